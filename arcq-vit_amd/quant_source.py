"""Source-side contract of the converter: a fake-quant linear shaped like the reference's
``QuantLinearPCARCQ`` (FQ/quant_backends.py:282-322) with quantizers that carry a ready,
frozen codebook (``_pc_cb``, ``_pc_thresholds``, ``bits``, ``group_size``, ``eps`` --
Q/dcarcq.py:433-455).

Only what conversion and model-level comparison need is here: eval-mode forward with a
compiled codebook (Q/dcarcq.py:512-578).  Codebook fitting and training are out of scope.
The converter matches the class by NAME (FQ/arcq_packed_convert.py:8-14), so a module
unpickled from a real ARCQ training run converts the same way.
"""
from __future__ import annotations

import torch
import torch.nn as nn
import torch.nn.functional as F


class FrozenARCQQuantizer(nn.Module):
    """Group-residual quantizer with a fixed codebook (eval behaviour of ``ARCQPCQuantizer``)."""

    def __init__(self, bits: int = 4, group_size: int = 64, eps: float = 1.0e-6):
        super().__init__()
        self.bits = int(bits)
        self.group_size = int(group_size)
        self.eps = float(eps)
        self.mean_preserve = True
        self._pc_ready = False
        self.register_buffer("_pc_cb", torch.empty(0))
        self.register_buffer("_pc_thresholds", torch.empty(0))

    def set_codebook(self, codebook: torch.Tensor) -> None:
        cb = codebook.detach().float().flatten().contiguous()
        if cb.numel() != 2 ** self.bits:
            raise ValueError(f"codebook size must be {2 ** self.bits}, got {cb.numel()}")
        self._pc_cb = cb.clone()
        self._pc_thresholds = ((cb[:-1] + cb[1:]) / 2.0).clone()  # Q/dcarcq.py:483
        self._pc_ready = True

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        if self.bits >= 8:
            return x
        if not self._pc_ready or self._pc_cb.numel() == 0:
            raise RuntimeError("quantizer has no compiled codebook; call set_codebook() or load a checkpoint")
        shape = x.shape
        c = shape[-1]
        x2 = x.reshape(-1, c)
        pad = (-c) % self.group_size
        if pad:
            x2 = F.pad(x2, (0, pad))
        rows, cp = x2.shape
        x3 = x2.reshape(rows, cp // self.group_size, self.group_size)
        center = x3.mean(dim=-1, keepdim=True)
        residual = x3 - center
        scale = (residual.square().mean(dim=-1, keepdim=True) + self.eps).sqrt()
        t = residual / scale
        cb = self._pc_cb.to(device=x.device, dtype=t.dtype)
        thr = self._pc_thresholds.to(device=x.device, dtype=t.dtype)
        t_hat = cb[torch.bucketize(t, thr)]
        if self.mean_preserve:
            t_hat = t_hat - t_hat.mean(dim=-1, keepdim=True)
        x_hat = (center + scale * t_hat).reshape(rows, cp)
        if pad:
            x_hat = x_hat[:, :c]
        x_hat = x_hat.reshape(shape)
        return x + (x_hat - x).detach()


class QuantLinearPCARCQ(nn.Module):
    """``linear`` + ``act_quant`` + ``weight_quant``; forward = fake-quant both, then ``F.linear``."""

    def __init__(self, in_f: int, out_f: int, bias: bool, w_bits: int, a_bits: int, group_size: int = 64):
        super().__init__()
        self.linear = nn.Linear(in_f, out_f, bias=bias)
        self.act_quant = FrozenARCQQuantizer(bits=a_bits, group_size=group_size)
        self.weight_quant = FrozenARCQQuantizer(bits=w_bits, group_size=group_size)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return F.linear(self.act_quant(x), self.weight_quant(self.linear.weight), self.linear.bias)


class QuantConv2dPCARCQ(nn.Module):
    """``conv`` + ``act_quant`` + ``weight_quant`` (FQ/quant_backends.py:329-384 without the DC conditioner, which the
    ``pcarcq_nodc`` backend leaves off): the activation is quantized in NHWC order, so a group is
    ``min(group_size, in_ch)`` channels of one pixel (three for RGB input), the weight as the 2-D matrix
    ``[out_ch, in_ch * kh * kw]`` in groups of ``group_size``; then ``F.conv2d``."""

    def __init__(self, in_ch: int, out_ch: int, k, s, p, bias: bool, w_bits: int, a_bits: int, group_size: int = 64):
        super().__init__()
        self.conv = nn.Conv2d(in_ch, out_ch, k, stride=s, padding=p, bias=bias)
        act_gs = min(group_size, in_ch) if in_ch > 0 else group_size
        self.act_quant = FrozenARCQQuantizer(bits=a_bits, group_size=act_gs)
        self.weight_quant = FrozenARCQQuantizer(bits=w_bits, group_size=group_size)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        w = self.conv.weight
        x_q = self.act_quant(x.permute(0, 2, 3, 1).contiguous()).permute(0, 3, 1, 2).contiguous()
        w_q = self.weight_quant(w.reshape(w.shape[0], -1)).reshape_as(w)
        c = self.conv
        return F.conv2d(x_q, w_q, c.bias, c.stride, c.padding, c.dilation, c.groups)


class LSQQuantizer(nn.Module):
    """Uniform quantizer with a learned step size, eval behaviour only.

    The reference constructs ``quant.lsq.LSQQuantizer(bits, signed, per_channel, ch_axis)``
    (FQ/quant_backends.py:125-136) but does not ship ``quant/lsq.py``; its checkpoint loader shows that the step
    size is a parameter named ``step`` whose shape may differ from the registered one
    (scripts/benchmark_arcq_packed_inference.py:93-95).  What is here is the published LSQ forward (Esser et al.,
    ICLR 2020): ``round(clamp(x / step, Qn, Qp)) * step`` with ``Qn = -2^(bits-1)``, ``Qp = 2^(bits-1) - 1`` for
    signed and ``0 .. 2^bits - 1`` for unsigned tensors; a per-channel step broadcasts along ``ch_axis``.  With no
    reference source to compare against, parity of this class is unpinned."""

    def __init__(self, bits: int = 8, signed: bool = True, per_channel: bool = False, ch_axis: int = 0):
        super().__init__()
        self.bits = int(bits)
        self.signed = bool(signed)
        self.per_channel = bool(per_channel)
        self.ch_axis = int(ch_axis)
        self.qn = -(1 << (self.bits - 1)) if self.signed else 0
        self.qp = (1 << (self.bits - 1)) - 1 if self.signed else (1 << self.bits) - 1
        self.step = nn.Parameter(torch.ones(1))

    def init_from(self, x: torch.Tensor) -> None:
        """Step size from data, the LSQ paper's initialisation ``2 mean|x| / sqrt(Qp)`` (per channel if so built)."""
        with torch.no_grad():
            if self.per_channel:
                dims = [d for d in range(x.dim()) if d != self.ch_axis % x.dim()]
                mean_abs = x.detach().abs().mean(dim=dims)
            else:
                mean_abs = x.detach().abs().mean().reshape(1)
            self.step = nn.Parameter((2.0 * mean_abs / (self.qp ** 0.5)).clamp_min(1e-8).float())

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        if self.bits >= 32:
            return x
        step = self.step.to(x.dtype)
        if step.numel() > 1:
            shape = [1] * x.dim()
            shape[self.ch_axis % x.dim()] = step.numel()
            step = step.reshape(shape)
        return torch.clamp(x / step, self.qn, self.qp).round() * step


class QuantLinearLSQ(nn.Module):
    """``linear`` + per-tensor activation LSQ + per-output-channel weight LSQ (FQ/quant_backends.py:125-136); the
    ``pcarcq_nodc`` backend uses it at 8/8 bits for the classifier head (:420-421)."""

    def __init__(self, in_f: int, out_f: int, bias: bool, w_bits: int = 8, a_bits: int = 8):
        super().__init__()
        self.linear = nn.Linear(in_f, out_f, bias=bias)
        self.act_quant = LSQQuantizer(bits=a_bits, signed=True, per_channel=False)
        self.weight_quant = LSQQuantizer(bits=w_bits, signed=True, per_channel=True, ch_axis=0)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return F.linear(self.act_quant(x), self.weight_quant(self.linear.weight), self.linear.bias)
