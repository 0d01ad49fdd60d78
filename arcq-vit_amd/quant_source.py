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
