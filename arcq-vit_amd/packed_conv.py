"""``ARCQPackedPatchConv``: inference form of the reference's ``QuantConv2dPCARCQ`` (FQ/quant_backends.py:329-384)
for a patch-embedding convolution, i.e. kernel == stride, no padding, dilation 1, one group.

The reference keeps this layer as fake quantization in its packed models (its converter only replaces linears,
FQ/arcq_packed_convert.py:8-14).  Here the layer runs on the same kernels as the packed linears:

* activation: pixels in NHWC order, one group = ``act_group_size`` channels of one pixel (three for RGB,
  ``min(64, in_ch)`` at :351), through the stage-1 kernel for arbitrary group sizes;
* weight: the ``[out_ch, in_ch*kh*kw]`` matrix encoded offline in groups of ``group_size`` exactly like a linear
  weight (:374-376), kept as packed codes + per-group metadata;
* the convolution over non-overlapping patches is a matrix product of the patch rows ``[B*Hp*Wp, in_ch*kh*kw]``
  with that matrix, done by the fused unpack+GEMM kernel (fp16 operands, fp32 accumulation).

Forward always runs the HIP kernels; there is no CPU forward.
"""
from __future__ import annotations

from typing import Dict, Optional

import torch
import torch.nn as nn

from . import ops
from .packed_linear import _pack, _quantize_weight_reference, _require_vector, infer_packed_hparams


class ARCQPackedPatchConv(nn.Module):
    _FP32_BUFFERS = ("weight_center", "weight_scale", "weight_code_sum", "weight_codebook", "activation_codebook",
                     "activation_thresholds", "bias")

    def __init__(self, source: Optional[nn.Module]):
        super().__init__()
        if source is None:  # filled in by from_packed_state()
            return
        conv = getattr(source, "conv", None)
        if conv is None or not hasattr(conv, "weight") or conv.weight.dim() != 4:
            raise TypeError("ARCQPackedPatchConv source must expose source.conv.weight [out, in, kh, kw]")
        act_quant = getattr(source, "act_quant", None)
        weight_quant = getattr(source, "weight_quant", None)
        if act_quant is None or weight_quant is None:
            raise TypeError("ARCQPackedPatchConv source must expose act_quant and weight_quant")
        kh, kw = (int(v) for v in conv.kernel_size)
        if (tuple(conv.stride) != (kh, kw) or tuple(int(p) for p in conv.padding) != (0, 0)
                or tuple(conv.dilation) != (1, 1) or conv.groups != 1):
            raise ValueError("only patch convolutions (kernel == stride, no padding, dilation 1, groups 1) are packed; "
                             f"got kernel={tuple(conv.kernel_size)} stride={tuple(conv.stride)} "
                             f"padding={tuple(conv.padding)} dilation={tuple(conv.dilation)} groups={conv.groups}")
        self.in_channels, self.out_channels = int(conv.in_channels), int(conv.out_channels)
        self.kernel_size = (kh, kw)
        self.group_size = int(getattr(weight_quant, "group_size", 64))
        self.act_group_size = int(getattr(act_quant, "group_size", min(64, self.in_channels)))
        self.bits = int(getattr(weight_quant, "bits", 4))
        self.act_bits = int(getattr(act_quant, "bits", self.bits))
        if self.bits != self.act_bits:
            raise ValueError(f"packed kernel currently requires W bits == A bits, got W{self.bits} A{self.act_bits}")
        if self.bits not in (2, 3, 4):
            raise ValueError(f"packed kernel supports bits 2/3/4, got {self.bits}")
        k = self.in_channels * kh * kw
        if k % self.group_size != 0:
            raise ValueError(f"in_ch*kh*kw={k} must be divisible by group_size={self.group_size}")
        if self.in_channels % self.act_group_size != 0:
            # the fake-quant forward pads the channel dimension (Q/dcarcq.py:528-533); no trained model needs it
            raise ValueError(f"in_channels={self.in_channels} must be divisible by the activation group size "
                             f"{self.act_group_size}")
        eps = float(getattr(weight_quant, "eps", getattr(act_quant, "eps", 1.0e-6)))
        a_cb = _require_vector("act_quant._pc_cb", getattr(act_quant, "_pc_cb", None))
        a_thr = _require_vector("act_quant._pc_thresholds", getattr(act_quant, "_pc_thresholds", None))
        w_cb = _require_vector("weight_quant._pc_cb", getattr(weight_quant, "_pc_cb", None))
        w_thr = _require_vector("weight_quant._pc_thresholds", getattr(weight_quant, "_pc_thresholds", None))
        if a_cb.numel() != 2 ** self.bits or w_cb.numel() != 2 ** self.bits:
            raise ValueError(f"codebook size must be {2 ** self.bits}, got A={a_cb.numel()} W={w_cb.numel()}")
        device = conv.weight.device
        w2 = conv.weight.detach().reshape(self.out_channels, k)
        codes, center, scale, code_sum = _quantize_weight_reference(w2, w_thr.to(device), w_cb.to(device),
                                                                    self.group_size, eps)
        bias = None if conv.bias is None else conv.bias.detach().to(device=device, dtype=torch.float32)
        self._register(_pack(codes, self.bits), center, scale, code_sum, w_cb.to(device), a_cb.to(device),
                       a_thr.to(device), bias)

    def _register(self, packed, center, scale, code_sum, w_cb, a_cb, a_thr, bias) -> None:
        device = packed.device
        self.register_buffer("packed_weight_codes", packed.contiguous())
        self.register_buffer("weight_center", center.float().contiguous())
        self.register_buffer("weight_scale", scale.float().contiguous())
        self.register_buffer("weight_code_sum", code_sum.float().contiguous())
        self.register_buffer("weight_codebook", w_cb.float().contiguous())
        self.register_buffer("activation_codebook", a_cb.float().contiguous())
        self.register_buffer("activation_thresholds", a_thr.float().contiguous())
        if bias is None or bias.numel() == 0:
            self.register_buffer("bias", torch.empty(0, device=device, dtype=torch.float32))
        else:
            self.register_buffer("bias", bias.float().contiguous())
        # what tensor shapes cannot tell a loader: [in_channels, kh, kw, activation group size]
        self.register_buffer("conv_geometry", torch.tensor(
            [self.in_channels, self.kernel_size[0], self.kernel_size[1], self.act_group_size], dtype=torch.int64,
            device=device))
        self.packed_weight_bytes = int(self.packed_weight_codes.numel())
        self.weight_meta_floats = int(
            self.weight_center.numel() + self.weight_scale.numel() + self.weight_code_sum.numel())

    @classmethod
    def from_packed_state(cls, state_dict: Dict[str, torch.Tensor], prefix: str = "") -> "ARCQPackedPatchConv":
        """Rebuild the layer from the buffers its ``state_dict`` holds under ``prefix``."""
        def get(name, required=True):
            t = state_dict.get(prefix + name)
            if t is None and required:
                raise KeyError(f"packed checkpoint has no '{prefix + name}'")
            return t

        packed, center, w_cb = get("packed_weight_codes"), get("weight_center"), get("weight_codebook")
        hp = infer_packed_hparams(packed, center, w_cb)
        geo = [int(v) for v in get("conv_geometry").tolist()]
        if len(geo) != 4 or geo[0] * geo[1] * geo[2] != hp["in_features"] or geo[3] <= 0 or geo[0] % geo[3] != 0:
            raise ValueError(f"conv_geometry {geo} does not match a packed row of {hp['in_features']} codes")
        self = cls(None)
        self.in_channels, self.out_channels = geo[0], hp["out_features"]
        self.kernel_size = (geo[1], geo[2])
        self.act_group_size = geo[3]
        self.group_size = hp["group_size"]
        self.bits = self.act_bits = hp["bits"]
        a_cb, a_thr = get("activation_codebook"), get("activation_thresholds")
        if a_cb.numel() != w_cb.numel() or a_thr.numel() != a_cb.numel() - 1:
            raise ValueError("activation codebook/thresholds do not match the weight codebook size")
        if a_thr.numel() > 1 and not bool((a_thr[1:] >= a_thr[:-1]).all()):
            raise ValueError("activation_thresholds must be non-decreasing")
        self._register(packed, center, get("weight_scale"), get("weight_code_sum"), w_cb, a_cb, a_thr,
                       get("bias", required=False))
        return self

    def _apply(self, fn, *args, **kwargs):
        # model.half() must not narrow the fp32 metadata; device moves still apply.
        keep = {n: self._buffers[n] for n in self._FP32_BUFFERS if self._buffers.get(n) is not None}
        super()._apply(fn, *args, **kwargs)
        for name, orig in keep.items():
            new = self._buffers[name]
            if new.dtype != orig.dtype:
                self._buffers[name] = orig.to(device=new.device)
        return self

    def extra_repr(self) -> str:
        return (f"in_channels={self.in_channels}, out_channels={self.out_channels}, kernel_size={self.kernel_size}, "
                f"bits={self.bits}, group_size={self.group_size}, act_group_size={self.act_group_size}, "
                f"packed_weight_bytes={self.packed_weight_bytes}")

    def estimated_storage_bytes(self) -> int:
        return int(sum(b.numel() * b.element_size() for b in self.buffers()))

    def patch_rows(self, x_hat_nhwc: torch.Tensor) -> torch.Tensor:
        """``[B, H, W, C]`` -> ``[B*Hp*Wp, C*kh*kw]`` with the column order ``(c, i, j)`` of ``conv.weight.reshape``."""
        b, h, w, c = x_hat_nhwc.shape
        kh, kw = self.kernel_size
        t = x_hat_nhwc.reshape(b, h // kh, kh, w // kw, kw, c).permute(0, 1, 3, 5, 2, 4)
        return t.reshape(b * (h // kh) * (w // kw), c * kh * kw)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        if x.dim() != 4 or x.shape[1] != self.in_channels:
            raise ValueError(f"expected input [B, {self.in_channels}, H, W], got {tuple(x.shape)}")
        kh, kw = self.kernel_size
        b, c, h, w = x.shape
        if h % kh != 0 or w % kw != 0:
            raise ValueError(f"image size {h}x{w} is not a multiple of the patch size {kh}x{kw}")
        dev = self.packed_weight_codes.device
        x = x.to(dev)
        if x.dtype not in (torch.float16, torch.float32):
            x = x.float()
        bias = self.bias if self.bias.numel() > 0 else None
        weights = (self.packed_weight_codes, self.weight_codebook, self.weight_center, self.weight_scale, self.weight_code_sum)
        m = b * (h // kh) * (w // kw)
        if (kh, kw) == (16, 16) and c == 3 and self.act_group_size == 3 and self.group_size == 64:
            # one launch for stage 1: the pixels' groups quantized and written as patch rows (same values, bit for bit,
            # as the general route below); from 512 patches on in the block layout of the weight-stationary GEMMs
            blocked = m >= 512
            rows = ops.quantize_patches(x, self.activation_thresholds, self.activation_codebook, self.bits, blocked=blocked)
            if blocked:
                y = ops.linear_fused_blocked(rows, m, c * kh * kw, *weights, bias, self.bits, out_dtype=x.dtype)
            else:
                y = ops.linear_fused(rows, *weights, bias, self.bits, self.group_size, out_dtype=x.dtype)
        else:
            pixels = x.permute(0, 2, 3, 1).contiguous().reshape(-1, c)
            x_hat = ops.dequant_activation_hip(pixels, self.activation_thresholds, self.activation_codebook,
                                               self.act_group_size)
            rows = self.patch_rows(x_hat.reshape(b, h, w, c)).to(torch.float16)
            y = ops.linear_fused(rows, *weights, bias, self.bits, self.group_size, out_dtype=x.dtype)
        return y.reshape(b, h // kh, w // kw, self.out_channels).permute(0, 3, 1, 2)
