"""``ARCQPackedLinear``: inference-only packed ARCQ linear with the reference's storage layout.

Mirrors FQ/arcq_packed_linear.py (``FQ`` = ``methods/fair_qat_framework/fair_qat``): same
constructor, buffer names/shapes/dtypes (:119-146), attributes, error conditions (:66-103,
:163-164) and the three runtime formats (:161-222).  A fourth format, ``"hip_fused"``, runs the
packed on-the-fly path (stage 1 -> fused unpack+GEMM) on the same buffers.

The offline encode (``_quantize_weight_reference``) is host logic and uses the same torch
calls as the reference, so on one machine it yields the same bytes as the reference converter.
Forward always runs the HIP kernels; there is no CPU forward.
"""
from __future__ import annotations

from typing import Dict, Optional, Tuple

import torch
import torch.nn as nn
import torch.nn.functional as F

from . import ops
from .pack_py import pack_codes_py, unpack_codes_py

_FORMATS = ("packed", "u8", "dequant_gemm", "hip_fused")


def _require_vector(name: str, value) -> torch.Tensor:
    """FQ/arcq_packed_linear.py:21-24."""
    if not isinstance(value, torch.Tensor) or value.numel() == 0:
        raise ValueError(f"{name} is missing; load a checkpoint with compiled ARCQ codebooks first")
    return value.detach().float().flatten().contiguous()


def _quantize_weight_reference(weight: torch.Tensor, thresholds: torch.Tensor, codebook: torch.Tensor,
                               group_size: int, eps: float) -> Tuple[torch.Tensor, ...]:
    """Offline weight encode, FQ/arcq_packed_linear.py:27-53: per group of ``group_size`` input
    channels, mean / sqrt(mean sq residual + eps) / bucketize / sum of looked-up values.

    Returns ``codes [N,K] int64``, ``center``, ``scale``, ``code_sum`` ``[N,G] fp32``.
    """
    if weight.dim() != 2:
        raise ValueError(f"ARCQPackedLinear expects 2D linear weight, got shape={tuple(weight.shape)}")
    out_features, in_features = weight.shape
    if in_features % group_size != 0:
        raise ValueError(
            f"in_features={in_features} must be divisible by group_size={group_size} "
            "for the first packed kernel version")
    w3 = weight.detach().float().contiguous().reshape(out_features, in_features // group_size, group_size)
    center = w3.mean(dim=-1)
    residual = w3 - center.unsqueeze(-1)
    scale = (residual.square().mean(dim=-1) + float(eps)).sqrt()
    t = residual / scale.unsqueeze(-1)
    codes = torch.bucketize(t, thresholds.to(device=t.device, dtype=t.dtype))
    code_sum = codebook.to(device=t.device, dtype=t.dtype)[codes].sum(dim=-1)
    return codes.reshape(out_features, in_features).to(torch.int64), center, scale, code_sum


def _pack(codes: torch.Tensor, bits: int) -> torch.Tensor:
    return ops.pack_codes(codes, bits) if codes.is_cuda else pack_codes_py(codes, bits)


def _unpack_u8(packed: torch.Tensor, bits: int, length: int) -> torch.Tensor:
    if packed.is_cuda:
        return ops.unpack_codes_u8(packed, bits, length)
    return unpack_codes_py(packed, bits, length).to(torch.uint8)


def infer_packed_hparams(packed_weight_codes: torch.Tensor, weight_center: torch.Tensor,
                         weight_codebook: torch.Tensor) -> Dict[str, int]:
    """Hyper-parameters are not stored in a packed ``state_dict``; recover them from shapes.

    ``N = packed.shape[0]``, ``G = center.shape[1]``, ``bits = log2(len(codebook))``; ``K`` is the
    row length whose packed size ``ceil(K*bits/8)`` equals ``packed.shape[1]`` and which ``G``
    divides (a row of 3-bit codes can end inside a byte, so up to three lengths share a packed size;
    a shape that leaves more than one of them is rejected as ambiguous), ``gs = K // G``.
    """
    levels = int(weight_codebook.numel())
    bits = levels.bit_length() - 1
    if levels != 1 << bits or bits not in (2, 3, 4):
        raise ValueError(f"weight_codebook has {levels} entries; expected 4, 8 or 16")
    n, pcols = packed_weight_codes.shape
    groups = int(weight_center.shape[1])
    k_max = (pcols * 8) // bits
    fits = [k for k in range(k_max, max(k_max - 8, 0), -1)
            if (k * bits + 7) // 8 == pcols and groups > 0 and k % groups == 0]
    if len(fits) != 1:
        raise ValueError(f"{'ambiguous' if fits else 'inconsistent'} packed shapes: "
                         f"packed={tuple(packed_weight_codes.shape)} groups={groups} bits={bits} "
                         f"(candidate in_features: {fits})")
    k = fits[0]
    return {"in_features": k, "out_features": int(n), "bits": bits, "group_size": k // groups}


class ARCQPackedLinear(nn.Module):
    """Replaces a trained ``QuantLinearPCARCQ``; keeps low-bit weight indices plus per-group
    metadata and never the full floating-point weight."""

    def __init__(self, source: Optional[nn.Module], runtime_code_format: str = "packed"):
        super().__init__()
        if runtime_code_format not in _FORMATS:
            raise ValueError(
                "runtime_code_format must be 'packed', 'u8', 'dequant_gemm', or 'hip_fused', "
                f"got {runtime_code_format}")
        self.runtime_code_format = runtime_code_format
        if source is None:  # filled in by from_packed_state()
            return
        linear = getattr(source, "linear", None)
        if linear is None or not hasattr(linear, "weight"):
            raise TypeError("ARCQPackedLinear source must expose source.linear.weight")
        act_quant = getattr(source, "act_quant", None)
        weight_quant = getattr(source, "weight_quant", None)
        if act_quant is None or weight_quant is None:
            raise TypeError("ARCQPackedLinear source must expose act_quant and weight_quant")

        self.in_features = int(linear.weight.shape[1])
        self.out_features = int(linear.weight.shape[0])
        self.group_size = int(getattr(weight_quant, "group_size", 64))
        self.bits = int(getattr(weight_quant, "bits", 4))
        self.act_bits = int(getattr(act_quant, "bits", self.bits))
        if self.bits != self.act_bits:
            raise ValueError(f"packed kernel currently requires W bits == A bits, got W{self.bits} A{self.act_bits}")
        if self.bits not in (2, 3, 4):
            raise ValueError(f"packed kernel supports bits 2/3/4, got {self.bits}")
        if self.in_features % self.group_size != 0:
            raise ValueError(f"in_features={self.in_features} must be divisible by group_size={self.group_size}")

        eps = float(getattr(weight_quant, "eps", getattr(act_quant, "eps", 1.0e-6)))
        a_cb = _require_vector("act_quant._pc_cb", getattr(act_quant, "_pc_cb", None))
        a_thr = _require_vector("act_quant._pc_thresholds", getattr(act_quant, "_pc_thresholds", None))
        w_cb = _require_vector("weight_quant._pc_cb", getattr(weight_quant, "_pc_cb", None))
        w_thr = _require_vector("weight_quant._pc_thresholds", getattr(weight_quant, "_pc_thresholds", None))
        if a_cb.numel() != 2 ** self.bits or w_cb.numel() != 2 ** self.bits:
            raise ValueError(f"codebook size must be {2 ** self.bits}, got A={a_cb.numel()} W={w_cb.numel()}")

        device = linear.weight.device
        codes, center, scale, code_sum = _quantize_weight_reference(
            linear.weight, w_thr.to(device), w_cb.to(device), self.group_size, eps)
        packed = _pack(codes, self.bits)
        bias = None if linear.bias is None else linear.bias.detach().to(device=device, dtype=torch.float32)
        self._register(packed, center, scale, code_sum, w_cb.to(device), a_cb.to(device), a_thr.to(device), bias,
                       codes=codes)

    # -- construction helpers -------------------------------------------------------------
    def _register(self, packed, center, scale, code_sum, w_cb, a_cb, a_thr, bias, codes=None) -> None:
        device = packed.device
        self.register_buffer("packed_weight_codes", packed.contiguous())
        if self.runtime_code_format == "u8":
            codes_u8 = _unpack_u8(self.packed_weight_codes, self.bits, self.in_features).contiguous()
        else:
            codes_u8 = torch.empty(0, device=device, dtype=torch.uint8)
        self.register_buffer("weight_codes_u8", codes_u8)
        if self.runtime_code_format == "dequant_gemm":
            # FQ/arcq_packed_linear.py:126-130: center + scale * (cb[codes] - code_sum/gs), two roundings.
            if codes is None:
                codes = unpack_codes_py(packed, self.bits, self.in_features) if not packed.is_cuda \
                    else ops.unpack_codes(packed, self.bits, self.in_features)
            vals = w_cb.float()[codes].reshape(self.out_features, self.in_features // self.group_size,
                                               self.group_size)
            off = vals - code_sum.float().unsqueeze(-1) / float(self.group_size)
            wd = center.float().unsqueeze(-1) + scale.float().unsqueeze(-1) * off
            wd = wd.reshape(self.out_features, self.in_features).to(torch.float16).contiguous()
        else:
            wd = torch.empty(0, device=device, dtype=torch.float16)
        self.register_buffer("weight_dequant", wd)
        self.register_buffer("weight_center", center.float().contiguous())
        self.register_buffer("weight_scale", scale.float().contiguous())
        self.register_buffer("weight_code_sum", code_sum.float().contiguous())
        self.register_buffer("weight_codebook", w_cb.float().contiguous())
        self.register_buffer("activation_codebook", a_cb.float().contiguous())
        self.register_buffer("activation_thresholds", a_thr.float().contiguous())
        self.register_buffer("product_table",
                             (a_cb.float().view(-1, 1) * w_cb.float().view(1, -1)).contiguous())
        if bias is None or bias.numel() == 0:
            self.register_buffer("bias", torch.empty(0, device=device, dtype=torch.float32))
        else:
            self.register_buffer("bias", bias.float().contiguous())
        self.packed_weight_bytes = int(self.packed_weight_codes.numel())
        self.weight_meta_floats = int(
            self.weight_center.numel() + self.weight_scale.numel() + self.weight_code_sum.numel())

    @classmethod
    def from_packed_state(cls, state_dict: Dict[str, torch.Tensor], prefix: str = "",
                          runtime_code_format: str = "hip_fused") -> "ARCQPackedLinear":
        """Rebuild a layer from the buffers a packed checkpoint holds under ``prefix``
        (what ``torch.save(model.state_dict())`` at scripts/convert_arcq_to_packed.py:86-95 wrote)."""
        def get(name, required=True):
            t = state_dict.get(prefix + name)
            if t is None and required:
                raise KeyError(f"packed checkpoint has no '{prefix + name}'")
            return t

        packed = get("packed_weight_codes")
        center, w_cb = get("weight_center"), get("weight_codebook")
        hp = infer_packed_hparams(packed, center, w_cb)
        self = cls(None, runtime_code_format)
        self.in_features, self.out_features = hp["in_features"], hp["out_features"]
        self.bits = self.act_bits = hp["bits"]
        self.group_size = hp["group_size"]
        a_cb, a_thr = get("activation_codebook"), get("activation_thresholds")
        if a_cb.numel() != w_cb.numel() or a_thr.numel() != a_cb.numel() - 1:
            raise ValueError("activation codebook/thresholds do not match the weight codebook size")
        if a_thr.numel() > 1 and not bool((a_thr[1:] >= a_thr[:-1]).all()):
            raise ValueError("activation_thresholds must be non-decreasing")
        bias = get("bias", required=False)
        if bias is None:
            bias = get("bias_tensor", required=False)  # spelling of the on-the-fly module
        self._register(packed, center, get("weight_scale"), get("weight_code_sum"), w_cb, a_cb, a_thr, bias)
        return self

    # -- nn.Module API --------------------------------------------------------------------
    def extra_repr(self) -> str:
        return (f"in_features={self.in_features}, out_features={self.out_features}, "
                f"bits={self.bits}, group_size={self.group_size}, "
                f"runtime_code_format={self.runtime_code_format}, "
                f"packed_weight_bytes={self.packed_weight_bytes}")

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        original_shape = x.shape
        if original_shape[-1] != self.in_features:
            raise ValueError(f"expected last dim {self.in_features}, got {original_shape[-1]}")
        dev = self.packed_weight_codes.device
        bias = self.bias if self.bias.numel() > 0 else None
        fmt = self.runtime_code_format
        if fmt == "hip_fused":
            x2 = x.reshape(-1, self.in_features).to(device=dev)
            if x2.dtype not in (torch.float16, torch.float32):
                x2 = x2.float()
            y2 = ops.linear_otf(x2.contiguous(), self.activation_thresholds, self.activation_codebook,
                                self.packed_weight_codes, self.weight_codebook, self.weight_center,
                                self.weight_scale, self.weight_code_sum, bias, self.bits, self.group_size,
                                out_dtype=torch.float32)
            return y2.reshape(*original_shape[:-1], self.out_features)
        x2 = x.reshape(-1, self.in_features).to(device=dev, dtype=torch.float32).contiguous()
        if fmt == "dequant_gemm" and self.group_size == 64 and x2.shape[0] > 0:
            # Stage 1 -> fp16 x_hat (the fp32 reconstruction rounded once, as `.half()` of the reference's fp32 x_hat),
            # then this library's MFMA GEMM on the cached dense weight (no vendor GEMM); the bias is added in fp32
            # before the one output rounding (the reference rounds it to fp16 first, FQ/arcq_packed_linear.py:175).
            xb = ops.quantize_activation_blocked(x2, self.activation_thresholds, self.activation_codebook, self.bits)
            y2 = ops.linear_fused_blocked(xb, x2.shape[0], self.in_features, self.packed_weight_codes, self.weight_codebook,
                                          self.weight_center, self.weight_scale, self.weight_code_sum, bias, self.bits,
                                          out_dtype=torch.float32, w_hat_ws=self.weight_dequant.reshape(-1),
                                          w_hat_ready=True)
        elif fmt == "dequant_gemm":          # other group sizes: the generic stage-1 kernel and a library GEMM
            x_hat = ops.quantize_activation_dequant(x2, self.activation_thresholds, self.activation_codebook,
                                                    self.bits, self.group_size)
            gemm_bias = self.bias.to(torch.float16) if bias is not None else None
            y2 = F.linear(x_hat.to(torch.float16), self.weight_dequant, gemm_bias).to(torch.float32)
        elif fmt == "u8":
            codes, xc, xs, xcs = ops.quantize_activation_u8(x2, self.activation_thresholds,
                                                            self.activation_codebook, self.bits, self.group_size)
            y2 = ops.arcq_linear_forward_u8(codes, xc, xs, xcs, self.weight_codes_u8, self.weight_center,
                                            self.weight_scale, self.weight_code_sum, self.product_table, bias,
                                            self.group_size)
        else:
            px, xc, xs, xcs = ops.quantize_activation(x2, self.activation_thresholds, self.activation_codebook,
                                                      self.bits, self.group_size)
            y2 = ops.arcq_linear_forward(px, xc, xs, xcs, self.packed_weight_codes, self.weight_center,
                                         self.weight_scale, self.weight_code_sum, self.product_table, bias,
                                         self.bits, self.group_size, self.in_features, self.out_features)
        return y2.reshape(*original_shape[:-1], self.out_features)

    def estimated_storage_bytes(self) -> int:
        """FQ/arcq_packed_linear.py:224-235: packed bytes + 4 bytes per metadata float."""
        meta = (self.weight_center.numel() + self.weight_scale.numel() + self.weight_code_sum.numel()
                + self.weight_codebook.numel() + self.activation_codebook.numel()
                + self.activation_thresholds.numel() + self.product_table.numel() + self.bias.numel()) * 4
        return int(self.packed_weight_codes.numel() + meta)

    def runtime_cache_bytes(self) -> int:
        """FQ/arcq_packed_linear.py:237-241."""
        return int(self.weight_codes_u8.numel() * self.weight_codes_u8.element_size()
                   + self.weight_dequant.numel() * self.weight_dequant.element_size())
