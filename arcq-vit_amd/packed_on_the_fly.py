"""``ARCQPackedLinearOnTheFly``: the packed on-the-fly layer (the path the reference's README
benchmarks), constructor and buffers as FQ/arcq_packed_on_the_fly.py:93-135.

Reference forward (:137-161): fp16 copy of x -> Triton quantize+reconstruct in place -> Triton
unpack of the whole weight into an fp16 buffer in HBM -> cuBLAS ``F.linear``.  Here the layer is one
or two HIP launches (``arcq_linear_otf_ws`` / ``arcq_linear_otf_ex``): stage 1 writes x_hat (fp16)
into a workspace or keeps it in LDS, and the fused unpack + fp16 MFMA GEMM follows.  Where the
dense weight lives depends on ``_weight_buffer`` (the flat fp16 scratch the reference's benchmark
shares between all layers, scripts/benchmark_arcq_on_the_fly.py:182-191, read at :148-158):
  * not set: the GEMM kernel rebuilds the weight tile by tile in LDS; the dense weight never exists
    in HBM;
  * set (what ``packed_convert.share_buffers`` and ``bench.py`` do): from 512 rows on the fp16
    weight is reconstructed into it inside the layer's first (or only) launch and the GEMM reads it
    from there, i.e. it does pass through memory (L2-resident, a few MB) -- the reference's
    unpack-then-GEMM order without a launch of its own; below 512 rows it is not used.
The result is bit-identical either way.

Differences from the reference module that a caller can observe (all on the side of more accuracy;
for these cases "same indices as the reference" is not pinned by any test):
  * the input tensor is never overwritten (the reference overwrites a contiguous fp16 input);
  * group statistics are taken in fp32 even for fp16 input (the Triton kernel reduces in fp16);
  * an fp32 input is quantized from its fp32 values (the reference first casts x to fp16, :139);
  * the bias is added in fp32 before the one output rounding (the reference rounds the bias to fp16);
  * ``model.half()`` leaves the fp32 metadata (codebooks, thresholds, center/scale/code_sum, bias)
    at their fp32 values (the reference's half chain leaves them rounded to fp16).
"""
from __future__ import annotations

import ctypes
from typing import Dict, Optional, Tuple

import torch
import torch.nn as nn

from . import _lib, ops
from ._lib import ARCQ_F16, ARCQ_F32

# Fallback fp16 x_hat workspace, one per (device, stream), for layers that were given no ``_x_hat_buffer``: layers
# run back to back on a stream, and stream order makes the reuse safe.  Grown on demand; ``clear_workspaces()``
# releases them.  Never used while a HIP graph is being captured: memory allocated during a capture belongs to
# that graph's private pool, so a capture gets a buffer of its own (kept alive by the graph's pool) instead of
# leaving one in this cache for a later capture to find.
_workspaces: Dict[Tuple[int, int], torch.Tensor] = {}


def _workspace(device: torch.device, numel: int) -> torch.Tensor:
    if torch.cuda.is_current_stream_capturing():
        return torch.empty(max(numel, 1), dtype=torch.float16, device=device)
    key = (device.index if device.index is not None else torch.cuda.current_device(),
           torch.cuda.current_stream(device).cuda_stream)
    ws = _workspaces.get(key)
    if ws is None or ws.numel() < numel:
        ws = torch.empty(max(numel, 1), dtype=torch.float16, device=device)
        _workspaces[key] = ws
    return ws


def clear_workspaces() -> None:
    """Drop the fallback x_hat workspaces (they are re-created on demand)."""
    _workspaces.clear()


class ARCQPackedLinearOnTheFly(nn.Module):
    """Stores packed codes + codebooks + per-group metadata + bias only (no dense weight)."""

    def __init__(self, in_features: int, out_features: int, bias: bool,
                 packed_weight_codes: torch.Tensor, weight_codebook: torch.Tensor,
                 weight_center: torch.Tensor, weight_scale: torch.Tensor, weight_code_sum: torch.Tensor,
                 activation_codebook: torch.Tensor, activation_thresholds: torch.Tensor,
                 bits: int, group_size: int, bias_tensor: Optional[torch.Tensor]):
        super().__init__()
        self.in_features = int(in_features)
        self.out_features = int(out_features)
        self.bits = int(bits)
        self.group_size = int(group_size)
        self.groups = self.in_features // self.group_size
        if self.bits not in (2, 3, 4):
            raise ValueError(f"packed kernel supports bits 2/3/4, got {self.bits}")
        if self.in_features % self.group_size != 0:
            raise ValueError(f"in_features={self.in_features} must be divisible by group_size={self.group_size}")
        if tuple(packed_weight_codes.shape) != (self.out_features, (self.in_features * self.bits + 7) // 8):
            raise ValueError(f"packed_weight_codes has shape {tuple(packed_weight_codes.shape)}, expected "
                             f"{(self.out_features, (self.in_features * self.bits + 7) // 8)}")
        self.register_buffer("packed_weight_codes", packed_weight_codes)
        self.register_buffer("weight_codebook", weight_codebook)
        self.register_buffer("weight_center", weight_center)
        self.register_buffer("weight_scale", weight_scale)
        self.register_buffer("weight_code_sum", weight_code_sum)
        self.register_buffer("activation_codebook", activation_codebook)
        self.register_buffer("activation_thresholds", activation_thresholds)
        if bias and bias_tensor is not None and bias_tensor.numel() > 0:
            self.register_buffer("bias_tensor", bias_tensor)
        else:
            self.register_buffer("bias_tensor", torch.empty(0))
        self.out_dtype = torch.float16
        self._prep = None
        # Opt-in: operands rounded to FP8 and the product on FP8 matrix units (ops.linear_otf_fp8).  Faster on the
        # large models, not the reference's numerics; see set_fp8_operands in packed_convert.
        self.fp8_operands = False
        self._fp8_mult = None

    def _prepare(self):
        """Validated, fp32-contiguous views of the buffers and their raw pointers, built once and reused by every
        forward until a buffer moves (``_apply``, ``load_state_dict``), is replaced or is written in place."""
        a = [ops._f32c(self.activation_thresholds), ops._f32c(self.activation_codebook)]
        w = [self.packed_weight_codes.contiguous(), ops._f32c(self.weight_codebook), ops._f32c(self.weight_center),
             ops._f32c(self.weight_scale), ops._f32c(self.weight_code_sum)]
        bias = ops._f32c(self.bias_tensor) if self.bias_tensor.numel() > 0 else None
        keep = a + w + [bias]
        self._prep = (keep, tuple(0 if t is None else t.data_ptr() for t in keep), self._buffers_key(),
                      self.packed_weight_codes.device)
        return self._prep

    _PREP_BUFFERS = ("activation_thresholds", "activation_codebook", "packed_weight_codes", "weight_codebook",
                     "weight_center", "weight_scale", "weight_code_sum", "bias_tensor")

    def _buffers_key(self):
        """Identity and version of every buffer the cached pointers were made from: replacing a buffer or writing into
        one in place changes it, and the next forward prepares again."""
        b = self._buffers
        return tuple((b[n].data_ptr(), b[n]._version) for n in self._PREP_BUFFERS)

    def _load_from_state_dict(self, *args, **kwargs):
        self._prep = None
        self._fp8_mult = None
        return super()._load_from_state_dict(*args, **kwargs)

    @classmethod
    def from_packed(cls, packed_layer: nn.Module) -> "ARCQPackedLinearOnTheFly":
        """From an ``ARCQPackedLinear`` (what scripts/benchmark_arcq_on_the_fly.py:151-170 does)."""
        b = packed_layer.bias if packed_layer.bias.numel() > 0 else None
        return cls(packed_layer.in_features, packed_layer.out_features, b is not None,
                   packed_layer.packed_weight_codes, packed_layer.weight_codebook, packed_layer.weight_center,
                   packed_layer.weight_scale, packed_layer.weight_code_sum, packed_layer.activation_codebook,
                   packed_layer.activation_thresholds, packed_layer.bits, packed_layer.group_size, b)

    _FP32_BUFFERS = ("weight_codebook", "weight_center", "weight_scale", "weight_code_sum",
                     "activation_codebook", "activation_thresholds", "bias_tensor")

    def _apply(self, fn, *args, **kwargs):
        # model.half() must not narrow the fp32 metadata.  (The reference casts the whole model and
        # then widens these buffers again, scripts/benchmark_arcq_on_the_fly.py:63-85, which leaves
        # them rounded to fp16.)  Device moves still apply; dtype changes of these buffers do not.
        keep = {n: self._buffers[n] for n in self._FP32_BUFFERS if self._buffers.get(n) is not None}
        self._prep = None
        super()._apply(fn, *args, **kwargs)
        for name, orig in keep.items():
            new = self._buffers[name]
            if new.dtype != orig.dtype:
                self._buffers[name] = orig.to(device=new.device)
        return self

    def can_quantize_for(self, consumer: nn.Module, rows: int) -> bool:
        """Whether ``forward(..., quantize_for=consumer)`` is available: this layer's launch then ends with the
        consumer's stage 1 (the consumer is called with ``input_is_xhat=True``).  From 512 rows on it needs the shared
        weight buffer (``_weight_buffer``)."""
        if not (isinstance(consumer, ARCQPackedLinearOnTheFly) and not self.fp8_operands and not consumer.fp8_operands
                and rows > 0 and self.group_size == 64 and consumer.group_size == 64 and self.bits == consumer.bits
                and consumer.in_features == self.out_features and self.out_features % 64 == 0
                and self.in_features % 64 == 0 and self.out_dtype == torch.float16):
            return False
        if rows < 512:                       # the small-M kernel's epilogue
            return self.in_features <= 1536
        # The block-layout GEMM kernels' epilogue: needs the weight workspace.  Not taken where this layer would run as
        # one launch with stage 1 inside (short rows: DeiT-S at batch 64): the consumer's stage 1 is then already hidden
        # under its own product and the chained pair measured slower (DeiT-S forward 1.86 -> 2.08 ms; DeiT-B 4.88 ->
        # 4.76, ViT-L 49.7 -> 48.5).
        if getattr(self, "_weight_buffer", None) is None or rows * self.in_features * 2 >= 2 ** 32:
            return False
        kernel = _lib.load().arcq_linear_otf_ws_kernel(rows, self.out_features, self.in_features, 1)
        return not kernel.startswith(b"otf_rows")

    def forward(self, x: torch.Tensor, layernorm: Optional[nn.LayerNorm] = None, activation: Optional[str] = None,
                residual: Optional[torch.Tensor] = None, quantize_for: Optional[nn.Module] = None,
                input_is_xhat: bool = False) -> torch.Tensor:
        """``residual + activation(linear(stage1(layernorm(x))))``.  The three optional parts (the LayerNorm in front
        of the layer, ``activation="gelu"`` and the skip connection behind it, as they surround the block linears in
        timm's ``Block``, FQ/timm_quant_models.py:63-121) are fused into the layer's launches where the library can
        (group size 64; for the LayerNorm K <= 1024 from 512 rows on and K <= 1536 below) and run as separate torch
        operations otherwise; without them this is the reference module's forward.  ``quantize_for=consumer`` (see
        ``can_quantize_for``): the result is the consumer's ``x_hat`` instead of this layer's output, to be passed to
        ``consumer(..., input_is_xhat=True)``, which skips its own stage 1."""
        original_shape = x.shape
        if original_shape[-1] != self.in_features:
            raise ValueError(f"expected last dim {self.in_features}, got {original_shape[-1]}")
        if not x.is_cuda or not self.packed_weight_codes.is_cuda:
            raise RuntimeError("x and the layer's buffers must be CUDA tensors (there is no CPU forward)")
        if activation not in (None, "gelu"):
            raise ValueError(f"activation must be None or 'gelu', got {activation!r}")
        x2 = x.reshape(-1, self.in_features)
        if x2.dtype not in (torch.float16, torch.float32):
            x2 = x2.to(torch.float16)
        x2 = x2.contiguous()
        m = x2.shape[0]
        chain = quantize_for is not None or input_is_xhat
        if quantize_for is not None and not self.can_quantize_for(quantize_for, m):
            raise ValueError("quantize_for: not available for this pair of layers / number of rows (see can_quantize_for)")
        if input_is_xhat and (x2.dtype != torch.float16 or layernorm is not None or self.fp8_operands):
            raise ValueError("input_is_xhat: x must be the float16 x_hat a producer made for this layer")
        ln_fusable = layernorm is None or (self.in_features <= (1024 if m >= 512 else 1536) and layernorm.elementwise_affine
                                           and tuple(layernorm.normalized_shape) == (self.in_features,))
        if chain and not ln_fusable:     # (a chained call cannot fall back as a whole: only the LayerNorm runs apart)
            x2, layernorm, ln_fusable = layernorm(x2).contiguous(), None, True
        extras = layernorm is not None or activation is not None or residual is not None or chain
        fuse = (extras and not self.fp8_operands and m > 0 and self.group_size == 64 and self.in_features % 64 == 0
                and ln_fusable)
        if extras and not fuse:          # separate operations around the plain layer
            if layernorm is not None:
                x2 = layernorm(x2)
            y = self.forward(x2)
            if activation == "gelu":
                y = torch.nn.functional.gelu(y)
            if residual is not None:
                y = y + residual.reshape(-1, self.out_features)
            return y.reshape(*original_shape[:-1], self.out_features)
        prep = self._prep
        if prep is None or prep[2] != self._buffers_key():
            prep = self._prepare()
            self._fp8_mult = None
        if prep[3] != x2.device:
            raise RuntimeError("x and the layer's buffers must be on the same device")
        if self.fp8_operands:
            if self.group_size != 64:
                raise ValueError("fp8_operands needs group_size 64")
            if self._fp8_mult is None:          # (reads the metadata back once per layer)
                self._fp8_mult = ops.fp8_weight_multiplier(self.weight_codebook, self.weight_center, self.weight_scale,
                                                           self.weight_code_sum)
            t = prep[0]
            y = ops.linear_otf_fp8(x2, t[0], t[1], t[2], t[3], t[4], t[5], t[6], t[7], self.bits,
                                   out_dtype=self.out_dtype, w_mult=self._fp8_mult)
            return y.reshape(*original_shape[:-1], self.out_features)
        ws = getattr(self, "_x_hat_buffer", None)       # a buffer the model owns (packed_convert.share_buffers)
        if ws is None or ws.numel() < x2.numel() or ws.device != x2.device:
            ws = _workspace(x2.device, x2.numel())
        w_ws = getattr(self, "_weight_buffer", None)
        if w_ws is not None and (not w_ws.is_cuda or w_ws.dtype != torch.float16 or not w_ws.is_contiguous()
                                 or w_ws.numel() < self.out_features * self.in_features):
            raise ValueError("_weight_buffer must be a contiguous float16 CUDA tensor of at least "
                             "out_features * in_features elements")
        y = torch.empty((m, self.out_features), dtype=self.out_dtype, device=x2.device)
        p = prep[1]
        f16 = ARCQ_F16 if x2.dtype == torch.float16 else ARCQ_F32
        y16 = ARCQ_F16 if self.out_dtype == torch.float16 else ARCQ_F32
        stream = torch.cuda.current_stream().cuda_stream
        with torch.cuda.device(x2.device):
            if not extras:
                _lib.check(_lib.load().arcq_linear_otf_ws(
                    x2.data_ptr(), f16, p[0], p[1], p[2], p[3], p[4], p[5], p[6], p[7], ws.data_ptr(),
                    0 if w_ws is None else w_ws.data_ptr(), y.data_ptr(), y16, m, self.out_features, self.in_features,
                    self.bits, self.group_size, stream))
            else:
                a = _lib.LinearExArgs()
                a.struct_size = ctypes.sizeof(_lib.LinearExArgs)
                a.x_dtype, a.y_dtype, a.bits, a.group_size = f16, y16, self.bits, self.group_size
                a.M, a.N, a.K = m, self.out_features, self.in_features
                a.x = x2.data_ptr()
                keep = []
                if layernorm is not None:
                    lw, lb = self._layernorm_params(layernorm)
                    keep = [lw, lb]
                    a.producer, a.ln_weight, a.ln_bias, a.ln_eps = (_lib.ARCQ_PRODUCER_LAYERNORM, lw.data_ptr(),
                                                                   lb.data_ptr(), float(layernorm.eps))
                a.activation = _lib.ARCQ_ACT_GELU if activation == "gelu" else _lib.ARCQ_ACT_NONE
                (a.a_thresholds, a.a_codebook, a.packed_w, a.w_codebook, a.w_center, a.w_scale, a.w_code_sum,
                 a.bias) = [v or None for v in p]
                if input_is_xhat:
                    a.producer = _lib.ARCQ_PRODUCER_XHAT
                if quantize_for is not None:
                    nprep = quantize_for._prep
                    if nprep is None or nprep[2] != quantize_for._buffers_key():
                        nprep = quantize_for._prepare()
                        quantize_for._fp8_mult = None
                    a.next_a_thresholds, a.next_a_codebook = nprep[1][0], nprep[1][1]
                if residual is not None:
                    r2 = residual.reshape(-1, self.out_features)
                    if r2.dtype != self.out_dtype or tuple(r2.shape) != (m, self.out_features) or r2.device != x2.device:
                        raise ValueError("residual must have the output's shape, dtype and device")
                    r2 = r2.contiguous()
                    keep.append(r2)
                    a.residual = r2.data_ptr()
                a.x_hat_ws, a.w_hat_ws, a.y = ws.data_ptr(), (None if w_ws is None else w_ws.data_ptr()), y.data_ptr()
                _lib.check(_lib.load().arcq_linear_otf_ex(ctypes.byref(a), stream))
        return y.reshape(*original_shape[:-1], self.out_features)

    def _layernorm_params(self, layernorm: nn.LayerNorm):
        """fp32 copies of a LayerNorm's weight and bias, cached per LayerNorm module and parameter version."""
        cache = self.__dict__.setdefault("_ln_cache", {})
        key = id(layernorm)
        ver = (layernorm.weight._version, layernorm.weight.data_ptr(),
               None if layernorm.bias is None else layernorm.bias._version)
        hit = cache.get(key)
        if hit is None or hit[0] != ver:
            w = layernorm.weight.detach().to(torch.float32).contiguous()
            b = (torch.zeros_like(w) if layernorm.bias is None
                 else layernorm.bias.detach().to(torch.float32).contiguous())
            hit = (ver, w, b)
            cache[key] = hit
        return hit[1], hit[2]

    def estimated_persistent_mb(self) -> float:
        """MiB held by this layer's buffers (FQ/arcq_packed_on_the_fly.py:163-169)."""
        return sum(b.numel() * b.element_size() for b in self.buffers()) / 1024 / 1024
