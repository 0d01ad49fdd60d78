"""Operator layer: the reference extension's eight functions, same names, argument order and
returns, on top of ``libarcq_hip.so``.

Reference binding table: FQ/arcq_infer_cuda/arcq_infer_bind.cpp:57-66 (``FQ`` =
``methods/fair_qat_framework/fair_qat``).  Also here: the two launchers of
FQ/arcq_packed_triton.py (``unpack_weight_triton`` :77-120, ``dequant_activation_triton``
:181-215) under HIP names, and the fused entry points that have no counterpart in the
reference (``linear_fused``, ``linear_otf``).

All tensors must live on the GPU; outputs are allocated with torch on the same device and the
kernels are enqueued on torch's current stream.  Nothing here synchronises.
"""
from __future__ import annotations

import ctypes
from typing import List, Optional

import torch

from . import _lib
from ._lib import ARCQ_F16, ARCQ_F32


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def _ptr(t: Optional[torch.Tensor]) -> int:
    return 0 if t is None else t.data_ptr()


def _check(cond: bool, msg: str) -> None:
    # TORCH_CHECK raises c10::Error, which Python sees as RuntimeError.
    if not cond:
        raise RuntimeError(msg)


def _dtype_code(t: torch.Tensor, name: str) -> int:
    if t.dtype == torch.float32:
        return ARCQ_F32
    if t.dtype == torch.float16:
        return ARCQ_F16
    raise RuntimeError(f"{name} must be float32 or float16")


def _check_bits(bits: int) -> None:
    _check(bits in (2, 3, 4), "bits must be 2, 3, or 4")


def _f32c(t: torch.Tensor) -> torch.Tensor:
    return t.to(torch.float32).contiguous()


# ---------------------------------------------------------------------------------------------
# bit packing -- EXT/arcq_pack_kernel.cu:94-158
# ---------------------------------------------------------------------------------------------
def pack_codes(codes: torch.Tensor, bits: int) -> torch.Tensor:
    """int codes ``[rows, length]`` -> ``uint8 [rows, ceil(length*bits/8)]`` (LSB-first bitstream)."""
    _check(codes.is_cuda, "codes must be CUDA tensor")
    _check_bits(bits)
    _check(codes.dim() == 2, "codes must have shape [rows, length]")
    c = codes.to(torch.int64).contiguous()
    rows, length = c.shape
    packed = torch.empty((rows, (length * bits + 7) // 8), dtype=torch.uint8, device=c.device)
    with torch.cuda.device(c.device):
        _lib.check(_lib.load().arcq_pack_codes(_ptr(c), _ptr(packed), rows, length, bits, _stream()))
    return packed


def _unpack(packed: torch.Tensor, bits: int, length: int, out_dtype: torch.dtype) -> torch.Tensor:
    _check(packed.is_cuda, "packed must be CUDA tensor")
    _check(packed.dtype == torch.uint8, "packed must be uint8")
    _check_bits(bits)
    _check(packed.dim() == 2, "packed must have shape [rows, packed_cols]")
    length = int(length)
    _check(length >= 0 and (length * bits + 7) // 8 <= packed.shape[1], "length exceeds the packed row")
    p = packed.contiguous()
    rows = p.shape[0]
    # The kernels index rows by ceil(length*bits/8); hand them exactly that row pitch.
    pc = (length * bits + 7) // 8
    if p.shape[1] != pc:
        p = p[:, :pc].contiguous()
    codes = torch.empty((rows, length), dtype=out_dtype, device=p.device)
    fn = _lib.load().arcq_unpack_codes if out_dtype == torch.int64 else _lib.load().arcq_unpack_codes_u8
    with torch.cuda.device(p.device):
        _lib.check(fn(_ptr(p), _ptr(codes), rows, length, bits, _stream()))
    return codes


def unpack_codes(packed: torch.Tensor, bits: int, length: int) -> torch.Tensor:
    """Inverse of :func:`pack_codes`, int64 out (EXT/arcq_pack_kernel.cu:116-136)."""
    return _unpack(packed, bits, length, torch.int64)


def unpack_codes_u8(packed: torch.Tensor, bits: int, length: int) -> torch.Tensor:
    """Inverse of :func:`pack_codes`, uint8 out (EXT/arcq_pack_kernel.cu:138-158)."""
    return _unpack(packed, bits, length, torch.uint8)


# ---------------------------------------------------------------------------------------------
# stage 1 -- EXT/arcq_activation_kernel.cu:188-326
# ---------------------------------------------------------------------------------------------
def _act_quant(x: torch.Tensor, thresholds: torch.Tensor, codebook: torch.Tensor, bits: int, group_size: int,
               want_packed: bool = False, want_u8: bool = False, want_meta: bool = False,
               x_hat: Optional[torch.Tensor] = None, strict_f32: bool = True, eps: float = 1.0e-6):
    _check(x.is_cuda, "x must be CUDA tensor")
    _check(thresholds.is_cuda, "thresholds must be CUDA tensor")
    _check(codebook.is_cuda, "codebook must be CUDA tensor")
    _check_bits(bits)
    _check(x.dim() == 2, "x must have shape [rows, cols]")
    if strict_f32:
        _check(x.dtype == torch.float32, "x must be float32")
    _check(thresholds.dtype == torch.float32, "thresholds must be float32")
    _check(codebook.dtype == torch.float32, "codebook must be float32")
    group_size = int(group_size)
    _check(group_size > 0 and x.shape[1] % group_size == 0, "in_features must be divisible by group_size")
    _check(codebook.numel() == (1 << bits), f"codebook must have {1 << bits} entries for {bits}-bit codes")
    _check(thresholds.numel() == codebook.numel() - 1, "thresholds must have one entry fewer than the codebook")
    x = x.contiguous()
    thresholds = thresholds.contiguous()
    codebook = codebook.contiguous()
    rows, cols = x.shape
    groups = cols // group_size
    dev = x.device
    packed = torch.empty((rows, (cols * bits + 7) // 8), dtype=torch.uint8, device=dev) if want_packed else None
    codes = torch.empty((rows, cols), dtype=torch.uint8, device=dev) if want_u8 else None
    center = torch.empty((rows, groups), dtype=torch.float32, device=dev) if want_meta else None
    scale = torch.empty((rows, groups), dtype=torch.float32, device=dev) if want_meta else None
    code_sum = torch.empty((rows, groups), dtype=torch.float32, device=dev) if want_meta else None
    with torch.cuda.device(dev):
        _lib.check(_lib.load().arcq_act_quant(
            _ptr(x), _dtype_code(x, "x"), _ptr(thresholds), _ptr(codebook), _ptr(packed), _ptr(codes), _ptr(center),
            _ptr(scale), _ptr(code_sum), _ptr(x_hat), _dtype_code(x_hat, "x_hat") if x_hat is not None else ARCQ_F32,
            rows, cols, bits, group_size, float(eps), _stream()))
    return packed, codes, center, scale, code_sum


def quantize_activation(x: torch.Tensor, thresholds: torch.Tensor, codebook: torch.Tensor, bits: int,
                        group_size: int) -> List[torch.Tensor]:
    """-> ``[packed u8 [rows, cols*bits/8], center, scale, code_sum f32 [rows, groups]]``
    (EXT/arcq_activation_kernel.cu:188-237)."""
    packed, _, center, scale, code_sum = _act_quant(x, thresholds, codebook, bits, group_size, want_packed=True,
                                                    want_meta=True)
    return [packed, center, scale, code_sum]


def quantize_activation_u8(x: torch.Tensor, thresholds: torch.Tensor, codebook: torch.Tensor, bits: int,
                           group_size: int) -> List[torch.Tensor]:
    """-> ``[codes u8 [rows, cols], center, scale, code_sum]`` (EXT/arcq_activation_kernel.cu:239-285)."""
    _, codes, center, scale, code_sum = _act_quant(x, thresholds, codebook, bits, group_size, want_u8=True,
                                                   want_meta=True)
    return [codes, center, scale, code_sum]


def quantize_activation_dequant(x: torch.Tensor, thresholds: torch.Tensor, codebook: torch.Tensor, bits: int,
                                group_size: int) -> torch.Tensor:
    """-> ``x_hat f32 [rows, cols]`` (EXT/arcq_activation_kernel.cu:287-326)."""
    _check(x.is_cuda, "x must be CUDA tensor")
    _check(x.dim() == 2, "x must have shape [rows, cols]")
    _check(x.dtype == torch.float32, "x must be float32")
    x = x.contiguous()
    x_hat = torch.empty_like(x)
    _act_quant(x, thresholds, codebook, bits, group_size, x_hat=x_hat)
    return x_hat


def dequant_activation_hip(x: torch.Tensor, thresholds: torch.Tensor, codebook: torch.Tensor, group_size: int,
                           out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Fused quantize+reconstruct, fp16 or fp32, optionally in place (``out=x``).

    Same contract as ``dequant_activation_triton`` (FQ/arcq_packed_triton.py:181-215), including its
    ``out`` checks; statistics are always taken in fp32, also for fp16 input.
    """
    _check(x.dim() == 2, "x must have shape [rows, cols]")
    x = x.contiguous()
    thresholds = thresholds.contiguous().float()
    codebook = codebook.contiguous().float()
    levels = codebook.numel()
    bits = levels.bit_length() - 1
    if out is None:
        out = torch.empty_like(x)
    else:
        if out.shape != x.shape:
            raise ValueError(f"dequant_activation out shape {tuple(out.shape)} != input shape {tuple(x.shape)}")
        if out.dtype != x.dtype:
            raise ValueError(f"dequant_activation out dtype {out.dtype} != input dtype {x.dtype}")
        if not out.is_contiguous():
            raise ValueError("dequant_activation out must be contiguous")
    _act_quant(x, thresholds, codebook, bits, group_size, x_hat=out, strict_f32=False)
    return out


# ---------------------------------------------------------------------------------------------
# stage 2 -- FQ/arcq_packed_triton.py:77-120
# ---------------------------------------------------------------------------------------------
def unpack_weight_hip(packed: torch.Tensor, codebook: torch.Tensor, center: torch.Tensor, scale: torch.Tensor,
                      code_sum: torch.Tensor, bits: int, group_size: int,
                      out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """packed codes + metadata -> fp16 weight ``[out_f, in_f]``.

    Same contract as ``unpack_weight_triton``: ``out`` may be a larger flat fp16 buffer shared by all
    layers (FQ/arcq_packed_on_the_fly.py:149-157); the first ``out_f*in_f`` elements are written and the
    buffer itself is returned.
    """
    _check(packed.is_cuda, "packed must be CUDA tensor")
    _check(packed.dtype == torch.uint8, "packed must be uint8")
    _check_bits(bits)
    out_f = packed.shape[0]
    groups = center.shape[1]
    in_f = groups * int(group_size)
    _check(packed.shape[1] == (in_f * bits + 7) // 8, "packed row length does not match in_features*bits/8")
    packed = packed.contiguous()
    codebook, center, scale, code_sum = _f32c(codebook), _f32c(center), _f32c(scale), _f32c(code_sum)
    if out is None:
        out = torch.empty((out_f, in_f), dtype=torch.float16, device=packed.device)
    else:
        _check(out.is_cuda and out.is_contiguous() and out.numel() >= out_f * in_f, "out buffer too small")
        _check(out.dtype in (torch.float16, torch.float32), "out must be float16 or float32")
    with torch.cuda.device(packed.device):
        _lib.check(_lib.load().arcq_weight_dequant(
            _ptr(packed), _ptr(codebook), _ptr(center), _ptr(scale), _ptr(code_sum), _ptr(out),
            _dtype_code(out, "out"), out_f, in_f, bits, int(group_size), _stream()))
    return out


# Import-compatible aliases for code written against FQ/arcq_packed_triton.py.
dequant_activation_triton = dequant_activation_hip
unpack_weight_triton = unpack_weight_hip


# ---------------------------------------------------------------------------------------------
# stages 2+3 fused / whole layer -- no counterpart function in the reference; they replace the
# unpack + F.linear pair at FQ/arcq_packed_on_the_fly.py:148-160
# ---------------------------------------------------------------------------------------------
def linear_fused(x_hat: torch.Tensor, packed_w: torch.Tensor, w_codebook: torch.Tensor, w_center: torch.Tensor,
                 w_scale: torch.Tensor, w_code_sum: torch.Tensor, bias: Optional[torch.Tensor], bits: int,
                 group_size: int, out_dtype: torch.dtype = torch.float16,
                 w_hat_ws: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``y = x_hat @ w_hat.T + bias`` with ``w_hat`` rebuilt from packed codes inside the GEMM.  ``w_hat_ws``
    (fp16, at least N*K elements; the role of the reference module's ``_weight_buffer``) lets shapes that would
    repeat the reconstruction in many workgroups rebuild the weights once instead; ``y`` is the same either way."""
    _check(x_hat.is_cuda and packed_w.is_cuda, "x_hat and packed_w must be CUDA tensors")
    _check(x_hat.dim() == 2 and x_hat.dtype == torch.float16, "x_hat must be float16 [M, K]")
    _check(packed_w.dtype == torch.uint8 and packed_w.dim() == 2, "packed_w must be uint8 [N, K*bits/8]")
    _check_bits(bits)
    x_hat = x_hat.contiguous()
    m, k = x_hat.shape
    n = packed_w.shape[0]
    _check(packed_w.shape[1] == (k * bits + 7) // 8, "packed_w row length does not match K*bits/8")
    y = torch.empty((m, n), dtype=out_dtype, device=x_hat.device)
    b = None if bias is None or bias.numel() == 0 else _f32c(bias)
    w = [packed_w.contiguous(), _f32c(w_codebook), _f32c(w_center), _f32c(w_scale), _f32c(w_code_sum)]
    _check_w_ws(w_hat_ws, n, k)
    with torch.cuda.device(x_hat.device):
        _lib.check(_lib.load().arcq_linear_fused_ws(
            _ptr(x_hat), *[_ptr(t) for t in w], _ptr(b), _ptr(w_hat_ws), _ptr(y), _dtype_code(y, "y"),
            m, n, k, bits, int(group_size), _stream()))
    return y


def _check_w_ws(w_hat_ws: Optional[torch.Tensor], n: int, k: int) -> None:
    if w_hat_ws is not None:
        _check(w_hat_ws.is_cuda and w_hat_ws.dtype == torch.float16 and w_hat_ws.is_contiguous()
               and w_hat_ws.numel() >= n * k, "w_hat_ws must be a contiguous float16 CUDA buffer of at least N*K elements")


def linear_otf(x: torch.Tensor, a_thresholds: torch.Tensor, a_codebook: torch.Tensor, packed_w: torch.Tensor,
               w_codebook: torch.Tensor, w_center: torch.Tensor, w_scale: torch.Tensor, w_code_sum: torch.Tensor,
               bias: Optional[torch.Tensor], bits: int, group_size: int, out_dtype: torch.dtype = torch.float16,
               x_hat_ws: Optional[torch.Tensor] = None, w_hat_ws: Optional[torch.Tensor] = None,
               scratch: bool = False) -> torch.Tensor:
    """Whole packed on-the-fly layer on ``x [M, K]`` (fp16 or fp32): stage 1 into ``x_hat_ws`` (fp16
    ``[M, K]``, allocated if not given), then the fused GEMM (``w_hat_ws``: see ``linear_fused``).

    With ``scratch=True`` or a ``w_hat_ws`` both workspaces are scratch only: ``y`` is the same bit for bit, but
    ``x_hat_ws`` may afterwards hold ``x_hat`` in the library's 32-row block layout instead of row-major (the
    faster path from 512 rows on).  Otherwise ``x_hat_ws`` holds ``x_hat`` row-major after the call."""
    _check(x.is_cuda and packed_w.is_cuda, "x and packed_w must be CUDA tensors")
    _check(x.dim() == 2, "x must have shape [M, K]")
    _check_bits(bits)
    x = x.contiguous()
    m, k = x.shape
    n = packed_w.shape[0]
    _check(packed_w.shape[1] == (k * bits + 7) // 8, "packed_w row length does not match K*bits/8")
    if x_hat_ws is None:
        x_hat_ws = torch.empty((m, k), dtype=torch.float16, device=x.device)
    else:
        _check(x_hat_ws.dtype == torch.float16 and x_hat_ws.is_contiguous() and x_hat_ws.numel() >= m * k,
               "x_hat_ws must be a contiguous float16 buffer of at least M*K elements")
    y = torch.empty((m, n), dtype=out_dtype, device=x.device)
    b = None if bias is None or bias.numel() == 0 else _f32c(bias)
    a = [_f32c(a_thresholds), _f32c(a_codebook)]
    w = [packed_w.contiguous(), _f32c(w_codebook), _f32c(w_center), _f32c(w_scale), _f32c(w_code_sum)]
    _check_w_ws(w_hat_ws, n, k)
    with torch.cuda.device(x.device):
        if scratch or w_hat_ws is not None:
            _lib.check(_lib.load().arcq_linear_otf_ws(
                _ptr(x), _dtype_code(x, "x"), *[_ptr(t) for t in a], *[_ptr(t) for t in w], _ptr(b), _ptr(x_hat_ws),
                _ptr(w_hat_ws), _ptr(y), _dtype_code(y, "y"), m, n, k, bits, int(group_size), _stream()))
        else:
            _lib.check(_lib.load().arcq_linear_otf(
                _ptr(x), _dtype_code(x, "x"), *[_ptr(t) for t in a], *[_ptr(t) for t in w], _ptr(b), _ptr(x_hat_ws),
                _ptr(y), _dtype_code(y, "y"), m, n, k, bits, int(group_size), _stream()))
    return y


def quantize_activation_blocked(x: torch.Tensor, thresholds: torch.Tensor, codebook: torch.Tensor, bits: int,
                                out: Optional[torch.Tensor] = None, weights=None,
                                w_hat: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Stage 1 (group size 64) with ``x_hat`` written as fp16 in the 32-row block layout
    ``[M/32, K/8, 32, 8]`` that ``linear_fused_blocked`` reads (a last block of ``r = M % 32`` rows follows as
    ``[K/8, r, 8]``); same values as ``dequant_activation_hip``.

    ``weights=(packed_w, w_codebook, w_center, w_scale, w_code_sum)`` with ``w_hat`` (fp16, N*K elements): the same
    launch also reconstructs the layer's weights into ``w_hat`` (what ``unpack_weight_hip`` would write)."""
    _check(x.is_cuda and x.dim() == 2, "x must be a CUDA tensor [M, K]")
    _check_bits(bits)
    x = x.contiguous()
    m, k = x.shape
    _check(k % 64 == 0, "the block layout needs K divisible by 64")
    if out is None:      # whole blocks: [M/32, K/8, 32, 8]; a ragged last block is stored compactly behind them: flat
        shape = (m // 32, k // 8, 32, 8) if m % 32 == 0 else (m * k,)
        out = torch.empty(shape, dtype=torch.float16, device=x.device)
    else:
        _check(out.is_cuda and out.dtype == torch.float16 and out.is_contiguous() and out.numel() >= m * k,
               "out must be a contiguous float16 CUDA buffer of at least M*K elements")
    thr, cbk = _f32c(thresholds), _f32c(codebook)
    with torch.cuda.device(x.device):
        if weights is None:
            _lib.check(_lib.load().arcq_act_quant_blocked(
                _ptr(x), _dtype_code(x, "x"), _ptr(thr), _ptr(cbk), _ptr(out), m, k, bits, 1.0e-6, _stream()))
        else:
            packed_w = weights[0].contiguous()
            n = packed_w.shape[0]
            _check(packed_w.is_cuda and packed_w.dtype == torch.uint8 and packed_w.dim() == 2
                   and packed_w.shape[1] == (k * bits + 7) // 8, "packed_w must be uint8 [N, K*bits/8]")
            _check(w_hat is not None, "weights need a w_hat buffer")
            _check_w_ws(w_hat, n, k)
            meta = [_f32c(t) for t in weights[1:]]
            _lib.check(_lib.load().arcq_act_quant_blocked_with_weights(
                _ptr(x), _dtype_code(x, "x"), _ptr(thr), _ptr(cbk), _ptr(out), m, k, bits, 1.0e-6,
                _ptr(packed_w), *[_ptr(t) for t in meta], _ptr(w_hat), n, _stream()))
    return out


def quantize_activation_blocked_ln(x: torch.Tensor, ln_weight: torch.Tensor, ln_bias: torch.Tensor, ln_eps: float,
                                   thresholds: torch.Tensor, codebook: torch.Tensor, bits: int,
                                   out: Optional[torch.Tensor] = None, weights=None,
                                   w_hat: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``quantize_activation_blocked`` of ``LayerNorm(x)`` (over the last dimension, result rounded to ``x``'s
    dtype) in one launch; ``64 <= K <= 1024``.  ``weights`` / ``w_hat`` as there."""
    _check(x.is_cuda and x.dim() == 2, "x must be a CUDA tensor [M, K]")
    _check_bits(bits)
    x = x.contiguous()
    m, k = x.shape
    _check(k % 64 == 0 and 64 <= k <= 1024, "the fused LayerNorm needs K divisible by 64 and at most 1024")
    if out is None:
        shape = (m // 32, k // 8, 32, 8) if m % 32 == 0 else (m * k,)
        out = torch.empty(shape, dtype=torch.float16, device=x.device)
    else:
        _check(out.is_cuda and out.dtype == torch.float16 and out.is_contiguous() and out.numel() >= m * k,
               "out must be a contiguous float16 CUDA buffer of at least M*K elements")
    thr, cbk, g, b = _f32c(thresholds), _f32c(codebook), _f32c(ln_weight), _f32c(ln_bias)
    _check(g.numel() == k and b.numel() == k, "ln_weight and ln_bias must have K elements")
    wp = [0, 0, 0, 0, 0, 0, 0]
    keep = None
    if weights is not None:
        packed_w = weights[0].contiguous()
        n = packed_w.shape[0]
        _check(w_hat is not None, "weights need a w_hat buffer")
        _check_w_ws(w_hat, n, k)
        keep = [packed_w] + [_f32c(t) for t in weights[1:]]
        wp = [_ptr(t) for t in keep] + [_ptr(w_hat), n]
    with torch.cuda.device(x.device):
        _lib.check(_lib.load().arcq_act_quant_blocked_ln(
            _ptr(x), _dtype_code(x, "x"), _ptr(g), _ptr(b), float(ln_eps), _ptr(thr), _ptr(cbk), _ptr(out), m, k, bits,
            1.0e-6, *wp, _stream()))
    return out


def quantize_patches(img: torch.Tensor, thresholds: torch.Tensor, codebook: torch.Tensor, bits: int,
                     blocked: bool = False) -> torch.Tensor:
    """Stage 1 of a quantized 16 x 16 patch convolution on three channels (``arcq_act_quant_patches``): every pixel's
    channels are one group; returns the reconstructed patch rows ``[B * patches, 768]`` fp16 (column order ``(c, i, j)``
    of ``conv.weight.reshape``), or with ``blocked`` the flat 32-row block layout ``linear_fused_blocked`` reads."""
    _check(img.is_cuda and img.dim() == 4 and img.shape[1] == 3 and img.dtype in (torch.float16, torch.float32),
           "img must be a CUDA fp16 or fp32 tensor [B, 3, H, W]")
    _check_bits(bits)
    b, _, h, w = img.shape
    _check(h % 16 == 0 and w % 16 == 0, "image sides must be multiples of 16")
    img = img.contiguous()
    m = b * (h // 16) * (w // 16)
    out = torch.empty(m * 768 if blocked else (m, 768), dtype=torch.float16, device=img.device)
    with torch.cuda.device(img.device):
        _lib.check(_lib.load().arcq_act_quant_patches(_ptr(img), _dtype_code(img, "img"), _ptr(_f32c(thresholds)),
                                                      _ptr(_f32c(codebook)), _ptr(out), b, 3, h, w, 16, bits, 1.0e-6,
                                                      int(bool(blocked)), _stream()))
    return out


def patch_embed_fwd(img: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor], cls_token: torch.Tensor,
                    pos_embed: torch.Tensor) -> torch.Tensor:
    """Front end of a ViT in one launch (``arcq_patch_embed_fwd``): 16 x 16 stride-16 patch convolution of ``img``
    ``[B, 3, H, W]`` with ``weight`` ``[N, 3, 16, 16]`` and ``bias``, the class token in front, ``pos_embed`` added ->
    ``[B, 1 + patches, N]``; everything fp16, fp32 accumulation, rounded as the separate torch operations round."""
    _check(img.is_cuda and img.dtype == torch.float16 and img.dim() == 4 and img.shape[1] == 3,
           "img must be a CUDA fp16 tensor [B, 3, H, W]")
    _check(weight.is_cuda and weight.dtype == torch.float16 and weight.dim() == 4 and tuple(weight.shape[1:]) == (3, 16, 16),
           "weight must be a CUDA fp16 tensor [N, 3, 16, 16]")
    _check(weight.shape[0] % 32 == 0, "the embedding width must be a multiple of 32")
    b, _, h, w_ = img.shape
    n = weight.shape[0]
    tokens = 1 + (h // 16) * (w_ // 16)
    _check(h % 16 == 0 and w_ % 16 == 0, "image sides must be multiples of 16")
    _check(cls_token.numel() == n and pos_embed.numel() == tokens * n, "cls_token / pos_embed do not match the patch grid")
    for t in (cls_token, pos_embed, bias):
        _check(t is None or (t.is_cuda and t.dtype == torch.float16), "bias, cls_token and pos_embed must be CUDA fp16 tensors")
    img, weight = img.contiguous(), weight.contiguous()
    cls_c, pos_c = cls_token.contiguous(), pos_embed.contiguous()
    bias_c = None if bias is None else bias.contiguous()
    out = torch.empty((b, tokens, n), dtype=torch.float16, device=img.device)
    with torch.cuda.device(img.device):
        _lib.check(_lib.load().arcq_patch_embed_fwd(_ptr(img), _ptr(weight), _ptr(bias_c), _ptr(cls_c), _ptr(pos_c), _ptr(out),
                                                    b, h, w_, 16, n, _stream()))
    return out


def attention_fwd(qkv: torch.Tensor, heads: int, scale: Optional[float] = None,
                  out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Softmax attention on the qkv layer's output ``[B, n, 3 C]`` fp16 (q, k, v of head h at columns
    ``(0|1|2) C + 64 h``) -> ``[B, n, C]`` fp16, the proj layer's input, in one launch with no reshaping copies
    (``arcq_attention_fwd``: head dimension 64, at most 256 tokens).  ``scale`` defaults to ``1 / sqrt(64)``."""
    _check(qkv.is_cuda and qkv.dtype == torch.float16 and qkv.dim() == 3, "qkv must be a CUDA fp16 tensor [B, n, 3 C]")
    _check(qkv.is_contiguous(), "qkv must be contiguous")
    b, n, c3 = qkv.shape
    _check(c3 % 3 == 0 and (c3 // 3) == heads * 64, f"head dimension must be 64 (C={c3 // 3}, heads={heads})")
    c = c3 // 3
    if out is None:
        out = torch.empty((b, n, c), dtype=torch.float16, device=qkv.device)
    else:
        _check(out.is_cuda and out.dtype == torch.float16 and out.is_contiguous() and out.numel() == b * n * c,
               "out must be a contiguous CUDA fp16 tensor of B * n * C elements")
    with torch.cuda.device(qkv.device):
        _lib.check(_lib.load().arcq_attention_fwd(_ptr(qkv), _ptr(out), b, n, heads, 64,
                                                  0.125 if scale is None else float(scale), _stream()))
    return out.view(b, n, c)


def xhat_layout(m: int) -> int:
    """Layout of an ``x_hat`` passed between two chained layers (``linear_otf_ex`` with ``next_quant`` / ``x_is_xhat``):
    0 = row-major, 1 = the 32-row block layout."""
    return int(_lib.load().arcq_xhat_layout(int(m)))


def linear_otf_ex(x: torch.Tensor, a_thresholds: torch.Tensor, a_codebook: torch.Tensor, packed_w: torch.Tensor,
                  w_codebook: torch.Tensor, w_center: torch.Tensor, w_scale: torch.Tensor, w_code_sum: torch.Tensor,
                  bias: Optional[torch.Tensor], bits: int, group_size: int, out_dtype: torch.dtype = torch.float16,
                  layernorm=None, gelu: bool = False, residual: Optional[torch.Tensor] = None,
                  x_hat_ws: Optional[torch.Tensor] = None, w_hat_ws: Optional[torch.Tensor] = None,
                  next_quant=None, x_is_xhat: bool = False) -> torch.Tensor:
    """``residual + gelu(linear(stage1(LayerNorm(x))))`` with the optional parts fused into the layer's two launches
    (``arcq_linear_otf_ex``): ``layernorm = (weight, bias, eps)`` or None, ``residual`` ``[M, N]`` of ``out_dtype`` or
    None.  Below 512 rows the whole layer with its options is one launch (or stage 1 + the split-K kernel with the
    GELU / residual in its epilogue); from 512 rows on the block-layout path.  Raises ``RuntimeError`` where the
    library does not fuse (LayerNorm with K > 1024 from 512 rows on, K > 1536 below).
    ``next_quant = (thresholds, codebook)`` of the layer that consumes the output: the result is that layer's ``x_hat``
    (stage 1 applied to the rounded output) in the layout ``xhat_layout(M)`` instead of the output itself; that layer is
    then called with ``x_is_xhat=True`` (its own stage 1 is skipped)."""
    _check(x.is_cuda and packed_w.is_cuda, "x and packed_w must be CUDA tensors")
    _check(x.dim() == 2, "x must have shape [M, K]")
    _check_bits(bits)
    x = x.contiguous()
    m, k = x.shape
    n = packed_w.shape[0]
    _check(packed_w.shape[1] == (k * bits + 7) // 8, "packed_w row length does not match K*bits/8")
    if x_hat_ws is None:
        x_hat_ws = torch.empty(m * k, dtype=torch.float16, device=x.device)
    y = torch.empty((m, n), dtype=out_dtype, device=x.device)
    keep = [_f32c(a_thresholds), _f32c(a_codebook), packed_w.contiguous(), _f32c(w_codebook), _f32c(w_center),
            _f32c(w_scale), _f32c(w_code_sum), None if bias is None or bias.numel() == 0 else _f32c(bias)]
    a = _lib.LinearExArgs()
    a.struct_size = ctypes.sizeof(_lib.LinearExArgs)
    a.x_dtype, a.y_dtype = _dtype_code(x, "x"), _dtype_code(y, "y")
    a.bits, a.group_size, a.M, a.N, a.K = bits, int(group_size), m, n, k
    a.x = _ptr(x)
    if layernorm is not None:
        lw, lb, eps = layernorm
        lw, lb = _f32c(lw), _f32c(lb)
        keep += [lw, lb]
        a.producer, a.ln_weight, a.ln_bias, a.ln_eps = _lib.ARCQ_PRODUCER_LAYERNORM, _ptr(lw), _ptr(lb), float(eps)
    if x_is_xhat:
        _check(layernorm is None and x.dtype == torch.float16, "x_is_xhat: x must be float16 and takes no LayerNorm")
        a.producer = _lib.ARCQ_PRODUCER_XHAT
    if next_quant is not None:
        nt, nc = _f32c(next_quant[0]), _f32c(next_quant[1])
        keep += [nt, nc]
        a.next_a_thresholds, a.next_a_codebook = _ptr(nt), _ptr(nc)
    a.activation = _lib.ARCQ_ACT_GELU if gelu else _lib.ARCQ_ACT_NONE
    (a.a_thresholds, a.a_codebook, a.packed_w, a.w_codebook, a.w_center, a.w_scale, a.w_code_sum,
     a.bias) = [_ptr(t) or None for t in keep[:8]]
    if residual is not None:
        _check(residual.is_cuda and residual.dtype == out_dtype and residual.is_contiguous()
               and tuple(residual.shape) == (m, n), "residual must be a contiguous [M, N] tensor of the output dtype")
        a.residual = _ptr(residual)
    _check_w_ws(w_hat_ws, n, k)
    a.x_hat_ws, a.w_hat_ws, a.y = _ptr(x_hat_ws), _ptr(w_hat_ws) or None, _ptr(y)
    with torch.cuda.device(x.device):
        _lib.check(_lib.load().arcq_linear_otf_ex(ctypes.byref(a), _stream()))
    return y


# ---------------------------------------------------------------------------------------------
# the layer with FP8 operands -- no counterpart in the reference; a faster, less exact stage 3
# ---------------------------------------------------------------------------------------------
FP8_MAX = 448.0          # largest finite OCP E4M3 value


def quantize_activation_fp8(x: torch.Tensor, thresholds: torch.Tensor, codebook: torch.Tensor, bits: int,
                            out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Stage 1 with the reconstruction rounded to FP8 (``torch.float8_e4m3fn``, row-major ``[M, K]``) instead of fp16;
    group size 64.  Codes, ``mu`` and ``s`` are those of ``quantize_activation``."""
    _check(x.is_cuda and x.dim() == 2, "x must be a CUDA tensor of shape [M, K]")
    _check_bits(bits)
    x = x.contiguous()
    m, k = x.shape
    if out is None:
        out = torch.empty((m, k), dtype=torch.float8_e4m3fn, device=x.device)
    else:
        _check(out.dtype == torch.float8_e4m3fn and out.is_contiguous() and out.numel() >= m * k,
               "out must be a contiguous float8_e4m3fn buffer of at least M*K elements")
    thresholds, codebook = _f32c(thresholds), _f32c(codebook)
    with torch.cuda.device(x.device):
        _lib.check(_lib.load().arcq_act_quant_fp8(_ptr(x), _dtype_code(x, "x"), _ptr(thresholds), _ptr(codebook), _ptr(out),
                                                  m, k, bits, 1.0e-6, _stream()))
    return out


def fp8_weight_multiplier(w_codebook: torch.Tensor, w_center: torch.Tensor, w_scale: torch.Tensor,
                          w_code_sum: torch.Tensor) -> float:
    """Power of two that moves a layer's reconstructed weights into FP8's normal range: the largest one that keeps a
    bound on ``|w_hat|`` (``|center| + |scale| (max |cb| + |code_sum| / 64)`` over all groups) at or below half the
    largest FP8 value.  Reads the metadata back to the host: compute it once per layer."""
    cb = float(w_codebook.abs().max())
    bound = float((w_center.abs() + w_scale.abs() * (cb + w_code_sum.abs() / 64.0)).max())
    if not bound > 0.0:
        return 1.0
    import math
    return float(2.0 ** math.floor(math.log2(FP8_MAX / 2.0 / bound)))


def unpack_weight_fp8(packed: torch.Tensor, codebook: torch.Tensor, center: torch.Tensor, scale: torch.Tensor,
                      code_sum: torch.Tensor, bits: int, w_mult: float, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Stage 2 with the weights rounded to FP8: ``fp8(w_mult * w_hat)``, row-major ``[N, K]``; group size 64."""
    _check(packed.is_cuda and packed.dtype == torch.uint8, "packed must be a CUDA uint8 tensor")
    _check_bits(bits)
    n = packed.shape[0]
    k = center.shape[1] * 64
    _check(packed.shape[1] == (k * bits + 7) // 8, "packed row length does not match in_features*bits/8")
    if out is None:
        out = torch.empty((n, k), dtype=torch.float8_e4m3fn, device=packed.device)
    else:
        _check(out.dtype == torch.float8_e4m3fn and out.is_contiguous() and out.numel() >= n * k,
               "out must be a contiguous float8_e4m3fn buffer of at least N*K elements")
    packed = packed.contiguous()
    codebook, center, scale, code_sum = _f32c(codebook), _f32c(center), _f32c(scale), _f32c(code_sum)
    with torch.cuda.device(packed.device):
        _lib.check(_lib.load().arcq_weight_dequant_fp8(_ptr(packed), _ptr(codebook), _ptr(center), _ptr(scale),
                                                       _ptr(code_sum), _ptr(out), n, k, bits, 64, float(w_mult), _stream()))
    return out


def fp8_padded_k(k: int) -> int:
    """Row length of the FP8 GEMM's operands: ``k`` rounded up to a multiple of 128 (the padding is zero)."""
    return (int(k) + 127) // 128 * 128


def linear_otf_fp8(x: torch.Tensor, a_thresholds: torch.Tensor, a_codebook: torch.Tensor, packed_w: torch.Tensor,
                   w_codebook: torch.Tensor, w_center: torch.Tensor, w_scale: torch.Tensor, w_code_sum: torch.Tensor,
                   bias: Optional[torch.Tensor], bits: int, out_dtype: torch.dtype = torch.float16,
                   w_mult: Optional[float] = None, x8_ws: Optional[torch.Tensor] = None,
                   w8_ws: Optional[torch.Tensor] = None) -> torch.Tensor:
    """The packed on-the-fly layer with FP8 operands (``arcq_linear_otf_fp8``, two launches): stage 1 and stage 2 as in
    ``linear_otf`` but rounded to FP8 (the weights first multiplied by ``w_mult``), then the library's own FP8 MFMA GEMM
    with fp32 accumulation, ``y = x8 w8^T / w_mult + bias``.  Faster where the layer is bound by the matrix units (the
    large models), NOT bit-compatible with the reference: each operand carries a rounding error of up to 2^-4 relative
    (fp16: 2^-11).  Group size 64.  ``x8_ws`` / ``w8_ws``: scratch of at least ``M * Kp`` / ``N * Kp`` bytes
    (``Kp = fp8_padded_k(K)``), any 1-byte dtype."""
    _check(x.is_cuda and x.dim() == 2, "x must be a CUDA tensor of shape [M, K]")
    _check_bits(bits)
    x = x.contiguous()
    m, k = x.shape
    n = packed_w.shape[0]
    _check(k % 64 == 0 and k > 0, "in_features must be a positive multiple of the group size 64")
    _check(packed_w.shape[1] == (k * bits + 7) // 8, "packed_w row length does not match K*bits/8")
    if w_mult is None:
        w_mult = fp8_weight_multiplier(w_codebook, w_center, w_scale, w_code_sum)
    kp = fp8_padded_k(k)
    if x8_ws is None:
        x8_ws = torch.empty(max(m * kp, 1), dtype=torch.uint8, device=x.device)
    if w8_ws is None:
        w8_ws = torch.empty(max(n * kp, 1), dtype=torch.uint8, device=x.device)
    for t, need, name in ((x8_ws, m * kp, "x8_ws"), (w8_ws, n * kp, "w8_ws")):
        _check(t.is_cuda and t.is_contiguous() and t.element_size() == 1 and t.numel() >= need,
               f"{name} must be a contiguous 1-byte CUDA buffer of at least {need} elements")
    y = torch.empty((m, n), dtype=out_dtype, device=x.device)
    a = [_f32c(a_thresholds), _f32c(a_codebook)]
    w = [packed_w.contiguous(), _f32c(w_codebook), _f32c(w_center), _f32c(w_scale), _f32c(w_code_sum)]
    b = None if bias is None or bias.numel() == 0 else _f32c(bias)
    with torch.cuda.device(x.device):
        _lib.check(_lib.load().arcq_linear_otf_fp8(
            _ptr(x), _dtype_code(x, "x"), *[_ptr(t) for t in a], *[_ptr(t) for t in w], _ptr(b), float(w_mult),
            _ptr(x8_ws), _ptr(w8_ws), _ptr(y), _dtype_code(y, "y"), m, n, k, bits, _stream()))
    return y


def linear_otf_fp8_library_gemm(x: torch.Tensor, a_thresholds: torch.Tensor, a_codebook: torch.Tensor,
                                packed_w: torch.Tensor, w_codebook: torch.Tensor, w_center: torch.Tensor,
                                w_scale: torch.Tensor, w_code_sum: torch.Tensor, bias: Optional[torch.Tensor], bits: int,
                                out_dtype: torch.dtype = torch.float16, w_mult: Optional[float] = None,
                                x8_ws: Optional[torch.Tensor] = None, w8_ws: Optional[torch.Tensor] = None) -> torch.Tensor:
    """The same layer with the product left to the vendor library's FP8 GEMM (``torch._scaled_mm``) on row-major
    operands, three launches: kept as a timing and cross-check reference for ``linear_otf_fp8``, not used by the
    modules."""
    _check(x.is_cuda and x.dim() == 2, "x must be a CUDA tensor of shape [M, K]")
    m, k = x.shape
    n = packed_w.shape[0]
    _check(k % 16 == 0 and n % 16 == 0, "the library's FP8 GEMM needs K and N to be multiples of 16")
    if w_mult is None:
        w_mult = fp8_weight_multiplier(w_codebook, w_center, w_scale, w_code_sum)
    x8 = quantize_activation_fp8(x, a_thresholds, a_codebook, bits, out=x8_ws)
    w8 = unpack_weight_fp8(packed_w, w_codebook, w_center, w_scale, w_code_sum, bits, w_mult, out=w8_ws)
    x8 = x8.view(-1)[:m * k].view(m, k)
    w8 = w8.view(-1)[:n * k].view(n, k)
    one = torch.ones((), dtype=torch.float32, device=x.device)
    inv = torch.full((), 1.0 / float(w_mult), dtype=torch.float32, device=x.device)
    has_bias = bias is not None and bias.numel() > 0
    if has_bias and out_dtype == torch.float16:      # (the library adds a bias of the output's type; fp16 only)
        return torch._scaled_mm(x8, w8.t(), scale_a=one, scale_b=inv, bias=bias.to(torch.float16), out_dtype=out_dtype)
    y = torch._scaled_mm(x8, w8.t(), scale_a=one, scale_b=inv, out_dtype=out_dtype)
    return y + bias.to(out_dtype) if has_bias else y


def linear_fused_blocked(x_hat_blocked: torch.Tensor, m: int, k: int, packed_w: torch.Tensor, w_codebook: torch.Tensor,
                         w_center: torch.Tensor, w_scale: torch.Tensor, w_code_sum: torch.Tensor,
                         bias: Optional[torch.Tensor], bits: int, out_dtype: torch.dtype = torch.float16,
                         w_hat_ws: Optional[torch.Tensor] = None, w_hat_ready: bool = False) -> torch.Tensor:
    """``linear_fused`` on ``x_hat`` ``[m, k]`` held in the 32-row block layout (``quantize_activation_blocked``).
    ``w_hat_ready``: ``w_hat_ws`` already holds the reconstructed fp16 weights and is used as is."""
    _check(x_hat_blocked.is_cuda and x_hat_blocked.dtype == torch.float16 and x_hat_blocked.is_contiguous()
           and x_hat_blocked.numel() >= m * k, "x_hat_blocked must be a contiguous float16 CUDA buffer of M*K elements")
    _check(packed_w.is_cuda and packed_w.dtype == torch.uint8 and packed_w.dim() == 2, "packed_w must be uint8 [N, K*bits/8]")
    _check_bits(bits)
    n = packed_w.shape[0]
    _check(packed_w.shape[1] == (k * bits + 7) // 8, "packed_w row length does not match K*bits/8")
    y = torch.empty((m, n), dtype=out_dtype, device=x_hat_blocked.device)
    b = None if bias is None or bias.numel() == 0 else _f32c(bias)
    w = [packed_w.contiguous(), _f32c(w_codebook), _f32c(w_center), _f32c(w_scale), _f32c(w_code_sum)]
    _check_w_ws(w_hat_ws, n, k)
    with torch.cuda.device(x_hat_blocked.device):
        _lib.check(_lib.load().arcq_linear_fused_blocked(
            _ptr(x_hat_blocked), *[_ptr(t) for t in w], _ptr(b), _ptr(w_hat_ws), int(bool(w_hat_ready)), _ptr(y),
            _dtype_code(y, "y"), m, n, k, bits, 64, _stream()))
    return y


# ---------------------------------------------------------------------------------------------
# index-space linears -- EXT/arcq_linear_kernel.cu:206-353
# ---------------------------------------------------------------------------------------------
def arcq_linear_forward(packed_x: torch.Tensor, x_center: torch.Tensor, x_scale: torch.Tensor,
                        x_code_sum: torch.Tensor, packed_w: torch.Tensor, w_center: torch.Tensor,
                        w_scale: torch.Tensor, w_code_sum: torch.Tensor, product_table: torch.Tensor,
                        bias: Optional[torch.Tensor], bits: int, group_size: int, in_features: int,
                        out_features: int) -> torch.Tensor:
    """fp64-accumulated product-table linear on packed codes (EXT/arcq_linear_kernel.cu:206-278)."""
    _check(packed_x.is_cuda, "packed_x must be CUDA tensor")
    _check(packed_w.is_cuda, "packed_w must be CUDA tensor")
    _check(packed_x.dtype == torch.uint8, "packed_x must be uint8")
    _check(packed_w.dtype == torch.uint8, "packed_w must be uint8")
    _check_bits(bits)
    _check(int(in_features) % int(group_size) == 0, "in_features must be divisible by group_size")
    _check(product_table.dtype == torch.float32, "product_table must be float32")
    pc = (int(in_features) * bits + 7) // 8
    _check(packed_x.dim() == 2 and packed_x.shape[1] == pc, "packed_x row length does not match in_features*bits/8")
    _check(packed_w.dim() == 2 and packed_w.shape == (int(out_features), pc),
           "packed_w shape does not match [out_features, in_features*bits/8]")
    rows = packed_x.shape[0]
    levels = product_table.shape[0]
    y = torch.empty((rows, int(out_features)), dtype=torch.float32, device=packed_x.device)
    b = None
    if bias is not None and bias.numel() > 0:
        _check(bias.is_cuda, "bias must be CUDA tensor")
        b = _f32c(bias)
    tensors = [packed_x.contiguous(), _f32c(x_center), _f32c(x_scale), _f32c(x_code_sum), packed_w.contiguous(),
               _f32c(w_center), _f32c(w_scale), _f32c(w_code_sum), _f32c(product_table)]
    with torch.cuda.device(packed_x.device):
        _lib.check(_lib.load().arcq_linear_forward_packed(
            *[_ptr(t) for t in tensors], _ptr(b), _ptr(y), rows, int(out_features), int(in_features), bits,
            int(group_size), levels, _stream()))
    return y


def arcq_linear_forward_u8(x_codes: torch.Tensor, x_center: torch.Tensor, x_scale: torch.Tensor,
                           x_code_sum: torch.Tensor, w_codes: torch.Tensor, w_center: torch.Tensor,
                           w_scale: torch.Tensor, w_code_sum: torch.Tensor, product_table: torch.Tensor,
                           bias: Optional[torch.Tensor], group_size: int) -> torch.Tensor:
    """fp32 product-table linear on byte codes, 32-lane summation order (EXT/arcq_linear_kernel.cu:280-353)."""
    _check(x_codes.is_cuda, "x_codes must be CUDA tensor")
    _check(w_codes.is_cuda, "w_codes must be CUDA tensor")
    _check(x_codes.dtype == torch.uint8, "x_codes must be uint8")
    _check(w_codes.dtype == torch.uint8, "w_codes must be uint8")
    _check(x_codes.dim() == 2, "x_codes must have shape [rows, in_features]")
    _check(w_codes.dim() == 2, "w_codes must have shape [out_features, in_features]")
    _check(x_codes.shape[1] == w_codes.shape[1], "x_codes and w_codes in_features must match")
    _check(x_codes.shape[1] % int(group_size) == 0, "in_features must be divisible by group_size")
    _check(product_table.dtype == torch.float32, "product_table must be float32")
    rows, in_features = x_codes.shape
    out_features = w_codes.shape[0]
    levels = product_table.shape[0]
    y = torch.empty((rows, out_features), dtype=torch.float32, device=x_codes.device)
    b = None
    if bias is not None and bias.numel() > 0:
        _check(bias.is_cuda, "bias must be CUDA tensor")
        b = _f32c(bias)
    tensors = [x_codes.contiguous(), _f32c(x_center), _f32c(x_scale), _f32c(x_code_sum), w_codes.contiguous(),
               _f32c(w_center), _f32c(w_scale), _f32c(w_code_sum), _f32c(product_table)]
    with torch.cuda.device(x_codes.device):
        _lib.check(_lib.load().arcq_linear_forward_u8(
            *[_ptr(t) for t in tensors], _ptr(b), _ptr(y), rows, out_features, in_features, int(group_size), levels,
            _stream()))
    return y
