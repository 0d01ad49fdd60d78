"""CPU oracle for the ARCQ packed quantized-linear path.  TEST INFRASTRUCTURE ONLY.

Only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of
``bench.py`` may import this module; the shipped package never does.  It holds

* ctypes bindings to ``libarcq_oracle.so`` (``arcq_oracle.c``: serial-order,
  IEEE fp32 restatement of the reference's CUDA kernels), and
* torch/numpy restatements of the reference's *torch* paths, which share the
  reduction order of whatever torch build runs them (the reference calls the
  same torch ops, so on one host the two agree bit for bit).

Reference paths are relative to the reference root; ``FQ`` =
``methods/fair_qat_framework/fair_qat``, ``EXT`` = ``FQ/arcq_infer_cuda``,
``Q`` = ``methods/fair_qat_framework/quant``.

Pinning status (tests that pin each function, none of which imports the
reference) is tabulated in ``oracle/README.md``.
"""
from __future__ import annotations

import ctypes
import os
import subprocess
from typing import Dict, Optional, Tuple

import numpy as np
import torch
import torch.nn.functional as F

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libarcq_oracle.so")
_lib = None


def build_c_oracle(force: bool = False) -> str:
    """Compile ``arcq_oracle.c`` with gcc (see ``oracle/Makefile``)."""
    src = os.path.join(_HERE, "arcq_oracle.c")
    stale = (not os.path.exists(_LIB_PATH)) or (os.path.exists(src) and os.path.getmtime(src) > os.path.getmtime(_LIB_PATH))
    if force or stale:
        subprocess.check_call(["make", "-C", _HERE, "-B" if force else "-s", "libarcq_oracle.so"])
    return _LIB_PATH


def _c():
    global _lib
    if _lib is None:
        build_c_oracle()
        lib = ctypes.CDLL(_LIB_PATH)
        lib.oracle_packed_cols.restype = ctypes.c_int64
        lib.oracle_packed_cols.argtypes = [ctypes.c_int64, ctypes.c_int]
        _lib = lib
    return _lib


def check_div_sequence(n: int, seed: int = 1) -> int:
    """Mismatches between the GPU kernel's fma-based divide and IEEE division on ``n`` random inputs."""
    lib = _c()
    lib.oracle_check_div_sequence.restype = ctypes.c_int64
    return int(lib.oracle_check_div_sequence(ctypes.c_int64(n), ctypes.c_uint64(seed)))


def _p(a: Optional[np.ndarray]):
    if a is None:
        return ctypes.c_void_p(0)
    assert a.flags["C_CONTIGUOUS"]
    return ctypes.c_void_p(a.ctypes.data)


def _f32(a) -> np.ndarray:
    if isinstance(a, torch.Tensor):
        a = a.detach().cpu().numpy()
    return np.ascontiguousarray(a, dtype=np.float32)


def _u8(a) -> np.ndarray:
    if isinstance(a, torch.Tensor):
        a = a.detach().cpu().numpy()
    return np.ascontiguousarray(a, dtype=np.uint8)


# --------------------------------------------------------------------------
# Bit layout (a1-a3)
# --------------------------------------------------------------------------
def packed_cols(length: int, bits: int) -> int:
    """``ceil(length*bits/8)`` -- EXT/arcq_pack_kernel.cu:101."""
    return (length * bits + 7) // 8


def pack_codes_c(codes, bits: int) -> np.ndarray:
    """C loop version of EXT/arcq_pack_kernel.cu:38-54."""
    codes = np.ascontiguousarray(codes, dtype=np.int64)
    rows, length = codes.shape
    out = np.empty((rows, packed_cols(length, bits)), dtype=np.uint8)
    _c().oracle_pack_codes(_p(codes), _p(out), ctypes.c_int64(rows), ctypes.c_int64(length), ctypes.c_int(bits))
    return out


def unpack_codes_c(packed, bits: int, length: int) -> np.ndarray:
    """EXT/arcq_pack_kernel.cu:56-72."""
    packed = _u8(packed)
    rows = packed.shape[0]
    out = np.empty((rows, length), dtype=np.int64)
    _c().oracle_unpack_codes(_p(packed), _p(out), ctypes.c_int64(rows), ctypes.c_int64(length), ctypes.c_int(bits))
    return out


def unpack_codes_u8_c(packed, bits: int, length: int) -> np.ndarray:
    """EXT/arcq_pack_kernel.cu:74-90."""
    packed = _u8(packed)
    rows = packed.shape[0]
    out = np.empty((rows, length), dtype=np.uint8)
    _c().oracle_unpack_codes_u8(_p(packed), _p(out), ctypes.c_int64(rows), ctypes.c_int64(length), ctypes.c_int(bits))
    return out


def pack_codes_np(codes, bits: int) -> np.ndarray:
    """Bitstream formulation of the layout FQ/arcq_packed_py.py:8-47 produces.

    Each code contributes its ``bits`` low bits, least significant first, to
    one long little-endian bit string per row; ``np.packbits(bitorder="little")``
    cuts that string into bytes.  Written independently of the C loop so the
    two can pin each other.
    """
    codes = np.asarray(codes).astype(np.int64)
    rows, length = codes.shape
    bit_planes = (codes[:, :, None] >> np.arange(bits)) & 1          # [rows, length, bits] LSB first
    stream = bit_planes.reshape(rows, length * bits).astype(np.uint8)
    pad = packed_cols(length, bits) * 8 - length * bits
    if pad:
        stream = np.concatenate([stream, np.zeros((rows, pad), dtype=np.uint8)], axis=1)
    return np.packbits(stream, axis=1, bitorder="little")


def unpack_codes_np(packed, bits: int, length: int) -> np.ndarray:
    """Inverse of :func:`pack_codes_np` -- FQ/arcq_packed_py.py:50-78."""
    packed = _u8(packed)
    rows = packed.shape[0]
    stream = np.unpackbits(packed, axis=1, bitorder="little")[:, : length * bits]
    planes = stream.reshape(rows, length, bits).astype(np.int64)
    return (planes << np.arange(bits)).sum(axis=-1)


# --------------------------------------------------------------------------
# Stage 1 (a6) -- serial order, C
# --------------------------------------------------------------------------
def act_quant_c(x, thresholds, codebook, bits: int, group_size: int, eps: float = 1e-6,
                fma: bool = True, want_xhat: bool = True) -> Dict[str, np.ndarray]:
    """EXT/arcq_activation_kernel.cu:24-184 in serial order with IEEE divide/sqrt.

    ``x`` may be fp16 or fp32; fp16 is widened exactly before any arithmetic
    (the half chain of FQ/arcq_packed_on_the_fly.py:139 hands fp16 in).
    Returns packed codes, byte codes, center, scale, code_sum and x_hat (fp32,
    not yet rounded to the output dtype).
    """
    x = _f32(x)
    thr, cb = _f32(thresholds), _f32(codebook)
    rows, cols = x.shape
    assert cols % group_size == 0 and cb.size == (1 << bits) and thr.size == cb.size - 1
    groups = cols // group_size
    out = {
        "packed": np.empty((rows, packed_cols(cols, bits)), dtype=np.uint8),
        "codes": np.empty((rows, cols), dtype=np.uint8),
        "center": np.empty((rows, groups), dtype=np.float32),
        "scale": np.empty((rows, groups), dtype=np.float32),
        "code_sum": np.empty((rows, groups), dtype=np.float32),
        "x_hat": np.empty((rows, cols), dtype=np.float32) if want_xhat else None,
    }
    _c().oracle_act_quant(
        _p(x), _p(thr), _p(cb), ctypes.c_int64(rows), ctypes.c_int64(cols), ctypes.c_int(bits),
        ctypes.c_int(group_size), ctypes.c_float(eps), ctypes.c_int(1 if fma else 0),
        _p(out["packed"]), _p(out["codes"]), _p(out["center"]), _p(out["scale"]), _p(out["code_sum"]),
        _p(out["x_hat"]))
    return out


# --------------------------------------------------------------------------
# Stage 2 (a9) -- C
# --------------------------------------------------------------------------
def weight_dequant_c(packed, codebook, center, scale, code_sum, bits: int, group_size: int,
                     fma: bool = True) -> np.ndarray:
    """FQ/arcq_packed_triton.py:33-74; returns fp32 (round with ``.astype(np.float16)``)."""
    packed, cb = _u8(packed), _f32(codebook)
    c, s, cs = _f32(center), _f32(scale), _f32(code_sum)
    n, groups = c.shape
    k = groups * group_size
    assert packed.shape == (n, packed_cols(k, bits))
    out = np.empty((n, k), dtype=np.float32)
    _c().oracle_weight_dequant(_p(packed), _p(cb), _p(c), _p(s), _p(cs), ctypes.c_int64(n), ctypes.c_int64(k),
                               ctypes.c_int(bits), ctypes.c_int(group_size), ctypes.c_int(1 if fma else 0), _p(out))
    return out


# --------------------------------------------------------------------------
# Stage 3 (a11) -- fp64 sum of exact fp16 products
# --------------------------------------------------------------------------
def linear_f64_c(a_f16, w_f16, bias=None) -> Tuple[np.ndarray, np.ndarray]:
    """``y = a @ w.T + bias`` summed in fp64, plus ``sum |a*w|`` per output."""
    a, w = _f32(a_f16), _f32(w_f16)
    b = None if bias is None else _f32(bias)
    m, k = a.shape
    n = w.shape[0]
    y = np.empty((m, n), dtype=np.float64)
    mag = np.empty((m, n), dtype=np.float64)
    _c().oracle_linear_f64(_p(a), _p(w), _p(b), ctypes.c_int64(m), ctypes.c_int64(n), ctypes.c_int64(k), _p(y), _p(mag))
    return y, mag


# --------------------------------------------------------------------------
# Index-space linears (a12) -- C
# --------------------------------------------------------------------------
def linear_forward_packed_c(packed_x, x_center, x_scale, x_code_sum, packed_w, w_center, w_scale, w_code_sum,
                            product_table, bias, bits: int, group_size: int, in_features: int,
                            out_features: int) -> np.ndarray:
    """EXT/arcq_linear_kernel.cu:22-78 (fp64 accumulate, serial)."""
    px, pw = _u8(packed_x), _u8(packed_w)
    pt = _f32(product_table)
    b = None if bias is None else _f32(bias)
    rows = px.shape[0]
    y = np.empty((rows, out_features), dtype=np.float32)
    _c().oracle_linear_forward_packed(
        _p(px), _p(_f32(x_center)), _p(_f32(x_scale)), _p(_f32(x_code_sum)),
        _p(pw), _p(_f32(w_center)), _p(_f32(w_scale)), _p(_f32(w_code_sum)),
        _p(pt), _p(b), ctypes.c_int64(rows), ctypes.c_int64(out_features), ctypes.c_int64(in_features),
        ctypes.c_int(bits), ctypes.c_int(group_size), ctypes.c_int(pt.shape[0]), _p(y))
    return y


def linear_forward_u8_c(x_codes, x_center, x_scale, x_code_sum, w_codes, w_center, w_scale, w_code_sum,
                        product_table, bias, group_size: int) -> np.ndarray:
    """EXT/arcq_linear_kernel.cu:136-202 (fp32, 32-lane strided partials + shuffle-down tree)."""
    xc, wc = _u8(x_codes), _u8(w_codes)
    pt = _f32(product_table)
    b = None if bias is None else _f32(bias)
    rows, in_features = xc.shape
    out_features = wc.shape[0]
    y = np.empty((rows, out_features), dtype=np.float32)
    _c().oracle_linear_forward_u8(
        _p(xc), _p(_f32(x_center)), _p(_f32(x_scale)), _p(_f32(x_code_sum)),
        _p(wc), _p(_f32(w_center)), _p(_f32(w_scale)), _p(_f32(w_code_sum)),
        _p(pt), _p(b), ctypes.c_int64(rows), ctypes.c_int64(out_features), ctypes.c_int64(in_features),
        ctypes.c_int(group_size), ctypes.c_int(pt.shape[0]), _p(y))
    return y


def linear_identity_f64_np(x_codes, x_center, x_scale, x_code_sum, w_codes, w_center, w_scale, w_code_sum,
                           cb_a, cb_w, bias, group_size: int) -> np.ndarray:
    """The closed form behind EXT/arcq_linear_kernel.cu:55-77, vectorised in fp64.

    ``sum_j xhat_j what_j = gs*mu_x*mu_w + s_x*s_w*(sum_j ca_j*cw_j - Sx*Sw/gs)``
    per group.  Independent of the C loops (einsum over codebook values rather
    than a product-table gather).
    """
    xc = np.asarray(x_codes).astype(np.int64)
    wc = np.asarray(w_codes).astype(np.int64)
    m, k = xc.shape
    n = wc.shape[0]
    g = k // group_size
    va = np.asarray(cb_a, dtype=np.float32).astype(np.float64)[xc].reshape(m, g, group_size)
    vw = np.asarray(cb_w, dtype=np.float32).astype(np.float64)[wc].reshape(n, g, group_size)
    cross = np.einsum("mgj,ngj->mng", va, vw)
    xm, xs, xS = (np.asarray(t, dtype=np.float64) for t in (x_center, x_scale, x_code_sum))
    wm, ws, wS = (np.asarray(t, dtype=np.float64) for t in (w_center, w_scale, w_code_sum))
    per_group = group_size * xm[:, None, :] * wm[None, :, :] + xs[:, None, :] * ws[None, :, :] * (
        cross - xS[:, None, :] * wS[None, :, :] / group_size)
    y = per_group.sum(-1)
    if bias is not None:
        y = y + np.asarray(bias, dtype=np.float64)[None, :]
    return y


# --------------------------------------------------------------------------
# Torch-order restatements (reduction order = the running torch build's)
# --------------------------------------------------------------------------
def group_stats_torch(x2: torch.Tensor, group_size: int, eps: float):
    """center / residual / scale / t exactly as Q/dcarcq.py:531-536 orders the ops."""
    rows, cols = x2.shape
    x3 = x2.reshape(rows, cols // group_size, group_size)
    center = x3.mean(dim=-1, keepdim=True)
    residual = x3 - center
    scale = (residual.square().mean(dim=-1, keepdim=True) + eps).sqrt()
    return x3, center, residual, scale, residual / scale


def quantize_weight_torch(weight: torch.Tensor, thresholds: torch.Tensor, codebook: torch.Tensor,
                          group_size: int, eps: float):
    """Offline weight encoder -- FQ/arcq_packed_linear.py:27-53.

    Returns ``codes [N,K] int64, center, scale, code_sum [N,G] fp32``.
    """
    w = weight.detach().float().contiguous()
    n, k = w.shape
    _, center, _, scale, t = group_stats_torch(w, group_size, float(eps))
    codes = torch.bucketize(t, thresholds.to(t.dtype))
    code_sum = codebook.to(t.dtype)[codes].sum(dim=-1)
    return codes.reshape(n, k).to(torch.int64), center.squeeze(-1), scale.squeeze(-1), code_sum


def dequant_activation_torch(x: torch.Tensor, thresholds: torch.Tensor, codebook: torch.Tensor,
                             group_size: int) -> torch.Tensor:
    """Torch stage 1, quantize + reconstruct -- FQ/arcq_packed_on_the_fly.py:66-90 (eps literal 1e-6)."""
    rows, cols = x.shape
    _, center, _, scale, t = group_stats_torch(x, group_size, 1e-6)
    codes = torch.bucketize(t, thresholds)
    vals = codebook[codes]
    code_mean = vals.sum(dim=-1, keepdim=True) / float(group_size)
    return (center + scale * (vals - code_mean)).reshape(rows, cols)


def act_quant_torch(x: torch.Tensor, thresholds: torch.Tensor, codebook: torch.Tensor, group_size: int,
                    eps: float = 1e-6):
    """Codes and metadata in torch order (same ops as :func:`dequant_activation_torch`)."""
    rows, cols = x.shape
    _, center, _, scale, t = group_stats_torch(x.float(), group_size, eps)
    codes = torch.bucketize(t, thresholds)
    code_sum = codebook[codes].sum(dim=-1)
    return codes.reshape(rows, cols), center.squeeze(-1), scale.squeeze(-1), code_sum, t.reshape(rows, cols)


def unpack_weight_torch(packed: torch.Tensor, codebook: torch.Tensor, center: torch.Tensor,
                        scale: torch.Tensor, code_sum: torch.Tensor, bits: int, group_size: int) -> torch.Tensor:
    """Torch stage 2 -- arithmetic of FQ/arcq_packed_on_the_fly.py:50-63 (``c + s*(v - cs/gs)`` -> fp16).

    The reference's byte gather at :36-48 reads one byte past the row for
    3-bit codes; codes are taken from :func:`unpack_codes_np` here instead.
    """
    n, groups = center.shape
    k = groups * group_size
    codes = torch.from_numpy(unpack_codes_np(packed.cpu().numpy(), bits, k))
    vals = codebook.float()[codes].reshape(n, groups, group_size)
    vals_c = vals - code_sum.float().unsqueeze(-1) / float(group_size)
    w = center.float().unsqueeze(-1) + scale.float().unsqueeze(-1) * vals_c
    return w.reshape(n, k).to(torch.float16)


def pcarcq_fake_quant(x: torch.Tensor, thresholds: torch.Tensor, codebook: torch.Tensor,
                      group_size: int = 64, eps: float = 1e-6) -> torch.Tensor:
    """Eval-mode forward of the phase-compiled quantizer with a ready codebook -- Q/dcarcq.py:512-578.

    Pads the last dim to a multiple of ``group_size`` (:522-527), quantizes,
    subtracts the group mean of the looked-up values (:555-556), reconstructs
    (:558) and returns ``x + (x_hat - x)`` (:564).
    """
    shape = x.shape
    c = shape[-1]
    x2 = x.reshape(-1, c)
    pad = (-c) % group_size
    if pad:
        x2 = F.pad(x2, (0, pad))
    rows, cp = x2.shape
    _, center, _, scale, t = group_stats_torch(x2, group_size, eps)
    codes = torch.bucketize(t, thresholds.to(t.dtype))
    t_hat = codebook.to(t.dtype)[codes]
    t_hat = t_hat - t_hat.mean(dim=-1, keepdim=True)
    x_hat = (center + scale * t_hat).reshape(rows, cp)
    if pad:
        x_hat = x_hat[:, :c]
    x_hat = x_hat.reshape(shape)
    return x + (x_hat - x)


def fake_quant_linear(x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor],
                      a_thr: torch.Tensor, a_cb: torch.Tensor, w_thr: torch.Tensor, w_cb: torch.Tensor,
                      group_size: int = 64, eps: float = 1e-6) -> torch.Tensor:
    """``QuantLinearPCARCQ.forward`` without the DC conditioner -- FQ/quant_backends.py:312-322.

    This is the "dcarcq quantize, reconstruct, then matmul" CPU path that
    ``bench.py`` times as ``cpu_baseline``; the weight is re-quantized on every
    call, as the reference does.
    """
    x_q = pcarcq_fake_quant(x, a_thr, a_cb, group_size, eps)
    w_q = pcarcq_fake_quant(weight, w_thr, w_cb, group_size, eps)
    return F.linear(x_q, w_q, bias)


# --------------------------------------------------------------------------
# LayerNorm in front of stage 1 (the fused producer of arcq_act_quant_blocked_ln) and the GELU of the
# fused epilogue.  The reference runs both as timm / torch modules around the packed linears
# (FQ/timm_quant_models.py:63-121: timm Block = LayerNorm -> Attention / Mlp with nn.GELU); timm is not
# available offline, so these restate torch.nn.LayerNorm / nn.GELU() semantics, in the summation order the
# HIP kernel documents, and are pinned against torch's own float64 layer_norm / erf in the tests.
# --------------------------------------------------------------------------
def layernorm_rows_np(x, weight, bias, eps: float, out_f16: bool) -> np.ndarray:
    """LayerNorm over the last dimension (a multiple of 64) in the kernel's fp32 order: serial sums over
    each run of 32 values, a row's partial sums added in order; mean = sum / K; var = the same over
    (x - mean)^2; y = ((x - mean) * (1 / sqrt(var + eps))) * weight + bias, one rounding per operation;
    optionally rounded to fp16 (what a stand-alone fp16 LayerNorm would store).  Returns fp32."""
    x = np.ascontiguousarray(_f32(x))
    rows, k = x.shape
    assert k % 64 == 0
    parts = k // 32
    x3 = x.reshape(rows, parts, 32)
    f32 = np.float32

    def serial(v):
        a = np.zeros(v.shape[:2], dtype=f32)
        for j in range(32):
            a = (a + v[:, :, j]).astype(f32)
        return a

    def total(p):
        acc = np.zeros(rows, dtype=f32)
        for i in range(parts):
            acc = (acc + p[:, i]).astype(f32)
        return acc

    mean = (total(serial(x3)) / f32(k)).astype(f32)
    d = (x3 - mean[:, None, None]).astype(f32)
    var = (total(serial((d * d).astype(f32))) / f32(k)).astype(f32)
    rstd = (f32(1.0) / np.sqrt((var + f32(eps)).astype(f32)).astype(f32)).astype(f32)
    t = (d * rstd[:, None, None]).astype(f32)
    u = (t * _f32(weight).reshape(1, parts, 32)).astype(f32)
    y = (u + _f32(bias).reshape(1, parts, 32)).astype(f32).reshape(rows, k)
    if out_f16:
        y = y.astype(np.float16).astype(f32)
    return y


def gelu_f64_np(x) -> np.ndarray:
    """Exact GELU ``0.5 x (1 + erf(x / sqrt 2))`` in float64 (nn.GELU(), approximate='none')."""
    import math
    x = np.asarray(x, dtype=np.float64)
    erf = np.vectorize(math.erf, otypes=[np.float64])
    return 0.5 * x * (1.0 + erf(x / math.sqrt(2.0)))


# --------------------------------------------------------------------------
# FP8 operands (the low-precision formulation of the layer; no reference counterpart)
# --------------------------------------------------------------------------
FP8_E4M3_MAX = 448.0


def fp8_e4m3_np(v) -> np.ndarray:
    """Round float values to OCP FP8 E4M3 (1 sign, 4 exponent bits with bias 7, 3 mantissa bits; no infinities,
    largest finite value 448): clamp to +-448, then round to nearest, ties to the even mantissa.  Normal numbers
    2^e (1 + m/8), e = -6 .. 8; below 2^-6 the spacing stays 2^-9 (subnormals).  Returns float32 holding the
    rounded values exactly.  Pinned in tests by hand-computed ties and against torch's ``float8_e4m3fn`` cast."""
    a = np.clip(np.asarray(v, dtype=np.float64), -FP8_E4M3_MAX, FP8_E4M3_MAX)
    mag = np.abs(a)
    e = np.floor(np.log2(np.where(mag > 0, mag, 1.0)))
    e = np.clip(e, -6, 8)
    step = np.exp2(e - 3)                      # spacing inside the binade (2^-9 for everything below 2^-6)
    q = np.rint(mag / step)                    # numpy rounds halves to even
    out = np.sign(a) * q * step                # (a mantissa carried to 16 steps is the next binade's first value)
    return out.astype(np.float32)
