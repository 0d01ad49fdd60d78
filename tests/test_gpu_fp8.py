"""GPU tests of the layer with FP8 operands (``ops.linear_otf_fp8``: stage 1 and stage 2 rounded to OCP E4M3, the
product on the library's own FP8 MFMA kernel).  The path has no counterpart in the reference and does not reproduce its
numbers; what is checked is that it is exactly what it says: the operands are the oracle's fp32 reconstructions
rounded to FP8 bit for bit, and the product is their exact product within fp32 accumulation error."""
import numpy as np
import pytest
import torch

import arcq_vit_amd as A
from arcq_vit_amd import ops, synth

pytestmark = pytest.mark.gpu


def _np(t):
    return t.detach().cpu().numpy()


def _layer(oracle, n, k, bits, seed):
    cb = synth.quantile_codebook(bits)
    thr = synth.midpoint_thresholds(cb)
    w = synth.make_weight(n, k, seed)
    codes, wc, ws, wcs = oracle.quantize_weight_torch(w, thr, cb, 64, 1e-6)
    return cb, thr, A.pack_codes_py(codes, bits), wc, ws, wcs, synth.make_bias(n, seed + 1)


def _fp8_bytes(values_f32: np.ndarray) -> np.ndarray:
    """Bit patterns of float32 values that are exactly representable in FP8 E4M3."""
    return torch.from_numpy(np.ascontiguousarray(values_f32)).to(torch.float8_e4m3fn).view(torch.uint8).numpy()


@pytest.mark.parametrize("m,k,bits,dtype", [(197, 192, 4, torch.float16), (1000, 384, 3, torch.float32),
                                            (4099, 1536, 2, torch.float16), (33, 64, 4, torch.float32)])
def test_stage1_fp8_is_the_oracle_reconstruction_rounded(cuda, oracle, m, k, bits, dtype):
    cb = synth.quantile_codebook(bits)
    thr = synth.midpoint_thresholds(cb)
    x = synth.make_activation(m, k, 7, "ln").to(dtype)
    x[0, :64] = 1000.0 * torch.linspace(-1, 1, 64).to(dtype)            # a group whose values leave FP8's range: clamped
    if m > 1:
        x[1, 5] = float("nan")                                          # a NaN poisons its group and stays a NaN in FP8
    x8 = ops.quantize_activation_fp8(x.to(cuda), thr.to(cuda), cb.to(cuda), bits)
    with np.errstate(invalid="ignore"):
        want = oracle.fp8_e4m3_np(oracle.act_quant_c(x.float().numpy(), thr, cb, bits, 64)["x_hat"])
    nan = np.isnan(want)
    assert np.nanmax(np.abs(want)) == 448.0 and (m == 1 or (nan[1, :64].all() and nan.sum() == 64))
    got = _np(x8.view(torch.uint8))
    assert np.array_equal((got & 0x7f) == 0x7f, nan)                     # E4M3: S.1111.111 is the only NaN
    assert np.array_equal(got[~nan], _fp8_bytes(np.where(nan, 0.0, want))[~nan])


@pytest.mark.parametrize("n,k,bits", [(384, 1536, 4), (96, 192, 3), (1024, 1024, 2)])
def test_stage2_fp8_is_the_oracle_reconstruction_scaled_and_rounded(cuda, oracle, n, k, bits):
    cb, thr, pw, wc, ws, wcs, _ = _layer(oracle, n, k, bits, 11)
    mult = ops.fp8_weight_multiplier(cb, wc, ws, wcs)
    w = oracle.weight_dequant_c(pw.numpy(), cb, wc, ws, wcs, bits, 64, fma=True)
    assert mult == 2.0 ** round(np.log2(mult)) and 1.0 < np.abs(w).max() * mult <= 224.0
    d = lambda t: t.to(cuda)
    w8 = ops.unpack_weight_fp8(d(pw), d(cb), d(wc), d(ws), d(wcs), bits, mult)
    assert np.array_equal(_np(w8.view(torch.uint8)), _fp8_bytes(oracle.fp8_e4m3_np(w * np.float32(mult))))
    # a multiplier that pushes weights past the range saturates them instead of producing NaNs
    w8 = ops.unpack_weight_fp8(d(pw), d(cb), d(wc), d(ws), d(wcs), bits, mult * 64)
    assert np.array_equal(_np(w8.view(torch.uint8)), _fp8_bytes(oracle.fp8_e4m3_np(w * np.float32(mult * 64))))


@pytest.mark.parametrize("m,n,k,bits,out", [(197, 384, 1536, 4, torch.float16), (3000, 768, 768, 3, torch.float32),
                                            (12608, 1152, 384, 4, torch.float16)])
def test_fp8_layer_is_the_exact_product_of_its_operands(cuda, oracle, m, n, k, bits, out):
    """y against the fp64 product of the FP8 operands (fp32 accumulation bound, as for the fp16 GEMMs, plus the
    rounding of the output), and its distance from the fp16 path, which is what the FP8 operands cost: a few per cent
    of the output's norm -- the reason this path is an option and not the default."""
    cb, thr, pw, wc, ws, wcs, bias = _layer(oracle, n, k, bits, 21)
    x = synth.make_activation(m, k, 23, "ln").to(torch.float16)
    d = lambda t: t.to(cuda)
    args = (d(x), d(thr), d(cb), d(pw), d(cb), d(wc), d(ws), d(wcs), d(bias), bits)
    y = ops.linear_otf_fp8(*args, out_dtype=out)
    mult = ops.fp8_weight_multiplier(cb, wc, ws, wcs)
    rows = torch.randint(0, m, (48,), generator=torch.Generator().manual_seed(3))
    rows[0], rows[1] = 0, m - 1
    a8 = oracle.fp8_e4m3_np(oracle.act_quant_c(x[rows].float().numpy(), thr, cb, bits, 64)["x_hat"])
    w8 = oracle.fp8_e4m3_np(oracle.weight_dequant_c(pw.numpy(), cb, wc, ws, wcs, bits, 64, fma=True) * np.float32(mult))
    y64, mag = oracle.linear_f64_c(a8, w8, None)
    y64, mag = y64 / mult + bias.numpy().astype(np.float64), mag / mult
    ulp = 2.0 ** -11 if out == torch.float16 else 2.0 ** -24
    tol = (k + 2) * 2.0 ** -24 * mag + 2 * np.abs(y64) * ulp + np.abs(bias.numpy()) * 2.0 ** -11 + 2.0 ** -20      # (bias added in the output type)
    err = np.abs(_np(y[rows.to(cuda)]).astype(np.float64) - y64)
    assert np.all(err <= tol), float((err / tol).max())
    y16 = ops.linear_otf(*args, 64, out_dtype=torch.float32)
    rel = float((y.float() - y16).norm() / y16.norm())
    assert 1e-4 < rel < 0.05, rel


def _fp8_blocked(a: np.ndarray, kp: int) -> np.ndarray:
    """[M, K] bytes -> the FP8 GEMM's block layout [M/32][kp/16][rows][16] (zero padding from K to kp), flat."""
    m, k = a.shape
    pad = np.zeros((m, kp), dtype=np.uint8)
    pad[:, :k] = a
    parts = []
    for r0 in range(0, m, 32):
        blk = pad[r0:r0 + 32]
        parts.append(np.ascontiguousarray(blk.reshape(blk.shape[0], kp // 16, 16).transpose(1, 0, 2)).reshape(-1))
    return np.concatenate(parts)


@pytest.mark.parametrize("m,n,k,bits,dtype", [(197, 96, 192, 4, torch.float16), (1000, 200, 384, 3, torch.float32),
                                              (4099, 64, 1536, 2, torch.float16), (33, 40, 64, 4, torch.float32)])
def test_stage1_fp8_blocked_with_weights(cuda, oracle, m, n, k, bits, dtype):
    """arcq_act_quant_fp8_blocked: the bytes of the row-major kernel in the block layout, zero padding to a multiple of
    128, and -- carried in the same launch -- the FP8 weights with the same padding."""
    cb, thr, pw, wc, ws, wcs, _ = _layer(oracle, n, k, bits, 13)
    x = synth.make_activation(m, k, 7, "ln").to(dtype)
    kp = ops.fp8_padded_k(k)
    mult = ops.fp8_weight_multiplier(cb, wc, ws, wcs)
    d = lambda t: t.to(cuda)
    x8 = torch.full((m * kp + 16,), 0x5a, dtype=torch.uint8, device=cuda)
    w8 = torch.full((n * kp + 16,), 0x5a, dtype=torch.uint8, device=cuda)
    lib = A._lib.load()
    xd, td, cd = d(x), d(thr), d(cb)
    wts = [d(t) for t in (pw, cb, wc, ws, wcs)]
    code = A._lib.ARCQ_F16 if dtype == torch.float16 else A._lib.ARCQ_F32
    A._lib.check(lib.arcq_act_quant_fp8_blocked(xd.data_ptr(), code, td.data_ptr(), cd.data_ptr(), x8.data_ptr(), m, k, bits,
                                               1e-6, *[t.data_ptr() for t in wts], w8.data_ptr(), n, mult, 0))
    torch.cuda.synchronize()
    want_x = _fp8_bytes(oracle.fp8_e4m3_np(oracle.act_quant_c(x.float().numpy(), thr, cb, bits, 64)["x_hat"]))
    assert np.array_equal(_np(x8)[:m * kp], _fp8_blocked(want_x, kp))
    w = oracle.weight_dequant_c(pw.numpy(), cb, wc, ws, wcs, bits, 64, fma=True)
    want_w = np.zeros((n, kp), dtype=np.uint8)
    want_w[:, :k] = _fp8_bytes(oracle.fp8_e4m3_np(w * np.float32(mult)))
    assert np.array_equal(_np(w8)[:n * kp].reshape(n, kp), want_w)
    assert bool((x8[m * kp:] == 0x5a).all()) and bool((w8[n * kp:] == 0x5a).all())


@pytest.mark.parametrize("m,n,k,out", [(50, 64, 128, torch.float32), (197, 384, 1536, torch.float16),
                                       (1000, 200, 256, torch.float32),       # ragged rows and columns
                                       (3000, 768, 768, torch.float16), (12608, 1152, 384, torch.float16),
                                       (8191, 4096, 1024, torch.float16)])    # sixteen row blocks and more per workgroup
def test_fp8_gemm_kernel_against_fp64(cuda, oracle, m, n, k, out):
    """arcq_linear_fp8_blocked on random FP8 operands against their fp64 product (fp32 accumulation bound + the output
    rounding) on sampled rows, and against the vendor library's FP8 GEMM on the same operands."""
    g = torch.Generator().manual_seed(5)
    a = (torch.randn(m, k, generator=g) * 1.5).to(torch.float8_e4m3fn)
    w = (torch.randn(n, k, generator=g) * 4.0).to(torch.float8_e4m3fn)
    bias = torch.randn(n, generator=g)
    mult = 16.0
    xb = torch.from_numpy(_fp8_blocked(a.view(torch.uint8).numpy(), k)).to(cuda)
    wd = w.to(cuda)
    y = torch.empty((m, n), dtype=out, device=cuda)
    A._lib.check(A._lib.load().arcq_linear_fp8_blocked(xb.data_ptr(), wd.data_ptr(), bias.to(cuda).data_ptr(), mult, y.data_ptr(),
                                                      A._lib.ARCQ_F16 if out == torch.float16 else A._lib.ARCQ_F32, m, n, k, 0))
    rows = torch.randint(0, m, (40,), generator=torch.Generator().manual_seed(3))
    rows[0], rows[1], rows[2] = 0, m - 1, (m // 32) * 32 - 1
    y64, mag = oracle.linear_f64_c(a[rows].float().numpy(), w.float().numpy(), None)
    y64, mag = y64 / mult + bias.numpy().astype(np.float64), mag / mult
    ulp = 2.0 ** -11 if out == torch.float16 else 2.0 ** -24
    # (the matrix unit sums the 64 products of one instruction internally, not as a chain of correctly rounded fp32
    # additions: twice the serial-fp32 bound is allowed for it; measured worst case 1.4 x)
    tol = 2 * (k + 2) * 2.0 ** -24 * mag + np.abs(y64) * ulp + 2.0 ** -24
    err = np.abs(_np(y[rows.to(cuda)]).astype(np.float64) - y64)
    assert np.all(err <= tol), float((err / tol).max())
    if out == torch.float16 and n % 16 == 0:
        one = torch.ones((), device=cuda)
        lib_y = torch._scaled_mm(a.to(cuda), wd.t(), scale_a=one, scale_b=one / mult, bias=bias.half().to(cuda), out_dtype=out)
        assert float((y.float() - lib_y.float()).abs().max()) <= 4e-3 * float(lib_y.float().abs().max())


def test_fp8_entry_points_reject_bad_arguments(cuda):
    lib = A._lib.load()
    x = torch.zeros(64 * 64, dtype=torch.float16, device=cuda)
    out = torch.zeros(64 * 64, dtype=torch.uint8, device=cuda)
    f = torch.zeros(64, dtype=torch.float32, device=cuda)
    F16 = A._lib.ARCQ_F16
    assert lib.arcq_act_quant_fp8(x.data_ptr(), F16, f.data_ptr(), f.data_ptr(), out.data_ptr(), 64, 64, 5, 1e-6, 0) != 0
    assert lib.arcq_act_quant_fp8(x.data_ptr(), F16, f.data_ptr(), f.data_ptr(), out.data_ptr(), 64, 96, 4, 1e-6, 0) != 0
    assert lib.arcq_act_quant_fp8(x.data_ptr(), F16, f.data_ptr(), f.data_ptr(), None, 64, 64, 4, 1e-6, 0) != 0
    assert lib.arcq_act_quant_fp8(None, F16, None, None, None, 0, 64, 4, 1e-6, 0) == 0          # nothing to do
    args = [out.data_ptr(), f.data_ptr(), f.data_ptr(), f.data_ptr(), f.data_ptr(), out.data_ptr()]
    assert lib.arcq_weight_dequant_fp8(*args, 8, 64, 4, 32, 1.0, 0) != 0                        # group size 64 only
    assert lib.arcq_weight_dequant_fp8(*args, 8, 64, 4, 64, 0.0, 0) != 0                        # multiplier must be positive
    assert lib.arcq_weight_dequant_fp8(*args, 8, 64, 7, 64, 1.0, 0) != 0
    y = torch.zeros(64 * 64, dtype=torch.float16, device=cuda)
    assert lib.arcq_linear_fp8_blocked(out.data_ptr(), out.data_ptr(), None, 1.0, y.data_ptr(), F16, 32, 64, 64, 0) != 0   # K % 128
    assert lib.arcq_linear_fp8_blocked(out.data_ptr(), out.data_ptr(), None, 0.0, y.data_ptr(), F16, 32, 64, 128, 0) != 0  # multiplier
    assert lib.arcq_linear_fp8_blocked(None, out.data_ptr(), None, 1.0, y.data_ptr(), F16, 32, 64, 128, 0) != 0
    assert lib.arcq_linear_fp8_blocked(None, None, None, 1.0, None, F16, 0, 64, 128, 0) == 0                              # nothing to do


def test_model_with_fp8_operands(cuda):
    """set_fp8_operands switches every packed layer of a model; the logits stay close to the fp16 path's (the layers
    differ by a few per cent each) and the switch back restores them bit for bit."""
    from arcq_vit_amd.vit import build_packed_vit
    vit = build_packed_vit("deit_tiny", 4, depth=2)
    x = torch.randn(8, 3, 224, 224, generator=torch.Generator().manual_seed(1)).half().to(cuda)
    with torch.no_grad():
        y16 = vit(x).float()
        assert A.set_fp8_operands(vit) == 8
        y8 = vit(x).float()
        assert A.set_fp8_operands(vit, False) == 8
        assert torch.equal(vit(x).float(), y16)
    cos = torch.nn.functional.cosine_similarity(y8.flatten(), y16.flatten(), dim=0).item()
    assert bool(torch.isfinite(y8).all()) and not torch.equal(y8, y16) and cos > 0.98, cos
