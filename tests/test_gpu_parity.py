"""GPU parity: every HIP entry point, called through the C ABI (via the ctypes shim in
``arcq_vit_amd.ops``), against the CPU oracle on the same seeded inputs.

Bars: bit-exact for codes, packed bytes, group metadata and reconstructions (integer work and
fp32 work with a fixed operation order); for the fp16 MFMA GEMM the fp32-accumulation error bound
stated in ``_gemm_tol``.
"""
import numpy as np
import pytest
import torch

from arcq_vit_amd import ops, synth

pytestmark = pytest.mark.gpu


def _cb(bits):
    cb = synth.quantile_codebook(bits)
    return cb, synth.midpoint_thresholds(cb)


def _np(t):
    return t.detach().cpu().numpy()


# ------------------------------------------------------------------------------------------------
# bit packing
# ------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("bits", [2, 3, 4])
@pytest.mark.parametrize("shape", [(1, 1), (3, 7), (5, 64), (17, 197), (768, 192), (384, 1536)])
def test_pack_unpack(cuda, oracle, bits, shape):
    rng = np.random.default_rng(bits * 31 + shape[1])
    codes = rng.integers(0, 1 << bits, size=shape, dtype=np.int64)
    packed = ops.pack_codes(torch.from_numpy(codes).to(cuda), bits)
    assert packed.dtype == torch.uint8 and tuple(packed.shape) == (shape[0], (shape[1] * bits + 7) // 8)
    assert np.array_equal(_np(packed), oracle.pack_codes_c(codes, bits))
    assert np.array_equal(_np(ops.unpack_codes(packed, bits, shape[1])), codes)
    u8 = ops.unpack_codes_u8(packed, bits, shape[1])
    assert u8.dtype == torch.uint8 and np.array_equal(_np(u8), codes.astype(np.uint8))


def test_pack_masks_and_overwrites(cuda, oracle):
    """High bits are dropped, and the output needs no pre-zeroing."""
    codes = torch.tensor([[0x1F, 0x23, -1, 7, 9]], dtype=torch.int64)
    for bits in (2, 3, 4):
        got = ops.pack_codes(codes.to(cuda), bits)
        assert np.array_equal(_np(got), oracle.pack_codes_c(codes.numpy(), bits))


def test_pack_empty(cuda):
    assert tuple(ops.pack_codes(torch.zeros((0, 8), dtype=torch.int64, device=cuda), 4).shape) == (0, 4)
    assert tuple(ops.unpack_codes(torch.zeros((4, 0), dtype=torch.uint8, device=cuda), 3, 0).shape) == (4, 0)


# ------------------------------------------------------------------------------------------------
# stage 1
# ------------------------------------------------------------------------------------------------
def _check_stage1(cuda, oracle, x, bits, gs=64):
    cb, thr = _cb(bits)
    ref = oracle.act_quant_c(x.numpy(), thr, cb, bits, gs)
    xd, thrd, cbd = x.to(cuda), thr.to(cuda), cb.to(cuda)
    packed, center, scale, code_sum = ops.quantize_activation(xd, thrd, cbd, bits, gs)
    assert np.array_equal(_np(packed), ref["packed"])
    assert np.array_equal(_np(center), ref["center"])
    assert np.array_equal(_np(scale), ref["scale"])
    assert np.array_equal(_np(code_sum), ref["code_sum"])
    codes, c2, s2, cs2 = ops.quantize_activation_u8(xd, thrd, cbd, bits, gs)
    assert np.array_equal(_np(codes), ref["codes"])
    assert torch.equal(c2, center) and torch.equal(s2, scale) and torch.equal(cs2, code_sum)
    x_hat = ops.quantize_activation_dequant(xd, thrd, cbd, bits, gs)
    assert x_hat.dtype == torch.float32 and np.array_equal(_np(x_hat), ref["x_hat"])
    return ref


@pytest.mark.parametrize("bits", [2, 3, 4])
@pytest.mark.parametrize("m,k,kind", [(197, 192, "ln"), (197, 384, "ln"), (197, 1536, "gelu"), (1, 64, "ln"),
                                      (63, 128, "ln"), (65, 64, "gelu"), (1000, 384, "ln")])
def test_stage1_bitexact_fp32(cuda, oracle, bits, m, k, kind):
    _check_stage1(cuda, oracle, synth.make_activation(m, k, 100 + bits, kind), bits)


@pytest.mark.parametrize("bits", [3, 4])
def test_stage1_bitexact_large_launch(cuda, oracle, bits):
    """More 64-group tiles (2 251, the last one a quarter full) than the 512 x 4 waves of the launch: waves walk two
    tiles, the second prefetched under the first; packed codes, byte codes, metadata and x_hat as the oracle's."""
    _check_stage1(cuda, oracle, synth.make_activation(9001, 1024, 300 + bits, "gelu"), bits)


@pytest.mark.parametrize("bits", [3, 4])
def test_stage1_fp16_chain_and_inplace(cuda, oracle, bits):
    """fp16 in -> fp16 out, as the on-the-fly layer runs it; fp16 is widened exactly, statistics are
    fp32, x_hat is rounded once to fp16.  In-place (out=x) gives the same bytes."""
    cb, thr = _cb(bits)
    x16 = synth.make_activation(197, 384, 7).to(torch.float16)
    ref = oracle.act_quant_c(x16.float().numpy(), thr, cb, bits, 64)
    want = ref["x_hat"].astype(np.float16)
    xd = x16.to(cuda)
    out = ops.dequant_activation_hip(xd, thr.to(cuda), cb.to(cuda), 64)
    assert out.dtype == torch.float16 and out.data_ptr() != xd.data_ptr()
    assert np.array_equal(_np(out).view(np.uint16), want.view(np.uint16))
    assert torch.equal(xd.cpu(), x16)                      # input untouched
    same = ops.dequant_activation_hip(xd, thr.to(cuda), cb.to(cuda), 64, out=xd)
    assert same.data_ptr() == xd.data_ptr()
    assert np.array_equal(_np(xd).view(np.uint16), want.view(np.uint16))
    # fp32 in place as well
    x32 = synth.make_activation(130, 192, 8).to(cuda)
    ref32 = oracle.act_quant_c(_np(x32), thr, cb, bits, 64)
    ops.dequant_activation_hip(x32, thr.to(cuda), cb.to(cuda), 64, out=x32)
    assert np.array_equal(_np(x32), ref32["x_hat"])


@pytest.mark.parametrize("gs,bits", [(32, 4), (128, 3), (16, 2), (192, 4)])
def test_stage1_other_group_sizes(cuda, oracle, gs, bits):
    _check_stage1(cuda, oracle, synth.make_activation(33, 384, gs, "ln"), bits, gs)


def test_stage1_ties_constant_and_extremes(cuda, oracle):
    """Exact ties (thresholds taken from occurring t values), constant groups (s = sqrt(eps)),
    large magnitudes and zeros."""
    bits = 4
    cb, _ = _cb(bits)
    x = synth.make_activation(16, 128, 3)
    x[0] = 2.5
    x[1, :64] = 0.0
    x[2] *= 3.0e4
    x[3] *= 1.0e-4
    ref0 = oracle.act_quant_c(x.numpy(), synth.midpoint_thresholds(cb), cb, bits, 64)
    t = ((x.numpy().reshape(16, 2, 64) - ref0["center"][..., None]) / ref0["scale"][..., None]).astype(np.float32)
    u = np.sort(np.unique(t))
    thr = torch.from_numpy(u[np.linspace(5, u.size - 6, 15).astype(np.int64)].copy())
    assert thr.numel() == 15 and bool((thr[1:] > thr[:-1]).all())
    ref = oracle.act_quant_c(x.numpy(), thr, cb, bits, 64)
    packed, center, scale, code_sum = ops.quantize_activation(x.to(cuda), thr.to(cuda), cb.to(cuda), bits, 64)
    assert np.array_equal(_np(packed), ref["packed"])
    assert np.array_equal(_np(scale), ref["scale"]) and np.array_equal(_np(code_sum), ref["code_sum"])
    assert _np(scale)[0, 0] == np.sqrt(np.float32(1e-6))


def test_stage1_fallback_paths(cuda, oracle):
    """The gs=64 kernel leaves its fast path (bucket-table search, fma-based divide) when two thresholds
    share a bucket, when thresholds are unsorted, or when a group's scale / mean is out of the guarded
    range; every fallback must give the same bits as the oracle."""
    bits = 4
    cb, thr = _cb(bits)
    x = synth.make_activation(70, 128, 9)
    d = lambda t: t.to(cuda)

    def check(xx, tt, eps=1e-6):
        ref = oracle.act_quant_c(xx.numpy(), tt, cb, bits, 64, eps=eps)
        out = ops._act_quant(d(xx), d(tt), d(cb), bits, 64, want_packed=True, want_meta=True, eps=eps)
        assert np.array_equal(_np(out[0]), ref["packed"])
        assert np.array_equal(_np(out[3]), ref["scale"]) and np.array_equal(_np(out[4]), ref["code_sum"])

    close = thr.clone()
    close[7] = close[6] + 1e-4                       # two thresholds inside one 1/32-wide bucket
    check(x, close)
    dup = thr.clone()
    dup[3] = dup[2]                                  # equal thresholds
    check(x, dup)
    unsorted = thr.clone()
    unsorted[[4, 9]] = unsorted[[9, 4]]              # while-loop semantics: stops at the first failing threshold
    check(x, unsorted)
    far = thr.clone()
    far[-1] = 9.5                                    # beyond the reachable range of t
    check(x, far)
    tiny = x.clone()
    tiny[3] *= 1e-30                                 # |mu| < 2^-66 with non-zero residuals
    tiny[5] = 0.0
    check(tiny, thr)
    huge = x.clone()
    huge[7] *= 3e18                                  # variance overflows to inf: s = inf, t = 0 or nan
    check(huge, thr)
    check(x * 1e-12, thr, eps=0.0)                   # eps = 0: s far below 2^-60... still exact
    check(x, thr, eps=1e-2)


def test_stage1_two_lane_fallback_paths(cuda, oracle):
    """The two-lanes-per-group kernels (small x_hat-only launches, block-layout output) through the same fallbacks:
    unusable bucket tables and groups outside the guarded range of the fma-based divide; x_hat equals the oracle's."""
    bits = 4
    cb, thr = _cb(bits)
    x = synth.make_activation(70, 128, 9)
    d = lambda t: t.to(cuda)

    def check(xx, tt):
        want = oracle.act_quant_c(xx.numpy(), tt, cb, bits, 64)["x_hat"]
        got = ops.dequant_activation_hip(d(xx), d(tt), d(cb), 64)                   # fp32 in, fp32 out: small kernel
        assert np.array_equal(_np(got).view(np.uint32), want.view(np.uint32))
        h = xx.clamp(-6.0e4, 6.0e4).to(torch.float16)      # finite in fp16: an inf group is all NaN, whose bits are free
        want16 = oracle.act_quant_c(h.float().numpy(), tt, cb, bits, 64)["x_hat"].astype(np.float16)
        got16 = ops.dequant_activation_hip(d(h), d(tt), d(cb), 64)
        assert np.array_equal(_np(got16).view(np.uint16), want16.view(np.uint16))
        blk = ops.quantize_activation_blocked(d(xx), d(tt), d(cb), bits).reshape(-1)   # block layout, fp32 in
        want_b = oracle.act_quant_c(xx.numpy(), tt, cb, bits, 64)["x_hat"].astype(np.float16)
        assert np.array_equal(_np(blk).view(np.uint16), _np(_to_blocked(torch.from_numpy(want_b))).view(np.uint16))

    close = thr.clone()
    close[7] = close[6] + 1e-4
    check(x, close)
    unsorted = thr.clone()
    unsorted[[4, 9]] = unsorted[[9, 4]]
    check(x, unsorted)
    far = thr.clone()
    far[-1] = 9.5
    check(x, far)
    tiny = x.clone()
    tiny[3] *= 1e-30
    tiny[5] = 0.0
    check(tiny, thr)
    huge = x.clone()
    huge[7] *= 3e18
    check(huge, thr)
    const = x.clone()
    const[11] = 2.5                                   # constant groups: s = sqrt(eps), every t = 0
    check(const, thr)


@pytest.mark.parametrize("bits", [4, 3, 2])
def test_stage1_threshold_neighbourhoods(cuda, oracle, bits):
    """Hard cases for the code decision t > thr with t = RN(d/s): thresholds that ARE occurring t values (exact ties:
    false), their neighbours one ulp below (true) and above, thresholds on round values and on / next to the
    boundaries of the kernels' lookup buckets (whole and shifted grids of 1/4 and 1/8), and a large launch for
    coverage; x_hat must equal the oracle's bit for bit in the small kernel, the block layout and fp16."""
    cb = synth.quantile_codebook(bits)
    n_thr = (1 << bits) - 1
    x = synth.make_activation(640, 384, 17)
    d = lambda t: t.to(cuda)

    def check(xx, tt):
        want = oracle.act_quant_c(xx.numpy(), tt, cb, bits, 64)["x_hat"]
        got = ops.dequant_activation_hip(d(xx), d(tt), d(cb), 64)
        assert np.array_equal(_np(got).view(np.uint32), want.view(np.uint32))
        blk = ops.quantize_activation_blocked(d(xx), d(tt), d(cb), bits).reshape(-1)
        assert np.array_equal(_np(blk).view(np.uint16),
                              _np(_to_blocked(torch.from_numpy(want.astype(np.float16)))).view(np.uint16))
        h = xx.to(torch.float16)
        want16 = oracle.act_quant_c(h.float().numpy(), tt, cb, bits, 64)["x_hat"].astype(np.float16)
        assert np.array_equal(_np(ops.dequant_activation_hip(d(h), d(tt), d(cb), 64)).view(np.uint16), want16.view(np.uint16))

    ref0 = oracle.act_quant_c(x.numpy(), synth.midpoint_thresholds(cb), cb, bits, 64)
    t = ((x.numpy().reshape(640, 6, 64) - ref0["center"][..., None]) / ref0["scale"][..., None]).astype(np.float32)
    u = np.sort(np.unique(t[np.abs(t) < 2.0]))
    ties = u[np.linspace(50, u.size - 51, n_thr).astype(np.int64)].copy()
    for thr in (ties, np.nextafter(ties, np.float32(-np.inf)), np.nextafter(ties, np.float32(np.inf))):
        thr = torch.from_numpy(thr.astype(np.float32))
        assert bool((thr[1:] - thr[:-1] > 0.13).all())          # wide apart: the coarse bucket table is in use
        check(x, thr)
    grid = torch.linspace(-1.75, 1.75, n_thr).mul(8).round().div(8)          # round values: 0, 1/4, 1/2 ...
    check(x, grid)
    for scale in (4.0, 8.0):                   # a grid shifted by a fraction of a bucket
        edge = (grid * scale - 0.381966) / scale
        check(x, edge)
        check(x, torch.from_numpy(np.nextafter(edge.numpy(), np.float32(np.inf))))
        check(x, edge + 3.0e-6)
    big = synth.make_activation(12608, 384, 18)
    check(big, synth.midpoint_thresholds(cb))


def test_stage1_empty(cuda):
    cb, thr = _cb(4)
    out = ops.quantize_activation(torch.zeros((0, 128), device=cuda), thr.to(cuda), cb.to(cuda), 4, 64)
    assert tuple(out[0].shape) == (0, 64) and tuple(out[1].shape) == (0, 2)


def test_stage1_torch_order_tie_audit(cuda, oracle):
    """Against the torch restatement (torch's own reduction order) codes may differ only at near-ties."""
    bits = 4
    cb, thr = _cb(bits)
    x = synth.make_activation(197, 384, 55)
    codes = _np(ops.quantize_activation_u8(x.to(cuda), thr.to(cuda), cb.to(cuda), bits, 64)[0])
    codes_t, _, _, _, _ = oracle.act_quant_torch(x, thr, cb, 64)
    diff = np.argwhere(codes != codes_t.numpy())
    assert len(diff) < 1e-3 * x.numel()
    x64 = x.double().reshape(197, -1, 64)
    mu = x64.mean(-1, keepdim=True)
    t64 = ((x64 - mu) / ((x64 - mu).square().mean(-1, keepdim=True) + 1e-6).sqrt()).reshape(197, 384).numpy()
    for r, c in diff:
        assert np.min(np.abs(thr.double().numpy() - t64[r, c])) < 4e-6 * max(1.0, abs(t64[r, c]))


# ------------------------------------------------------------------------------------------------
# stage 2
# ------------------------------------------------------------------------------------------------
def _packed_weight(oracle, n, k, bits, seed, gs=64):
    cb, thr = _cb(bits)
    w = synth.make_weight(n, k, seed)
    codes, center, scale, code_sum = oracle.quantize_weight_torch(w, thr, cb, gs, 1e-6)
    packed = torch.from_numpy(oracle.pack_codes_np(codes.numpy(), bits))
    return cb, packed, center, scale, code_sum


@pytest.mark.parametrize("bits", [2, 3, 4])
@pytest.mark.parametrize("n,k", [(768, 192), (384, 1536), (1152, 384), (5, 64)])
def test_stage2_bitexact(cuda, oracle, bits, n, k):
    cb, packed, center, scale, code_sum = _packed_weight(oracle, n, k, bits, 9)
    ref = oracle.weight_dequant_c(packed.numpy(), cb, center, scale, code_sum, bits, 64, fma=True)
    got = ops.unpack_weight_hip(packed.to(cuda), cb.to(cuda), center.to(cuda), scale.to(cuda), code_sum.to(cuda),
                                bits, 64)
    assert got.dtype == torch.float16 and tuple(got.shape) == (n, k)
    assert np.array_equal(_np(got).view(np.uint16), ref.astype(np.float16).view(np.uint16))
    out32 = torch.empty((n, k), dtype=torch.float32, device=cuda)
    ops.unpack_weight_hip(packed.to(cuda), cb.to(cuda), center.to(cuda), scale.to(cuda), code_sum.to(cuda), bits, 64,
                          out=out32)
    assert np.array_equal(_np(out32), ref)
    # against the two-rounding torch formulation: at most one fp16 ulp apart
    torch_w = oracle.unpack_weight_torch(packed, cb, center, scale, code_sum, bits, 64)
    d = np.abs(_np(got).view(np.int16).astype(np.int32) - torch_w.numpy().view(np.int16).astype(np.int32))
    assert d.max() <= 1 and (d != 0).mean() < 1e-3


def test_stage2_shared_buffer_and_odd_group(cuda, oracle):
    cb, packed, center, scale, code_sum = _packed_weight(oracle, 10, 96, 3, 4, gs=12)
    ref = oracle.weight_dequant_c(packed.numpy(), cb, center, scale, code_sum, 3, 12, fma=True)
    buf = torch.zeros(4096, dtype=torch.float16, device=cuda)
    out = ops.unpack_weight_hip(packed.to(cuda), cb.to(cuda), center.to(cuda), scale.to(cuda), code_sum.to(cuda),
                                3, 12, out=buf)
    assert out.data_ptr() == buf.data_ptr()
    assert np.array_equal(_np(buf[:960]).view(np.uint16), ref.astype(np.float16).ravel().view(np.uint16))
    assert not buf[960:].any()


# ------------------------------------------------------------------------------------------------
# stages 2+3 fused, whole layer
# ------------------------------------------------------------------------------------------------
def _gemm_tol(mag, k):
    """fp32 accumulation of exact fp16 products in any order: |err| <= (K+1) * 2^-24 * sum|a*w|
    (standard forward bound, gamma_K with u = 2^-24), plus one rounding of the result."""
    return (k + 2) * 2.0 ** -24 * mag


def _check_fused(cuda, oracle, m, n, k, bits, seed, with_bias=True, out_dtype=torch.float32):
    cb, packed, center, scale, code_sum = _packed_weight(oracle, n, k, bits, seed)
    kind = "gelu" if k > n else "ln"
    _, thr = _cb(bits)
    x = synth.make_activation(m, k, seed, kind)
    a = oracle.act_quant_c(x.numpy(), thr, cb, bits, 64)["x_hat"].astype(np.float16)
    w = oracle.weight_dequant_c(packed.numpy(), cb, center, scale, code_sum, bits, 64, fma=True).astype(np.float16)
    bias = synth.make_bias(n, seed) if with_bias else None
    y64, mag = oracle.linear_f64_c(a, w, None if bias is None else bias.numpy())
    y = ops.linear_fused(torch.from_numpy(a).to(cuda), packed.to(cuda), cb.to(cuda), center.to(cuda), scale.to(cuda),
                         code_sum.to(cuda), None if bias is None else bias.to(cuda), bits, 64, out_dtype=out_dtype)
    assert y.dtype == out_dtype and tuple(y.shape) == (m, n)
    got = _np(y).astype(np.float64)
    tol = _gemm_tol(mag, k)
    if out_dtype == torch.float16:
        tol = tol + np.abs(y64) * 2.0 ** -11 + 2.0 ** -25          # one fp16 rounding of the result
    assert np.all(np.abs(got - y64) <= tol), float(np.max(np.abs(got - y64) / tol))
    return y, y64


@pytest.mark.parametrize("bits", [2, 3, 4])
@pytest.mark.parametrize("m,n,k", [(197, 768, 192), (197, 1152, 384), (197, 384, 384), (197, 1536, 384),
                                   (197, 384, 1536), (1, 128, 64), (130, 200, 128), (64, 128, 64), (129, 129, 192)])
def test_fused_gemm_vs_fp64(cuda, oracle, bits, m, n, k):
    _check_fused(cuda, oracle, m, n, k, bits, seed=17)


def test_fused_gemm_fp16_out_no_bias_and_large_tile(cuda, oracle):
    _check_fused(cuda, oracle, 197, 384, 384, 4, seed=3, with_bias=False, out_dtype=torch.float16)
    _check_fused(cuda, oracle, 2100, 1152, 384, 4, seed=5, out_dtype=torch.float16)   # takes the 128-row tile
    _check_fused(cuda, oracle, 2100, 1152, 384, 3, seed=6, out_dtype=torch.float32)


@pytest.mark.parametrize("bits,out_dtype", [(4, torch.float16), (3, torch.float32), (2, torch.float16)])
@pytest.mark.parametrize("m,n,k", [(2100, 1152, 384),     # several passes per wave, K in one slab slice
                                   (1000, 200, 448),      # ragged N, 7 groups: a full slice plus a one-group slice
                                   (700, 130, 64),        # one group, last slab two columns wide
                                   (1500, 384, 1536),     # four slab slices
                                   (515, 520, 832)])      # 13 groups, ragged M and N
def test_fused_gemm_kernel_variants(cuda, oracle, monkeypatch, bits, out_dtype, m, n, k):
    """Every kernel behind arcq_linear_fused (pinned through ARCQ_GEMM_KERNEL) meets the fp64 bound, and the two
    large-M kernels, which accumulate in the same k order, agree bit for bit."""
    outs = {}
    for kern in ("stream", "slab", "small", "splitk"):
        monkeypatch.setenv("ARCQ_GEMM_KERNEL", kern)
        outs[kern], _ = _check_fused(cuda, oracle, m, n, k, bits, seed=29, out_dtype=out_dtype)
    monkeypatch.delenv("ARCQ_GEMM_KERNEL")
    assert torch.equal(outs["stream"], outs["slab"])
    auto, _ = _check_fused(cuda, oracle, m, n, k, bits, seed=29, out_dtype=out_dtype)
    assert torch.equal(auto, outs["slab"])


@pytest.mark.parametrize("bits,out_dtype", [(4, torch.float16), (3, torch.float32), (2, torch.float16)])
@pytest.mark.parametrize("m,n,k", [(1500, 384, 1536),     # four slab slices: the shape class the workspace is chosen for
                                   (1000, 200, 448),      # ragged N, a full slice plus a one-group slice
                                   (700, 130, 64),        # one group, last slab two columns wide
                                   (515, 520, 1216),      # 19 groups, ragged M and N
                                   (197, 384, 1536)])     # below 512 rows: the workspace is never used
def test_fused_gemm_weight_workspace(cuda, oracle, monkeypatch, bits, out_dtype, m, n, k):
    """arcq_linear_fused_ws: with a weight workspace the result is bit-identical to the one without, both when the
    library chooses (no override) and when the copy-from-workspace kernel is pinned; a pinned run leaves the
    reconstructed fp16 weight in the workspace, bit-equal to the oracle's; a run that does not take the workspace
    leaves it untouched."""
    cb, packed, center, scale, code_sum = _packed_weight(oracle, n, k, bits, 37)
    _, thr = _cb(bits)
    x = synth.make_activation(m, k, 37, "gelu" if k > n else "ln")
    a = torch.from_numpy(oracle.act_quant_c(x.numpy(), thr, cb, bits, 64)["x_hat"].astype(np.float16)).to(cuda)
    bias = synth.make_bias(n, 37).to(cuda)
    w = [t.to(cuda) for t in (packed, cb, center, scale, code_sum)]
    run = lambda ws: ops.linear_fused(a, *w, bias, bits, 64, out_dtype=out_dtype, w_hat_ws=ws)
    monkeypatch.delenv("ARCQ_GEMM_KERNEL", raising=False)
    plain = run(None)
    ws = torch.full((n * k + 8,), -3.0, dtype=torch.float16, device=cuda)   # longer than needed: the tail stays
    assert torch.equal(run(ws), plain)
    ws.fill_(-3.0)
    monkeypatch.setenv("ARCQ_GEMM_KERNEL", "prebuilt")
    assert torch.equal(run(ws), plain)
    monkeypatch.delenv("ARCQ_GEMM_KERNEL")
    got = _np(ws)
    assert np.all(got[n * k:] == np.float16(-3.0))
    if m >= 512:
        want = oracle.weight_dequant_c(packed.numpy(), cb, center, scale, code_sum, bits, 64, fma=True).astype(np.float16)
        assert np.array_equal(got[:n * k].view(np.uint16), want.reshape(-1).view(np.uint16))
    else:
        assert np.all(got == np.float16(-3.0))
    monkeypatch.setenv("ARCQ_GEMM_KERNEL", "stream")                       # another pinned kernel ignores the workspace
    ws.fill_(-3.0)
    assert torch.equal(run(ws), run(None))
    assert bool((ws == -3.0).all())


def test_layer_otf_weight_workspace(cuda, oracle, monkeypatch):
    """arcq_linear_otf_ws with both workspaces == without the weight workspace, on the shape the library picks the
    workspace for (fc2 of DeiT-S at 8 images) and through the module's ``_weight_buffer`` attribute."""
    from arcq_vit_amd.packed_on_the_fly import ARCQPackedLinearOnTheFly
    m, n, k, bits = 1576, 384, 1536, 4
    monkeypatch.delenv("ARCQ_GEMM_KERNEL", raising=False)
    cb, packed, center, scale, code_sum = _packed_weight(oracle, n, k, bits, 41)
    _, thr = _cb(bits)
    bias = synth.make_bias(n, 41)
    x = synth.make_activation(m, k, 41, "gelu").to(torch.float16).to(cuda)
    d = lambda t: t.to(cuda)
    args = (d(thr), d(cb), d(packed), d(cb), d(center), d(scale), d(code_sum), d(bias), bits, 64)
    plain = ops.linear_otf(x, *args, out_dtype=torch.float16)
    xw = torch.empty((m, k), dtype=torch.float16, device=cuda)
    ww = torch.zeros(n * k, dtype=torch.float16, device=cuda)
    assert torch.equal(ops.linear_otf(x, *args, out_dtype=torch.float16, x_hat_ws=xw, w_hat_ws=ww), plain)
    assert bool((ww != 0).any())                    # the library took the workspace for this shape
    layer = ARCQPackedLinearOnTheFly(k, n, True, d(packed), d(cb), d(center), d(scale), d(code_sum), d(cb), d(thr),
                                     bits, 64, d(bias))
    y0 = layer(x)
    layer._weight_buffer = torch.zeros(n * k + 64, dtype=torch.float16, device=cuda)
    assert torch.equal(layer(x), y0) and torch.equal(y0, plain)
    assert bool((layer._weight_buffer != 0).any())
    layer._weight_buffer = torch.zeros(16, dtype=torch.float16, device=cuda)
    with pytest.raises(ValueError):
        layer(x)


def _to_blocked(t):
    """Row-major [M, K] -> the 32-row block layout, flat: whole blocks as [M/32, K/8, 32, 8], then a last block of
    r = M % 32 rows as [K/8, r, 8]."""
    m, k = t.shape
    full = (m // 32) * 32
    parts = [t[:full].reshape(m // 32, 32, k // 8, 8).permute(0, 2, 1, 3).reshape(-1)]
    if full < m:
        parts.append(t[full:].reshape(m - full, k // 8, 8).permute(1, 0, 2).reshape(-1))
    return torch.cat(parts).contiguous()


@pytest.mark.parametrize("bits", [2, 3, 4])
@pytest.mark.parametrize("m,k,in_dtype", [(64, 384, torch.float16), (96, 448, torch.float32),    # 7 groups: a half-empty tile
                                          (32, 64, torch.float16),                               # one group per row
                                          (70, 384, torch.float16), (5, 64, torch.float32),      # a ragged last block
                                          (1024, 1536, torch.float16), (160, 832, torch.float32),
                                          (2752, 1536, torch.float16),     # 2 064 tiles: no builder wave, one tile per wave
                                          (6000, 1536, torch.float16),     # 4 512 tiles on 1 024 workgroups: waves walk 1-2 tiles, ragged end
                                          (4500, 1024, torch.float32),     # fp32 input without the builder wave
                                          (9001, 1024, torch.float32),     # fp32 input, waves walk 1-2 tiles, ragged end
                                          (12608, 1536, torch.float16)])   # the benchmark's largest stage 1: 2-3 tiles per wave
def test_stage1_block_layout(cuda, oracle, bits, m, k, in_dtype):
    """arcq_act_quant_blocked writes the values of the row-major stage 1 (and of the oracle), bit for bit, at
    [row / 32][k / 8][row % 32][k % 8]."""
    cb, thr = _cb(bits)
    x = synth.make_activation(m, k, 43, "gelu").to(in_dtype)
    want = oracle.act_quant_c(x.float().numpy(), thr, cb, bits, 64)["x_hat"].astype(np.float16)
    got = ops.quantize_activation_blocked(x.to(cuda), thr.to(cuda), cb.to(cuda), bits)
    assert tuple(got.shape) == ((m // 32, k // 8, 32, 8) if m % 32 == 0 else (m * k,)) and got.dtype == torch.float16
    got = got.reshape(-1)
    assert np.array_equal(_np(got).view(np.uint16), _np(_to_blocked(torch.from_numpy(want))).view(np.uint16))
    if in_dtype == torch.float16:
        assert torch.equal(_to_blocked(ops.dequant_activation_hip(x.to(cuda), thr.to(cuda), cb.to(cuda), 64)), got)
    # a larger out buffer is only written where the layout says
    buf = torch.full((m * k + 64,), -3.0, dtype=torch.float16, device=cuda)
    ops.quantize_activation_blocked(x.to(cuda), thr.to(cuda), cb.to(cuda), bits, out=buf)
    assert torch.equal(buf[:m * k], got) and bool((buf[m * k:] == -3.0).all())


@pytest.mark.parametrize("bits,out_dtype", [(4, torch.float16), (3, torch.float32), (2, torch.float16)])
@pytest.mark.parametrize("m,n,k", [(1504, 384, 1536),     # four slab slices; 47 blocks over 8 waves
                                   (1024, 200, 448),      # ragged N, a full slice plus a one-group slice (ring rotation by 1)
                                   (704, 130, 64),        # one group, last slab two columns wide
                                   (512, 520, 832),       # 13 groups (ring rotation by 1), ragged N
                                   (544, 256, 512),       # 8 groups: last slice of two (ring rotation by 2)
                                   (2112, 1152, 384),     # K in one slice, several passes per wave
                                   (1000, 200, 448), (531, 130, 64),      # a ragged last block (8 and 19 rows)
                                   (32, 128, 128), (7, 64, 128)])         # a single row block: seven waves idle
def test_fused_gemm_block_layout(cuda, oracle, monkeypatch, bits, out_dtype, m, n, k):
    """arcq_linear_fused_blocked on x_hat in the block layout == arcq_linear_fused on the same x_hat row-major: within
    the fp64 bound, bit-identical to the four-wave weight-stationary kernel (same k order), with and without a weight
    workspace and a bias."""
    monkeypatch.setenv("ARCQ_GEMM_KERNEL", "slab")
    ref, _ = _check_fused(cuda, oracle, m, n, k, bits, seed=47, out_dtype=out_dtype)
    monkeypatch.delenv("ARCQ_GEMM_KERNEL")
    cb, packed, center, scale, code_sum = _packed_weight(oracle, n, k, bits, 47)
    _, thr = _cb(bits)
    x = synth.make_activation(m, k, 47, "gelu" if k > n else "ln")
    a = torch.from_numpy(oracle.act_quant_c(x.numpy(), thr, cb, bits, 64)["x_hat"].astype(np.float16))
    xb = _to_blocked(a).to(cuda)
    bias = synth.make_bias(n, 47).to(cuda)
    w = [t.to(cuda) for t in (packed, cb, center, scale, code_sum)]
    y = ops.linear_fused_blocked(xb, m, k, *w, bias, bits, out_dtype=out_dtype)
    assert y.dtype == out_dtype and tuple(y.shape) == (m, n)
    if m >= 512:
        assert torch.equal(y, ref)
    else:       # below 512 rows the row-major entry point takes the split-K kernel: another summation order
        assert torch.allclose(y.float(), ref.float(), rtol=2e-3, atol=2e-3)
    ws = torch.full((n * k + 8,), -3.0, dtype=torch.float16, device=cuda)
    monkeypatch.setenv("ARCQ_GEMM_KERNEL", "prebuilt")
    assert torch.equal(ops.linear_fused_blocked(xb, m, k, *w, bias, bits, out_dtype=out_dtype, w_hat_ws=ws), y)
    monkeypatch.delenv("ARCQ_GEMM_KERNEL")
    want_w = oracle.weight_dequant_c(packed.numpy(), cb, center, scale, code_sum, bits, 64, fma=True).astype(np.float16)
    assert np.array_equal(_np(ws)[:n * k].view(np.uint16), want_w.reshape(-1).view(np.uint16))
    assert bool((ws[n * k:] == -3.0).all())
    assert torch.equal(ops.linear_fused_blocked(xb, m, k, *w, bias, bits, out_dtype=out_dtype, w_hat_ws=ws), y)   # library's choice
    # stage 1 with the weight reconstruction carried in its launch, then the GEMM on weights that are ready
    ws2 = torch.full((n * k + 8,), -3.0, dtype=torch.float16, device=cuda)
    xb2 = ops.quantize_activation_blocked(x.to(cuda), thr.to(cuda), cb.to(cuda), bits, weights=w, w_hat=ws2)
    assert torch.equal(xb2.reshape(-1), xb)
    assert np.array_equal(_np(ws2)[:n * k].view(np.uint16), want_w.reshape(-1).view(np.uint16))
    assert bool((ws2[n * k:] == -3.0).all())
    assert torch.equal(ops.linear_fused_blocked(xb2, m, k, *w, bias, bits, out_dtype=out_dtype, w_hat_ws=ws2,
                                                w_hat_ready=True), y)
    nb = ops.linear_fused_blocked(xb, m, k, *w, None, bits, out_dtype=torch.float32)
    yb = ops.linear_fused_blocked(xb, m, k, *w, bias, bits, out_dtype=torch.float32)
    assert torch.equal(nb + bias, yb)            # the bias is one fp32 addition before the output rounding


@pytest.mark.parametrize("bits,out_dtype", [(4, torch.float16), (3, torch.float32)])
@pytest.mark.parametrize("m,n,k", [(8960 + 7, 4096, 128),     # 8 ranges of 35-36 blocks: two full passes of pairs, 3-4 left (halves), ragged last block
                                   (10496, 4000, 192),        # 41 blocks per range: two full passes, 1 pair + 7 single blocks; ragged N
                                   (7936, 4096, 64),          # 31 blocks: one full pass, 7 pairs + 1 single block
                                   (4096, 4096, 448),         # 16 blocks, two slices: exactly one full pass, nothing left
                                   (3000, 1000, 832),         # 94 blocks over 32 ranges: 3 per workgroup (no full pass), three slices, ragged M and N
                                   (12608, 768, 768),         # DeiT-B proj: 10 blocks per workgroup: 2 pairs + 6 singles, two slices
                                   (6400, 2304, 1024)])       # 200 blocks over 14 ranges of 15: 7 pairs + 1 single, three slices
def test_fused_gemm_pair_kernel(cuda, oracle, monkeypatch, bits, out_dtype, m, n, k):
    """gemm_pair_kernel (two row blocks per wave and pass, weights ready in a workspace) against gemm_slab8_kernel on
    the same operands: bit-identical (same k order per output), whichever way a workgroup's blocks fall into pairs,
    single blocks and column halves; sampled rows against the fp64 oracle."""
    cb, packed, center, scale, code_sum = _packed_weight(oracle, n, k, bits, 61)
    _, thr = _cb(bits)
    x = synth.make_activation(m, k, 61, "gelu" if k > n else "ln").to(torch.float16)
    bias = synth.make_bias(n, 61).to(cuda)
    w = [t.to(cuda) for t in (packed, cb, center, scale, code_sum)]
    ws = torch.empty(n * k, dtype=torch.float16, device=cuda)
    xb = ops.quantize_activation_blocked(x.to(cuda), thr.to(cuda), cb.to(cuda), bits, weights=w, w_hat=ws)
    monkeypatch.setenv("ARCQ_PAIR", "0")
    ref = ops.linear_fused_blocked(xb, m, k, *w, bias, bits, out_dtype=out_dtype, w_hat_ws=ws, w_hat_ready=True)
    for variant in ("1", "2"):          # one slab buffer of six groups / two of three with the copy under the multiplication
        monkeypatch.setenv("ARCQ_PAIR", variant)
        y = ops.linear_fused_blocked(xb, m, k, *w, bias, bits, out_dtype=out_dtype, w_hat_ws=ws, w_hat_ready=True)
        assert torch.equal(y, ref), variant
    monkeypatch.delenv("ARCQ_PAIR")
    rows = torch.randint(0, m, (40,), generator=torch.Generator().manual_seed(2))
    rows[0], rows[1] = 0, m - 1
    a = oracle.act_quant_c(x[rows].float().numpy(), thr, cb, bits, 64)["x_hat"].astype(np.float16)
    w16 = oracle.weight_dequant_c(packed.numpy(), cb, center, scale, code_sum, bits, 64, fma=True).astype(np.float16)
    y64, mag = oracle.linear_f64_c(a, w16, _np(bias))
    tol = _gemm_tol(mag, k)
    if out_dtype == torch.float16:
        tol = tol + np.abs(y64) * 2.0 ** -11 + 2.0 ** -25
    assert np.all(np.abs(_np(y[rows.to(cuda)]).astype(np.float64) - y64) <= tol)


@pytest.mark.parametrize("m", [1504, 1576])     # whole 32-row blocks / a last block of 8 rows
def test_layer_otf_scratch_workspaces(cuda, oracle, monkeypatch, m):
    """arcq_linear_otf_ws (scratch-only workspaces) == arcq_linear_otf bit for bit, whichever layout it uses inside."""
    n, k, bits = 384, 1536, 4
    monkeypatch.delenv("ARCQ_GEMM_KERNEL", raising=False)
    cb, packed, center, scale, code_sum = _packed_weight(oracle, n, k, bits, 53)
    _, thr = _cb(bits)
    bias = synth.make_bias(n, 53)
    x = synth.make_activation(m, k, 53, "gelu").to(torch.float16).to(cuda)
    d = lambda t: t.to(cuda)
    args = (d(thr), d(cb), d(packed), d(cb), d(center), d(scale), d(code_sum), d(bias), bits, 64)
    xw = torch.empty((m, k), dtype=torch.float16, device=cuda)
    plain = ops.linear_otf(x, *args, out_dtype=torch.float16, x_hat_ws=xw)
    want_xhat = oracle.act_quant_c(x.float().cpu().numpy(), thr, cb, bits, 64)["x_hat"].astype(np.float16)
    assert np.array_equal(_np(xw).view(np.uint16), want_xhat.view(np.uint16))       # row-major without `scratch`
    xs = torch.empty((m, k), dtype=torch.float16, device=cuda)
    assert torch.equal(ops.linear_otf(x, *args, out_dtype=torch.float16, x_hat_ws=xs, scratch=True), plain)
    assert torch.equal(xs.reshape(-1), _to_blocked(xw))        # 512 rows or more: the block layout inside
    ww = torch.zeros(n * k, dtype=torch.float16, device=cuda)
    assert torch.equal(ops.linear_otf(x, *args, out_dtype=torch.float16, x_hat_ws=xs, w_hat_ws=ww), plain)
    want_w = oracle.weight_dequant_c(packed.numpy(), cb, center, scale, code_sum, bits, 64, fma=True).astype(np.float16)
    assert np.array_equal(_np(ww).view(np.uint16), want_w.reshape(-1).view(np.uint16))   # rebuilt in the stage-1 launch
    y32 = ops.linear_otf(x.float(), *args, out_dtype=torch.float32, scratch=True)   # fp32 in, fp32 out
    assert torch.allclose(y32, plain.float(), rtol=2e-3, atol=2e-3)


@pytest.mark.parametrize("m,n,k,bits,out_dtype", [(513, 7, 64, 2, torch.float16),        # one group, N below a vector store
                                                  (600, 33, 128, 3, torch.float32),
                                                  (1000, 129, 64, 4, torch.float16),     # second slab one column wide
                                                  (2048, 40000, 64, 4, torch.float16),   # more slabs than compute units
                                                  (700, 257, 2560, 3, torch.float32)])   # 40 groups: seven slab slices
def test_layer_otf_block_layout_odd_shapes(cuda, oracle, monkeypatch, m, n, k, bits, out_dtype):
    """Whole layer from 512 rows on (block layout, eight-wave GEMM, weights copied or rebuilt in the kernel) against the
    row-major four-wave kernel on awkward shapes: bit-identical."""
    cb, packed, center, scale, code_sum = _packed_weight(oracle, n, k, bits, 61)
    _, thr = _cb(bits)
    bias = synth.make_bias(n, 61)
    x = synth.make_activation(m, k, 61, "ln").to(torch.float16).to(cuda)
    d = lambda t: t.to(cuda)
    args = (x, d(thr), d(cb), d(packed), d(cb), d(center), d(scale), d(code_sum), d(bias), bits, 64)
    monkeypatch.setenv("ARCQ_GEMM_KERNEL", "slab")
    ref = ops.linear_otf(*args, out_dtype=out_dtype)
    monkeypatch.delenv("ARCQ_GEMM_KERNEL")
    ww = torch.empty(n * k, dtype=torch.float16, device=cuda)
    assert torch.equal(ops.linear_otf(*args, out_dtype=out_dtype, scratch=True), ref)
    assert torch.equal(ops.linear_otf(*args, out_dtype=out_dtype, w_hat_ws=ww), ref)
    monkeypatch.setenv("ARCQ_GEMM_KERNEL", "slab8")          # block layout, weights rebuilt inside the GEMM
    assert torch.equal(ops.linear_otf(*args, out_dtype=out_dtype, w_hat_ws=ww), ref)


@pytest.mark.parametrize("bits,in_dtype", [(3, torch.float32), (2, torch.float16)])
def test_layer_otf_weights_rebuilt_in_stage1_launch(cuda, oracle, monkeypatch, bits, in_dtype):
    """Whole layer in the block layout with a weight workspace (ragged N, seven groups, fp32 / fp16 input): the weights
    rebuilt alongside stage 1 equal the oracle's and y equals the path without workspaces, bit for bit."""
    m, n, k = 512, 200, 448
    monkeypatch.delenv("ARCQ_GEMM_KERNEL", raising=False)
    cb, packed, center, scale, code_sum = _packed_weight(oracle, n, k, bits, 59)
    _, thr = _cb(bits)
    bias = synth.make_bias(n, 59)
    x = synth.make_activation(m, k, 59, "ln").to(in_dtype).to(cuda)
    d = lambda t: t.to(cuda)
    args = (d(thr), d(cb), d(packed), d(cb), d(center), d(scale), d(code_sum), d(bias), bits, 64)
    plain = ops.linear_otf(x, *args, out_dtype=torch.float32)
    ww = torch.full((n * k + 8,), -3.0, dtype=torch.float16, device=cuda)
    assert torch.equal(ops.linear_otf(x, *args, out_dtype=torch.float32, w_hat_ws=ww), plain)
    want_w = oracle.weight_dequant_c(packed.numpy(), cb, center, scale, code_sum, bits, 64, fma=True).astype(np.float16)
    assert np.array_equal(_np(ww)[:n * k].view(np.uint16), want_w.reshape(-1).view(np.uint16))
    assert bool((ww[n * k:] == -3.0).all())


@pytest.mark.parametrize("bits,out_dtype", [(4, torch.float16), (3, torch.float32), (2, torch.float32)])
@pytest.mark.parametrize("m,n,k", [(197, 1152, 384), (197, 384, 1536), (1, 70, 64), (65, 130, 1088), (300, 64, 4096)])
def test_fused_gemm_small_m_kernels(cuda, oracle, monkeypatch, bits, out_dtype, m, n, k):
    """Small-M shapes through the split-K kernel (the default below 512 rows) and the tiled small kernel; the split-K
    reduction order is fixed, so two launches agree bit for bit."""
    monkeypatch.setenv("ARCQ_GEMM_KERNEL", "small")
    _check_fused(cuda, oracle, m, n, k, bits, seed=31, out_dtype=out_dtype)
    monkeypatch.setenv("ARCQ_GEMM_KERNEL", "splitk")
    a, _ = _check_fused(cuda, oracle, m, n, k, bits, seed=31, out_dtype=out_dtype)
    monkeypatch.delenv("ARCQ_GEMM_KERNEL")
    b, _ = _check_fused(cuda, oracle, m, n, k, bits, seed=31, out_dtype=out_dtype)
    assert torch.equal(a, b)


@pytest.mark.parametrize("bits", [3, 4])
def test_layer_otf_matches_stagewise(cuda, oracle, bits):
    """arcq_linear_otf == stage 1 then fused GEMM, and its activation matches the oracle bit for bit."""
    m, n, k = 197, 1152, 384
    cb, packed, center, scale, code_sum = _packed_weight(oracle, n, k, bits, 23)
    _, thr = _cb(bits)
    bias = synth.make_bias(n, 23)
    x = synth.make_activation(m, k, 23).to(torch.float16)
    d = lambda t: t.to(cuda)
    ws = torch.empty((m, k), dtype=torch.float16, device=cuda)
    y = ops.linear_otf(d(x), d(thr), d(cb), d(packed), d(cb), d(center), d(scale), d(code_sum), d(bias), bits, 64,
                       out_dtype=torch.float16, x_hat_ws=ws)
    want_xhat = oracle.act_quant_c(x.float().numpy(), thr, cb, bits, 64)["x_hat"].astype(np.float16)
    assert np.array_equal(_np(ws).view(np.uint16), want_xhat.view(np.uint16))
    y2 = ops.linear_fused(ws, d(packed), d(cb), d(center), d(scale), d(code_sum), d(bias), bits, 64,
                          out_dtype=torch.float16)
    assert torch.equal(y, y2)
    w = oracle.weight_dequant_c(packed.numpy(), cb, center, scale, code_sum, bits, 64).astype(np.float16)
    y64, mag = oracle.linear_f64_c(want_xhat, w, bias.numpy())
    tol = _gemm_tol(mag, k) + np.abs(y64) * 2.0 ** -11 + 2.0 ** -25
    assert np.all(np.abs(_np(y).astype(np.float64) - y64) <= tol)
    # against the fake-quant fp32 reference path (torch order, unrounded operands): fp16-level agreement
    fq = oracle.fake_quant_linear(x.float(), synth.make_weight(n, k, 23), bias, thr, cb, thr, cb, 64, 1e-6)
    cos = torch.nn.functional.cosine_similarity(y.float().cpu().flatten(), fq.flatten(), dim=0)
    assert cos > 0.9999
    assert (y.float().cpu() - fq).abs().max() < 2e-2 * fq.abs().max()


@pytest.mark.parametrize("bits,x_dtype,out_dtype", [(4, torch.float16, torch.float16), (3, torch.float32, torch.float32),
                                                    (2, torch.float16, torch.float32), (4, torch.float32, torch.float16)])
@pytest.mark.parametrize("m,n,k", [(197, 1152, 384), (1, 70, 64),
                                   (197, 768, 768),       # six 64-group tiles per row tile: two waves build the tables
                                   (100, 96, 1024),       # eight tiles: every wave has one, all build the tables
                                   (65, 130, 1088),       # nine tiles, and the partial tiles reuse the x_hat tile's LDS
                                   (197, 384, 1536), (500, 384, 1536),      # twelve tiles: two rounds for four waves
                                   (500, 64, 2048), (33, 200, 2112)])       # beyond the single launch: two launches
def test_layer_otf_single_launch(cuda, oracle, monkeypatch, bits, x_dtype, out_dtype, m, n, k):
    """Below 512 rows arcq_linear_otf can run the whole layer in one launch (ARCQ_OTF_FUSED=2: whenever K fits LDS; =1,
    the default: where that is faster; =0: never); all three must agree bit for bit, in y and in the x_hat workspace,
    and x_hat must equal the oracle's."""
    cb, packed, center, scale, code_sum = _packed_weight(oracle, n, k, bits, 37)
    _, thr = _cb(bits)
    bias = synth.make_bias(n, 37)
    x = synth.make_activation(m, k, 37, "gelu" if k > n else "ln").to(x_dtype)
    d = lambda t: t.to(cuda)
    args = (d(x), d(thr), d(cb), d(packed), d(cb), d(center), d(scale), d(code_sum), d(bias), bits, 64)
    outs = []
    for flag in ("2", "0", "1"):
        monkeypatch.setenv("ARCQ_OTF_FUSED", flag)
        ws = torch.full((m, k), float("nan"), dtype=torch.float16, device=cuda)
        y = ops.linear_otf(*args, out_dtype=out_dtype, x_hat_ws=ws)
        outs.append((y, ws))
    for other in outs[1:]:
        assert torch.equal(outs[0][0], other[0])
        assert torch.equal(outs[0][1], other[1])
    want_xhat = oracle.act_quant_c(x.float().numpy(), thr, cb, bits, 64)["x_hat"].astype(np.float16)
    assert np.array_equal(_np(outs[0][1]).view(np.uint16), want_xhat.view(np.uint16))
    w = oracle.weight_dequant_c(packed.numpy(), cb, center, scale, code_sum, bits, 64).astype(np.float16)
    y64, mag = oracle.linear_f64_c(want_xhat, w, bias.numpy())
    tol = _gemm_tol(mag, k) + (np.abs(y64) * 2.0 ** -11 + 2.0 ** -25 if out_dtype == torch.float16 else 0.0)
    assert np.all(np.abs(_np(outs[0][0]).astype(np.float64) - y64) <= tol)


def test_layer_otf_single_launch_fallback_thresholds(cuda, oracle):
    """Thresholds the bucket table cannot hold (two within one bucket) take the compare chain inside the fused kernel."""
    bits, m, n, k = 3, 130, 128, 256
    cb, packed, center, scale, code_sum = _packed_weight(oracle, n, k, bits, 39)
    thr = torch.tensor([-1.0, -0.5, -0.49, 0.0, 0.3, 0.31, 1.2], dtype=torch.float32)
    x = synth.make_activation(m, k, 39).to(torch.float16)
    d = lambda t: t.to(cuda)
    ws = torch.empty((m, k), dtype=torch.float16, device=cuda)
    ops.linear_otf(d(x), d(thr), d(cb), d(packed), d(cb), d(center), d(scale), d(code_sum), None, bits, 64,
                   out_dtype=torch.float16, x_hat_ws=ws)
    want = oracle.act_quant_c(x.float().numpy(), thr, cb, bits, 64)["x_hat"].astype(np.float16)
    assert np.array_equal(_np(ws).view(np.uint16), want.view(np.uint16))


# ------------------------------------------------------------------------------------------------
# index-space linears
# ------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("bits", [2, 3, 4])
@pytest.mark.parametrize("m,n,k", [(197, 768, 192), (33, 50, 128), (1, 1, 64)])
def test_index_linears_bitexact(cuda, oracle, bits, m, n, k):
    cb, packed_w, wc, ws, wcs = _packed_weight(oracle, n, k, bits, 41)
    _, thr = _cb(bits)
    x = synth.make_activation(m, k, 41)
    bias = synth.make_bias(n, 41)
    xa = oracle.act_quant_c(x.numpy(), thr, cb, bits, 64)
    table = (cb.view(-1, 1) * (cb * 1.25).view(1, -1)).float().contiguous()      # asymmetric on purpose
    wcodes = oracle.unpack_codes_u8_c(packed_w.numpy(), bits, k)
    d = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(cuda) if isinstance(a, np.ndarray) else a.to(cuda)
    for b in (bias, None):
        bn = None if b is None else b.numpy()
        want = oracle.linear_forward_packed_c(xa["packed"], xa["center"], xa["scale"], xa["code_sum"], packed_w.numpy(),
                                              wc, ws, wcs, table.numpy(), bn, bits, 64, k, n)
        got = ops.arcq_linear_forward(d(xa["packed"]), d(xa["center"]), d(xa["scale"]), d(xa["code_sum"]),
                                      d(packed_w), d(wc), d(ws), d(wcs), d(table), None if b is None else d(b),
                                      bits, 64, k, n)
        assert got.dtype == torch.float32 and np.array_equal(_np(got), want)
        want8 = oracle.linear_forward_u8_c(xa["codes"], xa["center"], xa["scale"], xa["code_sum"], wcodes, wc, ws,
                                           wcs, table.numpy(), bn, 64)
        got8 = ops.arcq_linear_forward_u8(d(xa["codes"]), d(xa["center"]), d(xa["scale"]), d(xa["code_sum"]),
                                          d(wcodes), d(wc), d(ws), d(wcs), d(table), None if b is None else d(b), 64)
        assert np.array_equal(_np(got8), want8)


def _index_case(oracle, m, n, k, bits, gs, seed):
    cb, packed_w, wc, ws, wcs = _packed_weight(oracle, n, k, bits, seed, gs=gs)
    _, thr = _cb(bits)
    x = synth.make_activation(m, k, seed)
    bias = synth.make_bias(n, seed)
    xa = oracle.act_quant_c(x.numpy(), thr, cb, bits, gs)
    table = (cb.view(-1, 1) * (cb * 1.25).view(1, -1)).float().contiguous()      # asymmetric on purpose
    wcodes = oracle.unpack_codes_u8_c(packed_w.numpy(), bits, k)
    return xa, packed_w.numpy(), wcodes, wc, ws, wcs, table, bias


def _index_both(cuda, oracle, case, bits, gs, k, n, rows=None):
    """Run both index-space formats on the GPU on all rows and compare the rows in ``rows`` (all if None) with the
    oracle evaluated on those rows only."""
    xa, packed_w, wcodes, wc, ws, wcs, table, bias = case
    d = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(cuda) if isinstance(a, np.ndarray) else a.to(cuda)
    sel = slice(None) if rows is None else rows
    got = ops.arcq_linear_forward(d(xa["packed"]), d(xa["center"]), d(xa["scale"]), d(xa["code_sum"]),
                                  d(packed_w), d(wc), d(ws), d(wcs), d(table), d(bias), bits, gs, k, n)
    want = oracle.linear_forward_packed_c(xa["packed"][sel], xa["center"][sel], xa["scale"][sel], xa["code_sum"][sel],
                                          packed_w, wc, ws, wcs, table.numpy(), bias.numpy(), bits, gs, k, n)
    assert got.dtype == torch.float32 and np.array_equal(_np(got)[sel], want)
    got8 = ops.arcq_linear_forward_u8(d(xa["codes"]), d(xa["center"]), d(xa["scale"]), d(xa["code_sum"]),
                                      d(wcodes), d(wc), d(ws), d(wcs), d(table), d(bias), gs)
    want8 = oracle.linear_forward_u8_c(xa["codes"][sel], xa["center"][sel], xa["scale"][sel], xa["code_sum"][sel],
                                       wcodes, wc, ws, wcs, table.numpy(), bias.numpy(), gs)
    assert np.array_equal(_np(got8)[sel], want8)


@pytest.mark.parametrize("bits", [2, 3, 4])
@pytest.mark.parametrize("m,n,k", [(2100, 300, 384), (8195, 71, 128)])
def test_index_linears_bitexact_many_tiles(cuda, oracle, bits, m, n, k):
    """Launches of more than 512 tiles of 16 rows x 64 outputs give every thread four outputs (a different
    instantiation from the one small launches take); rows % 16 and outputs % 64 are ragged on purpose."""
    assert ((m + 15) // 16) * ((n + 63) // 64) > 512
    _index_both(cuda, oracle, _index_case(oracle, m, n, k, bits, 64, 43), bits, 64, k, n)


@pytest.mark.parametrize("bits", [3, 4])
def test_index_linears_bitexact_batch64_sampled_rows(cuda, oracle, bits):
    """A DeiT-S projection at batch 64 (12 608 x 384 x 384: 4 728 tiles); the oracle is evaluated on 96 sampled rows
    that include the first and last tile and the ragged tail."""
    m, n, k = 12608, 384, 384
    rng = np.random.default_rng(5)
    rows = np.unique(np.concatenate([np.arange(0, 17), np.arange(m - 17, m), rng.integers(0, m, 62)]))
    _index_both(cuda, oracle, _index_case(oracle, m, n, k, bits, 64, 45), bits, 64, k, n, rows=rows)


@pytest.mark.parametrize("bits", [2, 3, 4])
@pytest.mark.parametrize("gs,m,n,k", [(32, 70, 45, 96), (128, 37, 50, 256), (16, 19, 33, 48)])
def test_index_linears_bitexact_other_group_sizes(cuda, oracle, bits, gs, m, n, k):
    """Group sizes other than 64 run the one-thread-per-output kernels."""
    _index_both(cuda, oracle, _index_case(oracle, m, n, k, bits, gs, 47), bits, gs, k, n)


# ------------------------------------------------------------------------------------------------
# argument errors surface as RuntimeError with the reference's wording
# ------------------------------------------------------------------------------------------------
def test_error_paths(cuda):
    cb, thr = _cb(4)
    x = torch.zeros((4, 128), device=cuda)
    with pytest.raises(RuntimeError, match="bits must be 2, 3, or 4"):
        ops.quantize_activation(x, thr.to(cuda), cb.to(cuda), 5, 64)
    with pytest.raises(RuntimeError, match="divisible by group_size"):
        ops.quantize_activation(x, thr.to(cuda), cb.to(cuda), 4, 48)
    with pytest.raises(RuntimeError, match="x must be float32"):
        ops.quantize_activation(x.half(), thr.to(cuda), cb.to(cuda), 4, 64)
    with pytest.raises(RuntimeError, match="x must be CUDA tensor"):
        ops.quantize_activation(x.cpu(), thr.to(cuda), cb.to(cuda), 4, 64)
    with pytest.raises(RuntimeError, match="codes must have shape"):
        ops.pack_codes(torch.zeros(8, dtype=torch.int64, device=cuda), 4)
    with pytest.raises(RuntimeError, match="packed must be uint8"):
        ops.unpack_codes(torch.zeros((2, 4), dtype=torch.int32, device=cuda), 4, 8)
    with pytest.raises(RuntimeError, match="only group_size 64"):
        ops.linear_fused(torch.zeros((4, 128), dtype=torch.float16, device=cuda),
                         torch.zeros((8, 64), dtype=torch.uint8, device=cuda), cb.to(cuda),
                         torch.zeros((8, 4), device=cuda), torch.ones((8, 4), device=cuda),
                         torch.zeros((8, 4), device=cuda), None, 4, 32)
    # the raw C ABI reports the same conditions as negative codes without launching anything
    from arcq_vit_amd import _lib
    lib = _lib.load()
    assert lib.arcq_pack_codes(0, 0, 4, 4, 7, 0) == -1
    assert lib.arcq_act_quant(x.data_ptr(), 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 4, 128, 4, 48, 1e-6, 0) == -2
    assert b"divisible" in lib.arcq_last_error()
    assert lib.arcq_act_quant(0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 4, 128, 4, 64, 1e-6, 0) == -3
    torch.cuda.synchronize()
