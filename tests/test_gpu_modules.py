"""GPU tests of the module layer and of the committed golden fixtures: the packed modules'
forwards (all runtime formats), checkpoint loading, the ViT skeleton (top-1 agreement against the
fake-quant model), HIP-graph replay, and size-independent properties at the benchmark's full
shapes."""
import os

import numpy as np
import pytest
import torch

import arcq_vit_amd as A
from arcq_vit_amd import ops, synth
from arcq_vit_amd.vit import build_fakequant_vit, build_packed_vit

pytestmark = pytest.mark.gpu
GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def _np(t):
    return t.detach().cpu().numpy()


@pytest.mark.parametrize("bits", [2, 3, 4])
def test_golden_fixtures(cuda, bits):
    """HIP results against the frozen vectors in tests/golden (no oracle call involved)."""
    g = np.load(os.path.join(GOLDEN, f"arcq_w{bits}a{bits}_g64.npz"))
    d = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(cuda)
    thr, cb = d(g["thresholds"]), d(g["codebook"])
    packed, center, scale, code_sum = ops.quantize_activation(d(g["x"]), thr, cb, bits, 64)
    assert np.array_equal(_np(packed), g["a32_packed"]) and np.array_equal(_np(center), g["a32_center"])
    assert np.array_equal(_np(scale), g["a32_scale"]) and np.array_equal(_np(code_sum), g["a32_code_sum"])
    assert np.array_equal(_np(ops.quantize_activation_u8(d(g["x"]), thr, cb, bits, 64)[0]), g["a32_codes"])
    assert np.array_equal(_np(ops.quantize_activation_dequant(d(g["x"]), thr, cb, bits, 64)), g["a32_x_hat"])
    xh16 = ops.dequant_activation_hip(d(g["x_f16"]), thr, cb, 64)
    assert np.array_equal(_np(xh16).view(np.uint16), g["a16_x_hat_f16"].view(np.uint16))
    w16 = ops.unpack_weight_hip(d(g["w_packed"]), cb, d(g["w_center"]), d(g["w_scale"]), d(g["w_code_sum"]), bits, 64)
    assert np.array_equal(_np(w16).view(np.uint16), g["w_dequant_f16"].view(np.uint16))
    assert np.array_equal(_np(ops.unpack_codes_u8(d(g["w_packed"]), bits, 128)), g["w_codes"])
    assert np.array_equal(_np(ops.pack_codes(d(g["w_codes"]).long(), bits)), g["w_packed"])
    y = ops.linear_otf(d(g["x_f16"]), thr, cb, d(g["w_packed"]), cb, d(g["w_center"]), d(g["w_scale"]),
                       d(g["w_code_sum"]), d(g["bias"]), bits, 64, out_dtype=torch.float32)
    tol = (128 + 2) * 2.0 ** -24 * g["y_abs_sum"]
    assert np.all(np.abs(_np(y).astype(np.float64) - g["y_f64"]) <= tol)
    yp = ops.arcq_linear_forward(d(g["a32_packed"]), d(g["a32_center"]), d(g["a32_scale"]), d(g["a32_code_sum"]),
                                 d(g["w_packed"]), d(g["w_center"]), d(g["w_scale"]), d(g["w_code_sum"]),
                                 d(g["product_table"]), d(g["bias"]), bits, 64, 128, 16)
    assert np.array_equal(_np(yp), g["y_index_packed"])
    yu = ops.arcq_linear_forward_u8(d(g["a32_codes"]), d(g["a32_center"]), d(g["a32_scale"]), d(g["a32_code_sum"]),
                                    d(g["w_codes"]), d(g["w_center"]), d(g["w_scale"]), d(g["w_code_sum"]),
                                    d(g["product_table"]), d(g["bias"]), 64)
    assert np.array_equal(_np(yu), g["y_index_u8"])


def _source(in_f, out_f, bits, seed=1, bias=True):
    src = A.QuantLinearPCARCQ(in_f, out_f, bias, bits, bits, 64)
    cb = synth.quantile_codebook(bits)
    src.act_quant.set_codebook(cb)
    src.weight_quant.set_codebook(cb)
    with torch.no_grad():
        src.linear.weight.copy_(synth.make_weight(out_f, in_f, seed))
        if bias:
            src.linear.bias.copy_(synth.make_bias(out_f, seed))
    return src.eval()


@pytest.mark.parametrize("bits", [3, 4])
def test_packed_linear_formats_agree_with_fake_quant(cuda, oracle, bits):
    """All runtime formats of ARCQPackedLinear against the fake-quant module they replace.  The
    reference's own acceptance numbers for this comparison are max-abs 1e-4 / mean-abs 1e-5 in fp32
    (scripts/debug_arcq_packed_correctness.py:221); the index-space formats meet them, the fp16
    formats are held to fp16 tolerance."""
    src = _source(384, 256, bits)
    x = synth.make_activation(197, 384, 12).reshape(1, 197, 384)
    want = src(x)
    outs = {}
    for fmt in ("packed", "u8", "dequant_gemm", "hip_fused"):
        layer = A.ARCQPackedLinear(src, fmt).to(cuda)
        y = layer(x.to(cuda))
        assert y.dtype == torch.float32 and tuple(y.shape) == (1, 197, 256)
        outs[fmt] = y.cpu()
    # Codes can differ from torch's at near-ties (different reduction order), which moves an output
    # by one codebook step times a weight; compare robustly, then exactly against the oracle chain.
    for fmt in ("packed", "u8"):
        diff = (outs[fmt] - want).abs()
        assert diff.mean() < 1e-5 and diff.median() < 2e-6
        assert (diff > 1e-4).float().mean() < 1e-3
    for fmt in ("dequant_gemm", "hip_fused"):
        diff = (outs[fmt] - want).abs()
        assert diff.max() < 1e-2 * want.abs().max() and diff.mean() < 2e-3 * want.abs().mean() + 1e-4
        assert torch.nn.functional.cosine_similarity(outs[fmt].flatten(), want.flatten(), dim=0) > 0.99999
    # "packed" and "u8" compute the same sum in fp64 / fp32
    assert (outs["packed"] - outs["u8"]).abs().max() < 1e-4
    # module forward == raw ops chain == oracle (bit-exact for the fp64 format)
    layer = A.ARCQPackedLinear(src, "packed")
    xa = oracle.act_quant_c(x.reshape(197, 384).numpy(), layer.activation_thresholds, layer.activation_codebook, bits, 64)
    ref = oracle.linear_forward_packed_c(xa["packed"], xa["center"], xa["scale"], xa["code_sum"],
                                         layer.packed_weight_codes.numpy(), layer.weight_center, layer.weight_scale,
                                         layer.weight_code_sum, layer.product_table.numpy(), layer.bias.numpy(), bits,
                                         64, 384, 256)
    assert np.array_equal(outs["packed"].reshape(197, 256).numpy(), ref)


def test_on_the_fly_and_fast_modules(cuda, oracle):
    src = _source(384, 1152, 4, seed=3)
    packed = A.ARCQPackedLinear(src, "packed")
    otf = A.ARCQPackedLinearOnTheFly.from_packed(packed).to(cuda)
    x = synth.make_activation(2 * 197, 384, 5).reshape(2, 197, 384).to(torch.float16)
    xd = x.to(cuda)
    y = otf(xd)
    assert y.dtype == torch.float16 and tuple(y.shape) == (2, 197, 1152)
    assert torch.equal(xd.cpu(), x)                                     # input not overwritten
    want = src(x.float())
    assert torch.nn.functional.cosine_similarity(y.float().cpu().flatten(), want.flatten(), dim=0) > 0.99999
    assert (y.float().cpu() - want).abs().max() < 2e-2 * want.abs().max()
    # fp32 input goes through the same kernels (widening is exact)
    y32 = otf(xd.float())
    assert torch.equal(y32, y)
    # .half() on the module keeps metadata fp32 and the result unchanged
    assert torch.equal(otf.half()(xd), y)
    # exact chain: oracle stage 1 + oracle stage 2 in fp16, fp64 product
    a = oracle.act_quant_c(x.reshape(-1, 384).float().numpy(), packed.activation_thresholds,
                           packed.activation_codebook, 4, 64)["x_hat"].astype(np.float16)
    w = oracle.weight_dequant_c(packed.packed_weight_codes.numpy(), packed.weight_codebook, packed.weight_center,
                                packed.weight_scale, packed.weight_code_sum, 4, 64).astype(np.float16)
    y64, mag = oracle.linear_f64_c(a, w, packed.bias.numpy())
    tol = (384 + 2) * 2.0 ** -24 * mag + np.abs(y64) * 2.0 ** -11 + 2.0 ** -25
    assert np.all(np.abs(_np(y).reshape(-1, 1152).astype(np.float64) - y64) <= tol)
    # the "fast" variant multiplies the UNQUANTIZED activation with the rebuilt weight, in fp32
    fast = A.ARCQPackedLinearFast(src, "packed").to(cuda)
    yf = fast(xd.float()).cpu()
    ref_fast = torch.nn.functional.linear(x.float().reshape(-1, 384), torch.from_numpy(w).float(), packed.bias)
    assert torch.allclose(yf.reshape(-1, 1152), ref_fast, rtol=1e-4, atol=1e-4)


def _oracle_layer(oracle, layer, x2):
    """fp64 value of one on-the-fly layer on input rows x2 (fp16 or fp32), and its error scale."""
    a = oracle.act_quant_c(x2.float().numpy(), layer.activation_thresholds.cpu(), layer.activation_codebook.cpu(),
                           layer.bits, 64)["x_hat"].astype(np.float16)
    w = oracle.weight_dequant_c(layer.packed_weight_codes.cpu().numpy(), layer.weight_codebook.cpu(),
                                layer.weight_center.cpu(), layer.weight_scale.cpu(), layer.weight_code_sum.cpu(),
                                layer.bits, 64).astype(np.float16)
    b = layer.bias_tensor.cpu().numpy() if layer.bias_tensor.numel() else None
    return oracle.linear_f64_c(a, w, b)


def test_vit_layerwise_parity(cuda, oracle):
    """Every packed linear of a full-depth model, checked where it sits: forward hooks capture each
    layer's actual input and output during one model forward (the method of
    scripts/debug_arcq_packed_correctness.py:198-225) and the output is compared with the oracle
    evaluated on that same input.  Deep random-init quantized nets amplify any perturbation (a code
    flip moves an activation by a whole codebook step), so end-to-end logits are only sanity-checked
    here; the per-layer check is the parity statement."""
    vit = build_packed_vit("deit_tiny", 4, num_classes=100, device="cuda", half_chain=True)
    captured = []
    hooks = [m.register_forward_hook(lambda mod, inp, out, name=n: captured.append((name, mod, inp[0], out)))
             for n, m in vit.named_modules() if isinstance(m, A.ARCQPackedLinearOnTheFly)]
    with torch.no_grad():
        logits = vit(synth.make_images(2, 1).to(cuda).half())
    for h in hooks:
        h.remove()
    assert len(captured) == 48 and bool(torch.isfinite(logits).all())
    worst = 0.0
    for name, mod, x, y in captured:
        k = mod.in_features
        y64, mag = _oracle_layer(oracle, mod, x.reshape(-1, k).cpu())
        tol = (k + 2) * 2.0 ** -24 * mag + np.abs(y64) * 2.0 ** -11 + 2.0 ** -25
        err = np.abs(_np(y).reshape(-1, mod.out_features).astype(np.float64) - y64)
        assert np.all(err <= tol), name
        worst = max(worst, float((err / tol).max()))
    print(f"48 layers within bound, worst err/tol = {worst:.3f}")


def test_vit_top1_agreement_and_checkpoint(cuda, tmp_path):
    """Packed model vs the fake-quant model it was converted from, on synthetic images (logits error
    and top-1 agreement, the metrics of scripts/debug_arcq_packed_correctness.py:227-242), on a
    2-block model so that quantization chaos does not swamp the comparison; then identical logits
    from a model rebuilt from the saved packed state_dict."""
    import copy
    from arcq_vit_amd.vit import VisionTransformer
    cbk = synth.quantile_codebook(4)

    def make(i, o, b):
        layer = A.QuantLinearPCARCQ(i, o, b, 4, 4, 64)
        layer.act_quant.set_codebook(cbk)
        layer.weight_quant.set_codebook(cbk)
        return layer

    torch.manual_seed(0)
    fq = VisionTransformer(192, 2, 3, 768, num_classes=100, linear=make).eval()
    g = torch.Generator().manual_seed(5)
    with torch.no_grad():
        for name, p in fq.named_parameters():
            if p.dim() >= 2:
                p.copy_(torch.randn(p.shape, generator=g) * (0.2 if name.startswith("head") else 0.05))
    imgs = synth.make_images(16, 1)
    with torch.no_grad():
        want = fq(imgs)
    packed = copy.deepcopy(fq)
    A.convert_arcq_linear_to_packed(packed, "packed")
    assert A.count_packed_linear(packed) == 8
    A.to_on_the_fly(packed)
    sd = {k: v.clone() for k, v in packed.state_dict().items()}
    packed = packed.to(cuda)
    with torch.no_grad():
        got32 = packed(imgs.to(cuda)).float().cpu()                      # fp32 trunk, fp16 packed linears
        got16 = packed.half()(imgs.to(cuda).half()).float().cpu()        # half chain
    # Yardstick: the fake-quant model is itself chaotic under rounding-sized noise (a code flip moves
    # an activation by a whole codebook step), so measure how far ITS logits move when every linear's
    # input gets fp16-rounding-sized relative noise, and hold the packed model to that scale.
    noisy = copy.deepcopy(fq)
    gen = torch.Generator().manual_seed(9)
    for mod in noisy.modules():
        if isinstance(mod, A.QuantLinearPCARCQ):
            mod.register_forward_pre_hook(
                lambda m_, inp: (inp[0] * (1 + 2.0 ** -11 * torch.randn(inp[0].shape, generator=gen)),))
    with torch.no_grad():
        ref_noise = (noisy(imgs) - want).pow(2).mean().sqrt()
    for got, factor in ((got32, 3.0), (got16, 4.0)):
        rms = (got - want).pow(2).mean().sqrt()
        assert rms < factor * ref_noise, (float(rms), float(ref_noise))
        assert torch.nn.functional.cosine_similarity(got.flatten(), want.flatten(), dim=0) > 0.98
    # top-1 must agree wherever the reference margin exceeds twice the observed logit error
    top2 = want.topk(2, dim=1).values
    decided = (top2[:, 0] - top2[:, 1]) > 2 * (got32 - want).abs().max()
    assert bool((got32.argmax(1) == want.argmax(1))[decided].all())
    print(f"top-1 agreement {(got32.argmax(1) == want.argmax(1)).float().mean():.3f} "
          f"(fp16 chain {(got16.argmax(1) == want.argmax(1)).float().mean():.3f}); logit rms err "
          f"{(got32 - want).pow(2).mean().sqrt():.4f} vs {ref_noise:.4f} for the fake-quant model under 2^-11 noise")
    torch.save(sd, tmp_path / "packed.pt")
    fresh = VisionTransformer(192, 2, 3, 768, num_classes=100)
    A.load_packed_state_dict(fresh, torch.load(tmp_path / "packed.pt", weights_only=True))
    with torch.no_grad():
        again = fresh.to(cuda)(imgs.to(cuda)).float().cpu()
    assert torch.equal(again, got32)


def test_hip_graph_replay(cuda):
    """The whole packed layer is capturable (no allocation or host read inside the C calls); replays
    interleaved with eager work reproduce the eager result every time."""
    vit = build_packed_vit("deit_tiny", 4, num_classes=10, device="cuda", half_chain=True)
    x = synth.make_images(1, 3).to(cuda).half()
    with torch.no_grad():
        eager = vit(x).clone()
        s = torch.cuda.Stream()
        s.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(s):
            for _ in range(2):
                vit(x)
        torch.cuda.current_stream().wait_stream(s)
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            out = vit(x)
        for i in range(4):
            g.replay()
            torch.cuda.synchronize()
            assert torch.equal(out, eager), f"replay {i}"
            other = vit(x * (1.0 + 0.1 * (i + 1)))                       # eager work between replays
            torch.cuda.synchronize()
            assert not torch.equal(other, eager)


# ------------------------------------------------------------------------------------------------
# full-size, size-independent properties (benchmark shapes: M = 12608)
# ------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("bits", [3, 4])
def test_fullsize_properties(cuda, oracle, bits):
    m, k, n = 12608, 384, 1152
    cb = synth.quantile_codebook(bits).to(cuda)
    thr = synth.midpoint_thresholds(cb.cpu()).to(cuda)
    x = synth.make_activation(m, k, 77).to(cuda)
    # (1) pack(unpack) round trip and byte codes == unpack(packed codes)
    packed, center, scale, code_sum = ops.quantize_activation(x, thr, cb, bits, 64)
    codes, c2, s2, cs2 = ops.quantize_activation_u8(x, thr, cb, bits, 64)
    assert torch.equal(ops.unpack_codes_u8(packed, bits, k), codes)
    assert torch.equal(ops.pack_codes(codes.long(), bits), packed)
    assert torch.equal(center, c2) and torch.equal(scale, s2) and torch.equal(code_sum, cs2)
    # (2) group invariants: code_sum is the serial sum of looked-up values; mean of x_hat is mu
    vals = cb[codes.long()].reshape(m, k // 64, 64)
    assert torch.allclose(vals.sum(-1), code_sum, atol=1e-4)
    x_hat = ops.quantize_activation_dequant(x, thr, cb, bits, 64)
    assert torch.allclose(x_hat.reshape(m, -1, 64).mean(-1), center, atol=2e-5)
    # (3) idempotent on already-constant groups, and row independence: a permutation of the tokens
    # permutes every output exactly
    perm = torch.randperm(m, device=cuda)
    p2, c3, _, _ = ops.quantize_activation(x[perm].contiguous(), thr, cb, bits, 64)
    assert torch.equal(p2, packed[perm]) and torch.equal(c3, center[perm])
    # (4) a random sample of rows against the oracle, bit for bit
    rows = torch.randint(0, m, (64,))
    ref = oracle.act_quant_c(_np(x[rows.to(cuda)]), thr.cpu(), cb.cpu(), bits, 64)
    assert np.array_equal(_np(packed[rows.to(cuda)]), ref["packed"])
    assert np.array_equal(_np(x_hat[rows.to(cuda)]), ref["x_hat"])
    # (5) fused GEMM: token permutation and M-split give identical rows (tiles do not interact);
    #     adding a bias shifts the fp32 result by exactly that bias up to one rounding
    w = synth.make_weight(n, k, 78)
    wcodes, wc, ws, wcs = oracle.quantize_weight_torch(w, thr.cpu(), cb.cpu(), 64, 1e-6)
    pw = A.pack_codes_py(wcodes, bits).to(cuda)
    wc, ws, wcs = wc.to(cuda), ws.to(cuda), wcs.to(cuda)
    xh = x_hat.half()
    y = ops.linear_fused(xh, pw, cb, wc, ws, wcs, None, bits, 64, out_dtype=torch.float32)
    yp = ops.linear_fused(xh[perm].contiguous(), pw, cb, wc, ws, wcs, None, bits, 64, out_dtype=torch.float32)
    assert torch.equal(yp, y[perm])
    y_half = ops.linear_fused(xh[:5000].contiguous(), pw, cb, wc, ws, wcs, None, bits, 64, out_dtype=torch.float32)
    assert torch.equal(y_half, y[:5000])
    bias = synth.make_bias(n, 79).to(cuda)
    yb = ops.linear_fused(xh, pw, cb, wc, ws, wcs, bias, bits, 64, out_dtype=torch.float32)
    assert torch.equal(yb, y + bias)
    # (6) against a library GEMM on the stage-2 output (fp16 operands, fp32 accumulate)
    w16 = ops.unpack_weight_hip(pw, cb, wc, ws, wcs, bits, 64)
    lib = torch.nn.functional.linear(xh.float(), w16.float())
    assert (y - lib).abs().max() < 1e-3 * lib.abs().max()
    # (7) sampled rows against the fp64 oracle with the fp32-accumulation bound
    y64, mag = oracle.linear_f64_c(_np(xh[rows.to(cuda)]), _np(w16), None)
    assert np.all(np.abs(_np(y[rows.to(cuda)]).astype(np.float64) - y64) <= (k + 2) * 2.0 ** -24 * mag)


@pytest.mark.parametrize("m,n,k,bits", [(12608, 384, 384, 4), (12608, 1536, 384, 4), (12608, 384, 1536, 4),
                                        (12608, 1536, 384, 3), (12608, 3072, 768, 4), (12608, 768, 3072, 3),
                                        (50432, 1024, 1024, 3)])
def test_fullsize_gemm_shapes(cuda, oracle, m, n, k, bits):
    """The remaining benchmark layer shapes (DeiT-S proj/fc1/fc2, DeiT-B fc1/fc2, ViT-L proj at batch 256) through
    whichever large-M kernel the dispatcher picks: row permutation and M-split leave rows unchanged (tiles do not
    interact), the result matches a library GEMM on the stage-2 output and, on sampled rows, the fp64 oracle within
    the fp32-accumulation bound."""
    cb = synth.quantile_codebook(bits)
    thr = synth.midpoint_thresholds(cb)
    x = synth.make_activation(m, k, 81, "gelu" if k > n else "ln").to(cuda)
    xh = ops.quantize_activation_dequant(x, thr.to(cuda), cb.to(cuda), bits, 64).half()
    del x
    w = synth.make_weight(n, k, 82)
    wcodes, wc, ws, wcs = oracle.quantize_weight_torch(w, thr, cb, 64, 1e-6)
    pw = A.pack_codes_py(wcodes, bits).to(cuda)
    cb, wc, ws, wcs = cb.to(cuda), wc.to(cuda), ws.to(cuda), wcs.to(cuda)
    bias = synth.make_bias(n, 83).to(cuda)
    y = ops.linear_fused(xh, pw, cb, wc, ws, wcs, bias, bits, 64, out_dtype=torch.float32)
    perm = torch.randperm(m, device=cuda)
    yp = ops.linear_fused(xh[perm].contiguous(), pw, cb, wc, ws, wcs, bias, bits, 64, out_dtype=torch.float32)
    assert torch.equal(yp, y[perm])
    del yp
    cut = 5000
    y_part = ops.linear_fused(xh[:cut].contiguous(), pw, cb, wc, ws, wcs, bias, bits, 64, out_dtype=torch.float32)
    assert torch.equal(y_part, y[:cut])
    y16 = ops.linear_fused(xh, pw, cb, wc, ws, wcs, bias, bits, 64, out_dtype=torch.float16)
    assert torch.equal(y16, y.half())                       # same fp32 value, rounded once
    w16 = ops.unpack_weight_hip(pw, cb, wc, ws, wcs, bits, 64)
    rows = torch.randint(0, m, (48,), device=cuda)
    lib = torch.nn.functional.linear(xh[rows].float(), w16.float(), bias)
    assert (y[rows] - lib).abs().max() < 1e-3 * lib.abs().max()
    y64, mag = oracle.linear_f64_c(_np(xh[rows]), _np(w16), _np(bias))
    assert np.all(np.abs(_np(y[rows]).astype(np.float64) - y64) <= (k + 2) * 2.0 ** -24 * mag)
    # The same product from x_hat in the 32-row block layout (eight waves per workgroup for the DeiT-S shapes, twelve
    # for the larger ones when the weights are ready): bit-identical, rebuilding the weights or copying them.
    del y_part, y16, lib
    xb = xh.reshape(m // 32, 32, k // 8, 8).permute(0, 2, 1, 3).contiguous()
    assert torch.equal(ops.linear_fused_blocked(xb, m, k, pw, cb, wc, ws, wcs, bias, bits, out_dtype=torch.float32), y)
    assert torch.equal(ops.linear_fused_blocked(xb, m, k, pw, cb, wc, ws, wcs, bias, bits, out_dtype=torch.float32,
                                                w_hat_ws=w16.reshape(-1), w_hat_ready=True), y)


def test_on_the_fly_layer_sees_replaced_and_updated_buffers(cuda):
    """The layer caches raw pointers of its buffers; swapping a buffer for another tensor, or writing into one in place,
    must show in the next forward."""
    from arcq_vit_amd.vit import build_packed_vit
    vit = build_packed_vit("deit_tiny", 4, depth=1)
    layer = vit.blocks[0].attn.proj
    x = synth.make_activation(197, layer.in_features, 3).to(cuda).half()
    with torch.no_grad():
        y0 = layer(x).clone()
        layer.bias_tensor = layer.bias_tensor * 64.0                     # replaced (a power of two: undone exactly below)
        y1 = layer(x).clone()
        assert not torch.equal(y1, y0)
        layer.bias_tensor.mul_(1.0 / 64.0)                               # in place
        assert torch.equal(layer(x), y0)
        layer.activation_thresholds = layer.activation_thresholds * 0.5  # another buffer than the packed codes
        assert not torch.equal(layer(x), y0)
