"""GPU tests of the elementwise work fused around the packed layer (arcq_linear_otf_ex / arcq_act_quant_blocked_ln):
LayerNorm inside the stage-1 launch, GELU and the skip connection inside the GEMM's epilogue, and the ViT block that
uses them."""
import numpy as np
import pytest
import torch

import arcq_vit_amd as A
from arcq_vit_amd import ops, synth
from arcq_vit_amd.vit import build_packed_vit

pytestmark = pytest.mark.gpu


def _np(t):
    return t.detach().cpu().numpy()


def _to_blocked(t):
    m, k = t.shape
    full = (m // 32) * 32
    parts = [t[:full].reshape(m // 32, 32, k // 8, 8).permute(0, 2, 1, 3).reshape(-1)]
    if full < m:
        parts.append(t[full:].reshape(m - full, k // 8, 8).permute(1, 0, 2).reshape(-1))
    return torch.cat(parts).contiguous()


def _cb(bits):
    cb = synth.quantile_codebook(bits)
    return cb, synth.midpoint_thresholds(cb)


def _weights(oracle, n, k, bits, seed):
    cb, thr = _cb(bits)
    codes, wc, ws, wcs = oracle.quantize_weight_torch(synth.make_weight(n, k, seed), thr, cb, 64, 1e-6)
    return A.pack_codes_py(codes, bits), cb, wc, ws, wcs


def _ln_params(k, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(k, generator=g) * 0.3 + 1.0, torch.randn(k, generator=g) * 0.2


@pytest.mark.parametrize("bits", [3, 4])
@pytest.mark.parametrize("m,k,in_dtype", [(512, 384, torch.float16), (1000, 192, torch.float16),     # ragged last block
                                          (70, 64, torch.float16), (640, 768, torch.float32),
                                          (600, 1024, torch.float16),       # sixteen waves per workgroup
                                          (12608, 384, torch.float16)])     # DeiT-S at batch 64
def test_layernorm_stage1_bitexact(cuda, oracle, bits, m, k, in_dtype):
    """arcq_act_quant_blocked_ln == oracle LayerNorm (in the documented summation order) -> oracle stage 1, bit for bit,
    in the block layout; with the weight reconstruction carried in the same launch as well."""
    cb, thr = _cb(bits)
    lw, lb = _ln_params(k, 5)
    x = (synth.make_activation(m, k, 21) * 1.7 + 0.3).to(in_dtype)
    xln = oracle.layernorm_rows_np(x.float().numpy(), lw.numpy(), lb.numpy(), 1e-6, out_f16=in_dtype == torch.float16)
    want = oracle.act_quant_c(xln, thr, cb, bits, 64)["x_hat"].astype(np.float16)
    d = lambda t: t.to(cuda)
    got = ops.quantize_activation_blocked_ln(d(x), d(lw), d(lb), 1e-6, d(thr), d(cb), bits)
    assert np.array_equal(_np(got.reshape(-1)).view(np.uint16), _np(_to_blocked(torch.from_numpy(want))).view(np.uint16))
    n = 200
    pw, _, wc, ws, wcs = _weights(oracle, n, k, bits, 22)
    w_hat = torch.full((n * k + 8,), -3.0, dtype=torch.float16, device=cuda)
    got2 = ops.quantize_activation_blocked_ln(d(x), d(lw), d(lb), 1e-6, d(thr), d(cb), bits,
                                              weights=[d(t) for t in (pw, cb, wc, ws, wcs)], w_hat=w_hat)
    assert torch.equal(got2, got)
    want_w = oracle.weight_dequant_c(pw.numpy(), cb, wc, ws, wcs, bits, 64, fma=True).astype(np.float16)
    assert np.array_equal(_np(w_hat)[:n * k].view(np.uint16), want_w.reshape(-1).view(np.uint16))
    assert bool((w_hat[n * k:] == -3.0).all())


@pytest.mark.parametrize("m,n,k,bits,ln,gelu,res", [
    (12608, 1152, 384, 4, True, False, False),      # qkv of DeiT-S: LayerNorm in front
    (12608, 384, 384, 4, False, False, True),       # proj: skip connection behind
    (12608, 1536, 384, 4, True, True, False),       # fc1: LayerNorm in front, GELU behind
    (12608, 384, 1536, 4, False, False, True),      # fc2: skip connection (eight-wave kernel, weights copied)
    (12608, 768, 3072, 3, False, False, True),      # DeiT-B fc2 at W3: the two-blocks-per-wave kernel
    (12608, 3072, 768, 4, True, True, False),       # DeiT-B fc1
    (1000, 200, 448, 4, True, True, True),          # ragged rows and columns, everything at once
    (600, 100, 1024, 3, True, False, True),
    # fewer than 512 rows (batch 1): one launch with everything inside, or stage 1 + split-K with the post-operations
    (197, 1152, 384, 4, True, False, False),        # qkv of DeiT-S at batch 1
    (197, 384, 384, 4, False, False, True),         # proj
    (197, 1536, 384, 4, True, True, False),         # fc1
    (197, 384, 1536, 4, False, False, True),        # fc2: two launches, residual in the split-K epilogue
    (197, 2304, 768, 3, True, False, False),        # DeiT-B qkv: one lane per group
    (197, 3072, 768, 4, True, True, False),         # DeiT-B fc1: the one-launch kernel because of the LayerNorm
    (394, 768, 192, 4, True, True, True),           # DeiT-tiny, batch 2
    (100, 200, 1024, 4, True, True, True),          # ragged rows and columns
    (37, 96, 1536, 3, True, False, True),           # LayerNorm over a long row: two rounds of stage-1 tiles
    (197, 100, 1536, 2, False, True, True),         # split-K epilogue, ragged columns
    (1, 64, 64, 4, True, True, True)])
def test_linear_otf_ex_equals_the_unfused_sequence(cuda, oracle, m, n, k, bits, ln, gelu, res):
    """arcq_linear_otf_ex == LayerNorm (oracle, rounded to fp16) -> arcq_linear_otf_ws -> torch GELU -> torch add, every
    step in fp16 as the unfused model runs them: bit for bit; sampled rows of the linear part against the fp64 oracle."""
    pw, cb, wc, ws, wcs = _weights(oracle, n, k, bits, 31)
    _, thr = _cb(bits)
    bias = synth.make_bias(n, 31)
    lw, lb = _ln_params(k, 6)
    x = (synth.make_activation(m, k, 32, "ln") * 1.3 - 0.2).to(torch.float16)
    r = (synth.make_activation(m, n, 33, "ln") * 0.7).to(torch.float16)
    d = lambda t: t.to(cuda)
    args = (d(thr), d(cb), d(pw), d(cb), d(wc), d(ws), d(wcs), d(bias), bits, 64)
    w_ws = torch.empty(n * k, dtype=torch.float16, device=cuda)
    y = ops.linear_otf_ex(d(x), *args, layernorm=(d(lw), d(lb), 1e-6) if ln else None, gelu=gelu,
                          residual=d(r) if res else None, w_hat_ws=w_ws)
    x_in = x
    if ln:
        x_in = torch.from_numpy(oracle.layernorm_rows_np(x.float().numpy(), lw.numpy(), lb.numpy(), 1e-6, True)).half()
    lin = ops.linear_otf(d(x_in), *args, w_hat_ws=w_ws)
    want = lin
    if gelu:
        want = torch.nn.functional.gelu(want)
    if res:
        want = want + d(r)
    assert y.dtype == torch.float16 and torch.equal(y, want)
    assert torch.equal(ops.linear_otf_ex(d(x), *args, layernorm=(d(lw), d(lb), 1e-6) if ln else None, gelu=gelu,
                                         residual=d(r) if res else None), y)          # without the weight workspace
    rows = torch.randint(0, m, (24,), generator=torch.Generator().manual_seed(4))
    rows[0], rows[1] = 0, m - 1
    a = oracle.act_quant_c(x_in[rows].float().numpy(), thr, cb, bits, 64)["x_hat"].astype(np.float16)
    w16 = oracle.weight_dequant_c(pw.numpy(), cb, wc, ws, wcs, bits, 64, fma=True).astype(np.float16)
    y64, mag = oracle.linear_f64_c(a, w16, bias.numpy())
    tol = (k + 2) * 2.0 ** -24 * mag + np.abs(y64) * 2.0 ** -11 + 2.0 ** -25
    assert np.all(np.abs(_np(lin[rows.to(cuda)]).astype(np.float64) - y64) <= tol)
    if gelu and not res:        # the epilogue's GELU against the float64 erf: within one fp16 step
        g64 = oracle.gelu_f64_np(_np(lin[rows.to(cuda)]).astype(np.float64))
        got = _np(y[rows.to(cuda)]).astype(np.float64)
        step = np.spacing(np.abs(g64).astype(np.float16)).astype(np.float64)
        assert np.all(np.abs(got - g64) <= step)


@pytest.mark.parametrize("m,k,h,bits", [(197, 384, 1536, 4), (100, 384, 1536, 3), (197, 192, 768, 4), (33, 768, 3072, 4),
                                        (1, 64, 64, 2),
                                        # from 512 rows on: the block-layout GEMM kernels, x_hat handed over in the block layout
                                        (1000, 384, 1536, 4),        # eight-wave kernel, ragged last block
                                        (3000, 192, 768, 3), (520, 64, 128, 2),
                                        (12608, 768, 3072, 4),       # DeiT-B: two row blocks per wave
                                        (8200, 1024, 4096, 3)])      # ViT-L widths
def test_two_layers_chained_through_x_hat(cuda, oracle, m, k, h, bits):
    """fc1 -> GELU -> fc2 with fc2's stage 1 inside fc1's launch (next_quant / x_is_xhat): the x_hat handed over equals
    the oracle's stage 1 of the stored GELU output bit for bit, and fc2's result equals the unfused sequence's."""
    pw1, cb, wc1, ws1, wcs1 = _weights(oracle, h, k, bits, 51)
    pw2, _, wc2, ws2, wcs2 = _weights(oracle, k, h, bits, 52)
    _, thr = _cb(bits)
    cb2 = cb * 1.1                                   # the consumer's own quantizer, different from the producer's
    thr2 = synth.midpoint_thresholds(cb2)
    b1, b2 = synth.make_bias(h, 51), synth.make_bias(k, 52)
    lw, lb = _ln_params(k, 9)
    x = (synth.make_activation(m, k, 53, "ln") * 1.2).to(torch.float16)
    d = lambda t: t.to(cuda)
    a1 = (d(thr), d(cb), d(pw1), d(cb), d(wc1), d(ws1), d(wcs1), d(b1), bits, 64)
    a2 = (d(thr2), d(cb2), d(pw2), d(cb), d(wc2), d(ws2), d(wcs2), d(b2), bits, 64)
    ln = (d(lw), d(lb), 1e-6)
    blocked = ops.xhat_layout(m) == 1
    assert blocked == (m >= 512)
    w1 = torch.empty(h * k, dtype=torch.float16, device=cuda)        # weight workspaces (the block-layout path needs one)
    xhat = ops.linear_otf_ex(d(x), *a1, layernorm=ln, gelu=True, next_quant=(d(thr2), d(cb2)), w_hat_ws=w1)
    y = ops.linear_otf_ex(xhat, *a2, residual=d(x), x_is_xhat=True, w_hat_ws=w1)
    g = ops.linear_otf_ex(d(x), *a1, layernorm=ln, gelu=True, w_hat_ws=w1)       # the stored GELU output
    want_xhat = torch.from_numpy(oracle.act_quant_c(_np(g).astype(np.float32), thr2, cb2, bits, 64)["x_hat"].astype(np.float16))
    if blocked:
        want_xhat = _to_blocked(want_xhat)
    assert xhat.dtype == torch.float16
    assert np.array_equal(_np(xhat).reshape(-1).view(np.uint16), want_xhat.numpy().reshape(-1).view(np.uint16))
    assert torch.equal(y, ops.linear_otf_ex(g, *a2, residual=d(x), w_hat_ws=w1))
    assert torch.equal(y, ops.linear_otf_ex(xhat, *a2, residual=d(x), x_is_xhat=True))     # consumer without a workspace


def test_linear_otf_ex_fp32_and_limits(cuda, oracle):
    n, k, bits = 256, 384, 4
    pw, cb, wc, ws, wcs = _weights(oracle, n, k, bits, 41)
    _, thr = _cb(bits)
    bias = synth.make_bias(n, 41)
    d = lambda t: t.to(cuda)
    args = (d(thr), d(cb), d(pw), d(cb), d(wc), d(ws), d(wcs), d(bias), bits, 64)
    x = synth.make_activation(640, k, 42).to(cuda)                       # fp32 in, fp32 out
    r = synth.make_activation(640, n, 43).to(cuda)
    y = ops.linear_otf_ex(x, *args, out_dtype=torch.float32, gelu=True, residual=r)
    lin = ops.linear_otf(x, *args, out_dtype=torch.float32)
    assert torch.equal(y, torch.nn.functional.gelu(lin) + r)
    assert torch.equal(ops.linear_otf_ex(x, *args, out_dtype=torch.float32), lin)      # no option: the plain layer
    small = x[:197].contiguous()
    lin_small = ops.linear_otf(small, *args, out_dtype=torch.float32)
    assert torch.equal(ops.linear_otf_ex(small, *args, out_dtype=torch.float32), lin_small)
    assert torch.equal(ops.linear_otf_ex(small, *args, out_dtype=torch.float32, gelu=True, residual=r[:197].contiguous()),
                       torch.nn.functional.gelu(lin_small) + r[:197])
    # fp32 input with a LayerNorm in front, below 512 rows: the LayerNorm's result is not rounded to fp16
    lw, lb = _ln_params(k, 8)
    xln = torch.from_numpy(oracle.layernorm_rows_np(small.cpu().numpy(), lw.numpy(), lb.numpy(), 1e-6, out_f16=False))
    assert torch.equal(ops.linear_otf_ex(small, *args, out_dtype=torch.float32, layernorm=(d(lw), d(lb), 1e-6)),
                       ops.linear_otf(d(xln), *args, out_dtype=torch.float32))
    with pytest.raises(RuntimeError, match="residual"):
        ops.linear_otf_ex(x, *args, out_dtype=torch.float32, residual=r.half())
    wide = synth.make_activation(8, 2048, 44).to(cuda)
    pw2, _, wc2, ws2, wcs2 = _weights(oracle, 64, 2048, bits, 45)
    with pytest.raises(RuntimeError, match="in_features <= 1536"):
        ops.linear_otf_ex(wide, d(thr), d(cb), d(pw2), d(cb), d(wc2), d(ws2), d(wcs2), None, bits, 64,
                          layernorm=(torch.ones(2048, device=cuda), torch.zeros(2048, device=cuda), 1e-6))


@pytest.mark.parametrize("model,batch", [("deit_small", 64), ("deit_tiny", 2)])
def test_vit_block_fusion(cuda, oracle, model, batch):
    """The ViT skeleton with LayerNorm / GELU / skip connections inside the packed layers' launches: every packed layer's
    output, captured by forward hooks, equals the oracle's value of the same fused layer on the captured input
    (LayerNorm restatement -> stage 1 -> fp64 product -> GELU / residual in fp16), and the logits stay close to the
    unfused model's (whose LayerNorm is torch's kernel: another summation order, so codes may differ at ties).  Batch 2
    (394 rows) takes the small-M kernels: one launch per layer with everything inside; the layers are hooked with fc1 and
    fc2 called separately, and the model with fc2's stage 1 inside fc1's launch must then give the same logits bit for bit."""
    kw = dict(num_classes=100, device="cuda", half_chain=True, depth=2, shared_buffers=True, max_rows=batch * synth.TOKENS)
    fused = build_packed_vit(model, 4, fuse_elementwise=True, **kw)
    plain = build_packed_vit(model, 4, fuse_elementwise=False, **kw)
    x = synth.make_images(batch, 1).to(cuda).half()
    captured = []

    def hook(mod, args, kwargs, out):
        rows = torch.arange(0, args[0].numel() // mod.in_features, max(1, args[0].numel() // mod.in_features // 24))
        x2 = args[0].reshape(-1, mod.in_features)[rows.to(cuda)].cpu()
        res = kwargs.get("residual")
        r2 = None if res is None else res.reshape(-1, mod.out_features)[rows.to(cuda)].cpu()
        captured.append((mod, kwargs.get("layernorm"), kwargs.get("activation"), x2, r2,
                         out.reshape(-1, mod.out_features)[rows.to(cuda)].cpu()))

    hooks = [m.register_forward_hook(hook, with_kwargs=True) for m in fused.modules()
             if isinstance(m, A.ARCQPackedLinearOnTheFly)]
    for blk in fused.blocks:
        blk.chain_mlp = False
    with torch.no_grad():
        lf, lp = fused(x), plain(x)
    for h in hooks:
        h.remove()
    for blk in fused.blocks:
        blk.chain_mlp = True
    with torch.no_grad():
        assert torch.equal(fused(x), lf)
    assert bool(torch.isfinite(lf).all())
    assert len(captured) == 8
    for mod, ln, act, x2, r2, y in captured:
        k = mod.in_features
        xin = x2.float().numpy()
        if ln is not None:
            xin = oracle.layernorm_rows_np(xin, ln.weight.detach().float().cpu().numpy(), ln.bias.detach().float().cpu().numpy(), ln.eps, True)
        a = oracle.act_quant_c(xin, mod.activation_thresholds.cpu(), mod.activation_codebook.cpu(), mod.bits, 64)["x_hat"]
        w = oracle.weight_dequant_c(mod.packed_weight_codes.cpu().numpy(), mod.weight_codebook.cpu(), mod.weight_center.cpu(),
                                    mod.weight_scale.cpu(), mod.weight_code_sum.cpu(), mod.bits, 64, fma=True)
        y64, mag = oracle.linear_f64_c(a.astype(np.float16), w.astype(np.float16), mod.bias_tensor.cpu().numpy())
        tol = (k + 2) * 2.0 ** -24 * mag + np.abs(y64) * 2.0 ** -11 + 2.0 ** -25
        want, slack = y64, tol
        if act == "gelu":       # GELU is 1-Lipschitz-ish (|gelu'| <= 1.13): carry the bound through, plus its own rounding
            want = oracle.gelu_f64_np(y64)
            slack = 1.13 * tol + np.abs(want) * 2.0 ** -11 + 2.0 ** -24
        if r2 is not None:
            want = want + r2.double().numpy()
            slack = slack + np.abs(want) * 2.0 ** -11 + 2.0 ** -24
        assert np.all(np.abs(y.double().numpy() - want) <= slack), (mod.in_features, mod.out_features, act)
    cos = torch.nn.functional.cosine_similarity(lf.float().flatten(), lp.float().flatten(), dim=0).item()
    assert cos > 0.98, cos
    print(f"{model} batch {batch}: fused vs unfused logits cosine {cos:.5f}, "
          f"top-1 agreement {(lf.argmax(1) == lp.argmax(1)).float().mean():.3f}")
