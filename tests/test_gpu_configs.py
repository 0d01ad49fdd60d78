"""GPU tests at the sizes of the named benchmark configurations: model forwards of DeiT-Base (W4A4, batch 64)
and ViT-Large (W3A3, batch 256) with every packed linear checked where it sits, the remaining DeiT-B / ViT-L layer
shapes through the fused GEMM, and the whole-layer call the benchmark times at its own size (M = 12 608)."""
import numpy as np
import pytest
import torch

import arcq_vit_amd as A
from arcq_vit_amd import _lib, ops, synth
from arcq_vit_amd.vit import build_packed_vit

pytestmark = pytest.mark.gpu


def _np(t):
    return t.detach().cpu().numpy()


def _to_blocked(t):
    """Row-major [M, K] -> the 32-row block layout, flat (whole blocks [M/32, K/8, 32, 8], then a ragged block)."""
    m, k = t.shape
    full = (m // 32) * 32
    parts = [t[:full].reshape(m // 32, 32, k // 8, 8).permute(0, 2, 1, 3).reshape(-1)]
    if full < m:
        parts.append(t[full:].reshape(m - full, k // 8, 8).permute(1, 0, 2).reshape(-1))
    return torch.cat(parts).contiguous()


def _oracle_rows(oracle, layer, x_rows):
    """fp64 value of one on-the-fly layer on the given input rows (fp16), and the error scale sum |a*w|."""
    a = oracle.act_quant_c(x_rows.float().numpy(), layer.activation_thresholds.cpu(), layer.activation_codebook.cpu(),
                           layer.bits, 64)["x_hat"].astype(np.float16)
    w = oracle.weight_dequant_c(layer.packed_weight_codes.cpu().numpy(), layer.weight_codebook.cpu(),
                                layer.weight_center.cpu(), layer.weight_scale.cpu(), layer.weight_code_sum.cpu(),
                                layer.bits, 64, fma=True).astype(np.float16)
    b = layer.bias_tensor.cpu().numpy() if layer.bias_tensor.numel() else None
    return oracle.linear_f64_c(a, w, b)


@pytest.mark.parametrize("model,bits,batch,depth", [("deit_base", 4, 64, 2), ("vit_large", 3, 256, 2),
                                                    ("deit_small", 4, 64, 2)])
def test_model_forward_layerwise_fullbatch(cuda, oracle, model, bits, batch, depth):
    """Model forward at the configuration's batch (M = 12 608 / 50 432 tokens) on `depth` blocks of the model's
    widths, through the module path with the shared weight scratch buffer the reference's benchmark sets up.
    Forward hooks take 48 sampled rows of every packed linear's input and output (the method of
    scripts/debug_arcq_packed_correctness.py:198-225); the output rows must equal the oracle's on those input rows
    within the fp32-accumulation bound plus one fp16 rounding.  Two blocks stand for the models' 12 / 24: every block
    has the same four layer shapes, so depth changes how often the kernels run, not which ones (the full-depth
    forwards that bench.py times check nothing and are not a substitute for this test)."""
    vit = build_packed_vit(model, bits, num_classes=100, device="cuda", half_chain=True, depth=depth,
                           shared_buffers=True, max_rows=batch * synth.TOKENS)
    gen = torch.Generator().manual_seed(7)
    captured = []

    def hook(mod, inp, out, name):
        x2 = inp[0].reshape(-1, mod.in_features)
        rows = torch.randint(0, x2.shape[0], (48,), generator=gen)
        rows[0], rows[1] = 0, x2.shape[0] - 1
        captured.append((name, mod, x2[rows.to(x2.device)].cpu(), out.reshape(-1, mod.out_features)[rows.to(x2.device)].cpu()))

    hooks = [m.register_forward_hook(lambda mod, inp, out, name=n: hook(mod, inp, out, name))
             for n, m in vit.named_modules() if isinstance(m, A.ARCQPackedLinearOnTheFly)]
    with torch.no_grad():
        logits = vit(synth.make_images(batch, 1).to(cuda).half())
    torch.cuda.synchronize()
    for h in hooks:
        h.remove()
    assert len(captured) == 4 * depth and tuple(logits.shape) == (batch, 100) and bool(torch.isfinite(logits).all())
    worst = 0.0
    for name, mod, x_rows, y_rows in captured:
        k = mod.in_features
        y64, mag = _oracle_rows(oracle, mod, x_rows)
        tol = (k + 2) * 2.0 ** -24 * mag + np.abs(y64) * 2.0 ** -11 + 2.0 ** -25
        err = np.abs(y_rows.numpy().astype(np.float64) - y64)
        assert np.all(err <= tol), (name, float((err / tol).max()))
        worst = max(worst, float((err / tol).max()))
    print(f"{model} W{bits}A{bits} batch {batch}: {len(captured)} layers within bound, worst err/tol = {worst:.3f}")


@pytest.mark.parametrize("name,k,n", synth.block_linear_shapes("deit_small"))
@pytest.mark.parametrize("bits", [4, 3])
def test_benchmarked_layer_call_fullsize(cuda, oracle, name, k, n, bits):
    """ops.linear_otf(..., w_hat_ws=ws) -- arcq_linear_otf_ws, the call bench.py times -- at M = 12 608 for the four
    DeiT-S shapes: where the layer runs as two launches the activation workspace holds the oracle's x_hat bit for bit
    (in the library's 32-row block layout), the weight workspace the oracle's w_hat (row-major, or in 32-column
    blocks after the one-launch kernel), and sampled rows of y match the fp64 oracle within the fp32-accumulation
    bound plus one fp16 rounding."""
    m = 64 * synth.TOKENS
    cb = synth.quantile_codebook(bits)
    thr = synth.midpoint_thresholds(cb)
    x = synth.make_activation(m, k, 91, "gelu" if name == "fc2" else "ln").to(torch.float16)
    w = synth.make_weight(n, k, 92)
    wcodes, wc, ws, wcs = oracle.quantize_weight_torch(w, thr, cb, 64, 1e-6)
    pw = A.pack_codes_py(wcodes, bits)
    bias = synth.make_bias(n, 93)
    d = lambda t: t.to(cuda)
    x_ws = torch.zeros(m * k, dtype=torch.float16, device=cuda)
    w_ws = torch.zeros(n * k, dtype=torch.float16, device=cuda)
    y = ops.linear_otf(d(x), d(thr), d(cb), d(pw), d(cb), d(wc), d(ws), d(wcs), d(bias), bits, 64,
                       out_dtype=torch.float16, x_hat_ws=x_ws, w_hat_ws=w_ws)
    torch.cuda.synchronize()
    path = _lib.load().arcq_linear_otf_ws_kernel(m, n, k, 1).decode()
    a = oracle.act_quant_c(x.float().numpy(), thr, cb, bits, 64)["x_hat"].astype(np.float16)
    w16 = oracle.weight_dequant_c(pw.numpy(), cb, wc, ws, wcs, bits, 64, fma=True).astype(np.float16)
    if "slab8" in path or "pair" in path:       # stage 1 wrote the block layout
        assert np.array_equal(_np(x_ws).view(np.uint16), _np(_to_blocked(torch.from_numpy(a))).view(np.uint16)), path
    if path.endswith("<copy>") or "pair" in path:       # the stage-1 launch rebuilt the weights
        assert np.array_equal(_np(w_ws).view(np.uint16), w16.reshape(-1).view(np.uint16)), path
    if path.startswith("otf_rows"):                     # one launch: x_hat stays in LDS, w_hat in 32-column blocks
        blocked = np.ascontiguousarray(w16.reshape(n // 32, 32, k // 8, 8).transpose(0, 2, 1, 3)).reshape(-1)
        assert np.array_equal(_np(w_ws).view(np.uint16), blocked.view(np.uint16)), path
    rows = torch.randint(0, m, (64,), generator=torch.Generator().manual_seed(3))
    rows[0], rows[1] = 0, m - 1
    y64, mag = oracle.linear_f64_c(a[rows.numpy()], w16, bias.numpy())
    tol = (k + 2) * 2.0 ** -24 * mag + np.abs(y64) * 2.0 ** -11 + 2.0 ** -25
    err = np.abs(_np(y[rows.to(cuda)]).astype(np.float64) - y64)
    assert np.all(err <= tol), (path, float((err / tol).max()))
    # and the same call without the weight workspace, and through the row-major entry point: same bits
    y2 = ops.linear_otf(d(x), d(thr), d(cb), d(pw), d(cb), d(wc), d(ws), d(wcs), d(bias), bits, 64,
                        out_dtype=torch.float16, scratch=True)
    y3 = ops.linear_otf(d(x), d(thr), d(cb), d(pw), d(cb), d(wc), d(ws), d(wcs), d(bias), bits, 64,
                        out_dtype=torch.float16)
    assert torch.equal(y2, y) and torch.equal(y3, y)


@pytest.mark.parametrize("m,n,k,bits", [(12608, 2304, 768, 4), (12608, 768, 768, 4), (12608, 768, 3072, 4),
                                        (50432, 3072, 1024, 3), (50432, 4096, 1024, 3), (50432, 1024, 4096, 3)])
def test_large_model_layer_shapes(cuda, oracle, m, n, k, bits):
    """DeiT-B qkv / proj / fc2 at W4 and ViT-L qkv / fc1 / fc2 at W3, whole layer through arcq_linear_otf_ws with
    both scratch buffers (what the module runs): sampled rows against the fp64 oracle, bit-identity with the
    row-major entry point and with the fused GEMM on the separately computed x_hat, and invariance under a
    permutation of the tokens."""
    cb = synth.quantile_codebook(bits)
    thr = synth.midpoint_thresholds(cb)
    x = synth.make_activation(m, k, 95, "gelu" if k > n else "ln").to(torch.float16)
    w = synth.make_weight(n, k, 96)
    wcodes, wc, ws, wcs = oracle.quantize_weight_torch(w, thr, cb, 64, 1e-6)
    pw = A.pack_codes_py(wcodes, bits)
    bias = synth.make_bias(n, 97)
    d = lambda t: t.to(cuda)
    args = (d(thr), d(cb), d(pw), d(cb), d(wc), d(ws), d(wcs), d(bias), bits, 64)
    xd = d(x)
    w_ws = torch.zeros(n * k, dtype=torch.float16, device=cuda)
    y = ops.linear_otf(xd, *args, out_dtype=torch.float16, w_hat_ws=w_ws)
    rows = torch.randint(0, m, (48,), generator=torch.Generator().manual_seed(5))
    rows[0], rows[1] = 0, m - 1
    a = oracle.act_quant_c(x[rows].float().numpy(), thr, cb, bits, 64)["x_hat"].astype(np.float16)
    w16 = oracle.weight_dequant_c(pw.numpy(), cb, wc, ws, wcs, bits, 64, fma=True).astype(np.float16)
    y64, mag = oracle.linear_f64_c(a, w16, bias.numpy())
    tol = (k + 2) * 2.0 ** -24 * mag + np.abs(y64) * 2.0 ** -11 + 2.0 ** -25
    err = np.abs(_np(y[rows.to(cuda)]).astype(np.float64) - y64)
    assert np.all(err <= tol), float((err / tol).max())
    assert torch.equal(ops.linear_otf(xd, *args, out_dtype=torch.float16), y)             # row-major entry point
    xh = ops.dequant_activation_hip(xd, d(thr), d(cb), 64)
    assert np.array_equal(_np(xh[rows.to(cuda)]).view(np.uint16), a.view(np.uint16))
    assert torch.equal(ops.linear_fused(xh, *args[2:], out_dtype=torch.float16), y)       # stage 1, then stages 2+3
    del xh
    perm = torch.randperm(m, device=cuda)
    yp = ops.linear_otf(xd[perm].contiguous(), *args, out_dtype=torch.float16, w_hat_ws=w_ws)
    assert torch.equal(yp, y[perm])
