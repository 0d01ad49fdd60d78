"""GPU tests of the packed patch-embedding convolution (``ARCQPackedPatchConv``) and of a model in the reference's
full quantization scope (ARCQ patch convolution + block linears, W8A8 LSQ head)."""
import numpy as np
import pytest
import torch

import arcq_vit_amd as A
from arcq_vit_amd import ops, synth
from arcq_vit_amd.vit import build_fakequant_vit, build_packed_vit

pytestmark = pytest.mark.gpu


def _np(t):
    return t.detach().cpu().numpy()


@pytest.mark.parametrize("bits", [4, 3, 2])
@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
def test_stage1_groups_of_three_channels(cuda, oracle, bits, dtype):
    """Stage 1 on pixels [B*H*W, 3] with one group of three channels per pixel (the activation grouping of
    FQ/quant_backends.py:351,366-368): bit-exact against the oracle, including constant pixels (scale = sqrt(eps))."""
    cb = synth.quantile_codebook(bits)
    thr = synth.midpoint_thresholds(cb)
    img = synth.make_images(2, 11)                                       # normalised U(0,1) images
    pix = img.permute(0, 2, 3, 1).reshape(-1, 3).contiguous().to(dtype)
    pix[:7] = pix[:7, :1]                                                # grey pixels: all residuals zero
    pix[7] = 0.0
    ref = oracle.act_quant_c(pix.float().numpy(), thr, cb, bits, 3)["x_hat"]
    got = ops.dequant_activation_hip(pix.to(cuda), thr.to(cuda), cb.to(cuda), 3)
    assert got.dtype == dtype
    want = ref.astype(np.float16) if dtype == torch.float16 else ref
    assert np.array_equal(_np(got).view(np.uint16 if dtype == torch.float16 else np.uint32),
                          want.view(np.uint16 if dtype == torch.float16 else np.uint32))


def _blocked(rows16: np.ndarray) -> np.ndarray:
    """[M, K] -> the 32-row block layout: whole blocks [M/32][K/8][32][8], a last block of r rows as [K/8][r][8]."""
    m, k = rows16.shape
    full = m // 32 * 32
    parts = [rows16[:full].reshape(full // 32, 32, k // 8, 8).transpose(0, 2, 1, 3).reshape(-1)]
    if m > full:
        parts.append(rows16[full:].reshape(m - full, k // 8, 8).transpose(1, 0, 2).reshape(-1))
    return np.concatenate(parts)


@pytest.mark.parametrize("bits,dtype,b,h,w", [(4, torch.float16, 2, 224, 224), (3, torch.float32, 3, 224, 224),
                                              (2, torch.float16, 1, 32, 48), (4, torch.float32, 5, 64, 16),
                                              (4, torch.float16, 64, 224, 224)])
def test_patch_rows_in_one_launch_equal_the_oracle(cuda, oracle, bits, dtype, b, h, w):
    """ops.quantize_patches (pixels quantized in groups of three channels and written as patch rows, one launch)
    against the oracle's stage 1 on the NHWC pixels, gathered into patch rows on the host: bit for bit, row-major and
    in the block layout (whole blocks and a ragged last one), grey and black pixels included."""
    cb = synth.quantile_codebook(bits)
    thr = synth.midpoint_thresholds(cb)
    g = torch.Generator().manual_seed(7 * b + h)
    img = (torch.rand(b, 3, h, w, generator=g) - 0.45) / 0.23
    img[0, :, :3, :5] = img[0, :1, :3, :5]                               # grey pixels: all residuals zero
    img[0, :, 4, :4] = 0.0
    img = img.to(dtype)
    pix = img.permute(0, 2, 3, 1).reshape(-1, 3).contiguous()
    xh = oracle.act_quant_c(pix.float().numpy(), thr, cb, bits, 3)["x_hat"].astype(np.float16)
    rows = xh.reshape(b, h // 16, 16, w // 16, 16, 3).transpose(0, 1, 3, 5, 2, 4).reshape(b * (h // 16) * (w // 16), 768)
    got = ops.quantize_patches(img.to(cuda), thr.to(cuda), cb.to(cuda), bits)
    assert got.shape == rows.shape and np.array_equal(_np(got).view(np.uint16), rows.view(np.uint16))
    gotb = ops.quantize_patches(img.to(cuda), thr.to(cuda), cb.to(cuda), bits, blocked=True)
    assert np.array_equal(_np(gotb).view(np.uint16), _blocked(rows).view(np.uint16))


def test_quantize_patches_argument_errors(cuda):
    lib = A._lib.load()
    img = torch.zeros(1, 3, 32, 32, dtype=torch.float16, device=cuda)
    t = torch.zeros(16, dtype=torch.float32, device=cuda)
    out = torch.zeros(4 * 768, dtype=torch.float16, device=cuda)
    call = lambda **k: lib.arcq_act_quant_patches(k.get("img", img.data_ptr()), k.get("dt", 1), t.data_ptr(), t.data_ptr(), out.data_ptr(),
                                                  1, k.get("c", 3), k.get("h", 32), 32, k.get("patch", 16), k.get("bits", 4), 1e-6, 0, None)
    assert call() == 0
    assert call(bits=5) == -1 and call(c=4) == -6 and call(patch=8) == -6 and call(h=40) == -4 and call(dt=7) == -5
    assert call(img=None) == -3 and call(img=img.data_ptr() + 2) == -7


@pytest.mark.parametrize("model,bits,batch,dtype", [("deit_small", 4, 8, torch.float16), ("deit_base", 3, 3, torch.float32),
                                                    ("deit_tiny", 2, 5, torch.float16)])
def test_packed_patch_conv_against_oracle(cuda, oracle, model, bits, batch, dtype):
    """The whole layer: oracle stage 1 on pixels -> fp16 -> patch rows -> fp64 product with the oracle's fp16
    weights, against the module's output, within the fp32-accumulation bound plus the output rounding; and against
    the fake-quant convolution it replaces (fp32 on the CPU), within the rounding of the operands to fp16."""
    dim = synth.MODEL_DIMS[model]["dim"]
    cb = synth.quantile_codebook(bits)
    thr = synth.midpoint_thresholds(cb)
    src = A.QuantConv2dPCARCQ(3, dim, 16, 16, 0, True, bits, bits)
    g = torch.Generator().manual_seed(21)
    with torch.no_grad():
        src.conv.weight.copy_(torch.randn(src.conv.weight.shape, generator=g) * 0.02)
        src.conv.bias.copy_(torch.randn(dim, generator=g) * 0.01)
    src.act_quant.set_codebook(cb)
    src.weight_quant.set_codebook(cb)
    layer = A.ARCQPackedPatchConv(src).to(cuda)
    x = synth.make_images(batch, 5).to(dtype)
    y = layer(x.to(cuda))
    torch.cuda.synchronize()
    assert tuple(y.shape) == (batch, dim, 14, 14) and y.dtype == dtype
    pix = x.permute(0, 2, 3, 1).reshape(-1, 3).contiguous()
    xh = oracle.act_quant_c(pix.float().numpy(), thr, cb, bits, 3)["x_hat"]
    if dtype == torch.float16:
        xh = xh.astype(np.float16).astype(np.float32)          # stage 1 writes the input's dtype, then fp16 rows
    rows = layer.patch_rows(torch.from_numpy(xh).reshape(batch, 224, 224, 3)).numpy().astype(np.float16)
    w16 = oracle.weight_dequant_c(_np(layer.packed_weight_codes), cb, _np(layer.weight_center), _np(layer.weight_scale),
                                  _np(layer.weight_code_sum), bits, 64, fma=True).astype(np.float16)
    y64, mag = oracle.linear_f64_c(rows, w16, _np(layer.bias))
    got = _np(y.permute(0, 2, 3, 1).reshape(-1, dim)).astype(np.float64)
    out_ulp = 2.0 ** -11 if dtype == torch.float16 else 2.0 ** -24
    tol = (768 + 2) * 2.0 ** -24 * mag + np.abs(y64) * out_ulp + 2.0 ** -25
    err = np.abs(got - y64)
    assert np.all(err <= tol), float((err / tol).max())
    with torch.no_grad():
        fq = src(x.float())                                     # fp32 fake quantization on the CPU
    # operands rounded to fp16 (2^-11 relative each) over a sum of |a*w|
    bound = 3 * 2.0 ** -11 * torch.from_numpy(mag).reshape(batch, 14, 14, dim).permute(0, 3, 1, 2) + 1e-4
    bad = ((y.float().cpu() - fq).abs() > bound).any(dim=1)            # [B, 14, 14]: patches with an output off
    # torch's reductions may order a sum differently from the serial kernel: a value on a threshold can then take the
    # neighbouring code, which moves every output of that one patch
    assert int(bad.sum()) <= 2, int(bad.sum())


def test_full_scope_model_forward(cuda):
    """DeiT-Small (two blocks) with the patch convolution packed and the LSQ head.  The head, given the features the
    GPU model produced, matches the same module on the CPU; the logits follow the fp32 fake-quant model's (codes that
    flip where fp16 operands move a value across a threshold keep the two from agreeing more closely than that)."""
    kw = dict(num_classes=100, depth=2, quantize_patch_embed=True, head_quant="w8a8")
    fq = build_fakequant_vit("deit_small", 4, **kw)
    vit = build_packed_vit("deit_small", 4, device="cuda", half_chain=False, **kw)
    assert isinstance(vit.patch_embed.proj, A.ARCQPackedPatchConv) and isinstance(vit.head, A.QuantLinearLSQ)
    seen = {}
    hook = vit.head.register_forward_hook(lambda mod, inp, out: seen.update(x=inp[0].detach().cpu(), y=out.detach().cpu()))
    x = synth.make_images(6, 2)
    with torch.no_grad():
        ref = fq(x)
        got = vit(x.to(cuda)).float().cpu()
        head_ref = fq.head(seen["x"].float())
    hook.remove()
    assert bool(torch.isfinite(got).all()) and tuple(got.shape) == (6, 100)
    assert float((seen["y"].float() - head_ref).abs().max()) <= 1e-4 * float(head_ref.abs().max()) + 1e-5
    cos = torch.nn.functional.cosine_similarity(got.flatten(), ref.flatten(), dim=0)
    assert float(cos) >= 0.9, float(cos)
    half = build_packed_vit("deit_small", 4, device="cuda", half_chain=True, **kw)
    with torch.no_grad():
        got16 = half(x.to(cuda).half()).float().cpu()
    cos16 = torch.nn.functional.cosine_similarity(got16.flatten(), ref.flatten(), dim=0)
    assert bool(torch.isfinite(got16).all()) and float(cos16) >= 0.9, float(cos16)
    print(f"logit cosine vs fp32 fake quantization: fp32 chain {float(cos):.4f}, half chain {float(cos16):.4f}")


def test_packed_checkpoint_round_trip_on_gpu(cuda, tmp_path):
    """Training checkpoint -> converter command line (patch convolution packed too) -> packed file -> plain skeleton
    via load_packed_state_dict -> GPU forward: the logits equal those of the model converted in memory, bit for bit
    (same buffers, same kernels)."""
    import yaml
    from arcq_vit_amd import convert
    from arcq_vit_amd.vit import VisionTransformer
    kw = dict(num_classes=10, quantize_patch_embed=True, head_quant="w8a8")
    src = build_fakequant_vit("deit_tiny", 4, **kw)
    ckpt = tmp_path / "best.pt"
    torch.save({"model": {"module." + k: v for k, v in src.state_dict().items()}, "epoch": 1}, ckpt)
    cfg = tmp_path / "cfg.yaml"
    cfg.write_text(yaml.safe_dump({"model_name": "deit_tiny_patch16_224", "num_classes": 10, "w_bits": 4, "a_bits": 4,
                                   "head_quant": "w8a8"}))
    convert.main(["--config", str(cfg), "--checkpoint", str(ckpt), "--output-dir", str(tmp_path), "--pack-patch-embed"])
    state = torch.load(tmp_path / "deit_tiny_w4a4_packed_packed.pt", map_location="cpu", weights_only=True)
    d = synth.MODEL_DIMS["deit_tiny"]
    loaded = A.load_packed_state_dict(VisionTransformer(d["dim"], d["depth"], d["heads"], d["mlp"], 10), state).to(cuda).eval()
    direct = build_packed_vit("deit_tiny", 4, device="cuda", half_chain=False, **kw)
    assert isinstance(loaded.patch_embed.proj, A.ARCQPackedPatchConv)
    assert sum(isinstance(m, A.ARCQPackedLinearOnTheFly) for m in loaded.modules()) == 48
    x = synth.make_images(4, 9).to(cuda)
    with torch.no_grad():
        assert torch.equal(loaded(x), direct(x))
