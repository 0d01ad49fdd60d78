"""GPU tests of the one-launch fp16 patch embedding (``ops.patch_embed_fwd``: 16 x 16 patch convolution from the NCHW
image, class token, position embedding).  The reference's models run this part in torch, so the check is the definition
in float64 with a bound for fp32 accumulation and the two fp16 roundings, plus agreement with the torch operations it
replaces inside the skeleton model."""
import pytest
import torch

from arcq_vit_amd import _lib, ops, synth
from arcq_vit_amd.vit import build_packed_vit

pytestmark = pytest.mark.gpu


def _reference(img, w, bias, cls, pos):
    b, _, h, wd = img.shape
    n = w.shape[0]
    patches = torch.nn.functional.unfold(img.double().cpu(), kernel_size=16, stride=16).transpose(1, 2)      # [B, np, 768]
    w2 = w.double().cpu().reshape(n, -1)
    y = patches @ w2.T
    mag = patches.abs() @ w2.abs().T
    if bias is not None:
        y = y + bias.double().cpu()
        mag = mag + bias.double().cpu().abs()
    return y, mag, cls.double().cpu().reshape(1, 1, n), pos.double().cpu().reshape(1, -1, n)


@pytest.mark.parametrize("b,h,w,n,with_bias", [(1, 224, 224, 384, True), (2, 224, 224, 192, True), (3, 32, 48, 64, False),
                                               (64, 224, 224, 384, True), (5, 224, 224, 768, True), (1, 16, 16, 32, True)])
def test_patch_embed_matches_float64(cuda, b, h, w, n, with_bias):
    g = torch.Generator().manual_seed(b * 1000 + n)
    img = torch.randn(b, 3, h, w, generator=g).half().to(cuda)
    wt = (torch.randn(n, 3, 16, 16, generator=g) * 0.05).half().to(cuda)
    bias = (torch.randn(n, generator=g) * 0.1).half().to(cuda) if with_bias else None
    tokens = 1 + (h // 16) * (w // 16)
    cls = torch.randn(1, 1, n, generator=g).half().to(cuda)
    pos = torch.randn(1, tokens, n, generator=g).half().to(cuda)
    got = ops.patch_embed_fwd(img, wt, bias, cls, pos).double().cpu()
    assert got.shape == (b, tokens, n)
    y, mag, c64, p64 = _reference(img, wt, bias, cls, pos)
    want = y + p64[:, 1:]
    # fp32 accumulation of 768 products and the bias, one rounding of the convolution's output, one of the sum
    tol = 770 * 2.0 ** -24 * mag + y.abs() * 2.0 ** -11 + want.abs() * 2.0 ** -11 + 2.0 ** -24
    assert bool(((got[:, 1:] - want).abs() <= tol).all())
    cls_want = (c64 + p64[:, :1]).expand(b, 1, n)
    assert bool(((got[:, :1] - cls_want).abs() <= cls_want.abs() * 2.0 ** -11 + 2.0 ** -24).all())


def test_patch_embed_equals_the_torch_operations_closely(cuda):
    g = torch.Generator().manual_seed(3)
    b, n = 4, 384
    img = torch.randn(b, 3, 224, 224, generator=g).half().to(cuda)
    conv = torch.nn.Conv2d(3, n, 16, 16).half().to(cuda)
    cls = torch.randn(1, 1, n, generator=g).half().to(cuda)
    pos = torch.randn(1, 197, n, generator=g).half().to(cuda)
    with torch.no_grad():
        x = conv(img).flatten(2).transpose(1, 2)
        ref = torch.cat([cls.expand(b, -1, -1), x], dim=1) + pos
        got = ops.patch_embed_fwd(img, conv.weight, conv.bias, cls, pos)
    assert torch.equal(got[:, 0], ref[:, 0])
    # same roundings; only the order of the fp32 accumulation differs
    assert float((got.float() - ref.float()).abs().max()) <= 2.0 ** -8


def test_patch_embed_argument_errors(cuda):
    lib = _lib.load()
    img = torch.zeros(1, 3, 32, 32, dtype=torch.float16, device=cuda)
    w = torch.zeros(64, 768, dtype=torch.float16, device=cuda)
    v = torch.zeros(5 * 64, dtype=torch.float16, device=cuda)
    out = torch.zeros(5 * 64, dtype=torch.float16, device=cuda)
    args = lambda **k: (k.get("img", img.data_ptr()), w.data_ptr(), None, v.data_ptr(), v.data_ptr(), out.data_ptr(), 1,
                        k.get("h", 32), 32, k.get("patch", 16), k.get("n", 64), None)
    assert lib.arcq_patch_embed_fwd(*args()) == 0
    assert lib.arcq_patch_embed_fwd(*args(patch=14)) == -6
    assert lib.arcq_patch_embed_fwd(*args(h=30)) == -4
    assert lib.arcq_patch_embed_fwd(*args(n=48)) == -6
    assert lib.arcq_patch_embed_fwd(*args(img=None)) == -3
    assert lib.arcq_patch_embed_fwd(*args(img=img.data_ptr() + 2)) == -7
    with pytest.raises(RuntimeError, match="3, 16, 16"):
        ops.patch_embed_fwd(img, torch.zeros(64, 3, 8, 8, dtype=torch.float16, device=cuda), None, v[:64], v)


@pytest.mark.parametrize("model,batch", [("deit_small", 4), ("deit_tiny", 1)])
def test_vit_with_own_patch_embed(cuda, model, batch):
    kw = dict(num_classes=100, device="cuda", half_chain=True, depth=2, shared_buffers=True,
              max_rows=batch * synth.TOKENS, fuse_elementwise=True, own_attention=True)
    own = build_packed_vit(model, 4, own_patch_embed=True, **kw)
    ref = build_packed_vit(model, 4, own_patch_embed=False, **kw)
    x = synth.make_images(batch, 1).to(cuda).half()
    seen = []
    h = own.blocks[0].attn.qkv.register_forward_hook(lambda m, a, o: seen.append(a[0]))
    h2 = ref.blocks[0].attn.qkv.register_forward_hook(lambda m, a, o: seen.append(a[0]))
    with torch.no_grad():
        a, b = own(x), ref(x)
    h.remove()
    h2.remove()
    # the blocks' input: same roundings, accumulation order aside
    assert seen[0].shape == seen[1].shape == (batch, synth.TOKENS, own.embed_dim)
    assert float((seen[0].float() - seen[1].float()).abs().max()) <= 2.0 ** -8
    cos = torch.nn.functional.cosine_similarity(a.float().flatten(), b.float().flatten(), dim=0).item()
    assert cos > 0.99, cos
