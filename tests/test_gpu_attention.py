"""GPU tests of the softmax attention kernel that sits between the packed qkv and proj layers (``ops.attention_fwd``).
The reference leaves attention to timm / torch, so there is nothing of its own to be bit-equal to: the check is the
mathematical definition in float64 on the same fp16 inputs, with an error bound derived from what the kernel rounds
(fp32 scores and accumulation, probabilities rounded to fp16, one fp16 rounding of the output)."""
import numpy as np
import pytest
import torch

from arcq_vit_amd import _lib, ops, synth
from arcq_vit_amd.vit import build_packed_vit

pytestmark = pytest.mark.gpu


def _reference(qkv: torch.Tensor, heads: int, scale: float):
    """float64 attention and the magnitude ``softmax @ |v|`` the error bound scales with."""
    b, n, c3 = qkv.shape
    c = c3 // 3
    q, k, v = qkv.double().cpu().reshape(b, n, 3, heads, c // heads).permute(2, 0, 3, 1, 4).unbind(0)
    p = torch.softmax(q @ k.transpose(-1, -2) * scale, dim=-1)
    out = (p @ v).transpose(1, 2).reshape(b, n, c)
    mag = (p @ v.abs()).transpose(1, 2).reshape(b, n, c)
    smax = (q @ k.transpose(-1, -2) * scale).abs().max().item()
    return out, mag, smax


def _check(qkv, heads, scale=None):
    got = ops.attention_fwd(qkv, heads, scale)
    want, mag, smax = _reference(qkv, heads, 0.125 if scale is None else scale)
    # probabilities: fp32 score error (64 products, ~2^-22 relative to the largest score) goes through exp, then one fp16
    # rounding (2^-11) of p and of the output, fp32 accumulation over n keys on top
    tol = (2.0 ** -10 + 2.0 ** -20 * max(smax, 1.0)) * mag + want.abs() * 2.0 ** -11 + 2.0 ** -24
    err = (got.double().cpu() - want).abs()
    assert bool((err <= tol).all()), (tuple(qkv.shape), heads, float((err / tol).max()))
    return got


@pytest.mark.parametrize("b,n,heads", [(1, 197, 6), (3, 197, 3), (2, 1, 2), (1, 32, 1), (2, 33, 4), (1, 256, 2),
                                       (5, 64, 12), (2, 50, 16), (1, 225, 3), (64, 197, 6)])
def test_attention_matches_float64(cuda, b, n, heads):
    g = torch.Generator().manual_seed(100 * n + heads)
    qkv = torch.randn(b, n, 3 * heads * 64, generator=g).half().to(cuda)
    _check(qkv, heads)


def test_attention_peaked_and_shifted_scores(cuda):
    """Large scores (softmax close to one-hot, |score| up to a few hundred) and a common offset on every key: the
    maximum is subtracted before the exponential, so neither overflows nor loses the small probabilities."""
    g = torch.Generator().manual_seed(5)
    b, n, heads = 2, 197, 3
    qkv = torch.randn(b, n, 3, heads, 64, generator=g)
    qkv[:, :, 0] *= 6.0                                  # q
    qkv[:, :, 1] += 2.0                                  # k: a shared component -> a per-query score offset
    qkv = qkv.reshape(b, n, 3 * heads * 64).half().to(cuda)
    _check(qkv, heads)
    _check(qkv, heads, scale=0.5)


def test_attention_equals_torch_closely_and_writes_into_out(cuda):
    g = torch.Generator().manual_seed(9)
    b, n, heads = 4, 197, 6
    qkv = torch.randn(b, n, 3 * heads * 64, generator=g).half().to(cuda)
    out = torch.full((b, n, heads * 64), float("nan"), dtype=torch.float16, device=cuda)
    got = ops.attention_fwd(qkv, heads, out=out)
    assert got.data_ptr() == out.data_ptr() and bool(torch.isfinite(out).all())
    q, k, v = qkv.reshape(b, n, 3, heads, 64).permute(2, 0, 3, 1, 4).unbind(0)
    ref = torch.nn.functional.scaled_dot_product_attention(q, k, v).transpose(1, 2).reshape(b, n, heads * 64)
    assert float((got.float() - ref.float()).abs().max()) < 4e-3


def test_attention_argument_errors(cuda):
    lib = _lib.load()
    x = torch.zeros(1, 8, 3 * 64, dtype=torch.float16, device=cuda)
    y = torch.zeros(1, 8, 64, dtype=torch.float16, device=cuda)
    assert lib.arcq_attention_fwd(x.data_ptr(), y.data_ptr(), 1, 8, 1, 32, 0.125, None) == -6
    assert b"head_dim" in lib.arcq_last_error()
    assert lib.arcq_attention_fwd(x.data_ptr(), y.data_ptr(), 1, 257, 1, 64, 0.125, None) == -6
    assert lib.arcq_attention_fwd(None, y.data_ptr(), 1, 8, 1, 64, 0.125, None) == -3
    assert lib.arcq_attention_fwd(x.data_ptr() + 2, y.data_ptr(), 1, 8, 1, 64, 0.125, None) == -7
    assert lib.arcq_attention_fwd(x.data_ptr(), y.data_ptr(), 0, 8, 1, 64, 0.125, None) == 0
    with pytest.raises(RuntimeError, match="head dimension"):
        ops.attention_fwd(torch.zeros(1, 8, 3 * 96, dtype=torch.float16, device=cuda), 2)


@pytest.mark.parametrize("model,batch", [("deit_small", 8), ("deit_tiny", 1)])
def test_vit_with_own_attention(cuda, model, batch):
    """The skeleton ViT with the library's attention kernel instead of torch's: the attention outputs differ in their
    last bits, which the next layer's quantizer may turn into different codes at ties, so the logits are close, not
    equal."""
    kw = dict(num_classes=100, device="cuda", half_chain=True, depth=2, shared_buffers=True,
              max_rows=batch * synth.TOKENS, fuse_elementwise=True)
    own = build_packed_vit(model, 4, own_attention=True, **kw)
    lib_attn = build_packed_vit(model, 4, own_attention=False, **kw)
    x = synth.make_images(batch, 1).to(cuda).half()
    seen = []
    hooks = [blk.attn.proj.register_forward_hook(lambda m, a, o: seen.append(a[0])) for blk in own.blocks]
    with torch.no_grad():
        a, b = own(x), lib_attn(x)
    for h in hooks:
        h.remove()
    assert len(seen) == 2 and all(t.shape == (batch, synth.TOKENS, own.blocks[0].attn.proj.in_features) for t in seen)
    assert bool(torch.isfinite(a).all())
    cos = torch.nn.functional.cosine_similarity(a.float().flatten(), b.float().flatten(), dim=0).item()
    assert cos > 0.99, cos
