"""Minimal DeiT / ViT skeleton whose submodule names match timm's ``VisionTransformer``
(``patch_embed.proj``, ``cls_token``, ``pos_embed``, ``blocks.N.{norm1,attn.{qkv,proj},norm2,
mlp.{fc1,fc2}}``, ``norm``, ``head``), so packed-checkpoint keys produced from a timm model
(FQ/timm_quant_models.py:155-182) line up.  timm itself is not available offline.

By default only the four block linears are quantized (the packed path's scope); patch embedding, LayerNorm,
softmax attention, GELU and the head stay in floating point, as the reference's README states.  The builders can
also give the model the reference's full quantization scope (FQ/timm_quant_models.py:63-121): the ARCQ wrapper on the
patch-embedding convolution and the W8A8 LSQ wrapper on the head.
"""
from __future__ import annotations

from typing import Callable, Optional

import torch
import torch.nn as nn
import torch.nn.functional as F

from .packed_convert import (convert_arcq_conv_to_packed, convert_arcq_linear_to_packed, share_buffers,
                             to_on_the_fly)
from .quant_source import QuantConv2dPCARCQ, QuantLinearLSQ, QuantLinearPCARCQ
from .synth import MODEL_DIMS, SEED, quantile_codebook

LinearFactory = Callable[[int, int, bool], nn.Module]


class PatchEmbed(nn.Module):
    def __init__(self, dim: int, patch: int = 16, in_ch: int = 3):
        super().__init__()
        self.proj = nn.Conv2d(in_ch, dim, kernel_size=patch, stride=patch)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return self.proj(x).flatten(2).transpose(1, 2)


class Attention(nn.Module):
    def __init__(self, dim: int, heads: int, linear: LinearFactory):
        super().__init__()
        self.num_heads = heads
        self.qkv = linear(dim, dim * 3, True)
        self.proj = linear(dim, dim, True)
        # True: the library's own attention kernel where it serves the shape (fp16 on the GPU, head dimension 64, at
        # most 256 tokens): one launch that reads qkv's output and writes proj's input as they lie.
        self.own_kernel = False

    def mix(self, qkv: torch.Tensor) -> torch.Tensor:
        """Softmax attention on the output of ``qkv`` ``[B, tokens, 3 C]`` -> ``[B, tokens, C]`` (input of ``proj``)."""
        b, n, c3 = qkv.shape
        c = c3 // 3
        if (self.own_kernel and qkv.is_cuda and qkv.dtype == torch.float16 and c == 64 * self.num_heads and n <= 256
                and qkv.is_contiguous()):
            from . import ops
            return ops.attention_fwd(qkv, self.num_heads)
        q, k, v = qkv.reshape(b, n, 3, self.num_heads, c // self.num_heads).permute(2, 0, 3, 1, 4).unbind(0)
        return F.scaled_dot_product_attention(q, k, v).transpose(1, 2).reshape(b, n, c)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return self.proj(self.mix(self.qkv(x)))


class Mlp(nn.Module):
    def __init__(self, dim: int, hidden: int, linear: LinearFactory):
        super().__init__()
        self.fc1 = linear(dim, hidden, True)
        self.act = nn.GELU()
        self.fc2 = linear(hidden, dim, True)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return self.fc2(self.act(self.fc1(x)))


class Block(nn.Module):
    def __init__(self, dim: int, heads: int, hidden: int, linear: LinearFactory):
        super().__init__()
        self.norm1 = nn.LayerNorm(dim, eps=1e-6)
        self.attn = Attention(dim, heads, linear)
        self.norm2 = nn.LayerNorm(dim, eps=1e-6)
        self.mlp = Mlp(dim, hidden, linear)
        # True (and the four linears on-the-fly packed layers): the LayerNorms, the GELU and the two skip connections
        # run inside the packed layers' launches (ARCQPackedLinearOnTheFly.forward's optional arguments).
        self.fuse_elementwise = False
        # With fuse_elementwise: let fc1's launch end with fc2's stage 1 where the layers can (the GELU output then never
        # exists as a tensor); results are the same bits either way.
        self.chain_mlp = True

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        if self.fuse_elementwise and isinstance(self.mlp.act, nn.GELU) and self.mlp.act.approximate == "none":
            a = self.attn
            x = a.proj(a.mix(a.qkv(x, layernorm=self.norm1)), residual=x)
            fc1, fc2 = self.mlp.fc1, self.mlp.fc2
            rows = x.numel() // x.shape[-1]
            if self.chain_mlp and hasattr(fc1, "can_quantize_for") and fc1.can_quantize_for(fc2, rows):
                # the GELU output is only ever consumed quantized: fc1's launch ends with fc2's stage 1
                h = fc1(x, layernorm=self.norm2, activation="gelu", quantize_for=fc2)
                return fc2(h, residual=x, input_is_xhat=True)
            return fc2(fc1(x, layernorm=self.norm2, activation="gelu"), residual=x)
        x = x + self.attn(self.norm1(x))
        return x + self.mlp(self.norm2(x))


class VisionTransformer(nn.Module):
    def __init__(self, dim: int, depth: int, heads: int, mlp: int, num_classes: int = 1000,
                 linear: Optional[LinearFactory] = None, img: int = 224, patch: int = 16):
        super().__init__()
        linear = linear or (lambda i, o, b: nn.Linear(i, o, bias=b))
        self.embed_dim = dim
        self.patch_embed = PatchEmbed(dim, patch)
        n_patches = (img // patch) ** 2
        self.cls_token = nn.Parameter(torch.zeros(1, 1, dim))
        self.pos_embed = nn.Parameter(torch.zeros(1, n_patches + 1, dim))
        self.blocks = nn.Sequential(*[Block(dim, heads, mlp, linear) for _ in range(depth)])
        self.norm = nn.LayerNorm(dim, eps=1e-6)
        self.head = nn.Linear(dim, num_classes)
        # True: the library's one-launch fp16 patch embedding where it serves the model (see forward_features)
        self.own_patch_embed = False

    def forward_features(self, x: torch.Tensor) -> torch.Tensor:
        conv = self.patch_embed.proj
        if (self.own_patch_embed and type(conv) is nn.Conv2d and x.is_cuda and x.dtype == torch.float16
                and conv.weight.dtype == torch.float16 and conv.kernel_size == (16, 16) and conv.stride == (16, 16)
                and conv.padding == (0, 0) and conv.in_channels == 3 and conv.out_channels % 32 == 0
                and x.shape[-1] % 16 == 0 and x.shape[-2] % 16 == 0):
            from . import ops       # convolution, class token and position embedding in one launch
            x = ops.patch_embed_fwd(x, conv.weight, conv.bias, self.cls_token, self.pos_embed)
        else:
            x = self.patch_embed(x)
            x = torch.cat([self.cls_token.expand(x.shape[0], -1, -1).to(x.dtype), x], dim=1) + self.pos_embed.to(x.dtype)
        x = self.blocks(x)
        # LayerNorm works token by token and the head reads the class token only: with own_patch_embed (the trimmed
        # trunk) only that row is normalised -- the same logits as normalising all tokens first, which is what timm's
        # forward_features does and what happens otherwise
        return self.norm(x[:, :1] if self.own_patch_embed else x)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return self.head(self.forward_features(x)[:, 0])


def build_fakequant_vit(model: str, bits: int, group_size: int = 64, seed: int = SEED,
                        num_classes: int = 1000, depth: Optional[int] = None, quantize_patch_embed: bool = False,
                        head_quant: str = "fp32") -> VisionTransformer:
    """Random-init ViT whose block linears are ``QuantLinearPCARCQ`` with quantile codebooks
    (weights N(0, 0.02^2), as timm's trunc_normal_(std=.02) init; biases N(0, 0.01^2)).
    ``depth`` overrides the model's number of blocks (a shallower model of the same widths).
    ``quantize_patch_embed`` wraps ``patch_embed.proj`` in ``QuantConv2dPCARCQ`` (same codebook), ``head_quant="w8a8"``
    the head in ``QuantLinearLSQ`` with step sizes initialised from the weights and from unit-variance input."""
    cfg = dict(MODEL_DIMS[model])
    if depth is not None:
        cfg["depth"] = int(depth)
    cb = quantile_codebook(bits)

    def make(i: int, o: int, b: bool) -> nn.Module:
        layer = QuantLinearPCARCQ(i, o, b, bits, bits, group_size)
        layer.act_quant.set_codebook(cb)
        layer.weight_quant.set_codebook(cb)
        return layer

    g = torch.Generator().manual_seed(int(seed))
    vit = VisionTransformer(cfg["dim"], cfg["depth"], cfg["heads"], cfg["mlp"], num_classes, linear=make)
    with torch.no_grad():
        for name, p in vit.named_parameters():
            if p.dim() >= 2:
                p.copy_(torch.randn(p.shape, generator=g) * 0.02)
            elif name.endswith("bias"):
                p.copy_(torch.randn(p.shape, generator=g) * 0.01)
            # LayerNorm weights keep their default of one
        if quantize_patch_embed:
            conv = vit.patch_embed.proj
            q = QuantConv2dPCARCQ(conv.in_channels, conv.out_channels, conv.kernel_size, conv.stride, conv.padding,
                                  True, bits, bits, group_size)
            q.conv.load_state_dict(conv.state_dict())
            q.act_quant.set_codebook(cb)
            q.weight_quant.set_codebook(cb)
            vit.patch_embed.proj = q
        if head_quant != "fp32":
            head = QuantLinearLSQ(vit.head.in_features, vit.head.out_features, True, 8, 8)
            head.linear.load_state_dict(vit.head.state_dict())
            head.weight_quant.init_from(head.linear.weight)
            head.act_quant.init_from(torch.randn(4096, generator=g))
            vit.head = head
    return vit.eval()


def build_packed_vit(model: str, bits: int, group_size: int = 64, seed: int = SEED, num_classes: int = 1000,
                     device: str = "cuda", half_chain: bool = True, depth: Optional[int] = None,
                     shared_buffers: bool = False, max_rows: int = 0, fuse_elementwise: bool = False,
                     quantize_patch_embed: bool = False, head_quant: str = "fp32",
                     own_attention: bool = False, own_patch_embed: bool = False) -> VisionTransformer:
    """Fake-quant ViT -> packed (``convert_arcq_linear_to_packed``) -> on-the-fly layers -> device,
    the sequence of scripts/benchmark_arcq_on_the_fly.py:88-199.  ``half_chain`` casts the
    floating-point rest of the model to fp16 (packed metadata stays fp32).  ``shared_buffers`` gives all
    layers one weight scratch buffer (:182-191 there) and, with ``max_rows`` tokens, one x_hat buffer.
    ``fuse_elementwise``: LayerNorm, GELU and the skip connections run inside the packed layers' launches.
    ``own_attention``: softmax attention on the library's kernel instead of torch's; ``own_patch_embed``: the fp16 patch
    convolution, class token and position embedding in one launch of the library's instead of four torch kernels.
    ``quantize_patch_embed``: the patch embedding is an ``ARCQPackedPatchConv``; ``head_quant="w8a8"``: LSQ head."""
    vit = build_fakequant_vit(model, bits, group_size, seed, num_classes, depth, quantize_patch_embed, head_quant)
    convert_arcq_linear_to_packed(vit, runtime_code_format="packed")
    convert_arcq_conv_to_packed(vit)
    to_on_the_fly(vit)
    vit = vit.to(device)
    if half_chain:
        vit = vit.half()
    if shared_buffers:
        share_buffers(vit, max_rows)
    for blk in vit.blocks:
        blk.fuse_elementwise = bool(fuse_elementwise)
        blk.attn.own_kernel = bool(own_attention)
    vit.own_patch_embed = bool(own_patch_embed)
    return vit.eval()
