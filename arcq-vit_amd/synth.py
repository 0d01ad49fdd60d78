"""Seeded synthetic inputs for the benchmark configurations (no datasets or checkpoints exist
offline): quantile codebooks, Gaussian weights, activations with outliers, GELU-shaped fc2
inputs, normalised images, and the DeiT / ViT linear shapes.
"""
from __future__ import annotations

from typing import Dict, List, Tuple

import torch

SEED = 20260630  # the seed scripts/debug_arcq_packed_correctness.py:133 uses
IMAGENET_MEAN = (0.485, 0.456, 0.406)
IMAGENET_STD = (0.229, 0.224, 0.225)

# (in_features, out_features) of the four block linears, by model width
MODEL_DIMS: Dict[str, Dict[str, int]] = {
    "deit_tiny": {"dim": 192, "depth": 12, "heads": 3, "mlp": 768},
    "deit_small": {"dim": 384, "depth": 12, "heads": 6, "mlp": 1536},
    "deit_base": {"dim": 768, "depth": 12, "heads": 12, "mlp": 3072},
    "vit_large": {"dim": 1024, "depth": 24, "heads": 16, "mlp": 4096},
}
TOKENS = 197  # 14*14 patches + cls


def block_linear_shapes(model: str) -> List[Tuple[str, int, int]]:
    """``[(name, K, N)]`` for qkv / proj / fc1 / fc2 of one transformer block."""
    d, h = MODEL_DIMS[model]["dim"], MODEL_DIMS[model]["mlp"]
    return [("qkv", d, 3 * d), ("proj", d, d), ("fc1", d, h), ("fc2", h, d)]


def quantile_codebook(bits: int) -> torch.Tensor:
    """``2^bits`` levels at the standard-normal quantiles ``Phi^-1((i + 1/2) / L)``, fp32, sorted."""
    levels = 1 << bits
    p = (torch.arange(levels, dtype=torch.float64) + 0.5) / levels
    return torch.special.ndtri(p).to(torch.float32)


def midpoint_thresholds(codebook: torch.Tensor) -> torch.Tensor:
    """Adjacent midpoints, computed in fp32 as Q/dcarcq.py:483 does."""
    cb = codebook.float()
    return (cb[:-1] + cb[1:]) / 2.0


def gen(seed: int) -> torch.Generator:
    return torch.Generator().manual_seed(int(seed))


def make_weight(n: int, k: int, seed: int) -> torch.Tensor:
    """``W ~ N(0, 0.02^2)``."""
    return torch.randn(n, k, generator=gen(seed)) * 0.02


def make_bias(n: int, seed: int) -> torch.Tensor:
    """``b ~ N(0, 0.01^2)``."""
    return torch.randn(n, generator=gen(seed + 1)) * 0.01


def make_activation(m: int, k: int, seed: int, kind: str = "ln") -> torch.Tensor:
    """``kind="ln"``: N(0,1) with 0.5 % of entries set to +-8 (post-LayerNorm-like, with outliers).
    ``kind="gelu"``: GELU of N(0,1)*1.5 (heavy-tailed, non-negative-skewed fc2 input)."""
    g = gen(seed + 2)
    x = torch.randn(m, k, generator=g)
    if kind == "gelu":
        return torch.nn.functional.gelu(x * 1.5)
    mask = torch.rand(m, k, generator=g) < 0.005
    sign = torch.where(torch.rand(m, k, generator=g) < 0.5, -1.0, 1.0)
    return torch.where(mask, 8.0 * sign, x)


def make_images(batch: int, seed: int, size: int = 224) -> torch.Tensor:
    """``U(0,1)`` images normalised with the ImageNet mean/std (FW/data.py:25-26)."""
    x = torch.rand(batch, 3, size, size, generator=gen(seed + 3))
    mean = torch.tensor(IMAGENET_MEAN).view(1, 3, 1, 1)
    std = torch.tensor(IMAGENET_STD).view(1, 3, 1, 1)
    return (x - mean) / std


def algorithmic_bytes(m: int, n: int, k: int, bits: int, gs: int = 64, io_bytes: int = 2) -> int:
    """HBM bytes one packed linear call has to move: packed W + (mu, s, S) per group + codebooks and
    thresholds + bias + x in + y out."""
    levels = 1 << bits
    return n * k * bits // 8 + 12 * n * k // gs + 4 * (3 * levels - 1) + 4 * n + io_bytes * m * k + io_bytes * m * n


def algorithmic_flops(m: int, n: int, k: int) -> int:
    return 2 * m * n * k
