"""Host-side (CPU, NumPy) bit packing used when a model is converted on the CPU.

Same role and byte layout as the reference's ``pack_codes_py`` / ``unpack_codes_py``
(FQ/arcq_packed_py.py:8-47, :50-78), which its converter patches in for CPU conversion
(scripts/convert_arcq_to_packed.py:56-59).  Conversion is offline host work; the forward path
never comes through here.
"""
from __future__ import annotations

import numpy as np
import torch


def pack_codes_py(codes: torch.Tensor, bits: int) -> torch.Tensor:
    """``[rows, length]`` integer codes -> ``uint8 [rows, ceil(length*bits/8)]``."""
    assert codes.dim() == 2, f"codes must be 2D, got {codes.dim()}"
    assert bits in (2, 3, 4), f"bits must be 2/3/4, got {bits}"
    c = codes.detach().cpu().numpy().astype(np.uint64) & np.uint64((1 << bits) - 1)
    rows, length = c.shape
    pcols = (length * bits + 7) // 8
    # Accumulate every code, shifted to its bit position inside its first byte, into 16-bit cells
    # (a code touches at most two bytes), then fold the spill into the following byte.
    bit_off = np.arange(length, dtype=np.int64) * bits
    byte_idx = bit_off >> 3
    shifted = (c << (bit_off & 7).astype(np.uint64)).astype(np.uint32)
    lo = np.zeros((rows, pcols + 1), dtype=np.uint32)
    np.add.at(lo, (slice(None), byte_idx), shifted & 0xFF)
    np.add.at(lo, (slice(None), byte_idx + 1), shifted >> 8)
    # Contributions to one byte occupy disjoint bits, so the sum equals the bitwise OR.
    return torch.from_numpy(lo[:, :pcols].astype(np.uint8)).to(device=codes.device)


def unpack_codes_py(packed: torch.Tensor, bits: int, length: int) -> torch.Tensor:
    """Inverse of :func:`pack_codes_py`; int64 ``[rows, length]``."""
    p = packed.detach().cpu().numpy().astype(np.uint32)
    rows = p.shape[0]
    p = np.concatenate([p, np.zeros((rows, 1), dtype=np.uint32)], axis=1)
    bit_off = np.arange(length, dtype=np.int64) * bits
    byte_idx = bit_off >> 3
    two = p[:, byte_idx] | (p[:, byte_idx + 1] << 8)
    codes = (two >> (bit_off & 7).astype(np.uint32)) & ((1 << bits) - 1)
    return torch.from_numpy(codes.astype(np.int64)).to(device=packed.device)
