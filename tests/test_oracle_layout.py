"""Pins the oracle's bit layout (EXT/arcq_pack_kernel.cu:8-36; FQ/arcq_packed_py.py) without the
reference: hand-derived byte vectors, the closed form byte[(j*b)>>3] >> ((j*b)&7), brute force
over all code values, round trips, and agreement of three independently written packers
(C loop, numpy bitstream, numpy two-byte scatter of the shipped host helper)."""
import itertools

import numpy as np
import pytest
import torch


def test_hand_vectors(oracle):
    # 4-bit: byte k = c[2k] | c[2k+1] << 4
    assert oracle.pack_codes_c(np.array([[1, 2, 3, 4]]), 4).tolist() == [[0x21, 0x43]]
    # 3-bit: 8 codes form a 24-bit little-endian word, code i at bit 3i:
    # 1 + 2<<3 + 3<<6 + 4<<9 + 5<<12 + 6<<15 + 7<<18 + 0<<21 = 0x1F58D1
    assert oracle.pack_codes_c(np.array([[1, 2, 3, 4, 5, 6, 7, 0]]), 3).tolist() == [[0xD1, 0x58, 0x1F]]
    # 2-bit: 4 codes per byte
    assert oracle.pack_codes_c(np.array([[3, 0, 1, 2]]), 2).tolist() == [[0b10010011]]
    # a ragged tail: 3 codes of 3 bits = 9 bits -> 2 bytes, top 7 bits zero
    assert oracle.pack_codes_c(np.array([[7, 7, 7]]), 3).tolist() == [[0xFF, 0x01]]


@pytest.mark.parametrize("bits", [2, 3, 4])
def test_single_code_closed_form(oracle, bits):
    """Setting only code j to v must set exactly bits [j*bits, (j+1)*bits) of the stream."""
    length = 19
    for j in range(length):
        for v in range(1 << bits):
            codes = np.zeros((1, length), dtype=np.int64)
            codes[0, j] = v
            packed = oracle.pack_codes_c(codes, bits)[0]
            stream = int.from_bytes(packed.tobytes(), "little")
            assert stream == v << (j * bits)


@pytest.mark.parametrize("bits", [2, 3, 4])
def test_bruteforce_all_pairs(oracle, bits):
    """Every pair of neighbouring code values at every alignment (covers every byte straddle)."""
    levels = 1 << bits
    pairs = np.array(list(itertools.product(range(levels), repeat=2)), dtype=np.int64)
    for offset in range(8):
        codes = np.zeros((len(pairs), offset + 2), dtype=np.int64)
        codes[:, offset:] = pairs
        packed = oracle.pack_codes_c(codes, bits)
        for row, (a, b) in zip(packed, pairs):
            stream = int.from_bytes(row.tobytes(), "little")
            assert (stream >> (offset * bits)) & (levels - 1) == a
            assert (stream >> ((offset + 1) * bits)) & (levels - 1) == b
        assert np.array_equal(oracle.unpack_codes_c(packed, bits, offset + 2), codes)


@pytest.mark.parametrize("bits", [2, 3, 4])
@pytest.mark.parametrize("length", [1, 7, 8, 64, 192, 197, 384])
def test_three_packers_agree_and_roundtrip(oracle, bits, length):
    from arcq_vit_amd.pack_py import pack_codes_py, unpack_codes_py
    rng = np.random.default_rng(bits * 1000 + length)
    codes = rng.integers(0, 1 << bits, size=(5, length), dtype=np.int64)
    pc = oracle.pack_codes_c(codes, bits)
    pn = oracle.pack_codes_np(codes, bits)
    pp = pack_codes_py(torch.from_numpy(codes), bits).numpy()
    assert pc.shape == (5, (length * bits + 7) // 8)
    assert np.array_equal(pc, pn) and np.array_equal(pc, pp)
    assert np.array_equal(oracle.unpack_codes_c(pc, bits, length), codes)
    assert np.array_equal(oracle.unpack_codes_np(pc, bits, length), codes)
    assert np.array_equal(oracle.unpack_codes_u8_c(pc, bits, length), codes.astype(np.uint8))
    assert np.array_equal(unpack_codes_py(torch.from_numpy(pc), bits, length).numpy(), codes)


def test_codes_are_masked(oracle):
    """set_packed_code_u8 masks to the low `bits` bits (EXT/arcq_pack_kernel.cu:30-31)."""
    from arcq_vit_amd.pack_py import pack_codes_py
    codes = np.array([[0x1F, 0x23, -1, 7]], dtype=np.int64)
    for bits in (2, 3, 4):
        want = oracle.pack_codes_c(codes & ((1 << bits) - 1), bits)
        assert np.array_equal(oracle.pack_codes_c(codes, bits), want)
        assert np.array_equal(pack_codes_py(torch.from_numpy(codes), bits).numpy(), want)


def test_group_bytes(oracle):
    """A 64-code group is 32 / 24 / 16 bytes for 4 / 3 / 2 bits, so groups never share a byte."""
    for bits, nbytes in ((4, 32), (3, 24), (2, 16)):
        codes = np.zeros((1, 128), dtype=np.int64)
        codes[0, 64:] = (1 << bits) - 1
        packed = oracle.pack_codes_c(codes, bits)[0]
        assert not packed[:nbytes].any() and (packed[nbytes:] == 0xFF).all()


def test_empty(oracle):
    assert oracle.pack_codes_c(np.zeros((0, 8), dtype=np.int64), 4).shape == (0, 4)
    assert oracle.pack_codes_c(np.zeros((3, 0), dtype=np.int64), 3).shape == (3, 0)
