"""Pins the oracle's list layout against the closed form of the interleaved format (no GPU).

Layout: list extents [ceil(n/32), ceil(pq_dim / (128 / pq_bits)), 32, 16] bytes
(cuVS cpp/include/cuvs/neighbors/ivf_pq.hpp:222-296); code j of row i lives in chunk j / cpc at
bit (j % cpc) * pq_bits of the 16-byte little-endian word at
((i / 32) * n_chunks + chunk) * 512 + (i % 32) * 16  (ivf_pq_codepacking.cuh:29-168).
"""
import os

import numpy as np
import pytest

GOLD = os.path.join(os.path.dirname(__file__), "golden")


def closed_form_get(list_bytes, i, j, pq_dim, pq_bits):
    cpc = 128 // pq_bits
    n_chunks = -(-pq_dim // cpc)
    base = ((i // 32) * n_chunks + j // cpc) * 512 + (i % 32) * 16
    word = int.from_bytes(bytes(list_bytes[base:base + 16]), "little")
    return (word >> ((j % cpc) * pq_bits)) & ((1 << pq_bits) - 1)


def test_derived_dimensions(orc):
    # cuVS cpp/src/neighbors/ivf_pq_index.cu:78-111
    assert [orc.dim_ext(d) for d in (128, 96, 768, 7, 8, 15)] == [136, 104, 776, 8, 16, 16]
    assert orc.pq_len(128, 64) == 2 and orc.rot_dim(128, 64) == 128
    assert orc.pq_len(100, 32) == 4 and orc.rot_dim(100, 32) == 128
    # list extents for one group of 32 rows: chunks * 512 bytes
    assert orc.list_bytes(32, 64, 8) == 4 * 512
    assert orc.list_bytes(33, 48, 8) == 2 * 3 * 512
    assert orc.list_bytes(1, 32, 8) == 2 * 512
    assert orc.list_bytes(1, 384, 4) == 12 * 512
    assert orc.list_bytes(1, 25, 5) == 512 and orc.list_bytes(1, 26, 5) == 1024   # cpc = 25
    assert orc.list_bytes(1, 21, 6) == 512 and orc.list_bytes(1, 22, 6) == 1024   # cpc = 21
    assert orc.list_bytes(1, 18, 7) == 512 and orc.list_bytes(1, 19, 7) == 1024   # cpc = 18
    assert orc.list_bytes(0, 64, 8) == 0


@pytest.mark.parametrize("pq_bits,pq_dim,n_rows", [(4, 8, 1), (4, 40, 70), (5, 8, 33), (5, 32, 64),
                                                   (6, 12, 31), (6, 44, 100), (7, 16, 32),
                                                   (7, 40, 45), (8, 3, 65), (8, 64, 96)])
def test_pack_matches_closed_form_and_round_trips(orc, pq_bits, pq_dim, n_rows):
    rng = np.random.default_rng(pq_bits * 1000 + pq_dim)
    codes = rng.integers(0, 1 << pq_bits, (n_rows, pq_dim)).astype(np.uint8)
    packed = orc.pack_list(codes, pq_bits)
    assert packed.size == orc.list_bytes(n_rows, pq_dim, pq_bits)
    for i in rng.integers(0, n_rows, 20):
        for j in range(pq_dim):
            assert closed_form_get(packed, int(i), j, pq_dim, pq_bits) == codes[i, j]
    assert np.array_equal(orc.unpack_list(packed, n_rows, pq_dim, pq_bits), codes)
    # unused high bits of every chunk stay zero
    cpc = 128 // pq_bits
    used = cpc * pq_bits
    if used < 128:
        words = packed.reshape(-1, 16)
        top = words[:, used // 8:]
        mask = np.zeros(16 - used // 8, dtype=np.uint8)
        mask[0] = (0xFF << (used % 8)) & 0xFF
        mask[1:] = 0xFF
        assert not np.any(top & mask)
    # erase and re-pack with an offset: bytes of the untouched rows survive
    if n_rows > 3:
        again = packed.copy()
        orc.pack_list(codes[2:5], pq_bits, out=again, row_offset=2)
        assert np.array_equal(again, packed)


@pytest.mark.parametrize("pq_bits,pq_dim", [(4, 8), (5, 8), (6, 12), (7, 16), (8, 20)])
def test_contiguous_unpack_is_one_bit_stream_per_row(orc, pq_bits, pq_dim):
    rng = np.random.default_rng(7 + pq_bits)
    n_rows = 50
    codes = rng.integers(0, 1 << pq_bits, (n_rows, pq_dim)).astype(np.uint8)
    packed = orc.pack_list(codes, pq_bits)
    flat = orc.unpack_list_contiguous(packed, n_rows - 3, pq_dim, pq_bits, row_offset=3)
    assert flat.shape == (n_rows - 3, (pq_dim * pq_bits + 7) // 8)
    for r in range(n_rows - 3):
        stream = int.from_bytes(bytes(flat[r]), "little")
        for j in range(pq_dim):
            assert (stream >> (j * pq_bits)) & ((1 << pq_bits) - 1) == codes[r + 3, j]


def test_committed_pack_cases(orc):
    gold = np.load(os.path.join(GOLD, "pack_cases.npz"))
    for pq_bits in (4, 5, 6, 7, 8):
        codes, want = gold[f"codes_{pq_bits}"], gold[f"list_{pq_bits}"]
        assert np.array_equal(orc.pack_list(codes, pq_bits), want)
        for i in range(codes.shape[0]):
            for j in range(codes.shape[1]):
                assert closed_form_get(want, i, j, codes.shape[1], pq_bits) == codes[i, j]
