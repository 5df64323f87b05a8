"""Pins the oracle's scalar codecs against closed forms and numpy (no GPU).

fp_8bit<5, Signed>: cuVS cpp/src/neighbors/ivf_pq/ivf_pq_fp_8bit.cuh:31-100.  The known answers
below are derived from the formulas in that file by hand, not by calling the oracle.
"""
import json
import os

import numpy as np

GOLD = os.path.join(os.path.dirname(__file__), "golden")


def _bits(f):
    return int(np.float32(f).view(np.uint32))


def _from_bits(u):
    return float(np.uint32(u).view(np.float32))


def test_fp8_known_answers(orc):
    L = orc.lib()
    assert L.orc_fp8_encode(1.0, 0) == 0x78
    assert L.orc_fp8_decode(0x78, 0) == 1.0625
    assert _bits(L.orc_fp8_decode(0x00, 0)) == 0x38080000
    assert L.orc_fp8_decode(0x00, 0) == 2.0 ** -15 * 1.0625
    assert _bits(L.orc_fp8_decode(0xFF, 0)) == 0x47F80000
    assert L.orc_fp8_decode(0xFF, 0) == 126976.0
    # everything below 2^-15, including negatives, collapses to zero
    for v in (0.0, -1.0, 2.0 ** -16, np.nextafter(np.float32(2.0 ** -15), np.float32(0))):
        assert L.orc_fp8_encode(float(v), 0) == 0
    assert L.orc_fp8_encode(2.0 ** -15, 0) == 0
    assert L.orc_fp8_encode(float(np.nextafter(np.float32(2.0 ** -15), np.float32(1))), 0) == 0
    # saturation at 2^16 * (2 - 1/8)
    assert L.orc_fp8_encode(122880.0, 0) == 0xFF
    assert L.orc_fp8_encode(float(np.nextafter(np.float32(122880.0), np.float32(0))), 0) == 0xFE
    assert L.orc_fp8_encode(1e30, 0) == 0xFF
    # signed variant: the mantissa LSB is the sign
    assert L.orc_fp8_encode(-1.0, 1) == 0x79
    assert L.orc_fp8_decode(0x79, 1) == -1.0625
    assert L.orc_fp8_encode(1.2, 0) == 0x79
    assert L.orc_fp8_encode(1.2, 1) == 0x78
    assert L.orc_fp8_decode(0x78, 1) == 1.0625
    # half decode of the same byte
    assert L.orc_fp8_decode_half(0x78, 0) == 0x3C40
    assert L.orc_fp8_decode_half(0x79, 1) == 0xBC40


def test_fp8_encode_is_truncation_of_the_float_bits(orc):
    """For in-range v the byte is ((exponent + 15 - 127) << 3 | top 3 mantissa bits)."""
    L = orc.lib()
    rng = np.random.default_rng(0)
    vals = np.exp(rng.uniform(np.log(2.0 ** -14), np.log(1e5), 5000)).astype(np.float32)
    for v in vals:
        b = _bits(v)
        expo = (b >> 23) & 0xFF
        mant3 = (b >> 20) & 0x7
        want = ((expo - 127 + 15) << 3) | mant3
        assert L.orc_fp8_encode(float(v), 0) == want


def test_fp8_decode_table_and_round_trip(orc):
    L = orc.lib()
    table = [L.orc_fp8_decode(u, 0) for u in range(256)]
    assert all(b > a for a, b in zip(table, table[1:])), "decode must be strictly increasing"
    for u in range(256):
        # closed form: 2^(e-15) * (1 + (m + 0.5) / 8) with e = u >> 3, m = u & 7
        e, m = u >> 3, u & 7
        want = 2.0 ** (e - 15) * (1.0 + (m + 0.5) / 8.0)
        if e == 0:
            # exponent field 0 of the fp32 pattern 0x38080000 is still a normal number
            want = 2.0 ** -15 * (1.0 + (m + 0.5) / 8.0)
        assert table[u] == want
        assert L.orc_fp8_encode(table[u], 0) == u
        hb = L.orc_fp8_decode_half(u, 0)
        assert hb == 0x0040 + (u << 7)
        if 1 <= e <= 30:
            # inside the binary16 normal range both decodes give the same number; exponent
            # field 0 lands on binary16 subnormals and field 31 on the inf/NaN patterns
            assert float(np.uint16(hb).view(np.float16)) == want
    rng = np.random.default_rng(1)
    vals = np.exp(rng.uniform(np.log(2.0 ** -14), np.log(1e5), 5000)).astype(np.float32)
    for v in vals:
        d = L.orc_fp8_decode(L.orc_fp8_encode(float(v), 0), 0)
        assert v * (1 - 1 / 16) <= d <= v * (1 + 1 / 16)
    # signed: decode ignores the LSB for the magnitude
    for u in range(256):
        want = table[u & 0xFE] * (-1.0 if u & 1 else 1.0)
        assert L.orc_fp8_decode(u, 1) == want


def test_fp8_matches_committed_table(orc):
    with open(os.path.join(GOLD, "fp8_tables.json")) as f:
        gold = json.load(f)
    L = orc.lib()
    assert [_bits(L.orc_fp8_decode(u, 0)) for u in range(256)] == gold["decode_unsigned_bits"]
    assert [_bits(L.orc_fp8_decode(u, 1)) for u in range(256)] == gold["decode_signed_bits"]
    assert [L.orc_fp8_decode_half(u, 0) for u in range(256)] == gold["decode_half_unsigned_bits"]
    for bits, want_u, want_s in gold["encode_cases"]:
        v = _from_bits(bits)
        assert L.orc_fp8_encode(v, 0) == want_u
        assert L.orc_fp8_encode(v, 1) == want_s


def test_half_conversions_against_numpy(orc):
    L = orc.lib()
    # every binary16 pattern widens exactly like numpy
    allh = np.arange(65536, dtype=np.uint16)
    ref = allh.view(np.float16).astype(np.float32)
    for u in range(0, 65536, 7):
        got = L.orc_half_to_float(u)
        if np.isnan(ref[u]):
            assert np.isnan(got)
        else:
            assert got == ref[u]
    # float -> half is round-to-nearest-even like numpy, including subnormals, ties and overflow
    rng = np.random.default_rng(2)
    vals = np.concatenate([
        rng.standard_normal(4000).astype(np.float32) * 100,
        np.exp(rng.uniform(np.log(1e-9), np.log(1e6), 4000)).astype(np.float32),
        np.array([0.0, -0.0, 65504.0, 65519.99, 65520.0, 65536.0, 1e10, 2.0 ** -24, 2.0 ** -25,
                  2.0 ** -25 * 1.0001, 2.0 ** -14, 6.1e-5, 1.0009765625, 1.00048828125,
                  1.00146484375], dtype=np.float32)])
    # exact ties between two halves
    h = rng.integers(0, 0x7BFF, 2000).astype(np.uint16)
    lo = h.view(np.float16).astype(np.float32)
    hi = (h + 1).astype(np.uint16).view(np.float16).astype(np.float32)
    vals = np.concatenate([vals, (lo + hi) / 2, -(lo + hi) / 2])
    with np.errstate(over="ignore"):
        want = vals.astype(np.float16).view(np.uint16)
    for v, w in zip(vals, want):
        assert L.orc_float_to_half(float(v)) == int(w), (v, hex(int(w)))


def test_half_add_against_numpy(orc):
    L = orc.lib()
    rng = np.random.default_rng(3)
    a = rng.integers(0, 0x7C00, 4000).astype(np.uint16)
    b = rng.integers(0, 0x7C00, 4000).astype(np.uint16)
    sign = rng.integers(0, 2, 4000).astype(np.uint16) << 15
    b = b | sign
    with np.errstate(over="ignore"):
        want = (a.view(np.float16) + b.view(np.float16)).view(np.uint16)
        # numpy adds halves in float32 and rounds once; cross-check with float64 as well
        want64 = (a.view(np.float16).astype(np.float64) + b.view(np.float16).astype(np.float64)
                  ).astype(np.float16).view(np.uint16)
    assert np.array_equal(want, want64)
    for x, y, w in zip(a, b, want):
        assert L.orc_half_add(int(x), int(y)) == int(w)
