"""Pins the oracle's rounding / RNG / integer helpers against what the
mathematics fixes (no GPU needed)."""
import json
import os

import numpy as np
import pytest

import oracle as orc
from oracle import ref_numpy as rn

HERE = os.path.dirname(os.path.abspath(__file__))


def test_f16_rz_exact_values_round_trip():
    # every finite fp16 value is exactly representable in fp32: RZ must be identity
    h = np.arange(0, 1 << 16, dtype=np.uint16)
    f = h.view(np.float16)
    finite = np.isfinite(f)
    got = orc.f32_to_f16_rz(f.astype(np.float32))
    assert np.array_equal(got[finite], h[finite])
    inf = np.isinf(f)
    assert np.array_equal(got[inf], h[inf])


def test_f16_rz_truncates_toward_zero():
    rng = np.random.default_rng(0)
    x = np.concatenate([
        rng.uniform(-70000, 70000, 200000),
        rng.uniform(-1e-4, 1e-4, 200000),
        rng.uniform(-1e-7, 1e-7, 100000),
        [65504.0, 65519.9, 65520.0, 65535.9, 65536.0, 1e30, -1e30, 2.0 ** -24, 2.0 ** -25,
         0.99 * 2.0 ** -24, 0.0, -0.0],
    ]).astype(np.float32)
    got = orc.f32_to_f16_rz(x).view(np.float16).astype(np.float64)
    xd = x.astype(np.float64)
    # never larger in magnitude, same sign, and within one fp16 step below
    assert np.all(np.abs(got) <= np.abs(xd))
    assert np.all((np.signbit(got) == np.signbit(x)))
    rn = x.astype(np.float16)
    # nearest and toward-zero differ by at most one fp16 ulp
    up = np.nextafter(got.astype(np.float16), np.float16(np.inf) * np.sign(x).astype(np.float16))
    clipped = np.abs(xd) >= 65520
    ok = (rn.astype(np.float64) == got) | (rn == up) | clipped
    assert ok.all()
    assert np.all(np.abs(got[clipped]) == 65504.0)


def test_round_int_is_half_even_and_saturating():
    x = np.array([0.5, 1.5, 2.5, -0.5, -1.5, 126.5, 127.5, 300.0, -300.0, 254.5, 255.5], dtype=np.float32)
    assert orc.round_int(x, np.int8).tolist() == [0, 2, 2, 0, -2, 126, 127, 127, -128, 127, 127]
    assert orc.round_int(x, np.uint8).tolist() == [0, 2, 2, 0, 0, 126, 128, 255, 0, 254, 255]


def test_rand32_is_a_bijection_of_idx_and_stream_sensitive():
    idx = np.arange(1 << 16, dtype=np.uint32)
    a = orc.rand32(1234, 7, idx)
    assert np.unique(a).size == idx.size
    b = orc.rand32(1234, 8, idx)
    c = orc.rand32(1235, 7, idx)
    assert (a != b).mean() > 0.99 and (a != c).mean() > 0.99
    # top bits roughly uniform
    assert abs((a >> 31).mean() - 0.5) < 0.01


def test_rand32_golden_vectors():
    with open(os.path.join(HERE, "golden", "rand32.json")) as f:
        g = json.load(f)
    for case in g["cases"]:
        got = orc.rand32(case["seed"], case["stream"], np.array(case["idx"], dtype=np.uint32))
        assert got.tolist() == case["out"]


@pytest.mark.parametrize("bits", [1, 4, 10])
def test_sr_fp16_invariants(bits):
    rng = np.random.default_rng(bits)
    x = rng.uniform(-4, 4, 50000).astype(np.float32)
    r = rng.integers(0, 2 ** 32, x.size, dtype=np.uint64).astype(np.uint32)
    got = orc.round_stochastic_fp16(x, bits, r).astype(np.float64)
    # bracket: truncation at `bits` <= |got| <= truncation + one unit
    e = np.floor(np.log2(np.abs(x.astype(np.float64))))
    unit = 2.0 ** (e - bits)
    lo = np.floor(np.abs(x.astype(np.float64)) / unit) * unit
    assert np.all(np.abs(got) >= lo - 1e-12)
    assert np.all(np.abs(got) <= lo + unit + 1e-12)
    assert np.all(np.sign(got) == np.sign(x))
    # r == 0 -> plain truncation; r == max -> rounds up unless exact
    t = orc.round_stochastic_fp16(x, bits, np.zeros_like(r)).astype(np.float64)
    assert np.array_equal(np.abs(t), lo)
    # exactly representable values pass through for any r
    xe = (np.round(x * 4) / 4).astype(np.float32) if bits >= 4 else np.sign(x).astype(np.float32)
    assert np.array_equal(orc.round_stochastic_fp16(xe, bits, r).astype(np.float32), xe)


def test_sr_fp16_is_unbiased():
    # E[result] == v over a uniform sweep of r
    v = np.float32(1.0 + 3.0 / 4096 + 1.0 / 16384)   # needs 14 mantissa bits
    r = (np.arange(1 << 16, dtype=np.uint64) << 16).astype(np.uint32)
    got = orc.round_stochastic_fp16(np.full(r.size, v, np.float32), 10, r).astype(np.float64)
    assert abs(got.mean() - float(v)) < 1e-7
    assert set(np.unique(got)) == {1.0, 1.0 + 2.0 ** -10}


def test_sr_fp32_masks_and_saturates():
    x = np.array([1.0000001, -3.14159, 3.3e38, np.inf, -np.inf], dtype=np.float32)
    r = np.full(x.size, 0xFFFFFFFF, dtype=np.uint32)
    got = orc.round_stochastic_fp32(x, 15, r)
    assert np.all((got.view(np.uint32)[:3] & 0xFF) == 0)
    assert np.isfinite(got[2]) and np.isinf(got[3]) and np.isinf(got[4])
    assert abs(got[1]) >= abs(x[1])


def test_round_store_dispatch():
    x = np.array([0.1, 1000.7, -2.5], dtype=np.float32)
    assert orc.round_store(x, np.float16).dtype == np.float16
    assert orc.round_store(x, np.float32) is not None
    assert orc.round_store(x, np.int8).tolist() == [0, 127, -2]


@pytest.mark.parametrize("d", [1, 2, 3, 5, 7, 9, 11, 27, 121, 363])
def test_magic32_exhaustive(d):
    nmax = 65535
    m, s = orc.magic32(nmax, d)
    n = np.arange(nmax + 1, dtype=np.uint64)
    assert np.array_equal(n // d, (n * m) >> s)
    assert nmax * m < 2 ** 64


def test_tile_heuristic_matches_both_reference_statements():
    # spot values worked by hand from the decision tree
    assert orc.gemm_tile_heuristic("nn", 4096, 128, 256) == "128x128"
    assert orc.gemm_tile_heuristic("nn", 4096, 32, 256) == "128x32"
    assert orc.gemm_tile_heuristic("tn", 32, 4096, 256) == "128x128"
    assert orc.gemm_tile_heuristic("nn", 60, 4096, 24) == "32x128"


def test_fast_ew_dims():
    assert orc.fast_ew_dims(1024 * 1024)[0] == (4096, 256)
    assert orc.fast_ew_dims(96)[0] == (1, 96)
    shp, strd = orc.fast_ew_dims(7 * 13)
    assert shp[0] * shp[1] == 91 and strd == (shp[1], 1)


def test_sr10_short_form_is_the_same_function():
    """The device rounds at the default 10 bits with a shorter expression
    (ng_sr10_bump in csrc/ng_device_common.h): no mask, the increment added to
    the signed pattern as it is, and values whose magnitude lies within 2^13
    patterns of the largest finite fp32 (or beyond: infinities, NaNs) passed on
    unchanged instead of clamp + infinity test.  It must be the oracle's
    function bit for bit, NaN payloads included."""
    U = np.uint32

    def short_form(x, r):
        x = np.ascontiguousarray(x, dtype=np.float32)
        u = x.view(np.uint32)
        with np.errstate(over="ignore", invalid="ignore"):
            bumped = (u + (r >> U(19))).astype(np.uint32)
            keep = np.abs(x) < np.array([0x7F7FE000], dtype=np.uint32).view(np.float32)[0]
        return rn.f32_to_f16_rz(np.where(keep, bumped, u).astype(np.uint32).view(np.float32))

    rng = np.random.default_rng(3)
    for case in range(4):
        bits = rng.integers(0, 2 ** 32, 500_000, dtype=np.uint64).astype(np.uint32)
        if case == 1:    # exponents around the fp16 range, subnormal results included
            bits = (bits & U(0x807FFFFF)) | (rng.integers(100, 146, bits.size).astype(np.uint32) << U(23))
        if case == 2:    # around the largest finite fp32, infinities and NaNs
            bits = (bits & U(0x8000FFFF)) | U(0x7F7F0000) | ((bits >> U(3)) & U(0x00810000))
        r = rng.integers(0, 2 ** 32, bits.size, dtype=np.uint64).astype(np.uint32)
        if case == 3:
            r |= U(0xFFF80000)
        ref = orc.round_stochastic_fp16(bits.view(np.float32), 10, r).view(np.uint16)
        assert np.array_equal(ref, short_form(bits.view(np.float32), r).view(np.uint16))
    sp = np.array([0x7F800000, 0xFF800000, 0x7FC00000, 0xFFFFFFFF, 0x7FFFFFFF, 0x7F7FFFFF, 0xFF7FFFFF, 0x7F7FE000,
                   0x7F7FE001, 0x477FE000, 0x477FDFFF, 0x477FFFFF, 0x47800000, 0, 0x80000000, 1, 0x33800000,
                   0x337FFFFF, 0x38800000, 0x387FFFFF], dtype=np.uint32)
    for rv in (0, 0xFFFFFFFF, 0x80000000, 0x0007FFFF, 0xFFF80000):
        r = np.full(sp.shape, rv, dtype=np.uint32)
        assert np.array_equal(orc.round_stochastic_fp16(sp.view(np.float32), 10, r).view(np.uint16),
                              short_form(sp.view(np.float32), r).view(np.uint16))
