"""Max / average pooling fprop and bprop on the GPU against the numpy oracle
(gather + np.max/np.argmax/np.mean of benchmarks/pool_test.py:71-146)."""
import numpy as np
import pytest

import oracle as orc
from util import assert_fp16_within_ulp

pytestmark = pytest.mark.gpu

# N, C, D, H, W, J, T, R, S, pad(j,d,h,w), stride(j,d,h,w)
CASES = [
    (32, 32, 1, 32, 32, 2, 1, 3, 3, (0, 0, 0, 0), (2, 1, 2, 2)),     # benchmarks/pool_test.py:31-37
    (64, 16, 1, 16, 16, 1, 1, 2, 2, (0, 0, 0, 0), (1, 1, 2, 2)),     # non-overlapping, tiles exactly
    (16, 8, 1, 15, 15, 1, 1, 2, 2, (0, 0, 0, 0), (1, 1, 2, 2)),      # ragged edge
    (8, 12, 1, 13, 13, 1, 1, 3, 3, (0, 0, 1, 1), (1, 1, 2, 2)),      # padded, overlapping
    (8, 6, 4, 9, 7, 1, 2, 3, 2, (0, 1, 1, 0), (1, 1, 2, 1)),         # 3-D window
    (24, 9, 1, 6, 6, 3, 1, 1, 1, (0, 0, 0, 0), (3, 1, 1, 1)),        # maxout over feature maps only
    (12, 5, 1, 9, 9, 1, 1, 3, 3, (0, 0, 0, 0), (1, 1, 4, 4)),        # stride > window: uncovered inputs
    (4, 4, 1, 8, 8, 1, 1, 3, 3, (0, 0, 0, 0), (1, 1, 1, 1)),         # N not a multiple of 8 (scalar path)
    (16, 3, 2, 12, 10, 1, 1, 3, 3, (0, 0, 0, 0), (1, 1, 2, 2)),      # 3x3/2 on even extents: last row / column uncovered
    (8, 4, 1, 7, 9, 1, 1, 3, 3, (0, 0, 1, 1), (1, 1, 2, 2)),         # 3x3/2 padded, odd non-square extents
    (4, 5, 1, 9, 11, 1, 1, 3, 3, (0, 0, 0, 1), (1, 1, 2, 2)),        # 3x3/2, four images: vector path only in fp32
    (16, 6, 1, 10, 9, 1, 1, 3, 3, (0, 0, 1, 1), (1, 1, 1, 1)),       # 3x3/1 padded (inception pooling branch), vector path
    (8, 10, 1, 5, 5, 3, 1, 1, 1, (1, 0, 0, 0), (2, 1, 1, 1)),        # overlapping, padded windows over feature maps
    (8, 4, 7, 6, 6, 1, 3, 2, 2, (0, 1, 0, 0), (1, 2, 2, 2)),         # overlapping in depth only
    (8, 3, 1, 9, 8, 1, 1, 2, 2, (0, 0, 0, 0), (1, 1, 1, 1)),         # 2x2/1: overlapping, no compiled cell shape
    # feature maps in multiples of 8 and several workgroups of cells per map: the backward kernel numbers its
    # workgroups so that an XCD takes whole maps
    (64, 16, 1, 13, 13, 1, 1, 3, 3, (0, 0, 0, 0), (1, 1, 2, 2)),     # 3x3/2, two workgroups per map
    (32, 24, 1, 20, 18, 1, 1, 3, 3, (0, 0, 1, 1), (1, 1, 2, 2)),     # 3x3/2 padded, 24 maps
    (32, 8, 1, 10, 9, 1, 1, 3, 3, (0, 0, 1, 1), (1, 1, 1, 1)),       # 3x3/1 padded
]


def _layer(ng, dtype, op, case):
    N, C, D, H, W, J, T, R, S, pad, strd = case
    return ng.pool_layer(dtype, op, N, C, D, H, W, J, T, R, S, pad[0], pad[1], pad[2], pad[3],
                         strd[0], strd[1], strd[2], strd[3])


@pytest.mark.parametrize("dtype", [np.float16, np.float32])
@pytest.mark.parametrize("op", ["max", "avg"])
@pytest.mark.parametrize("case", CASES)
def test_pool_full_compare(ng, dtype, op, case):
    layer = _layer(ng, dtype, op, case)
    rng = np.random.default_rng(7)
    I = rng.uniform(0, 1, layer.dimI).astype(np.float16).astype(dtype)
    E = rng.uniform(-1, 1, layer.dimO).astype(np.float16).astype(dtype)
    dI, dE = ng.array(I, dtype=dtype), ng.array(E, dtype=dtype)
    dO = ng.empty(layer.dimO, dtype=dtype)
    dB = ng.empty(layer.dimI, dtype=dtype)
    dB.fill(9)
    ng.fprop_pool(layer, dI, dO)
    ng.bprop_pool(layer, dI, dE, dB)
    refO = orc.ref_pool_fprop(I, op, layer.JTRS, layer.padding, layer.strides)
    refB = orc.ref_pool_bprop(I, E, op, layer.JTRS, layer.padding, layer.strides)
    if op == "max":
        assert np.array_equal(dO.get(), refO.astype(dtype))          # max is exact
    elif dtype == np.float16:
        assert_fp16_within_ulp(dO.get(), refO, 1.0, "avg fprop", 1e-6)
    else:
        np.testing.assert_allclose(dO.get(), refO, rtol=1e-5, atol=1e-6)
    if dtype == np.float16:
        assert_fp16_within_ulp(dB.get(), refB, 1.0, "%s bprop" % op, 1e-6)
    else:
        np.testing.assert_allclose(dB.get(), refB, rtol=1e-5, atol=1e-6)


def test_max_pool_ties_and_out_of_bounds(ng):
    """first maximum in (j,t,r,s) scan order wins (kernels/sass/hpool_max.sass:264-282)"""
    layer = ng.pool_layer(np.float16, "max", 8, 4, 1, 6, 6, 1, 1, 3, 3, 0, 0, 1, 1, 1, 1, 1, 1)
    I = np.ones(layer.dimI, np.float16)          # every window is all ties
    E = np.full(layer.dimO, 1.0, np.float16)
    dB = ng.empty(layer.dimI)
    ng.bprop_pool(layer, ng.array(I), ng.array(E), dB)
    ref = orc.ref_pool_bprop(I, E, "max", layer.JTRS, layer.padding, layer.strides)
    assert np.array_equal(dB.get(), ref.astype(np.float16))


@pytest.mark.parametrize("dtype", [np.float16, np.float32])
def test_max_pool_negative_inputs_padding_and_signed_zero_ties(ng, dtype):
    """padding never wins a window (all inputs negative), and among +0 / -0 ties the
    first element in scan order receives the error (numeric, not bitwise, equality)"""
    rng = np.random.default_rng(12)
    for (N, C, H, W, R, pad, strd) in ((16, 6, 9, 10, 3, 1, 2), (16, 4, 8, 8, 2, 1, 2), (8, 5, 7, 7, 3, 1, 1)):
        layer = ng.pool_layer(dtype, "max", N, C, 1, H, W, 1, 1, R, R, 0, 0, pad, pad, 1, 1, strd, strd)
        I = rng.uniform(-2, -1, layer.dimI).astype(dtype)
        E = rng.uniform(-1, 1, layer.dimO).astype(dtype)
        for variant in ("negative", "zeros"):
            if variant == "zeros":
                # non-positive data with many exact zeros of both signs: windows tie on zero
                I = np.where(rng.random(layer.dimI) < 0.5, 0.0, I).astype(dtype)
                I[(I == 0) & (rng.random(layer.dimI) < 0.5)] = -0.0
                assert np.signbit(I[I == 0]).any() and (~np.signbit(I[I == 0])).any()
            dI, dE = ng.array(I, dtype=dtype), ng.array(E, dtype=dtype)
            dO, dB = ng.empty(layer.dimO, dtype=dtype), ng.empty(layer.dimI, dtype=dtype)
            ng.fprop_pool(layer, dI, dO)
            ng.bprop_pool(layer, dI, dE, dB)
            refO = orc.ref_pool_fprop(I, "max", layer.JTRS, layer.padding, layer.strides)
            refB = orc.ref_pool_bprop(I, E, "max", layer.JTRS, layer.padding, layer.strides)
            assert np.array_equal(dO.get(), refO.astype(dtype)), variant
            if dtype == np.float16:
                assert_fp16_within_ulp(dB.get(), refB, 1.0, "max bprop " + variant, 1e-6)
            else:
                np.testing.assert_allclose(dB.get(), refB, rtol=1e-5, atol=1e-6)


@pytest.mark.parametrize("dtype", [np.float16, np.float32])
@pytest.mark.parametrize("geom", [(2, 2, 2, 2), (3, 3, 3, 2), (2, 3, 3, 1), (3, 3, 4, 3)])
def test_max_pool_window_wholly_outside_the_image(ng, dtype, geom):
    """A window that lies in the padding only: the reference's scan starts at
    -FLT_MAX and finds nothing larger (kernels/sass/hpool_max.sass:218-219), so the
    output is -FLT_MAX in fp32 and -inf once narrowed to fp16, on the compiled
    2x2 / 3x3 window shapes and on the generic loop alike; the error of such a
    window goes nowhere."""
    R, S, pad, strd = geom
    layer = ng.pool_layer(dtype, "max", 8, 3, 1, 7, 7, 1, 1, R, S, 0, 0, pad, pad, 1, 1, strd, strd)
    rng = np.random.default_rng(13)
    I = rng.uniform(-1, 1, layer.dimI).astype(dtype)
    E = rng.uniform(0.5, 1, layer.dimO).astype(dtype)
    dI, dE = ng.array(I, dtype=dtype), ng.array(E, dtype=dtype)
    dO, dB = ng.empty(layer.dimO, dtype=dtype), ng.empty(layer.dimI, dtype=dtype)
    ng.fprop_pool(layer, dI, dO)
    ng.bprop_pool(layer, dI, dE, dB)
    refO = orc.ref_pool_fprop(I, "max", layer.JTRS, layer.padding, layer.strides)
    assert (refO == np.finfo(np.float32).min).any(), "geometry was meant to have windows in the padding only"
    got = dO.get()
    with np.errstate(over="ignore"):
        exp = refO.astype(dtype)
    assert np.array_equal(got, exp)
    outside = refO == np.finfo(np.float32).min
    assert np.all(got[outside] == (-np.inf if dtype == np.float16 else np.finfo(np.float32).min))
    refB = orc.ref_pool_bprop(I, E, "max", layer.JTRS, layer.padding, layer.strides)
    if dtype == np.float16:
        assert_fp16_within_ulp(dB.get(), refB, 1.0, "max bprop", 1e-6)
    else:
        np.testing.assert_allclose(dB.get(), refB, rtol=1e-5, atol=1e-6)


def test_config4_vgg_pool_shapes(ng):
    """2x2/2 max pooling at the five block ends of config 4, full shapes, every
    element: the forward result against a reshape + max, and the structure of
    the backward result (each window passes its error to exactly one element)"""
    rng = np.random.default_rng(3)
    for C, HW in ((64, 224), (128, 112), (256, 56), (512, 28), (512, 14)):
        layer = ng.pool_layer(np.float16, "max", 64, C, 1, HW, HW, 1, 1, 2, 2)
        I = rng.standard_normal(layer.dimI, dtype=np.float32).astype(np.float16)
        E = rng.standard_normal(layer.dimO, dtype=np.float32).astype(np.float16)
        dI, dE = ng.array(I), ng.array(E)
        dO, dB = ng.empty(layer.dimO), ng.empty(layer.dimI)
        ng.fprop_pool(layer, dI, dO)
        ng.bprop_pool(layer, dI, dE, dB)
        ref = I.astype(np.float32).reshape(C, 1, HW // 2, 2, HW // 2, 2, 64).max(axis=(3, 5))
        assert np.array_equal(dO.get(), ref.astype(np.float16))
        del ref
        B = dB.get().astype(np.float32)
        # each window passes its error to exactly one element: the first maximum
        assert np.array_equal(B.reshape(C, 1, HW // 2, 2, HW // 2, 2, 64).sum(axis=(3, 5)), E.astype(np.float32))
        assert np.count_nonzero(B) <= E.size
        If = I.astype(np.float32)
        at_max = If == np.repeat(np.repeat(dO.get().astype(np.float32), 2, axis=2), 2, axis=3)
        assert not np.any(B[~at_max])            # nothing lands on an element that is not a maximum
        del B, If, at_max


def test_config5_pool_sampled(ng):
    """3x3/2 on C=256, 56x56, N=128: sampled windows / pixels vs the oracle"""
    rng = np.random.default_rng(4)
    for op in ("max", "avg"):
        layer = ng.pool_layer(np.float16, op, 128, 256, 1, 56, 56, 1, 1, 3, 3, 0, 0, 0, 0, 1, 1, 2, 2)
        assert layer.MPQ == (1, 27, 27)
        I = rng.uniform(0, 1, layer.dimI).astype(np.float16)
        E = rng.uniform(-1, 1, layer.dimO).astype(np.float16)
        dI, dE = ng.array(I), ng.array(E)
        dO, dB = ng.empty(layer.dimO), ng.empty(layer.dimI)
        ng.fprop_pool(layer, dI, dO)
        ng.bprop_pool(layer, dI, dE, dB)
        O = dO.get()
        wins = [(int(rng.integers(256)), 0, int(rng.integers(27)), int(rng.integers(27))) for _ in range(256)]
        wins += [(int(rng.integers(256)), 0, e, int(rng.integers(27))) for e in (0, 26) for _ in range(8)]
        wins += [(int(rng.integers(256)), 0, int(rng.integers(27)), e) for e in (0, 26) for _ in range(8)]
        wins += [(0, 0, 0, 0), (255, 0, 26, 26), (7, 0, 0, 26), (9, 0, 26, 0)]
        ref = orc.ref_pool_fprop_pixels(I, op, layer.JTRS, wins, layer.padding, layer.strides)
        got = np.stack([O[w] for w in wins])
        assert_fp16_within_ulp(got, ref, 1.0 if op == "avg" else 0.0, "%s fprop" % op, 1e-7 if op == "avg" else 0.0)
        # bprop: compare whole channels against the oracle run on those channels only
        B = dB.get()
        for c in (0, 131, 255):
            refB = orc.ref_pool_bprop(I[c:c + 1], E[c:c + 1], op, layer.JTRS, layer.padding, layer.strides)
            assert_fp16_within_ulp(B[c:c + 1], refB, 1.0, "%s bprop" % op, 1e-6)


@pytest.mark.parametrize("dtype", [np.float16, np.float32])
@pytest.mark.parametrize("case", CASES)
def test_l2_pool_fprop(ng, dtype, case):
    """l2 pooling (named at nervanagpu/nervanagpu.py:746, defined at benchmarks/pool_test.py:145-146):
    the square root of the sum of squares over the window, slots outside the tensor counting as zero;
    every geometry of the max / avg cases (unrolled 2x2 and 3x3 windows, generic loops, padding,
    feature-map windows, the scalar path).  The reference defines no derivative: bprop refuses."""
    layer = _layer(ng, dtype, "l2", case)
    rng = np.random.default_rng(17)
    I = rng.uniform(-1, 1, layer.dimI).astype(np.float16).astype(dtype)
    dO = ng.empty(layer.dimO, dtype=dtype)
    dO.fill(9)
    ng.fprop_pool(layer, ng.array(I, dtype=dtype), dO)
    ref = orc.ref_pool_fprop(I, "l2", layer.JTRS, layer.padding, layer.strides)
    if dtype == np.float16:
        assert_fp16_within_ulp(dO.get(), ref, 1.0, "l2 fprop", 1e-6)
    else:
        np.testing.assert_allclose(dO.get(), ref, rtol=1e-5, atol=1e-6)
    with pytest.raises(ValueError):
        ng.bprop_pool(layer, ng.empty(layer.dimI, dtype=dtype), ng.empty(layer.dimO, dtype=dtype),
                      ng.empty(layer.dimI, dtype=dtype))


def test_pool_errors(ng):
    layer = ng.pool_layer(np.float16, "median", 8, 4, 1, 6, 6, 1, 1, 2, 2)
    with pytest.raises(ValueError):
        ng.fprop_pool(layer, ng.empty(layer.dimI), ng.empty(layer.dimO))
    ok = ng.pool_layer(np.float16, "max", 8, 4, 1, 6, 6, 1, 1, 2, 2)
    with pytest.raises(AssertionError):
        ng.fprop_pool(ok, ng.empty(layer.dimI), ng.empty((4, 1, 3, 3, 16)))
    with pytest.raises(AssertionError):
        ng.bprop_pool(ok, ng.empty(ok.dimI), ng.empty(ok.dimO), ng.empty(ok.dimI, dtype=np.float32))


@pytest.mark.parametrize("dtype", [np.float16, np.float32])
def test_max_pool_bprop_with_rectifier_mask(ng, dtype):
    """bprop_pool(..., relu_mask=True) = bprop_pool followed by the reference's
    relu derivative step `grad *= I > 0` (nervanagpu/layers.py:89-91), on every
    backward path: exact tiling 2x2 and 3x3, generic exact tiling, overlapping
    3x3/2 by cells, overlapping with padding, feature-map pooling, N = 4 lanes."""
    rng = np.random.default_rng(23)
    cases = [  # N, C, D, H, W, J, T, R, S, pads (j,d,h,w), strides (j,d,h,w)
        (16, 6, 1, 8, 8, 1, 1, 2, 2, (0, 0, 0, 0), (1, 1, 2, 2)),
        (16, 4, 1, 9, 9, 1, 1, 3, 3, (0, 0, 0, 0), (1, 1, 3, 3)),
        (8, 4, 2, 8, 6, 1, 2, 2, 3, (0, 0, 0, 0), (1, 2, 2, 3)),
        (16, 5, 1, 13, 13, 1, 1, 3, 3, (0, 0, 0, 0), (1, 1, 2, 2)),
        (16, 3, 1, 12, 10, 1, 1, 3, 3, (0, 0, 1, 1), (1, 1, 2, 2)),
        (8, 6, 1, 7, 7, 2, 1, 3, 3, (0, 0, 1, 1), (2, 1, 1, 1)),
        (4, 3, 1, 9, 9, 1, 1, 3, 3, (0, 0, 0, 0), (1, 1, 2, 2)),
    ]
    for (N, C, D, H, W, J, T, R, S, pads, strides) in cases:
        layer = ng.pool_layer(dtype, "max", N, C, D, H, W, J, T, R, S, *pads, *strides)
        # about half of the inputs are zero (a rectifier's output), some windows entirely
        x = np.maximum(rng.standard_normal(layer.dimI), 0).astype(dtype)
        x[:, :, : H // 3, : W // 3, :] = 0
        e = rng.uniform(-1, 1, layer.dimO).astype(dtype)
        dI, dE = ng.array(x, dtype=dtype), ng.array(e, dtype=dtype)
        plain, masked = ng.empty(layer.dimI, dtype=dtype), ng.empty(layer.dimI, dtype=dtype)
        ng.bprop_pool(layer, dI, dE, plain)
        ng.bprop_pool(layer, dI, dE, masked, relu_mask=True)
        want = plain.get() * (x > 0)
        assert np.array_equal(masked.get(), want), (N, C, D, H, W, J, T, R, S)
        ref = orc.ref_pool_bprop(x.astype(np.float32), e.astype(np.float32), "max", layer.JTRS, layer.padding,
                                 layer.strides) * (x > 0)
        assert np.allclose(masked.get().astype(np.float32), ref.astype(dtype).astype(np.float32), rtol=2e-3, atol=1e-6)
        # inputs that are not a rectifier's output: the mask is still (I > 0)
        x2 = rng.standard_normal(layer.dimI).astype(dtype)
        dI.set(x2)
        ng.bprop_pool(layer, dI, dE, plain)
        ng.bprop_pool(layer, dI, dE, masked, relu_mask=True)
        assert np.array_equal(masked.get(), plain.get() * (x2 > 0))
    avg = ng.pool_layer(np.float16, "avg", 16, 4, 1, 8, 8, 1, 1, 2, 2)
    A, E, B = ng.empty(avg.dimI), ng.empty(avg.dimO), ng.empty(avg.dimI)
    with pytest.raises(Exception):
        ng.bprop_pool(avg, A, E, B, relu_mask=True)
