"""The small data-movement entry points of the C ABI (2-D transpose, filter
dimension shuffle, fp32 -> storage-type convert; counterparts of
nervanagpu/float_ew.py:1325-1428) against numpy, called through the library."""
import ctypes

import numpy as np
import pytest

import oracle as orc

pytestmark = pytest.mark.gpu

vp = ctypes.c_void_p
CODES = {np.dtype(np.float16): 0, np.dtype(np.float32): 1, np.dtype(np.uint8): 2, np.dtype(np.int8): 3}


@pytest.mark.parametrize("dtype", [np.float16, np.float32, np.uint8])
@pytest.mark.parametrize("shape", [(64, 64), (1, 1), (63, 65), (200, 7), (5, 513), (130, 257)])
def test_transpose(ng, dtype, shape):
    from nervanagpu_amd import _lib
    rng = np.random.default_rng(31)
    a = rng.integers(0, 200, shape).astype(dtype)
    dA = ng.array(a, dtype=dtype)
    dO = ng.empty(shape[::-1], dtype=dtype)
    dO.fill(3)
    _lib.call("ng_transpose", CODES[np.dtype(dtype)], vp(dA.ptr), vp(dO.ptr), shape[0], shape[1], None)
    assert np.array_equal(dO.get(), orc.ref_transpose(a))


@pytest.mark.parametrize("dtype", [np.float16, np.float32])
@pytest.mark.parametrize("dims", [(64, 1, 3, 3, 64), (3, 1, 11, 11, 64), (72, 2, 3, 1, 40), (1, 1, 1, 1, 8), (130, 1, 2, 2, 67)])
def test_dimshuffle(ng, dtype, dims):
    from nervanagpu_amd import _lib
    rng = np.random.default_rng(32)
    f = rng.standard_normal(dims).astype(dtype)
    C, T, R, S, K = dims
    dF = ng.array(f, dtype=dtype)
    dO = ng.empty((K, T, R, S, C), dtype=dtype)
    dO.fill(3)
    _lib.call("ng_dimshuffle", CODES[np.dtype(dtype)], vp(dF.ptr), vp(dO.ptr), C, T * R * S, K, None)
    assert np.array_equal(dO.get(), orc.ref_dimshuffle(f))


@pytest.mark.parametrize("dtype", [np.float16, np.float32, np.uint8, np.int8])
@pytest.mark.parametrize("count", [1, 255, 256, 100003])
def test_fp32_convert(ng, dtype, count):
    """nearest-even rounding; integer targets also saturate (NaN -> 0)"""
    from nervanagpu_amd import _lib
    rng = np.random.default_rng(33)
    src = (rng.standard_normal(count) * 100).astype(np.float32)
    special = np.array([0.5, 1.5, 2.5, -0.5, -1.5, 127.5, 128.5, 254.5, 255.5, -128.5, -129.0, 300.0, -300.0,
                        np.inf, -np.inf, np.nan, 65504.0, 65520.0, 70000.0, 2.0 ** -25, 2.0 ** -24 * 1.5, 1e-8],
                       dtype=np.float32)
    n = min(count, special.size)
    src[:n] = special[:n]
    dS = ng.array(src.reshape(1, -1), dtype=np.float32)
    dD = ng.empty((1, count), dtype=dtype)
    _lib.call("ng_fp32_convert", CODES[np.dtype(dtype)], vp(dS.ptr), vp(dD.ptr), count, None)
    with np.errstate(over="ignore", invalid="ignore"):
        exp = orc.round_store(src, dtype)
    got = dD.get().reshape(-1)
    assert np.array_equal(got.view(np.uint8), np.asarray(exp).view(np.uint8))


def test_null_and_empty_arguments(ng):
    from nervanagpu_amd import _lib
    lib = _lib.load()
    assert lib.ng_transpose(0, None, None, 0, 5, None) == 0          # empty: nothing to do
    assert lib.ng_transpose(0, None, None, 4, 5, None) != 0
    assert lib.ng_dimshuffle(0, None, None, 4, 5, 8, None) != 0
    assert lib.ng_fp32_convert(0, None, None, 8, None) != 0
    assert lib.ng_fp32_convert(9, vp(1), vp(1), 8, None) != 0        # unknown dtype, nothing launched
