"""Shared helpers of the parity tests."""
import numpy as np


def fp16_ulp(ref):
    """size of one fp16 unit in the last place at |ref| (float64 array)"""
    a = np.abs(np.asarray(ref, dtype=np.float64))
    a16 = np.minimum(a, 65504.0).astype(np.float16)
    return np.spacing(a16).astype(np.float64)


EPS32 = 2.0 ** -24


def acc_atol(absdot):
    """bound on the fp32 accumulation error of a dot product whose absolute
    terms sum to `absdot`: it only matters where the result cancels to ~0"""
    return 4.0 * EPS32 * np.asarray(absdot, dtype=np.float64)


def assert_fp16_within_ulp(out, ref32, ulps=1.0, what="", atol=0.0):
    """fp16 result within `ulps` fp16 units of the fp32-accumulated reference
    (plus `atol`, the accumulation error of the fp32 value itself)"""
    out = np.asarray(out)
    assert out.dtype == np.float16, out.dtype
    ref = np.asarray(ref32, dtype=np.float64)
    assert out.shape == ref.shape, (out.shape, ref.shape)
    o = out.astype(np.float64)
    # beyond the fp16 range nearest rounding gives infinity (from 65520 on; the
    # band between the largest fp16 value and that threshold may go either way
    # within the accumulation error and is left out)
    over = np.isfinite(ref) & (np.abs(ref) > 65520.0 * (1.0 + 1e-3))
    if over.any():
        assert np.all(np.isinf(o[over]) & (np.sign(o[over]) == np.sign(ref[over]))), \
            "%s: values beyond the fp16 range must round to infinity" % what
    fin = np.isfinite(ref) & (np.abs(ref) < 65504.0)
    err = np.abs(o[fin] - ref[fin])
    atol = np.broadcast_to(np.asarray(atol, dtype=np.float64), ref.shape)[fin]
    tol = ulps * fp16_ulp(ref[fin]) * (1.0 + 1e-6) + atol
    bad = err > tol
    if bad.any():
        i = np.argmax(err / tol)
        raise AssertionError("%s: %d of %d elements off by more than %g fp16 ulp (worst: got %r ref %r)"
                             % (what, bad.sum(), bad.size, ulps, o[fin][i], ref[fin][i]))


def assert_fp32_close(out, ref32, rel=1e-5, what=""):
    """max|d| / mean|ref| <= rel (metric form of benchmarks/cublas_test.py:169-171)"""
    out = np.asarray(out, dtype=np.float64)
    ref = np.asarray(ref32, dtype=np.float64)
    assert out.shape == ref.shape, (out.shape, ref.shape)
    nz = ref != 0          # exact zeros (e.g. produced by relu) do not dilute the scale
    scale = max(np.abs(ref[nz]).mean() if nz.any() else 0.0, 1e-30)
    err = np.abs(out - ref).max() / scale
    assert err <= rel, "%s: max|d|/mean|ref| = %.3g > %.3g" % (what, err, rel)


def assert_fp32_sum_close(out, ref64, abs_sum, nterms, what=""):
    """fp32 result of a sum of `nterms` products against its float64 value.

    Rounding in an fp32 accumulation chain moves a sum of n terms by at most
    n * 2^-24 * sum|a_i b_i| whatever the order of the additions, and by about
    sqrt(n) * 2^-24 * sum|a_i b_i| when the rounding errors are independent
    (Higham & Mary 2019, probabilistic bound with constant 1).  The test takes
    the square-root form, per element, with `abs_sum` = the same sum over the
    absolute values of the operands, plus one rounding of the result; an index
    or term mistake moves a result by the size of a term, thousands of times more.
    Sums of at most 512 terms must also meet max|d| / mean|ref| <= 1e-5."""
    out = np.asarray(out, dtype=np.float64)
    ref = np.asarray(ref64, dtype=np.float64)
    abs_sum = np.asarray(abs_sum, dtype=np.float64)
    assert out.shape == ref.shape == abs_sum.shape, (out.shape, ref.shape, abs_sum.shape)
    tol = np.sqrt(float(nterms)) * EPS32 * abs_sum + EPS32 * np.abs(ref)
    err = np.abs(out - ref)
    bad = err > tol
    if bad.any():
        i = np.argmax(err - tol)
        raise AssertionError("%s: %d of %d elements beyond sqrt(n) 2^-24 sum|a||b| (worst: got %r ref %r bound %.3g)"
                             % (what, bad.sum(), bad.size, out.flat[i], ref.flat[i], tol.flat[i]))
    if nterms <= 512:
        assert_fp32_close(out, ref, 1e-5, what)
