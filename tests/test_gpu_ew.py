"""Elementwise / reduction / broadcast expressions on the GPU against the numpy
oracle: the reference's own unit test matrix (nervanagpu/tests/test_tensor.py:
46-82) plus reductions, broadcasting, transposes, take/onehot, batch
normalisation (README.md:113) and stochastic-rounding stores."""
import numpy as np
import pytest

import oracle as orc
from util import assert_fp16_within_ulp, assert_fp32_close

pytestmark = pytest.mark.gpu

DIMS = (1024, 1024)


def rand_unif(dtype, dims, rng):
    if np.dtype(dtype).kind == "f":
        return rng.uniform(-1, 1, dims).astype(dtype)
    info = np.iinfo(dtype)
    return np.around(rng.uniform(info.min, info.max, dims)).clip(info.min, info.max)


def numpy_math(op, a, b):
    a, b = a.astype(np.float32), b.astype(np.float32)
    return {"+": lambda: a + b, "-": lambda: a - b, "*": lambda: a * b, "/": lambda: a / b,
            ">": lambda: a > b, ">=": lambda: a >= b, "<": lambda: a < b, "<=": lambda: a <= b}[op]()


def gpu_math(ng, op, inA, inB, dtype):
    A = ng.array(inA, dtype=dtype)
    B = ng.array(inB, dtype=dtype)
    C = ng.empty(inB.shape, dtype=dtype)
    if op == "+": C[:] = A + B
    elif op == "-": C[:] = A - B
    elif op == "*": C[:] = A * B
    elif op == "/": C[:] = A / B
    elif op == ">": C[:] = A > B
    elif op == ">=": C[:] = A >= B
    elif op == "<": C[:] = A < B
    elif op == "<=": C[:] = A <= B
    return C


@pytest.mark.parametrize("dtype", [np.float32, np.float16, np.int8, np.uint8])
def test_math_matrix(ng, dtype):
    """nervanagpu/tests/test_tensor.py:68-82; tolerance atol 1e-5 as in the reference
    (which makes the fp16 and integer cases bit-exact)"""
    rng = np.random.default_rng(0)
    inA, inB = rand_unif(dtype, DIMS, rng), rand_unif(dtype, DIMS, rng)
    for op in ("+", "-", "*", ">", ">=", "<", "<="):
        ref = numpy_math(op, inA.astype(dtype), inB.astype(dtype)).astype(np.float32)
        if np.dtype(dtype).kind in "iu":
            ref = np.around(ref).clip(np.iinfo(dtype).min, np.iinfo(dtype).max)
        ref = ref.astype(dtype)
        got = gpu_math(ng, op, inA, inB, dtype).get()
        np.testing.assert_allclose(got.astype(np.float64), ref.astype(np.float64), atol=1e-5, rtol=0,
                                   err_msg="%s %s" % (np.dtype(dtype), op))
    if np.dtype(dtype).kind == "f":
        inB = np.where(np.abs(inB) < 0.05, dtype(0.5), inB)
        ref = numpy_math("/", inA, inB).astype(dtype)
        got = gpu_math(ng, "/", inA, inB, dtype).get()
        # the reference compiles with fast-math division (nervanagpu/float_ew.py:1030);
        # here x / y is x * rcp(y): within 2 ulp in fp32, then rounded to nearest
        if dtype is np.float32:
            np.testing.assert_allclose(got, ref, rtol=2.5e-7, atol=0)
        else:
            assert_fp16_within_ulp(got, inA.astype(np.float32) / inB.astype(np.float32), 1, "fp16 division")


def test_unary_ops_and_constants(ng):
    rng = np.random.default_rng(1)
    a = rng.uniform(0.1, 2.0, (300, 200)).astype(np.float32)
    A = ng.array(a, dtype=np.float32)
    C = ng.empty(a.shape, dtype=np.float32)
    # sqrt and division are the hardware approximations (fast-math in the reference)
    cases = [
        (lambda: ng.sqrt(A), np.sqrt(a), 2.5e-7), (lambda: ng.square(A), a * a, 0),
        (lambda: ng.exp(A), np.exp(a), 2e-6), (lambda: ng.log(A), np.log(a), 2e-6),
        (lambda: ng.exp2(A), np.exp2(a), 2e-6), (lambda: ng.log2(A), np.log2(a), 2e-6),
        (lambda: ng.sig(A), 1 / (1 + np.exp(-a)), 2e-6), (lambda: ng.tanh(A), np.tanh(a), 2e-6),
        (lambda: ng.tanh2(A), (np.exp2(2 * a) - 1) / (np.exp2(2 * a) + 1), 4e-6),
        (lambda: ng.sig2(A), 1 / (1 + np.exp2(-a)), 2e-6),
        (lambda: ng.reciprocal(A), (1 / a), 2.5e-7), (lambda: -A, -a, 0), (lambda: abs(A - 1.0), np.abs(a - np.float32(1)), 0),
        (lambda: ng.sgn(A - 1.0), np.copysign(1, a - np.float32(1)), 0),
        (lambda: ng.power(A, 1.5), np.power(a, np.float32(1.5)), 4e-6),
        (lambda: ng.clip(A, 0.5, 1.0), np.clip(a, 0.5, 1.0), 0),
        (lambda: ng.maximum(A, 1.25), np.maximum(a, 1.25), 0), (lambda: ng.minimum(A, 1.25), np.minimum(a, 1.25), 0),
        (lambda: 2.5 * A * A + 1, np.float32(2.5) * a * a + 1, 0),
        (lambda: 1 - A, 1 - a, 0), (lambda: 2.0 / A, np.float32(2) / a, 2.5e-7),
        (lambda: (A == A) + (A != A), np.ones_like(a), 0),
        (lambda: ng.finite(ng.log(A - 1.0)), np.isfinite(np.log(a - np.float32(1))).astype(np.float32), 0),
    ]
    with np.errstate(all="ignore"):
        for i, (expr, ref, rtol) in enumerate(cases):
            C[:] = expr()
            got = C.get()
            if rtol == 0:
                assert np.array_equal(got, ref.astype(np.float32)), "case %d" % i
            else:
                np.testing.assert_allclose(got, ref.astype(np.float32), rtol=rtol, atol=1e-7, err_msg="case %d" % i)


@pytest.mark.parametrize("dtype", [np.float32, np.float16])
@pytest.mark.parametrize("shape", [(64, 8192), (333, 1000), (1000, 37), (7, 5), (4096, 50000 // 8 * 8 + 8)])
def test_reductions_axis1_and_axis0(ng, dtype, shape):
    rng = np.random.default_rng(2)
    if shape[0] * shape[1] > 3e7:
        shape = (shape[0] // 16, shape[1])
    a = rng.uniform(-1, 1, shape).astype(dtype)
    A = ng.array(a, dtype=dtype)
    a32 = a.astype(np.float32)
    for axis in (1, 0):
        oshape = (shape[0], 1) if axis == 1 else (1, shape[1])
        O = ng.empty(oshape, dtype=np.float32)
        n = shape[axis]
        ng.sum(A, axis=axis, out=O)
        np.testing.assert_allclose(O.get(), a32.astype(np.float64).sum(axis=axis, keepdims=True),
                                   rtol=1e-5, atol=1e-5 * np.sqrt(n))
        ng.max(A, axis=axis, out=O)
        assert np.array_equal(O.get(), a32.max(axis=axis, keepdims=True))
        ng.min(A, axis=axis, out=O)
        assert np.array_equal(O.get(), a32.min(axis=axis, keepdims=True))
        ng.mean(A, axis=axis, out=O)
        np.testing.assert_allclose(O.get(), a32.astype(np.float64).mean(axis=axis, keepdims=True), rtol=1e-5, atol=2e-6)
        ng.var(A, axis=axis, out=O)
        assert_fp32_close(O.get(), a32.astype(np.float64).var(axis=axis, keepdims=True), 1e-5, "var axis %d" % axis)
        ng.std(A, axis=axis, out=O)
        assert_fp32_close(O.get(), a32.astype(np.float64).std(axis=axis, keepdims=True), 1e-5, "std axis %d" % axis)
        Oi = ng.empty(oshape, dtype=np.int32)
        ng.argmax(A, axis=axis, out=Oi)
        assert np.array_equal(Oi.get(), np.expand_dims(np.argmax(a32, axis=axis), axis))
        ng.argmin(A, axis=axis, out=Oi)
        assert np.array_equal(Oi.get(), np.expand_dims(np.argmin(a32, axis=axis), axis))


def test_argmax_ties_take_lower_index(ng):
    a = np.zeros((5, 700), np.float32)
    a[:, [3, 64, 650]] = 2.0
    A = ng.array(a, dtype=np.float32)
    Oi = ng.empty((5, 1), dtype=np.int32)
    ng.argmax(A, axis=1, out=Oi)
    assert np.all(Oi.get() == 3)
    ng.argmin(-A, axis=1, out=Oi)
    assert np.all(Oi.get() == 3)


def test_full_reduction_with_partial_and_layer_stats(ng):
    rng = np.random.default_rng(3)
    a = rng.uniform(-1, 1, (513, 257)).astype(np.float16)
    A = ng.array(a)
    partial = ng.empty((513, 1), dtype=np.float32)
    out = partial[0:1, 0:1]
    got = float(ng.mean(abs(A), partial=partial, out=out).get()[0, 0])
    assert abs(got - np.abs(a.astype(np.float64)).mean()) < 1e-5
    got = float(ng.max(abs(A), partial=partial, out=out).get()[0, 0])
    assert got == np.abs(a.astype(np.float32)).max()
    got = float(ng.sum(A, partial=partial, out=out).get()[0, 0])
    assert abs(got - a.astype(np.float64).sum()) < 1e-2


def test_broadcast_transpose_inplace(ng):
    rng = np.random.default_rng(4)
    a = rng.uniform(-1, 1, (200, 300)).astype(np.float32)
    col = rng.uniform(-1, 1, (200, 1)).astype(np.float32)
    row = rng.uniform(-1, 1, (1, 300)).astype(np.float32)
    A, Cc, Rr = ng.array(a, dtype=np.float32), ng.array(col, dtype=np.float32), ng.array(row, dtype=np.float32)
    O = ng.empty(a.shape, dtype=np.float32)
    O[:] = A * Cc + Rr
    assert np.array_equal(O.get(), a * col + row)
    O[:] = Rr + 0 * Cc          # both operands broadcast
    assert np.array_equal(O.get(), np.broadcast_to(row, a.shape) + 0 * col)
    Ot = ng.empty((300, 200), dtype=np.float32)
    Ot[:] = A.T
    assert np.array_equal(Ot.get(), a.T)
    A.transpose(out=Ot)
    assert np.array_equal(Ot.get(), a.T)
    Ot[:] = A.T * 2 + Ot
    assert np.array_equal(Ot.get(), a.T * 2 + a.T)
    A += 1
    A *= Rr
    assert np.array_equal(A.get(), (a + 1) * row)
    # slices (non-contiguous views) on both sides
    O.fill(0)
    O[10:20, 5:50] = A[30:40, 100:145] - 3
    ref = np.zeros_like(a)
    ref[10:20, 5:50] = ((a + 1) * row)[30:40, 100:145] - 3
    assert np.array_equal(O.get(), ref)
    O[3, :] = 7
    ref[3, :] = 7
    assert np.array_equal(O.get(), ref)
    with pytest.raises(TypeError):
        O[:] = A + ng.empty((200, 299), dtype=np.float32)
    with pytest.raises(ValueError):
        O[:] = ng.sum(A, axis=1) + ng.sum(A, axis=0)
    with pytest.raises(ValueError):
        ng.sum(A, axis=2, out=O)


def test_fill_copy_reshape_share_dtypes(ng):
    for dtype in (np.float16, np.float32, np.int8, np.uint8, np.int32):
        z = ng.zeros((33, 17), dtype=dtype)
        o = ng.ones((33, 17), dtype=dtype)
        assert np.all(z.get() == 0) and np.all(o.get() == 1)
        o.fill(3)
        assert np.all(o.get() == 3) and o.get().dtype == dtype
        z.copy(o)
        assert np.all(z.get() == 3)
    a = np.arange(24, dtype=np.float32).reshape(4, 6)
    A = ng.array(a, dtype=np.float32)
    assert np.array_equal(A.reshape(6, 4).get(), a.reshape(6, 4))
    assert np.array_equal(A.reshape((2, 12)).get(), a.reshape(2, 12))
    assert np.array_equal(A.share((3, 4)).get(), a.reshape(-1)[:12].reshape(3, 4))
    assert np.array_equal(A[1:3].get(), a[1:3])
    assert np.array_equal(A[2].get(), a[2])
    with pytest.raises(ValueError):
        A.reshape(5, 5)
    with pytest.raises(ValueError):
        A.share((5, 5))
    with pytest.raises(IndexError):
        A[7]
    # conversions between dtypes round half to even and saturate
    f = np.array([[0.5, 1.5, 2.5, -0.5, 300.0, -300.0, 126.5, 3.7]], dtype=np.float32)
    F = ng.array(f, dtype=np.float32)
    I8 = ng.empty(f.shape, dtype=np.int8)
    U8 = ng.empty(f.shape, dtype=np.uint8)
    I8[:] = F
    U8[:] = F
    assert np.array_equal(I8.get(), orc.round_int(f, np.int8))
    assert np.array_equal(U8.get(), orc.round_int(f, np.uint8))
    H = ng.empty(f.shape, dtype=np.float16)
    H[:] = U8
    assert np.array_equal(H.get(), orc.round_int(f, np.uint8).astype(np.float16))


def test_take_and_onehot(ng):
    rng = np.random.default_rng(5)
    a = rng.uniform(-1, 1, (50, 40)).astype(np.float32)
    A = ng.array(a, dtype=np.float32)
    idx = rng.integers(0, 50, 20).astype(np.int32)
    O = ng.empty((20, 40), dtype=np.float32)
    A.take(idx, axis=0, out=O)
    assert np.array_equal(O.get(), a[idx])
    idx1 = rng.integers(0, 40, 16).astype(np.int32)
    O1 = ng.empty((50, 16), dtype=np.float32)
    ng.take(A, idx1, 1, out=O1)
    assert np.array_equal(O1.get(), a[:, idx1])
    # one-hot along axis 0: out[i, j] = (idx[j] == i)
    labels = rng.integers(0, 10, 40).astype(np.int32)
    L = ng.array(labels.reshape(1, -1), dtype=np.int32)
    H0 = ng.empty((10, 40), dtype=np.float32)
    ng.onehot(L, axis=0, out=H0)
    assert np.array_equal(H0.get(), (np.arange(10)[:, None] == labels[None, :]).astype(np.float32))
    labels1 = rng.integers(0, 40, 10).astype(np.int32)
    L1 = ng.array(labels1.reshape(-1, 1), dtype=np.int32)
    H1 = ng.empty((10, 40), dtype=np.float32)
    ng.onehot(L1, axis=1, out=H1)
    assert np.array_equal(H1.get(), (np.arange(40)[None, :] == labels1[:, None]).astype(np.float32))


def bn_expr(ng, A, eps):
    return (A - ng.mean(A, axis=1)) / ng.sqrt(ng.var(A, axis=1) + eps)


@pytest.mark.parametrize("shape", [(64, 512), (37, 1000), (16, 8192), (4, 20000)])
def test_batchnorm_expression(ng, shape):
    rng = np.random.default_rng(6)
    a = rng.uniform(0, 1, shape).astype(np.float16)
    A = ng.array(a)
    O32 = ng.empty(shape, dtype=np.float32)
    O32[:] = bn_expr(ng, A, 1e-3)
    ref = orc.ref_batchnorm_rows(a, 1e-3)
    np.testing.assert_allclose(O32.get(), ref, rtol=1e-5, atol=1e-5)
    A[:] = bn_expr(ng, A, 1e-3)             # in place, fp16 nearest
    assert_fp16_within_ulp(A.get(), ref, 1.0, "bn fp16", atol=1e-5)
    # the postfix stack evaluated by the oracle's generic evaluator gives the same answer
    A2 = ng.array(a)
    stack = bn_expr(ng, A2, 1e-3).traverse([])
    st = [a if item is A2 else item for item in stack]
    np.testing.assert_allclose(O32.get(), orc.ref_ew(st, shape), rtol=2e-5, atol=2e-5)


def test_config5_batchnorm_full_shape(ng):
    """(4096, 8192) fp16 rows, the benchmark's own shape: nearest rounding within
    one ulp of the float64 closed form; the stochastic store bit-exact against the
    numpy restatement fed the kernel's own fp32 values and the same stream"""
    from nervanagpu_amd import NervanaGPU
    shape = (4096, 8192)
    a = np.random.default_rng(4).uniform(0, 1, shape).astype(np.float16)
    A = ng.array(a)
    A[:] = bn_expr(ng, A, 1e-3)
    ref = orc.ref_batchnorm_rows(a, 1e-3)
    assert_fp16_within_ulp(A.get(), ref, 1.0, "bn fp16 full shape", atol=1e-5)
    assert np.abs(A.get().astype(np.float64).mean(axis=1)).max() < 2e-3      # rows end up centred

    ngs = NervanaGPU(stochastic_round=True, seed=4)
    S = ngs.array(a)
    assert S.rounding == 10
    P = ngs.empty(shape, dtype=np.float32)
    P.rounding = 0
    P[:] = bn_expr(ngs, S, 1e-3)
    S[:] = bn_expr(ngs, S, 1e-3)
    r = orc.rand_sr16(4, ngs.rng_counter, np.arange(a.size, dtype=np.uint32)).reshape(shape)
    assert np.array_equal(S.get().view(np.uint16), orc.round_stochastic_fp16(P.get(), 10, r).view(np.uint16))


def test_stochastic_rounding_store_bit_exact(ng):
    """fp16 SR store: bit-exact against the numpy restatement fed the same stream"""
    from nervanagpu_amd import NervanaGPU
    ngs = NervanaGPU(stochastic_round=True, seed=77)
    rng = np.random.default_rng(7)
    for shape in ((64, 1024), (33, 250), (33, 251)):
        a = (rng.standard_normal(shape) * 3).astype(np.float32)
        A = ngs.array(a, dtype=np.float32)
        H = ngs.empty(shape)                # fp16, rounding=10
        assert H.rounding == 10
        H[:] = A                            # plain contiguous copy-convert
        r = orc.rand_sr16(77, ngs.rng_counter, np.arange(a.size, dtype=np.uint32)).reshape(shape)
        assert np.array_equal(H.get().view(np.uint16), orc.round_stochastic_fp16(a, 10, r).view(np.uint16))
        # row-mode kernel (reduction + broadcast) with SR store: take the kernel's own
        # fp32 values from a second, unrounded run of the same expression
        P = ngs.empty(shape, dtype=np.float32)
        P.rounding = 0
        P[:] = bn_expr(ngs, A, 1e-3)
        H[:] = bn_expr(ngs, A, 1e-3)
        r = orc.rand_sr16(77, ngs.rng_counter, np.arange(a.size, dtype=np.uint32)).reshape(shape)
        assert np.array_equal(H.get().view(np.uint16), orc.round_stochastic_fp16(P.get(), 10, r).view(np.uint16))
        # fewer bits, transposed output walk (axis 0 reduction)
        H.rounding = 4
        H[:] = A - ng_mean0(ngs, A)
        P[:] = A - ng_mean0(ngs, A)
        r = orc.rand_sr16(77, ngs.rng_counter, np.arange(a.size, dtype=np.uint32)).reshape(shape)
        assert np.array_equal(H.get().view(np.uint16), orc.round_stochastic_fp16(P.get(), 4, r).view(np.uint16))
        H.rounding = 10
    # fp32 SR
    F = ngs.empty((64, 1024), dtype=np.float32)
    F.rounding = 15
    a = rng.standard_normal((64, 1024)).astype(np.float32)
    F[:] = ngs.array(a, dtype=np.float32) * 1.0
    r = orc.rand32(77, ngs.rng_counter, np.arange(a.size, dtype=np.uint32)).reshape(a.shape)
    assert np.array_equal(F.get().view(np.uint32), orc.round_stochastic_fp32(a, 15, r).view(np.uint32))
    # special values through the device conversion
    sp = np.array([0.0, -0.0, 65504.0, 65519.0, 70000.0, -70000.0, 1e-8, 6e-8, 6.1e-5, -3e-5, 1e30, 2.0 ** -24,
                   np.inf, -np.inf, 3.4028235e38, -3.4028235e38, 3.4028e38, 65503.99, 65535.99, 65536.0,
                   2.0 ** -14, 2.0 ** -14 - 2.0 ** -30, 5.9e-8, -2.9e-8], dtype=np.float32)
    spb = np.concatenate([sp.view(np.uint32), np.array([0x7FC00000, 0xFFC00000, 0x7F800001, 0xFFFFFFFF, 0x7FFFFFFF,
                                                        0x7F7FE000, 0x7F7FE001, 0x477FDFFF], dtype=np.uint32)])
    # every value at even and odd positions, under many different draws, at full and reduced precision
    sp = np.tile(spb, 64).reshape(64, spb.size).view(np.float32)
    sp = np.concatenate([sp, np.roll(sp, 1, axis=1)], axis=0)
    S = ngs.empty(sp.shape)
    for bits in (10, 7):
        S.rounding = bits
        S[:] = ngs.array(sp, dtype=np.float32)
        r = orc.rand_sr16(77, ngs.rng_counter, np.arange(sp.size, dtype=np.uint32)).reshape(sp.shape)
        got, ref = S.get().view(np.uint16), orc.round_stochastic_fp16(sp, bits, r).view(np.uint16)
        nan = np.isnan(sp)
        assert np.array_equal(got[~nan], ref[~nan]), bits
        assert np.all(np.isnan(S.get()[nan]))   # NaN stays NaN (payload bits are not compared)


def ng_mean0(ngs, A):
    return ngs.mean(A, axis=0)


def test_rand_and_dropout(ng):
    from nervanagpu_amd import NervanaGPU
    ngs = NervanaGPU(seed=5)
    R = ngs.empty((128, 512), dtype=np.float32)
    ngs.rand(out=R)
    got = R.get()
    assert got.min() >= 0 and got.max() <= 1 and abs(got.mean() - 0.5) < 0.01
    exp = orc.rand_uniform(5, ngs.rng_counter + 0x1000193 * 1, np.arange(got.size, dtype=np.uint32)).reshape(got.shape)
    assert np.array_equal(got, exp)
    D = ngs.empty((128, 512), dtype=np.float32)
    ngs.dropout(keep=0.3, out=D)
    assert abs(D.get().mean() - 0.3) < 0.02


def test_compensated_sum(ng):
    rng = np.random.default_rng(8)
    s = np.zeros((64, 128), np.float16)
    c = np.zeros((64, 128), np.float16)
    S, Cm = ng.array(s), ng.array(c)
    for _ in range(5):
        a = rng.uniform(0, 0.01, s.shape).astype(np.float16)
        ng.compensated_sum(S, Cm, ng.array(a), 1.0, 0.5)
        s, c = orc.ref_compensated_sum(s, c, a, 1.0, 0.5)
        assert np.array_equal(S.get(), s) and np.array_equal(Cm.get(), c)


def test_compensated_sum_stochastic_and_strided():
    """the fused accumulate with a stochastic store of the running sum (bit exact
    against the numpy restatement on the same stream, one stream per call), fp32
    storage, and strided 2-D views (scalar path)"""
    from nervanagpu_amd import NervanaGPU
    ngs = NervanaGPU(stochastic_round=10, seed=31)
    rng = np.random.default_rng(9)
    s = rng.uniform(-1, 1, (48, 264)).astype(np.float16)
    c = np.zeros_like(s)
    S, Cm = ngs.array(s), ngs.array(c)
    for step in range(3):
        a = rng.uniform(-0.01, 0.01, s.shape).astype(np.float16)
        before = ngs.rng_counter
        ngs.compensated_sum(S, Cm, ngs.array(a), 0.75, 1.5)
        assert ngs.rng_counter == before + 1
        r = orc.rand_sr16(31, ngs.rng_counter, np.arange(s.size, dtype=np.uint32)).reshape(s.shape)
        s, c = orc.ref_compensated_sum(s, c, a, 0.75, 1.5, rounding=10, r=r)
        assert np.array_equal(S.get().view(np.uint16), s.view(np.uint16)), step
        assert np.array_equal(Cm.get().view(np.uint16), c.view(np.uint16)), step
    # fp32 storage, nearest rounding, on column slices of wider tensors
    ngn = NervanaGPU(stochastic_round=False)
    s32 = rng.uniform(-1, 1, (33, 70)).astype(np.float32)
    c32 = rng.uniform(-1e-6, 1e-6, (33, 70)).astype(np.float32)
    a32 = rng.uniform(-1e-3, 1e-3, (33, 70)).astype(np.float32)
    S32, C32, A32 = (ngn.array(x, dtype=np.float32) for x in (s32, c32, a32))
    ngn.compensated_sum(S32[:, 3:61], C32[:, 3:61], A32[:, 3:61], 1.0, 2.0)
    es, ec = orc.ref_compensated_sum(s32[:, 3:61], c32[:, 3:61], a32[:, 3:61], 1.0, 2.0, dtype=np.float32)
    gs, gc = S32.get(), C32.get()
    assert np.array_equal(gs[:, 3:61], es) and np.array_equal(gc[:, 3:61], ec)
    assert np.array_equal(gs[:, :3], s32[:, :3]) and np.array_equal(gs[:, 61:], s32[:, 61:])
    # the reset of the compensation after kahan_reset calls
    C32.kahan_reset = 1
    C32.kahan_count = 2
    ngn.compensated_sum(S32, C32, A32)
    es2, _ = orc.ref_compensated_sum(gs, gc, a32, 0.0, 1.0, dtype=np.float32)
    assert np.array_equal(S32.get(), es2) and C32.kahan_count == 1
