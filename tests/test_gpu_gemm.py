"""GEMM parity on the GPU: NervanaGPU.dot / batched_dot through the C ABI
against the numpy oracle (np.dot check of benchmarks/gemm_test.py:27-70,
all-ones known answer of benchmarks/gemm_test2.py:40-41 and
kernels/C_interface/test.cu:27-124)."""
import ctypes
import os
import subprocess

import numpy as np
import pytest

import oracle as orc
from util import acc_atol, assert_fp16_within_ulp, assert_fp32_close

pytestmark = pytest.mark.gpu


def _operands(ng, op, m, n, k, dtype, rng, lo=-1.0, hi=1.0):
    A = rng.uniform(lo, hi, (m, k)).astype(dtype)
    B = rng.uniform(lo, hi, (k, n)).astype(dtype)
    devA = ng.array(np.ascontiguousarray(A.T) if op[0] == "t" else A, dtype=dtype)
    devB = ng.array(np.ascontiguousarray(B.T) if op[1] == "t" else B, dtype=dtype)
    if op[0] == "t":
        devA = devA.T
    if op[1] == "t":
        devB = devB.T
    return A, B, devA, devB


def _absdot(A, B):
    return np.abs(A.astype(np.float32)) @ np.abs(B.astype(np.float32))


def _check(out, ref, dtype, what, atol=0.0):
    if dtype == np.float16:
        assert_fp16_within_ulp(out, ref, 1.0, what, atol)
    else:
        assert_fp32_close(out, ref, 1e-5, what)


SMALL = (1, 2, 3, 7, 8, 9, 16, 33, 64, 65, 127, 128, 192)


@pytest.mark.parametrize("dtype", [np.float32, np.float16])
@pytest.mark.parametrize("op", ["nn", "nt", "tn"])
def test_dot_odd_sizes(ng, dtype, op):
    # subset of the small/medium lists of benchmarks/gemm_test.py:29-31
    rng = np.random.default_rng(11)
    sizes = [(m, n, k) for m in SMALL for n in (1, 9, 65, 128) for k in (1, 8, 72, 127)]
    sizes += [(778, 64, 787), (785, 794, 192), (1, 786, 64), (257, 255, 129), (1537, 64, 1532)]
    for (m, n, k) in sizes[::3] + sizes[-5:]:
        A, B, dA, dB = _operands(ng, op, m, n, k, dtype, rng)
        C = ng.empty((m, n), dtype=dtype)
        ng.dot(dA, dB, C)
        _check(C.get(), orc.ref_dot(A, B), dtype, "%s %s m,n,k=%d,%d,%d" % (np.dtype(dtype), op, m, n, k),
               acc_atol(_absdot(A, B)))


# 16-byte aligned operands whose extents are not multiples of any tile: one
# shape per tile shape of the dispatcher (64x64, 64x128, 128x128, 256x256),
# so the direct-to-LDS pipeline meets ragged edges in m, n and k
ALIGNED_RAGGED = [(1000, 136, 520), (520, 128, 1032), (1032, 1000, 72), (2056, 2040, 136), (3080, 3080, 520),
                  (8, 8, 8), (72, 4104, 264)]


@pytest.mark.parametrize("dtype", [np.float16, np.float32])
@pytest.mark.parametrize("op", ["nn", "nt", "tn"])
def test_dot_aligned_ragged_edges(ng, dtype, op):
    rng = np.random.default_rng(12)
    for (m, n, k) in ALIGNED_RAGGED:
        A, B, dA, dB = _operands(ng, op, m, n, k, dtype, rng)
        C = ng.empty((m, n), dtype=dtype)
        ng.dot(dA, dB, C)
        _check(C.get(), orc.ref_dot(A, B), dtype, "%s %s m,n,k=%d,%d,%d" % (np.dtype(dtype), op, m, n, k),
               acc_atol(_absdot(A, B)))


@pytest.mark.parametrize("op", ["nn", "nt", "tn"])
def test_dot_mid_size_long_contraction_fp16(ng, op):
    # between half a chip and a chip of 128x128 tiles with 48 or more 64-deep
    # contraction tiles: 128x128 tiles in two slices, ragged in m, n and k
    rng = np.random.default_rng(19)
    m, n, k = 1544, 1800, 3080
    A, B, dA, dB = _operands(ng, op, m, n, k, np.float16, rng)
    C = ng.empty((m, n), dtype=np.float16)
    ng.dot(dA, dB, C)
    _check(C.get(), orc.ref_dot(A, B), np.float16, "float16 %s m,n,k=%d,%d,%d" % (op, m, n, k), acc_atol(_absdot(A, B)))


# small outputs over long contractions: the contraction is cut into many slices
# and the fp32 partial sums are added by several lanes per output group
LONG_K = [(64, 64, 8192), (72, 136, 16400), (200, 8, 32768), (8, 24, 4104)]


@pytest.mark.parametrize("dtype", [np.float16, np.float32])
@pytest.mark.parametrize("op", ["nn", "nt", "tn"])
def test_dot_long_contraction_small_output(ng, dtype, op):
    rng = np.random.default_rng(17)
    for (m, n, k) in LONG_K:
        A, B, dA, dB = _operands(ng, op, m, n, k, dtype, rng)
        C = ng.empty((m, n), dtype=dtype)
        ng.dot(dA, dB, C, relu=True)
        first = C.get()
        _check(first, orc.ref_dot(A, B, relu=True), dtype, "%s %s m,n,k=%d,%d,%d" % (np.dtype(dtype), op, m, n, k),
               acc_atol(_absdot(A, B)))
        # the order of the additions is fixed: a second run gives the same bits
        C.fill(0)
        ng.dot(dA, dB, C, relu=True)
        assert np.array_equal(first.view(np.uint8), C.get().view(np.uint8))


@pytest.mark.parametrize("op", ["nn", "tn"])
def test_config1_fp32_1024(ng, op):
    rng = np.random.default_rng(0)
    A = rng.standard_normal((1024, 1024)).astype(np.float32)
    B = rng.standard_normal((1024, 1024)).astype(np.float32)
    dA = ng.array(np.ascontiguousarray(A.T), dtype=np.float32).T if op == "tn" else ng.array(A, dtype=np.float32)
    dB = ng.array(B, dtype=np.float32)
    C = ng.empty((1024, 1024), dtype=np.float32)
    ng.dot(dA, dB, C, relu=False)
    assert_fp32_close(C.get(), orc.ref_dot(A, B), 1e-5, "cfg1 " + op)


@pytest.mark.parametrize("size", [257, 256, 255, 129, 128, 127, 65, 64, 17, 16, 15])
def test_c_api_known_answers(ng, size):
    """kernels/C_interface/test.cu: sgemm of ones == size everywhere, hgemm of zeros == 0"""
    from nervanagpu_amd import _lib
    lib = _lib.load()
    ones = ng.ones((257, 257), dtype=np.float32)
    zeros = ng.zeros((257, 257), dtype=np.float16)
    outf = ng.empty((size, size), dtype=np.float32)
    outh = ng.ones((size, size), dtype=np.float16)
    assert lib.nervana_loadKernels(b"../cubin/")
    assert lib.nervana_randStateSizeBytes() == 2048 * 32 * 4
    vp = ctypes.c_void_p
    for a_t, b_t in ((False, False), (False, True), (True, False)):
        assert lib.nervana_sgemm(vp(ones.ptr), vp(ones.ptr), vp(outf.ptr), a_t, b_t, size, size, size,
                                 size, size, size, 1.0, 0.0, None, False, False, None, -1)
        assert np.all(outf.get() == size)
        assert lib.nervana_hgemm(vp(zeros.ptr), vp(zeros.ptr), vp(outh.ptr), a_t, b_t, size, size, size,
                                 size, size, size, 1.0, 0.0, None, False, False, None, -1)
        assert np.all(outh.get() == 0)
    # column-major wrapper: C_cm = A_cm . B_cm
    rng = np.random.default_rng(size)
    m, n, k = size, max(size // 2, 1), size + 3
    A = rng.uniform(-1, 1, (m, k)).astype(np.float32)
    B = rng.uniform(-1, 1, (k, n)).astype(np.float32)
    dA = ng.array(np.asfortranarray(A).T.copy(), dtype=np.float32)   # column-major bytes of A
    dB = ng.array(np.asfortranarray(B).T.copy(), dtype=np.float32)
    dC = ng.empty((n, m), dtype=np.float32)
    assert lib.nervana_sgemm_colmajor(vp(dA.ptr), vp(dB.ptr), vp(dC.ptr), False, False, m, n, k,
                                      m, k, m, 1.0, 0.0, None, False, False, None, -1)
    assert_fp32_close(dC.get().T, orc.ref_dot(A, B), 1e-5, "colmajor")


def test_all_ones_fp16_known_answer(ng):
    # benchmarks/gemm_test2.py:40-41: every element equals k, exactly representable in fp16
    m, n, k = 384, 256, 2048
    A = ng.ones((m, k), dtype=np.float16)
    B = ng.ones((k, n), dtype=np.float16)
    C = ng.empty((m, n), dtype=np.float16)
    ng.dot(A, B, C)
    assert np.all(C.get() == k)


@pytest.mark.parametrize("dtype", [np.float16, np.float32])
@pytest.mark.parametrize("op", ["nn", "nt", "tn"])
def test_alpha_beta_relu_and_strided_views(ng, dtype, op):
    rng = np.random.default_rng(5)
    m, n, k = 200, 136, 264
    A, B, dA, dB = _operands(ng, op, m, n, k, dtype, rng)
    C0 = rng.uniform(-1, 1, (m, n + 8)).astype(dtype)
    Cbig = ng.array(C0, dtype=dtype)
    C = Cbig[:, 8:]          # ldc > n, offset pointer
    for alpha, beta, relu in ((0.5, 0.5, False), (1.0, 0.0, True), (2.0, -1.0, True)):
        Cbig.set(C0)
        ng.dot(dA, dB, C, alpha=alpha, beta=beta, relu=relu)
        got = Cbig.get()
        ref = orc.ref_dot(A, B, C0[:, 8:], alpha, beta, relu)
        _check(got[:, 8:], ref, dtype, "alpha/beta/relu %s" % op, acc_atol(abs(alpha) * _absdot(A, B) + 1))
        assert np.array_equal(got[:, :8], C0[:, :8]), "columns outside the view were modified"


FC = [(4096, 9216), (4096, 4096), (1000, 4096)]


@pytest.mark.parametrize("MK", FC)
@pytest.mark.parametrize("op", ["nn", "nt", "tn"])
@pytest.mark.parametrize("relu", [False, True])
def test_config2_fc_shapes(ng, MK, op, relu):
    """fp16 FC-layer shapes with minibatch 128 (op <-> role mapping of benchmarks/cublas.py:68-71)"""
    M, K = MK
    N = 128
    rng = np.random.default_rng(1)
    if op == "nn":
        m, n, k = M, N, K
    elif op == "tn":
        m, n, k = K, N, M
    else:
        m, n, k = M, K, N
    A, B, dA, dB = _operands(ng, op, m, n, k, np.float16, rng)
    C = ng.empty((m, n), dtype=np.float16)
    ng.dot(dA, dB, C, relu=relu)
    assert_fp16_within_ulp(C.get(), orc.ref_dot(A, B, relu=relu), 1.0, "fc %s %s" % (MK, op),
                           acc_atol(_absdot(A, B)))


def test_config2_square_and_batched(ng):
    rng = np.random.default_rng(1)
    A, B, dA, dB = _operands(ng, "nn", 4096, 4096, 4096, np.float16, rng)
    C = ng.empty((4096, 4096), dtype=np.float16)
    ng.dot(dA, dB, C)
    assert_fp16_within_ulp(C.get(), orc.ref_dot(A, B), 1.0, "4096^3", acc_atol(_absdot(A, B)))
    # linearity: dot(A, 2B) == 2 dot(A, B) exactly (power-of-two scaling)
    dB2 = ng.array((B * np.float16(2)).astype(np.float16), dtype=np.float16)
    C2 = ng.empty((4096, 4096), dtype=np.float16)
    ng.dot(dA, dB2, C2)
    got, got2 = C.get().astype(np.float32), C2.get().astype(np.float32)
    fin = (np.abs(got2) < 60000) & (np.abs(got) > 2.0 ** -13)   # fp16 normal range only
    assert np.array_equal(got[fin] * 2, got2[fin])

    Ab = rng.uniform(-1, 1, (32, 512, 512)).astype(np.float16)
    Bb = rng.uniform(-1, 1, (32, 512, 512)).astype(np.float16)
    dAb, dBb = ng.array(Ab, dtype=np.float16), ng.array(Bb, dtype=np.float16)
    Cb = ng.empty((32, 512, 512), dtype=np.float16)
    ng.batched_dot(dAb, dBb, Cb)
    assert_fp16_within_ulp(Cb.get(), orc.ref_batched_dot(Ab, Bb), 1.0, "batched 32x512^3", acc_atol(512 * 0.3))


@pytest.mark.parametrize("dtype", [np.float16, np.float32])
def test_batched_dot_forms(ng, dtype):
    """fprop / bprop / update forms of benchmarks/batched_dot_test.py:41-74"""
    rng = np.random.default_rng(9)
    X, nOut, nIn, N = 5, 96, 72, 32
    W = rng.uniform(-1, 1, (nOut, nIn)).astype(dtype)
    I = rng.uniform(-1, 1, (X, nIn, N)).astype(dtype)
    E = rng.uniform(-1, 1, (X, nOut, N)).astype(dtype)
    dW, dI, dE = ng.array(W, dtype=dtype), ng.array(I, dtype=dtype), ng.array(E, dtype=dtype)
    dO = ng.empty((X, nOut, N), dtype=dtype)
    dB = ng.empty((X, nIn, N), dtype=dtype)
    dU = ng.empty((nOut, nIn), dtype=dtype)
    ng.batched_dot(dW, dI, dO)                 # 2-D A broadcast over the batch
    ng.batched_dot(dW.T, dE, dB)               # transposed 2-D A
    ng.batched_dot(dE, dI.T, dU)               # summed over the batch into 2-D C
    _check(dO.get(), orc.ref_batched_dot(W, I), dtype, "fprop", acc_atol(nIn))
    _check(dB.get(), orc.ref_batched_dot(W.T, E), dtype, "bprop", acc_atol(nOut))
    _check(dU.get(), orc.ref_batched_dot(E, np.transpose(I, (0, 2, 1)), out_3d=False), dtype, "update",
           acc_atol(X * N))


@pytest.mark.parametrize("dtype", [np.float16, np.float32])
def test_batched_dot_forms_minibatch_major(ng, dtype):
    """the second layout of benchmarks/batched_dot_test.py:54-57 (Nin = False): activations (X, N, C),
    3-D A with a transposed 2-D B, and a transposed 3-D A summed over the batch into a 2-D C"""
    rng = np.random.default_rng(10)
    X, nOut, nIn, N = 5, 96, 72, 32
    W = rng.uniform(-1, 1, (nOut, nIn)).astype(dtype)
    I = rng.uniform(-1, 1, (X, N, nIn)).astype(dtype)
    E = rng.uniform(-1, 1, (X, N, nOut)).astype(dtype)
    dW, dI, dE = ng.array(W, dtype=dtype), ng.array(I, dtype=dtype), ng.array(E, dtype=dtype)
    dO = ng.empty((X, N, nOut), dtype=dtype)
    dB = ng.empty((X, N, nIn), dtype=dtype)
    dU = ng.empty((nOut, nIn), dtype=dtype)
    ng.batched_dot(dI, dW.T, dO)               # fprop
    ng.batched_dot(dE, dW, dB)                 # bprop
    ng.batched_dot(dE.T, dI, dU)               # update: summed over the batch
    _check(dO.get(), orc.ref_batched_dot(I, W.T), dtype, "fprop", acc_atol(nIn))
    _check(dB.get(), orc.ref_batched_dot(E, W), dtype, "bprop", acc_atol(nOut))
    _check(dU.get(), orc.ref_batched_dot(np.transpose(E, (0, 2, 1)), I, out_3d=False), dtype, "update",
           acc_atol(X * N))


def test_batched_dot_reference_scale_accumulate():
    """batch accumulation at the reference's scale (benchmarks/batched_dot_test.py:19-23, 53: X = 100,
    (3072, 32) operands): E (X,K,N) . I^T (X,N,C) summed over the batch into (K,C), 3200 terms per
    output; dyadic operands, so the fp32 sums are exact in any order and the stochastic store is
    compared bit for bit, as is a 3-D output with a stochastic store"""
    from nervanagpu_amd import NervanaGPU
    ngs = NervanaGPU(stochastic_round=10, seed=77)
    rng = np.random.default_rng(13)
    X, K, C, N = 100, 3072, 3072, 32
    E, I = _dyadic(rng, (X, K, N)), _dyadic(rng, (X, C, N))
    dE, dI = ngs.array(E), ngs.array(I)
    dU = ngs.empty((K, C))
    ngs.batched_dot(dE, dI.T, dU)
    E2 = np.ascontiguousarray(np.transpose(E, (1, 0, 2))).reshape(K, X * N).astype(np.float32)
    I2 = np.ascontiguousarray(np.transpose(I, (1, 0, 2))).reshape(C, X * N).astype(np.float32)
    pre = E2 @ I2.T                                                                      # exact
    r = orc.rand_sr16(77, ngs.rng_counter, np.arange(K * C, dtype=np.uint32)).reshape(K, C)
    assert np.array_equal(dU.get().view(np.uint16), orc.round_stochastic_fp16(pre, 10, r).view(np.uint16))
    # nearest rounding of the same sums
    ngn = NervanaGPU(stochastic_round=False)
    dUn = ngn.empty((K, C))
    ngn.batched_dot(ngn.array(E), ngn.array(I).T, dUn)
    assert np.array_equal(dUn.get().view(np.uint16), pre.astype(np.float16).view(np.uint16))
    # 3-D output (one product per batch entry) with a stochastic store: the stream index runs over (z, i, j)
    W = _dyadic(rng, (256, C))
    dO = ngs.empty((8, 256, N))
    ngs.batched_dot(ngs.array(W), dI[0:8], dO, relu=True)
    pre = np.maximum(np.matmul(W.astype(np.float32)[None], I[0:8].astype(np.float32)), 0)
    r = orc.rand_sr16(77, ngs.rng_counter, np.arange(pre.size, dtype=np.uint32)).reshape(pre.shape)
    assert np.array_equal(dO.get().view(np.uint16), orc.round_stochastic_fp16(pre, 10, r).view(np.uint16))


@pytest.mark.parametrize("op", ["nn", "nt", "tn"])
def test_dot_one_round_of_128_tiles_three_stages(op):
    """256 tiles of 128x128 on 256 CUs with 16 or more contraction tiles: the three-stage pipeline
    (m = n = 2048); ragged k, beta and relu against the oracle, and a stochastic store bit for bit"""
    from nervanagpu_amd import NervanaGPU
    rng = np.random.default_rng(23)
    ngn = NervanaGPU(stochastic_round=False)
    m, n, k = 2048, 2048, 2056
    A, B, dA, dB = _operands(ngn, op, m, n, k, np.float16, rng)
    C0 = rng.uniform(-1, 1, (m, n)).astype(np.float16)
    C = ngn.array(C0)
    ngn.dot(dA, dB, C, alpha=0.5, beta=0.25, relu=True)
    assert_fp16_within_ulp(C.get(), orc.ref_dot(A, B, C0, 0.5, 0.25, True), 1.0, "2048x2048x2056 %s" % op,
                           acc_atol(0.5 * _absdot(A, B) + 0.25))
    ngs = NervanaGPU(stochastic_round=10, seed=6)
    k = 1032
    A, B = _dyadic(rng, (m, k)), _dyadic(rng, (k, n))
    dA = ngs.array(np.ascontiguousarray(A.T)).T if op[0] == "t" else ngs.array(A)
    dB = ngs.array(np.ascontiguousarray(B.T)).T if op[1] == "t" else ngs.array(B)
    C = ngs.empty((m, n))
    ngs.dot(dA, dB, C)
    pre = orc.ref_dot(A, B, acc_dtype=np.float32)
    r = orc.rand_sr16(6, ngs.rng_counter, np.arange(m * n, dtype=np.uint32)).reshape(m, n)
    assert np.array_equal(C.get().view(np.uint16), orc.round_stochastic_fp16(pre, 10, r).view(np.uint16))


def test_stochastic_rounding_bit_exact(ng):
    """SR output bit-exact against the numpy restatement fed the same stream.
    Operands are small dyadic rationals so every fp32 sum is exact and the
    pre-rounding value is known without ambiguity."""
    from nervanagpu_amd import NervanaGPU
    ngs = NervanaGPU(stochastic_round=10, seed=1234)
    rng = np.random.default_rng(3)
    for op, (m, n, k) in (("nn", (256, 128, 192)), ("tn", (130, 72, 64)), ("nt", (64, 264, 40))):
        A = (rng.integers(-64, 65, (m, k)) / 1024.0).astype(np.float16)
        B = (rng.integers(-64, 65, (k, n)) / 64.0).astype(np.float16)
        dA = ngs.array(np.ascontiguousarray(A.T) if op[0] == "t" else A)
        dB = ngs.array(np.ascontiguousarray(B.T) if op[1] == "t" else B)
        dA = dA.T if op[0] == "t" else dA
        dB = dB.T if op[1] == "t" else dB
        C = ngs.empty((m, n))
        assert C.rounding == 10
        ngs.dot(dA, dB, C, relu=True)
        stream = ngs.rng_counter
        pre = orc.ref_dot(A, B, relu=True)                      # exact in fp32
        assert np.array_equal(pre.astype(np.float64), np.maximum(A.astype(np.float64) @ B.astype(np.float64), 0))
        r = orc.rand_sr16(1234, stream, np.arange(m * n, dtype=np.uint32)).reshape(m, n)
        exp = orc.round_stochastic_fp16(pre, 10, r)
        got = C.get()
        assert np.array_equal(got.view(np.uint16), exp.view(np.uint16)), op
        # and it is not plain nearest rounding
        assert not np.array_equal(got.view(np.uint16), pre.astype(np.float16).view(np.uint16))
    # fp32 output keeps `bits` mantissa bits
    ngs32 = NervanaGPU(stochastic_round=7, seed=99)
    A = rng.uniform(-1, 1, (128, 64)).astype(np.float32)
    B = rng.uniform(-1, 1, (64, 136)).astype(np.float32)
    C = ngs32.empty((128, 136), dtype=np.float32)
    ngs32.dot(ngs32.array(A, dtype=np.float32), ngs32.array(B, dtype=np.float32), C)
    got = C.get()
    assert np.all((got.view(np.uint32) & ((1 << 16) - 1)) == 0)
    ref = orc.ref_dot(A, B)
    assert np.all(np.abs(got - ref) <= 2.0 ** -7 * np.abs(ref) * 1.01 + 1e-5)   # within one unit at 7 bits


def test_batched_dot_stochastic_rounding_bit_exact():
    """stochastic stores through batched_dot: one product per batch entry (the random stream is indexed
    by the flat position in the (batch, m, n) result) and the sum over the batch into a 2-D result, both
    bit for bit against the numpy restatement fed the same stream.  Dyadic operands: every fp32 sum is
    exact, so the value before rounding is known without ambiguity."""
    from nervanagpu_amd import NervanaGPU
    ngs = NervanaGPU(stochastic_round=10, seed=77)
    rng = np.random.default_rng(21)
    X, nOut, nIn, N = 6, 96, 72, 32
    W = _dyadic(rng, (nOut, nIn), 32)
    I = _dyadic(rng, (X, nIn, N), 32)
    E = _dyadic(rng, (X, nOut, N), 32)
    dW, dI, dE = ngs.array(W), ngs.array(I), ngs.array(E)
    dO = ngs.empty((X, nOut, N))
    ngs.batched_dot(dW, dI, dO, relu=True)
    pre = np.maximum(orc.ref_batched_dot(W, I, acc_dtype=np.float32), 0)
    assert np.array_equal(pre.astype(np.float64), np.maximum(np.einsum("oi,xin->xon", W.astype(np.float64), I.astype(np.float64)), 0))
    r = orc.rand_sr16(77, ngs.rng_counter, np.arange(pre.size, dtype=np.uint32)).reshape(pre.shape)
    got = dO.get()
    assert np.array_equal(got.view(np.uint16), orc.round_stochastic_fp16(pre, 10, r).view(np.uint16))
    assert not np.array_equal(got.view(np.uint16), pre.astype(np.float16).view(np.uint16))
    dU = ngs.empty((nOut, nIn))
    ngs.batched_dot(dE, dI.T, dU)
    pre = orc.ref_batched_dot(E, np.transpose(I, (0, 2, 1)), out_3d=False, acc_dtype=np.float32)
    assert np.array_equal(pre.astype(np.float64), np.einsum("xon,xin->oi", E.astype(np.float64), I.astype(np.float64)))
    r = orc.rand_sr16(77, ngs.rng_counter, np.arange(pre.size, dtype=np.uint32)).reshape(pre.shape)
    assert np.array_equal(dU.get().view(np.uint16), orc.round_stochastic_fp16(pre, 10, r).view(np.uint16))


def _dyadic(rng, shape, step=16):
    """multiples of 1/step in [-1, 1]: products are multiples of 1/step^2, and
    sums of up to 2^14 of them are exact in fp32 in any order"""
    return (rng.integers(-step, step + 1, shape) / float(step)).astype(np.float16)


def _fc_problem(op, M, K, N=128):
    if op == "nn":
        return M, N, K
    if op == "tn":
        return K, N, M
    return M, K, N


@pytest.mark.parametrize("MK", FC)
@pytest.mark.parametrize("op", ["nn", "nt", "tn"])
def test_config2_fc_shapes_stochastic_rounding_bit_exact(MK, op):
    """The nine FC cases with stochastic-round outputs: contraction slices with
    fp32 partial sums, the fixed-order reduce and its stochastic store (nn, tn),
    and the one-launch store (nt), bit for bit against the numpy restatement of
    fp32_to_fp16_rand (nervanagpu/float_ew.py:182-201) fed the same stream."""
    from nervanagpu_amd import NervanaGPU
    ngs = NervanaGPU(stochastic_round=10, seed=4321)
    rng = np.random.default_rng(21)
    m, n, k = _fc_problem(op, *MK)
    A, B = _dyadic(rng, (m, k)), _dyadic(rng, (k, n))
    dA = ngs.array(np.ascontiguousarray(A.T)).T if op[0] == "t" else ngs.array(A)
    dB = ngs.array(np.ascontiguousarray(B.T)).T if op[1] == "t" else ngs.array(B)
    for relu, beta in ((False, 0.0), (True, 0.5)):
        C0 = (rng.integers(-64, 65, (m, n)) / 16.0).astype(np.float16)
        C = ngs.array(C0)
        ngs.dot(dA, dB, C, beta=beta, relu=relu)
        pre = orc.ref_dot(A, B, C0, 1.0, beta, relu, acc_dtype=np.float32)     # exact
        r = orc.rand_sr16(4321, ngs.rng_counter, np.arange(m * n, dtype=np.uint32)).reshape(m, n)
        exp = orc.round_stochastic_fp16(pre, 10, r)
        got = C.get()
        assert np.array_equal(got.view(np.uint16), exp.view(np.uint16)), (op, MK, relu, beta)
        assert not np.array_equal(got.view(np.uint16), pre.astype(np.float16).view(np.uint16))


def test_config2_square_stochastic_rounding_bit_exact():
    """4096^3 (256x256 tiles, one launch) with a stochastic store, with and without beta"""
    from nervanagpu_amd import NervanaGPU
    ngs = NervanaGPU(stochastic_round=10, seed=8)
    rng = np.random.default_rng(22)
    m = n = k = 4096
    A, B = _dyadic(rng, (m, k)), _dyadic(rng, (k, n))
    dA, dB = ngs.array(A), ngs.array(B)
    for relu, beta in ((True, 0.0), (False, -0.5)):
        C0 = (rng.integers(-64, 65, (m, n)) / 16.0).astype(np.float16)
        C = ngs.array(C0)
        ngs.dot(dA, dB, C, beta=beta, relu=relu)
        pre = orc.ref_dot(A, B, C0, 1.0, beta, relu, acc_dtype=np.float32)
        r = orc.rand_sr16(8, ngs.rng_counter, np.arange(m * n, dtype=np.uint32)).reshape(m, n)
        assert np.array_equal(C.get().view(np.uint16), orc.round_stochastic_fp16(pre, 10, r).view(np.uint16)), (relu, beta)


@pytest.mark.parametrize("shape", [(256, 128, 192), (130, 72, 64), (4096, 128, 1024)])
def test_fp16_overflow_in_the_store(shape):
    """|value| beyond the largest fp16: nearest rounding gives infinity,
    stochastic rounding truncates to 65504 (round toward zero past the top,
    nervanagpu/float_ew.py:182-201); exact operands, so the comparison is on bits.
    Shapes: aligned one-launch store, ragged store, sliced contraction + reduce."""
    from nervanagpu_amd import NervanaGPU
    m, n, k = shape
    rng = np.random.default_rng(23)
    # integers -4..4 times powers of two chosen so that the sums have a spread of
    # about 50000: every partial sum is an exact multiple of sa*sb below 2^24 units
    e = int(round(np.log2(9821.0 / np.sqrt(k))))
    sa, sb = 2.0 ** (e // 2), 2.0 ** (e - e // 2)
    A = (rng.integers(-4, 5, (m, k)) * sa).astype(np.float16)
    B = (rng.integers(-4, 5, (k, n)) * sb).astype(np.float16)
    pre = orc.ref_dot(A, B, acc_dtype=np.float32)
    assert (np.abs(pre) > 65504).mean() > 0.05 and (np.abs(pre) < 65504).mean() > 0.05
    ngn = NervanaGPU(stochastic_round=False)
    C = ngn.empty((m, n))
    ngn.dot(ngn.array(A), ngn.array(B), C)
    with np.errstate(over="ignore"):
        exp = pre.astype(np.float16)
    got = C.get()
    assert np.isinf(exp).any()
    assert np.array_equal(got.view(np.uint16), exp.view(np.uint16))
    ngs = NervanaGPU(stochastic_round=10, seed=77)
    C = ngs.empty((m, n))
    ngs.dot(ngs.array(A), ngs.array(B), C)
    r = orc.rand_sr16(77, ngs.rng_counter, np.arange(m * n, dtype=np.uint32)).reshape(m, n)
    exp = orc.round_stochastic_fp16(pre, 10, r)
    got = C.get()
    assert np.array_equal(got.view(np.uint16), exp.view(np.uint16))
    assert np.all(np.isfinite(got)) and (np.abs(got.astype(np.float32)) == 65504).any()


@pytest.mark.parametrize("dtype", [np.float16, np.float32])
@pytest.mark.parametrize("shape", [(128, 136, 64), (130, 67, 40)])
def test_nan_and_infinities_reach_the_output(ng, dtype, shape):
    """Without relu nothing clamps: a NaN or an infinity in A shows up in every
    output of its row (aligned 16-byte stores and the ragged element-wise path);
    with relu the reference's max(v, 0) turns NaN and -inf into 0."""
    m, n, k = shape
    rng = np.random.default_rng(24)
    A = rng.uniform(0.5, 1, (m, k)).astype(dtype)
    B = rng.uniform(0.5, 1, (k, n)).astype(dtype)
    A[3, 5] = np.nan
    A[7, 1] = np.inf
    A[9, 2] = -np.inf
    C = ng.empty((m, n), dtype=dtype)
    ng.dot(ng.array(A, dtype=dtype), ng.array(B, dtype=dtype), C)
    got = C.get()
    assert np.all(np.isnan(got[3])) and np.all(got[7] == np.inf) and np.all(got[9] == -np.inf)
    rest = np.ones(m, dtype=bool)
    rest[[3, 7, 9]] = False
    assert np.all(np.isfinite(got[rest]))
    ng.dot(ng.array(A, dtype=dtype), ng.array(B, dtype=dtype), C, relu=True)
    got = C.get()
    assert np.all(got[3] == 0) and np.all(got[7] == np.inf) and np.all(got[9] == 0)


def test_c_api_hgemm_colmajor(ng):
    """nervana_hgemm_colmajor (kernels/C_interface/nervana_c_api.cu:402-420): the
    column-major product is the row-major product of the swapped operands"""
    from nervanagpu_amd import _lib
    lib = _lib.load()
    vp = ctypes.c_void_p
    rng = np.random.default_rng(25)
    m, n, k = 136, 72, 200
    A = rng.uniform(-1, 1, (m, k)).astype(np.float16)
    B = rng.uniform(-1, 1, (k, n)).astype(np.float16)
    dA = ng.array(np.ascontiguousarray(A.T))       # column-major bytes of A(m,k)
    dB = ng.array(np.ascontiguousarray(B.T))
    dC = ng.empty((n, m), dtype=np.float16)        # column-major bytes of C(m,n)
    assert lib.nervana_hgemm_colmajor(vp(dA.ptr), vp(dB.ptr), vp(dC.ptr), False, False, m, n, k,
                                      m, k, m, 1.0, 0.0, None, False, True, None, -1)
    assert_fp16_within_ulp(dC.get().T, orc.ref_dot(A, B, relu=True), 1.0, "hgemm colmajor", acc_atol(_absdot(A, B)))
    # transposed A: stored (m,k) row-major = column-major (k,m), lda = k
    dAt = ng.array(A)
    assert lib.nervana_hgemm_colmajor(vp(dAt.ptr), vp(dB.ptr), vp(dC.ptr), True, False, m, n, k,
                                      k, k, m, 1.0, 0.0, None, False, False, None, -1)
    assert_fp16_within_ulp(dC.get().T, orc.ref_dot(A, B), 1.0, "hgemm colmajor tn", acc_atol(_absdot(A, B)))


KAT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "c_api", "kat")


def _run_kat(*args):
    """the native caller of the C interface (tests/c_api/kat.cpp, built by build()), as a fresh process"""
    assert os.path.exists(KAT), "tests/c_api/kat is not built: run __graft_entry__.build()"
    done = subprocess.run([KAT] + list(args), stdout=subprocess.PIPE, stderr=subprocess.STDOUT, timeout=300)
    assert done.returncode == 0, done.stdout.decode("utf-8", "replace")[-2000:]
    return done.stdout.decode("utf-8", "replace")


def test_c_api_native_caller_known_answers():
    """kernels/C_interface/test.cu:27-124 compiled against include/nervana_hip.h, 17-argument calls:
    sgemm of ones == size and hgemm of zeros == 0 for 11 sizes x {nn, nt, tn}"""
    assert "known answers: 0 mismatches" in _run_kat()


def test_c_api_native_caller_stochastic_rounding(tmp_path):
    """nervana_hgemm(stochastic_round=true) from a fresh native process: seed 0 and one rounding stream
    per call, numbered from 1; an unsliced shape, two fully-connected shapes whose partial sums go
    through the library's static array (the second on another stream) and an nt shape, bit for bit
    against the numpy restatement of fp32_to_fp16_rand (nervanagpu/float_ew.py:182-201)"""
    out = str(tmp_path / "sr.bin")
    _run_kat("sr", out)
    raw = np.fromfile(out, dtype=np.uint8)
    pos, call = 0, 0
    while pos < raw.size:
        m, n, k, a_t, b_t, relu = (int(v) for v in raw[pos:pos + 24].view(np.int32))
        pos += 24
        call += 1
        A = raw[pos:pos + 2 * m * k].view(np.float16).reshape((k, m) if a_t else (m, k)); pos += 2 * m * k
        B = raw[pos:pos + 2 * k * n].view(np.float16).reshape((n, k) if b_t else (k, n)); pos += 2 * k * n
        C = raw[pos:pos + 2 * m * n].view(np.uint16).reshape(m, n); pos += 2 * m * n
        A = A.T if a_t else A
        B = B.T if b_t else B
        pre = orc.ref_dot(A, B, relu=bool(relu), acc_dtype=np.float32)      # exact: dyadic operands
        assert np.array_equal(pre.astype(np.float64), np.maximum(A.astype(np.float64) @ B.astype(np.float64),
                                                                 0 if relu else -np.inf))
        r = orc.rand_sr16(0, call, np.arange(m * n, dtype=np.uint32)).reshape(m, n)
        exp = orc.round_stochastic_fp16(pre, 10, r)
        assert np.array_equal(C, exp.view(np.uint16)), (call, m, n, k, a_t, b_t)
        assert not np.array_equal(C, pre.astype(np.float16).view(np.uint16))
    assert call == 4


def test_error_paths(ng):
    A = ng.empty((8, 8), dtype=np.float16)
    B = ng.empty((8, 8), dtype=np.float32)
    with pytest.raises(AssertionError):
        ng.dot(A, B, A)
    with pytest.raises(AssertionError):
        ng.dot(A.T, A.T, A)        # "tt" is not supported
    with pytest.raises(AssertionError):
        ng.dot(A, ng.empty((9, 8), dtype=np.float16), A)
    Ci = ng.empty((8, 8), dtype=np.int8)
    with pytest.raises((TypeError, AssertionError)):
        ng.dot(Ci, Ci, Ci)
