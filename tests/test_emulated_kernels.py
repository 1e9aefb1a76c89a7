"""The HIP kernels run lane by lane on the CPU (tests/emu): the kernel sources of nervanagpu_amd/csrc
are compiled for the host against a stand-in HIP runtime in which every thread of a workgroup is a
fiber, barriers and wavefront-wide instructions (MFMA, transposing LDS reads, readlane) are rendezvous
points, buffer descriptors apply the hardware's out-of-range rule, every global access is checked
against the registered buffers, and loads that write LDS directly land either at once or only when the
issuing wavefront's s_waitcnt covers them (`late_loads`), with the fibers resumed in a shuffled order.
That checks index arithmetic, tile layouts, barriers and wait counts without a GPU, against the same
numpy oracle as the GPU parity tests.  It is test infrastructure: the product never loads this library,
and the results say nothing about speed."""
import os
import subprocess
import sys

import numpy as np
import pytest

import oracle as orc
from util import acc_atol, assert_fp16_within_ulp, assert_fp32_close

sys.path.insert(0, os.path.join(os.path.dirname(os.path.abspath(__file__)), "emu"))


@pytest.fixture(scope="module")
def emu():
    import emu as module
    module.build()          # incremental: a few seconds when the library is current
    module.load()
    return module


def _operands(rng, m, n, k, ta, tb, dtype=np.float16):
    A = rng.uniform(-1, 1, (k, m) if ta else (m, k)).astype(dtype)
    B = rng.uniform(-1, 1, (n, k) if tb else (k, n)).astype(dtype)
    return A, B, (A.T if ta else A), (B.T if tb else B)


GEMM_CASES = [  # m, n, k, A transposed, B transposed: on 8 emulated CUs these reach the tile shapes named
    (64, 64, 64, 0, 0),          # 64x64 tiles
    (128, 136, 72, 0, 1),        # 128x128 half-depth tiles, ragged n and k
    (72, 64, 136, 1, 0),         # transposed A: row-contiguous tiles, transposing LDS reads
    (512, 128, 1024, 0, 0),      # minibatch-wide: 64x128 tiles, two contraction slices + fixed-order reduce
    (392, 104, 1032, 1, 0),      # ... ragged in m, n and k
    (256, 520, 256, 0, 0),       # 256x256 tiles (more than half of the emulated chip)
    (136, 1032, 128, 0, 1),      # outer-product shape: output stream
]


@pytest.mark.parametrize("late_loads,shuffle", [(False, 0), (True, 7)])
@pytest.mark.parametrize("case", GEMM_CASES)
def test_emulated_gemm_fp16(emu, case, late_loads, shuffle):
    m, n, k, ta, tb = case
    rng = np.random.default_rng(m + n + k)
    A, B, a, b = _operands(rng, m, n, k, ta, tb)
    C0 = rng.uniform(-1, 1, (m, n)).astype(np.float16)
    got = emu.gemm(A, B, ta, tb, alpha=0.5, beta=0.25, relu=True, C=C0, late_loads=late_loads, shuffle=shuffle)
    absdot = np.abs(a).astype(np.float32) @ np.abs(b).astype(np.float32)
    assert_fp16_within_ulp(got, orc.ref_dot(a, b, C0, 0.5, 0.25, True), 1.0, str(case), acc_atol(0.5 * absdot + 0.25))


def test_emulated_gemm_fp32_and_unaligned(emu):
    rng = np.random.default_rng(3)
    for (m, n, k, ta, tb) in [(96, 72, 40, 0, 0), (65, 33, 17, 1, 0), (40, 96, 24, 0, 1)]:
        A, B, a, b = _operands(rng, m, n, k, ta, tb, np.float32)
        assert_fp32_close(emu.gemm(A, B, ta, tb), orc.ref_dot(a, b), 1e-5, "fp32 %s" % ((m, n, k, ta, tb),))
    # fp16 with extents that are not multiples of 8: the element-wise loader
    A, B, a, b = _operands(rng, 37, 21, 53, 0, 0)
    assert_fp16_within_ulp(emu.gemm(A, B), orc.ref_dot(a, b), 1.0, "ragged fp16",
                           acc_atol(np.abs(a).astype(np.float32) @ np.abs(b).astype(np.float32)))


def test_emulated_gemm_stochastic_rounding_bit_exact(emu):
    """sliced contraction + stochastic store in the reduce, and the one-launch store"""
    rng = np.random.default_rng(4)
    for (m, n, k, ta, tb) in [(256, 128, 1024, 0, 0), (128, 264, 64, 0, 1)]:
        A = (rng.integers(-16, 17, (m, k)) / 16.0).astype(np.float16)
        B = (rng.integers(-16, 17, (n, k) if tb else (k, n)) / 16.0).astype(np.float16)
        got = emu.gemm(A, B, ta, tb, sr_bits=10, seed=99, stream=3, late_loads=True, shuffle=1)
        pre = orc.ref_dot(A, B.T if tb else B, acc_dtype=np.float32)       # exact
        r = orc.rand_sr16(99, 3, np.arange(m * n, dtype=np.uint32)).reshape(m, n)
        assert np.array_equal(got.view(np.uint16), orc.round_stochastic_fp16(pre, 10, r).view(np.uint16))


CONV_CASES = [  # N, C, K, DHW, TRS, pad, strides
    (16, 3, 8, (1, 12, 12), (1, 3, 3), (0, 1, 1), (1, 1, 1)),       # first layer: row-by-row gather / streamed columns
    (8, 16, 32, (1, 9, 8), (1, 3, 3), (0, 1, 1), (1, 2, 2)),        # strided: one class per residue
    (64, 64, 72, (1, 4, 8), (1, 3, 3), (0, 1, 1), (1, 1, 1)),       # blocked channels, shared taps, ring update
    (8, 8, 16, (3, 5, 5), (2, 3, 3), (1, 0, 1), (1, 1, 2)),         # 3-D
]


@pytest.mark.parametrize("case", CONV_CASES)
def test_emulated_convolution(emu, case):
    N, C, K, DHW, TRS, pad, strd = case
    conv = emu.Conv(np.float16, N, C, K, DHW, TRS, pad, strd)
    rng = np.random.default_rng(N + C + K)
    I = rng.uniform(-1, 1, conv.dimI).astype(np.float16)
    F = rng.uniform(-1, 1, conv.dimF).astype(np.float16)
    E = rng.uniform(-1, 1, conv.dimO).astype(np.float16)
    taps = int(np.prod(TRS))
    assert_fp16_within_ulp(conv.fprop(I, F, alpha=0.5, relu=True, late_loads=True, shuffle=2),
                           orc.ref_conv_fprop(I, F, pad, strd, 0.5, True), 1.0, "fprop", acc_atol(C * taps))
    assert_fp16_within_ulp(conv.bprop(F, E, late_loads=True, shuffle=3),
                           orc.ref_conv_bprop(F, E, conv.dimI, pad, strd), 1.0, "bprop", acc_atol(K * taps))
    assert_fp32_close(conv.update(I, E, late_loads=True, shuffle=4), orc.ref_conv_update(I, E, conv.dimF, pad, strd),
                      1e-5, "update")


POOL_CASES = [  # C, D, H, W, N, JTRS, pad, strides
    (4, 1, 9, 9, 8, (1, 1, 3, 3), (0, 0, 0, 0), (1, 1, 2, 2)),       # overlapping: argmax bytes + gather by cells
    (3, 1, 8, 8, 16, (1, 1, 2, 2), (0, 0, 0, 0), (1, 1, 2, 2)),      # exact tiling: one pass
    (6, 2, 7, 7, 8, (2, 1, 3, 3), (0, 0, 1, 1), (2, 1, 2, 2)),       # feature-map window, padded: generic loops
    (3, 1, 7, 9, 4, (1, 1, 3, 3), (0, 0, 1, 1), (1, 1, 2, 2)),       # four images: scalar path in fp16
]


@pytest.mark.parametrize("case", POOL_CASES)
def test_emulated_pooling(emu, case):
    C, D, H, W, N, JTRS, pad, strd = case
    rng = np.random.default_rng(C + H + N)
    I = rng.uniform(-1, 1, (C, D, H, W, N)).astype(np.float16)
    for op, name in ((0, "max"), (1, "avg"), (2, "l2")):
        O = emu.pool(op, I, JTRS, pad, strd)
        assert_fp16_within_ulp(O, orc.ref_pool_fprop(I, name, JTRS, pad, strd), 1.0, name, 1e-6)
        if name != "l2":
            E = rng.uniform(-1, 1, O.shape).astype(np.float16)
            assert_fp16_within_ulp(emu.pool(op, I, JTRS, pad, strd, E=E), orc.ref_pool_bprop(I, E, name, JTRS, pad, strd),
                                   1.0, name + " bprop", 1e-6)


CANDIDATES = [("fc", {"NG_FC_CFG": "1"}), ("fc", {"NG_FC_CFG": "2"}), ("fc", {"NG_FC_CFG": "3"}),
              ("fc", {"NG_FC_CFG": "7"}), ("fc", {"NG_FC_CFG": "8"}),
              ("nt", {"NG_NT_STREAM": "1"}), ("nt", {"NG_NT_STREAM": "2"}), ("rows", {"NG_CONV_ROWS": "1"}),
              ("strips", {"NG_UPDATE_STRIPS": "1"}), ("stages", {"NG_CONV_STAGES": "3"})]


@pytest.mark.parametrize("what,switch", CANDIDATES)
def test_emulated_candidate_kernels(emu, what, switch):
    """kernels that wait behind environment switches for their first measurement on a device
    (tests/emu/candidates.py): split k-steps inside a workgroup, the streamed outer-product GEMM,
    the first-layer forward with decoded taps, the weight gradient on strips"""
    env = dict(os.environ)
    env.update(switch)
    done = subprocess.run([sys.executable, os.path.join(os.path.dirname(os.path.abspath(__file__)), "emu", "candidates.py"), what],
                          env=env, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, timeout=900)
    assert done.returncode == 0 and b"ok " + what.encode() in done.stdout, done.stdout.decode("utf-8", "replace")[-2000:]
