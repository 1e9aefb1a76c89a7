"""Checks of the candidate kernels that sit behind environment switches until they are measured on a
device (the switches are read once per process, hence this separate script):

    NG_FC_CFG=1..13    minibatch-wide GEMM: workgroups whose wavefront groups split the k-steps of a tile,
                       or that spend a whole CU of LDS on stages of the weight stream
    NG_NT_STREAM=1|2   outer-product GEMM: rows of A resident in registers, output columns streamed
    NG_CONV_ROWS=1     first-layer forward with large filters: taps decoded from the contraction row
    NG_UPDATE_STRIPS=1 weight gradient of 3x3 filters with at most 64 channels and output maps: strips of four
                       output columns, all nine taps on one ring of input pixels

    NG_CONV_STAGES=3   forward / data gradient on 128x256x64 tiles of a grid of at most one workgroup per CU:
                       three LDS stages

usage: python tests/emu/candidates.py fc|nt|rows|strips|stages   (with the switch set in the environment)
Every case runs with loads landing at once and with loads landing as late as the wait counts allow."""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
sys.path.insert(0, os.path.dirname(HERE))
sys.path.insert(0, HERE)

import emu  # noqa: E402
import oracle as orc  # noqa: E402
from util import acc_atol, assert_fp16_within_ulp  # noqa: E402

MODES = ((False, 0), (True, 3))


def fc():
    rng = np.random.default_rng(0)
    for (m, n, k, ta, tb) in [(512, 128, 2048, 0, 0), (456, 72, 1032, 0, 0), (512, 128, 1024, 1, 0), (392, 104, 1992, 1, 0)]:
        A = rng.uniform(-1, 1, (k, m) if ta else (m, k)).astype(np.float16)
        B = rng.uniform(-1, 1, (k, n)).astype(np.float16)
        a = A.T if ta else A
        ref = orc.ref_dot(a, B, relu=True)
        absd = np.abs(a).astype(np.float32) @ np.abs(B).astype(np.float32)
        for late, shuffle in MODES:
            for ws in (True, False):          # sliced with a fixed-order reduce, and unsliced
                got = emu.gemm(A, B, ta, tb, relu=True, late_loads=late, shuffle=shuffle, workspace=ws)
                assert_fp16_within_ulp(got, ref, 1.0, "fc %s" % ((m, n, k, ta, tb, late, ws),), acc_atol(absd))
    # stochastic store of the reduce, bit exact on dyadic operands
    A = (rng.integers(-16, 17, (384, 1024)) / 16.0).astype(np.float16)
    B = (rng.integers(-16, 17, (1024, 128)) / 16.0).astype(np.float16)
    got = emu.gemm(A, B, sr_bits=10, seed=5, stream=2, late_loads=True, shuffle=1)
    r = orc.rand_sr16(5, 2, np.arange(384 * 128, dtype=np.uint32)).reshape(384, 128)
    exp = orc.round_stochastic_fp16(orc.ref_dot(A, B, acc_dtype=np.float32), 10, r)
    assert np.array_equal(got.view(np.uint16), exp.view(np.uint16))


def nt():
    rng = np.random.default_rng(1)
    for (m, n, k) in [(136, 1032, 128), (64, 1024, 64), (200, 1288, 72), (128, 2048, 104)]:
        A = rng.uniform(-1, 1, (m, k)).astype(np.float16)
        B = rng.uniform(-1, 1, (n, k)).astype(np.float16)
        ref = orc.ref_dot(A, B.T, alpha=0.5, relu=True)
        absd = np.abs(A).astype(np.float32) @ np.abs(B.T).astype(np.float32)
        for late, shuffle in MODES:
            got = emu.gemm(A, B, False, True, alpha=0.5, relu=True, late_loads=late, shuffle=shuffle)
            assert_fp16_within_ulp(got, ref, 1.0, "nt %s" % ((m, n, k, late),), acc_atol(absd))
        Ad = (rng.integers(-16, 17, (m, k)) / 16.0).astype(np.float16)
        Bd = (rng.integers(-16, 17, (n, k)) / 16.0).astype(np.float16)
        got = emu.gemm(Ad, Bd, False, True, sr_bits=10, seed=77, stream=5, late_loads=True, shuffle=9)
        r = orc.rand_sr16(77, 5, np.arange(m * n, dtype=np.uint32)).reshape(m, n)
        exp = orc.round_stochastic_fp16(orc.ref_dot(Ad, Bd.T, acc_dtype=np.float32), 10, r)
        assert np.array_equal(got.view(np.uint16), exp.view(np.uint16)), (m, n, k)


def rows():
    rng = np.random.default_rng(2)
    for (N, C, K, DHW, TRS, pad, strd) in [(16, 3, 64, (1, 75, 75), (1, 11, 11), (0, 2, 2), (1, 4, 4)),
                                           (16, 3, 24, (1, 46, 50), (1, 7, 7), (0, 3, 3), (1, 2, 2)),
                                           (8, 3, 40, (2, 40, 45), (2, 5, 5), (1, 0, 2), (1, 1, 1))]:
        conv = emu.Conv(np.float16, N, C, K, DHW, TRS, pad, strd)
        I = rng.uniform(-1, 1, conv.dimI).astype(np.float16)
        F = rng.uniform(-1, 1, conv.dimF).astype(np.float16)
        ref = orc.ref_conv_fprop(I, F, pad, strd, 0.5, True)
        for late, shuffle in MODES:
            got = conv.fprop(I, F, alpha=0.5, relu=True, late_loads=late, shuffle=shuffle)
            assert_fp16_within_ulp(got, ref, 1.0, "rows %s" % ((N, C, K, DHW, TRS, late),), acc_atol(C * np.prod(TRS)))


def strips():
    rng = np.random.default_rng(4)
    # (N, C, K, H, W): widths that are and are not multiples of the strip, fewer channels / maps than 64,
    # one CU (a single slice walks every strip) and eight (slices start inside strips)
    for (N, C, K, H, W, cus) in [(64, 64, 64, 6, 8, 8), (64, 64, 64, 9, 10, 1), (64, 40, 24, 5, 13, 8), (64, 64, 48, 12, 9, 3)]:
        conv = emu.Conv(np.float16, N, C, K, (1, H, W), (1, 3, 3), (0, 1, 1), (1, 1, 1), cus=cus)
        I = rng.uniform(-1, 1, conv.dimI).astype(np.float16)
        E = rng.uniform(-1, 1, conv.dimO).astype(np.float16)
        ref = orc.ref_conv_update(I, E, conv.dimF, (0, 1, 1), (1, 1, 1), 0.25)
        scale = np.abs(ref).mean()
        for late, shuffle in MODES:
            got = conv.update(I, E, alpha=0.25, late_loads=late, shuffle=shuffle, cus=cus)
            err = np.abs(got - ref).max() / scale
            assert err < 2e-5, ("strips", (N, C, K, H, W, cus, late), err)


def stages():
    rng = np.random.default_rng(6)
    # channels in blocks of 32, image rows that do not share taps (14 and 7 pixels), 128-row tiles, at most 8 column tiles
    for (N, C, K, H, W) in [(64, 128, 128, 2, 14), (16, 160, 256, 7, 7)]:
        conv = emu.Conv(np.float16, N, C, K, (1, H, W), (1, 3, 3), (0, 1, 1), (1, 1, 1))
        I = rng.uniform(-1, 1, conv.dimI).astype(np.float16)
        F = rng.uniform(-1, 1, conv.dimF).astype(np.float16)
        E = rng.uniform(-1, 1, conv.dimO).astype(np.float16)
        for late, shuffle in MODES:
            O = conv.fprop(I, F, relu=True, late_loads=late, shuffle=shuffle)
            assert_fp16_within_ulp(O, orc.ref_conv_fprop(I, F, (0, 1, 1), (1, 1, 1), 1.0, True), 1.0, "stages fprop", acc_atol(C * 9))
            B = conv.bprop(F, E, late_loads=late, shuffle=shuffle)
            assert_fp16_within_ulp(B, orc.ref_conv_bprop(F, E, conv.dimI, (0, 1, 1), (1, 1, 1)), 1.0, "stages bprop", acc_atol(K * 9))


if __name__ == "__main__":
    {"fc": fc, "nt": nt, "rows": rows, "strips": strips, "stages": stages}[sys.argv[1]]()
    print("ok", sys.argv[1])
