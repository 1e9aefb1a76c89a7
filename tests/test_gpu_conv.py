"""Convolution fprop / bprop / update parity on the GPU against the numpy
oracle (per-pixel gather + np.dot of benchmarks/conv_test.py:99-167).
Full-tensor comparison at reduced shapes; sampled pixels / filter rows plus
border positions at the configured layer shapes."""
import numpy as np
import pytest

import oracle as orc
from util import acc_atol, assert_fp16_within_ulp, assert_fp32_close, assert_fp32_sum_close

pytestmark = pytest.mark.gpu

# N, C, K, D, H, W, T, R, S, pad(d,h,w), stride(d,h,w)
SMALL = [
    (16, 3, 8, 1, 64, 64, 1, 3, 3, (0, 1, 1), (1, 1, 1)),        # benchmarks/conv_test.py:36-42
    (8, 3, 16, 1, 35, 35, 1, 11, 11, (0, 2, 2), (1, 4, 4)),       # strided, C=3 (AlexNet conv1 style)
    (16, 64, 72, 1, 13, 13, 1, 3, 3, (0, 1, 1), (1, 1, 1)),
    (32, 40, 64, 1, 14, 9, 1, 5, 3, (0, 2, 0), (1, 2, 1)),
    (8, 16, 32, 5, 9, 8, 3, 3, 3, (1, 0, 1), (1, 1, 2)),          # 3-D
    (64, 8, 8, 1, 7, 7, 1, 1, 1, (0, 0, 0), (1, 1, 1)),           # 1x1
    (8, 20, 24, 1, 12, 12, 1, 2, 2, (0, 0, 0), (1, 3, 3)),        # stride > filter: unreached input pixels
    (8, 72, 64, 1, 12, 11, 1, 3, 3, (0, 1, 1), (1, 2, 2)),        # strided, classes * C > 256: one launch per class
    # channel counts that are not multiples of the contraction tile: blocks padded with unread rows
    (16, 96, 112, 1, 9, 9, 1, 3, 3, (0, 1, 1), (1, 1, 1)),
    (16, 144, 48, 1, 7, 7, 1, 1, 1, (0, 0, 0), (1, 1, 1)),        # 1x1 (inception style)
    (8, 96, 112, 1, 11, 10, 1, 3, 3, (0, 1, 1), (1, 2, 2)),       # strided, one launch per class
    (8, 48, 208, 1, 6, 6, 1, 2, 2, (0, 1, 1), (1, 1, 1)),
    # one-dimensional filters with one-sided extents, depth stride with depth padding, a filter as large as the image
    (8, 16, 24, 1, 9, 12, 1, 1, 7, (0, 0, 3), (1, 1, 1)),
    (8, 16, 24, 1, 12, 9, 1, 7, 1, (0, 3, 0), (1, 1, 1)),
    (8, 8, 8, 6, 7, 7, 3, 3, 3, (1, 1, 1), (2, 2, 2)),
    (8, 8, 16, 1, 5, 5, 1, 5, 5, (0, 0, 0), (1, 1, 1)),
    # 64 images, three taps per filter row, unit strides, output rows of a multiple of four pixels:
    # forward runs with the taps of a filter row sharing one activation tile
    (64, 32, 64, 1, 8, 8, 1, 3, 3, (0, 1, 1), (1, 1, 1)),
    (64, 160, 72, 1, 5, 14, 1, 3, 3, (0, 0, 0), (1, 1, 1)),        # no padding, five channel blocks, ragged K
    (64, 32, 32, 4, 6, 8, 2, 3, 3, (1, 1, 1), (1, 1, 1)),          # 3-D
    (64, 64, 136, 1, 5, 8, 1, 1, 3, (0, 0, 1), (1, 1, 1)),         # one filter row
    (64, 32, 16, 1, 4, 4, 1, 3, 3, (0, 1, 3), (1, 1, 1)),          # padding wider than the filter reach
    (32, 32, 128, 2, 5, 8, 2, 3, 3, (1, 1, 1), (1, 1, 1)),         # 32 images: tiles of 128 columns, 3-D
    (32, 64, 136, 1, 6, 12, 1, 3, 3, (0, 1, 1), (1, 1, 1)),        # 32 images, ragged rows
    # output rows of 11 and 23 pixels: forward pads them to 12 and 24 and folds the padding away in the store
    (64, 32, 64, 1, 6, 13, 1, 3, 3, (0, 1, 0), (1, 1, 1)),
    (32, 32, 128, 1, 5, 25, 1, 3, 3, (0, 0, 0), (1, 1, 1)),
    # the data gradient shares taps when the image rows are a multiple of four pixels and the output
    # maps come in blocks of 32 (the taps are mirrored: two-row filter, ragged channel count)
    (64, 72, 96, 1, 5, 12, 1, 3, 3, (0, 0, 0), (1, 1, 1)),
    (64, 40, 32, 1, 4, 4, 1, 2, 3, (0, 1, 3), (1, 1, 1)),
    (64, 32, 64, 3, 4, 8, 3, 2, 3, (2, 0, 1), (1, 1, 1)),          # 3-D, padding only in depth and width
    # very few channels, 64 images, three taps per filter row: the data gradient runs with rows
    # (channel, horizontal tap) over strips of six pixels (ragged last strip, ragged block of output
    # maps, 3-D, no / wide horizontal padding, ten channels = 30 rows)
    (64, 3, 32, 1, 9, 14, 1, 3, 3, (0, 1, 1), (1, 1, 1)),
    (64, 5, 72, 2, 5, 7, 2, 2, 3, (1, 0, 2), (1, 1, 1)),
    (64, 10, 16, 1, 4, 6, 1, 3, 3, (0, 1, 0), (1, 1, 1)),
    # first layers on many pixels: forward keeps the filter in registers and streams the output
    # columns (one to four contraction tiles of 32 rows, strided, ragged last column tile and rows);
    # the thin data gradient streams its halo strips the same way (three and six contraction tiles)
    (8, 3, 24, 1, 95, 97, 1, 3, 3, (0, 1, 1), (1, 1, 1)),
    (16, 4, 16, 1, 66, 64, 1, 3, 3, (0, 1, 1), (1, 1, 1)),
    (16, 3, 16, 1, 131, 131, 1, 5, 5, (0, 2, 2), (1, 2, 2)),
    (16, 3, 8, 1, 70, 70, 1, 6, 6, (0, 2, 2), (1, 1, 1)),
    (64, 3, 64, 1, 20, 80, 1, 3, 3, (0, 1, 1), (1, 1, 1)),
    (64, 5, 32, 1, 24, 72, 1, 3, 3, (0, 1, 1), (1, 1, 1)),
    # 288 column tiles of 256 on a 256-CU chip: the 32 tiles beyond a whole round run as 64x64 tiles in a
    # second launch (forward with 128 output maps; data gradient with 128 channels)
    (64, 32, 128, 1, 36, 32, 1, 3, 3, (0, 1, 1), (1, 1, 1)),
    (64, 128, 32, 1, 36, 32, 1, 3, 3, (0, 1, 1), (1, 1, 1)),
    # 128 images: shared taps with two pixels per 256-column tile (128- and 256-row tiles, forward with
    # 13-pixel output rows padded to 14 and folded, 3-D without horizontal padding, data gradient of 512 channels)
    (128, 32, 128, 1, 6, 8, 1, 3, 3, (0, 1, 1), (1, 1, 1)),
    (128, 32, 128, 1, 5, 13, 1, 3, 3, (0, 1, 1), (1, 1, 1)),
    (128, 64, 160, 2, 5, 8, 2, 3, 3, (1, 0, 0), (1, 1, 1)),
    (128, 32, 512, 1, 10, 14, 1, 3, 3, (0, 1, 1), (1, 1, 1)),
    (128, 512, 32, 1, 10, 14, 1, 3, 3, (0, 1, 1), (1, 1, 1)),
    (128, 64, 32, 1, 4, 13, 1, 3, 3, (0, 1, 1), (1, 1, 1)),          # data gradient with 13-pixel image rows padded to 14
    # the same tail launch on the kernels with separate taps (16 images: forward with 128 output maps,
    # data gradient with 128 channels, 288 column tiles each)
    (16, 64, 128, 1, 64, 72, 1, 3, 3, (0, 1, 1), (1, 1, 1)),
    (16, 128, 64, 1, 64, 72, 1, 3, 3, (0, 1, 1), (1, 1, 1)),
    # weight gradient of three-tap filters with at most 64 output maps: the horizontal taps share a ring of
    # input pixels (192-row workgroups with ragged rows and columns and an odd image width; slices of four
    # positions that cross image rows; the other cases with 64 images, 3x3 filters and K <= 64 take it too)
    (64, 120, 24, 1, 5, 9, 1, 3, 3, (0, 1, 1), (1, 1, 1)),
    (64, 64, 64, 1, 20, 20, 1, 3, 3, (0, 1, 1), (1, 1, 1)),
    # ... and with 65 to 128 output maps on maps of 8192 pixels or more: 128-row workgroups, two column blocks per wavefront
    (64, 128, 72, 1, 91, 91, 1, 1, 3, (0, 0, 1), (1, 1, 1)),
    # two row tiles x 144 column tiles = 288 workgroups: the 32 beyond a whole round leave the main launch as
    # 16 column tiles and run as small tiles behind it (64 and 128 images, forward and data gradient)
    (64, 32, 512, 1, 24, 24, 1, 3, 3, (0, 1, 1), (1, 1, 1)),
    (64, 512, 32, 1, 24, 24, 1, 3, 3, (0, 1, 1), (1, 1, 1)),
    (128, 32, 512, 1, 16, 18, 1, 3, 3, (0, 1, 1), (1, 1, 1)),
    (128, 512, 32, 1, 16, 18, 1, 3, 3, (0, 1, 1), (1, 1, 1)),
    # grids much smaller than the chip with long contractions (7x7 maps): forward and data gradient cut the
    # contraction into slices with fp32 partial sums (blocked and row-by-row forward)
    (16, 128, 128, 1, 7, 7, 1, 3, 3, (0, 1, 1), (1, 1, 1)),
    (16, 24, 64, 1, 7, 7, 1, 5, 5, (0, 2, 2), (1, 1, 1)),
    # long pixel ranges with filter rows in multiples of 192: the weight gradient's 192-row tiles
    (64, 64, 32, 1, 24, 24, 1, 3, 3, (0, 1, 1), (1, 1, 1)),
    (64, 64, 96, 1, 24, 24, 1, 3, 3, (0, 1, 1), (1, 1, 1)),
    # at most 64 channels and 64 output maps on maps of four column tiles per CU or more: the filter stays in
    # registers and the activations stream (forward and data gradient); 64 and 32 channels, whole and partial
    # shares of column tiles per workgroup, no padding (forward only: the data gradient wants W % 4 == 0)
    (64, 64, 64, 1, 64, 64, 1, 3, 3, (0, 1, 1), (1, 1, 1)),
    (64, 32, 32, 1, 40, 104, 1, 3, 3, (0, 1, 1), (1, 1, 1)),
    (64, 64, 48, 1, 66, 66, 1, 3, 3, (0, 0, 0), (1, 1, 1)),
    # 128 rows over a round and a half or more of 512-column tiles (eight pixels per tile), with a tail launch: forward / data gradient
    (64, 32, 128, 1, 80, 80, 1, 3, 3, (0, 1, 1), (1, 1, 1)),
    (64, 128, 32, 1, 80, 80, 1, 3, 3, (0, 1, 1), (1, 1, 1)),
    # 128 rows on the kernels with separate taps (16 images) and more 256-column tiles than CUs: 512-column tiles
    (16, 64, 128, 1, 72, 72, 1, 3, 3, (0, 1, 1), (1, 1, 1)),
    (16, 128, 64, 1, 72, 72, 1, 3, 3, (0, 1, 1), (1, 1, 1)),
    # 192 output maps: the weight gradient's 192-column tiles
    (64, 32, 192, 1, 20, 20, 1, 3, 3, (0, 1, 1), (1, 1, 1)),
    # output maps in multiples of 192 over more than a round of column tiles: 192-row forward tiles
    (16, 64, 192, 1, 80, 80, 1, 3, 3, (0, 1, 1), (1, 1, 1)),
    # ... and the data gradient of at most 32 channels (first layers) as one block of 32 rows, 64 and 32 output maps
    (64, 3, 64, 1, 64, 64, 1, 3, 3, (0, 1, 1), (1, 1, 1)),
    (64, 5, 32, 1, 40, 104, 1, 3, 3, (0, 1, 1), (1, 1, 1)),
    # ... 33 to 64 channels from 32 output maps (64 rows, one block of output maps)
    (64, 48, 32, 1, 64, 64, 1, 3, 3, (0, 1, 1), (1, 1, 1)),
    # forward with shared taps wants channel blocks of 64 (32 channels run row by row): the forward twins of the
    # cases above with 64 channels: plain, folded 13- and 25-pixel rows, main + tail launch with one and two row
    # tiles, 128 images (two-pixel tiles, folded rows, 256-row tiles, tail launch), 512-column tiles
    (64, 64, 72, 1, 8, 8, 1, 3, 3, (0, 1, 1), (1, 1, 1)),
    (64, 64, 64, 1, 6, 13, 1, 3, 3, (0, 1, 0), (1, 1, 1)),
    (32, 64, 128, 1, 5, 25, 1, 3, 3, (0, 0, 0), (1, 1, 1)),
    (64, 64, 128, 1, 36, 32, 1, 3, 3, (0, 1, 1), (1, 1, 1)),
    (64, 64, 512, 1, 24, 24, 1, 3, 3, (0, 1, 1), (1, 1, 1)),
    (128, 64, 128, 1, 6, 8, 1, 3, 3, (0, 1, 1), (1, 1, 1)),
    (128, 64, 128, 1, 5, 13, 1, 3, 3, (0, 1, 1), (1, 1, 1)),
    (128, 64, 512, 1, 10, 14, 1, 3, 3, (0, 1, 1), (1, 1, 1)),
    (128, 64, 512, 1, 16, 18, 1, 3, 3, (0, 1, 1), (1, 1, 1)),
    (64, 64, 128, 1, 80, 80, 1, 3, 3, (0, 1, 1), (1, 1, 1)),
]


def _layer(ng, dtype, case):
    N, C, K, D, H, W, T, R, S, pad, strd = case
    return ng.conv_layer(dtype, N, C, K, D, H, W, T, R, S, pad[0], pad[1], pad[2], strd[0], strd[1], strd[2])


def _data(layer, dtype, seed):
    rng = np.random.default_rng(seed)
    I = rng.uniform(-1, 1, layer.dimI).astype(dtype)
    F = rng.uniform(-1, 1, layer.dimF).astype(dtype)
    E = rng.uniform(-1, 1, layer.dimO).astype(dtype)
    return I, F, E


def _check(out, ref, dtype, what, nterms, abs_sum=None):
    """fp16: one unit in the last place of the fp32-accumulated value; fp32: the
    accumulation bound derived from the sum over absolute operands (abs_sum: a
    callable that evaluates the same op on |operands|), and 1e-5 of the mean
    magnitude for sums of at most 512 terms"""
    if np.dtype(dtype) == np.float16:
        assert_fp16_within_ulp(out, ref, 1.0, what, acc_atol(nterms))
    else:
        assert_fp32_sum_close(out, ref, abs_sum(), nterms, what)


@pytest.mark.parametrize("dtype", [np.float16, np.float32])
@pytest.mark.parametrize("case", SMALL)
def test_conv_small_full_compare(ng, dtype, case):
    layer = _layer(ng, dtype, case)
    I, F, E = _data(layer, dtype, 2)
    dI, dF, dE = ng.array(I, dtype=dtype), ng.array(F, dtype=dtype), ng.array(E, dtype=dtype)
    crst = layer.dimF2[0]

    dO = ng.empty(layer.dimO, dtype=dtype)
    ng.fprop_conv(layer, dI, dF, dO, alpha=1.0)
    aI, aF, aE = np.abs(I), np.abs(F), np.abs(E)
    _check(dO.get(), orc.ref_conv_fprop(I, F, layer.padding, layer.strides), dtype, "fprop", crst,
           lambda: orc.ref_conv_fprop(aI, aF, layer.padding, layer.strides))
    ng.fprop_conv(layer, dI, dF, dO, alpha=0.5, relu=True)
    _check(dO.get(), orc.ref_conv_fprop(I, F, layer.padding, layer.strides, 0.5, True), dtype, "fprop relu", crst,
           lambda: orc.ref_conv_fprop(aI, aF, layer.padding, layer.strides, 0.5))

    dB = ng.empty(layer.dimI, dtype=dtype)
    dB.fill(7)   # every element must be overwritten
    ng.bprop_conv(layer, dF, dE, dB, alpha=1.0)
    krst = layer.K * np.prod(layer.TRS)
    _check(dB.get(), orc.ref_conv_bprop(F, E, layer.dimI, layer.padding, layer.strides), dtype, "bprop", krst,
           lambda: orc.ref_conv_bprop(aF, aE, layer.dimI, layer.padding, layer.strides))

    ref_u = orc.ref_conv_update(I, E, layer.dimF, layer.padding, layer.strides)
    depth = np.prod(layer.MPQ) * layer.N
    dU = ng.empty(layer.dimF, dtype=np.float32)
    ng.update_conv(layer, dI, dE, dU, alpha=1.0)
    assert_fp32_close(dU.get(), ref_u, 1e-5, "update fp32 out")
    if dtype == np.float16:
        dUh = ng.empty(layer.dimF, dtype=np.float16)
        ng.update_conv(layer, dI, dE, dUh, alpha=2.0)
        assert_fp16_within_ulp(dUh.get(), 2 * ref_u, 1.0, "update fp16 out", acc_atol(2 * depth))


def test_conv_uint8_input_bit_exact(ng):
    """bytes are converted exactly on load: the result must equal the run on the
    same values stored as fp16, bit for bit (README.md:37)"""
    case = (16, 3, 16, 1, 31, 31, 1, 5, 5, (0, 2, 2), (1, 2, 2))
    layer = _layer(ng, np.float16, case)
    rng = np.random.default_rng(4)
    I8 = rng.integers(0, 256, layer.dimI).astype(np.uint8)
    F = (rng.standard_normal(layer.dimF) * 0.01).astype(np.float16)
    E = rng.uniform(-1, 1, layer.dimO).astype(np.float16)
    dF, dE = ng.array(F), ng.array(E)
    dI8 = ng.array(I8, dtype=np.uint8)
    dIh = ng.array(I8.astype(np.float16))
    O8, Oh = ng.empty(layer.dimO), ng.empty(layer.dimO)
    ng.fprop_conv(layer, dI8, dF, O8, relu=True)
    ng.fprop_conv(layer, dIh, dF, Oh, relu=True)
    assert np.array_equal(O8.get().view(np.uint16), Oh.get().view(np.uint16))
    assert_fp16_within_ulp(O8.get(), orc.ref_conv_fprop(I8.astype(np.float32), F, layer.padding, layer.strides, 1.0, True),
                           1.0, "u8 fprop", acc_atol(255.0 * 75))
    U8, Uh = ng.empty(layer.dimF, dtype=np.float32), ng.empty(layer.dimF, dtype=np.float32)
    ng.update_conv(layer, dI8, dE, U8)
    ng.update_conv(layer, dIh, dE, Uh)
    assert np.array_equal(U8.get(), Uh.get())
    # signed bytes
    Is8 = rng.integers(-128, 128, layer.dimI).astype(np.int8)
    ng.fprop_conv(layer, ng.array(Is8, dtype=np.int8), dF, O8)
    ng.fprop_conv(layer, ng.array(Is8.astype(np.float16)), dF, Oh)
    assert np.array_equal(O8.get().view(np.uint16), Oh.get().view(np.uint16))
    ng.update_conv(layer, ng.array(Is8, dtype=np.int8), dE, U8)
    ng.update_conv(layer, ng.array(Is8.astype(np.float16)), dE, Uh)
    assert np.array_equal(U8.get(), Uh.get())
    assert_fp32_close(U8.get(), orc.ref_conv_update(Is8.astype(np.float32), E, layer.dimF, layer.padding, layer.strides),
                      1e-5, "i8 update")


def test_conv_adjoint_identity_gpu(ng):
    """<fprop(I,F),E> == <I,bprop(F,E)> == <F,update(I,E)> with fp32 tensors"""
    case = (16, 24, 40, 1, 17, 15, 1, 3, 5, (0, 1, 2), (1, 2, 1))
    layer = _layer(ng, np.float32, case)
    I, F, E = _data(layer, np.float32, 5)
    dI, dF, dE = (ng.array(x, dtype=np.float32) for x in (I, F, E))
    dO, dB, dU = (ng.empty(s, dtype=np.float32) for s in (layer.dimO, layer.dimI, layer.dimF))
    ng.fprop_conv(layer, dI, dF, dO)
    ng.bprop_conv(layer, dF, dE, dB)
    ng.update_conv(layer, dI, dE, dU)
    a = np.vdot(dO.get().astype(np.float64), E)
    b = np.vdot(I, dB.get().astype(np.float64))
    c = np.vdot(F, dU.get().astype(np.float64))
    assert abs(a - b) <= 1e-5 * abs(a) and abs(a - c) <= 1e-5 * abs(a)


ALEXNET = [  # C,H,W,K,R,S,stride,pad at N=128 (benchmark configuration 3)
    (3, 224, 224, 64, 11, 11, 4, 2), (64, 27, 27, 192, 5, 5, 1, 2), (192, 13, 13, 384, 3, 3, 1, 1),
    (384, 13, 13, 256, 3, 3, 1, 1), (256, 13, 13, 256, 3, 3, 1, 1)]
VGG = [  # C,HW,K at N=64, 3x3 s1 p1 (benchmark configuration 4)
    (3, 224, 64), (64, 224, 64), (64, 112, 128), (128, 112, 128), (128, 56, 256), (256, 56, 256),
    (256, 28, 512), (512, 28, 512), (512, 14, 512)]


def _sampled_layer_check(ng, layer, seed, gen, npix=256, nrows=6, in_dtype=np.float16):
    rng = np.random.default_rng(seed)
    I, F, E = gen(rng, layer)
    dI = ng.array(I, dtype=in_dtype)
    dF, dE = ng.array(F), ng.array(E)
    M, P, Q = layer.MPQ
    D, H, W = layer.DHW
    crst = layer.dimF2[0]
    If = I.astype(np.float32)
    scale_i, scale_f, scale_e = np.abs(If).max(), np.abs(F.astype(np.float32)).max(), np.abs(E.astype(np.float32)).max()

    def sample(dims):
        """npix random positions, the corners of the volume, and positions on
        every face (first / last index of one coordinate, the others random):
        the places where padding and ragged tiles show"""
        pts = [tuple(int(rng.integers(0, d)) for d in dims) for _ in range(npix)]
        pts += [tuple(0 for _ in dims), tuple(d - 1 for d in dims), (0, 0, dims[2] - 1), (0, dims[1] - 1, 0),
                (dims[0] - 1, 0, 0), (dims[0] - 1, dims[1] - 1, 0), (dims[0] - 1, 0, dims[2] - 1), (0, dims[1] - 1, dims[2] - 1)]
        for axis in range(3):
            for edge in (0, dims[axis] - 1):
                for _ in range(3):
                    pt = [int(rng.integers(0, d)) for d in dims]
                    pt[axis] = edge
                    pts.append(tuple(pt))
        return sorted(set(pts))

    dO = ng.empty(layer.dimO)
    ng.fprop_conv(layer, dI, dF, dO, relu=True)
    O = dO.get()
    pix = sample((M, P, Q))
    ref = orc.ref_conv_fprop_pixels(If, F, pix, layer.padding, layer.strides, 1.0, True)
    got = np.stack([O[:, m, p, q, :] for (m, p, q) in pix])
    assert_fp16_within_ulp(got, ref, 1.0, "fprop %s" % layer, acc_atol(crst * scale_i * scale_f))
    del O

    if in_dtype == np.float16:
        dB = ng.empty(layer.dimI)
        ng.bprop_conv(layer, dF, dE, dB)
        B = dB.get()
        ipix = sample((D, H, W))
        refb = orc.ref_conv_bprop_pixels(F, E, layer.dimI, ipix, layer.padding, layer.strides)
        gotb = np.stack([B[:, z, y, x, :] for (z, y, x) in ipix])
        assert_fp16_within_ulp(gotb, refb, 1.0, "bprop %s" % layer,
                               acc_atol(layer.K * np.prod(layer.TRS) * scale_f * scale_e))
        del B, dB

    dU = ng.empty(layer.dimF, dtype=np.float32)
    ng.update_conv(layer, dI, dE, dU)
    U = dU.get().reshape(crst, layer.K)
    rows = np.unique(np.concatenate([rng.integers(0, crst, nrows), [0, crst - 1]]))
    refu = orc.ref_conv_update_rows(If, E, layer.dimF, rows, layer.padding, layer.strides)
    assert_fp32_close(U[rows], refu, 1e-5, "update %s" % layer)
    # the same gradient stored as fp16 (nervanagpu/nervanagpu.py:695-698, 723-724: fp32 accumulation, one
    # rounding), at the configured shape: one unit in the last place of the fp32-accumulated value plus
    # the accumulation slack of the sums over the absolute operands
    dUh = ng.empty(layer.dimF, dtype=np.float16)
    ng.update_conv(layer, dI, dE, dUh)
    Uh = dUh.get().reshape(crst, layer.K)
    absu = orc.ref_conv_update_rows(np.abs(If), np.abs(E.astype(np.float32)), layer.dimF, rows, layer.padding, layer.strides)
    assert_fp16_within_ulp(Uh[rows], refu, 1.0, "update (fp16 out) %s" % layer, acc_atol(absu))


def _alexnet_data(rng, layer):
    I = rng.uniform(0, 1, layer.dimI).astype(np.float16)
    F = (rng.standard_normal(layer.dimF) * 0.01).astype(np.float16)
    E = rng.uniform(-1, 1, layer.dimO).astype(np.float16)
    E *= (rng.uniform(0, 1, layer.dimO) > 0.5)           # relu mask
    return I, F, E


@pytest.mark.parametrize("cfg", ALEXNET)
def test_config3_alexnet_layers(ng, cfg):
    C, H, W, K, R, S, strd, pad = cfg
    layer = ng.conv_layer(np.float16, 128, C, K, 1, H, W, 1, R, S, 0, pad, pad, 1, strd, strd)
    _sampled_layer_check(ng, layer, 2, _alexnet_data, npix=256)


def test_config3_first_layer_uint8(ng):
    C, H, W, K, R, S, strd, pad = ALEXNET[0]
    layer = ng.conv_layer(np.float16, 128, C, K, 1, H, W, 1, R, S, 0, pad, pad, 1, strd, strd)

    def gen(rng, layer):
        I = rng.integers(0, 256, layer.dimI).astype(np.uint8)
        F = (rng.standard_normal(layer.dimF) * 0.01).astype(np.float16)
        E = rng.uniform(-1, 1, layer.dimO).astype(np.float16)
        return I, F, E
    _sampled_layer_check(ng, layer, 2, gen, in_dtype=np.uint8)


@pytest.mark.parametrize("cfg", VGG)
def test_config4_vgg_layers(ng, cfg):
    C, HW, K = cfg
    layer = ng.conv_layer(np.float16, 64, C, K, 1, HW, HW, 1, 3, 3, 0, 1, 1, 1, 1, 1)

    def gen(rng, layer):
        I = rng.standard_normal(layer.dimI, dtype=np.float32).astype(np.float16)
        F = (rng.standard_normal(layer.dimF) * np.sqrt(2.0 / (C * 9))).astype(np.float16)
        E = rng.standard_normal(layer.dimO, dtype=np.float32).astype(np.float16)
        return I, F, E
    _sampled_layer_check(ng, layer, 3, gen, npix=256, nrows=4)


def test_config5_conv3d(ng):
    layer = ng.conv_layer(np.float16, 32, 64, 128, 16, 28, 28, 3, 3, 3)
    assert layer.MPQ == (14, 26, 26)

    def gen(rng, layer):
        I = rng.uniform(-1, 1, layer.dimI).astype(np.float16)
        F = (rng.standard_normal(layer.dimF) * 0.05).astype(np.float16)
        E = rng.uniform(-1, 1, layer.dimO).astype(np.float16)
        return I, F, E
    _sampled_layer_check(ng, layer, 4, gen, npix=256, nrows=4)


@pytest.mark.parametrize("dtype", [np.float16, np.float32])
@pytest.mark.parametrize("geom", [(10, 10, 3, 3, 0, 0, 2, 2), (9, 12, 5, 3, 2, 1, 2, 1), (7, 7, 2, 2, 0, 0, 2, 2)])
def test_deconv_layer_ops(ng, dtype, geom):
    """DeconvLayer (nervanagpu/layers.py:509-537) is a ConvLayer whose input extent
    H,W is derived from the wanted P,Q; a deconvolution runs it backwards: its
    forward pass is bprop_conv (K maps of PxQ -> C maps of HxW), its backward pass
    fprop_conv, its weight gradient update_conv.  All three against the oracle."""
    P, Q, R, S, pad_h, pad_w, str_h, str_w = geom
    N, C, K = 16, 24, 32
    layer = ng.deconv_layer(dtype, N, C, K, P, Q, R, S, 0, pad_h, pad_w, 1, str_h, str_w)
    assert layer.MPQ == (1, P, Q)
    assert layer.DHW == (1, (P - 1) * str_h - 2 * pad_h + R, (Q - 1) * str_w - 2 * pad_w + S)
    assert layer.dimO == (K, 1, P, Q, N) and layer.dimF == (C, 1, R, S, K)
    small, F, big = _data(layer, dtype, 41)       # dimI-shaped, filters, dimO-shaped
    dF = ng.array(F, dtype=dtype)
    # forward of the deconvolution: upsample the (K,P,Q) maps to (C,H,W)
    up = ng.empty(layer.dimI, dtype=dtype)
    up.fill(7)
    ng.bprop_conv(layer, dF, ng.array(big, dtype=dtype), up)
    _check(up.get(), orc.ref_conv_bprop(F, big, layer.dimI, layer.padding, layer.strides), dtype, "deconv forward",
           K * R * S, lambda: orc.ref_conv_bprop(np.abs(F), np.abs(big), layer.dimI, layer.padding, layer.strides))
    # backward of the deconvolution: gradient w.r.t. the (K,P,Q) maps
    down = ng.empty(layer.dimO, dtype=dtype)
    ng.fprop_conv(layer, ng.array(small, dtype=dtype), dF, down)
    _check(down.get(), orc.ref_conv_fprop(small, F, layer.padding, layer.strides), dtype, "deconv backward", C * R * S,
           lambda: orc.ref_conv_fprop(np.abs(small), np.abs(F), layer.padding, layer.strides))
    # weight gradient
    dU = ng.empty(layer.dimF, dtype=np.float32)
    ng.update_conv(layer, ng.array(small, dtype=dtype), ng.array(big, dtype=dtype), dU)
    assert_fp32_close(dU.get(), orc.ref_conv_update(small, big, layer.dimF, layer.padding, layer.strides), 1e-5,
                      "deconv update")


def test_deconv_layer_and_errors(ng):
    layer = ng.deconv_layer(np.float16, 16, 8, 16, 10, 12, 3, 3, 0, 1, 1, 1, 2, 2)
    assert layer.MPQ[1:] == (10, 12)
    with pytest.raises(AssertionError):
        ng.conv_layer(np.float16, 12, 3, 8, 1, 8, 8, 1, 3, 3)        # N % 8
    with pytest.raises(AssertionError):
        ng.conv_layer(np.float16, 16, 3, 6, 1, 8, 8, 1, 3, 3)        # K % 8
    small = ng.conv_layer(np.float16, 16, 3, 8, 1, 8, 8, 1, 3, 3)
    with pytest.raises(AssertionError):
        ng.fprop_conv(small, ng.empty((3, 1, 8, 8, 8)), ng.empty(small.dimF), ng.empty(small.dimO))
    with pytest.raises(AssertionError):
        ng.fprop_conv(small, ng.empty(small.dimI), ng.empty(small.dimF, dtype=np.float32), ng.empty(small.dimO))


@pytest.mark.parametrize("dtype", [np.float16, np.float32])
def test_bprop_with_rectifier_mask(ng, dtype):
    """bprop_conv(..., relu_mask=act) = bprop_conv followed by the reference's
    relu derivative step `grad *= act > 0` (nervanagpu/layers.py:89-91), on the
    blocked, the row-by-row and the shared-tap form, full and ragged tiles; strided layers refuse."""
    rng = np.random.default_rng(29)
    for case in (SMALL[0], SMALL[2], SMALL[5], SMALL[8], SMALL[11],
                 (64, 72, 96, 1, 5, 12, 1, 3, 3, (0, 0, 0), (1, 1, 1)),        # shared taps
                 (64, 32, 64, 3, 4, 8, 3, 2, 3, (2, 0, 1), (1, 1, 1)),         # shared taps, 3-D
                 (16, 64, 64, 1, 20, 20, 1, 3, 3, (0, 1, 1), (1, 1, 1)),
                 (64, 128, 32, 1, 36, 32, 1, 3, 3, (0, 1, 1), (1, 1, 1)),      # main launch + tail launch
                 (128, 32, 128, 1, 6, 8, 1, 3, 3, (0, 1, 1), (1, 1, 1)),       # shared taps, 128 images
                 (128, 64, 32, 1, 4, 13, 1, 3, 3, (0, 1, 1), (1, 1, 1)),       # ... with padded image rows
                 (16, 128, 64, 1, 64, 72, 1, 3, 3, (0, 1, 1), (1, 1, 1)),       # separate taps, main + tail launch
                 (16, 128, 128, 1, 7, 7, 1, 3, 3, (0, 1, 1), (1, 1, 1))):       # sliced contraction: the mask is applied by the reduce
        layer = _layer(ng, dtype, case)
        I, F, E = _data(layer, dtype, 31)
        act = np.maximum(rng.standard_normal(layer.dimI), 0).astype(dtype)     # about half zeros
        dF, dE, dA = ng.array(F, dtype=dtype), ng.array(E, dtype=dtype), ng.array(act, dtype=dtype)
        plain, masked = ng.empty(layer.dimI, dtype=dtype), ng.empty(layer.dimI, dtype=dtype)
        ng.bprop_conv(layer, dF, dE, plain)
        masked.fill(7)
        ng.bprop_conv(layer, dF, dE, masked, relu_mask=dA)
        assert np.array_equal(masked.get(), plain.get() * (act > 0)), case
        # a mask with negative entries and negative zeros: only > 0 passes
        act2 = rng.standard_normal(layer.dimI).astype(dtype)
        act2[..., ::3] = -0.0
        dA.set(act2)
        ng.bprop_conv(layer, dF, dE, masked, relu_mask=dA)
        assert np.array_equal(masked.get(), plain.get() * (act2 > 0)), case
    strided = _layer(ng, dtype, SMALL[7])
    I, F, E = _data(strided, dtype, 31)
    out = ng.empty(strided.dimI, dtype=dtype)
    with pytest.raises(Exception):
        ng.bprop_conv(strided, ng.array(F, dtype=dtype), ng.array(E, dtype=dtype), out, relu_mask=ng.empty(strided.dimI, dtype=dtype))
