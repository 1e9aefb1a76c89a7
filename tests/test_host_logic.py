"""CPU-only tests: the C-ABI library loads and exports every symbol declared in
include/nervana_hip.h, the host-side tensor/view/expression logic, kernel source
generation (compiled for gfx950 with hiprtc, no device needed), layer geometry."""
import os
import re

import numpy as np
import pytest

import oracle as orc
from nervanagpu_amd import GPUTensor, NervanaGPU, _lib, float_ew
from nervanagpu_amd import layers as L
from nervanagpu_amd.nervanagpu import OpTreeNode

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_functions():
    text = open(os.path.join(ROOT, "include", "nervana_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    names = re.findall(r"\b(ng_[a-z0-9_]+|nervana_[A-Za-z_]+)\s*\(", text)
    return sorted(set(n for n in names if not n.endswith("_params")))


def test_library_exports_every_declared_symbol():
    import ctypes
    assert os.path.exists(_lib.LIB_PATH), "build the library first (__graft_entry__.build())"
    lib = ctypes.CDLL(_lib.LIB_PATH)
    declared = declared_functions()
    assert len(declared) >= 45
    for name in declared:
        assert hasattr(lib, name), "missing export " + name
    # and the Python binding covers the same set
    assert sorted(_lib.EXPORTS) == declared
    _lib.load()


def test_no_gpu_means_loud_failure():
    if _lib.device_count() > 0:
        pytest.skip("a GPU is present")
    ng = NervanaGPU()
    with pytest.raises(_lib.NervanaGPUError):
        ng.empty((4, 4))


def test_gemm_workspace_of_the_fully_connected_shapes_fits_the_static_scratch():
    """ng_gemm_workspace_bytes is host arithmetic (no device: 256 CUs assumed).  The minibatch-wide shapes of the
    benchmark (benchmarks/cublas.py:64-71) only fill the chip with their contraction cut into slices; the
    partial sums of every schedule the dispatcher may pick must fit the 32 MiB array that ng_gemm_noalloc and
    the nervana_* entry points use, and an outer product (k = 128) or a chip-filling square needs none."""
    import ctypes
    lib = ctypes.CDLL(_lib.LIB_PATH)
    lib.ng_gemm_workspace_bytes.restype = ctypes.c_size_t
    lib.ng_gemm_workspace_bytes.argtypes = [ctypes.c_int] * 8
    lib.ng_gemm_static_scratch_bytes.restype = ctypes.c_size_t
    cap = lib.ng_gemm_static_scratch_bytes()
    assert cap == 32 << 20
    for (M, K) in ((4096, 9216), (4096, 4096), (1000, 4096)):
        for (ta, m, n, k) in ((0, M, 128, K), (1, K, 128, M)):
            need = lib.ng_gemm_workspace_bytes(0, ta, 0, m, n, k, 1, 1)
            assert 0 < need <= cap, (ta, m, n, k, need)
            assert need % (m * n * 4) == 0 and need // (m * n * 4) >= 2      # whole fp32 slices, at least two
        assert lib.ng_gemm_workspace_bytes(0, 0, 1, M, K, 128, 1, 1) == 0
    assert lib.ng_gemm_workspace_bytes(0, 0, 0, 4096, 4096, 4096, 1, 1) == 0


def fake(ng, shape, dtype=np.float16, addr=0x100000, **kw):
    return GPUTensor(ng, shape, dtype, gpudata=addr, **kw)


def test_views_strides_and_offsets():
    ng = NervanaGPU()
    A = fake(ng, (6, 8, 10), np.float32)
    assert A.strides == (80, 10, 1) and A.is_contiguous and A.nbytes == 1920
    v = A[1:5:2, 3, ::-1]
    assert v.shape == (2, 10) and v.strides == (160, -1)
    assert int(v.gpudata) == 0x100000 + (80 * 1 + 10 * 3 + 9) * 4 and v.base is A
    assert A[..., 2].shape == (6, 8) and A[2, ...].shape == (8, 10)
    assert int(A[-1].gpudata) == 0x100000 + 5 * 80 * 4
    t = fake(ng, (4, 9))
    assert t.T.shape == (9, 4) and t.T.strides == (1, 9) and t.T.is_trans and not t.T.T.is_trans
    b = fake(ng, (3, 4, 9))
    assert b.T.shape == (3, 9, 4) and b.T.strides == (36, 1, 9)     # batched: outer dim kept
    assert t.reshape(6, 6).shape == (6, 6) and t.reshape((36,)).strides == (1,)
    assert t.share((2, 3), dtype=np.float32).dtype == np.float32
    with pytest.raises(TypeError):
        t.T.reshape(6, 6)
    with pytest.raises(IndexError):
        t[1, 2, 3, 4]
    with pytest.raises(IndexError):
        A[..., 1, ...]
    assert len(t) == 4 and isinstance(hash(t), int) and {t: 1}[t] == 1
    assert isinstance(t == t, OpTreeNode)


def test_postfix_stack_and_shape():
    ng = NervanaGPU()
    A, B = fake(ng, (32, 64)), fake(ng, (32, 1), addr=0x200000)
    node = 2.5 * A * B + 1
    stack = node.traverse([])
    ops = [s["op"] if isinstance(s, dict) else s for s in stack]
    assert ops == [2.5, A, "mul", B, "mul", 1, "add"]
    assert OpTreeNode.shape(node) == (32, 64)
    bn = (A - ng.mean(A, axis=1)) / ng.sqrt(ng.var(A, axis=1) + 1e-3)
    names = [s["op"] for s in bn.traverse([]) if isinstance(s, dict)]
    assert names == ["sum", "mul", "sub", "sum", "mul", "sub", "sqr", "sum", "mul", "add", "sqrt", "div"]


def _plan_and_source(out, expr):
    stack = OpTreeNode({"op": "assign"}, out, expr).traverse([])
    plan = float_ew.analyse(stack)
    src, order = float_ew.generate_source(plan.spec, "k")
    _lib.rtc_syntax_check(src, "k")            # compiles for gfx950 without a device
    return plan, src, order


def test_ew_generator_specialisations_compile():
    ng = NervanaGPU()
    A = fake(ng, (4096, 8192), addr=0x10000000)
    B = fake(ng, (4096, 8192), addr=0x20000000)
    C = fake(ng, (4096, 8192), addr=0x30000000, rounding=10)
    plan, src, _ = _plan_and_source(C, A * B + 1.5)
    assert plan.mode == "flat" and plan.vec == 8 and "ng_sr_f16" in src
    # batch norm: row cached in registers, the three reductions collapse into two stages
    plan, src, _ = _plan_and_source(C, (A - ng.mean(A, axis=1)) / ng.sqrt(ng.var(A, axis=1) + 1e-3))
    assert plan.mode == "row" and plan.items > 0 and plan.vec == 8 and plan.n == 8192 and plan.rows == 4096
    assert src.count("__shfl_xor") == 2 and src.count("reinterpret_cast<const vt_*>") == 1   # one read of A
    # axis-0 reduction walks strided columns; output one value per column
    O0 = fake(ng, (1, 8192), np.float32, addr=0x40000000)
    plan, src, _ = _plan_and_source(O0, ng.sum(A, axis=0))
    assert plan.rows == 8192 and plan.n == 4096 and plan.n_out == 1 and plan.vec == 1
    # broadcast of a column and a row vector, int8 output saturates
    col, rowv = fake(ng, (4096, 1), addr=0x50000000), fake(ng, (1, 8192), addr=0x60000000)
    I8 = fake(ng, (4096, 8192), np.int8, addr=0x70000000)
    plan, src, _ = _plan_and_source(I8, A * col + rowv)
    assert plan.mode == "row" and "ng_rint_sat" in src
    # transpose, argmax, rand, unaligned pointer falls back to narrower vectors
    At = fake(ng, (8192, 4096), addr=0x10000000).T
    _plan_and_source(C, At + A)
    Oi = fake(ng, (4096, 1), np.int32, addr=0x80000000)
    _plan_and_source(Oi, ng.argmax(A, axis=1))
    _plan_and_source(C, ng.rand() * A)
    U = fake(ng, (4096, 8192), addr=0x10000002)
    plan, _, _ = _plan_and_source(C, U + 1)
    assert plan.vec == 1
    U4 = fake(ng, (4096, 8192), addr=0x10000008)
    plan, _, _ = _plan_and_source(C, U4 + 1)
    assert plan.vec == 4
    # errors raised before any launch (same exception types as the reference)
    with pytest.raises(ValueError):
        float_ew.analyse(OpTreeNode({"op": "assign"}, C, ng.sum(A, axis=1) + ng.sum(A, axis=0)).traverse([]))
    with pytest.raises(TypeError):
        float_ew.analyse(OpTreeNode({"op": "assign"}, C, A + fake(ng, (4096, 100))).traverse([]))
    with pytest.raises(ValueError):
        float_ew.analyse([C, fake(ng, (2, 3, 4)), fake(ng, (1, 4)), {"op": "add"}, {"op": "assign"}])


def test_fast_ew_dims_and_strides_match_oracle():
    for size in (1024 * 1024, 96, 91, 255 * 7, 4096 * 8192):
        assert float_ew._get_fast_ew_dims(size) == orc.fast_ew_dims(size)


CONV_CFGS = [
    dict(N=128, C=3, K=64, H=224, W=224, R=11, S=11, pad_h=2, pad_w=2, str_h=4, str_w=4),
    dict(N=128, C=64, K=192, H=27, W=27, R=5, S=5, pad_h=2, pad_w=2),
    dict(N=64, C=512, K=512, H=14, W=14, R=3, S=3, pad_h=1, pad_w=1),
    dict(N=32, C=64, K=128, D=16, H=28, W=28, T=3, R=3, S=3),
]


@pytest.mark.parametrize("cfg", CONV_CFGS)
def test_conv_layer_geometry(cfg):
    ng = NervanaGPU()
    layer = ng.conv_layer(np.float16, **cfg)
    D, H, W = layer.DHW
    assert layer.MPQ == orc.conv_out_dims((D, H, W), layer.TRS, layer.padding, layer.strides)
    M, P, Q = layer.MPQ
    assert layer.dimI == (cfg["C"], D, H, W, cfg["N"]) and layer.dimO == (cfg["K"], M, P, Q, cfg["N"])
    assert layer.dimF == (cfg["C"],) + layer.TRS + (cfg["K"],)
    assert layer.flops == 2.0 * M * P * Q * cfg["K"] * cfg["N"] * cfg["C"] * np.prod(layer.TRS)
    assert layer.sizeO == np.prod(layer.dimO) and layer.nOut == M * P * Q * cfg["K"]
    assert layer.dtypeU is np.float32


def test_known_layer_sizes_of_the_configs():
    ng = NervanaGPU()
    p = [ng.conv_layer(np.float16, **c).MPQ[1] for c in CONV_CFGS[:2]]
    assert p == [55, 27]
    assert ng.conv_layer(np.float16, **CONV_CFGS[3]).MPQ == (14, 26, 26)
    flops = [ng.conv_layer(np.float16, **c).flops / 1e9 for c in CONV_CFGS]
    np.testing.assert_allclose(flops, [17.99, 57.33, 59.19, 133.97], rtol=1e-3)
    pool = ng.pool_layer(np.float16, "max", 128, 256, 1, 56, 56, 1, 1, 3, 3, 0, 0, 0, 0, 1, 1, 2, 2)
    assert pool.MPQ == (1, 27, 27) and pool.overlap == 4 and pool.K == 256
    assert (pool.K,) + pool.MPQ == orc.pool_out_dims((256, 1, 56, 56), pool.JTRS, pool.padding, pool.strides)
    dflt = ng.pool_layer(np.float16, "max", 64, 64, 1, 224, 224, 1, 1, 2, 2)
    assert dflt.strides == (1, 1, 2, 2) and dflt.overlap == 0 and dflt.MPQ == (1, 112, 112)
    fc = L.FullLayer(ng, np.float16, 128, 9216, 4096)
    assert fc.flops == 2.0 * 128 * 9216 * 4096 and fc.dimF == (4096, 9216)


def test_layer_create_chain_without_device():
    ng = NervanaGPU()
    confs = [
        {"layer": L.DataLayer, "N": 64, "C": 3, "H": 224, "W": 224},
        {"layer": L.ConvLayer, "common": {"R": 3, "S": 3, "pad_h": 1, "pad_w": 1}, "K": 64},
        {"layer": L.PoolLayer, "op": "max", "R": 2, "S": 2},
        {"layer": L.ConvLayer, "R": 3, "S": 3, "pad_h": 1, "pad_w": 1, "K": 128, np.float16: {"grid_P": 2}},
        {"layer": L.FullLayer, "nOut": 1000},
    ]
    prev, layers = None, []
    for conf in confs:
        prev = L.Layer.create(ng, conf, prev, np.float16)
        layers.append(prev)
    assert layers[1].dimO == (64, 1, 224, 224, 64) and layers[2].dimO == (64, 1, 112, 112, 64)
    assert layers[3].C == 64 and layers[3].grid_P == 2 and layers[4].nIn == 128 * 112 * 112


@pytest.mark.parametrize("nmax,d", [(65535, 7), (3025 * 4, 55), (363, 121), (1 << 20, 1000), (9, 9), (100, 1)])
def test_magic32(nmax, d):
    m, s = L._magic32(nmax, d)
    assert (m, s) == orc.magic32(nmax, d)
    n = np.arange(nmax + 1, dtype=np.uint64)
    assert np.array_equal(n // d, (n * m) >> s)
    assert L._flatten([1, [2, (3, [4])], 5]) == [1, 2, 3, 4, 5]


def test_network_tables_and_flops():
    """host logic only: the four benchmark networks chain their geometry like the
    reference tables (benchmarks/convnet-benchmarks.py:120-200)"""
    from nervanagpu_amd import convnet_benchmarks as cb
    from nervanagpu_amd.layers import Inception
    assert len(cb.network_config("Alexnet")) == 12
    assert len(cb.network_config("VGG")) == 17
    assert len(cb.network_config("VGG_E")) == 25
    assert cb.PUBLISHED_TITAN_X_MS[("VGG", "float16")][2] == 491.382

    # inception modules: output channels are the sum of the branch tails
    def tail_k(conf):
        return [part[-1].get("K") for part in conf["partitions"]]
    g1 = cb.network_config("GoogLeNet1")
    assert len(g1) == 19 and sum(c["layer"] is Inception for c in g1) == 9
    assert sum(tail_k(g1[6])) == 256 and sum(tail_k(g1[7])) == 480 and sum(tail_k(g1[-3])) == 1024
    assert g1[-2]["op"] == "avg" and g1[-2]["R"] == 7 and g1[1]["str_h"] == 2 and g1[1]["pad_h"] == 3
    g2 = cb.network_config("GoogLeNet2")
    assert len(g2) == 20 and sum(c["layer"] is Inception for c in g2) == 10
    assert tail_k(g2[6]) == [64, 64, 96, 32] and [len(p) for p in g2[6]["partitions"]] == [1, 2, 3, 2]
    # a zero width drops the 1x1 branch and the 1x1 after the pool: the pool passes its channels through
    assert tail_k(g2[8]) == [160, 96, None] and g2[8]["partitions"][-1][0]["op"] == "max"
    assert g2[9]["K"] == 576 and g2[9]["R"] == 2 and g2[9]["str_w"] == 2

    # chained through Layer.create: the published GoogLeNet channel / map sizes
    # (http://arxiv.org/abs/1409.4842 table 1)
    ng, prev, widths = NervanaGPU(), None, []
    for conf in g1:
        prev = L.Layer.create(ng, conf, prev, np.float16)
        if type(prev) is Inception:
            widths.append((prev.K, prev.P))
    assert widths == [(256, 28), (480, 28), (512, 14), (512, 14), (512, 14), (528, 14), (832, 14), (832, 7), (1024, 7)]
    assert prev.nIn == 1024 and prev.nOut == 1000
