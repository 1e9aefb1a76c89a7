"""ng_gemm_noalloc (the GEMM entry point that allocates nothing: split partial
sums in a fixed device array of the library image) against ng_gemm given a
caller workspace, both through the C ABI.  Same slicing, same order of
additions: the outputs must be identical bit for bit.  Two calls in a row share
the array, the second one smaller than the first."""
import ctypes

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

vp = ctypes.c_void_p
F16 = 0


def _gemm_pair(ng, lib_mod, op, m, n, k, flags, seed, stream_id, rng, beta=0.0):
    """run the same product through ng_gemm (+workspace) and ng_gemm_noalloc"""
    ta, tb = op[0] == "t", op[1] == "t"
    A = rng.uniform(-1, 1, (k, m) if ta else (m, k)).astype(np.float16)
    B = rng.uniform(-1, 1, (n, k) if tb else (k, n)).astype(np.float16)
    C0 = rng.uniform(-1, 1, (m, n)).astype(np.float16)
    dA, dB = ng.array(A), ng.array(B)
    need = lib_mod.load().ng_gemm_workspace_bytes(F16, ta, tb, m, n, k, 1, 1)
    ws = lib_mod.mem_alloc(need) if need else None
    out = []
    for entry in ("ng_gemm", "ng_gemm_noalloc"):
        dC = ng.array(C0)
        args = [F16, int(ta), int(tb), m, n, k, vp(dA.ptr), A.shape[1], vp(dB.ptr), B.shape[1], vp(dC.ptr), n,
                1.0, beta, flags, seed, stream_id, 1, 0, 0, 0, 1]
        if entry == "ng_gemm":
            args += [vp(int(ws)) if ws else None, need, None]
        else:
            args += [None]
        lib_mod.call(entry, *args)
        out.append(dC.get())
    return need, out[0], out[1], (A.T if ta else A), (B.T if tb else B)


def test_noalloc_matches_workspace_entry_on_two_calls_in_a_row(ng):
    import oracle as orc
    from nervanagpu_amd import _lib
    from util import acc_atol, assert_fp16_within_ulp
    rng = np.random.default_rng(77)
    cap = _lib.load().ng_gemm_static_scratch_bytes()
    assert cap == 32 << 20
    # first the largest minibatch-wide shape (sliced contraction, ~12 MB of
    # partial sums), then a smaller one that reuses the front of the array,
    # then stochastic rounding with beta, then a shape that needs no slices
    cases = [("nn", 4096, 128, 9216, 2, 0.0), ("tn", 4096, 128, 1000, 0, 0.0),
             ("nn", 1000, 128, 4096, 1 | (10 << 16), 0.5), ("nt", 520, 264, 136, 2, 0.0)]
    used_scratch = 0
    for i, (op, m, n, k, flags, beta) in enumerate(cases):
        need, ref_out, got, A, B = _gemm_pair(ng, _lib, op, m, n, k, flags, 5, 40 + i, rng, beta)
        assert need <= cap
        used_scratch += need > 0
        assert np.array_equal(ref_out.view(np.uint16), got.view(np.uint16)), (op, m, n, k)
        if not (flags & 1):
            absdot = np.abs(A.astype(np.float32)) @ np.abs(B.astype(np.float32))
            assert_fp16_within_ulp(got, orc.ref_dot(A, B, relu=bool(flags & 2)), 1.0, "noalloc %s" % op, acc_atol(absdot))
    assert used_scratch >= 3, "the cases were meant to exercise the static scratch"


def test_noalloc_refuses_what_does_not_fit(ng):
    from nervanagpu_amd import _lib
    lib = _lib.load()
    m, n, k = 1664, 1792, 4096
    need = lib.ng_gemm_workspace_bytes(F16, 0, 0, m, n, k, 1, 1)
    assert need > lib.ng_gemm_static_scratch_bytes()
    A = ng.zeros((m, k), dtype=np.float16)
    B = ng.zeros((k, n), dtype=np.float16)
    C = ng.ones((m, n), dtype=np.float16)
    with pytest.raises(_lib.NervanaGPUError, match="static scratch"):
        _lib.call("ng_gemm_noalloc", F16, 0, 0, m, n, k, vp(A.ptr), k, vp(B.ptr), n, vp(C.ptr), n,
                  1.0, 0.0, 0, 0, 0, 1, 0, 0, 0, 1, None)
    assert np.all(C.get() == 1), "a refused call must not touch the output"
