"""ctypes driver of tests/emu/libnervana_emu.so: the kernel sources compiled for the host and run
lane by lane on the CPU (see shim/hip/hip_runtime.h).  Test infrastructure only."""
import ctypes
import os
import subprocess

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
LIB = os.path.join(HERE, "libnervana_emu.so")
c_int, c_long, c_float, c_uint, c_size_t, c_void_p = (ctypes.c_int, ctypes.c_long, ctypes.c_float, ctypes.c_uint,
                                                       ctypes.c_size_t, ctypes.c_void_p)
NG_F16, NG_F32 = 0, 1
_lib = None


def build():
    subprocess.check_call(["make", "-C", HERE, "-j", "4"], stdout=subprocess.DEVNULL)


def load():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB):
            build()
        _lib = ctypes.CDLL(LIB)
        _lib.ng_last_error.restype = ctypes.c_char_p
        _lib.ng_gemm.argtypes = [c_int] * 6 + [c_void_p, c_int, c_void_p, c_int, c_void_p, c_int, c_float, c_float,
                                              c_uint, c_uint, c_uint, c_int, c_long, c_long, c_long, c_int,
                                              c_void_p, c_size_t, c_void_p]
        _lib.ng_gemm_workspace_bytes.restype = c_size_t
        _lib.ng_gemm_workspace_bytes.argtypes = [c_int] * 8
        _lib.emu_register_buffer.argtypes = [c_void_p, c_size_t]
        _lib.emu_unregister_buffer.argtypes = [c_void_p]
        assert _lib.ng_init(0) == 0, _lib.ng_last_error()
    return _lib


def aligned(shape, dtype, fill=None):
    """numpy array whose data is 256-byte aligned (device allocations are)"""
    n = int(np.prod(shape)) * np.dtype(dtype).itemsize
    raw = np.empty(n + 256, dtype=np.uint8)
    off = (-raw.ctypes.data) % 256
    a = raw[off:off + n].view(dtype).reshape(shape)
    if fill is not None:
        a[...] = fill
    return a


def gemm(A, B, trans_a=False, trans_b=False, alpha=1.0, beta=0.0, relu=False, C=None, sr_bits=0, seed=0, stream=0,
         cus=8, late_loads=False, shuffle=0, workspace=True):
    """C = beta*C + relu(alpha * op(A).op(B)) through the emulated ng_gemm.  A and B are the stored
    matrices (row-major); trans_* say whether the product uses them transposed."""
    lib = load()
    lib.emu_set_cus(cus)
    lib.emu_set_late_loads(1 if late_loads else 0)
    lib.emu_set_shuffle(shuffle)
    dtype = A.dtype
    code = NG_F16 if dtype == np.float16 else NG_F32
    m = A.shape[1] if trans_a else A.shape[0]
    k = A.shape[0] if trans_a else A.shape[1]
    n = B.shape[0] if trans_b else B.shape[1]
    dA, dB = aligned(A.shape, dtype, A), aligned(B.shape, dtype, B)
    dC = aligned((m, n), dtype, C if C is not None else 7)
    need = lib.ng_gemm_workspace_bytes(code, int(trans_a), int(trans_b), m, n, k, 1, 1) if workspace else 0
    ws = aligned((max(need, 16),), np.uint8, 0xAB)
    for buf in (dA, dB, dC, ws):
        lib.emu_register_buffer(buf.ctypes.data, buf.nbytes)
    flags = (1 | (sr_bits << 16) if sr_bits else 0) | (2 if relu else 0)
    try:
        rc = lib.ng_gemm(code, int(trans_a), int(trans_b), m, n, k, dA.ctypes.data, A.shape[1], dB.ctypes.data,
                         B.shape[1], dC.ctypes.data, n, alpha, beta, flags, seed, stream, 1, 0, 0, 0, 1,
                         ws.ctypes.data if need else None, need, None)
        assert rc == 0, lib.ng_last_error()
    finally:
        for buf in (dA, dB, dC, ws):
            lib.emu_unregister_buffer(buf.ctypes.data)
    return np.array(dC)


# ---- convolution and pooling through the emulated ABI ------------------------------------------

class ConvParams(ctypes.Structure):
    _fields_ = [(n, c_int) for n in ("N", "C", "K", "D", "H", "W", "T", "R", "S", "M", "P", "Q",
                                     "pad_d", "pad_h", "pad_w", "str_d", "str_h", "str_w")]


class PoolParams(ctypes.Structure):
    _fields_ = [(n, c_int) for n in ("N", "C", "D", "H", "W", "J", "T", "R", "S", "K", "M", "P", "Q",
                                     "pad_j", "pad_d", "pad_h", "pad_w", "str_j", "str_d", "str_h", "str_w")]


def _configure(cus, late_loads, shuffle):
    lib = load()
    lib.emu_set_cus(cus)
    lib.emu_set_late_loads(1 if late_loads else 0)
    lib.emu_set_shuffle(shuffle)
    return lib


def _out_dim(x, w, pad, strd):
    return -(-(x - w + 1 + 2 * pad) // strd)


class Conv(object):
    """one convolution geometry: N, C, K, (D,H,W), (T,R,S), padding, strides as in ConvLayer"""

    def __init__(self, dtype, N, C, K, DHW, TRS, pad=(0, 0, 0), strd=(1, 1, 1), cus=8):
        lib = _configure(cus, False, 0)
        self.dtype = np.dtype(dtype)
        self.code = NG_F16 if self.dtype == np.float16 else NG_F32
        D, H, W = DHW
        T, R, S = TRS
        M, P, Q = (_out_dim(D, T, pad[0], strd[0]), _out_dim(H, R, pad[1], strd[1]), _out_dim(W, S, pad[2], strd[2]))
        self.p = ConvParams(N, C, K, D, H, W, T, R, S, M, P, Q, pad[0], pad[1], pad[2], strd[0], strd[1], strd[2])
        self.dimI, self.dimF, self.dimO = (C, D, H, W, N), (C, T, R, S, K), (K, M, P, Q, N)
        self.padding, self.strides = tuple(pad), tuple(strd)
        self.plan = c_void_p()
        lib.ng_conv_plan_create.argtypes = [ctypes.POINTER(ConvParams), c_int, ctypes.POINTER(c_void_p)]
        assert lib.ng_conv_plan_create(ctypes.byref(self.p), self.code, ctypes.byref(self.plan)) == 0, lib.ng_last_error()
        lib.ng_conv_plan_workspace_bytes.restype = c_size_t
        lib.ng_conv_plan_workspace_bytes.argtypes = [c_void_p]
        self.ws_bytes = lib.ng_conv_plan_workspace_bytes(self.plan)

    def _run(self, call, tensors, late_loads, shuffle, cus=8):
        lib = _configure(cus, late_loads, shuffle)
        ws = aligned((max(self.ws_bytes, 16),), np.uint8, 0xAB)
        bufs = list(tensors) + [ws]
        for b in bufs:
            lib.emu_register_buffer(b.ctypes.data, b.nbytes)
        try:
            rc = call(lib, ws)
            assert rc == 0, lib.ng_last_error()
        finally:
            for b in bufs:
                lib.emu_unregister_buffer(b.ctypes.data)

    def fprop(self, I, F, alpha=1.0, relu=False, late_loads=False, shuffle=0):
        dI, dF = aligned(I.shape, I.dtype, I), aligned(F.shape, F.dtype, F)
        dO = aligned(self.dimO, self.dtype, 7)
        in_code = {np.dtype(np.float16): NG_F16, np.dtype(np.float32): NG_F32, np.dtype(np.uint8): 2, np.dtype(np.int8): 3}[I.dtype]
        def call(lib, ws):
            lib.ng_conv_fprop.argtypes = [c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_float, c_uint, c_void_p, c_size_t, c_void_p]
            return lib.ng_conv_fprop(self.plan, in_code, dI.ctypes.data, dF.ctypes.data, dO.ctypes.data, alpha,
                                     2 if relu else 0, ws.ctypes.data, self.ws_bytes, None)
        self._run(call, (dI, dF, dO), late_loads, shuffle)
        return np.array(dO)

    def bprop(self, F, E, alpha=1.0, late_loads=False, shuffle=0):
        dF, dE = aligned(F.shape, F.dtype, F), aligned(E.shape, E.dtype, E)
        dB = aligned(self.dimI, self.dtype, 7)
        def call(lib, ws):
            lib.ng_conv_bprop.argtypes = [c_void_p, c_void_p, c_void_p, c_void_p, c_float, c_void_p, c_void_p, c_size_t, c_void_p]
            return lib.ng_conv_bprop(self.plan, dF.ctypes.data, dE.ctypes.data, dB.ctypes.data, alpha, None,
                                     ws.ctypes.data, self.ws_bytes, None)
        self._run(call, (dF, dE, dB), late_loads, shuffle)
        return np.array(dB)

    def update(self, I, E, alpha=1.0, late_loads=False, shuffle=0, cus=8, workspace=True):
        dI, dE = aligned(I.shape, I.dtype, I), aligned(E.shape, E.dtype, E)
        dU = aligned(self.dimF, np.float32, 7)
        def call(lib, ws):
            lib.ng_conv_update.argtypes = [c_void_p, c_int, c_int, c_void_p, c_void_p, c_void_p, c_float, c_void_p, c_size_t, c_void_p]
            return lib.ng_conv_update(self.plan, self.code, NG_F32, dI.ctypes.data, dE.ctypes.data, dU.ctypes.data, alpha,
                                      ws.ctypes.data if workspace else None, self.ws_bytes if workspace else 0, None)
        self._run(call, (dI, dE, dU), late_loads, shuffle, cus)
        return np.array(dU)


def pool(op, I, JTRS, pad=(0, 0, 0, 0), strd=None, E=None, relu_mask=False):
    """fprop (E is None) or bprop of one pooling geometry; op 0 max, 1 avg, 2 l2"""
    lib = _configure(8, False, 0)
    C, D, H, W, N = I.shape
    J, T, R, S = JTRS
    strd = strd or JTRS
    K, M, P, Q = (_out_dim(C, J, pad[0], strd[0]), _out_dim(D, T, pad[1], strd[1]), _out_dim(H, R, pad[2], strd[2]),
                  _out_dim(W, S, pad[3], strd[3]))
    p = PoolParams(N, C, D, H, W, J, T, R, S, K, M, P, Q, pad[0], pad[1], pad[2], pad[3], strd[0], strd[1], strd[2], strd[3])
    code = NG_F16 if I.dtype == np.float16 else NG_F32
    dI = aligned(I.shape, I.dtype, I)
    bufs = [dI]
    if E is None:
        dO = aligned((K, M, P, Q, N), I.dtype, 7)
        bufs.append(dO)
    else:
        dE, dB = aligned(E.shape, E.dtype, E), aligned(I.shape, I.dtype, 7)
        lib.ng_pool_workspace_bytes.restype = c_size_t
        lib.ng_pool_workspace_bytes.argtypes = [ctypes.POINTER(PoolParams), c_int, c_int]
        need = lib.ng_pool_workspace_bytes(ctypes.byref(p), code, op)
        ws = aligned((max(need, 16),), np.uint8, 0xAB)
        bufs += [dE, dB, ws]
    for b in bufs:
        lib.emu_register_buffer(b.ctypes.data, b.nbytes)
    try:
        if E is None:
            lib.ng_pool_fprop.argtypes = [ctypes.POINTER(PoolParams), c_int, c_int, c_void_p, c_void_p, c_void_p]
            rc = lib.ng_pool_fprop(ctypes.byref(p), code, op, dI.ctypes.data, dO.ctypes.data, None)
            out = dO
        else:
            lib.ng_pool_bprop.argtypes = [ctypes.POINTER(PoolParams), c_int, c_int, c_void_p, c_void_p, c_void_p, c_uint,
                                          c_void_p, c_size_t, c_void_p]
            rc = lib.ng_pool_bprop(ctypes.byref(p), code, op, dI.ctypes.data, dE.ctypes.data, dB.ctypes.data,
                                   2 if relu_mask else 0, ws.ctypes.data if need else None, need, None)
            out = dB
        assert rc == 0, lib.ng_last_error()
    finally:
        for b in bufs:
            lib.emu_unregister_buffer(b.ctypes.data)
    return np.array(out)
