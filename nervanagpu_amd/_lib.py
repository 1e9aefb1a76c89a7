"""
ctypes binding of libnervana_hip.so (the C ABI declared in include/nervana_hip.h).

This module is the only place that touches the shared library.  It replaces
what the reference imports from pycuda (nervanagpu/nervanagpu.py:18-21).  There
is no CPU fallback: if the library is missing or no gfx950 device is present,
every device call raises NervanaGPUError.
"""
import ctypes
import os
import threading
from ctypes import (POINTER, c_bool, c_char_p, c_float, c_int, c_long, c_size_t,
                    c_uint, c_void_p)

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libnervana_hip.so")
COMMON_HEADER = os.path.join(_HERE, "csrc", "ng_device_common.h")

NG_F16, NG_F32, NG_U8, NG_I8 = 0, 1, 2, 3
FLAG_SR, FLAG_RELU = 1, 2


class NervanaGPUError(RuntimeError):
    """Raised for any failing call into the HIP library (pycuda's drv.Error)."""


class ConvParams(ctypes.Structure):
    _fields_ = [(n, c_int) for n in (
        "N", "C", "K", "D", "H", "W", "T", "R", "S", "M", "P", "Q",
        "pad_d", "pad_h", "pad_w", "str_d", "str_h", "str_w")]


class PoolParams(ctypes.Structure):
    _fields_ = [(n, c_int) for n in (
        "N", "C", "D", "H", "W", "J", "T", "R", "S", "K", "M", "P", "Q",
        "pad_j", "pad_d", "pad_h", "pad_w", "str_j", "str_d", "str_h", "str_w")]


# name -> (restype, argtypes); every int-returning entry is status-checked
_SIGNATURES = {
    "ng_init": (c_int, [c_int]),
    "ng_device_count": (c_int, [POINTER(c_int)]),
    "ng_device_attr": (c_int, [c_int, POINTER(c_int)]),
    "ng_device_name": (c_int, [c_char_p, c_size_t]),
    "ng_last_error": (c_char_p, []),
    "ng_malloc": (c_int, [POINTER(c_void_p), c_size_t]),
    "ng_free": (c_int, [c_void_p]),
    "ng_mem_info": (c_int, [POINTER(c_size_t), POINTER(c_size_t)]),
    "ng_memcpy_h2d": (c_int, [c_void_p, c_void_p, c_size_t, c_void_p]),
    "ng_memcpy_d2h": (c_int, [c_void_p, c_void_p, c_size_t, c_void_p]),
    "ng_memcpy_d2d": (c_int, [c_void_p, c_void_p, c_size_t, c_void_p]),
    "ng_memset8": (c_int, [c_void_p, c_uint, c_size_t, c_void_p]),
    "ng_memset16": (c_int, [c_void_p, c_uint, c_size_t, c_void_p]),
    "ng_memset32": (c_int, [c_void_p, c_uint, c_size_t, c_void_p]),
    "ng_stream_create": (c_int, [POINTER(c_void_p)]),
    "ng_stream_sync": (c_int, [c_void_p]),
    "ng_stream_destroy": (c_int, [c_void_p]),
    "ng_event_create": (c_int, [POINTER(c_void_p)]),
    "ng_event_record": (c_int, [c_void_p, c_void_p]),
    "ng_event_sync": (c_int, [c_void_p]),
    "ng_event_elapsed_ms": (c_int, [POINTER(c_float), c_void_p, c_void_p]),
    "ng_event_destroy": (c_int, [c_void_p]),
    "ng_rtc_compile": (c_int, [c_char_p, c_char_p, POINTER(c_char_p), c_int,
                               POINTER(c_void_p), c_char_p, c_size_t]),
    "ng_module_get_function": (c_int, [POINTER(c_void_p), c_void_p, c_char_p]),
    "ng_module_unload": (c_int, [c_void_p]),
    "ng_launch": (c_int, [c_void_p, POINTER(c_uint), POINTER(c_uint), c_uint, c_void_p,
                          POINTER(c_void_p)]),
    "ng_gemm": (c_int, [c_int, c_int, c_int, c_int, c_int, c_int,
                        c_void_p, c_int, c_void_p, c_int, c_void_p, c_int,
                        c_float, c_float, c_uint, c_uint, c_uint,
                        c_int, c_long, c_long, c_long, c_int,
                        c_void_p, c_size_t, c_void_p]),
    "ng_gemm_workspace_bytes": (c_size_t, [c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int]),
    "ng_gemm_static_scratch_bytes": (c_size_t, []),
    "ng_gemm_noalloc": (c_int, [c_int, c_int, c_int, c_int, c_int, c_int,
                                c_void_p, c_int, c_void_p, c_int, c_void_p, c_int,
                                c_float, c_float, c_uint, c_uint, c_uint,
                                c_int, c_long, c_long, c_long, c_int, c_void_p]),
    "nervana_loadKernels": (c_bool, [c_char_p]),
    "nervana_unloadKernels": (c_bool, []),
    "nervana_randStateSizeBytes": (c_size_t, []),
    "nervana_sgemm": (c_bool, [c_void_p, c_void_p, c_void_p, c_bool, c_bool, c_int, c_int, c_int,
                               c_int, c_int, c_int, c_float, c_float, c_void_p, c_bool, c_bool,
                               c_void_p, c_int]),
    "nervana_hgemm": (c_bool, [c_void_p, c_void_p, c_void_p, c_bool, c_bool, c_int, c_int, c_int,
                               c_int, c_int, c_int, c_float, c_float, c_void_p, c_bool, c_bool,
                               c_void_p, c_int]),
    "nervana_sgemm_colmajor": (c_bool, [c_void_p, c_void_p, c_void_p, c_bool, c_bool, c_int, c_int,
                                        c_int, c_int, c_int, c_int, c_float, c_float, c_void_p,
                                        c_bool, c_bool, c_void_p, c_int]),
    "nervana_hgemm_colmajor": (c_bool, [c_void_p, c_void_p, c_void_p, c_bool, c_bool, c_int, c_int,
                                        c_int, c_int, c_int, c_int, c_float, c_float, c_void_p,
                                        c_bool, c_bool, c_void_p, c_int]),
    "ng_conv_plan_create": (c_int, [POINTER(ConvParams), c_int, POINTER(c_void_p)]),
    "ng_conv_plan_destroy": (c_int, [c_void_p]),
    "ng_conv_plan_workspace_bytes": (c_size_t, [c_void_p]),
    "ng_conv_fprop": (c_int, [c_void_p, c_int, c_void_p, c_void_p, c_void_p,
                              c_float, c_uint, c_void_p, c_size_t, c_void_p]),
    "ng_conv_bprop": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p,
                              c_float, c_void_p, c_void_p, c_size_t, c_void_p]),
    "ng_conv_update": (c_int, [c_void_p, c_int, c_int, c_void_p, c_void_p, c_void_p,
                               c_float, c_void_p, c_size_t, c_void_p]),
    "ng_pool_fprop": (c_int, [POINTER(PoolParams), c_int, c_int, c_void_p, c_void_p, c_void_p]),
    "ng_pool_workspace_bytes": (c_size_t, [POINTER(PoolParams), c_int, c_int]),
    "ng_pool_bprop": (c_int, [POINTER(PoolParams), c_int, c_int, c_void_p, c_void_p, c_void_p, c_uint,
                              c_void_p, c_size_t, c_void_p]),
    "ng_transpose": (c_int, [c_int, c_void_p, c_void_p, c_int, c_int, c_void_p]),
    "ng_dimshuffle": (c_int, [c_int, c_void_p, c_void_p, c_int, c_int, c_int, c_void_p]),
    "ng_fp32_convert": (c_int, [c_int, c_void_p, c_void_p, c_size_t, c_void_p]),
}

EXPORTS = tuple(_SIGNATURES)

_lib = None
_lock = threading.Lock()
_initialised_device = None


def load():
    """dlopen the library (no device call is made)."""
    global _lib
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is not None:
            return _lib
        if not os.path.exists(LIB_PATH):
            raise NervanaGPUError(
                "%s not found: build it with `python -c 'import __graft_entry__ as g; g.build()'` "
                "or `make -C nervanagpu_amd/csrc`" % LIB_PATH)
        lib = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in _SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype = res
            fn.argtypes = args
        _lib = lib
    return _lib


def check(status):
    if status != 0:
        msg = load().ng_last_error()
        raise NervanaGPUError("%s (status %d)" % (msg.decode("utf-8", "replace") if msg else "?", status))


def call(name, *args):
    """Invoke a status-returning entry point and raise on failure."""
    check(getattr(load(), name)(*args))


def device_count():
    n = c_int(0)
    try:
        st = load().ng_device_count(ctypes.byref(n))
    except NervanaGPUError:
        return 0
    return n.value if st == 0 else 0


_default_device = 0


def set_default_device(device):
    """device used by the lazy initialisation (NervanaGPU(device=...))"""
    global _default_device
    _default_device = int(device)


def init(device=None):
    """Lazy device initialisation (replaces `import pycuda.autoinit`); raises
    NervanaGPUError when the library or a gfx950 device is missing."""
    global _initialised_device
    if device is None:
        device = _default_device
    if _initialised_device == device:
        return
    call("ng_init", device)
    _initialised_device = device


def device_attr(attr):
    init()
    v = c_int(0)
    call("ng_device_attr", attr, ctypes.byref(v))
    return v.value


def device_name():
    init()
    buf = ctypes.create_string_buffer(256)
    call("ng_device_name", buf, 256)
    return buf.value.decode()


class DeviceAllocation(object):
    """Owning device buffer (pycuda's DeviceAllocation): int() gives the address,
    memory is released when the object is collected."""

    __slots__ = ("ptr", "nbytes", "__weakref__")

    def __init__(self, nbytes):
        init()
        p = c_void_p()
        call("ng_malloc", ctypes.byref(p), max(int(nbytes), 1))
        self.ptr = p.value
        self.nbytes = int(nbytes)

    def __int__(self):
        return self.ptr

    def __index__(self):
        return self.ptr

    def free(self):
        if self.ptr:
            lib = _lib
            if lib is not None:
                lib.ng_free(c_void_p(self.ptr))
            self.ptr = 0

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


def mem_alloc(nbytes):
    return DeviceAllocation(nbytes)


def memcpy_htod(dst, host_array, stream=None):
    call("ng_memcpy_h2d", c_void_p(int(dst)), host_array.ctypes.data_as(c_void_p),
         host_array.nbytes, stream)


def memcpy_dtoh(host_array, src, stream=None):
    call("ng_memcpy_d2h", host_array.ctypes.data_as(c_void_p), c_void_p(int(src)),
         host_array.nbytes, stream)


def memcpy_dtod(dst, src, nbytes, stream=None):
    call("ng_memcpy_d2d", c_void_p(int(dst)), c_void_p(int(src)), nbytes, stream)


def memset(dst, value_bits, count, itemsize, stream=None):
    name = {1: "ng_memset8", 2: "ng_memset16", 4: "ng_memset32"}[itemsize]
    call(name, c_void_p(int(dst)), value_bits, count, stream)


def stream_sync(stream=None):
    call("ng_stream_sync", stream)


class Event(object):
    """drv.Event: record / synchronize / time_since (milliseconds)."""

    def __init__(self):
        init()
        e = c_void_p()
        call("ng_event_create", ctypes.byref(e))
        self.handle = e

    def record(self, stream=None):
        call("ng_event_record", self.handle, stream)
        return self

    def synchronize(self):
        call("ng_event_sync", self.handle)
        return self

    def time_since(self, start):
        ms = c_float(0)
        call("ng_event_elapsed_ms", ctypes.byref(ms), start.handle, self.handle)
        return ms.value

    def __del__(self):
        try:
            if _lib is not None and self.handle:
                _lib.ng_event_destroy(self.handle)
        except Exception:
            pass


_RTC_OPTIONS = [b"--offload-arch=gfx950", b"-O3", b"-ffp-contract=off", b"-std=c++17",
                b"-Xclang", b"-target-feature", b"-Xclang", b"-packed-fp32-ops"]


class Function(object):
    """A kernel of a run-time compiled module (pycuda Function after prepare())."""

    def __init__(self, module, handle, name):
        self.module = module
        self.handle = handle
        self.name = name

    def launch(self, grid, block, stream, args, shared_bytes=0):
        """args: list of ctypes scalars (c_void_p / c_int / c_float / c_uint)."""
        n = len(args)
        ptrs = (c_void_p * n)(*[ctypes.cast(ctypes.pointer(a), c_void_p) for a in args])
        g = (c_uint * 3)(*grid)
        b = (c_uint * 3)(*block)
        call("ng_launch", self.handle, g, b, shared_bytes, stream, ptrs)


class Module(object):
    """pycuda.compiler.SourceModule on hiprtc."""

    def __init__(self, source, name="ew_kernel", require_device=True):
        if require_device:
            init()
        opts = (c_char_p * len(_RTC_OPTIONS))(*_RTC_OPTIONS)
        log = ctypes.create_string_buffer(16384)
        mod = c_void_p()
        self.source = source
        call("ng_rtc_compile", source.encode(), (name + ".hip").encode(), opts, len(_RTC_OPTIONS),
             ctypes.byref(mod), log, len(log))
        self.handle = mod
        self.log = log.value.decode("utf-8", "replace")

    def get_function(self, name):
        f = c_void_p()
        call("ng_module_get_function", ctypes.byref(f), self.handle, name.encode())
        return Function(self, f, name)


def rtc_syntax_check(source, name="check"):
    """Compile `source` for gfx950 without loading it (works without a GPU).
    Returns the compiler log; raises NervanaGPUError if compilation fails."""
    rtc = ctypes.CDLL("libhiprtc.so")
    prog = c_void_p()
    rtc.hiprtcCreateProgram.argtypes = [POINTER(c_void_p), c_char_p, c_char_p, c_int, c_void_p, c_void_p]
    if rtc.hiprtcCreateProgram(ctypes.byref(prog), source.encode(), (name + ".hip").encode(), 0, None, None):
        raise NervanaGPUError("hiprtcCreateProgram failed")
    opts = (c_char_p * len(_RTC_OPTIONS))(*_RTC_OPTIONS)
    rtc.hiprtcCompileProgram.argtypes = [c_void_p, c_int, POINTER(c_char_p)]
    rc = rtc.hiprtcCompileProgram(prog, len(_RTC_OPTIONS), opts)
    size = c_size_t()
    rtc.hiprtcGetProgramLogSize.argtypes = [c_void_p, POINTER(c_size_t)]
    rtc.hiprtcGetProgramLogSize(prog, ctypes.byref(size))
    log = ctypes.create_string_buffer(size.value + 1)
    rtc.hiprtcGetProgramLog.argtypes = [c_void_p, c_char_p]
    rtc.hiprtcGetProgramLog(prog, log)
    rtc.hiprtcDestroyProgram.argtypes = [POINTER(c_void_p)]
    rtc.hiprtcDestroyProgram(ctypes.byref(prog))
    text = log.value.decode("utf-8", "replace")
    if rc != 0:
        raise NervanaGPUError("hiprtc compile failed:\n" + text)
    return text


def common_header_text():
    with open(COMMON_HEADER) as f:
        return f.read()
