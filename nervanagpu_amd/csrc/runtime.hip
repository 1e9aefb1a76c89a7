// Runtime primitives of the C ABI: device, memory, streams, events, run-time
// compilation and generic launch.  These replace what the reference's host code
// takes from pycuda.driver / pycuda.compiler (nervanagpu/nervanagpu.py:18-21,
// nervanagpu/float_ew.py:1030).
#include "ng_internal.h"

#include <hip/hiprtc.h>

#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <mutex>
#include <string>
#include <vector>

namespace ng {

static thread_local char g_err[1024] = "";

int fail(int code, const char* fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code ? code : -1;
}

int hip_fail(hipError_t e, const char* what)
{
    return fail((int)e, "%s: %s", what, hipGetErrorString(e));
}

static std::mutex g_init_mutex;
static int g_device = -1;
static hipDeviceProp_t g_prop;

int device_cu_count()
{
    return g_device >= 0 ? g_prop.multiProcessorCount : 256;
}

template <typename T>
__global__ void fill_kernel(T* dst, T value, size_t count)
{
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    size_t stride = (size_t)gridDim.x * blockDim.x;
    for (; i < count; i += stride) dst[i] = value;
}

template <typename T>
static int fill(void* dst, T value, size_t count, void* stream)
{
    if (count == 0) return 0;
    if (!dst) return fail(-2, "ng_memset: null destination");
    size_t blocks = (count + 255) / 256;
    if (blocks > 65536) blocks = 65536;
    hipLaunchKernelGGL(fill_kernel<T>, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream,
                       (T*)dst, value, count);
    NG_CHECK_LAUNCH("fill");
    return 0;
}

}  // namespace ng

using namespace ng;

extern "C" {

const char* ng_last_error(void) { return g_err; }

int ng_device_count(int* count)
{
    int c = 0;
    hipError_t e = hipGetDeviceCount(&c);
    if (e != hipSuccess) { *count = 0; return hip_fail(e, "hipGetDeviceCount"); }
    *count = c;
    return 0;
}

int ng_init(int device)
{
    std::lock_guard<std::mutex> lock(g_init_mutex);
    NG_HIP(hipSetDevice(device));
    NG_HIP(hipGetDeviceProperties(&g_prop, device));
    if (strncmp(g_prop.gcnArchName, "gfx950", 6) != 0)
        return fail(-3, "libnervana_hip is built for gfx950 only, device reports %s", g_prop.gcnArchName);
    int rc = gemm_static_scratch_setup(device);
    if (rc) return rc;
    g_device = device;
    return 0;
}

int ng_device_attr(int attr, int* value)
{
    if (g_device < 0) return fail(-4, "ng_init has not been called");
    switch (attr) {
    case 0: *value = g_prop.multiProcessorCount; break;
    case 1: *value = (int)g_prop.sharedMemPerBlock; break;
    case 2: *value = g_prop.warpSize; break;
    case 3: *value = g_prop.clockRate; break;
    case 4: *value = g_prop.memoryClockRate; break;
    case 5: *value = g_prop.l2CacheSize; break;
    default: return fail(-5, "unknown device attribute %d", attr);
    }
    return 0;
}

int ng_device_name(char* buf, size_t cap)
{
    if (g_device < 0) return fail(-4, "ng_init has not been called");
    snprintf(buf, cap, "%s (%s)", g_prop.name, g_prop.gcnArchName);
    return 0;
}

int ng_malloc(void** ptr, size_t bytes)
{
    *ptr = nullptr;
    NG_HIP(hipMalloc(ptr, bytes));
    return 0;
}

int ng_free(void* ptr)
{
    if (ptr) NG_HIP(hipFree(ptr));
    return 0;
}

int ng_mem_info(size_t* free_bytes, size_t* total_bytes)
{
    NG_HIP(hipMemGetInfo(free_bytes, total_bytes));
    return 0;
}

int ng_memcpy_h2d(void* dst, const void* src, size_t bytes, void* stream)
{
    if (!bytes) return 0;
    // pageable source: the copy is staged by the runtime before returning
    NG_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, (hipStream_t)stream));
    NG_HIP(hipStreamSynchronize((hipStream_t)stream));
    return 0;
}

int ng_memcpy_d2h(void* dst, const void* src, size_t bytes, void* stream)
{
    if (!bytes) return 0;
    NG_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, (hipStream_t)stream));
    NG_HIP(hipStreamSynchronize((hipStream_t)stream));
    return 0;
}

int ng_memcpy_d2d(void* dst, const void* src, size_t bytes, void* stream)
{
    if (!bytes) return 0;
    NG_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, (hipStream_t)stream));
    return 0;
}

int ng_memset8(void* dst, unsigned value, size_t count, void* stream)
{
    // widen to 32-bit stores when the range allows it
    if (((uintptr_t)dst & 3) == 0 && (count & 3) == 0) {
        unsigned v = value & 0xFF;
        return fill<unsigned>(dst, v | (v << 8) | (v << 16) | (v << 24), count / 4, stream);
    }
    return fill<unsigned char>(dst, (unsigned char)value, count, stream);
}

int ng_memset16(void* dst, unsigned value, size_t count, void* stream)
{
    if (((uintptr_t)dst & 3) == 0 && (count & 1) == 0) {
        unsigned v = value & 0xFFFF;
        return fill<unsigned>(dst, v | (v << 16), count / 2, stream);
    }
    return fill<unsigned short>(dst, (unsigned short)value, count, stream);
}

int ng_memset32(void* dst, unsigned value, size_t count, void* stream)
{
    return fill<unsigned>(dst, value, count, stream);
}

int ng_stream_create(void** stream)
{
    hipStream_t s;
    NG_HIP(hipStreamCreate(&s));
    *stream = (void*)s;
    return 0;
}

int ng_stream_sync(void* stream)
{
    NG_HIP(hipStreamSynchronize((hipStream_t)stream));
    return 0;
}

int ng_stream_destroy(void* stream)
{
    if (stream) NG_HIP(hipStreamDestroy((hipStream_t)stream));
    return 0;
}

int ng_event_create(void** event)
{
    hipEvent_t e;
    NG_HIP(hipEventCreate(&e));
    *event = (void*)e;
    return 0;
}

int ng_event_record(void* event, void* stream)
{
    NG_HIP(hipEventRecord((hipEvent_t)event, (hipStream_t)stream));
    return 0;
}

int ng_event_sync(void* event)
{
    NG_HIP(hipEventSynchronize((hipEvent_t)event));
    return 0;
}

int ng_event_elapsed_ms(float* ms, void* start, void* end)
{
    NG_HIP(hipEventElapsedTime(ms, (hipEvent_t)start, (hipEvent_t)end));
    return 0;
}

int ng_event_destroy(void* event)
{
    if (event) NG_HIP(hipEventDestroy((hipEvent_t)event));
    return 0;
}

int ng_rtc_compile(const char* source, const char* name,
                   const char** options, int n_options,
                   void** module, char* log, size_t log_cap)
{
    *module = nullptr;
    if (log && log_cap) log[0] = 0;
    hiprtcProgram prog;
    hiprtcResult r = hiprtcCreateProgram(&prog, source, name, 0, nullptr, nullptr);
    if (r != HIPRTC_SUCCESS) return fail(-10, "hiprtcCreateProgram: %s", hiprtcGetErrorString(r));

    std::vector<const char*> opts(options, options + n_options);
    r = hiprtcCompileProgram(prog, (int)opts.size(), opts.data());

    size_t log_size = 0;
    hiprtcGetProgramLogSize(prog, &log_size);
    std::string full_log(log_size, '\0');
    if (log_size) hiprtcGetProgramLog(prog, &full_log[0]);
    if (log && log_cap) {
        strncpy(log, full_log.c_str(), log_cap - 1);
        log[log_cap - 1] = 0;
    }
    if (r != HIPRTC_SUCCESS) {
        hiprtcDestroyProgram(&prog);
        return fail(-11, "hiprtcCompileProgram(%s): %s\n%.700s", name, hiprtcGetErrorString(r), full_log.c_str());
    }
    size_t code_size = 0;
    hiprtcGetCodeSize(prog, &code_size);
    std::vector<char> code(code_size);
    hiprtcGetCode(prog, code.data());
    hiprtcDestroyProgram(&prog);

    hipModule_t mod;
    NG_HIP(hipModuleLoadData(&mod, code.data()));
    *module = (void*)mod;
    return 0;
}

int ng_module_get_function(void** function, void* module, const char* name)
{
    hipFunction_t f;
    NG_HIP(hipModuleGetFunction(&f, (hipModule_t)module, name));
    *function = (void*)f;
    return 0;
}

int ng_module_unload(void* module)
{
    if (module) NG_HIP(hipModuleUnload((hipModule_t)module));
    return 0;
}

int ng_launch(void* function, const unsigned grid[3], const unsigned block[3],
              unsigned shared_bytes, void* stream, void** args)
{
    if (!function) return fail(-12, "ng_launch: null function");
    if (grid[0] == 0 || grid[1] == 0 || grid[2] == 0) return 0;
    if ((size_t)block[0] * block[1] * block[2] > 1024) return fail(-13, "ng_launch: block too large");
    NG_HIP(hipModuleLaunchKernel((hipFunction_t)function, grid[0], grid[1], grid[2],
                                 block[0], block[1], block[2], shared_bytes,
                                 (hipStream_t)stream, args, nullptr));
    return 0;
}

}  // extern "C"
