// Fiber runtime of the lane-level CPU emulation (see shim/hip/hip_runtime.h) and the few
// library-internal functions the kernel translation units expect from runtime.hip.
// One OS thread runs one workgroup at a time; every lane is a ucontext fiber.
#include <hip/hip_runtime.h>

#include <ucontext.h>

#include <cstdarg>
#include <deque>
#include <map>
#include <random>
#include <vector>

#include "ng_internal.h"

namespace emu {

Lane* cur = nullptr;
dim3 g_grid, g_block, g_bidx;

namespace {

constexpr size_t STACK_BYTES = 256 * 1024;

struct PendingLoad { char* dst; bool is_dma; bool zero; unsigned char data[16]; };

struct Wave {
    int live = 0;                 // lanes that have not returned
    int arrived = 0;
    unsigned generation = 0;
    int parity = 0;               // which of the two slot sets the next rendezvous uses
    char slots[2][64 * 64];
};

struct Fiber {
    Lane lane;
    ucontext_t ctx;
    std::vector<char> stack;
    bool done = false;
    std::deque<PendingLoad> vmem;   // per lane, in issue order (all lanes of a wavefront issue alike)
};

ucontext_t g_main;
std::vector<Fiber> g_fibers;
std::vector<Wave> g_waves;
Fiber* g_cur = nullptr;
const std::function<void()>* g_body = nullptr;
int g_wg_live = 0, g_wg_arrived = 0;
unsigned g_wg_generation = 0;
unsigned long g_progress = 0;       // bumped whenever a fiber passes a rendezvous or returns
bool g_late_loads = false;          // LDS-bound loads land only when s_waitcnt covers them
unsigned g_shuffle_seed = 0;        // != 0: fibers are resumed in a shuffled order
int g_cus = 8;

void yield() { swapcontext(&g_cur->ctx, &g_main); }

void apply(const PendingLoad& p)
{
    if (!p.is_dma) return;
    if (p.zero) std::memset(p.dst, 0, 16);
    else std::memcpy(p.dst, p.data, 16);
}

void fiber_entry()
{
    (*g_body)();
    Fiber* f = g_cur;
    for (const PendingLoad& p : f->vmem) apply(p);   // a wavefront's loads land before it ends
    f->vmem.clear();
    f->done = true;
    g_waves[f->lane.wave].live--;
    g_wg_live--;
    g_progress++;
    // a lane that returns may complete a rendezvous the others wait in
    Wave& w = g_waves[f->lane.wave];
    if (w.live > 0 && w.arrived == w.live) { w.arrived = 0; w.generation++; w.parity ^= 1; }
    if (g_wg_live > 0 && g_wg_arrived == g_wg_live) { g_wg_arrived = 0; g_wg_generation++; }
    swapcontext(&f->ctx, &g_main);
}

}  // namespace

void wg_sync()
{
    const unsigned gen = g_wg_generation;
    if (++g_wg_arrived == g_wg_live) { g_wg_arrived = 0; g_wg_generation++; g_progress++; return; }
    while (g_wg_generation == gen) yield();
    g_progress++;
}

char* wave_exchange_begin()
{
    Wave& w = g_waves[cur->wave];
    return w.slots[w.parity];
}

void wave_exchange_sync()
{
    Wave& w = g_waves[cur->wave];
    const unsigned gen = w.generation;
    if (++w.arrived == w.live) { w.arrived = 0; w.generation++; w.parity ^= 1; g_progress++; return; }
    while (w.generation == gen) yield();
    g_progress++;
}

void vmem_issue(char* lds_dst, const void* src16)
{
    PendingLoad p;
    p.dst = lds_dst; p.is_dma = true; p.zero = src16 == nullptr;
    if (src16) std::memcpy(p.data, src16, 16);
    if (g_late_loads) g_cur->vmem.push_back(p);
    else { apply(p); p.is_dma = false; g_cur->vmem.push_back(p); }
}

void vmem_issue_plain()
{
    PendingLoad p;
    p.dst = nullptr; p.is_dma = false; p.zero = false;
    g_cur->vmem.push_back(p);
}

void vmem_wait(int outstanding)
{
    std::deque<PendingLoad>& q = g_cur->vmem;
    while ((int)q.size() > outstanding) { apply(q.front()); q.pop_front(); }
}

void launch(dim3 grid, dim3 block, const std::function<void()>& body, const char* name)
{
    const int nthreads = (int)(block.x * block.y * block.z);
    const int nwaves = (nthreads + 63) / 64;
    g_grid = grid; g_block = block;
    g_body = &body;
    static const bool trace = std::getenv("EMU_TRACE") != nullptr;
    if (trace) std::fprintf(stderr, "emu: launch grid (%u,%u,%u) block %u  %.400s\n", grid.x, grid.y, grid.z, block.x, name ? name : "");
    std::mt19937 rng(g_shuffle_seed);
    std::vector<int> order(nthreads);
    for (unsigned bz = 0; bz < grid.z; bz++)
        for (unsigned by = 0; by < grid.y; by++)
            for (unsigned bx = 0; bx < grid.x; bx++) {
                g_bidx = dim3(bx, by, bz);
                if ((int)g_fibers.size() != nthreads) g_fibers = std::vector<Fiber>(nthreads);
                g_waves.assign(nwaves, Wave());
                g_wg_live = nthreads; g_wg_arrived = 0;
                for (int t = 0; t < nthreads; t++) {
                    Fiber& f = g_fibers[t];
                    f.lane.tid = dim3((unsigned)t % block.x, ((unsigned)t / block.x) % block.y, (unsigned)t / (block.x * block.y));
                    f.lane.lane = t & 63; f.lane.wave = t >> 6;
                    f.done = false; f.vmem.clear();
                    if (f.stack.empty()) f.stack.resize(STACK_BYTES);
                    getcontext(&f.ctx);
                    f.ctx.uc_stack.ss_sp = f.stack.data();
                    f.ctx.uc_stack.ss_size = f.stack.size();
                    f.ctx.uc_link = &g_main;
                    makecontext(&f.ctx, fiber_entry, 0);
                    g_waves[t >> 6].live++;
                    order[t] = t;
                }
                while (g_wg_live > 0) {
                    if (g_shuffle_seed) {
                        // whole wavefronts in a shuffled order, and the lanes inside each
                        std::shuffle(order.begin(), order.end(), rng);
                    }
                    const unsigned long before = g_progress;
                    for (int idx : order) {
                        Fiber& f = g_fibers[idx];
                        if (f.done) continue;
                        g_cur = &f; cur = &f.lane;
                        swapcontext(&g_main, &f.ctx);
                    }
                    if (g_progress == before && g_wg_live > 0) {
                        std::fprintf(stderr, "emu: deadlock in workgroup (%u,%u,%u): %d lanes alive, %d at the workgroup barrier\n",
                                     bx, by, bz, g_wg_live, g_wg_arrived);
                        std::abort();
                    }
                }
            }
    g_body = nullptr; g_cur = nullptr; cur = nullptr;
}

}  // namespace emu

// ---- registered buffers: every global access of a kernel must fall inside one -------------
static std::map<uintptr_t, size_t> g_buffers;
static bool g_check_access = true;

void emu_check_access(const void* p, size_t bytes, const char* what)
{
    if (!g_check_access || g_buffers.empty()) return;
    const uintptr_t a = (uintptr_t)p;
    auto it = g_buffers.upper_bound(a);
    if (it != g_buffers.begin()) {
        --it;
        if (a >= it->first && a + bytes <= it->first + it->second) return;
    }
    std::fprintf(stderr, "emu: %s at %p (%zu bytes) is outside every registered buffer (workgroup %u,%u,%u thread %u)\n",
                 what, p, bytes, emu::g_bidx.x, emu::g_bidx.y, emu::g_bidx.z, emu::cur ? emu::cur->tid.x : 0u);
    std::abort();
}

void* emu_alloc(size_t bytes)
{
    void* p = nullptr;
    if (posix_memalign(&p, 256, bytes ? bytes : 256)) return nullptr;
    g_buffers[(uintptr_t)p] = bytes;
    return p;
}

void emu_free(void* p)
{
    if (!p) return;
    g_buffers.erase((uintptr_t)p);
    std::free(p);
}

// ---- what the kernel translation units expect from runtime.hip --------------------------------
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
int hip_fail(hipError_t e, const char* what) { return fail((int)e ? (int)e : -1, "%s: emulated runtime error", what); }
int device_cu_count() { return emu::g_cus; }

}  // namespace ng

// ---- run-time compilation: the host compiler against the same stand-in headers --------------
#include <dlfcn.h>
#include <unistd.h>

#include <regex>
#include <string>

namespace {

struct EmuModule { void* handle; std::string dir; };

std::string this_library()
{
    Dl_info info;
    if (dladdr((void*)&this_library, &info) && info.dli_fname) return info.dli_fname;
    return "libnervana_emu.so";
}

std::string shim_dir()
{
    const std::string so = this_library();
    const size_t slash = so.find_last_of('/');
    return (slash == std::string::npos ? std::string(".") : so.substr(0, slash)) + "/shim";
}

// `extern "C" __global__ ... void NAME(T0 a0, T1 a1, ...)` -> a trampoline NAME__emu(void** args)
// that unpacks the argument block of ng_launch (pointers to the values, as hipModuleLaunchKernel takes)
std::string trampolines(const std::string& src)
{
    std::string out;
    std::regex head(R"(extern\s+"C"\s+__global__[\s\S]*?void\s+(\w+)\s*\(([^\)]*)\))");
    for (std::sregex_iterator it(src.begin(), src.end(), head), end; it != end; ++it) {
        const std::string name = (*it)[1], params = (*it)[2];
        std::vector<std::string> types;
        size_t pos = 0;
        while (pos < params.size()) {
            size_t comma = params.find(',', pos);
            if (comma == std::string::npos) comma = params.size();
            std::string p = params.substr(pos, comma - pos);
            pos = comma + 1;
            // drop the parameter name (the last identifier)
            size_t e = p.find_last_not_of(" \t\n");
            if (e == std::string::npos) continue;
            size_t b = e;
            while (b > 0 && (std::isalnum((unsigned char)p[b - 1]) || p[b - 1] == '_')) b--;
            std::string type = p.substr(0, b);
            type = std::regex_replace(type, std::regex("__restrict__"), "");
            types.push_back(type);
        }
        out += "extern \"C\" void " + name + "__emu(void** args)\n{\n    " + name + "(";
        for (size_t i = 0; i < types.size(); i++)
            out += (i ? ", " : "") + std::string("*(") + types[i] + "*)args[" + std::to_string(i) + "]";
        out += ");\n}\n";
    }
    return out;
}

}  // namespace

extern "C" {

const char* ng_last_error(void) { return ng::g_err; }
int ng_init(int device) { return ng::gemm_static_scratch_setup(device); }

int ng_device_count(int* count) { *count = 1; return 0; }
int ng_device_attr(int attr, int* value)
{
    switch (attr) {
    case 0: *value = emu::g_cus; break;
    case 1: *value = 160 * 1024; break;
    case 2: *value = 64; break;
    case 3: *value = 2400000; break;
    case 4: *value = 2000000; break;
    case 5: *value = 4 << 20; break;
    default: return ng::fail(-5, "unknown device attribute %d", attr);
    }
    return 0;
}
int ng_device_name(char* buf, size_t cap) { snprintf(buf, cap, "lane-level CPU emulation (gfx950 kernels)"); return 0; }
int ng_malloc(void** ptr, size_t bytes) { *ptr = emu_alloc(bytes); return *ptr ? 0 : ng::fail(-6, "out of memory"); }
int ng_free(void* ptr) { emu_free(ptr); return 0; }
int ng_mem_info(size_t* free_bytes, size_t* total_bytes) { *free_bytes = *total_bytes = (size_t)8 << 30; return 0; }
int ng_memcpy_h2d(void* dst, const void* src, size_t bytes, void*) { std::memcpy(dst, src, bytes); return 0; }
int ng_memcpy_d2h(void* dst, const void* src, size_t bytes, void*) { std::memcpy(dst, src, bytes); return 0; }
int ng_memcpy_d2d(void* dst, const void* src, size_t bytes, void*) { std::memmove(dst, src, bytes); return 0; }
int ng_memset8(void* dst, unsigned value, size_t count, void*) { std::memset(dst, (int)(value & 0xFF), count); return 0; }
int ng_memset16(void* dst, unsigned value, size_t count, void*)
{
    unsigned short* p = (unsigned short*)dst;
    for (size_t i = 0; i < count; i++) p[i] = (unsigned short)value;
    return 0;
}
int ng_memset32(void* dst, unsigned value, size_t count, void*)
{
    unsigned* p = (unsigned*)dst;
    for (size_t i = 0; i < count; i++) p[i] = value;
    return 0;
}
int ng_stream_create(void** stream) { *stream = nullptr; return 0; }
int ng_stream_sync(void*) { return 0; }
int ng_stream_destroy(void*) { return 0; }
int ng_event_create(void** event) { *event = (void*)1; return 0; }
int ng_event_record(void*, void*) { return 0; }
int ng_event_sync(void*) { return 0; }
int ng_event_elapsed_ms(float* ms, void*, void*) { *ms = 1.0f; return 0; }
int ng_event_destroy(void*) { return 0; }

int ng_rtc_compile(const char* source, const char* name, const char** /*options*/, int /*n_options*/,
                   void** module, char* log, size_t log_cap)
{
    *module = nullptr;
    if (log && log_cap) log[0] = 0;
    char tmpl[] = "/tmp/ng_emu_rtc_XXXXXX";
    if (!mkdtemp(tmpl)) return ng::fail(-10, "mkdtemp failed");
    const std::string dir(tmpl), cpp = dir + "/k.cpp", so = dir + "/k.so", err = dir + "/err.txt";
    {
        std::string text = std::string("#include <hip/hip_runtime.h>\n") + source + "\n" + trampolines(source);
        FILE* f = fopen(cpp.c_str(), "w");
        if (!f) return ng::fail(-10, "cannot write %s", cpp.c_str());
        fwrite(text.data(), 1, text.size(), f);
        fclose(f);
    }
    const std::string cmd = "/opt/rocm/llvm/bin/clang++ -std=c++17 -O1 -fPIC -shared -ffp-contract=off -I " + shim_dir() +
                            " -Wno-psabi -Wno-unused-value -Wno-ignored-attributes -Wno-macro-redefined -x c++ " + cpp + " -x none " + this_library() +
                            " -o " + so +
                            " 2> " + err;
    const int rc = system(cmd.c_str());
    if (rc != 0) {
        std::string msg;
        if (FILE* f = fopen(err.c_str(), "r")) { char buf[2048]; size_t n = fread(buf, 1, sizeof(buf) - 1, f); buf[n] = 0; msg = buf; fclose(f); }
        if (log && log_cap) { strncpy(log, msg.c_str(), log_cap - 1); log[log_cap - 1] = 0; }
        return ng::fail(-11, "host compile of %s failed:\n%.700s", name, msg.c_str());
    }
    // the module finds emu::* and the other runtime symbols in this library (already loaded, global)
    void* h = dlopen(so.c_str(), RTLD_NOW | RTLD_LOCAL);
    if (!h) return ng::fail(-11, "dlopen(%s): %s", so.c_str(), dlerror());
    *module = new EmuModule{h, dir};
    return 0;
}

int ng_module_get_function(void** function, void* module, const char* name)
{
    EmuModule* m = (EmuModule*)module;
    void* f = dlsym(m->handle, (std::string(name) + "__emu").c_str());
    if (!f) return ng::fail(-12, "kernel %s not found in the emulated module", name);
    *function = f;
    return 0;
}

int ng_module_unload(void* module)
{
    EmuModule* m = (EmuModule*)module;
    if (m) { dlclose(m->handle); delete m; }
    return 0;
}

int ng_launch(void* function, const unsigned grid[3], const unsigned block[3], unsigned /*shared_bytes*/, void* /*stream*/,
              void** args)
{
    if (!function) return ng::fail(-12, "ng_launch: null function");
    if (grid[0] == 0 || grid[1] == 0 || grid[2] == 0) return 0;
    if ((size_t)block[0] * block[1] * block[2] > 1024) return ng::fail(-13, "ng_launch: block too large");
    void (*tramp)(void**) = (void (*)(void**))function;
    emu::launch(dim3(grid[0], grid[1], grid[2]), dim3(block[0], block[1], block[2]), [=]() { tramp(args); });
    return 0;
}


// controls of the emulation
void emu_set_cus(int cus) { emu::g_cus = cus; }
void emu_set_late_loads(int late) { emu::g_late_loads = late != 0; }
void emu_set_shuffle(unsigned seed) { emu::g_shuffle_seed = seed; }
void emu_register_buffer(const void* p, size_t bytes) { g_buffers[(uintptr_t)p] = bytes; }
void emu_unregister_buffer(const void* p) { g_buffers.erase((uintptr_t)p); }

}  // extern "C"
