// libdlgrad_hip.so -- device layer under dlgrad's `device="hip"` runtime.
//
// Host C++ plus one device-side object, the static scratch array of the allocation-free
// reduction (no kernels live here: they arrive as HIP source strings from
// dlgrad_amd/codegen/hip_kernel.py and are compiled by hiprtc for gfx950).
// Implements include/dlgrad_hip.h: a size-bucketed caching allocator over
// hipMalloc, synchronous transfers, hiprtc compile, code-object load, kernel
// launch from a packed argument block, events and error strings.
//
// One device, one default-priority stream, one process.  The allocator hands a
// freed block to the next request of the same bucket without waiting for the
// GPU: that is safe because every consumer of the block was enqueued on the
// same stream before the free and every producer is enqueued after it.

#include "../../include/dlgrad_hip.h"

#include <hip/hip_runtime.h>
#include <hip/hiprtc.h>

#include <atomic>
#include <cstddef>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <map>
#include <mutex>
#include <string>
#include <unordered_map>
#include <vector>

// Partial results of dlg_hip_reduce_full_static: one float per block of the first stage.  Device
// memory that belongs to the library's code object; every GPU the library is loaded on holds its
// own copy until the process ends.  Host code never uses this name as an address: the device
// address is looked up once per device (dlg_hip_init) and kept in g_scratch_ptr.
static __device__ __align__(256) unsigned char scratch[DLG_HIP_STATIC_SCRATCH_BYTES];

namespace {

constexpr int kMaxDevices = 64;
void *g_scratch_ptr[kMaxDevices] = {};            // device address of `scratch`, per device

thread_local std::string g_err;
thread_local std::string g_log;

std::mutex g_mu;
bool g_inited = false;
int g_device = -1;
hipStream_t g_stream = nullptr;

struct Kernel {
    hipModule_t module;
    hipFunction_t fn;
};
std::vector<Kernel> g_kernels;                   // handle = index + 1
std::vector<hipModule_t> g_modules;

// ---- allocator state --------------------------------------------------------
// Arena 0 is the ordinary pool.  Other arenas are private pools for captured graphs: a
// block handed out while an arena is current returns to that arena when freed and is
// never given to anybody else, because a graph replays writes to its addresses.
struct Block { size_t bucket; uint64_t arena; void *base; };
// Large blocks are handed out at base + colour * 4 KiB, colour cycling 0..3 from one large allocation
// to the next.  Driver allocations of this size all start on the same multi-MiB alignment, so element i
// of two operands of an element-wise kernel falls on the same DRAM channel and bank at the same moment;
// 4 KiB between them is worth 5 % of a 16384x8192 add (6.26 -> 6.60 TB/s, measured over the offsets 0..1 MiB).
constexpr size_t kStaggerMin = size_t(8) << 20, kStagger = 4096, kColours = 4;
unsigned g_colour = 0;
std::map<uint64_t, std::map<size_t, std::vector<void *>>> g_free;   // arena -> bucket -> cached blocks
std::unordered_map<void *, Block> g_live;                            // block -> bucket, arena
std::map<uint64_t, bool> g_arena_alive;                              // arenas that still exist
struct Usage { size_t live = 0, peak = 0; };                         // blocks of one bucket of one arena: in use now, most at once
std::map<uint64_t, std::map<size_t, Usage>> g_usage;                 // arena (never 0) -> bucket -> usage
uint64_t g_arena = 0, g_next_arena = 1;
uint64_t g_bytes_in_use = 0, g_bytes_cached = 0, g_device_allocs = 0;
std::atomic<bool> g_capturing{false};                            // read by calls that refuse to run inside a capture
std::map<void *, size_t> g_pinned;                                   // page-locked host blocks handed out
std::vector<hipGraphExec_t> g_graphs;                                // handle = index + 1 (null once destroyed)
std::vector<hipEvent_t> g_events;                                    // handle = index + 1 (null once destroyed)

int fail(const char *what, hipError_t e) {
    char buf[512];
    std::snprintf(buf, sizeof buf, "%s: %s (%d)", what, hipGetErrorString(e), (int)e);
    g_err = buf;
    return -(int)e - 1000;
}
int fail_msg(int code, const std::string &msg) {
    g_err = msg;
    return code;
}
#define HIP_TRY(expr)                                   \
    do {                                                \
        hipError_t e__ = (expr);                        \
        if (e__ != hipSuccess) return fail(#expr, e__); \
    } while (0)

#define NEED_INIT()                                                          \
    do {                                                                     \
        if (!g_inited) return fail_msg(-2, "dlg_hip_init has not succeeded"); \
    } while (0)

size_t bucket_of(size_t n) {
    if (n < 256) n = 256;
    if (n <= (size_t(1) << 20)) {             // up to 1 MiB: next power of two
        size_t b = 256;
        while (b < n) b <<= 1;
        return b;
    }
    const size_t mib = size_t(1) << 20;       // above: whole MiB
    return (n + mib - 1) / mib * mib;
}

void trim_arena_locked(uint64_t arena) {
    auto it = g_free.find(arena);
    if (it == g_free.end()) return;
    for (auto &kv : it->second)
        for (void *p : kv.second) {
            (void)hipFree(p);
            g_bytes_cached -= kv.first;
        }
    g_free.erase(it);
}

void trim_locked() {                              // the ordinary pool only: graph arenas keep their blocks
    trim_arena_locked(0);
}

int alloc_locked(size_t nbytes, void **out) {
    const bool stagger = nbytes >= kStaggerMin;
    size_t b = bucket_of(stagger ? nbytes + (kColours - 1) * kStagger : nbytes);
    auto &lists = g_free[g_arena];
    auto it = lists.find(b);
    if (it != lists.end() && !it->second.empty()) {
        *out = it->second.back();
        it->second.pop_back();
        g_bytes_cached -= b;
    } else {
        if (g_capturing) {                    // a device allocation (and the wait of its retry) is no part of a graph:
            *out = nullptr;                   // the step being captured must find every block in its arena
            char buf[256];
            std::snprintf(buf, sizeof buf,
                          "allocation of %zu bytes missed the arena during a capture: run the step once inside the "
                          "arena first, with the same shapes", nbytes);
            return fail_msg(-9, buf);
        }
        void *p = nullptr;
        hipError_t e = hipMalloc(&p, b);
        if (e != hipSuccess) {                // give cached blocks back and retry once
            (void)hipGetLastError();
            (void)hipStreamSynchronize(g_stream);
            trim_locked();
            e = hipMalloc(&p, b);
        }
        if (e != hipSuccess || p == nullptr) {
            (void)hipGetLastError();
            *out = nullptr;
            char buf[160];
            std::snprintf(buf, sizeof buf, "Failed to allocate %zu bytes of device memory", nbytes);
            return fail_msg(-3, buf);
        }
        ++g_device_allocs;
        *out = p;
    }
    void *base = *out;
    if (stagger) *out = static_cast<char *>(base) + (g_colour++ % kColours) * kStagger;
    g_live[*out] = Block{b, g_arena, base};
    g_bytes_in_use += b;
    if (g_arena != 0) {
        Usage &u = g_usage[g_arena][b];
        if (++u.live > u.peak) u.peak = u.live;
    }
    return 0;
}

}  // namespace

extern "C" {

const char *dlg_hip_last_error(void) { return g_err.c_str(); }
const char *dlg_hip_compile_log(void) { return g_log.c_str(); }

int dlg_hip_device_count(int *count) {
    if (!count) return fail_msg(-1, "count is NULL");
    *count = 0;
    hipError_t e = hipGetDeviceCount(count);
    if (e != hipSuccess) {
        *count = 0;
        return fail("hipGetDeviceCount", e);
    }
    return 0;
}

int dlg_hip_init(int device) {
    std::lock_guard<std::mutex> lk(g_mu);
    if (g_inited) {
        if (device == g_device) return 0;
        return fail_msg(-4, "already initialised on another device");
    }
    int n = 0;
    hipError_t e = hipGetDeviceCount(&n);
    if (e != hipSuccess || n <= 0) {
        (void)hipGetLastError();
        return fail_msg(-5, "no HIP device available");
    }
    if (device < 0 || device >= n) return fail_msg(-6, "device index out of range");
    if (device >= kMaxDevices) return fail_msg(-6, "device index out of range");
    HIP_TRY(hipSetDevice(device));
    {                                             // with this device current: where its copy of `scratch` lives
        void *p = nullptr;
        HIP_TRY(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
        if (!p) return fail_msg(-40, "hipGetSymbolAddress returned no address for the static scratch array");
        g_scratch_ptr[device] = p;
    }
    HIP_TRY(hipStreamCreateWithFlags(&g_stream, hipStreamNonBlocking));
    g_device = device;
    g_inited = true;
    return 0;
}

int dlg_hip_shutdown(void) {
    std::lock_guard<std::mutex> lk(g_mu);
    if (!g_inited) return 0;
    (void)hipStreamSynchronize(g_stream);
    for (hipGraphExec_t ge : g_graphs) if (ge) (void)hipGraphExecDestroy(ge);
    g_graphs.clear();
    for (hipEvent_t ev : g_events) if (ev) (void)hipEventDestroy(ev);
    g_events.clear();
    while (!g_free.empty()) trim_arena_locked(g_free.begin()->first);
    g_arena = 0;
    g_capturing = false;
    for (auto &kv : g_pinned) (void)hipHostFree(kv.first);
    g_pinned.clear();
    for (hipModule_t m : g_modules) (void)hipModuleUnload(m);
    g_modules.clear();
    g_kernels.clear();
    (void)hipStreamDestroy(g_stream);
    g_stream = nullptr;
    g_inited = false;
    g_device = -1;
    return 0;
}

int dlg_hip_props(dlg_hip_props_t *out) {
    NEED_INIT();
    if (!out) return fail_msg(-1, "out is NULL");
    hipDeviceProp_t p;
    HIP_TRY(hipGetDeviceProperties(&p, g_device));
    std::memset(out, 0, sizeof *out);
    std::snprintf(out->name, sizeof out->name, "%s", p.name);
    if (!out->name[0]) {                          // some driver stacks leave the property empty: ask by name, then fall back to the arch
        char nm[128] = {0};
        if (hipDeviceGetName(nm, sizeof nm, g_device) == hipSuccess && nm[0]) std::snprintf(out->name, sizeof out->name, "%s", nm);
        else std::snprintf(out->name, sizeof out->name, "%s", p.gcnArchName);
        (void)hipGetLastError();
    }
    std::snprintf(out->arch, sizeof out->arch, "%s", p.gcnArchName);
    out->compute_units = p.multiProcessorCount;
    out->wavefront_size = p.warpSize;
    out->clock_khz = p.clockRate;
    out->mem_clock_khz = p.memoryClockRate;
    out->mem_bus_bits = p.memoryBusWidth;
    out->lds_bytes = (int32_t)p.sharedMemPerBlock;
    out->l2_bytes = p.l2CacheSize;
    out->total_mem = p.totalGlobalMem;
    return 0;
}

// ---- memory -------------------------------------------------------------------

int dlg_hip_alloc(size_t nbytes, void **out) {
    NEED_INIT();
    if (!out) return fail_msg(-1, "out is NULL");
    std::lock_guard<std::mutex> lk(g_mu);
    return alloc_locked(nbytes, out);
}

int dlg_hip_alloc_zero(size_t nbytes, void **out) {
    NEED_INIT();
    if (!out) return fail_msg(-1, "out is NULL");
    if (g_capturing) return fail_msg(-9, "dlg_hip_alloc_zero records a memset node; clear with a kernel while capturing");
    {
        std::lock_guard<std::mutex> lk(g_mu);
        int rc = alloc_locked(nbytes, out);
        if (rc) return rc;
    }
    if (nbytes) HIP_TRY(hipMemsetAsync(*out, 0, nbytes, g_stream));
    return 0;
}

int dlg_hip_fill_f32(void *dst, float value, size_t count) {
    NEED_INIT();
    if (!count) return 0;
    if (g_capturing) return fail_msg(-9, "dlg_hip_fill_f32 records a memset node; fill with a kernel while capturing");
    uint32_t bits;
    std::memcpy(&bits, &value, 4);
    HIP_TRY(hipMemsetD32Async((hipDeviceptr_t)dst, (int)bits, count, g_stream));
    return 0;
}

int dlg_hip_free(void *ptr) {
    if (!ptr) return 0;
    std::lock_guard<std::mutex> lk(g_mu);
    if (!g_inited) return 0;                  // after shutdown the driver owns nothing
    auto it = g_live.find(ptr);
    if (it == g_live.end()) return fail_msg(-7, "dlg_hip_free: pointer was not allocated here");
    Block blk = it->second;
    g_live.erase(it);
    g_bytes_in_use -= blk.bucket;
    if (blk.arena != 0) {
        auto ua = g_usage.find(blk.arena);
        if (ua != g_usage.end()) {
            auto ub = ua->second.find(blk.bucket);
            if (ub != ua->second.end() && ub->second.live) --ub->second.live;
        }
    }
    if (blk.arena != 0 && !g_arena_alive[blk.arena]) {      // its graph is gone: give the memory back
        (void)hipFree(blk.base);
        return 0;
    }
    g_free[blk.arena][blk.bucket].push_back(blk.base);
    g_bytes_cached += blk.bucket;
    return 0;
}

int dlg_hip_pool_stats(uint64_t *in_use, uint64_t *cached, uint64_t *n_allocs) {
    std::lock_guard<std::mutex> lk(g_mu);
    if (in_use) *in_use = g_bytes_in_use;
    if (cached) *cached = g_bytes_cached;
    if (n_allocs) *n_allocs = g_device_allocs;
    return 0;
}

int dlg_hip_pool_trim(void) {
    NEED_INIT();
    HIP_TRY(hipStreamSynchronize(g_stream));
    std::lock_guard<std::mutex> lk(g_mu);
    trim_locked();
    return 0;
}

// ---- transfers ------------------------------------------------------------------

int dlg_hip_h2d(void *dst, const void *src, size_t n) {
    NEED_INIT();
    if (!n) return 0;
    if (g_capturing) return fail_msg(-9, "dlg_hip_h2d is a synchronous transfer and cannot be part of a captured graph");
    HIP_TRY(hipMemcpyAsync(dst, src, n, hipMemcpyHostToDevice, g_stream));
    HIP_TRY(hipStreamSynchronize(g_stream));
    return 0;
}

int dlg_hip_d2h(void *dst, const void *src, size_t n) {
    NEED_INIT();
    if (!n) return 0;
    if (g_capturing) return fail_msg(-9, "dlg_hip_d2h is a synchronous transfer and cannot be part of a captured graph");
    HIP_TRY(hipMemcpyAsync(dst, src, n, hipMemcpyDeviceToHost, g_stream));
    HIP_TRY(hipStreamSynchronize(g_stream));
    return 0;
}

int dlg_hip_d2d(void *dst, const void *src, size_t n) {
    NEED_INIT();
    if (!n) return 0;
    HIP_TRY(hipMemcpyAsync(dst, src, n, hipMemcpyDeviceToDevice, g_stream));
    return 0;
}

// ---- pinned staging ---------------------------------------------------------------

int dlg_hip_host_alloc(size_t nbytes, void **out) {
    NEED_INIT();
    if (!out) return fail_msg(-1, "out is NULL");
    *out = nullptr;
    void *p = nullptr;
    hipError_t e = hipHostMalloc(&p, nbytes ? nbytes : 1, hipHostMallocDefault);
    if (e != hipSuccess || !p) {
        (void)hipGetLastError();
        char buf[160];
        std::snprintf(buf, sizeof buf, "Failed to allocate %zu bytes of pinned host memory", nbytes);
        return fail_msg(-3, buf);
    }
    std::lock_guard<std::mutex> lk(g_mu);
    g_pinned[p] = nbytes;
    *out = p;
    return 0;
}

int dlg_hip_host_free(void *ptr) {
    if (!ptr) return 0;
    {
        std::lock_guard<std::mutex> lk(g_mu);
        if (!g_inited) return 0;
        auto it = g_pinned.find(ptr);
        if (it == g_pinned.end()) return fail_msg(-7, "dlg_hip_host_free: pointer was not allocated here");
        g_pinned.erase(it);
    }
    (void)hipStreamSynchronize(g_stream);        // a copy out of it may still be queued
    HIP_TRY(hipHostFree(ptr));
    return 0;
}

int dlg_hip_h2d_async(void *dst, const void *src, size_t n) {
    NEED_INIT();
    if (!n) return 0;
    {                                            // pageable memory would make this copy synchronous or unsafe
        std::lock_guard<std::mutex> lk(g_mu);
        bool ok = false;
        for (const auto &kv : g_pinned) {
            const char *b = (const char *)kv.first;
            if ((const char *)src >= b && (const char *)src + n <= b + kv.second) { ok = true; break; }
        }
        if (!ok) return fail_msg(-8, "dlg_hip_h2d_async: the source is not inside a dlg_hip_host_alloc block");
    }
    HIP_TRY(hipMemcpyAsync(dst, src, n, hipMemcpyHostToDevice, g_stream));
    return 0;
}

// ---- kernels ----------------------------------------------------------------------

int dlg_hip_compile(const char *source, const char *name, const char *const *options,
                    int n_options, void **code, size_t *code_size) {
    if (!source || !code || !code_size) return fail_msg(-1, "NULL argument");
    *code = nullptr;
    *code_size = 0;
    g_log.clear();
    hiprtcProgram prog;
    hiprtcResult r = hiprtcCreateProgram(&prog, source, name ? name : "kernel.hip", 0, nullptr, nullptr);
    if (r != HIPRTC_SUCCESS)
        return fail_msg(-10, std::string("hiprtcCreateProgram: ") + hiprtcGetErrorString(r));
    r = hiprtcCompileProgram(prog, n_options, const_cast<const char **>(options));
    size_t log_size = 0;
    if (hiprtcGetProgramLogSize(prog, &log_size) == HIPRTC_SUCCESS && log_size > 1) {
        g_log.resize(log_size);
        (void)hiprtcGetProgramLog(prog, &g_log[0]);
    }
    if (r != HIPRTC_SUCCESS) {
        (void)hiprtcDestroyProgram(&prog);
        return fail_msg(-11, std::string("Compilation failed: ") + hiprtcGetErrorString(r));
    }
    size_t sz = 0;
    r = hiprtcGetCodeSize(prog, &sz);
    if (r != HIPRTC_SUCCESS || sz == 0) {
        (void)hiprtcDestroyProgram(&prog);
        return fail_msg(-12, "hiprtcGetCodeSize failed");
    }
    void *buf = std::malloc(sz);
    if (!buf) {
        (void)hiprtcDestroyProgram(&prog);
        return fail_msg(-13, "out of host memory for code object");
    }
    r = hiprtcGetCode(prog, (char *)buf);
    (void)hiprtcDestroyProgram(&prog);
    if (r != HIPRTC_SUCCESS) {
        std::free(buf);
        return fail_msg(-14, "hiprtcGetCode failed");
    }
    *code = buf;
    *code_size = sz;
    return 0;
}

int dlg_hip_code_free(void *code) {
    std::free(code);
    return 0;
}

int dlg_hip_module_load(const void *code, size_t code_size, const char *kernel_name,
                        uint64_t *handle) {
    NEED_INIT();
    if (!code || !code_size || !kernel_name || !handle) return fail_msg(-1, "NULL argument");
    hipModule_t mod;
    HIP_TRY(hipModuleLoadData(&mod, code));
    hipFunction_t fn;
    hipError_t e = hipModuleGetFunction(&fn, mod, kernel_name);
    if (e != hipSuccess) {
        (void)hipModuleUnload(mod);
        return fail(kernel_name, e);
    }
    std::lock_guard<std::mutex> lk(g_mu);
    g_modules.push_back(mod);
    g_kernels.push_back({mod, fn});
    *handle = (uint64_t)g_kernels.size();
    return 0;
}

int dlg_hip_launch(uint64_t handle, uint32_t gx, uint32_t gy, uint32_t gz, uint32_t bx,
                   uint32_t by, uint32_t bz, uint32_t shared_bytes, const void *args,
                   size_t args_size) {
    NEED_INIT();
    hipFunction_t fn;
    {                                             // module_load on another thread may grow the table
        std::lock_guard<std::mutex> lk(g_mu);
        if (handle == 0 || handle > g_kernels.size()) return fail_msg(-20, "bad kernel handle");
        fn = g_kernels[handle - 1].fn;
    }
    if (!gx || !gy || !gz || !bx || !by || !bz) return fail_msg(-21, "empty grid or block");
    if ((uint64_t)bx * by * bz > 1024) return fail_msg(-22, "block larger than 1024 threads");
    if (!args && args_size) return fail_msg(-23, "argument block is NULL");
    void *config[] = {HIP_LAUNCH_PARAM_BUFFER_POINTER, const_cast<void *>(args),
                      HIP_LAUNCH_PARAM_BUFFER_SIZE, &args_size, HIP_LAUNCH_PARAM_END};
    HIP_TRY(hipModuleLaunchKernel(fn, gx, gy, gz, bx, by, bz, shared_bytes, g_stream, nullptr, config));
    return 0;
}

int dlg_hip_kernel_attrs(uint64_t handle, int32_t *num_regs, int32_t *lds_bytes,
                         int32_t *scratch_bytes, int32_t *max_threads) {
    NEED_INIT();
    hipFunction_t fn;
    {
        std::lock_guard<std::mutex> lk(g_mu);
        if (handle == 0 || handle > g_kernels.size()) return fail_msg(-20, "bad kernel handle");
        fn = g_kernels[handle - 1].fn;
    }
    int v = 0;
    if (num_regs) { HIP_TRY(hipFuncGetAttribute(&v, HIP_FUNC_ATTRIBUTE_NUM_REGS, fn)); *num_regs = v; }
    if (lds_bytes) { HIP_TRY(hipFuncGetAttribute(&v, HIP_FUNC_ATTRIBUTE_SHARED_SIZE_BYTES, fn)); *lds_bytes = v; }
    if (scratch_bytes) { HIP_TRY(hipFuncGetAttribute(&v, HIP_FUNC_ATTRIBUTE_LOCAL_SIZE_BYTES, fn)); *scratch_bytes = v; }
    if (max_threads) { HIP_TRY(hipFuncGetAttribute(&v, HIP_FUNC_ATTRIBUTE_MAX_THREADS_PER_BLOCK, fn)); *max_threads = v; }
    return 0;
}

// ---- full reduction as one call ---------------------------------------------------------------
namespace {

struct ReduceArgs {                               // argument block of hip_kernel.reduce_full_kernel
    const void *x;
    void *out;
    uint32_t n;
    float divisor;
    uint32_t chunk;
};
constexpr size_t kReduceArgsSize = offsetof(ReduceArgs, chunk) + sizeof(uint32_t);
constexpr uint32_t kReduceChunk = 2048;           // vector items one block of the first stage folds
constexpr uint64_t kReduceMaxBlocks = 65536;      // partials one block of the second stage folds

int launch_reduce_stage(hipFunction_t fn, uint32_t blocks, ReduceArgs a) {
    size_t size = kReduceArgsSize;
    void *config[] = {HIP_LAUNCH_PARAM_BUFFER_POINTER, &a, HIP_LAUNCH_PARAM_BUFFER_SIZE, &size, HIP_LAUNCH_PARAM_END};
    HIP_TRY(hipModuleLaunchKernel(fn, blocks, 1, 1, 256, 1, 1, 0, g_stream, nullptr, config));
    return 0;
}

// Both entry points: the first stage writes one partial per block into `part`, the second folds them.
int reduce_full_into(uint64_t k_stage, uint64_t k_fold, const void *x, uint64_t n, uint32_t vec, float divisor,
                     void *out, void *part, size_t part_bytes, const char *who) {
    if (!x || !out) return fail_msg(-1, std::string(who) + ": NULL operand");
    if (vec != 1 && vec != 4) return fail_msg(-41, std::string(who) + ": vec must be 1 or 4");
    if (n == 0 || n >= (uint64_t(1) << 31)) return fail_msg(-42, std::string(who) + ": n must be in [1, 2^31)");
    if (vec == 4 && ((uintptr_t)x & 15)) return fail_msg(-43, std::string(who) + ": vec = 4 needs a 16-byte aligned input");
    hipFunction_t f_stage, f_fold;
    {
        std::lock_guard<std::mutex> lk(g_mu);
        if (k_stage == 0 || k_stage > g_kernels.size() || k_fold == 0 || k_fold > g_kernels.size())
            return fail_msg(-20, "bad kernel handle");
        f_stage = g_kernels[k_stage - 1].fn;
        f_fold = g_kernels[k_fold - 1].fn;
    }
    const uint64_t items = (n + vec - 1) / vec;
    const uint64_t blocks = (items + kReduceChunk - 1) / kReduceChunk;
    if (blocks == 1)                                              // one block folds everything: no partials
        return launch_reduce_stage(f_stage, 1, ReduceArgs{x, out, (uint32_t)n, divisor, (uint32_t)items});
    if (blocks > kReduceMaxBlocks) {
        char buf[200];
        std::snprintf(buf, sizeof buf, "%s: %llu elements need %llu partial results, at most %llu fit one call", who,
                      (unsigned long long)n, (unsigned long long)blocks, (unsigned long long)kReduceMaxBlocks);
        return fail_msg(-44, buf);
    }
    if (!part || ((uintptr_t)part & 15) || part_bytes < blocks * sizeof(float)) {
        char buf[200];
        std::snprintf(buf, sizeof buf, "%s: the partial results need %llu bytes, 16-byte aligned (got %zu)", who,
                      (unsigned long long)(blocks * sizeof(float)), part_bytes);
        return fail_msg(-45, buf);
    }
    int rc = launch_reduce_stage(f_stage, (uint32_t)blocks, ReduceArgs{x, part, (uint32_t)n, 1.0f, kReduceChunk});
    if (rc) return rc;
    return launch_reduce_stage(f_fold, 1, ReduceArgs{part, out, (uint32_t)blocks, divisor, (uint32_t)((blocks + 3) / 4)});
}

}  // namespace

int dlg_hip_reduce_full(uint64_t k_stage, uint64_t k_fold, const void *x, uint64_t n, uint32_t vec,
                        float divisor, void *out, void *workspace, size_t workspace_bytes) {
    NEED_INIT();
    return reduce_full_into(k_stage, k_fold, x, n, vec, divisor, out, workspace, workspace_bytes, "dlg_hip_reduce_full");
}

int dlg_hip_reduce_full_static(uint64_t k_stage, uint64_t k_fold, const void *x, uint64_t n, uint32_t vec,
                               float divisor, void *out) {
    NEED_INIT();
    void *part = g_scratch_ptr[g_device];                         // never the array's name: that is a host-side stand-in
    if (!part) return fail_msg(-40, "dlg_hip_reduce_full_static: the static scratch array was not located at init");
    return reduce_full_into(k_stage, k_fold, x, n, vec, divisor, out, part, DLG_HIP_STATIC_SCRATCH_BYTES,
                            "dlg_hip_reduce_full_static");
}

// ---- arenas and graphs ----------------------------------------------------------------

int dlg_hip_arena_create(uint64_t *arena) {
    NEED_INIT();
    if (!arena) return fail_msg(-1, "arena is NULL");
    std::lock_guard<std::mutex> lk(g_mu);
    *arena = g_next_arena++;
    g_arena_alive[*arena] = true;
    return 0;
}

int dlg_hip_arena_set(uint64_t arena) {
    NEED_INIT();
    std::lock_guard<std::mutex> lk(g_mu);
    if (arena != 0 && !g_arena_alive[arena]) return fail_msg(-30, "no such arena");
    g_arena = arena;
    return 0;
}

int dlg_hip_arena_reserve(uint64_t arena) {
    NEED_INIT();
    if (g_capturing) return fail_msg(-9, "dlg_hip_arena_reserve allocates device memory and cannot run inside a capture");
    std::lock_guard<std::mutex> lk(g_mu);
    if (arena == 0 || !g_arena_alive[arena]) return fail_msg(-30, "no such arena");
    // A pass that repeats what the arena has seen needs, per bucket, as many blocks at once as the most that
    // were ever in use together; blocks of the earlier pass that are still held do not come back for it.
    for (auto &kv : g_usage[arena]) {
        std::vector<void *> &cached = g_free[arena][kv.first];
        while (cached.size() < kv.second.peak) {
            void *p = nullptr;
            hipError_t e = hipMalloc(&p, kv.first);
            if (e != hipSuccess || !p) {
                (void)hipGetLastError();
                char buf[160];
                std::snprintf(buf, sizeof buf, "Failed to reserve %zu bytes of device memory for an arena", kv.first);
                return fail_msg(-3, buf);
            }
            ++g_device_allocs;
            cached.push_back(p);
            g_bytes_cached += kv.first;
        }
    }
    return 0;
}

int dlg_hip_arena_destroy(uint64_t arena) {
    NEED_INIT();
    if (arena == 0) return fail_msg(-30, "the default pool cannot be destroyed");
    HIP_TRY(hipStreamSynchronize(g_stream));
    std::lock_guard<std::mutex> lk(g_mu);
    if (g_arena == arena) g_arena = 0;
    g_arena_alive[arena] = false;
    g_usage.erase(arena);
    trim_arena_locked(arena);
    return 0;
}

int dlg_hip_graph_begin(void) {
    NEED_INIT();
    if (g_capturing) return fail_msg(-31, "a capture is already in progress");
    HIP_TRY(hipStreamBeginCapture(g_stream, hipStreamCaptureModeRelaxed));
    g_capturing = true;
    return 0;
}

int dlg_hip_graph_end(uint64_t *graph, uint64_t *n_nodes) {
    NEED_INIT();
    if (!g_capturing) return fail_msg(-31, "no capture in progress");
    g_capturing = false;
    hipGraph_t g = nullptr;
    HIP_TRY(hipStreamEndCapture(g_stream, &g));
    if (!graph) {                                  // caller only wants the capture abandoned
        if (g) (void)hipGraphDestroy(g);
        return 0;
    }
    size_t nodes = 0;
    (void)hipGraphGetNodes(g, nullptr, &nodes);
    hipGraphExec_t ge = nullptr;
    hipError_t e = hipGraphInstantiate(&ge, g, nullptr, nullptr, 0);
    (void)hipGraphDestroy(g);
    if (e != hipSuccess) return fail("hipGraphInstantiate", e);
    std::lock_guard<std::mutex> lk(g_mu);
    g_graphs.push_back(ge);
    *graph = (uint64_t)g_graphs.size();
    if (n_nodes) *n_nodes = nodes;
    return 0;
}

int dlg_hip_graph_launch(uint64_t graph) {
    NEED_INIT();
    hipGraphExec_t ge;
    {
        std::lock_guard<std::mutex> lk(g_mu);
        if (graph == 0 || graph > g_graphs.size() || !g_graphs[graph - 1]) return fail_msg(-32, "bad graph handle");
        ge = g_graphs[graph - 1];
    }
    HIP_TRY(hipGraphLaunch(ge, g_stream));
    return 0;
}

int dlg_hip_graph_destroy(uint64_t graph) {
    NEED_INIT();
    hipGraphExec_t ge;
    {
        std::lock_guard<std::mutex> lk(g_mu);
        if (graph == 0 || graph > g_graphs.size() || !g_graphs[graph - 1]) return fail_msg(-32, "bad graph handle");
        ge = g_graphs[graph - 1];
        g_graphs[graph - 1] = nullptr;
    }
    HIP_TRY(hipStreamSynchronize(g_stream));
    HIP_TRY(hipGraphExecDestroy(ge));
    return 0;
}

// ---- ordering and timing ------------------------------------------------------------

int dlg_hip_sync(void) {
    NEED_INIT();
    HIP_TRY(hipStreamSynchronize(g_stream));
    return 0;
}

namespace {
// The event behind a handle, or nullptr (with the error text set) for a handle this library never gave out.
hipEvent_t event_of(uint64_t handle) {
    std::lock_guard<std::mutex> lk(g_mu);
    if (handle == 0 || handle > g_events.size() || !g_events[handle - 1]) {
        g_err = "bad event handle";
        return nullptr;
    }
    return g_events[handle - 1];
}
}  // namespace

int dlg_hip_event_create(uint64_t *event) {
    NEED_INIT();
    if (!event) return fail_msg(-1, "event is NULL");
    hipEvent_t ev;
    HIP_TRY(hipEventCreate(&ev));
    std::lock_guard<std::mutex> lk(g_mu);
    g_events.push_back(ev);
    *event = (uint64_t)g_events.size();
    return 0;
}

int dlg_hip_event_record(uint64_t event) {
    NEED_INIT();
    hipEvent_t ev = event_of(event);
    if (!ev) return -33;
    HIP_TRY(hipEventRecord(ev, g_stream));
    return 0;
}

int dlg_hip_event_sync(uint64_t event) {
    NEED_INIT();
    hipEvent_t ev = event_of(event);
    if (!ev) return -33;
    HIP_TRY(hipEventSynchronize(ev));
    return 0;
}

int dlg_hip_event_elapsed_ms(uint64_t start, uint64_t stop, float *ms) {
    NEED_INIT();
    if (!ms) return fail_msg(-1, "ms is NULL");
    hipEvent_t a = event_of(start), b = event_of(stop);
    if (!a || !b) return -33;
    HIP_TRY(hipEventElapsedTime(ms, a, b));
    return 0;
}

int dlg_hip_event_destroy(uint64_t event) {
    NEED_INIT();
    hipEvent_t ev;
    {
        std::lock_guard<std::mutex> lk(g_mu);
        if (event == 0 || event > g_events.size() || !g_events[event - 1]) return fail_msg(-33, "bad event handle");
        ev = g_events[event - 1];
        g_events[event - 1] = nullptr;
    }
    HIP_TRY(hipEventDestroy(ev));
    return 0;
}

}  // extern "C"
