// libappy_hip.so - device runtime behind the APPy HIP code generator.
//
// hiprtc compilation, code-object loading, a pooled device allocator, stream-ordered
// copies, kernel launch and HIP-event timing, exported through the C ABI declared in
// include/appy_hip.h.  The generated kernels themselves are produced at run time by
// the Python code generator and compiled here through hiprtc for gfx950; the only
// device-side object of this file is the static scratch buffer of
// appy_hip_launch_static_scratch.
#include "appy_hip.h"

#include <hip/hip_runtime.h>
#include <hip/hiprtc.h>

#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <algorithm>
#include <atomic>
#include <map>
#include <mutex>
#include <string>
#include <thread>
#include <unordered_map>
#include <vector>

// Scratch memory for launches that may not allocate (appy_hip_launch_static_scratch): part of
// the library's code object, so every GPU the library runs on holds a copy of its own until the
// process ends.  Host code never uses this name as an address: the address on a device comes
// from hipGetSymbolAddress (static_scratch_of below).
static __device__ __align__(256) unsigned char scratch[APPY_HIP_STATIC_SCRATCH_BYTES];

namespace {

thread_local std::string g_last_error;
thread_local std::string g_compile_log;

int fail_hip(hipError_t e, const char* what) {
    g_last_error = std::string(what) + ": " + hipGetErrorName(e) + " (" + hipGetErrorString(e) + ")";
    // Clear the sticky per-thread error so that the next call reports its own.
    (void)hipGetLastError();
    return static_cast<int>(e);
}

int fail_rtc(hiprtcResult r, const char* what) {
    g_last_error = std::string(what) + ": " + hiprtcGetErrorString(r);
    return 10000 + static_cast<int>(r);
}

int fail_arg(const char* what) {
    g_last_error = std::string("invalid argument: ") + what;
    return static_cast<int>(hipErrorInvalidValue);
}

}  // namespace

// error reporting for the other source files of the library (not exported)
__attribute__((visibility("hidden"))) int appy_hip_internal_fail(hipError_t e, const char* what) { return fail_hip(e, what); }
__attribute__((visibility("hidden"))) int appy_hip_internal_fail_arg(const char* what) { return fail_arg(what); }

namespace {

#define HIP_TRY(expr)                                   \
    do {                                                \
        hipError_t e__ = (expr);                        \
        if (e__ != hipSuccess) return fail_hip(e__, #expr); \
    } while (0)

// ---------------------------------------------------------------------------
// Pooled device allocator.  Sizes are rounded up to a bucket (powers of two up
// to 1 MiB, then multiples of 2 MiB); freed blocks are kept per (device,bucket)
// and handed out again.  The pool is bounded by APPY_HIP_POOL_MAX_BYTES
// (default 64 GiB, a fraction of the 288 GB of HBM3E); beyond that blocks are
// returned to the driver.
// ---------------------------------------------------------------------------
struct Block {
    int device;
    size_t bucket;
};

struct Pool {
    std::mutex mu;
    std::unordered_map<void*, Block> live;                       // handed out
    std::map<std::pair<int, size_t>, std::vector<void*>> cached; // free lists
    uint64_t bytes_in_use = 0;
    uint64_t bytes_cached = 0;
    uint64_t max_cached = 64ull << 30;
    Pool() {
        if (const char* s = std::getenv("APPY_HIP_POOL_MAX_BYTES")) {
            max_cached = std::strtoull(s, nullptr, 10);
        }
    }
};

Pool& pool() {
    static Pool* p = new Pool();  // intentionally leaked: outlives HIP teardown order
    return *p;
}

size_t bucket_of(size_t n) {
    if (n < 256) n = 256;
    const size_t one_mib = size_t(1) << 20;
    if (n <= one_mib) {
        size_t b = 256;
        while (b < n) b <<= 1;
        return b;
    }
    const size_t two_mib = size_t(2) << 20;
    return (n + two_mib - 1) / two_mib * two_mib;
}

std::vector<char> pack_copy(const void* args, size_t nbytes) {
    std::vector<char> buf(nbytes ? nbytes : 1);
    if (nbytes) std::memcpy(buf.data(), args, nbytes);
    return buf;
}

hipError_t launch_packed(hipFunction_t f, uint32_t gx, uint32_t gy, uint32_t gz,
                         uint32_t bx, uint32_t by, uint32_t bz, uint32_t lds,
                         hipStream_t s, void* argbuf, size_t nbytes) {
    void* extra[] = {HIP_LAUNCH_PARAM_BUFFER_POINTER, argbuf,
                     HIP_LAUNCH_PARAM_BUFFER_SIZE, &nbytes, HIP_LAUNCH_PARAM_END};
    return hipModuleLaunchKernel(f, gx, gy, gz, bx, by, bz, lds, s, nullptr, extra);
}

bool launch_shape_ok(uint32_t gx, uint32_t gy, uint32_t gz, uint32_t bx, uint32_t by, uint32_t bz) {
    if (gx == 0 || gy == 0 || gz == 0 || bx == 0 || by == 0 || bz == 0) return false;
    if (uint64_t(bx) * by * bz > 1024) return false;
    // HIP limits the total number of threads per grid dimension to < 2^32.
    if (uint64_t(gx) * bx > 0xFFFFFFFFull) return false;
    if (uint64_t(gy) * by > 0xFFFFFFFFull) return false;
    if (uint64_t(gz) * bz > 0xFFFFFFFFull) return false;
    return true;
}

// ---------------------------------------------------------------------------
// Host memory.  Pinned (page-locked) blocks handed out by appy_hip_host_alloc
// are remembered by address range: a copy whose host side lies inside one is a
// single DMA at link speed.  Any other host pointer is pageable memory: the
// driver's own path for it moves 17-30 GB/s, so large pageable copies go
// through the staging engine below instead.
// ---------------------------------------------------------------------------
struct HostBlocks {
    std::mutex mu;
    std::map<uintptr_t, size_t> ranges;   // base -> bytes
    bool contains(const void* p, size_t n) {
        std::lock_guard<std::mutex> g(mu);
        const uintptr_t a = reinterpret_cast<uintptr_t>(p);
        auto it = ranges.upper_bound(a);
        if (it == ranges.begin()) return false;
        --it;
        return a >= it->first && a + n <= it->first + it->second;
    }
};

HostBlocks& host_blocks() {
    static HostBlocks* h = new HostBlocks();
    return *h;
}

// Staging engine for pageable host memory: the buffer is cut into kLanes
// contiguous slices; one host thread per slice copies its slice through a ring
// of two pinned chunks of its own, on a stream of its own, so that the memcpy of
// chunk k+1 overlaps the DMA of chunk k and the slices overlap each other.  Four
// lanes of 8 MiB chunks reach the link rate measured for pinned memory
// (53 of 57 GB/s in both directions on MI355X; one lane gives 28 GB/s).
constexpr int kLanes = 4;
constexpr int kRing = 2;
constexpr size_t kChunk = size_t(8) << 20;
constexpr size_t kStagedMin = size_t(16) << 20;   // below this the plain copy is as fast

struct StageLane {
    char* pinned[kRing] = {nullptr, nullptr};
    hipEvent_t done[kRing] = {nullptr, nullptr};
    hipStream_t stream = nullptr;
};

struct Stager {
    std::mutex mu;            // one staged copy at a time per device
    bool ready = false;
    bool broken = false;      // pinned memory could not be had: use the plain path
    StageLane lanes[kLanes];
};

Stager& stager(int device) {
    static std::mutex mu;
    static std::map<int, Stager*>* all = new std::map<int, Stager*>();
    std::lock_guard<std::mutex> g(mu);
    auto it = all->find(device);
    if (it == all->end()) it = all->emplace(device, new Stager()).first;
    return *it->second;
}

void stager_release(Stager& st) {
    for (auto& lane : st.lanes) {
        for (int r = 0; r < kRing; ++r) {
            if (lane.done[r]) (void)hipEventDestroy(lane.done[r]);
            if (lane.pinned[r]) (void)hipHostFree(lane.pinned[r]);
            lane.done[r] = nullptr;
            lane.pinned[r] = nullptr;
        }
        if (lane.stream) (void)hipStreamDestroy(lane.stream);
        lane.stream = nullptr;
    }
}

hipError_t stager_prepare(Stager& st) {
    if (st.ready) return hipSuccess;
    hipError_t e = hipSuccess;
    for (auto& lane : st.lanes) {
        e = hipStreamCreateWithFlags(&lane.stream, hipStreamNonBlocking);   // default priority
        for (int r = 0; r < kRing && e == hipSuccess; ++r) {
            e = hipHostMalloc(reinterpret_cast<void**>(&lane.pinned[r]), kChunk, hipHostMallocDefault);
            if (e == hipSuccess) e = hipEventCreateWithFlags(&lane.done[r], hipEventDisableTiming);
        }
        if (e != hipSuccess) break;
    }
    if (e != hipSuccess) {
        stager_release(st);     // a partial set-up is of no use: give back what it took
        return e;
    }
    st.ready = true;
    return hipSuccess;
}

// One lane's share of a staged copy.  to_device: host -> pinned -> device;
// otherwise device -> pinned -> host, the host memcpy trailing the DMA by one slot.
hipError_t stage_slice(StageLane& lane, int device, char* dev, char* host, size_t n, bool to_device) {
    hipError_t e = hipSetDevice(device);
    if (e != hipSuccess) return e;
    size_t pend_off[kRing] = {0, 0}, pend_len[kRing] = {0, 0};
    size_t off = 0;
    // a slice is cut into at least eight pieces so that the host memcpy of one piece
    // hides behind the DMA of the one before it, also for slices of a few MiB
    size_t piece = std::min(kChunk, std::max(size_t(1) << 20, (n / 8 + 4095) & ~size_t(4095)));
    for (int i = 0; off < n; ++i) {
        const int r = i % kRing;
        const size_t m = std::min(piece, n - off);
        if (i >= kRing) {
            if ((e = hipEventSynchronize(lane.done[r])) != hipSuccess) return e;
            if (!to_device) std::memcpy(host + pend_off[r], lane.pinned[r], pend_len[r]);
        }
        if (to_device) {
            std::memcpy(lane.pinned[r], host + off, m);
            e = hipMemcpyAsync(dev + off, lane.pinned[r], m, hipMemcpyHostToDevice, lane.stream);
        } else {
            e = hipMemcpyAsync(lane.pinned[r], dev + off, m, hipMemcpyDeviceToHost, lane.stream);
        }
        if (e != hipSuccess) return e;
        if ((e = hipEventRecord(lane.done[r], lane.stream)) != hipSuccess) return e;
        pend_off[r] = off;
        pend_len[r] = m;
        off += m;
    }
    if ((e = hipStreamSynchronize(lane.stream)) != hipSuccess) return e;
    if (!to_device) {
        // the last (up to kRing) chunks are still in the ring
        const size_t chunks = (n + piece - 1) / piece;
        const size_t first = chunks > size_t(kRing) ? chunks - kRing : 0;
        for (size_t c = first; c < chunks; ++c) {
            const int r = int(c % kRing);
            std::memcpy(host + pend_off[r], lane.pinned[r], pend_len[r]);
        }
    }
    return hipSuccess;
}

// Returns hipErrorNotSupported when the staged path is not available (the caller
// then uses the plain copy).
hipError_t staged_copy(void* dev, void* host, size_t n, bool to_device, hipStream_t order_after) {
    int device = 0;
    hipError_t e = hipGetDevice(&device);
    if (e != hipSuccess) return e;
    Stager& st = stager(device);
    std::lock_guard<std::mutex> g(st.mu);
    if (st.broken) return hipErrorNotSupported;
    if ((e = stager_prepare(st)) != hipSuccess) {
        st.broken = true;
        (void)hipGetLastError();
        return hipErrorNotSupported;
    }
    // work already queued on the caller's stream (the kernel whose results are
    // fetched, or earlier users of the destination) comes first
    if ((e = hipStreamSynchronize(order_after)) != hipSuccess) return e;
    size_t per = (n + kLanes - 1) / kLanes;
    per = (per + 4095) & ~size_t(4095);
    hipError_t results[kLanes];
    std::thread workers[kLanes];
    bool inline_slices[kLanes] = {};
    int used = 0;
    for (int t = 0; t < kLanes; ++t) {
        results[t] = hipSuccess;
        const size_t o = per * size_t(t);
        if (o >= n) break;
        const size_t m = std::min(per, n - o);
        char* d = static_cast<char*>(dev) + o;
        char* h = static_cast<char*>(host) + o;
        StageLane* lane = &st.lanes[t];
        hipError_t* out = &results[t];
        if (t == 0) continue;   // the calling thread takes the first slice itself, below
        try {
            workers[t] = std::thread([=] { *out = stage_slice(*lane, device, d, h, m, to_device); });
        } catch (...) {
            // no thread to be had: the calling thread copies this slice too (no exception may
            // cross the C boundary)
            inline_slices[t] = true;
        }
        used = t;
    }
    results[0] = stage_slice(st.lanes[0], device, static_cast<char*>(dev), static_cast<char*>(host),
                             std::min(per, n), to_device);
    for (int t = 1; t <= used; ++t) {
        if (inline_slices[t]) {
            const size_t o = per * size_t(t);
            results[t] = stage_slice(st.lanes[t], device, static_cast<char*>(dev) + o, static_cast<char*>(host) + o,
                                     std::min(per, n - o), to_device);
        } else {
            workers[t].join();
        }
    }
    for (int t = 0; t < kLanes; ++t)
        if (results[t] != hipSuccess) return results[t];
    return hipSuccess;
}

// Address of the static scratch buffer on each device, looked up once per device with that
// device current.
constexpr int kMaxDevices = 64;
std::mutex g_scratch_mu;
void* g_scratch_ptr[kMaxDevices] = {};

hipError_t static_scratch_of(int device, void** out) {
    if (device < 0 || device >= kMaxDevices) return hipErrorInvalidDevice;
    std::lock_guard<std::mutex> g(g_scratch_mu);
    if (!g_scratch_ptr[device]) {
        int current = -1;
        hipError_t e = hipGetDevice(&current);
        if (e != hipSuccess) return e;
        if (current != device) return hipErrorInvalidDevice;    // the caller makes the device current first
        void* p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return e;
        if (!p) return hipErrorInvalidSymbol;
        g_scratch_ptr[device] = p;
    }
    *out = g_scratch_ptr[device];
    return hipSuccess;
}

bool staging_enabled() {
    static const bool on = [] {
        const char* s = std::getenv("APPY_HIP_NO_STAGING");
        return !(s && s[0] == '1');
    }();
    return on;
}

}  // namespace

extern "C" {

int appy_hip_abi_version(void) { return APPY_HIP_ABI_VERSION; }

const char* appy_hip_last_error(void) { return g_last_error.c_str(); }

// ---- device ---------------------------------------------------------------

int appy_hip_device_count(int* count_out) {
    if (!count_out) return fail_arg("count_out is NULL");
    int n = 0;
    hipError_t e = hipGetDeviceCount(&n);
    if (e == hipErrorNoDevice) {
        (void)hipGetLastError();
        *count_out = 0;
        return 0;
    }
    if (e != hipSuccess) return fail_hip(e, "hipGetDeviceCount");
    *count_out = n;
    return 0;
}

int appy_hip_init(int device) {
    HIP_TRY(hipSetDevice(device));
    HIP_TRY(hipFree(nullptr));  // forces creation of the primary context
    // the device's copy of the static scratch buffer (appy_hip_launch_static_scratch)
    void* p = nullptr;
    HIP_TRY(static_scratch_of(device, &p));
    return 0;
}

int appy_hip_device_props(int device, appy_hip_props* out) {
    if (!out) return fail_arg("out is NULL");
    hipDeviceProp_t p;
    HIP_TRY(hipGetDeviceProperties(&p, device));
    std::memset(out, 0, sizeof(*out));
    std::snprintf(out->name, sizeof(out->name), "%s", p.name);
    std::snprintf(out->arch, sizeof(out->arch), "%s", p.gcnArchName);
    out->compute_units = p.multiProcessorCount;
    out->wavefront_size = p.warpSize;
    out->max_threads_per_block = p.maxThreadsPerBlock;
    out->lds_bytes_per_block = static_cast<int32_t>(p.sharedMemPerBlock);
    out->l2_bytes = p.l2CacheSize;
    out->clock_khz = p.clockRate;
    out->mem_clock_khz = p.memoryClockRate;
    out->mem_bus_bits = p.memoryBusWidth;
    out->hbm_bytes = p.totalGlobalMem;
    return 0;
}

int appy_hip_device_topology(int device, appy_hip_topology* out) {
    if (!out) return fail_arg("out is NULL");
    std::memset(out, 0, sizeof(*out));
    int xcds = 0, cus = 0, l2 = 0, lds = 0;
    if (hipDeviceGetAttribute(&xcds, hipDeviceAttributeNumberOfXccs, device) != hipSuccess || xcds < 1) {
        (void)hipGetLastError();
        xcds = 1;
    }
    HIP_TRY(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, device));
    HIP_TRY(hipDeviceGetAttribute(&l2, hipDeviceAttributeL2CacheSize, device));
    HIP_TRY(hipDeviceGetAttribute(&lds, hipDeviceAttributeMaxSharedMemoryPerMultiprocessor, device));
    out->xcds = xcds;
    out->compute_units = cus;
    out->l2_bytes_per_xcd = l2;
    out->lds_bytes_per_cu = lds;
    return 0;
}

// ---- run-time compilation ---------------------------------------------------

int appy_hip_compile(const char* src, const char* name, const char* arch,
                     const char* const* opts, int nopts,
                     void** code_out, size_t* size_out) {
    g_compile_log.clear();
    if (!src || !code_out || !size_out) return fail_arg("src/code_out/size_out is NULL");
    if (nopts < 0 || (nopts > 0 && !opts)) return fail_arg("opts");
    *code_out = nullptr;
    *size_out = 0;

    hiprtcProgram prog = nullptr;
    hiprtcResult r = hiprtcCreateProgram(&prog, src, name ? name : "appy_kernel.hip", 0, nullptr, nullptr);
    if (r != HIPRTC_SUCCESS) return fail_rtc(r, "hiprtcCreateProgram");

    std::string arch_opt = std::string("--offload-arch=") + ((arch && *arch) ? arch : "gfx950");
    std::vector<const char*> all;
    all.push_back(arch_opt.c_str());
    for (int i = 0; i < nopts; ++i) all.push_back(opts[i]);

    r = hiprtcCompileProgram(prog, static_cast<int>(all.size()), all.data());

    size_t log_size = 0;
    if (hiprtcGetProgramLogSize(prog, &log_size) == HIPRTC_SUCCESS && log_size > 1) {
        g_compile_log.resize(log_size);
        if (hiprtcGetProgramLog(prog, &g_compile_log[0]) != HIPRTC_SUCCESS) g_compile_log.clear();
        while (!g_compile_log.empty() && g_compile_log.back() == '\0') g_compile_log.pop_back();
    }
    if (r != HIPRTC_SUCCESS) {
        hiprtcDestroyProgram(&prog);
        int rc = fail_rtc(r, "hiprtcCompileProgram");
        if (!g_compile_log.empty()) g_last_error += "\n" + g_compile_log;
        return rc;
    }

    size_t code_size = 0;
    r = hiprtcGetCodeSize(prog, &code_size);
    if (r != HIPRTC_SUCCESS || code_size == 0) {
        hiprtcDestroyProgram(&prog);
        return fail_rtc(r == HIPRTC_SUCCESS ? HIPRTC_ERROR_INTERNAL_ERROR : r, "hiprtcGetCodeSize");
    }
    void* code = std::malloc(code_size);
    if (!code) {
        hiprtcDestroyProgram(&prog);
        g_last_error = "out of host memory for code object";
        return static_cast<int>(hipErrorOutOfMemory);
    }
    r = hiprtcGetCode(prog, static_cast<char*>(code));
    hiprtcDestroyProgram(&prog);
    if (r != HIPRTC_SUCCESS) {
        std::free(code);
        return fail_rtc(r, "hiprtcGetCode");
    }
    *code_out = code;
    *size_out = code_size;
    return 0;
}

int appy_hip_rtc_version(int* version_out) {
    if (!version_out) return fail_arg("version_out is NULL");
    int major = 0, minor = 0;
    hiprtcResult r = hiprtcVersion(&major, &minor);
    if (r != HIPRTC_SUCCESS) return fail_rtc(r, "hiprtcVersion");
    *version_out = major * 1000 + minor;
    return 0;
}

const char* appy_hip_compile_log(void) { return g_compile_log.c_str(); }

void appy_hip_code_free(void* code) { std::free(code); }

int appy_hip_module_load(const void* code, size_t size, void** module_out) {
    if (!code || size == 0 || !module_out) return fail_arg("code/size/module_out");
    hipModule_t m = nullptr;
    HIP_TRY(hipModuleLoadData(&m, code));
    *module_out = m;
    return 0;
}

int appy_hip_module_get_function(void* module, const char* kernel_name, void** func_out) {
    if (!module || !kernel_name || !func_out) return fail_arg("module/kernel_name/func_out");
    hipFunction_t f = nullptr;
    HIP_TRY(hipModuleGetFunction(&f, static_cast<hipModule_t>(module), kernel_name));
    *func_out = f;
    return 0;
}

int appy_hip_module_unload(void* module) {
    if (!module) return 0;
    HIP_TRY(hipModuleUnload(static_cast<hipModule_t>(module)));
    return 0;
}

int appy_hip_func_get_info(void* func, appy_hip_func_info* out) {
    if (!func || !out) return fail_arg("func/out");
    hipFunction_t f = static_cast<hipFunction_t>(func);
    int v = 0;
    std::memset(out, 0, sizeof(*out));
    HIP_TRY(hipFuncGetAttribute(&v, HIP_FUNC_ATTRIBUTE_NUM_REGS, f));
    out->num_vgprs = v;
    HIP_TRY(hipFuncGetAttribute(&v, HIP_FUNC_ATTRIBUTE_SHARED_SIZE_BYTES, f));
    out->static_lds_bytes = v;
    HIP_TRY(hipFuncGetAttribute(&v, HIP_FUNC_ATTRIBUTE_LOCAL_SIZE_BYTES, f));
    out->scratch_bytes = v;
    HIP_TRY(hipFuncGetAttribute(&v, HIP_FUNC_ATTRIBUTE_MAX_THREADS_PER_BLOCK, f));
    out->max_threads_per_block = v;
    return 0;
}

int appy_hip_occupancy(void* func, int block_threads, size_t dynamic_lds_bytes, int* blocks_per_cu_out) {
    if (!func || !blocks_per_cu_out || block_threads <= 0) return fail_arg("func/blocks_per_cu_out/block_threads");
    int n = 0;
    HIP_TRY(hipModuleOccupancyMaxActiveBlocksPerMultiprocessor(
        &n, static_cast<hipFunction_t>(func), block_threads, dynamic_lds_bytes));
    *blocks_per_cu_out = n;
    return 0;
}

// ---- device memory ----------------------------------------------------------

int appy_hip_malloc(size_t nbytes, void** dptr_out) {
    if (!dptr_out) return fail_arg("dptr_out is NULL");
    *dptr_out = nullptr;
    int dev = 0;
    HIP_TRY(hipGetDevice(&dev));
    const size_t b = bucket_of(nbytes);
    Pool& p = pool();
    {
        std::lock_guard<std::mutex> lk(p.mu);
        auto it = p.cached.find({dev, b});
        if (it != p.cached.end() && !it->second.empty()) {
            void* d = it->second.back();
            it->second.pop_back();
            p.bytes_cached -= b;
            p.bytes_in_use += b;
            p.live[d] = Block{dev, b};
            *dptr_out = d;
            return 0;
        }
    }
    void* d = nullptr;
    hipError_t e = hipMalloc(&d, b);
    if (e == hipErrorOutOfMemory) {
        // Give the cached blocks back to the driver and try once more.
        (void)hipGetLastError();
        appy_hip_pool_trim();
        e = hipMalloc(&d, b);
    }
    if (e != hipSuccess) return fail_hip(e, "hipMalloc");
    {
        std::lock_guard<std::mutex> lk(p.mu);
        p.live[d] = Block{dev, b};
        p.bytes_in_use += b;
    }
    *dptr_out = d;
    return 0;
}

int appy_hip_free(void* dptr) {
    if (!dptr) return 0;
    Pool& p = pool();
    Block blk{};
    bool keep = false;
    {
        std::lock_guard<std::mutex> lk(p.mu);
        auto it = p.live.find(dptr);
        if (it == p.live.end()) return fail_arg("pointer was not allocated by appy_hip_malloc");
        blk = it->second;
        p.live.erase(it);
        p.bytes_in_use -= blk.bucket;
        if (p.bytes_cached + blk.bucket <= p.max_cached) {
            p.cached[{blk.device, blk.bucket}].push_back(dptr);
            p.bytes_cached += blk.bucket;
            keep = true;
        }
    }
    if (!keep) HIP_TRY(hipFree(dptr));
    return 0;
}

int appy_hip_pool_trim(void) {
    Pool& p = pool();
    std::vector<void*> victims;
    {
        std::lock_guard<std::mutex> lk(p.mu);
        for (auto& kv : p.cached) {
            for (void* d : kv.second) victims.push_back(d);
            kv.second.clear();
        }
        p.bytes_cached = 0;
    }
    int rc = 0;
    for (void* d : victims) {
        hipError_t e = hipFree(d);
        if (e != hipSuccess && rc == 0) rc = fail_hip(e, "hipFree");
    }
    return rc;
}

int appy_hip_pool_stats(uint64_t* bytes_in_use_out, uint64_t* bytes_cached_out) {
    Pool& p = pool();
    std::lock_guard<std::mutex> lk(p.mu);
    if (bytes_in_use_out) *bytes_in_use_out = p.bytes_in_use;
    if (bytes_cached_out) *bytes_cached_out = p.bytes_cached;
    return 0;
}

int appy_hip_memcpy_h2d(void* dst_dev, const void* src_host, size_t nbytes, void* stream) {
    if (nbytes == 0) return 0;
    if (!dst_dev || !src_host) return fail_arg("dst_dev/src_host is NULL");
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (nbytes >= kStagedMin && staging_enabled() && !host_blocks().contains(src_host, nbytes)) {
        hipError_t e = staged_copy(dst_dev, const_cast<void*>(src_host), nbytes, true, s);
        if (e == hipSuccess) return 0;
        if (e != hipErrorNotSupported) return fail_hip(e, "staged host-to-device copy");
    }
    HIP_TRY(hipMemcpyAsync(dst_dev, src_host, nbytes, hipMemcpyHostToDevice, s));
    HIP_TRY(hipStreamSynchronize(s));
    return 0;
}

int appy_hip_memcpy_h2d_async(void* dst_dev, const void* src_pinned, size_t nbytes, void* stream) {
    if (nbytes == 0) return 0;
    if (!dst_dev || !src_pinned) return fail_arg("dst_dev/src_pinned is NULL");
    if (!host_blocks().contains(src_pinned, nbytes))
        return fail_arg("asynchronous uploads take memory from appy_hip_host_alloc only");
    HIP_TRY(hipMemcpyAsync(dst_dev, src_pinned, nbytes, hipMemcpyHostToDevice, static_cast<hipStream_t>(stream)));
    return 0;
}

int appy_hip_memcpy_d2h(void* dst_host, const void* src_dev, size_t nbytes, void* stream) {
    if (nbytes == 0) return 0;
    if (!dst_host || !src_dev) return fail_arg("dst_host/src_dev is NULL");
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (nbytes >= kStagedMin && staging_enabled() && !host_blocks().contains(dst_host, nbytes)) {
        hipError_t e = staged_copy(const_cast<void*>(src_dev), dst_host, nbytes, false, s);
        if (e == hipSuccess) return 0;
        if (e != hipErrorNotSupported) return fail_hip(e, "staged device-to-host copy");
    }
    HIP_TRY(hipMemcpyAsync(dst_host, src_dev, nbytes, hipMemcpyDeviceToHost, s));
    HIP_TRY(hipStreamSynchronize(s));
    return 0;
}

int appy_hip_host_alloc(size_t nbytes, void** out) {
    if (!out) return fail_arg("out is NULL");
    *out = nullptr;
    void* p = nullptr;
    HIP_TRY(hipHostMalloc(&p, nbytes ? nbytes : 1, hipHostMallocDefault));
    {
        std::lock_guard<std::mutex> g(host_blocks().mu);
        host_blocks().ranges[reinterpret_cast<uintptr_t>(p)] = nbytes ? nbytes : 1;
    }
    *out = p;
    return 0;
}

int appy_hip_host_free(void* p) {
    if (!p) return 0;
    {
        std::lock_guard<std::mutex> g(host_blocks().mu);
        auto it = host_blocks().ranges.find(reinterpret_cast<uintptr_t>(p));
        if (it == host_blocks().ranges.end()) return fail_arg("pointer was not returned by appy_hip_host_alloc");
        host_blocks().ranges.erase(it);
    }
    HIP_TRY(hipHostFree(p));
    return 0;
}

int appy_hip_host_is_pinned(const void* p, size_t nbytes) {
    return host_blocks().contains(p, nbytes) ? 1 : 0;
}

int appy_hip_memcpy_d2d_async(void* dst_dev, const void* src_dev, size_t nbytes, void* stream) {
    if (nbytes == 0) return 0;
    if (!dst_dev || !src_dev) return fail_arg("dst_dev/src_dev is NULL");
    HIP_TRY(hipMemcpyAsync(dst_dev, src_dev, nbytes, hipMemcpyDeviceToDevice, static_cast<hipStream_t>(stream)));
    return 0;
}

int appy_hip_memset_async(void* dst_dev, int byte_value, size_t nbytes, void* stream) {
    if (nbytes == 0) return 0;
    if (!dst_dev) return fail_arg("dst_dev is NULL");
    if (stream) {
        // memset nodes are kept out of graphs (replays of such nodes are not reliable
        // on this platform): clear with a kernel inside a capture instead
        hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
        HIP_TRY(hipStreamIsCapturing(static_cast<hipStream_t>(stream), &st));
        if (st != hipStreamCaptureStatusNone) return fail_arg("memset on a stream that is being captured");
    }
    HIP_TRY(hipMemsetAsync(dst_dev, byte_value, nbytes, static_cast<hipStream_t>(stream)));
    return 0;
}

// ---- launch -----------------------------------------------------------------

int appy_hip_launch(void* func,
                    uint32_t grid_x, uint32_t grid_y, uint32_t grid_z,
                    uint32_t block_x, uint32_t block_y, uint32_t block_z,
                    uint32_t dynamic_lds_bytes, void* stream,
                    const void* args, size_t args_bytes) {
    if (!func) return fail_arg("func is NULL");
    if (args_bytes > 0 && !args) return fail_arg("args is NULL");
    if (!launch_shape_ok(grid_x, grid_y, grid_z, block_x, block_y, block_z))
        return fail_arg("grid/block shape out of range");
    std::vector<char> buf = pack_copy(args, args_bytes);
    HIP_TRY(launch_packed(static_cast<hipFunction_t>(func), grid_x, grid_y, grid_z,
                          block_x, block_y, block_z, dynamic_lds_bytes,
                          static_cast<hipStream_t>(stream), buf.data(), args_bytes));
    return 0;
}

int appy_hip_sync(void* stream) {
    HIP_TRY(hipStreamSynchronize(static_cast<hipStream_t>(stream)));
    return 0;
}

int appy_hip_device_sync(void) {
    HIP_TRY(hipDeviceSynchronize());
    return 0;
}

int appy_hip_launch_static_scratch(void* func,
                                   uint32_t grid_x, uint32_t grid_y, uint32_t grid_z,
                                   uint32_t block_x, uint32_t block_y, uint32_t block_z,
                                   uint32_t dynamic_lds_bytes, void* stream,
                                   const void* args, size_t args_bytes,
                                   size_t scratch_arg_offset, size_t scratch_bytes) {
    constexpr size_t kMaxArgs = 4096;
    if (!func) return fail_arg("func is NULL");
    if (!args || args_bytes == 0) return fail_arg("args is NULL or empty");
    if (args_bytes > kMaxArgs) return fail_arg("argument block larger than 4096 bytes");
    if (scratch_arg_offset % alignof(void*) || args_bytes < sizeof(void*) || scratch_arg_offset > args_bytes - sizeof(void*))
        return fail_arg("scratch_arg_offset does not name a pointer inside the argument block");
    if (scratch_bytes > APPY_HIP_STATIC_SCRATCH_BYTES)
        return fail_arg("scratch_bytes exceeds APPY_HIP_STATIC_SCRATCH_BYTES (the static scratch buffer holds 8 MiB)");
    if (!launch_shape_ok(grid_x, grid_y, grid_z, block_x, block_y, block_z))
        return fail_arg("grid/block shape out of range");
    int device = 0;
    HIP_TRY(hipGetDevice(&device));
    void* dev_scratch = nullptr;
    HIP_TRY(static_scratch_of(device, &dev_scratch));
    alignas(16) char buf[kMaxArgs];                 // no heap: the argument block is copied on the stack
    std::memcpy(buf, args, args_bytes);
    std::memcpy(buf + scratch_arg_offset, &dev_scratch, sizeof(void*));
    HIP_TRY(launch_packed(static_cast<hipFunction_t>(func), grid_x, grid_y, grid_z,
                          block_x, block_y, block_z, dynamic_lds_bytes,
                          static_cast<hipStream_t>(stream), buf, args_bytes));
    return 0;
}

// ---- streams and graphs -------------------------------------------------------

int appy_hip_stream_create(void** stream_out) {
    if (!stream_out) return fail_arg("stream_out is NULL");
    hipStream_t s = nullptr;
    HIP_TRY(hipStreamCreateWithFlags(&s, hipStreamNonBlocking));   // default priority
    *stream_out = s;
    return 0;
}

int appy_hip_stream_destroy(void* stream) {
    if (!stream) return 0;
    HIP_TRY(hipStreamDestroy(static_cast<hipStream_t>(stream)));
    return 0;
}

int appy_hip_graph_begin(void* stream) {
    if (!stream) return fail_arg("the null stream cannot be captured");
    // Relaxed: code-object loads and pool growth triggered by the first launch of a
    // kernel are legal while capturing; they are simply not part of the graph.
    HIP_TRY(hipStreamBeginCapture(static_cast<hipStream_t>(stream), hipStreamCaptureModeRelaxed));
    return 0;
}

int appy_hip_graph_end(void* stream, void** graph_exec_out) {
    if (!stream || !graph_exec_out) return fail_arg("stream/graph_exec_out is NULL");
    *graph_exec_out = nullptr;
    hipGraph_t g = nullptr;
    HIP_TRY(hipStreamEndCapture(static_cast<hipStream_t>(stream), &g));
    if (!g) return fail_arg("the capture recorded nothing");
    hipGraphExec_t ex = nullptr;
    hipError_t e = hipGraphInstantiate(&ex, g, nullptr, nullptr, 0);
    (void)hipGraphDestroy(g);
    if (e != hipSuccess) return fail_hip(e, "hipGraphInstantiate");
    *graph_exec_out = ex;
    return 0;
}

int appy_hip_graph_launch(void* graph_exec, void* stream) {
    if (!graph_exec) return fail_arg("graph_exec is NULL");
    HIP_TRY(hipGraphLaunch(static_cast<hipGraphExec_t>(graph_exec), static_cast<hipStream_t>(stream)));
    return 0;
}

int appy_hip_graph_destroy(void* graph_exec) {
    if (!graph_exec) return 0;
    HIP_TRY(hipGraphExecDestroy(static_cast<hipGraphExec_t>(graph_exec)));
    return 0;
}

// ---- timing -----------------------------------------------------------------

int appy_hip_event_create(void** event_out) {
    if (!event_out) return fail_arg("event_out is NULL");
    hipEvent_t e = nullptr;
    HIP_TRY(hipEventCreate(&e));
    *event_out = e;
    return 0;
}

int appy_hip_event_record(void* event, void* stream) {
    if (!event) return fail_arg("event is NULL");
    HIP_TRY(hipEventRecord(static_cast<hipEvent_t>(event), static_cast<hipStream_t>(stream)));
    return 0;
}

int appy_hip_event_sync(void* event) {
    if (!event) return fail_arg("event is NULL");
    HIP_TRY(hipEventSynchronize(static_cast<hipEvent_t>(event)));
    return 0;
}

int appy_hip_event_elapsed_ms(void* start, void* stop, float* ms_out) {
    if (!start || !stop || !ms_out) return fail_arg("start/stop/ms_out");
    HIP_TRY(hipEventElapsedTime(ms_out, static_cast<hipEvent_t>(start), static_cast<hipEvent_t>(stop)));
    return 0;
}

int appy_hip_event_destroy(void* event) {
    if (!event) return 0;
    HIP_TRY(hipEventDestroy(static_cast<hipEvent_t>(event)));
    return 0;
}

int appy_hip_launch_timed(void* func,
                          uint32_t grid_x, uint32_t grid_y, uint32_t grid_z,
                          uint32_t block_x, uint32_t block_y, uint32_t block_z,
                          uint32_t dynamic_lds_bytes, void* stream,
                          const void* args, size_t args_bytes,
                          int warmup, int reps, float* mean_ms_out) {
    if (!func || !mean_ms_out) return fail_arg("func/mean_ms_out");
    if (reps <= 0 || warmup < 0) return fail_arg("reps/warmup");
    if (args_bytes > 0 && !args) return fail_arg("args is NULL");
    if (!launch_shape_ok(grid_x, grid_y, grid_z, block_x, block_y, block_z))
        return fail_arg("grid/block shape out of range");
    hipFunction_t f = static_cast<hipFunction_t>(func);
    hipStream_t s = static_cast<hipStream_t>(stream);
    std::vector<char> buf = pack_copy(args, args_bytes);
    for (int i = 0; i < warmup; ++i)
        HIP_TRY(launch_packed(f, grid_x, grid_y, grid_z, block_x, block_y, block_z,
                              dynamic_lds_bytes, s, buf.data(), args_bytes));
    hipEvent_t e0 = nullptr, e1 = nullptr;
    HIP_TRY(hipEventCreate(&e0));
    hipError_t err = hipEventCreate(&e1);
    if (err != hipSuccess) {
        (void)hipEventDestroy(e0);
        return fail_hip(err, "hipEventCreate");
    }
    err = hipEventRecord(e0, s);
    for (int i = 0; i < reps && err == hipSuccess; ++i)
        err = launch_packed(f, grid_x, grid_y, grid_z, block_x, block_y, block_z,
                            dynamic_lds_bytes, s, buf.data(), args_bytes);
    if (err == hipSuccess) err = hipEventRecord(e1, s);
    if (err == hipSuccess) err = hipEventSynchronize(e1);
    float ms = 0.f;
    if (err == hipSuccess) err = hipEventElapsedTime(&ms, e0, e1);
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    if (err != hipSuccess) return fail_hip(err, "timed launch");
    *mean_ms_out = ms / static_cast<float>(reps);
    return 0;
}

}  // extern "C"
