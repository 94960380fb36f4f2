// libappy_hip.so - device runtime behind the APPy HIP code generator.
//
// Host-only translation unit: hiprtc compilation, code-object loading, a pooled
// device allocator, stream-ordered copies, kernel launch and HIP-event timing,
// exported through the C ABI declared in include/appy_hip.h.  The generated
// kernels themselves are produced at run time by the Python code generator and
// compiled here through hiprtc for gfx950.
#include "appy_hip.h"

#include <hip/hip_runtime.h>
#include <hip/hiprtc.h>

#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <map>
#include <mutex>
#include <string>
#include <unordered_map>
#include <vector>

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
    HIP_TRY(hipMemcpyAsync(dst_dev, src_host, nbytes, hipMemcpyHostToDevice, s));
    HIP_TRY(hipStreamSynchronize(s));
    return 0;
}

int appy_hip_memcpy_d2h(void* dst_host, const void* src_dev, size_t nbytes, void* stream) {
    if (nbytes == 0) return 0;
    if (!dst_host || !src_dev) return fail_arg("dst_host/src_dev is NULL");
    hipStream_t s = static_cast<hipStream_t>(stream);
    HIP_TRY(hipMemcpyAsync(dst_host, src_dev, nbytes, hipMemcpyDeviceToHost, s));
    HIP_TRY(hipStreamSynchronize(s));
    return 0;
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
