/*
 * appy_hip.h - C ABI of libappy_hip.so, the device runtime underneath the APPy
 * HIP code generator (gfx950 / MI355X).
 *
 * The reference has no native layer: its generated host launchers reach the GPU
 * through PyTorch + Triton calls emitted as Python text.  Each entry point below
 * names the reference construct whose job it takes over (paths are relative to
 * the reference tree).  All functions are plain C: pointers, sizes and ints,
 * no C++ or torch types.  Every function returns 0 on success; a non-zero value
 * is a hipError_t (1..9999) or 10000 + hiprtcResult, and appy_hip_last_error()
 * returns the matching text for the calling thread.
 *
 * Threading: all entry points may be called from several host threads at once.
 * Streams are caller supplied (NULL = the null stream); launches and *_async
 * calls are asynchronous with respect to the host.
 */
#ifndef APPY_HIP_H
#define APPY_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* 2: page-locked host memory, streams and graphs, appy_hip_rtc_version; 3: appy_hip_launch_static_scratch;
 * 4: row plans (appy_hip_rowplan_*), appy_hip_device_sync, appy_hip_memcpy_h2d_async, appy_hip_device_topology
 * (additions only: every entry point of the earlier versions is unchanged). */
#define APPY_HIP_ABI_VERSION 5

typedef struct appy_hip_props {
    char     name[128];        /* marketing name */
    char     arch[64];         /* gcnArchName, e.g. "gfx950:sramecc+:xnack-" */
    int32_t  compute_units;    /* CUs on the device */
    int32_t  wavefront_size;   /* 64 on CDNA */
    int32_t  max_threads_per_block;
    int32_t  lds_bytes_per_block;
    int32_t  l2_bytes;
    int32_t  clock_khz;
    int32_t  mem_clock_khz;
    int32_t  mem_bus_bits;
    uint64_t hbm_bytes;
} appy_hip_props;

typedef struct appy_hip_func_info {
    int32_t num_vgprs;         /* hipFuncAttributes.numRegs */
    int32_t static_lds_bytes;  /* sharedSizeBytes */
    int32_t scratch_bytes;     /* localSizeBytes: >0 means register spills */
    int32_t max_threads_per_block;
} appy_hip_func_info;

/* ---- library ---------------------------------------------------------- */

/* ABI version of the loaded library (APPY_HIP_ABI_VERSION). */
int appy_hip_abi_version(void);

/* Text of the last error raised on the calling thread ("" if none). */
const char* appy_hip_last_error(void);

/* ---- device ------------------------------------------------------------
 * Replaces the reference's device discovery: shutil.which("nvidia-smi") in
 * appy/dispatcher.py:37 and the literal 'cuda' device string in
 * appy/backends/triton/passes/host_passes/gen_data_movement.py:48-62. */
int appy_hip_device_count(int* count_out);
int appy_hip_init(int device);                 /* make `device` current for this thread */
int appy_hip_device_props(int device, appy_hip_props* out);
/* How the compute units are grouped (ABI 4; appy_hip_props keeps its layout).  On MI355X: 8 accelerator dies
 * (XCDs) of 32 CUs, each with an L2 of its own (appy_hip_props.l2_bytes is that of one die) - the launch
 * heuristics size grids by the CUs and pin stripes of gathered operands to dies, workgroup number modulo `xcds`. */
typedef struct appy_hip_topology {
    int32_t xcds;               /* accelerator dies with an L2 each; 1 where the device does not say */
    int32_t compute_units;      /* all of them, as appy_hip_props.compute_units */
    int32_t l2_bytes_per_xcd;
    int32_t lds_bytes_per_cu;
} appy_hip_topology;
int appy_hip_device_topology(int device, appy_hip_topology* out);

/* ---- run-time compilation ----------------------------------------------
 * Replaces @triton.jit on the generated `_kernel_loop_N`
 * (appy/backends/triton/passes/gen_device_code.py:36-41) and the
 * load_module_from_str step (appy/backends/triton/codegen.py:51-55): HIP C++
 * source text -> gfx950 code object, via hiprtc.  Needs no GPU.
 * `arch` is e.g. "gfx950"; `opts` are extra hiprtc options.  On success
 * *code_out / *size_out hold a malloc'ed code object (free with
 * appy_hip_code_free).  The compiler log of the last compile on this thread
 * (warnings or errors) is returned by appy_hip_compile_log(). */
int appy_hip_compile(const char* src, const char* name, const char* arch,
                     const char* const* opts, int nopts,
                     void** code_out, size_t* size_out);
const char* appy_hip_compile_log(void);
/* hiprtc's version as major * 1000 + minor (part of the key of code-object caches). */
int appy_hip_rtc_version(int* version_out);
void appy_hip_code_free(void* code);

/* Load a code object on the current device / look up an extern "C" kernel. */
int appy_hip_module_load(const void* code, size_t size, void** module_out);
int appy_hip_module_get_function(void* module, const char* kernel_name, void** func_out);
int appy_hip_module_unload(void* module);
int appy_hip_func_get_info(void* func, appy_hip_func_info* out);
/* Resident workgroups per CU for `func` at this block size / dynamic LDS. */
int appy_hip_occupancy(void* func, int block_threads, size_t dynamic_lds_bytes,
                       int* blocks_per_cu_out);

/* ---- device memory ------------------------------------------------------
 * Replaces `__tg_x = __tc_x.to('cuda')` and `__tc_x.copy_(__tg_x)`
 * (appy/backends/triton/passes/host_passes/gen_data_movement.py:25-87) for
 * NumPy / CPU-tensor arguments.  Buffers come from a size-bucketed pool so a
 * repeated call does not pay hipMalloc/hipFree; appy_hip_pool_trim releases
 * everything the pool holds.  appy_hip_free does not wait for the GPU: the
 * block may be handed out again at once, so synchronise the streams that still
 * use it first (appy_hip_memcpy_d2h and appy_hip_sync do). */
int appy_hip_malloc(size_t nbytes, void** dptr_out);
int appy_hip_free(void* dptr);
int appy_hip_pool_trim(void);
int appy_hip_pool_stats(uint64_t* bytes_in_use_out, uint64_t* bytes_cached_out);
/* Stream-ordered copies; both return after the copy has completed.  Host
 * memory from appy_hip_host_alloc moves as one DMA; any other (pageable) host
 * memory of 16 MiB or more is moved by four host threads through pinned staging
 * chunks on streams of their own, after the work queued on `stream` has
 * finished (set APPY_HIP_NO_STAGING=1 to use the driver's pageable path). */
int appy_hip_memcpy_h2d(void* dst_dev, const void* src_host, size_t nbytes, void* stream);
int appy_hip_memcpy_d2h(void* dst_host, const void* src_dev, size_t nbytes, void* stream);
/* Upload from page-locked memory (appy_hip_host_alloc; anything else is refused) that returns once the copy is
 * queued on `stream`: the caller leaves the host bytes alone until it has waited for the stream.  Used for the
 * one-element buffers of `shared()` scalars (appy/frontend/process_shared.py:27-53), which travel with every launch. */
int appy_hip_memcpy_h2d_async(void* dst_dev, const void* src_pinned, size_t nbytes, void* stream);
/* Page-locked host memory for arrays that travel often.  Replaces the device-
 * visible buffers behind the reference's shared NumPy arrays
 * (`device.buffer(n)` + `np.frombuffer`, appy/np_shared.py:11-17): on a
 * discrete GPU the array lives in pinned host memory and is mirrored in HBM.
 * appy_hip_host_is_pinned returns 1 if [p, p+nbytes) lies inside such a block. */
int appy_hip_host_alloc(size_t nbytes, void** host_out);
int appy_hip_host_free(void* host_ptr);
int appy_hip_host_is_pinned(const void* p, size_t nbytes);
int appy_hip_memcpy_d2d_async(void* dst_dev, const void* src_dev, size_t nbytes, void* stream);
int appy_hip_memset_async(void* dst_dev, int byte_value, size_t nbytes, void* stream);

/* ---- launch --------------------------------------------------------------
 * Replaces `_kernel_loop_N[grid](args..., num_warps=4)`
 * (appy/backends/triton/passes/host_passes/gen_kernel_launch.py:27-66).
 * `args` is the kernel's argument block laid out as the C struct of its
 * parameters (natural alignment); it is copied before the call returns. */
int appy_hip_launch(void* func,
                    uint32_t grid_x, uint32_t grid_y, uint32_t grid_z,
                    uint32_t block_x, uint32_t block_y, uint32_t block_z,
                    uint32_t dynamic_lds_bytes, void* stream,
                    const void* args, size_t args_bytes);
int appy_hip_sync(void* stream);               /* hipStreamSynchronize */
/* Wait for everything queued on the current device, on every stream (hipDeviceSynchronize): what a caller
 * does before it gives back memory that launches on streams it no longer knows may still use. */
int appy_hip_device_sync(void);

/* appy_hip_launch for a kernel that takes a scratch buffer among its arguments (the partial results
 * of a loop that runs as two kernels), without any allocation: the library keeps one buffer of
 * APPY_HIP_STATIC_SCRATCH_BYTES per GPU inside its own code object, and writes that buffer's address
 * over the 8 bytes at `scratch_arg_offset` of (its copy of) the argument block before the launch.
 * `scratch_bytes` is what the kernel will use of it: more than APPY_HIP_STATIC_SCRATCH_BYTES is refused
 * (invalid value), as is an argument block of more than 4096 bytes.
 * Nothing in the reference corresponds to this.  It is for callers that cannot call hipMalloc where
 * they launch: code under stream capture, serving loops with a fixed memory budget, harnesses that
 * forbid allocation.  Neither device nor host memory is allocated or freed by the call.
 * Every call on a GPU shares that GPU's buffer, which keeps what the last kernel left in it: kernels
 * must write what they read (the two-phase kernels generated here do), and two launches that use it
 * may not overlap on one GPU (same stream, or otherwise ordered by the caller). */
#define APPY_HIP_STATIC_SCRATCH_BYTES (8u << 20)
int appy_hip_launch_static_scratch(void* func,
                                   uint32_t grid_x, uint32_t grid_y, uint32_t grid_z,
                                   uint32_t block_x, uint32_t block_y, uint32_t block_z,
                                   uint32_t dynamic_lds_bytes, void* stream,
                                   const void* args, size_t args_bytes,
                                   size_t scratch_arg_offset, size_t scratch_bytes);

/* ---- row plans ------------------------------------------------------------
 * The reference runs the CSR loop of examples/03-spmv.py:5-16
 * (tests/integration/triton/tutorial/test_spmv.py:10-21) one row per program, every launch from the raw
 * arrays.  When the same arrays come back launch after launch, the order in which the elements of
 * `s += f(A[j], X[IDX[j]])` are walked can be worked out once ("inspector") and kept: a row plan.  A
 * generated kernel turns every position j of the streamed arrays into
 *     key  = (block of 2^APPY_HIP_ROWPLAN_ROW_BITS rows) << line_bits | (IDX[j] >> 5)   (0xFFFFFFFF: no element here)
 *     val  = bits of A[j] | (row within the block) << 32 | (IDX[j] & 31) << (32 + APPY_HIP_ROWPLAN_ROW_BITS)
 * and appy_hip_rowplan_build orders them, on `stream`, without waiting for it and without allocating:
 *   keys_sorted / elements   the pairs sorted by key (stable); `elements` is then rewritten in place to
 *                            bits of A[j] | (column within its group | slot << col_bits) << 32
 *   cell_start[cells + 1]    cell c = block c / groups, column range c % groups (`group_width` columns each):
 *                            elements [cell_start[c], cell_start[c + 1]); cell_start[cells] = all elements
 *   tile_base[cells + 1]     number of tiles (of `tile` elements, the last of a cell shorter) before cell c
 *   row_stream               per tile, at word (first element >> 1) + 4 * (tile number): one word
 *                            singles | runs << 16; the rows of the slots [0, singles) as 16-bit numbers
 *                            (rows that occur once in the tile); then runs + 1 words row | first slot <<
 *                            APPY_HIP_ROWPLAN_ROW_BITS of the rows that occur several times, whose elements
 *                            hold consecutive slots from `singles` on (the last word: the end)
 * Within a tile no row appears in two slots of the singles or in two runs, so a kernel may add the slots
 * to per-row sums with plain loads and stores.  appy_hip_rowplan_sizes gives the bytes of `sort_temp`, the
 * most tiles there can be and the words of `row_stream`.  Shapes that do not fit a 32-bit key or packed
 * word are refused (invalid value). */
#define APPY_HIP_ROWPLAN_ROW_BITS 15
typedef struct appy_hip_rowplan_shape {
    uint64_t entries;       /* positions of the streamed arrays (pairs to sort), < 2^31 */
    uint32_t row_blocks;    /* blocks of 2^APPY_HIP_ROWPLAN_ROW_BITS rows */
    uint32_t groups;        /* column ranges of X (8: one per XCD) */
    uint32_t group_width;   /* columns per range, a multiple of 32 */
    uint32_t col_bits;      /* bits of the column within its range in a packed word */
    uint32_t tile;          /* elements per tile: 4096 or 6144 */
    uint32_t line_bits;     /* bits of IDX[j] >> 5 in a key */
    uint32_t full;          /* 1: every position holds an element (no key is 0xFFFFFFFF), so the sort may leave
                               out the bit that only such keys have set - one pass less; 0: not known */
} appy_hip_rowplan_shape;
int appy_hip_rowplan_sizes(const appy_hip_rowplan_shape* shape, size_t* sort_temp_bytes_out, size_t* max_tiles_out,
                           size_t* stream_words_out);
int appy_hip_rowplan_build(const appy_hip_rowplan_shape* shape, const uint32_t* keys, const uint64_t* vals,
                           uint32_t* keys_sorted, uint64_t* elements, void* sort_temp, size_t sort_temp_bytes,
                           uint32_t* cell_start, uint32_t* tile_base, uint32_t* row_stream, void* stream);

/* ---- streams and graphs -----------------------------------------------------
 * A loop nest that launches many short kernels (a time-stepping host loop
 * around parallel loops, e.g. tests/integration/triton/npbench/test_jacobi_1d.py)
 * is bound by the host's launch rate.  The launches can be recorded once into a
 * HIP graph and replayed as one submission.  Nothing in the reference
 * corresponds to this (its launches go through Triton one at a time,
 * appy/backends/triton/passes/host_passes/gen_kernel_launch.py:27-66).
 * Streams have the default priority.  Between graph_begin and graph_end only
 * appy_hip_launch and appy_hip_memcpy_d2d_async may be issued on `stream`;
 * appy_hip_memset_async is refused while a capture is active on the stream. */
int appy_hip_stream_create(void** stream_out);
int appy_hip_stream_destroy(void* stream);
int appy_hip_graph_begin(void* stream);
int appy_hip_graph_end(void* stream, void** graph_exec_out);
int appy_hip_graph_launch(void* graph_exec, void* stream);
int appy_hip_graph_destroy(void* graph_exec);

/* ---- timing ---------------------------------------------------------------
 * Replaces torch.utils.benchmark.Timer in examples/benchmark_utils.py:4-15:
 * HIP events recorded on the stream the kernel is launched on. */
int appy_hip_event_create(void** event_out);
int appy_hip_event_record(void* event, void* stream);
int appy_hip_event_sync(void* event);
int appy_hip_event_elapsed_ms(void* start, void* stop, float* ms_out);
int appy_hip_event_destroy(void* event);
/* `reps` back-to-back launches of one kernel between two events, after
 * `warmup` untimed launches; *mean_ms_out = elapsed / reps. */
int appy_hip_launch_timed(void* func,
                          uint32_t grid_x, uint32_t grid_y, uint32_t grid_z,
                          uint32_t block_x, uint32_t block_y, uint32_t block_z,
                          uint32_t dynamic_lds_bytes, void* stream,
                          const void* args, size_t args_bytes,
                          int warmup, int reps, float* mean_ms_out);

#ifdef __cplusplus
}
#endif
#endif /* APPY_HIP_H */
