// Row plans: the part of libappy_hip.so that orders the elements of a sum over a gathered operand
// (`s += f(A[j], X[IDX[j]])` under a parallel loop over rows) once, so that later launches of the loop
// can walk them in an order that suits the memory system.
//
// A generated kernel has turned every element into a key (block of 32768 rows, 128-byte line of X) and a
// value (the 32 bits of A[j], the row within the block, the column within the line).  From those this file
// builds, all on the device and in a fixed order (no atomics: the same input gives the same plan):
//   1. the pairs sorted by key (stable radix sort);
//   2. cells - one block of rows x one of the `groups` column ranges of X - as ranges of the sorted pairs,
//      cut into tiles of `tile` elements;
//   3. per tile, the place ("slot") of every element in the order sorted by row, rows that occur once
//      first, then the runs of rows that occur several times; and the stream of row numbers in that order.
// The kernel that runs a plan gathers X in column order (adjacent lanes read the same lines), drops each
// product into its slot in LDS, and then adds the slots to the sums of their rows, also in LDS, one lane
// per row: no two lanes ever touch the same sum at once, so the result does not depend on timing.
#include "appy_hip.h"

#include <cstdint>
#include <cstring>
#include <string>

#include <hip/hip_runtime.h>
#include <rocprim/rocprim.hpp>

__attribute__((visibility("hidden"))) int appy_hip_internal_fail(hipError_t e, const char* what);
__attribute__((visibility("hidden"))) int appy_hip_internal_fail_arg(const char* what);

namespace {

#define PLAN_TRY(expr)                                                      \
    do {                                                                    \
        hipError_t e__ = (expr);                                            \
        if (e__ != hipSuccess) return appy_hip_internal_fail(e__, #expr);   \
    } while (0)

constexpr uint32_t ROW_BITS = APPY_HIP_ROWPLAN_ROW_BITS;
constexpr uint32_t BLOCK_ROWS = 1u << ROW_BITS;
constexpr uint32_t LINE_SHIFT = 5;      // 32 four-byte elements of X per 128-byte line

// first position whose key is not below `bound`
__device__ inline uint64_t lower_bound(const uint32_t* __restrict__ keys, uint64_t n, uint32_t bound) {
    uint64_t lo = 0, hi = n;
    while (lo < hi) {
        const uint64_t mid = (lo + hi) >> 1;
        if (keys[mid] < bound) lo = mid + 1; else hi = mid;
    }
    return lo;
}

// cell c = block c / groups, column range c % groups; cell_start[cells] = number of real elements
__global__ __launch_bounds__(256) void cell_bounds(const uint32_t* __restrict__ keys, uint64_t n, uint32_t cells,
                                                  uint32_t groups, uint32_t group_lines, uint32_t line_bits,
                                                  uint32_t* __restrict__ cell_start) {
    const uint32_t c = blockIdx.x * 256 + threadIdx.x;
    if (c > cells) return;
    const uint32_t b = c / groups, g = c % groups;
    cell_start[c] = (uint32_t)lower_bound(keys, n, (b << line_bits) | (g * group_lines));
}

// tile_base[c] = tiles of the cells before c; one workgroup
__global__ __launch_bounds__(1024) void tile_bases(const uint32_t* __restrict__ cell_start, uint32_t cells, uint32_t tile,
                                                  uint32_t* __restrict__ tile_base) {
    __shared__ uint32_t part[1024];
    const uint32_t per = (cells + 1023) / 1024;
    const uint32_t c0 = threadIdx.x * per;
    uint32_t sum = 0;
    for (uint32_t c = c0; c < c0 + per && c < cells; ++c) sum += (cell_start[c + 1] - cell_start[c] + tile - 1) / tile;
    part[threadIdx.x] = sum;
    __syncthreads();
    if (threadIdx.x == 0) {
        uint32_t run = 0;
        for (int t = 0; t < 1024; ++t) { const uint32_t v = part[t]; part[t] = run; run += v; }
    }
    __syncthreads();
    uint32_t run = part[threadIdx.x];
    for (uint32_t c = c0; c < c0 + per && c < cells; ++c) {
        tile_base[c] = run;
        run += (cell_start[c + 1] - cell_start[c] + tile - 1) / tile;
    }
    if (c0 < cells && c0 + per >= cells) tile_base[cells] = run;
    if (cells == 0 && threadIdx.x == 0) tile_base[0] = 0;
}

// where the row stream of a tile starts (32-bit words): half a word per element before it, four words per tile before it
__host__ __device__ inline uint64_t stream_word(uint64_t first_element, uint64_t tile_number) {
    return (first_element >> 1) + 4 * tile_number;
}

template <int U>
__global__ __launch_bounds__(1024) void build_tiles(const uint32_t* __restrict__ keys, uint64_t* __restrict__ ent,
                                                   const uint32_t* __restrict__ cell_start, const uint32_t* __restrict__ tile_base,
                                                   uint32_t cells, uint32_t groups, uint32_t group_width, uint32_t line_bits,
                                                   uint32_t col_bits, uint32_t* __restrict__ row_stream) {
    constexpr int T = U * 1024;
    using sort_t = rocprim::block_radix_sort<uint16_t, 1024, U, uint16_t>;
    using scan_t = rocprim::block_scan<uint64_t, 1024>;
    __shared__ union {
        typename sort_t::storage_type sort;
        typename scan_t::storage_type scan;
    } tmp;
    __shared__ uint16_t row_of[T + 2];      // rows in sorted order, a guard on either side
    __shared__ uint16_t slot_of[T];         // slot of the element at each position of the tile
    __shared__ uint32_t found_cell;

    const uint32_t ti = blockIdx.x;
    if (ti >= tile_base[cells]) return;
    if (threadIdx.x == 0) {
        uint32_t lo = 0, hi = cells;        // the last cell whose first tile is not beyond ti (cells without tiles are passed over)
        while (hi - lo > 1) {
            const uint32_t mid = (lo + hi) >> 1;
            if (tile_base[mid] <= ti) lo = mid; else hi = mid;
        }
        found_cell = lo;
    }
    __syncthreads();
    const uint32_t c = found_cell;
    const uint32_t g = c % groups;
    const uint64_t p0 = (uint64_t)cell_start[c] + (uint64_t)(ti - tile_base[c]) * T;
    const uint32_t left = cell_start[c + 1] - (uint32_t)p0;
    const uint32_t cnt = left < (uint32_t)T ? left : (uint32_t)T;
    const uint32_t line_mask = (1u << line_bits) - 1u;

    uint32_t carried[U], colg[U];
    uint16_t skey[U], sval[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
        const uint32_t i = threadIdx.x * U + u;
        if (i < cnt) {
            const uint32_t k = keys[p0 + i];
            const uint64_t v = ent[p0 + i];
            carried[u] = (uint32_t)v;
            colg[u] = (((k & line_mask) << LINE_SHIFT) | (uint32_t)((v >> (32 + ROW_BITS)) & 31u)) - g * group_width;
            skey[u] = (uint16_t)((v >> 32) & (BLOCK_ROWS - 1u));
        } else {
            carried[u] = 0; colg[u] = 0; skey[u] = 0xFFFFu;
        }
        sval[u] = (uint16_t)i;
    }
    sort_t().sort(skey, sval, tmp.sort, 0, 16);
    __syncthreads();
    if (threadIdx.x == 0) { row_of[0] = 0xFFFFu; row_of[T + 1] = 0xFFFFu; }
#pragma unroll
    for (int u = 0; u < U; ++u) row_of[1 + threadIdx.x * U + u] = skey[u];
    __syncthreads();
    // rows that occur once in the tile, elements of the other rows, first elements of those rows
    bool single[U], head[U];
    uint64_t mine = 0;
#pragma unroll
    for (int u = 0; u < U; ++u) {
        const uint32_t k = threadIdx.x * U + u;
        const bool valid = k < cnt;
        const bool first = valid && row_of[k] != skey[u];              // row_of[k] is the row before (guard for k = 0)
        const bool last = valid && (k + 1 >= cnt || row_of[k + 2] != skey[u]);
        single[u] = first && last;
        head[u] = first && !last;
        mine += (single[u] ? 1ull : 0ull) | ((valid && !single[u]) ? (1ull << 21) : 0ull) | (head[u] ? (1ull << 42) : 0ull);
    }
    uint64_t before = 0, total = 0;
    scan_t().exclusive_scan(mine, before, 0ull, total, tmp.scan);
    __syncthreads();
    const uint32_t ns = (uint32_t)(total & 0x1FFFFFu), nm = (uint32_t)(total >> 42);
    uint32_t at_single = (uint32_t)(before & 0x1FFFFFu), at_multi = (uint32_t)((before >> 21) & 0x1FFFFFu), at_head = (uint32_t)(before >> 42);
    uint32_t* seg = row_stream + stream_word(p0, ti);
    uint16_t* singles = reinterpret_cast<uint16_t*>(seg + 1);
    uint32_t* runs = seg + 1 + (ns + 1) / 2;
    if (threadIdx.x == 0) {
        seg[0] = ns | (nm << 16);
        runs[nm] = cnt << ROW_BITS;
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
        const uint32_t k = threadIdx.x * U + u;
        if (k >= cnt) continue;
        uint32_t slot;
        if (single[u]) {
            slot = at_single++;
            singles[slot] = skey[u];
        } else {
            slot = ns + at_multi++;
            if (head[u]) runs[at_head++] = (uint32_t)skey[u] | (slot << ROW_BITS);
        }
        slot_of[sval[u]] = (uint16_t)slot;
    }
    __syncthreads();
#pragma unroll
    for (int u = 0; u < U; ++u) {
        const uint32_t i = threadIdx.x * U + u;
        if (i < cnt)
            ent[p0 + i] = (uint64_t)carried[u] | ((uint64_t)(colg[u] | ((uint32_t)slot_of[i] << col_bits)) << 32);
    }
}

bool shape_ok(const appy_hip_rowplan_shape* s) {
    if (!s || s->groups == 0 || s->groups > 64 || s->group_width == 0 || s->group_width % 32 != 0) return false;
    if (s->tile != 4096 && s->tile != 6144) return false;
    // a packed word holds the column within the group and the slot within the tile
    uint32_t slot_bits = s->tile <= 4096 ? 12 : 13;
    if (s->col_bits + slot_bits > 32 || (1ull << s->col_bits) < s->group_width) return false;
    if (s->line_bits == 0 || s->line_bits > 27) return false;
    if ((uint64_t)s->groups * (s->group_width >> LINE_SHIFT) > (1ull << s->line_bits)) return false;
    // keys of real elements stay below 2^31: the key of a position without an element (all ones) sorts behind them
    if (s->row_blocks == 0 || ((uint64_t)s->row_blocks << s->line_bits) > (1ull << 31)) return false;
    if (s->entries == 0 || s->entries >= (1ull << 31)) return false;
    return true;
}

uint32_t key_bits(const appy_hip_rowplan_shape* s) {
    uint32_t bits = s->line_bits;
    while ((1ull << bits) < ((uint64_t)s->row_blocks << s->line_bits)) ++bits;
    return bits + (s->full ? 0 : 1);        // and the bit that only positions without an element have set
}

}  // namespace

extern "C" {

int appy_hip_rowplan_sizes(const appy_hip_rowplan_shape* shape, size_t* sort_temp_bytes_out, size_t* max_tiles_out,
                           size_t* stream_words_out) {
    if (!shape_ok(shape) || !sort_temp_bytes_out || !max_tiles_out || !stream_words_out) return appy_hip_internal_fail_arg("rowplan shape");
    size_t temp = 0;
    PLAN_TRY(rocprim::radix_sort_pairs(nullptr, temp, (uint32_t*)nullptr, (uint32_t*)nullptr, (uint64_t*)nullptr, (uint64_t*)nullptr,
                                       (size_t)shape->entries, 0u, key_bits(shape), (hipStream_t) nullptr));
    const size_t cells = (size_t)shape->row_blocks * shape->groups;
    const size_t tiles = shape->entries / shape->tile + cells + 1;
    *sort_temp_bytes_out = temp ? temp : 256;
    *max_tiles_out = tiles;
    *stream_words_out = (size_t)(shape->entries >> 1) + 4 * tiles + 8;
    return 0;
}

int appy_hip_rowplan_build(const appy_hip_rowplan_shape* shape, const uint32_t* keys, const uint64_t* vals,
                           uint32_t* keys_sorted, uint64_t* elements, void* sort_temp, size_t sort_temp_bytes,
                           uint32_t* cell_start, uint32_t* tile_base, uint32_t* row_stream, void* stream) {
    if (!shape_ok(shape) || !keys || !vals || !keys_sorted || !elements || !sort_temp || !cell_start || !tile_base || !row_stream)
        return appy_hip_internal_fail_arg("rowplan build");
    hipStream_t s = static_cast<hipStream_t>(stream);
    size_t temp = sort_temp_bytes;
    PLAN_TRY(rocprim::radix_sort_pairs(sort_temp, temp, keys, keys_sorted, vals, elements, (size_t)shape->entries, 0u,
                                       key_bits(shape), s));
    const uint32_t cells = shape->row_blocks * shape->groups;
    cell_bounds<<<(cells + 1 + 255) / 256, 256, 0, s>>>(keys_sorted, shape->entries, cells, shape->groups,
                                                       shape->group_width >> LINE_SHIFT, shape->line_bits, cell_start);
    PLAN_TRY(hipGetLastError());
    tile_bases<<<1, 1024, 0, s>>>(cell_start, cells, shape->tile, tile_base);
    PLAN_TRY(hipGetLastError());
    const uint32_t tiles = (uint32_t)(shape->entries / shape->tile + cells + 1);
    if (shape->tile == 4096)
        build_tiles<4><<<tiles, 1024, 0, s>>>(keys_sorted, elements, cell_start, tile_base, cells, shape->groups, shape->group_width,
                                             shape->line_bits, shape->col_bits, row_stream);
    else
        build_tiles<6><<<tiles, 1024, 0, s>>>(keys_sorted, elements, cell_start, tile_base, cells, shape->groups, shape->group_width,
                                             shape->line_bits, shape->col_bits, row_stream);
    PLAN_TRY(hipGetLastError());
    return 0;
}

}  // extern "C"
