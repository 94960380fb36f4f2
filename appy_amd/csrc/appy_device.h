// appy_device.h - device-side support code for generated kernels (gfx950).
//
// This text is placed in front of every generated kernel before it is handed
// to hiprtc, so it may only use compiler builtins and the HIP device headers.
// Wavefronts are 64 lanes wide; a "team" is a power-of-two group of adjacent
// lanes (2..64) that executes one iteration of a parallel loop together.
#if !defined(__HIPCC_RTC__)
#include <hip/hip_runtime.h>  // hiprtc has the device API built in; hipcc needs the header
#endif

namespace appy {

typedef long long i64;

// ---- unaligned-tolerant vector access ---------------------------------------
// Element-aligned vectors: global memory accepts dwordx2/x4 accesses at any
// element-aligned address, so rows that start at arbitrary offsets can still be
// streamed with wide loads.
template <typename T, int V>
struct vec {
    typedef T type __attribute__((ext_vector_type(V), aligned(alignof(T))));
};

template <typename T, int V>
__device__ __forceinline__ typename vec<T, V>::type vload(const T* p) {
    return *reinterpret_cast<const typename vec<T, V>::type*>(p);
}

template <typename T, int V>
__device__ __forceinline__ void vstore(T* p, typename vec<T, V>::type v) {
    *reinterpret_cast<typename vec<T, V>::type*>(p) = v;
}

// LDS tiles are 16-byte aligned and indexed in whole vectors: naturally aligned
// vector types give single ds_read_b128 / ds_write_b128 accesses.
template <typename T, int V>
struct avec {
    typedef T type __attribute__((ext_vector_type(V)));
};

template <typename T, int V>
__device__ __forceinline__ typename vec<T, V>::type lds_vload(const T* p) {
    typename avec<T, V>::type a = *reinterpret_cast<const typename avec<T, V>::type*>(p);
    typename vec<T, V>::type r;
#pragma unroll
    for (int k = 0; k < V; ++k) r[k] = a[k];
    return r;
}

template <typename T, int V>
__device__ __forceinline__ void lds_vstore(T* p, typename vec<T, V>::type v) {
    typename avec<T, V>::type a;
#pragma unroll
    for (int k = 0; k < V; ++k) a[k] = v[k];
    *reinterpret_cast<typename avec<T, V>::type*>(p) = a;
}

// Streaming variants: data that is touched once should not displace reused
// lines (x of SpMV/GEMV, B rows of SpMM) from the L2.
template <typename T, int V>
__device__ __forceinline__ typename vec<T, V>::type vload_stream(const T* p) {
    return __builtin_nontemporal_load(reinterpret_cast<const typename vec<T, V>::type*>(p));
}

template <typename T, int V>
__device__ __forceinline__ void vstore_stream(T* p, typename vec<T, V>::type v) {
    __builtin_nontemporal_store(v, reinterpret_cast<typename vec<T, V>::type*>(p));
}

template <typename T>
__device__ __forceinline__ T load_stream(const T* p) {
    return __builtin_nontemporal_load(p);
}

// ---- bounds-checked kernels --------------------------------------------------------
// A checked kernel never leaves its arrays: an index outside its dimension is
// reported (site number + 1 in *oob; any offending site may win) and the load
// goes to element 0 instead, the store is dropped.  The host turns the report
// into an IndexError after the launch.
__device__ __forceinline__ bool inside(i64 idx, i64 extent) { return idx >= 0 && idx < extent; }

__device__ __forceinline__ void report(int* oob, int site) { *oob = site + 1; }

__device__ __forceinline__ i64 at(i64 idx, i64 extent, int site, int* oob) {
    if (inside(idx, extent)) return idx;
    report(oob, site);
    return 0;
}

// ---- Python arithmetic that differs from C ------------------------------------
// (integer division by zero gives 0, as NumPy's floor_divide and remainder do)
template <typename T>
__device__ __forceinline__ T floordiv_int(T a, T b) {
    if (b == 0) return 0;
    T q = a / b;
    T r = a % b;
    return ((r != 0) && ((r < 0) != (b < 0))) ? q - 1 : q;
}

template <typename T>
__device__ __forceinline__ T mod_int(T a, T b) {
    if (b == 0) return 0;
    T r = a % b;
    return ((r != 0) && ((r < 0) != (b < 0))) ? r + b : r;
}

template <typename T>
__device__ __forceinline__ T div_unsigned(T a, T b) {
    return b == 0 ? (T)0 : (T)(a / b);
}

template <typename T>
__device__ __forceinline__ T mod_unsigned(T a, T b) {
    return b == 0 ? (T)0 : (T)(a % b);
}

// Floating-point `%` and `//` follow NumPy's (and CPython's) divmod: the remainder comes from
// fmod, which is exact, and the quotient is derived from it, so that a / b rounding up to
// a whole number does not push the floor one too high.
__device__ __forceinline__ float mod_float(float a, float b) {
    float r = fmodf(a, b);
    if (r != 0.0f) return ((r < 0.0f) != (b < 0.0f)) ? r + b : r;
    return (b == 0.0f) ? r : copysignf(0.0f, b);
}

__device__ __forceinline__ double mod_float(double a, double b) {
    double r = fmod(a, b);
    if (r != 0.0) return ((r < 0.0) != (b < 0.0)) ? r + b : r;
    return (b == 0.0) ? r : copysign(0.0, b);
}

__device__ __forceinline__ float floordiv_float(float a, float b) {
    if (b == 0.0f) return a / b;
    const float r = fmodf(a, b);
    float div = (a - r) / b;
    if (r != 0.0f && ((b < 0.0f) != (r < 0.0f))) div -= 1.0f;
    if (div == 0.0f) return copysignf(0.0f, a / b);
    float q = floorf(div);
    if (div - q > 0.5f) q += 1.0f;
    return q;
}

__device__ __forceinline__ double floordiv_float(double a, double b) {
    if (b == 0.0) return a / b;
    const double r = fmod(a, b);
    double div = (a - r) / b;
    if (r != 0.0 && ((b < 0.0) != (r < 0.0))) div -= 1.0;
    if (div == 0.0) return copysign(0.0, a / b);
    double q = floor(div);
    if (div - q > 0.5) q += 1.0;
    return q;
}

template <typename T>
__device__ __forceinline__ T ipow(T base, i64 e) {
    T r = (T)1;
    if (e < 0) return (T)0;
    while (e) {
        if (e & 1) r *= base;
        base *= base;
        e >>= 1;
    }
    return r;
}

// ---- reduction operators --------------------------------------------------------
struct OpAdd {
    template <typename T>
    __device__ static __forceinline__ T f(T a, T b) { return a + b; }
};
struct OpMul {
    template <typename T>
    __device__ static __forceinline__ T f(T a, T b) { return a * b; }
};
struct OpMax {  // Python's max(a, b): b only if it is greater
    template <typename T>
    __device__ static __forceinline__ T f(T a, T b) { return (b > a) ? b : a; }
};
struct OpMin {
    template <typename T>
    __device__ static __forceinline__ T f(T a, T b) { return (b < a) ? b : a; }
};

// ---- cross-lane movement ----------------------------------------------------------
// DPP controls (GFX9): quad_perm[1,0,3,2]=0xB1, quad_perm[2,3,0,1]=0x4E,
// row_half_mirror=0x141, row_mirror=0x140.  All four stay inside a row of 16
// lanes, so teams of up to 16 lanes reduce without touching the LDS crossbar.
template <int CTRL>
__device__ __forceinline__ int dpp_i32(int x) {
    return __builtin_amdgcn_update_dpp(x, x, CTRL, 0xf, 0xf, false);
}

template <int CTRL, typename T>
__device__ __forceinline__ T dpp_move(T v) {
    static_assert(sizeof(T) == 4 || sizeof(T) == 8, "cross-lane values are 4 or 8 bytes");
    if constexpr (sizeof(T) == 4) {
        return __builtin_bit_cast(T, dpp_i32<CTRL>(__builtin_bit_cast(int, v)));
    } else {
        unsigned long long u = __builtin_bit_cast(unsigned long long, v);
        unsigned lo = (unsigned)dpp_i32<CTRL>((int)(unsigned)(u & 0xffffffffull));
        unsigned hi = (unsigned)dpp_i32<CTRL>((int)(unsigned)(u >> 32));
        return __builtin_bit_cast(T, ((unsigned long long)hi << 32) | (unsigned long long)lo);
    }
}

template <typename T>
__device__ __forceinline__ T lane_xor(T v, int mask) {
    static_assert(sizeof(T) == 4 || sizeof(T) == 8, "cross-lane values are 4 or 8 bytes");
    const int src = ((int)__lane_id() ^ mask) << 2;
    if constexpr (sizeof(T) == 4) {
        return __builtin_bit_cast(T, __builtin_amdgcn_ds_bpermute(src, __builtin_bit_cast(int, v)));
    } else {
        unsigned long long u = __builtin_bit_cast(unsigned long long, v);
        unsigned lo = (unsigned)__builtin_amdgcn_ds_bpermute(src, (int)(unsigned)(u & 0xffffffffull));
        unsigned hi = (unsigned)__builtin_amdgcn_ds_bpermute(src, (int)(unsigned)(u >> 32));
        return __builtin_bit_cast(T, ((unsigned long long)hi << 32) | (unsigned long long)lo);
    }
}

// Butterfly reduction over a team of W adjacent lanes (W = 1,2,4,...,64, teams
// aligned to W).  Every lane of the team must be active; every lane returns the
// same total.
template <typename Op, int W, typename T>
__device__ __forceinline__ T team_reduce(T v) {
    static_assert(W >= 1 && W <= 64 && (W & (W - 1)) == 0, "team width is a power of two up to 64");
    if constexpr (W >= 2) v = Op::f(v, dpp_move<0xB1>(v));
    if constexpr (W >= 4) v = Op::f(v, dpp_move<0x4E>(v));
    if constexpr (W >= 8) v = Op::f(v, dpp_move<0x141>(v));
    if constexpr (W >= 16) v = Op::f(v, dpp_move<0x140>(v));
    if constexpr (W >= 32) v = Op::f(v, lane_xor(v, 16));
    if constexpr (W >= 64) v = Op::f(v, lane_xor(v, 32));
    return v;
}

// The same butterfly for a width that is only known at run time (the same for the whole
// wavefront: rows binned by length are dealt to wavefronts class by class).
template <typename Op, typename T>
__device__ __forceinline__ T team_reduce_dyn(T v, int w) {
    if (w >= 2) v = Op::f(v, dpp_move<0xB1>(v));
    if (w >= 4) v = Op::f(v, dpp_move<0x4E>(v));
    if (w >= 8) v = Op::f(v, dpp_move<0x141>(v));
    if (w >= 16) v = Op::f(v, dpp_move<0x140>(v));
    if (w >= 32) v = Op::f(v, lane_xor(v, 16));
    if (w >= 64) v = Op::f(v, lane_xor(v, 32));
    return v;
}

// Running maximum over the lanes of a team of W adjacent lanes (lane k gets the maximum of
// lanes 0..k of its team).  Every lane of the team must be active.
template <int W>
__device__ __forceinline__ i64 team_running_max(i64 v, int lane) {
    static_assert(W >= 1 && W <= 64 && (W & (W - 1)) == 0, "team width is a power of two up to 64");
#pragma unroll
    for (int d = 1; d < W; d <<= 1) {
        const int src = ((int)__lane_id() - d) << 2;
        const unsigned long long u = (unsigned long long)v;
        const unsigned lo = (unsigned)__builtin_amdgcn_ds_bpermute(src, (int)(unsigned)(u & 0xffffffffull));
        const unsigned hi = (unsigned)__builtin_amdgcn_ds_bpermute(src, (int)(unsigned)(u >> 32));
        const i64 o = (i64)(((unsigned long long)hi << 32) | (unsigned long long)lo);
        if (lane >= d && o > v) v = o;
    }
    return v;
}

// The value of the lane below in a team of W adjacent lanes (lane 0 of a team gets an unspecified value).
template <int W>
__device__ __forceinline__ i64 team_lane_below(i64 v, int lane) {
    const int src = ((int)__lane_id() - 1) << 2;
    const unsigned long long u = (unsigned long long)v;
    const unsigned lo = (unsigned)__builtin_amdgcn_ds_bpermute(src, (int)(unsigned)(u & 0xffffffffull));
    const unsigned hi = (unsigned)__builtin_amdgcn_ds_bpermute(src, (int)(unsigned)(u >> 32));
    (void)lane;
    return (i64)(((unsigned long long)hi << 32) | (unsigned long long)lo);
}

// A number that is the same in every lane, kept in scalar registers whatever it was computed from: with such an offset
// from a kernel argument, loads at `base + offset + lane offset` take the scalar-base form of the memory instructions
// (one 32-bit register per lane for the lane's offset instead of a 64-bit address worked out per lane).
// A 64-bit index as a 32-bit one; what does not fit becomes -1 (kernels that group elements drop negative indices).
__device__ __forceinline__ int narrow_index(long long v) {
    return v >= 0 && v <= 0x7fffffffll ? (int)v : -1;
}
__device__ __forceinline__ vec<int, 4>::type narrow_indices(vec<long long, 4>::type v) {
    vec<int, 4>::type r;
#pragma unroll
    for (int k = 0; k < 4; ++k) r[k] = narrow_index(v[k]);
    return r;
}

__device__ __forceinline__ unsigned lane_offset(unsigned v) {
    // (the compiler may not look through this: a lane's offset stays one 32-bit register next to the scalar base, where it
    //  would otherwise widen offsets chosen under a condition to 64 bits and add the base lane by lane)
    asm("" : "+v"(v));
    return v;
}

__device__ __forceinline__ i64 uniform_i64(i64 v) {
    const unsigned long long u = (unsigned long long)v;
    const unsigned lo = (unsigned)__builtin_amdgcn_readfirstlane((int)(unsigned)(u & 0xffffffffull));
    const unsigned hi = (unsigned)__builtin_amdgcn_readfirstlane((int)(unsigned)(u >> 32));
    return (i64)(((unsigned long long)hi << 32) | (unsigned long long)lo);
}

// Between two loops that the lanes of one wavefront share: what any lane stored in the first is
// visible to every lane in the second, and nothing of the second is started before the first is
// through.  The hardware runs the lanes in lockstep; this keeps the compiler from moving one
// lane's loads and stores of the second loop over those of the first when it can prove that
// lane's own addresses distinct (the overlap is between lanes).  No instruction is generated.
__device__ __forceinline__ void wave_fence() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// Workgroup reduction: wavefront butterfly, one LDS slot per wavefront, then a
// butterfly over the slots.  Must be reached by every thread of the workgroup.
// The total is returned in every lane of wavefront 0 (only).
template <typename Op, int BLOCK, typename T>
__device__ __forceinline__ T block_reduce(T v, T identity) {
    static_assert(BLOCK % 64 == 0 && BLOCK <= 1024, "workgroup is a whole number of wavefronts");
    constexpr int NW = BLOCK / 64;
    v = team_reduce<Op, 64>(v);
    if constexpr (NW == 1) {
        return v;
    } else {
        __shared__ T slots[NW];
        const int wave = threadIdx.x >> 6;
        const int lane = threadIdx.x & 63;
        if (lane == 0) slots[wave] = v;
        __syncthreads();
        T r = identity;
        if (wave == 0) {
            r = (lane < NW) ? slots[lane] : identity;
            constexpr int W2 = NW <= 2 ? 2 : NW <= 4 ? 4 : NW <= 8 ? 8 : 16;
            r = team_reduce<Op, W2>(r);
        }
        __syncthreads();  // slots may be reused by the next reduction
        return r;
    }
}

// Workgroup reduction whose total is returned in every thread (a team that
// spans the whole workgroup).  Must be reached by every thread.
template <typename Op, int BLOCK, typename T>
__device__ __forceinline__ T workgroup_reduce_all(T v, T identity) {
    static_assert(BLOCK % 64 == 0 && BLOCK <= 1024, "workgroup is a whole number of wavefronts");
    constexpr int NW = BLOCK / 64;
    v = team_reduce<Op, 64>(v);
    if constexpr (NW == 1) {
        return v;
    } else {
        __shared__ T slots[NW];
        const int wave = threadIdx.x >> 6;
        const int lane = threadIdx.x & 63;
        if (lane == 0) slots[wave] = v;
        __syncthreads();
        constexpr int W2 = NW <= 2 ? 2 : NW <= 4 ? 4 : NW <= 8 ? 8 : 16;
        const int slot = lane & (W2 - 1);   // every aligned group of W2 lanes reduces the same NW slots
        T r = (slot < NW) ? slots[slot] : identity;
        r = team_reduce<Op, W2>(r);
        __syncthreads();                    // slots may be reused by the next reduction
        return r;
    }
}

// ---- atomics on device memory -------------------------------------------------------
template <int N>
struct uint_of;
template <>
struct uint_of<4> {
    typedef unsigned int type;
};
template <>
struct uint_of<8> {
    typedef unsigned long long type;
};

template <typename Op, typename T>
__device__ __forceinline__ void atomic_cas_combine(T* p, T v) {
    typedef typename uint_of<sizeof(T)>::type U;
    U* up = reinterpret_cast<U*>(p);
    U seen = __hip_atomic_load(up, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    for (;;) {
        const T next = Op::f(__builtin_bit_cast(T, seen), v);
        const U want = __builtin_bit_cast(U, next);
        if (want == seen) return;
        if (__hip_atomic_compare_exchange_strong(up, &seen, want, __ATOMIC_RELAXED, __ATOMIC_RELAXED,
                                                 __HIP_MEMORY_SCOPE_AGENT))
            return;
    }
}

// 8- and 16-bit elements: compare-and-swap on the aligned 32-bit word that holds the element
// (device allocations are whole multiples of four bytes, so the word is inside the allocation).
template <int N>
struct small_uint_of;
template <>
struct small_uint_of<1> {
    typedef unsigned char type;
};
template <>
struct small_uint_of<2> {
    typedef unsigned short type;
};

template <typename Op, typename T>
__device__ __forceinline__ void atomic_subword_combine(T* p, T v) {
    typedef typename small_uint_of<sizeof(T)>::type U;
    const unsigned long long addr = reinterpret_cast<unsigned long long>(p);
    unsigned int* word = reinterpret_cast<unsigned int*>(addr & ~3ull);
    const unsigned int shift = static_cast<unsigned int>(addr & 3ull) * 8u;
    const unsigned int mask = (sizeof(T) == 1 ? 0xFFu : 0xFFFFu) << shift;
    unsigned int seen = __hip_atomic_load(word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    for (;;) {
        const T cur = __builtin_bit_cast(T, static_cast<U>((seen & mask) >> shift));
        const T next = Op::f(cur, v);
        const unsigned int want = (seen & ~mask) | (static_cast<unsigned int>(__builtin_bit_cast(U, next)) << shift);
        if (want == seen) return;
        if (__hip_atomic_compare_exchange_strong(word, &seen, want, __ATOMIC_RELAXED, __ATOMIC_RELAXED,
                                                 __HIP_MEMORY_SCOPE_AGENT))
            return;
    }
}

template <typename Op, typename T, int N = sizeof(T)>
struct atomic_combine {
    __device__ static __forceinline__ void run(T* p, T v) { atomic_cas_combine<Op, T>(p, v); }
};
template <typename Op, typename T>
struct atomic_combine<Op, T, 1> {
    __device__ static __forceinline__ void run(T* p, T v) { atomic_subword_combine<Op, T>(p, v); }
};
template <typename Op, typename T>
struct atomic_combine<Op, T, 2> {
    __device__ static __forceinline__ void run(T* p, T v) { atomic_subword_combine<Op, T>(p, v); }
};
template <typename T>
struct atomic_combine<OpAdd, T, 4> {  // hardware add for 32/64-bit integers, float and double
    __device__ static __forceinline__ void run(T* p, T v) {
        __hip_atomic_fetch_add(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
};
template <typename T>
struct atomic_combine<OpAdd, T, 8> {
    __device__ static __forceinline__ void run(T* p, T v) {
        __hip_atomic_fetch_add(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
};

}  // namespace appy
