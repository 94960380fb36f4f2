// kernel for spmv_kernel_loop_1_xcells: team_b1024_v1_u6_w1024_r_s8_xcells
extern "C" __global__ void __launch_bounds__(1024)
_spmv_kernel_loop_1_xcells(
    const int* __restrict__ A_indptr,
    const float* __restrict__ A_data,
    const float* __restrict__ x,
    const int* __restrict__ A_indices,
    float* __restrict__ y,
    const unsigned long long* __ent,
    const unsigned* __cstart,
    const unsigned* __tbase,
    const unsigned* __rstream,
    const appy::i64 __ncell,
    const appy::i64 __split,
    const appy::i64 __gwidth,
    const int __colbits,
    const appy::i64 __nx,
    double* __scratch,
    const appy::i64 __lo,
    const appy::i64 __hi)
{
    const unsigned __tid = threadIdx.x;
    __shared__ float __sum[32768];        // the sums of the rows of the cell
    __shared__ __attribute__((aligned(8))) float __prod[6144];       // the terms of a tile, sorted by row
    const appy::i64 __n = __hi - __lo;
    const unsigned __cmask = (1u << __colbits) - 1u;
    const unsigned __xlast = (unsigned)(__nx - 1);
    const char* __xb = reinterpret_cast<const char*>(x);
    // a cell may be shared by __split workgroups, each with a run of its tiles and a slot of its own for the sums
    for (appy::i64 __vc = blockIdx.x; __vc < __ncell * __split; __vc += gridDim.x) {
        const int __g = (int)(__vc & 7);
        const appy::i64 __b = (__vc >> 3) / __split;
        const int __part = (int)((__vc >> 3) % __split);
        const appy::i64 __cell = __b * 8 + __g;
        const appy::i64 __ce = __cstart[__cell + 1];
        const int __nta = (int)(__tbase[__cell + 1] - __tbase[__cell]);
        const int __tlo = (int)((appy::i64)__part * __nta / __split), __nt = (int)((appy::i64)(__part + 1) * __nta / __split) - __tlo;
        const appy::i64 __cs = (appy::i64)__cstart[__cell] + (appy::i64)__tlo * 6144;
        const unsigned __x0 = (unsigned)(__g * __gwidth);
        // tile t of this workgroup: elements at __eb + t * TILE, row stream at __sb + t * SEG
        const char* __eb = reinterpret_cast<const char*>(__ent + __cs);
        const char* __sb = reinterpret_cast<const char*>(__rstream + ((__cs >> 1) + 4 * ((appy::i64)__tbase[__cell] + __tlo)));
        #pragma unroll
        for (int __k = 0; __k < 32; ++__k) __sum[__k * 1024 + __tid] = 0;
        unsigned long long __e0[6], __e1[6], __e2[6];
        float __xv[6], __x1[6];
        unsigned __r0[3], __r1[3];
        unsigned __da0, __db0, __da1, __db1;
        unsigned __h0, __h1, __h2;
        { const bool __in = (0) < __nt;
          const char* __p = __eb + (appy::i64)(0) * 49152;
        #pragma unroll
          for (int __u = 0; __u < 6; ++__u)
              __e0[__u] = __builtin_nontemporal_load(reinterpret_cast<const unsigned long long*>(__p + (__in ? (unsigned)((__u * 1024 + __tid) * 8) : 0u)));
          __h0 = __builtin_amdgcn_readfirstlane(*reinterpret_cast<const unsigned*>(__sb + (appy::i64)(0) * 12304)); }
        { const bool __in = (1) < __nt;
          const char* __p = __eb + (appy::i64)(1) * 49152;
        #pragma unroll
          for (int __u = 0; __u < 6; ++__u)
              __e1[__u] = __builtin_nontemporal_load(reinterpret_cast<const unsigned long long*>(__p + (__in ? (unsigned)((__u * 1024 + __tid) * 8) : 0u)));
          __h1 = __builtin_amdgcn_readfirstlane(*reinterpret_cast<const unsigned*>(__sb + (appy::i64)(1) * 12304)); }
        { const bool __in = (0) < __nt;
          const char* __p = __sb + (appy::i64)(0) * 12304;
        #pragma unroll
          for (int __u = 0; __u < 3; ++__u)
              __r0[__u] = __builtin_nontemporal_load(reinterpret_cast<const unsigned*>(__p + (__in ? (unsigned)((1 + __u * 1024 + __tid) * 4) : 0u)));
          const unsigned __runs = (__h0 >> 16);
          const char* __q = __p + (__in ? (appy::i64)(1 + (((__h0 & 0xffffu) + 1) >> 1)) * 4 : 0);     // (a header beyond the run of tiles may hold anything)
          const unsigned __at = __in && __tid < __runs ? __tid * 4 : 0u;        // (lanes without a run: one position)
          __da0 = *reinterpret_cast<const unsigned*>(__q + __at);
          __db0 = *reinterpret_cast<const unsigned*>(__q + __at + 4); }
        { const bool __in = (0) < __nt;
        #pragma unroll
          for (int __u = 0; __u < 6; ++__u) {
            unsigned __c = __x0 + ((unsigned)(__e0[__u] >> 32) & __cmask);
            __c = __c < __xlast ? __c : __xlast;        // (what was read beyond the cell may hold anything)
            __xv[__u] = *reinterpret_cast<const float*>(__xb + (__in ? (unsigned)(__c << 2) : 0u));
          } }
        __syncthreads();
        for (int __t = 0; __t < __nt; ++__t) {
            const appy::i64 __left = __ce - (__cs + (appy::i64)__t * 6144);
            const unsigned __cnt = (unsigned)(__left < 6144 ? __left : 6144);
            const unsigned __ns = __h0 & 0xffffu, __nm = __h0 >> 16;
            if (__cnt == 6144u) {
            #pragma unroll
                for (int __u = 0; __u < 6; ++__u) {
                    float __val;
                    { const float __cv = __int_as_float((int)(unsigned)(__e0[__u])); const float __cx = __xv[__u]; __val = (__cv * __cx); }
                    __prod[(unsigned)(__e0[__u] >> 32) >> __colbits] = __val;
                }
            } else {
            #pragma unroll
                for (int __u = 0; __u < 6; ++__u) {
                    float __val;
                    { const float __cv = __int_as_float((int)(unsigned)(__e0[__u])); const float __cx = __xv[__u]; __val = (__cv * __cx); }
                    if (__u * 1024 + __tid < __cnt) __prod[(unsigned)(__e0[__u] >> 32) >> __colbits] = __val;
                }
            }
            // the elements of the tile after the next, the row numbers and the gathers of the next one travel while this one is added up
            { const bool __in = (__t + 2) < __nt;
              const char* __p = __eb + (appy::i64)(__t + 2) * 49152;
            #pragma unroll
              for (int __u = 0; __u < 6; ++__u)
                  __e2[__u] = __builtin_nontemporal_load(reinterpret_cast<const unsigned long long*>(__p + (__in ? (unsigned)((__u * 1024 + __tid) * 8) : 0u)));
              __h2 = __builtin_amdgcn_readfirstlane(*reinterpret_cast<const unsigned*>(__sb + (appy::i64)(__t + 2) * 12304)); }
            { const bool __in = (__t + 1) < __nt;
              const char* __p = __sb + (appy::i64)(__t + 1) * 12304;
            #pragma unroll
              for (int __u = 0; __u < 3; ++__u)
                  __r1[__u] = __builtin_nontemporal_load(reinterpret_cast<const unsigned*>(__p + (__in ? (unsigned)((1 + __u * 1024 + __tid) * 4) : 0u)));
              const unsigned __runs = (__h1 >> 16);
              const char* __q = __p + (__in ? (appy::i64)(1 + (((__h1 & 0xffffu) + 1) >> 1)) * 4 : 0);     // (a header beyond the run of tiles may hold anything)
              const unsigned __at = __in && __tid < __runs ? __tid * 4 : 0u;        // (lanes without a run: one position)
              __da1 = *reinterpret_cast<const unsigned*>(__q + __at);
              __db1 = *reinterpret_cast<const unsigned*>(__q + __at + 4); }
            { const bool __in = (__t + 1) < __nt;
            #pragma unroll
              for (int __u = 0; __u < 6; ++__u) {
                unsigned __c = __x0 + ((unsigned)(__e1[__u] >> 32) & __cmask);
                __c = __c < __xlast ? __c : __xlast;        // (what was read beyond the cell may hold anything)
                __x1[__u] = *reinterpret_cast<const float*>(__xb + (__in ? (unsigned)(__c << 2) : 0u));
              } }
            __syncthreads();
            {
                float __sa[3], __sb_[3];
                appy::vec<float, 2>::type __pp[3];
            #pragma unroll
                for (int __u = 0; __u < 3; ++__u) {
                    __pp[__u] = *reinterpret_cast<const appy::vec<float, 2>::type*>(&__prod[2 * (__u * 1024 + __tid)]);
                    __sa[__u] = __sum[__r0[__u] & 0x7fffu]; __sb_[__u] = __sum[(__r0[__u] >> 16) & 0x7fffu];
                }
            #pragma unroll
                for (int __u = 0; __u < 3; ++__u) {
                    const unsigned __s = 2 * (__u * 1024 + __tid);
                    if (__s < __ns) __sum[__r0[__u] & 0x7fffu] = __sa[__u] + __pp[__u][0];
                    if (__s + 1 < __ns) __sum[(__r0[__u] >> 16) & 0x7fffu] = __sb_[__u] + __pp[__u][1];
                }
            }
            if (__nm > 0) {
                if (__tid < __nm) {
                    { const int __row = (int)(__da0 & 32767u), __from = (int)(__da0 >> 15), __to = (int)(__db0 >> 15);
                      float __acc = __sum[__row];
                      for (int __k = __from; __k < __to; __k += 4) {
                          const float __p0 = __prod[__k], __p1 = __k + 1 < __to ? __prod[__k + 1] : 0, __p2 = __k + 2 < __to ? __prod[__k + 2] : 0, __p3 = __k + 3 < __to ? __prod[__k + 3] : 0;
                          __acc += __p0;
                          if (__k + 1 < __to) __acc += __p1;
                          if (__k + 2 < __to) __acc += __p2;
                          if (__k + 3 < __to) __acc += __p3;
                      }
                      __sum[__row] = __acc; }
                }
                if (__nm > 1024) {
                    const unsigned* __runs = reinterpret_cast<const unsigned*>(__sb + (appy::i64)__t * 12304) + 1 + ((__ns + 1) >> 1);
                    for (unsigned __m = __tid + 1024; __m < __nm; __m += 1024) {
                        const unsigned __d = __runs[__m], __d1 = __runs[__m + 1];
                        { const int __row = (int)(__d & 32767u), __from = (int)(__d >> 15), __to = (int)(__d1 >> 15);
                          float __acc = __sum[__row];
                          for (int __k = __from; __k < __to; __k += 4) {
                              const float __p0 = __prod[__k], __p1 = __k + 1 < __to ? __prod[__k + 1] : 0, __p2 = __k + 2 < __to ? __prod[__k + 2] : 0, __p3 = __k + 3 < __to ? __prod[__k + 3] : 0;
                              __acc += __p0;
                              if (__k + 1 < __to) __acc += __p1;
                              if (__k + 2 < __to) __acc += __p2;
                              if (__k + 3 < __to) __acc += __p3;
                          }
                          __sum[__row] = __acc; }
                    }
                }
            }
            __syncthreads();
            #pragma unroll
            for (int __u = 0; __u < 6; ++__u) { __e0[__u] = __e1[__u]; __e1[__u] = __e2[__u]; __xv[__u] = __x1[__u]; }
            #pragma unroll
            for (int __u = 0; __u < 3; ++__u) __r0[__u] = __r1[__u];
            __h0 = __h1; __h1 = __h2; __da0 = __da1; __db0 = __db1;
        }
        float* __out = reinterpret_cast<float*>(__scratch) + ((appy::i64)__part * 8 + __g) * __n + __b * 32768;
        if ((__b + 1) * 32768 <= __n) {
        #pragma unroll
            for (int __k = 0; __k < 32; ++__k) __out[__k * 1024 + __tid] = __sum[__k * 1024 + __tid];
        } else {
            for (int __k = 0; __k < 32; ++__k)
                if (__b * 32768 + __k * 1024 + __tid < __n) __out[__k * 1024 + __tid] = __sum[__k * 1024 + __tid];
        }
        __syncthreads();
    }
}
