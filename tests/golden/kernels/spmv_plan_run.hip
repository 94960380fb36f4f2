// kernel for spmv_kernel_loop_1_xcells: team_b1024_v1_u6_w1024_r_s8_xcells
extern "C" __global__ void __launch_bounds__(1024)
_spmv_kernel_loop_1_xcells(
    const int* __restrict__ A_indptr,
    const float* __restrict__ A_data,
    const float* __restrict__ x,
    const int* __restrict__ A_indices,
    float* __restrict__ y,
    const unsigned long long* __restrict__ __ent,
    const unsigned* __restrict__ __cstart,
    const unsigned* __restrict__ __tbase,
    const unsigned* __restrict__ __rstream,
    const appy::i64 __ncell,
    const appy::i64 __split,
    const unsigned* __restrict__ __order,
    const appy::i64 __norder,
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
    // A cell may be shared by __split workgroups, each with a run of its tiles and a slot of its own for the sums: a
    // run is numbered (block * __split + part) * 8 + range.  The workgroup takes the runs that the entries blockIdx.x,
    // blockIdx.x + gridDim.x, ... of __order name (dealt out on the host by size; the grid is a multiple of eight
    // workgroups and all runs of a workgroup read the same range) and walks their tiles as one sequence, so that
    // the loads of a run's first tiles travel while the run before it is finished.
    const unsigned __nrun = (unsigned)(__ncell * __split), __spl = (unsigned)__split;
    const unsigned __g = blockIdx.x & 7u;
    const unsigned __x0 = __g * (unsigned)__gwidth;
    #pragma unroll
    for (int __k = 0; __k < 32; ++__k) __sum[__k * 1024 + __tid] = 0;
    unsigned long long __e0[6], __e1[6], __e2[6];
    float __xv[6], __x1[6];
    unsigned __r0[3], __r1[3];
    unsigned __da0, __db0, __da1, __db1;
    unsigned __h0, __h1, __hv2;        // headers of the tiles in flight (the newest as it was loaded, in a vector register)
    // the tile the next load fetches: run, tile within the run; of the run: its tiles, where its elements and its row
    // stream start, the elements from there to the end of the cell
    unsigned __vi = blockIdx.x, __tt = 0, __nt = 0;
    unsigned __vc = __vi < __norder ? __order[__vi] : 0xffffffffu;        // (no run: a number beyond them all)
    appy::i64 __eb = 0, __sb = 0;      // (in bytes from the start of the elements and of the row stream)
    const char* __entb = reinterpret_cast<const char*>(__ent);
    const char* __rsb = reinterpret_cast<const char*>(__rstream);
    appy::i64 __left = 0;
    // of the tiles in flight (0: the one that is added up, 1: the one whose gathers travel, 2: the one just requested):
    // whether it exists, its elements, whether it ends its run, the run, its part of the row stream
    bool __in0, __in1, __in2, __end0, __end1, __end2, __any0, __any1, __any2;
    unsigned __cnt0, __cnt1, __cnt2, __run0, __run1, __run2;
    appy::i64 __ps0, __ps1, __ps2;
    if (__vc < __nrun) {
        const unsigned __b = (__vc >> 3) / __spl, __part = (__vc >> 3) % __spl;
        const appy::i64 __cell = (appy::i64)__b * 8 + __g;
        const unsigned __nta = __tbase[__cell + 1] - __tbase[__cell];
        const unsigned __tlo = __part * __nta / __spl;        // (at most 32 parts, and tiles of thousands of elements)
        __nt = (__part + 1) * __nta / __spl - __tlo;
        const appy::i64 __cs = (appy::i64)__cstart[__cell] + (appy::i64)__tlo * 6144;
        __left = (appy::i64)__cstart[__cell + 1] - __cs;
        __eb = __cs * 8;
        __sb = ((__cs >> 1) + 4 * ((appy::i64)__tbase[__cell] + __tlo)) * 4;
    } else {
        __nt = 0;
    }
    {
      __any2 = __vc < __nrun; __in2 = __any2 && __tt < __nt; __end2 = __tt + 1 >= __nt; __run2 = __vc;
      const char* __p = __entb + appy::uniform_i64(__in2 ? __eb + (appy::i64)__tt * 49152 : 0);
      __ps2 = appy::uniform_i64(__in2 ? __sb + (appy::i64)__tt * 12304 : 0);
      __hv2 = *reinterpret_cast<const unsigned*>(__rsb + __ps2 + appy::lane_offset(0u));
      const appy::i64 __l = __left - (appy::i64)__tt * 6144;
      __cnt2 = __in2 ? (unsigned)(__l < 6144 ? __l : 6144) : 0u;
    #pragma unroll
      for (int __u = 0; __u < 6; ++__u)
          __e0[__u] = __builtin_nontemporal_load(reinterpret_cast<const unsigned long long*>(__p + appy::lane_offset(__in2 ? (unsigned)((__u * 1024 + __tid) * 8) : 0u)));
      if (__any2) {
          if (!__end2) ++__tt;
          else {
              __vi += gridDim.x; __vc = __vi < __norder ? __order[__vi] : 0xffffffffu; __tt = 0;
                if (__vc < __nrun) {
                    const unsigned __b = (__vc >> 3) / __spl, __part = (__vc >> 3) % __spl;
                    const appy::i64 __cell = (appy::i64)__b * 8 + __g;
                    const unsigned __nta = __tbase[__cell + 1] - __tbase[__cell];
                    const unsigned __tlo = __part * __nta / __spl;        // (at most 32 parts, and tiles of thousands of elements)
                    __nt = (__part + 1) * __nta / __spl - __tlo;
                    const appy::i64 __cs = (appy::i64)__cstart[__cell] + (appy::i64)__tlo * 6144;
                    __left = (appy::i64)__cstart[__cell + 1] - __cs;
                    __eb = __cs * 8;
                    __sb = ((__cs >> 1) + 4 * ((appy::i64)__tbase[__cell] + __tlo)) * 4;
                } else {
                    __nt = 0;
                }
          }
      }
    }
    __h0 = __builtin_amdgcn_readfirstlane(__hv2);
    __in0 = __in2; __end0 = __end2; __any0 = __any2; __cnt0 = __cnt2; __run0 = __run2; __ps0 = __ps2;
    {
      __any2 = __vc < __nrun; __in2 = __any2 && __tt < __nt; __end2 = __tt + 1 >= __nt; __run2 = __vc;
      const char* __p = __entb + appy::uniform_i64(__in2 ? __eb + (appy::i64)__tt * 49152 : 0);
      __ps2 = appy::uniform_i64(__in2 ? __sb + (appy::i64)__tt * 12304 : 0);
      __hv2 = *reinterpret_cast<const unsigned*>(__rsb + __ps2 + appy::lane_offset(0u));
      const appy::i64 __l = __left - (appy::i64)__tt * 6144;
      __cnt2 = __in2 ? (unsigned)(__l < 6144 ? __l : 6144) : 0u;
    #pragma unroll
      for (int __u = 0; __u < 6; ++__u)
          __e1[__u] = __builtin_nontemporal_load(reinterpret_cast<const unsigned long long*>(__p + appy::lane_offset(__in2 ? (unsigned)((__u * 1024 + __tid) * 8) : 0u)));
      if (__any2) {
          if (!__end2) ++__tt;
          else {
              __vi += gridDim.x; __vc = __vi < __norder ? __order[__vi] : 0xffffffffu; __tt = 0;
                if (__vc < __nrun) {
                    const unsigned __b = (__vc >> 3) / __spl, __part = (__vc >> 3) % __spl;
                    const appy::i64 __cell = (appy::i64)__b * 8 + __g;
                    const unsigned __nta = __tbase[__cell + 1] - __tbase[__cell];
                    const unsigned __tlo = __part * __nta / __spl;        // (at most 32 parts, and tiles of thousands of elements)
                    __nt = (__part + 1) * __nta / __spl - __tlo;
                    const appy::i64 __cs = (appy::i64)__cstart[__cell] + (appy::i64)__tlo * 6144;
                    __left = (appy::i64)__cstart[__cell + 1] - __cs;
                    __eb = __cs * 8;
                    __sb = ((__cs >> 1) + 4 * ((appy::i64)__tbase[__cell] + __tlo)) * 4;
                } else {
                    __nt = 0;
                }
          }
      }
    }
    __h1 = __builtin_amdgcn_readfirstlane(__hv2);
    __in1 = __in2; __end1 = __end2; __any1 = __any2; __cnt1 = __cnt2; __run1 = __run2; __ps1 = __ps2;
    {
    #pragma unroll
      for (int __u = 0; __u < 3; ++__u)
          __r0[__u] = __builtin_nontemporal_load(reinterpret_cast<const unsigned*>(__rsb + __ps0 + appy::lane_offset(__in0 ? (unsigned)((1 + __u * 1024 + __tid) * 4) : 0u)));
      const unsigned __runs = (__h0 >> 16);
      const char* __q = __rsb + (__ps0 + (__in0 ? (appy::i64)(1 + (((__h0 & 0xffffu) + 1) >> 1)) * 4 : 0));     // (the header of a tile that does not exist may hold anything)
      const unsigned __at = appy::lane_offset(__in0 && __tid < __runs ? __tid * 4 : 0u);        // (lanes without a run: one position)
      __da0 = *reinterpret_cast<const unsigned*>(__q + __at);
      __db0 = *reinterpret_cast<const unsigned*>(__q + __at + 4); }
    {
    #pragma unroll
      for (int __u = 0; __u < 6; ++__u) {
        unsigned __c = __x0 + ((unsigned)(__e0[__u] >> 32) & __cmask);
        __c = __c < __xlast ? __c : __xlast;        // (what was read beyond the cell may hold anything)
        __xv[__u] = *reinterpret_cast<const float*>(__xb + appy::lane_offset(__in0 ? (unsigned)(__c << 2) : 0u));
      } }
    __syncthreads();
    while (__any0) {
        const unsigned __ns = __in0 ? __h0 & 0xffffu : 0u, __nm = __in0 ? __h0 >> 16 : 0u;
        {
          __any2 = __vc < __nrun; __in2 = __any2 && __tt < __nt; __end2 = __tt + 1 >= __nt; __run2 = __vc;
          const char* __p = __entb + appy::uniform_i64(__in2 ? __eb + (appy::i64)__tt * 49152 : 0);
          __ps2 = appy::uniform_i64(__in2 ? __sb + (appy::i64)__tt * 12304 : 0);
          __hv2 = *reinterpret_cast<const unsigned*>(__rsb + __ps2 + appy::lane_offset(0u));
          const appy::i64 __l = __left - (appy::i64)__tt * 6144;
          __cnt2 = __in2 ? (unsigned)(__l < 6144 ? __l : 6144) : 0u;
        #pragma unroll
          for (int __u = 0; __u < 6; ++__u)
              __e2[__u] = __builtin_nontemporal_load(reinterpret_cast<const unsigned long long*>(__p + appy::lane_offset(__in2 ? (unsigned)((__u * 1024 + __tid) * 8) : 0u)));
          if (__any2) {
              if (!__end2) ++__tt;
              else {
                  __vi += gridDim.x; __vc = __vi < __norder ? __order[__vi] : 0xffffffffu; __tt = 0;
                    if (__vc < __nrun) {
                        const unsigned __b = (__vc >> 3) / __spl, __part = (__vc >> 3) % __spl;
                        const appy::i64 __cell = (appy::i64)__b * 8 + __g;
                        const unsigned __nta = __tbase[__cell + 1] - __tbase[__cell];
                        const unsigned __tlo = __part * __nta / __spl;        // (at most 32 parts, and tiles of thousands of elements)
                        __nt = (__part + 1) * __nta / __spl - __tlo;
                        const appy::i64 __cs = (appy::i64)__cstart[__cell] + (appy::i64)__tlo * 6144;
                        __left = (appy::i64)__cstart[__cell + 1] - __cs;
                        __eb = __cs * 8;
                        __sb = ((__cs >> 1) + 4 * ((appy::i64)__tbase[__cell] + __tlo)) * 4;
                    } else {
                        __nt = 0;
                    }
              }
          }
        }
        if (__cnt0 == 6144u) {
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
                if (__u * 1024 + __tid < __cnt0) __prod[(unsigned)(__e0[__u] >> 32) >> __colbits] = __val;
            }
        }
        {
        #pragma unroll
          for (int __u = 0; __u < 3; ++__u)
              __r1[__u] = __builtin_nontemporal_load(reinterpret_cast<const unsigned*>(__rsb + __ps1 + appy::lane_offset(__in1 ? (unsigned)((1 + __u * 1024 + __tid) * 4) : 0u)));
          const unsigned __runs = (__h1 >> 16);
          const char* __q = __rsb + (__ps1 + (__in1 ? (appy::i64)(1 + (((__h1 & 0xffffu) + 1) >> 1)) * 4 : 0));     // (the header of a tile that does not exist may hold anything)
          const unsigned __at = appy::lane_offset(__in1 && __tid < __runs ? __tid * 4 : 0u);        // (lanes without a run: one position)
          __da1 = *reinterpret_cast<const unsigned*>(__q + __at);
          __db1 = *reinterpret_cast<const unsigned*>(__q + __at + 4); }
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
        {
        #pragma unroll
          for (int __u = 0; __u < 3; ++__u) {
            unsigned __c = __x0 + ((unsigned)(__e1[__u] >> 32) & __cmask);
            __c = __c < __xlast ? __c : __xlast;        // (what was read beyond the cell may hold anything)
            __x1[__u] = *reinterpret_cast<const float*>(__xb + appy::lane_offset(__in1 ? (unsigned)(__c << 2) : 0u));
          } }
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
                const unsigned* __runs = reinterpret_cast<const unsigned*>(__rsb + __ps0) + 1 + ((__ns + 1) >> 1);
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
        {
        #pragma unroll
          for (int __u = 3; __u < 6; ++__u) {
            unsigned __c = __x0 + ((unsigned)(__e1[__u] >> 32) & __cmask);
            __c = __c < __xlast ? __c : __xlast;        // (what was read beyond the cell may hold anything)
            __x1[__u] = *reinterpret_cast<const float*>(__xb + appy::lane_offset(__in1 ? (unsigned)(__c << 2) : 0u));
          } }
        __syncthreads();
        if (__end0) {
            // the run is through: its sums go out and start again at zero (every lane clears what it has read itself; the next
            // tile's terms are added after the barrier that follows their scatter)
            const unsigned __b = (__run0 >> 3) / __spl, __part = (__run0 >> 3) % __spl;
            float* __out = reinterpret_cast<float*>(__scratch) + ((appy::i64)__part * 8 + __g) * __n + (appy::i64)__b * 32768;
            if (((appy::i64)__b + 1) * 32768 <= __n) {
            #pragma unroll
                for (int __k = 0; __k < 32; ++__k) { __out[__k * 1024 + __tid] = __sum[__k * 1024 + __tid]; __sum[__k * 1024 + __tid] = 0; }
            } else {
                for (int __k = 0; __k < 32; ++__k) {
                    if ((appy::i64)__b * 32768 + __k * 1024 + __tid < __n) __out[__k * 1024 + __tid] = __sum[__k * 1024 + __tid];
                    __sum[__k * 1024 + __tid] = 0;
                }
            }
        }
        #pragma unroll
        for (int __u = 0; __u < 6; ++__u) { __e0[__u] = __e1[__u]; __e1[__u] = __e2[__u]; __xv[__u] = __x1[__u]; }
        #pragma unroll
        for (int __u = 0; __u < 3; ++__u) __r0[__u] = __r1[__u];
        __h0 = __h1; __h1 = __builtin_amdgcn_readfirstlane(__hv2); __da0 = __da1; __db0 = __db1;
        __in0 = __in1; __end0 = __end1; __any0 = __any1; __cnt0 = __cnt1; __run0 = __run1; __ps0 = __ps1;
        __in1 = __in2; __end1 = __end2; __any1 = __any2; __cnt1 = __cnt2; __run1 = __run2; __ps1 = __ps2;
    }
}
