// kernel for spmv_kernel_loop_1_rkeys: team_b256_v1_u1_w64_r_rkeys_R256
extern "C" __global__ void __launch_bounds__(256)
_spmv_kernel_loop_1_rkeys(
    const int* __restrict__ A_indptr,
    const float* __restrict__ A_data,
    const float* __restrict__ x,
    const int* __restrict__ A_indices,
    float* __restrict__ y,
    unsigned* __keys,
    unsigned long long* __vals,
    const appy::i64 __len,
    const appy::i64 __nx,
    const int __lbits,
    long long* __flag,
    const appy::i64 __lo,
    const appy::i64 __hi)
{
    const int __lid = threadIdx.x & 63;
    const int __wvl = threadIdx.x >> 6;
    __shared__ int __lp_all[4][257];      // where the rows of the block start; the last entry: where it ends
    __shared__ int __hq_all[4][257];      // where they end
    int* __lp = __lp_all[__wvl];
    int* __hq = __hq_all[__wvl];
    const appy::i64 __nblk = (__hi - __lo + 255) / 256;
    for (appy::i64 __b = (appy::i64)blockIdx.x * 4 + __wvl; __b < __nblk; __b += (appy::i64)gridDim.x * 4) {
        const appy::i64 __r0 = __lo + __b * 256;
        const int __nr = (int)((__hi - __r0) < 256 ? (__hi - __r0) : 256);
        appy::wave_fence();       // the block before this one has been read out of __lp
        bool __good = true;
        #pragma unroll
        for (int __k = 0; __k < 5; ++__k) {      // and the first row of the next block, if there is one
            const int __r = __k * 64 + __lid;
            if (__r <= __nr && __r0 + __r < __hi && (__k < 4 || __lid == 0)) {
                const appy::i64 i = __r0 + __r;
                int start = 0;
                int end = 0;
                double s = 0;
                start = A_indptr[i];
                end = A_indptr[(i + 1LL)];
                s = 0.0;
                const appy::i64 __rlo = ((long long)(start));
                const appy::i64 __rhi = ((long long)(end));
                if (__rlo < 0 || __rhi < __rlo || __rhi > __len) __good = false;
                __lp[__r] = (int)__rlo;
                if (__r < __nr) __hq[__r] = (int)__rhi;
            }
        }
        appy::wave_fence();
        // every row ends where the next one starts; the block ends no later than the next one starts
        #pragma unroll
        for (int __k = 0; __k < 4; ++__k) {
            const int __r = __k * 64 + __lid;
            if (__r < __nr - 1) __good = __good && __lp[__r + 1] == __hq[__r];
            else if (__r == __nr - 1 && __r0 + __nr < __hi) __good = __good && __lp[__nr] >= __hq[__r];
        }
        __good = __ballot(!__good) == 0ull;
        const int __first = __good ? __lp[0] : 0, __end = __good ? __hq[__nr - 1] : 0;
        appy::wave_fence();
        #pragma unroll
        for (int __k = 0; __k < 5; ++__k) {
            const int __r = __k * 64 + __lid;
            if (__r >= __nr && __r <= 256 && (__k < 4 || __lid == 0)) __lp[__r] = __end;
        }
        appy::wave_fence();
        if (!__good) {
            if (__lid == 0) __flag[0] = 1;
            continue;
        }
        // (how many positions the rows of all blocks cover: when it is every position, no key stays unset and the sort needs a bit less)
        if (__lid == 0) atomicAdd(reinterpret_cast<unsigned long long*>(__flag) + 1, (unsigned long long)(__end - __first));
        const unsigned __rel0 = (unsigned)(__b * 256);       // first row of the block, counted from the start of the range
        bool __inside = true;
        for (int __j0 = __first; __j0 < __end; __j0 += 1024) {
            #pragma unroll
            for (int __k = 0; __k < 4; ++__k) {
                const int __j = __j0 + __k * 256 + __lid * 4;
                if (__j >= __end) continue;
                appy::vec<int, 4>::type __c;
                appy::vec<int, 4>::type __v;
                if (__j + 4 <= __end) __c = appy::vload<int, 4>(A_indices + __j);
                else {
                #pragma unroll
                    for (int __q = 0; __q < 4; ++__q) __c[__q] = __j + __q < __end ? A_indices[__j + __q] : 0;
                }
                if (__j + 4 <= __end) __v = appy::vload<int, 4>(reinterpret_cast<const int*>(A_data) + __j);
                else {
                #pragma unroll
                    for (int __q = 0; __q < 4; ++__q) __v[__q] = __j + __q < __end ? reinterpret_cast<const int*>(A_data)[__j + __q] : 0;
                }
                int __row = 0, __past = 256;       // the last row that starts at or before __j
                #pragma unroll
                for (int __it = 0; __it < 8; ++__it) {
                    const int __mid = (__row + __past) >> 1;
                    if (__lp[__mid] <= __j) __row = __mid; else __past = __mid;
                }
                appy::vec<unsigned, 4>::type __kq;
                appy::vec<unsigned long long, 4>::type __vq;
                bool __all = __j + 4 <= __end;
                #pragma unroll
                for (int __q = 0; __q < 4; ++__q) {
                    if (__j + __q < __end) while (__lp[__row + 1] <= __j + __q) ++__row;
                    const int __cq = __c[__q];
                    const bool __in = __cq >= 0 && __cq < __nx;
                    if (__j + __q < __end && !__in) __inside = false;
                    __all = __all && __in;
                    const unsigned __rel = __rel0 + (unsigned)__row;
                    __kq[__q] = ((__rel >> 15) << __lbits) | ((unsigned)__cq >> 5);
                    __vq[__q] = (unsigned long long)(unsigned)__v[__q] | ((unsigned long long)((__rel & 32767u) | (((unsigned)__cq & 31u) << 15)) << 32);
                }
                if (__all) {
                    appy::vstore<unsigned, 4>(__keys + __j, __kq);
                    appy::vstore<unsigned long long, 4>(__vals + __j, __vq);
                } else {
                #pragma unroll
                    for (int __q = 0; __q < 4; ++__q) {
                        const int __cq = __c[__q];
                        if (__j + __q < __end && __cq >= 0 && __cq < __nx) { __keys[__j + __q] = __kq[__q]; __vals[__j + __q] = __vq[__q]; }
                    }
                }
            }
        }
        if (__ballot(!__inside) != 0ull && __lid == 0) __flag[0] = 1;      // an index outside the gathered operand: no plan
    }
}
