// kernel for spmv_kernel_loop_1_group: team_b256_v1_u1_w64_r_s8_group_R256
extern "C" __global__ void __launch_bounds__(256)
_spmv_kernel_loop_1_group(
    const int* __restrict__ A_indptr,
    const float* __restrict__ A_data,
    const float* __restrict__ x,
    const int* __restrict__ A_indices,
    float* __restrict__ y,
    long long* __ent,
    int* __desc,
    const int __shiftc,
    const appy::i64 __len,
    const appy::i64 __rowmax,
    long long* __hint,
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
    const int __cmask = (1 << __shiftc) - 1;
    for (appy::i64 __b = (appy::i64)blockIdx.x * 4 + __wvl; __b < __nblk; __b += (appy::i64)gridDim.x * 4) {
        const appy::i64 __r0 = __lo + __b * 256;
        const int __nr = (int)((__hi - __r0) < 256 ? (__hi - __r0) : 256);
        appy::wave_fence();       // the block before this one has been read out of __lp
        bool __good = true, __long = false;
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
                if (__r < __nr) { __hq[__r] = (int)__rhi; __long = __long || (__rhi - __rlo > __rowmax); }
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
        if (__ballot(__long) != 0ull && __lid == 0) __hint[0] = 2;      // rows too long for this treatment: the next launch sorts them
        const int __first = __good ? __lp[0] : 0, __end = __good ? __hq[__nr - 1] : 0;
        appy::wave_fence();
        #pragma unroll
        for (int __k = 0; __k < 5; ++__k) {
            const int __r = __k * 64 + __lid;
            if (__r >= __nr && __r <= 256 && (__k < 4 || __lid == 0)) __lp[__r] = __end;
        }
        appy::wave_fence();
        if (!__good) {
            // refused: the launch runs the loop row by row instead; the cells of this block stay empty
            if (__lid == 0) __flag[0] = 1;
            if (__lid <= 8) __desc[__b * 9 + __lid] = 0;
            continue;
        }
        int __cnt[8], __at[9];
        #pragma unroll
        for (int __s = 0; __s < 8; ++__s) __cnt[__s] = 0;
        for (int __j0 = __first; __j0 < __end; __j0 += 1024) {
            appy::vec<int, 4>::type __c[4];
            #pragma unroll
            for (int __k = 0; __k < 4; ++__k) {
                { const int __j = __j0 + __k * 256 + __lid * 4;
                if (__j + 4 <= __end) __c[__k] = appy::vload<int, 4>(A_indices + __j);
                else {
                #pragma unroll
                    for (int __q = 0; __q < 4; ++__q) __c[__k][__q] = __j + __q < __end ? A_indices[__j + __q] : -1;
                } }
            }
            #pragma unroll
            for (int __k = 0; __k < 4; ++__k) {
                #pragma unroll
                for (int __q = 0; __q < 4; ++__q)
                #pragma unroll
                    for (int __s = 0; __s < 8; ++__s) __cnt[__s] += __popcll(__ballot((__c[__k][__q] >> __shiftc) == __s));
            }
        }
        __at[0] = __first;
        #pragma unroll
        for (int __s = 0; __s < 8; ++__s) __at[__s + 1] = __at[__s] + __cnt[__s];
        #pragma unroll
        for (int __s = 0; __s <= 8; ++__s) if (__lid == __s) __desc[__b * 9 + __s] = __at[__s];
        int __atv = 0;       // lane s: where the next element of stripe s goes
        #pragma unroll
        for (int __s = 0; __s < 8; ++__s) __atv = __lid == __s ? __at[__s] : __atv;
        for (int __j0 = __first; __j0 < __end; __j0 += 1024) {
            appy::vec<int, 4>::type __c[4], __v[4];
            #pragma unroll
            for (int __k = 0; __k < 4; ++__k) {
                { const int __j = __j0 + __k * 256 + __lid * 4;
                if (__j + 4 <= __end) __c[__k] = appy::vload<int, 4>(A_indices + __j);
                else {
                #pragma unroll
                    for (int __q = 0; __q < 4; ++__q) __c[__k][__q] = __j + __q < __end ? A_indices[__j + __q] : -1;
                } }
                { const int __j = __j0 + __k * 256 + __lid * 4;
                if (__j + 4 <= __end) __v[__k] = appy::vload<int, 4>(reinterpret_cast<const int*>(A_data) + __j);
                else {
                #pragma unroll
                    for (int __q = 0; __q < 4; ++__q) __v[__k][__q] = __j + __q < __end ? reinterpret_cast<const int*>(A_data)[__j + __q] : 0;
                } }
            }
            #pragma unroll
            for (int __k = 0; __k < 4; ++__k) {
                const int __j = __j0 + __k * 256 + __lid * 4;
                int __row = 0, __past = 256;       // the last row that starts at or before __j
                #pragma unroll
                for (int __it = 0; __it < 8; ++__it) {
                    const int __mid = (__row + __past) >> 1;
                    if (__lp[__mid] <= __j) __row = __mid; else __past = __mid;
                }
                #pragma unroll
                for (int __q = 0; __q < 4; ++__q) {
                    if (__j + __q < __end) while (__lp[__row + 1] <= __j + __q) ++__row;
                    const int __cq = __c[__k][__q];
                    const int __sq = __cq >> __shiftc;          // negative past the end (and for negative indices: such elements are dropped)
                    const bool __ok = __sq >= 0 && __sq < 8;
                    const unsigned long long __okm = __ballot(__ok);
                    unsigned __olo = (unsigned)__okm, __ohi = (unsigned)(__okm >> 32);
                    #pragma unroll
                    for (int __bit = 0; __bit < 3; ++__bit) {
                        const unsigned __e = (unsigned)((__sq << (31 - __bit)) >> 31);       // all ones where the bit is set
                        const unsigned long long __bm = __ballot(__e != 0u);
                        __olo &= ~((unsigned)__bm ^ __e);
                        __ohi &= ~((unsigned)(__bm >> 32) ^ __e);
                    }
                    const int __pos = __builtin_amdgcn_ds_bpermute(__sq << 2, __atv) + (int)__builtin_amdgcn_mbcnt_hi(__ohi, __builtin_amdgcn_mbcnt_lo(__olo, 0u));
                    // every lane tells the lane of its stripe how many elements the stripe takes in this step (all of them the same
                    // number; a lane that no one tells receives zero; a lane without an element tells what holds for the number it has)
                    __atv += __builtin_amdgcn_ds_permute(__sq << 2, __popc(__olo) + __popc(__ohi));
                    if (__ok)
                        __ent[__pos] = (long long)(((unsigned long long)(((unsigned)__row << 22) | (unsigned)(__cq & __cmask)) << 32) | (unsigned long long)(unsigned)__v[__k][__q]);
                }
            }
        }
    }
}
