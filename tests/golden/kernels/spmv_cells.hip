// kernel for spmv_kernel_loop_1_cells: team_b256_v1_u1_w64_r_s8_cells_R256_if1
extern "C" __global__ void __launch_bounds__(256)
_spmv_kernel_loop_1_cells(
    const int* __restrict__ A_indptr,
    const float* __restrict__ A_data,
    const float* __restrict__ x,
    const int* __restrict__ A_indices,
    float* __restrict__ y,
    const long long* __ent,
    const int* __desc,
    const int __shiftc,
    double* __scratch,
    const long long* __flag,
    const appy::i64 __lo,
    const appy::i64 __hi)
{
    if ((__flag[0] != 0) == true) return;
    const int __lid = threadIdx.x & 63;
    const int __wvl = threadIdx.x >> 6;
    __shared__ float __acc_all[4][256];        // the sums of the rows of a cell, one cell per wavefront
    float* __acc = __acc_all[__wvl];
    const appy::i64 __nblk = (__hi - __lo + 255) / 256;
    // workgroup g serves the stripes g mod 8, g mod 8 + 8, ...: workgroups go to the eight XCDs in turn, so every L2
    // holds one stripe of the gathered operand at a time
    const appy::i64 __w0 = (appy::i64)(blockIdx.x >> 3) * 4 + __wvl, __nw = (appy::i64)(gridDim.x >> 3) * 4;
    for (int __pass = 0; __pass < 1; ++__pass) {
        const int __s = (int)(blockIdx.x & 7) + 8 * __pass;
        const appy::i64 __x0 = (appy::i64)__s << __shiftc;
        for (appy::i64 __b = __w0; __b < __nblk; __b += __nw) {
            const int __clo = __desc[__b * 9 + __s], __chi = __desc[__b * 9 + __s + 1];
            #pragma unroll
            for (int __k = 0; __k < 4; ++__k) __acc[__k * 64 + __lid] = 0;
            appy::wave_fence();
            for (int __j0 = __clo; __j0 < __chi; __j0 += 512) {
                long long __e[8];
                float __xv[8];
                #pragma unroll
                for (int __k = 0; __k < 8; ++__k) {
                    const int __j = __j0 + __k * 64 + __lid;
                    __e[__k] = __j < __chi ? __builtin_nontemporal_load(__ent + __j) : 0ll;
                }
                #pragma unroll
                for (int __k = 0; __k < 8; ++__k) {
                    const int __j = __j0 + __k * 64 + __lid;
                    __xv[__k] = x[__j < __chi ? __x0 + (appy::i64)((unsigned)((unsigned long long)__e[__k] >> 32) & 0x3fffffu) : 0];
                }
                #pragma unroll
                for (int __k = 0; __k < 8; ++__k) {
                    const int __j = __j0 + __k * 64 + __lid;
                    if (__j < __chi) {
                        const float __cv = __int_as_float((int)(unsigned)(unsigned long long)__e[__k]);
                        const float __cx = __xv[__k];
                        atomicAdd(&__acc[(unsigned)((unsigned long long)__e[__k] >> 54)], (__cv * __cx));
                    }
                }
            }
            appy::wave_fence();
            #pragma unroll
            for (int __k = 0; __k < 4; ++__k) {
                const appy::i64 __row = __b * 256 + __k * 64 + __lid;
                if (__row < __hi - __lo) reinterpret_cast<float*>(__scratch)[(appy::i64)__s * (__hi - __lo) + __row] = __acc[__k * 64 + __lid];
            }
            appy::wave_fence();
        }
    }
}
