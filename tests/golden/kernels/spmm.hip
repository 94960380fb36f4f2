// kernel for spmm_kernel_loop_1: team_b256_v4_u1_w32_r_e128
extern "C" __global__ void __launch_bounds__(256)
_spmm_kernel_loop_1(
    const int* __restrict__ A_indptr,
    float* __restrict__ y,
    const float* __restrict__ A_data,
    const float* __restrict__ B,
    const int* __restrict__ A_indices,
    const appy::i64 y_stride_0,
    const appy::i64 B_stride_0,
    const appy::i64 __lo,
    const appy::i64 __hi)
{
    const int __lane = threadIdx.x & 31;
    const appy::i64 __team = threadIdx.x / 32;
    for (appy::i64 __i = __lo + blockIdx.x * 8LL + __team; __i < __hi; __i += gridDim.x * 8LL) {
        {
            const appy::i64 i = __i;
            int start = 0;
            int end = 0;
            start = A_indptr[i];
            end = A_indptr[(i + 1LL)];
            {
                // row accumulators: extent 128 is fixed at compile time (asserted by the launcher)
                appy::vec<float, 4>::type __acc1;
                { __acc1.x = ((float)(0LL)); __acc1.y = ((float)(0LL)); __acc1.z = ((float)(0LL)); __acc1.w = ((float)(0LL)); }
                const appy::i64 __hi2 = ((long long)(end));
                #pragma unroll 4
                for (appy::i64 k = ((long long)(start)); k < __hi2; ++k) {
                    {
                        const appy::vec<float, 4>::type __ld_B_3 = appy::vload<float, 4>(B + (((long long)(A_indices[k])) * B_stride_0 + ((0LL + __lane) * 4)));
                        { const appy::i64 __c2 = ((0LL + __lane) * 4) + 0;
                          __acc1.x = (__acc1.x + (A_data[k] * __ld_B_3.x)); }
                        { const appy::i64 __c2 = ((0LL + __lane) * 4) + 1;
                          __acc1.y = (__acc1.y + (A_data[k] * __ld_B_3.y)); }
                        { const appy::i64 __c2 = ((0LL + __lane) * 4) + 2;
                          __acc1.z = (__acc1.z + (A_data[k] * __ld_B_3.z)); }
                        { const appy::i64 __c2 = ((0LL + __lane) * 4) + 3;
                          __acc1.w = (__acc1.w + (A_data[k] * __ld_B_3.w)); }
                    }
                }
                appy::vstore<float, 4>(y + (i * y_stride_0 + ((0LL + __lane) * 4)), __acc1);
                appy::wave_fence();     // the row is stored: later loops of the team may read other lanes' elements
            }
        }
    }
}
