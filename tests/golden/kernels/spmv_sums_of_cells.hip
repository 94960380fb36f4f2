// kernel for spmv_kernel_loop_1_sums: team_b256_v4_u1_w1_r_p2_if1
extern "C" __global__ void __launch_bounds__(256)
_spmv_kernel_loop_1_sums(
    const int* __restrict__ A_indptr,
    const float* __restrict__ A_data,
    const float* __restrict__ x,
    const int* __restrict__ A_indices,
    float* __restrict__ y,
    double* __scratch,
    const appy::i64 __nsplit,
    const long long* __flag,
    const appy::i64 __lo,
    const appy::i64 __hi)
{
    if ((__flag[0] != 0) == true) return;
    const int __lane = threadIdx.x & 0;
    const appy::i64 __team = threadIdx.x / 1;
    for (appy::i64 __i = __lo + blockIdx.x * 256LL + __team; __i < __hi; __i += gridDim.x * 256LL) {
        {
            const appy::i64 i = __i;
            int start = 0;
            int end = 0;
            float s = 0;
            start = A_indptr[i];
            end = A_indptr[(i + 1LL)];
            s = ((float)(0.0));
            {
                const appy::i64 __lo1 = ((long long)(start));
                const appy::i64 __hi2 = ((long long)(end));
                float __part_s_3 = ((float)0);
                #pragma unroll 16
                for (appy::i64 __c = 0; __c < __nsplit; ++__c) __part_s_3 = appy::OpAdd::f<float>(__part_s_3, reinterpret_cast<float*>(__scratch)[(0 * __nsplit + __c) * (__hi - __lo) + (i - __lo)]);
                s = appy::OpAdd::f<float>(s, __part_s_3);
            }
            if (__lane == 0) { y[i] = s; }
        }
    }
}
