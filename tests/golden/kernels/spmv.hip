// kernel for spmv_kernel_loop_1: team_b256_v4_u1_w4_r_nt
extern "C" __global__ void __launch_bounds__(256)
_spmv_kernel_loop_1(
    const int* __restrict__ A_indptr,
    const float* __restrict__ A_data,
    const float* __restrict__ x,
    const int* __restrict__ A_indices,
    float* __restrict__ y,
    const appy::i64 __lo,
    const appy::i64 __hi)
{
    const int __lane = threadIdx.x & 3;
    const appy::i64 __team = threadIdx.x / 4;
    for (appy::i64 __i = __lo + blockIdx.x * 64LL + __team; __i < __hi; __i += gridDim.x * 64LL) {
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
                const appy::i64 __nv4 = (__hi2 - __lo1) / 4;
                #pragma unroll 2
                for (appy::i64 __q5 = __lane; __q5 < __nv4; __q5 += 4) {
                    const appy::i64 __j6 = __lo1 + __q5 * 4;
                    const appy::vec<float, 4>::type __ld_A_data_7 = appy::vload_stream<float, 4>(A_data + (__j6));
                    const appy::vec<int, 4>::type __ld_A_indices_8 = appy::vload_stream<int, 4>(A_indices + (__j6));
                    {
                        const appy::i64 j = __j6 + 0;
                        __part_s_3 = appy::OpAdd::f<float>(__part_s_3, (__ld_A_data_7.x * x[((long long)(__ld_A_indices_8.x))]));
                    }
                    {
                        const appy::i64 j = __j6 + 1;
                        __part_s_3 = appy::OpAdd::f<float>(__part_s_3, (__ld_A_data_7.y * x[((long long)(__ld_A_indices_8.y))]));
                    }
                    {
                        const appy::i64 j = __j6 + 2;
                        __part_s_3 = appy::OpAdd::f<float>(__part_s_3, (__ld_A_data_7.z * x[((long long)(__ld_A_indices_8.z))]));
                    }
                    {
                        const appy::i64 j = __j6 + 3;
                        __part_s_3 = appy::OpAdd::f<float>(__part_s_3, (__ld_A_data_7.w * x[((long long)(__ld_A_indices_8.w))]));
                    }
                }
                for (appy::i64 j = __lo1 + __nv4 * 4 + __lane; j < __hi2; j += 4) {
                    __part_s_3 = appy::OpAdd::f<float>(__part_s_3, (A_data[j] * x[((long long)(A_indices[j]))]));
                }
                s = appy::OpAdd::f<float>(s, appy::team_reduce<appy::OpAdd, 4, float>(__part_s_3));
            }
            if (__lane == 0) { y[i] = s; }
        }
    }
}
