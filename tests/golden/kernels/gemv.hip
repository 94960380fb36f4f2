// kernel for gemv_kernel_loop_1: team_b256_v4_u1_w32_r_nt
extern "C" __global__ void __launch_bounds__(256)
_gemv_kernel_loop_1(
    const float* __restrict__ A,
    const float* __restrict__ x,
    float* __restrict__ y,
    const appy::i64 A_stride_0,
    const long long A_shape_1,
    const appy::i64 __lo,
    const appy::i64 __hi)
{
    const int __lane = threadIdx.x & 31;
    const appy::i64 __team = threadIdx.x / 32;
    for (appy::i64 __i = __lo + blockIdx.x * 8LL + __team; __i < __hi; __i += gridDim.x * 8LL) {
        {
            const appy::i64 i = __i;
            float yi = 0;
            yi = ((float)(0.0));
            {
                const appy::i64 __lo1 = 0LL;
                const appy::i64 __hi2 = A_shape_1;
                float __part_yi_3 = ((float)0);
                const appy::i64 __nv4 = (__hi2 - __lo1) / 4;
                #pragma unroll 2
                for (appy::i64 __q5 = __lane; __q5 < __nv4; __q5 += 32) {
                    const appy::i64 __j6 = __lo1 + __q5 * 4;
                    const appy::vec<float, 4>::type __ld_A_7 = appy::vload_stream<float, 4>(A + (i * A_stride_0 + __j6));
                    const appy::vec<float, 4>::type __ld_x_8 = appy::vload<float, 4>(x + (__j6));
                    {
                        const appy::i64 j = __j6 + 0;
                        __part_yi_3 = appy::OpAdd::f<float>(__part_yi_3, (__ld_A_7.x * __ld_x_8.x));
                    }
                    {
                        const appy::i64 j = __j6 + 1;
                        __part_yi_3 = appy::OpAdd::f<float>(__part_yi_3, (__ld_A_7.y * __ld_x_8.y));
                    }
                    {
                        const appy::i64 j = __j6 + 2;
                        __part_yi_3 = appy::OpAdd::f<float>(__part_yi_3, (__ld_A_7.z * __ld_x_8.z));
                    }
                    {
                        const appy::i64 j = __j6 + 3;
                        __part_yi_3 = appy::OpAdd::f<float>(__part_yi_3, (__ld_A_7.w * __ld_x_8.w));
                    }
                }
                for (appy::i64 j = __lo1 + __nv4 * 4 + __lane; j < __hi2; j += 32) {
                    __part_yi_3 = appy::OpAdd::f<float>(__part_yi_3, (A[i * A_stride_0 + j] * x[j]));
                }
                yi = appy::OpAdd::f<float>(yi, appy::team_reduce<appy::OpAdd, 32, float>(__part_yi_3));
            }
            if (__lane == 0) { y[i] = yi; }
        }
    }
}
