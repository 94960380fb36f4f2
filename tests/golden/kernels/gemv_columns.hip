// kernel for gemv_columns_kernel_loop_1: strip_b1024_v1_u8_w1_r_nt
extern "C" __global__ void __launch_bounds__(1024)
_gemv_columns_kernel_loop_1(
    const float* __restrict__ A,
    const float* __restrict__ y,
    float* __restrict__ x,
    const appy::i64 A_stride_0,
    const long long A_shape_0,
    const appy::i64 __lo,
    const appy::i64 __hi)
{
    const int __lane = threadIdx.x & 63;
    const int __wave = threadIdx.x >> 6;
    __shared__ float __strip_s[16][64];
    for (appy::i64 __s = blockIdx.x; __lo + __s * 64 < __hi; __s += gridDim.x) {
        const appy::i64 j = __lo + __s * 64 + __lane;
        const bool __active = j < __hi;
        float s = 0;
        float __part_s = ((float)0);
        if (__active) {
            s = ((float)(0.0));
            const appy::i64 __hi1 = A_shape_0;
            #pragma unroll 8
            for (appy::i64 i = 0LL + __wave; i < __hi1; i += 16) {
                __part_s = appy::OpAdd::f<float>(__part_s, (__builtin_nontemporal_load(&A[i * A_stride_0 + j]) * y[i]));
            }
        }
        __strip_s[__wave][__lane] = __part_s;
        __syncthreads();
        if (__wave == 0 && __active) {
            for (int __w = 1; __w < 16; ++__w) __part_s = appy::OpAdd::f<float>(__part_s, __strip_s[__w][__lane]);
            s = appy::OpAdd::f<float>(s, __part_s);
            x[j] = s;
        }
        __syncthreads();   // the slots are free for the next strip
    }
}
