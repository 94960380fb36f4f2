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
    __shared__ double __strip_slots[16][64];   // one slot per wavefront and lane, any 4- or 8-byte type
    for (appy::i64 __s = blockIdx.x; __lo + __s * 64 < __hi; __s += gridDim.x) {
        const bool __active = __lo + __s * 64 + __lane < __hi;
        const appy::i64 j = __active ? __lo + __s * 64 + __lane : __hi - 1;
        float s = 0;
        s = ((float)(0.0));
        {
            const appy::i64 __lo1 = 0LL;
            const appy::i64 __hi2 = A_shape_0;
            float __part_s_3 = ((float)0);
            if (__active) {
                #pragma unroll 8
                for (appy::i64 i = __lo1 + __wave; i < __hi2; i += 16) {
                    __part_s_3 = appy::OpAdd::f<float>(__part_s_3, (__builtin_nontemporal_load(&A[i * A_stride_0 + j]) * y[i]));
                }
            }
            reinterpret_cast<float*>(&__strip_slots[0][0])[__wave * 64 + __lane] = __part_s_3;
            __syncthreads();
            float __tot4 = reinterpret_cast<float*>(&__strip_slots[0][0])[__lane];
            for (int __w = 1; __w < 16; ++__w) __tot4 = appy::OpAdd::f<float>(__tot4, reinterpret_cast<float*>(&__strip_slots[0][0])[__w * 64 + __lane]);
            s = appy::OpAdd::f<float>(s, __tot4);
            __syncthreads();   // the slots are free again
        }
        if (__wave == 0 && __active) { x[j] = s; }
    }
}
