// kernel for spmv_kernel_loop_1_bins: team_b1024_v1_u1_w1_r_bins
extern "C" __global__ void __launch_bounds__(1024)
_spmv_kernel_loop_1_bins(
    const int* __restrict__ A_indptr,
    const float* __restrict__ A_data,
    const float* __restrict__ x,
    const int* __restrict__ A_indices,
    float* __restrict__ y,
    int* __rows,
    int* __counts,
    int* __zero,
    const appy::i64 __m,
    const int __base,
    const appy::i64 __t0,
    const appy::i64 __t1,
    const appy::i64 __t2,
    const appy::i64 __lo,
    const appy::i64 __hi)
{
    __shared__ int __cnt[4];
    __shared__ int __first[4];
    if (blockIdx.x == 0 && threadIdx.x < 136) __zero[threadIdx.x] = 0;     // 8 counters, 64 part loads of 8 bytes
    for (appy::i64 __c0 = __lo + (appy::i64)blockIdx.x * 4096; __c0 < __hi; __c0 += (appy::i64)gridDim.x * 4096) {
        if (threadIdx.x < 4) __cnt[threadIdx.x] = 0;
        __syncthreads();
        int __cl[4], __pos[4];
        #pragma unroll
        for (int __r = 0; __r < 4; ++__r) {
            const appy::i64 __i = __c0 + (appy::i64)__r * 1024 + threadIdx.x;
            __cl[__r] = -1;
            __pos[__r] = 0;
            if (__i < __hi) {
                const appy::i64 i = __i;
                int start = 0;
                int end = 0;
                double s = 0;
                start = A_indptr[i];
                end = A_indptr[(i + 1LL)];
                s = 0.0;
                const appy::i64 __trip = (((long long)(end))) - (((long long)(start)));
                const int __c = __trip <= __t0 ? 0 : __trip <= __t1 ? 1 : __trip <= __t2 ? 2 : 3;
                if (__c != __base) { __cl[__r] = __c; __pos[__r] = atomicAdd(&__cnt[__c], 1); }
            }
        }
        __syncthreads();
        if (threadIdx.x < 4) __first[threadIdx.x] = __cnt[threadIdx.x] ? atomicAdd(&__counts[threadIdx.x], __cnt[threadIdx.x]) : 0;
        __syncthreads();
        #pragma unroll
        for (int __r = 0; __r < 4; ++__r) {
            if (__cl[__r] >= 0) __rows[(appy::i64)__cl[__r] * __m + __first[__cl[__r]] + __pos[__r]] = (int)(__c0 + (appy::i64)__r * 1024 + threadIdx.x);
        }
        __syncthreads();
    }
}
