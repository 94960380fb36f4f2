// kernel for spmv_kernel_loop_1_plan: team_b256_v1_u1_w8_r_list_s8_plan
extern "C" __global__ void __launch_bounds__(256)
_spmv_kernel_loop_1_plan(
    const int* __restrict__ A_indptr,
    const float* __restrict__ A_data,
    const float* __restrict__ x,
    const int* __restrict__ A_indices,
    float* __restrict__ y,
    const int* __rows,
    const int* __nrows,
    int* __bnd,
    const appy::i64 __cap,
    appy::i64* __start,
    const appy::i64 __stripe,
    unsigned long long* __load,
    const appy::i64 __lo,
    const appy::i64 __hi)
{
    const int __lane = threadIdx.x & 7;
    const appy::i64 __team = threadIdx.x / 8;
    const appy::i64 __listed = (appy::i64)__nrows[0];
    const appy::i64 __n = __listed < __cap ? __listed : __cap;
    __shared__ unsigned long long __work[8];
    if (threadIdx.x < 8) __work[threadIdx.x] = 0;
    __syncthreads();
    unsigned long long __mine = 0;      // elements in the part of this lane, over the rows of its team
    for (appy::i64 __t = (appy::i64)blockIdx.x * 32 + __team; __t < __n; __t += (appy::i64)gridDim.x * 32) {
        {
            const appy::i64 i = (appy::i64)__rows[__t];
            int start = 0;
            int end = 0;
            double s = 0;
            start = A_indptr[i];
            end = A_indptr[(i + 1LL)];
            s = 0.0;
            const appy::i64 __rlo = ((long long)(start));
            const appy::i64 __rhi = (((long long)(end))) > __rlo ? (((long long)(end))) : __rlo;
            appy::i64 __b = __rhi;
            if (__lane < 7 && __rhi > __rlo) {
                const appy::i64 __target = (appy::i64)(__lane + 1) * __stripe;
                appy::i64 __a = __rlo, __z = __rhi;       // the cut lies in [__a, __z]: indices before __a are below the target
                const appy::i64 __guess = __rlo + ((__rhi - __rlo) * (__lane + 1)) / 8;
                appy::i64 __step = 16;
                if ((appy::i64)A_indices[__guess] < __target) {
                    __a = __guess + 1;
                    while (__a < __z) {
                        const appy::i64 __p = (__a + __step - 1) < (__z - 1) ? (__a + __step - 1) : (__z - 1);
                        if ((appy::i64)A_indices[__p] < __target) { __a = __p + 1; __step *= 4; } else { __z = __p; break; }
                    }
                } else {
                    __z = __guess;
                    while (__a < __z) {
                        const appy::i64 __p = (__z - __step) > __a ? (__z - __step) : __a;
                        if ((appy::i64)A_indices[__p] < __target) { __a = __p + 1; break; } else { __z = __p; __step *= 4; }
                    }
                }
                while (__a < __z) {
                    const appy::i64 __mid = __a + ((__z - __a) >> 1);
                    if ((appy::i64)A_indices[__mid] < __target) __a = __mid + 1; else __z = __mid;
                }
                __b = __a;
            }
            __b = appy::team_running_max<8>(__b, __lane);
            if (__lane == 0) { __bnd[__t] = 0; __start[__t] = __rlo; }
            const appy::i64 __cut = (__lane < 7 ? __b : __rhi) - __rlo;      // where part __lane ends
            if (__lane < 8) __bnd[(appy::i64)(__lane + 1) * __cap + __t] = (int)__cut;
            const appy::i64 __before = appy::team_lane_below<8>(__cut, __lane);
            if (__lane < 8 && __cut > (__lane ? __before : 0)) __mine += (unsigned long long)(__cut - (__lane ? __before : 0));
        }
    }
    if (__lane < 8 && __mine) atomicAdd(&__work[__lane], __mine);
    __syncthreads();
    if (threadIdx.x < 8 && __work[threadIdx.x]) atomicAdd(&__load[threadIdx.x], __work[threadIdx.x]);
}
