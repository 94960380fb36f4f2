// kernel for spmv_kernel_loop_1: team_b256_v4_u1_w64_r_nt_mixed
extern "C" __global__ void __launch_bounds__(256)
_spmv_kernel_loop_1(
    const int* __restrict__ A_indptr,
    const float* __restrict__ A_data,
    const float* __restrict__ x,
    const int* __restrict__ A_indices,
    float* __restrict__ y,
    const int* __rows,
    const int* __counts,
    const appy::i64 __m,
    const int __base,
    const int __wl0,
    const int __wl1,
    const int __wl2,
    const int __wl3,
    const appy::i64 __skip3,
    long long* __hint,
    const appy::i64 __tlo,
    const appy::i64 __thi,
    const appy::i64 __lo,
    const appy::i64 __hi)
{
    const int __lid = threadIdx.x & 63;
    const appy::i64 __wv = (appy::i64)blockIdx.x * 4 + __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const appy::i64 __nwv = (appy::i64)gridDim.x * 4;
    const appy::i64 __l0 = (appy::i64)__counts[0] - 0;
    const appy::i64 __n0 = (__base == 0) ? (__hi - __lo) : (__l0 > 0 ? __l0 : 0);
    const appy::i64 __e0 = 0 + (((__n0 << __wl0) + 63) >> 6);
    const appy::i64 __l1 = (appy::i64)__counts[1] - 0;
    const appy::i64 __n1 = (__base == 1) ? (__hi - __lo) : (__l1 > 0 ? __l1 : 0);
    const appy::i64 __e1 = __e0 + (((__n1 << __wl1) + 63) >> 6);
    const appy::i64 __l2 = (appy::i64)__counts[2] - 0;
    const appy::i64 __n2 = (__base == 2) ? (__hi - __lo) : (__l2 > 0 ? __l2 : 0);
    const appy::i64 __e2 = __e1 + (((__n2 << __wl2) + 63) >> 6);
    const appy::i64 __l3 = (appy::i64)__counts[3] - __skip3;
    const appy::i64 __n3 = (__base == 3) ? (__hi - __lo) : (__l3 > 0 ? __l3 : 0);
    const appy::i64 __e3 = __e2 + (((__n3 << __wl3) + 63) >> 6);
    if (blockIdx.x == 0 && threadIdx.x == 0) {
        const appy::i64 __others = (__base == 0 ? 0 : (appy::i64)__counts[0]) + (__base == 1 ? 0 : (appy::i64)__counts[1]) + (__base == 2 ? 0 : (appy::i64)__counts[2]) + (__base == 3 ? 0 : (appy::i64)__counts[3]);
        __hint[1] = (__base == 0) ? (__hi - __lo) - __others : (appy::i64)__counts[0];
        __hint[2] = (__base == 1) ? (__hi - __lo) - __others : (appy::i64)__counts[1];
        __hint[3] = (__base == 2) ? (__hi - __lo) - __others : (appy::i64)__counts[2];
        __hint[4] = (__base == 3) ? (__hi - __lo) - __others : (appy::i64)__counts[3];
        __hint[0] = 1;
    }
    for (appy::i64 __v = __wv; __v < __e3; __v += __nwv) {
        const int __c = (int)(__v >= __e0) + (int)(__v >= __e1) + (int)(__v >= __e2);
        const int __wl = __c == 0 ? __wl0 : __c == 1 ? __wl1 : __c == 2 ? __wl2 : __wl3;
        const int __W = 1 << __wl;
        const int __lane = __lid & (__W - 1);
        const appy::i64 __vb = __c == 0 ? 0 : __c == 1 ? __e0 : __c == 2 ? __e1 : __e2;
        const appy::i64 __nc = __c == 0 ? __n0 : __c == 1 ? __n1 : __c == 2 ? __n2 : __n3;
        const appy::i64 __t = ((__v - __vb) << (6 - __wl)) + (__lid >> __wl);
        if (__t < __nc) {
            const appy::i64 __i = (__c == __base) ? (__lo + __t) : (appy::i64)__rows[(appy::i64)__c * __m + (__c == 3 ? __skip3 : 0) + __t];
            {
                const appy::i64 i = __i;
                int start = 0;
                int end = 0;
                float s = 0;
                start = A_indptr[i];
                end = A_indptr[(i + 1LL)];
                s = ((float)(0.0));
                const appy::i64 __trip = (((long long)(end))) - (((long long)(start)));
                if (__c != __base || (__trip > __tlo && __trip <= __thi)) {
                    {
                        const appy::i64 __lo1 = ((long long)(start));
                        const appy::i64 __hi2 = ((long long)(end));
                        float __part_s_3 = ((float)0);
                        const appy::i64 __nv4 = (__hi2 - __lo1) / 4;
                        #pragma unroll 2
                        for (appy::i64 __q5 = __lane; __q5 < __nv4; __q5 += __W) {
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
                        for (appy::i64 j = __lo1 + __nv4 * 4 + __lane; j < __hi2; j += __W) {
                            __part_s_3 = appy::OpAdd::f<float>(__part_s_3, (A_data[j] * x[((long long)(A_indices[j]))]));
                        }
                        s = appy::OpAdd::f<float>(s, appy::team_reduce_dyn<appy::OpAdd, float>(__part_s_3, __W));
                    }
                    if (__lane == 0) { y[i] = s; }
                }
            }
        }
    }
}
