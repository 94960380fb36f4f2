// kernel for spmv_kernel_loop_1_parts: team_b256_v4_u1_w16_r_nt_p1_list_s8
extern "C" __global__ void __launch_bounds__(256)
_spmv_kernel_loop_1_parts(
    const int* __restrict__ A_indptr,
    const float* __restrict__ A_data,
    const float* __restrict__ x,
    const int* __restrict__ A_indices,
    float* __restrict__ y,
    double* __scratch,
    const appy::i64 __nsplit,
    const int* __rows,
    const int* __nrows,
    const int* __bnd,
    const appy::i64 __cap,
    const appy::i64* __start,
    const unsigned long long* __load,
    const appy::i64 __lo,
    const appy::i64 __hi)
{
    const int __lane = threadIdx.x & 15;
    const appy::i64 __team = threadIdx.x / 16;
    const appy::i64 __listed = (appy::i64)__nrows[0];
    const appy::i64 __n = __listed < __cap ? __listed : __cap;
    unsigned long long __tot = 0, __most = 0;
    for (int __x = 0; __x < 8; ++__x) {
        unsigned long long __sum = 0;
        for (int __p = __x; __p < 8; __p += 8) __sum += __load[__p];
        __tot += __sum;
        __most = __sum > __most ? __sum : __most;
    }
    const bool __even = __most * 16 <= __tot * 3;
    const appy::i64 __t0 = (__even ? (appy::i64)(blockIdx.x >> 3) : (appy::i64)blockIdx.x) * 16 + __team;
    const appy::i64 __dt = (__even ? (appy::i64)(gridDim.x >> 3) : (appy::i64)gridDim.x) * 16;
    for (appy::i64 __pass = 0; __pass < (__even ? 1 : 8); ++__pass) {
        const appy::i64 __chunk = __even ? (appy::i64)(blockIdx.x & 7) + 8 * __pass : __pass;
        for (appy::i64 __t = __t0; __t < __n; __t += __dt) {
            {
                const appy::i64 i = (appy::i64)__rows[__t];
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
                    const appy::i64 __first = __start[__t];     // (from the plan: no need to wait for the set-up's loads)
                    const appy::i64 __lo4 = __first + __bnd[__chunk * __cap + __t];
                    const appy::i64 __hi5 = __first + __bnd[(__chunk + 1) * __cap + __t];
                    const appy::i64 __nv6 = (__hi5 - __lo4) / 4;
                    #pragma unroll 2
                    for (appy::i64 __q7 = __lane; __q7 < __nv6; __q7 += 16) {
                        const appy::i64 __j8 = __lo4 + __q7 * 4;
                        const appy::vec<float, 4>::type __ld_A_data_9 = appy::vload_stream<float, 4>(A_data + (__j8));
                        const appy::vec<int, 4>::type __ld_A_indices_10 = appy::vload_stream<int, 4>(A_indices + (__j8));
                        {
                            const appy::i64 j = __j8 + 0;
                            __part_s_3 = appy::OpAdd::f<float>(__part_s_3, (__ld_A_data_9.x * x[((long long)(__ld_A_indices_10.x))]));
                        }
                        {
                            const appy::i64 j = __j8 + 1;
                            __part_s_3 = appy::OpAdd::f<float>(__part_s_3, (__ld_A_data_9.y * x[((long long)(__ld_A_indices_10.y))]));
                        }
                        {
                            const appy::i64 j = __j8 + 2;
                            __part_s_3 = appy::OpAdd::f<float>(__part_s_3, (__ld_A_data_9.z * x[((long long)(__ld_A_indices_10.z))]));
                        }
                        {
                            const appy::i64 j = __j8 + 3;
                            __part_s_3 = appy::OpAdd::f<float>(__part_s_3, (__ld_A_data_9.w * x[((long long)(__ld_A_indices_10.w))]));
                        }
                    }
                    for (appy::i64 j = __lo4 + __nv6 * 4 + __lane; j < __hi5; j += 16) {
                        __part_s_3 = appy::OpAdd::f<float>(__part_s_3, (A_data[j] * x[((long long)(A_indices[j]))]));
                    }
                    const float __tot11 = appy::team_reduce<appy::OpAdd, 16, float>(__part_s_3);
                    if (__lane == 0) *reinterpret_cast<float*>(__scratch + ((0 * __nsplit + __chunk) * __cap + __t)) = __tot11;
                }
            }
        }
    }
}
