// kernel for vec_add_kernel_loop_1: flat_b1024_v4_u1_w1_r_nt_nts
extern "C" __global__ void __launch_bounds__(1024)
_vec_add_kernel_loop_1(
    float* __restrict__ c,
    const float* __restrict__ a,
    const float* __restrict__ b,
    const appy::i64 __lo,
    const appy::i64 __hi)
{
    const appy::i64 __tid = threadIdx.x;
    const appy::i64 __nblk = gridDim.x;
    const appy::i64 __ntiles = (__hi - __lo) / 4096;
    for (appy::i64 __t = blockIdx.x; __t < __ntiles; __t += __nblk) {
        const appy::i64 __tile0 = __lo + __t * 4096 + __tid * 4;
        const appy::vec<float, 4>::type __ld_a_1 = appy::vload_stream<float, 4>(a + (__tile0));
        const appy::vec<float, 4>::type __ld_b_2 = appy::vload_stream<float, 4>(b + (__tile0));
        appy::vec<float, 4>::type __st_c_3;
        {
            const appy::i64 i = __tile0 + 0;
            __st_c_3.x = (__ld_a_1.x + __ld_b_2.x);
        }
        {
            const appy::i64 i = __tile0 + 1;
            __st_c_3.y = (__ld_a_1.y + __ld_b_2.y);
        }
        {
            const appy::i64 i = __tile0 + 2;
            __st_c_3.z = (__ld_a_1.z + __ld_b_2.z);
        }
        {
            const appy::i64 i = __tile0 + 3;
            __st_c_3.w = (__ld_a_1.w + __ld_b_2.w);
        }
        appy::vstore_stream<float, 4>(c + (__tile0), __st_c_3);
    }
    const appy::i64 __rest0 = __lo + __ntiles * 4096;
    const appy::i64 __nrv = (__hi - __rest0) / 4;
    for (appy::i64 __q = blockIdx.x * 1024LL + __tid; __q < __nrv; __q += __nblk * 1024LL) {
        const appy::i64 __vb = __rest0 + __q * 4;
        const appy::vec<float, 4>::type __ld_a_4 = appy::vload_stream<float, 4>(a + (__vb));
        const appy::vec<float, 4>::type __ld_b_5 = appy::vload_stream<float, 4>(b + (__vb));
        appy::vec<float, 4>::type __st_c_6;
        {
            const appy::i64 i = __vb + 0;
            __st_c_6.x = (__ld_a_4.x + __ld_b_5.x);
        }
        {
            const appy::i64 i = __vb + 1;
            __st_c_6.y = (__ld_a_4.y + __ld_b_5.y);
        }
        {
            const appy::i64 i = __vb + 2;
            __st_c_6.z = (__ld_a_4.z + __ld_b_5.z);
        }
        {
            const appy::i64 i = __vb + 3;
            __st_c_6.w = (__ld_a_4.w + __ld_b_5.w);
        }
        appy::vstore_stream<float, 4>(c + (__vb), __st_c_6);
    }
    for (appy::i64 __i = __rest0 + __nrv * 4 + blockIdx.x * 1024LL + __tid; __i < __hi; __i += __nblk * 1024LL) {
        {
            const appy::i64 i = __i;
            c[i] = (a[i] + b[i]);
        }
    }
}
