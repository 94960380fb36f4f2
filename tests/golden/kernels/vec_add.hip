// kernel for vec_add_kernel_loop_1: flat_b256_v4_u2_w1_r
extern "C" __global__ void __launch_bounds__(256)
_vec_add_kernel_loop_1(
    float* __restrict__ c,
    const float* __restrict__ a,
    const float* __restrict__ b,
    const appy::i64 __lo,
    const appy::i64 __hi)
{
    const appy::i64 __tid = threadIdx.x;
    const appy::i64 __nblk = gridDim.x;
    const appy::i64 __ntiles = (__hi - __lo) / 2048;
    for (appy::i64 __t = blockIdx.x; __t < __ntiles; __t += __nblk) {
        const appy::i64 __tile0 = __lo + __t * 2048 + __tid * 4;
        const appy::vec<float, 4>::type __ld_a_1 = appy::vload<float, 4>(a + ((__tile0 + 0)));
        const appy::vec<float, 4>::type __ld_b_2 = appy::vload<float, 4>(b + ((__tile0 + 0)));
        const appy::vec<float, 4>::type __ld_a_3 = appy::vload<float, 4>(a + ((__tile0 + 1024)));
        const appy::vec<float, 4>::type __ld_b_4 = appy::vload<float, 4>(b + ((__tile0 + 1024)));
        appy::vec<float, 4>::type __st_c_5;
        appy::vec<float, 4>::type __st_c_6;
        {
            const appy::i64 i = (__tile0 + 0) + 0;
            __st_c_5.x = (__ld_a_1.x + __ld_b_2.x);
        }
        {
            const appy::i64 i = (__tile0 + 0) + 1;
            __st_c_5.y = (__ld_a_1.y + __ld_b_2.y);
        }
        {
            const appy::i64 i = (__tile0 + 0) + 2;
            __st_c_5.z = (__ld_a_1.z + __ld_b_2.z);
        }
        {
            const appy::i64 i = (__tile0 + 0) + 3;
            __st_c_5.w = (__ld_a_1.w + __ld_b_2.w);
        }
        {
            const appy::i64 i = (__tile0 + 1024) + 0;
            __st_c_6.x = (__ld_a_3.x + __ld_b_4.x);
        }
        {
            const appy::i64 i = (__tile0 + 1024) + 1;
            __st_c_6.y = (__ld_a_3.y + __ld_b_4.y);
        }
        {
            const appy::i64 i = (__tile0 + 1024) + 2;
            __st_c_6.z = (__ld_a_3.z + __ld_b_4.z);
        }
        {
            const appy::i64 i = (__tile0 + 1024) + 3;
            __st_c_6.w = (__ld_a_3.w + __ld_b_4.w);
        }
        appy::vstore<float, 4>(c + ((__tile0 + 0)), __st_c_5);
        appy::vstore<float, 4>(c + ((__tile0 + 1024)), __st_c_6);
    }
    const appy::i64 __rest0 = __lo + __ntiles * 2048;
    const appy::i64 __nrv = (__hi - __rest0) / 4;
    for (appy::i64 __q = blockIdx.x * 256LL + __tid; __q < __nrv; __q += __nblk * 256LL) {
        const appy::i64 __vb = __rest0 + __q * 4;
        const appy::vec<float, 4>::type __ld_a_7 = appy::vload<float, 4>(a + (__vb));
        const appy::vec<float, 4>::type __ld_b_8 = appy::vload<float, 4>(b + (__vb));
        appy::vec<float, 4>::type __st_c_9;
        {
            const appy::i64 i = __vb + 0;
            __st_c_9.x = (__ld_a_7.x + __ld_b_8.x);
        }
        {
            const appy::i64 i = __vb + 1;
            __st_c_9.y = (__ld_a_7.y + __ld_b_8.y);
        }
        {
            const appy::i64 i = __vb + 2;
            __st_c_9.z = (__ld_a_7.z + __ld_b_8.z);
        }
        {
            const appy::i64 i = __vb + 3;
            __st_c_9.w = (__ld_a_7.w + __ld_b_8.w);
        }
        appy::vstore<float, 4>(c + (__vb), __st_c_9);
    }
    for (appy::i64 __i = __rest0 + __nrv * 4 + blockIdx.x * 256LL + __tid; __i < __hi; __i += __nblk * 256LL) {
        {
            const appy::i64 i = __i;
            c[i] = (a[i] + b[i]);
        }
    }
}
