// kernel for copy_kernel_loop_1: flat_b512_v4_u1_w1_r_nt_nts
extern "C" __global__ void __launch_bounds__(512)
_copy_kernel_loop_1(
    float* __restrict__ c,
    const float* __restrict__ a,
    const appy::i64 __lo,
    const appy::i64 __hi)
{
    const appy::i64 __tid = threadIdx.x;
    const appy::i64 __nblk = gridDim.x;
    const appy::i64 __ntiles = (__hi - __lo) / 2048;
    for (appy::i64 __t = blockIdx.x; __t < __ntiles; __t += __nblk) {
        const appy::i64 __tile0 = __lo + __t * 2048 + __tid * 4;
        const appy::vec<float, 4>::type __ld_a_1 = appy::vload_stream<float, 4>(a + (__tile0));
        appy::vec<float, 4>::type __st_c_2;
        {
            const appy::i64 i = __tile0 + 0;
            __st_c_2.x = __ld_a_1.x;
        }
        {
            const appy::i64 i = __tile0 + 1;
            __st_c_2.y = __ld_a_1.y;
        }
        {
            const appy::i64 i = __tile0 + 2;
            __st_c_2.z = __ld_a_1.z;
        }
        {
            const appy::i64 i = __tile0 + 3;
            __st_c_2.w = __ld_a_1.w;
        }
        appy::vstore_stream<float, 4>(c + (__tile0), __st_c_2);
    }
    const appy::i64 __rest0 = __lo + __ntiles * 2048;
    const appy::i64 __nrv = (__hi - __rest0) / 4;
    for (appy::i64 __q = blockIdx.x * 512LL + __tid; __q < __nrv; __q += __nblk * 512LL) {
        const appy::i64 __vb = __rest0 + __q * 4;
        const appy::vec<float, 4>::type __ld_a_3 = appy::vload_stream<float, 4>(a + (__vb));
        appy::vec<float, 4>::type __st_c_4;
        {
            const appy::i64 i = __vb + 0;
            __st_c_4.x = __ld_a_3.x;
        }
        {
            const appy::i64 i = __vb + 1;
            __st_c_4.y = __ld_a_3.y;
        }
        {
            const appy::i64 i = __vb + 2;
            __st_c_4.z = __ld_a_3.z;
        }
        {
            const appy::i64 i = __vb + 3;
            __st_c_4.w = __ld_a_3.w;
        }
        appy::vstore_stream<float, 4>(c + (__vb), __st_c_4);
    }
    for (appy::i64 __i = __rest0 + __nrv * 4 + blockIdx.x * 512LL + __tid; __i < __hi; __i += __nblk * 512LL) {
        {
            const appy::i64 i = __i;
            c[i] = a[i];
        }
    }
}
