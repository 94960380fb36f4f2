// kernel for masked_sum_kernel_loop_1: flat_b256_v4_u2_w1_r_nt
extern "C" __global__ void __launch_bounds__(256)
_masked_sum_kernel_loop_1(
    double* __restrict__ s,
    const unsigned char* __restrict__ M,
    const float* __restrict__ A,
    const appy::i64 __lo,
    const appy::i64 __hi)
{
    double __acc0 = ((double)0);
    const appy::i64 __tid = threadIdx.x;
    const appy::i64 __nblk = gridDim.x;
    const appy::i64 __ntiles = (__hi - __lo) / 2048;
    for (appy::i64 __t = blockIdx.x; __t < __ntiles; __t += __nblk) {
        const appy::i64 __tile0 = __lo + __t * 2048 + __tid * 4;
        const appy::vec<unsigned char, 4>::type __ld_M_1 = appy::vload_stream<unsigned char, 4>(M + ((__tile0 + 0)));
        const appy::vec<float, 4>::type __ld_A_2 = appy::vload_stream<float, 4>(A + ((__tile0 + 0)));
        const appy::vec<unsigned char, 4>::type __ld_M_3 = appy::vload_stream<unsigned char, 4>(M + ((__tile0 + 1024)));
        const appy::vec<float, 4>::type __ld_A_4 = appy::vload_stream<float, 4>(A + ((__tile0 + 1024)));
        {
            const appy::i64 i = (__tile0 + 0) + 0;
            __acc0 = appy::OpAdd::f<double>(__acc0, ((double)(((__ld_M_1.x != 0) ? __ld_A_2.x : ((float)(0.0))))));
        }
        {
            const appy::i64 i = (__tile0 + 0) + 1;
            __acc0 = appy::OpAdd::f<double>(__acc0, ((double)(((__ld_M_1.y != 0) ? __ld_A_2.y : ((float)(0.0))))));
        }
        {
            const appy::i64 i = (__tile0 + 0) + 2;
            __acc0 = appy::OpAdd::f<double>(__acc0, ((double)(((__ld_M_1.z != 0) ? __ld_A_2.z : ((float)(0.0))))));
        }
        {
            const appy::i64 i = (__tile0 + 0) + 3;
            __acc0 = appy::OpAdd::f<double>(__acc0, ((double)(((__ld_M_1.w != 0) ? __ld_A_2.w : ((float)(0.0))))));
        }
        {
            const appy::i64 i = (__tile0 + 1024) + 0;
            __acc0 = appy::OpAdd::f<double>(__acc0, ((double)(((__ld_M_3.x != 0) ? __ld_A_4.x : ((float)(0.0))))));
        }
        {
            const appy::i64 i = (__tile0 + 1024) + 1;
            __acc0 = appy::OpAdd::f<double>(__acc0, ((double)(((__ld_M_3.y != 0) ? __ld_A_4.y : ((float)(0.0))))));
        }
        {
            const appy::i64 i = (__tile0 + 1024) + 2;
            __acc0 = appy::OpAdd::f<double>(__acc0, ((double)(((__ld_M_3.z != 0) ? __ld_A_4.z : ((float)(0.0))))));
        }
        {
            const appy::i64 i = (__tile0 + 1024) + 3;
            __acc0 = appy::OpAdd::f<double>(__acc0, ((double)(((__ld_M_3.w != 0) ? __ld_A_4.w : ((float)(0.0))))));
        }
    }
    const appy::i64 __rest0 = __lo + __ntiles * 2048;
    const appy::i64 __nrv = (__hi - __rest0) / 4;
    for (appy::i64 __q = blockIdx.x * 256LL + __tid; __q < __nrv; __q += __nblk * 256LL) {
        const appy::i64 __vb = __rest0 + __q * 4;
        const appy::vec<unsigned char, 4>::type __ld_M_5 = appy::vload_stream<unsigned char, 4>(M + (__vb));
        const appy::vec<float, 4>::type __ld_A_6 = appy::vload_stream<float, 4>(A + (__vb));
        {
            const appy::i64 i = __vb + 0;
            __acc0 = appy::OpAdd::f<double>(__acc0, ((double)(((__ld_M_5.x != 0) ? __ld_A_6.x : ((float)(0.0))))));
        }
        {
            const appy::i64 i = __vb + 1;
            __acc0 = appy::OpAdd::f<double>(__acc0, ((double)(((__ld_M_5.y != 0) ? __ld_A_6.y : ((float)(0.0))))));
        }
        {
            const appy::i64 i = __vb + 2;
            __acc0 = appy::OpAdd::f<double>(__acc0, ((double)(((__ld_M_5.z != 0) ? __ld_A_6.z : ((float)(0.0))))));
        }
        {
            const appy::i64 i = __vb + 3;
            __acc0 = appy::OpAdd::f<double>(__acc0, ((double)(((__ld_M_5.w != 0) ? __ld_A_6.w : ((float)(0.0))))));
        }
    }
    for (appy::i64 __i = __rest0 + __nrv * 4 + blockIdx.x * 256LL + __tid; __i < __hi; __i += __nblk * 256LL) {
        {
            const appy::i64 i = __i;
            __acc0 = appy::OpAdd::f<double>(__acc0, ((double)(((M[i] != 0) ? A[i] : ((float)(0.0))))));
        }
    }
    {
        const double __tot = appy::block_reduce<appy::OpAdd, 256, double>(__acc0, ((double)0));
        if (threadIdx.x == 0) appy::atomic_combine<appy::OpAdd, double>::run(&s[0], __tot);
    }
}
