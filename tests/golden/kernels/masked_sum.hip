// kernel for masked_sum_kernel_loop_1: flat_b512_v4_u4_w1_r_nt
extern "C" __global__ void __launch_bounds__(512)
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
    const appy::i64 __ntiles = (__hi - __lo) / 8192;
    for (appy::i64 __t = blockIdx.x; __t < __ntiles; __t += __nblk) {
        const appy::i64 __tile0 = __lo + __t * 8192 + __tid * 4;
        const appy::vec<unsigned char, 4>::type __ld_M_1 = appy::vload_stream<unsigned char, 4>(M + ((__tile0 + 0)));
        const appy::vec<float, 4>::type __ld_A_2 = appy::vload_stream<float, 4>(A + ((__tile0 + 0)));
        const appy::vec<unsigned char, 4>::type __ld_M_3 = appy::vload_stream<unsigned char, 4>(M + ((__tile0 + 2048)));
        const appy::vec<float, 4>::type __ld_A_4 = appy::vload_stream<float, 4>(A + ((__tile0 + 2048)));
        const appy::vec<unsigned char, 4>::type __ld_M_5 = appy::vload_stream<unsigned char, 4>(M + ((__tile0 + 4096)));
        const appy::vec<float, 4>::type __ld_A_6 = appy::vload_stream<float, 4>(A + ((__tile0 + 4096)));
        const appy::vec<unsigned char, 4>::type __ld_M_7 = appy::vload_stream<unsigned char, 4>(M + ((__tile0 + 6144)));
        const appy::vec<float, 4>::type __ld_A_8 = appy::vload_stream<float, 4>(A + ((__tile0 + 6144)));
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
            const appy::i64 i = (__tile0 + 2048) + 0;
            __acc0 = appy::OpAdd::f<double>(__acc0, ((double)(((__ld_M_3.x != 0) ? __ld_A_4.x : ((float)(0.0))))));
        }
        {
            const appy::i64 i = (__tile0 + 2048) + 1;
            __acc0 = appy::OpAdd::f<double>(__acc0, ((double)(((__ld_M_3.y != 0) ? __ld_A_4.y : ((float)(0.0))))));
        }
        {
            const appy::i64 i = (__tile0 + 2048) + 2;
            __acc0 = appy::OpAdd::f<double>(__acc0, ((double)(((__ld_M_3.z != 0) ? __ld_A_4.z : ((float)(0.0))))));
        }
        {
            const appy::i64 i = (__tile0 + 2048) + 3;
            __acc0 = appy::OpAdd::f<double>(__acc0, ((double)(((__ld_M_3.w != 0) ? __ld_A_4.w : ((float)(0.0))))));
        }
        {
            const appy::i64 i = (__tile0 + 4096) + 0;
            __acc0 = appy::OpAdd::f<double>(__acc0, ((double)(((__ld_M_5.x != 0) ? __ld_A_6.x : ((float)(0.0))))));
        }
        {
            const appy::i64 i = (__tile0 + 4096) + 1;
            __acc0 = appy::OpAdd::f<double>(__acc0, ((double)(((__ld_M_5.y != 0) ? __ld_A_6.y : ((float)(0.0))))));
        }
        {
            const appy::i64 i = (__tile0 + 4096) + 2;
            __acc0 = appy::OpAdd::f<double>(__acc0, ((double)(((__ld_M_5.z != 0) ? __ld_A_6.z : ((float)(0.0))))));
        }
        {
            const appy::i64 i = (__tile0 + 4096) + 3;
            __acc0 = appy::OpAdd::f<double>(__acc0, ((double)(((__ld_M_5.w != 0) ? __ld_A_6.w : ((float)(0.0))))));
        }
        {
            const appy::i64 i = (__tile0 + 6144) + 0;
            __acc0 = appy::OpAdd::f<double>(__acc0, ((double)(((__ld_M_7.x != 0) ? __ld_A_8.x : ((float)(0.0))))));
        }
        {
            const appy::i64 i = (__tile0 + 6144) + 1;
            __acc0 = appy::OpAdd::f<double>(__acc0, ((double)(((__ld_M_7.y != 0) ? __ld_A_8.y : ((float)(0.0))))));
        }
        {
            const appy::i64 i = (__tile0 + 6144) + 2;
            __acc0 = appy::OpAdd::f<double>(__acc0, ((double)(((__ld_M_7.z != 0) ? __ld_A_8.z : ((float)(0.0))))));
        }
        {
            const appy::i64 i = (__tile0 + 6144) + 3;
            __acc0 = appy::OpAdd::f<double>(__acc0, ((double)(((__ld_M_7.w != 0) ? __ld_A_8.w : ((float)(0.0))))));
        }
    }
    const appy::i64 __rest0 = __lo + __ntiles * 8192;
    const appy::i64 __nrv = (__hi - __rest0) / 4;
    for (appy::i64 __q = blockIdx.x * 512LL + __tid; __q < __nrv; __q += __nblk * 512LL) {
        const appy::i64 __vb = __rest0 + __q * 4;
        const appy::vec<unsigned char, 4>::type __ld_M_9 = appy::vload_stream<unsigned char, 4>(M + (__vb));
        const appy::vec<float, 4>::type __ld_A_10 = appy::vload_stream<float, 4>(A + (__vb));
        {
            const appy::i64 i = __vb + 0;
            __acc0 = appy::OpAdd::f<double>(__acc0, ((double)(((__ld_M_9.x != 0) ? __ld_A_10.x : ((float)(0.0))))));
        }
        {
            const appy::i64 i = __vb + 1;
            __acc0 = appy::OpAdd::f<double>(__acc0, ((double)(((__ld_M_9.y != 0) ? __ld_A_10.y : ((float)(0.0))))));
        }
        {
            const appy::i64 i = __vb + 2;
            __acc0 = appy::OpAdd::f<double>(__acc0, ((double)(((__ld_M_9.z != 0) ? __ld_A_10.z : ((float)(0.0))))));
        }
        {
            const appy::i64 i = __vb + 3;
            __acc0 = appy::OpAdd::f<double>(__acc0, ((double)(((__ld_M_9.w != 0) ? __ld_A_10.w : ((float)(0.0))))));
        }
    }
    for (appy::i64 __i = __rest0 + __nrv * 4 + blockIdx.x * 512LL + __tid; __i < __hi; __i += __nblk * 512LL) {
        {
            const appy::i64 i = __i;
            __acc0 = appy::OpAdd::f<double>(__acc0, ((double)(((M[i] != 0) ? A[i] : ((float)(0.0))))));
        }
    }
    {
        const double __tot = appy::block_reduce<appy::OpAdd, 512, double>(__acc0, ((double)0));
        if (threadIdx.x == 0) appy::atomic_combine<appy::OpAdd, double>::run(&s[0], __tot);
    }
}
