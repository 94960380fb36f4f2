// kernel for vector_sum_kernel_loop_1: flat_b512_v4_u2_w1_r_nt
extern "C" __global__ void __launch_bounds__(512)
_vector_sum_kernel_loop_1(
    double* __restrict__ s,
    const float* __restrict__ A,
    const appy::i64 __lo,
    const appy::i64 __hi)
{
    double __acc0 = ((double)0);
    const appy::i64 __tid = threadIdx.x;
    const appy::i64 __nblk = gridDim.x;
    const appy::i64 __ntiles = (__hi - __lo) / 4096;
    for (appy::i64 __t = blockIdx.x; __t < __ntiles; __t += __nblk) {
        const appy::i64 __tile0 = __lo + __t * 4096 + __tid * 4;
        const appy::vec<float, 4>::type __ld_A_1 = appy::vload_stream<float, 4>(A + ((__tile0 + 0)));
        const appy::vec<float, 4>::type __ld_A_2 = appy::vload_stream<float, 4>(A + ((__tile0 + 2048)));
        {
            const appy::i64 i = (__tile0 + 0) + 0;
            __acc0 = appy::OpAdd::f<double>(__acc0, ((double)(__ld_A_1.x)));
        }
        {
            const appy::i64 i = (__tile0 + 0) + 1;
            __acc0 = appy::OpAdd::f<double>(__acc0, ((double)(__ld_A_1.y)));
        }
        {
            const appy::i64 i = (__tile0 + 0) + 2;
            __acc0 = appy::OpAdd::f<double>(__acc0, ((double)(__ld_A_1.z)));
        }
        {
            const appy::i64 i = (__tile0 + 0) + 3;
            __acc0 = appy::OpAdd::f<double>(__acc0, ((double)(__ld_A_1.w)));
        }
        {
            const appy::i64 i = (__tile0 + 2048) + 0;
            __acc0 = appy::OpAdd::f<double>(__acc0, ((double)(__ld_A_2.x)));
        }
        {
            const appy::i64 i = (__tile0 + 2048) + 1;
            __acc0 = appy::OpAdd::f<double>(__acc0, ((double)(__ld_A_2.y)));
        }
        {
            const appy::i64 i = (__tile0 + 2048) + 2;
            __acc0 = appy::OpAdd::f<double>(__acc0, ((double)(__ld_A_2.z)));
        }
        {
            const appy::i64 i = (__tile0 + 2048) + 3;
            __acc0 = appy::OpAdd::f<double>(__acc0, ((double)(__ld_A_2.w)));
        }
    }
    const appy::i64 __rest0 = __lo + __ntiles * 4096;
    const appy::i64 __nrv = (__hi - __rest0) / 4;
    for (appy::i64 __q = blockIdx.x * 512LL + __tid; __q < __nrv; __q += __nblk * 512LL) {
        const appy::i64 __vb = __rest0 + __q * 4;
        const appy::vec<float, 4>::type __ld_A_3 = appy::vload_stream<float, 4>(A + (__vb));
        {
            const appy::i64 i = __vb + 0;
            __acc0 = appy::OpAdd::f<double>(__acc0, ((double)(__ld_A_3.x)));
        }
        {
            const appy::i64 i = __vb + 1;
            __acc0 = appy::OpAdd::f<double>(__acc0, ((double)(__ld_A_3.y)));
        }
        {
            const appy::i64 i = __vb + 2;
            __acc0 = appy::OpAdd::f<double>(__acc0, ((double)(__ld_A_3.z)));
        }
        {
            const appy::i64 i = __vb + 3;
            __acc0 = appy::OpAdd::f<double>(__acc0, ((double)(__ld_A_3.w)));
        }
    }
    for (appy::i64 __i = __rest0 + __nrv * 4 + blockIdx.x * 512LL + __tid; __i < __hi; __i += __nblk * 512LL) {
        {
            const appy::i64 i = __i;
            __acc0 = appy::OpAdd::f<double>(__acc0, ((double)(A[i])));
        }
    }
    {
        const double __tot = appy::block_reduce<appy::OpAdd, 512, double>(__acc0, ((double)0));
        if (threadIdx.x == 0) appy::atomic_combine<appy::OpAdd, double>::run(&s[0], __tot);
    }
}
