// Compile check of the device support header with the offline compiler:
// instantiates every template once for the element types kernels use.
#include "appy_device.h"

extern "C" __global__ void __launch_bounds__(256)
appy_device_check(const float* __restrict__ a, const double* __restrict__ b, const int* __restrict__ c,
                  float* __restrict__ of, double* __restrict__ od, long long* __restrict__ ol, long long n) {
    const long long t = blockIdx.x * 256ll + threadIdx.x;
    float f = 0.f;
    double d = 0.0;
    long long l = 0;
    if (t * 4 + 4 <= n) {
        auto v = appy::vload<float, 4>(a + t * 4);
        auto w = appy::vload_stream<double, 2>(b + t * 2);
        auto u = appy::vload<int, 4>(c + t * 4);
        f = v.x + v.y + v.z + v.w;
        d = w.x + w.y;
        l = appy::floordiv_int<long long>(u.x, 3) + appy::mod_int<int>(u.y, 5) + appy::ipow<long long>(u.z, 2);
        appy::vstore<float, 4>(of + t * 4, v);
    }
    f = appy::team_reduce<appy::OpAdd, 16>(f);
    d = appy::team_reduce<appy::OpMax, 64>(d);
    l = appy::team_reduce<appy::OpMin, 4>(l);
    const float bf = appy::block_reduce<appy::OpAdd, 256>(f, 0.f);
    const double bd = appy::block_reduce<appy::OpMax, 256>(d, -__builtin_inf());
    const long long bl = appy::block_reduce<appy::OpAdd, 256>(l, 0ll);
    if (threadIdx.x == 0) {
        appy::atomic_combine<appy::OpAdd, float>::run(of, bf);
        appy::atomic_combine<appy::OpMax, double>::run(od, bd);
        appy::atomic_combine<appy::OpAdd, long long>::run(ol, bl);
        appy::atomic_combine<appy::OpMul, double>::run(od + 1, appy::mod_float(bd, 3.0));
    }
    {
        const float wf = appy::workgroup_reduce_all<appy::OpAdd, 256>(f, 0.f);
        if (threadIdx.x == 255) of[1] = wf;
    }
}
