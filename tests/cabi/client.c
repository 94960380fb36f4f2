/* A C client of libappy_hip.so: proves that include/appy_hip.h is plain C and
 * that the library can be driven without Python.  Usage:
 *   client compile   - compile a kernel through the C ABI (no GPU needed), print "compiled <bytes>"
 *   client run       - compile, load, launch c[i] = a[i] + b[i] on device 0, verify on the host
 */
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "appy_hip.h"

static const char* SRC =
    "extern \"C\" __global__ void add(float* c, const float* a, const float* b, long long n) {\n"
    "  long long i = blockIdx.x * 256ll + threadIdx.x;\n"
    "  if (i < n) c[i] = a[i] + b[i];\n"
    "}\n";

#define CHECK(call)                                                              \
    do {                                                                         \
        int rc__ = (call);                                                       \
        if (rc__ != 0) {                                                         \
            fprintf(stderr, "%s failed (%d): %s\n", #call, rc__, appy_hip_last_error()); \
            return 1;                                                            \
        }                                                                        \
    } while (0)

struct add_args {
    void* c;
    const void* a;
    const void* b;
    long long n;
};

int main(int argc, char** argv) {
    const char* opts[] = {"-O3", "-ffp-contract=off"};
    void* code = NULL;
    size_t size = 0;
    if (appy_hip_abi_version() != APPY_HIP_ABI_VERSION) {
        fprintf(stderr, "ABI version mismatch\n");
        return 1;
    }
    CHECK(appy_hip_compile(SRC, "add.hip", "gfx950", opts, 2, &code, &size));
    if (argc < 2 || strcmp(argv[1], "compile") == 0) {
        printf("compiled %zu\n", size);
        appy_hip_code_free(code);
        return 0;
    }
    {
        enum { N = 100003 };
        float *a = malloc(N * sizeof(float)), *b = malloc(N * sizeof(float)), *c = malloc(N * sizeof(float));
        void *da, *db, *dc, *mod, *fn;
        struct add_args args;
        long long i, bad = 0;
        for (i = 0; i < N; ++i) { a[i] = (float)i * 0.5f; b[i] = (float)(N - i); c[i] = -1.0f; }
        CHECK(appy_hip_init(0));
        CHECK(appy_hip_module_load(code, size, &mod));
        CHECK(appy_hip_module_get_function(mod, "add", &fn));
        CHECK(appy_hip_malloc(N * sizeof(float), &da));
        CHECK(appy_hip_malloc(N * sizeof(float), &db));
        CHECK(appy_hip_malloc(N * sizeof(float), &dc));
        CHECK(appy_hip_memcpy_h2d(da, a, N * sizeof(float), NULL));
        CHECK(appy_hip_memcpy_h2d(db, b, N * sizeof(float), NULL));
        args.c = dc; args.a = da; args.b = db; args.n = N;
        CHECK(appy_hip_launch(fn, (N + 255) / 256, 1, 1, 256, 1, 1, 0, NULL, &args, sizeof(args)));
        CHECK(appy_hip_memcpy_d2h(c, dc, N * sizeof(float), NULL));
        for (i = 0; i < N; ++i) bad += (c[i] != a[i] + b[i]);
        CHECK(appy_hip_free(da));
        CHECK(appy_hip_free(db));
        CHECK(appy_hip_free(dc));
        CHECK(appy_hip_module_unload(mod));
        appy_hip_code_free(code);
        free(a); free(b); free(c);
        printf("ran %d elements, %lld mismatches\n", (int)N, bad);
        return bad ? 2 : 0;
    }
}
