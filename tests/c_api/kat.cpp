// Native caller of the GEMM-only C interface, the counterpart of the reference's
// own test program (kernels/C_interface/test.cu:27-124): it includes nothing but
// the interface header and the HIP runtime, and calls nervana_sgemm / nervana_hgemm
// in the reference's 17-argument form (no `grid`).
//
//   kat               known answers: sgemm of ones == size for 11 sizes x {nn, nt, tn},
//                     hgemm of zeros == 0 (test.cu:42-51, 27-40); exit status 1 on any mismatch
//   kat sr FILE       stochastic-round hgemm calls on dyadic operands; operands and raw
//                     results are written to FILE for the caller to compare with the
//                     rounding stream (seed 0, one stream per call, numbered from 1)
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>

#include "nervana_hip.h"

#define HIP_OK(expr)                                                                 \
    do {                                                                             \
        hipError_t e_ = (expr);                                                      \
        if (e_ != hipSuccess) {                                                      \
            std::fprintf(stderr, "%s: %s\n", #expr, hipGetErrorString(e_));          \
            std::exit(2);                                                            \
        }                                                                            \
    } while (0)

static int mismatches = 0;

static void expect_sgemm(float* a, float* b, float* c, bool a_t, bool b_t, int size)
{
    if (!nervana_sgemm(a, b, c, a_t, b_t, size, size, size, size, size, size, 1.0, 0.0, NULL, false, false, 0)) {
        mismatches++;
        return;
    }
    std::vector<float> h((size_t)size * size);
    HIP_OK(hipMemcpy(h.data(), c, sizeof(float) * h.size(), hipMemcpyDeviceToHost));
    for (size_t i = 0; i < h.size(); ++i)
        if (h[i] != (float)size) {
            if (mismatches++ < 10) std::printf("sgemm %d%d size %d: mismatch at %zu: %g != %d\n", a_t, b_t, size, i, h[i], size);
        }
}

static void expect_hgemm(short* a, short* b, short* c, bool a_t, bool b_t, int size)
{
    if (!nervana_hgemm(a, b, c, a_t, b_t, size, size, size, size, size, size, 1.0, 0.0, NULL, false, false, 0)) {
        mismatches++;
        return;
    }
    std::vector<short> h((size_t)size * size);
    HIP_OK(hipMemcpy(h.data(), c, sizeof(short) * h.size(), hipMemcpyDeviceToHost));
    for (size_t i = 0; i < h.size(); ++i)
        if (h[i] != 0) {
            if (mismatches++ < 10) std::printf("hgemm %d%d size %d: mismatch at %zu: %d != 0\n", a_t, b_t, size, i, h[i]);
        }
}

static int known_answers()
{
    const int sizes[] = {257, 256, 255, 129, 128, 127, 65, 64, 17, 16, 15};
    const int big = sizes[0];
    {
        std::vector<float> ones((size_t)big * big, 1.f);
        float *a, *b, *c;
        HIP_OK(hipMalloc(&a, sizeof(float) * ones.size()));
        HIP_OK(hipMalloc(&b, sizeof(float) * ones.size()));
        HIP_OK(hipMalloc(&c, sizeof(float) * ones.size()));
        HIP_OK(hipMemcpy(a, ones.data(), sizeof(float) * ones.size(), hipMemcpyHostToDevice));
        HIP_OK(hipMemcpy(b, ones.data(), sizeof(float) * ones.size(), hipMemcpyHostToDevice));
        for (int size : sizes) {
            expect_sgemm(a, b, c, false, false, size);
            expect_sgemm(a, b, c, false, true, size);
            expect_sgemm(a, b, c, true, false, size);
        }
        HIP_OK(hipFree(a)); HIP_OK(hipFree(b)); HIP_OK(hipFree(c));
    }
    {
        std::vector<short> zeros((size_t)big * big, 0);
        short *a, *b, *c;
        HIP_OK(hipMalloc(&a, sizeof(short) * zeros.size()));
        HIP_OK(hipMalloc(&b, sizeof(short) * zeros.size()));
        HIP_OK(hipMalloc(&c, sizeof(short) * zeros.size()));
        HIP_OK(hipMemcpy(a, zeros.data(), sizeof(short) * zeros.size(), hipMemcpyHostToDevice));
        HIP_OK(hipMemcpy(b, zeros.data(), sizeof(short) * zeros.size(), hipMemcpyHostToDevice));
        HIP_OK(hipMemset(c, 0x3c, sizeof(short) * zeros.size()));   // every output must be overwritten
        for (int size : sizes) {
            expect_hgemm(a, b, c, false, false, size);
            expect_hgemm(a, b, c, false, true, size);
            expect_hgemm(a, b, c, true, false, size);
        }
        HIP_OK(hipFree(a)); HIP_OK(hipFree(b)); HIP_OK(hipFree(c));
    }
    std::printf("known answers: %d mismatches\n", mismatches);
    return mismatches ? 1 : 0;
}

// fp16 bits of j/16 for j in [-16, 16]: products are multiples of 1/256, and sums of
// up to 2^14 of them are exact in fp32 in any order
static short dyadic16(unsigned& state)
{
    static const unsigned short pos[17] = {0x0000, 0x2c00, 0x3000, 0x3200, 0x3400, 0x3500, 0x3600, 0x3700, 0x3800,
                                           0x3880, 0x3900, 0x3980, 0x3a00, 0x3a80, 0x3b00, 0x3b80, 0x3c00};
    state = state * 1664525u + 1013904223u;
    const int j = (int)((state >> 8) % 33u) - 16;
    return (short)(j < 0 ? (pos[-j] | 0x8000) : pos[j]);
}

struct SrCase { int m, n, k, a_t, b_t, relu, other_stream; };

static int stochastic_cases(const char* path)
{
    // an unsliced shape, then a fully-connected shape whose contraction is cut into slices
    // (partial sums in the library's static array), the latter again on a second stream
    const SrCase cases[] = {{256, 128, 192, 0, 0, 1, 0}, {1000, 128, 4096, 0, 0, 0, 0}, {4096, 128, 1000, 1, 0, 0, 1},
                            {136, 264, 128, 0, 1, 1, 1}};
    std::FILE* f = std::fopen(path, "wb");
    if (!f) { std::perror(path); return 2; }
    hipStream_t second;
    HIP_OK(hipStreamCreate(&second));
    unsigned state = 2024u;
    for (const SrCase& c : cases) {
        const size_t na = (size_t)c.m * c.k, nb = (size_t)c.k * c.n, nc = (size_t)c.m * c.n;
        std::vector<short> ha(na), hb(nb), hc(nc);
        for (short& v : ha) v = dyadic16(state);
        for (short& v : hb) v = dyadic16(state);
        short *a, *b, *d;
        HIP_OK(hipMalloc(&a, 2 * na)); HIP_OK(hipMalloc(&b, 2 * nb)); HIP_OK(hipMalloc(&d, 2 * nc));
        HIP_OK(hipMemcpy(a, ha.data(), 2 * na, hipMemcpyHostToDevice));
        HIP_OK(hipMemcpy(b, hb.data(), 2 * nb, hipMemcpyHostToDevice));
        // A is stored (m,k), or (k,m) when transposed; B (k,n), or (n,k) when transposed
        const int lda = c.a_t ? c.m : c.k, ldb = c.b_t ? c.k : c.n;
        std::vector<unsigned> rand_state(nervana_randStateSizeBytes() / sizeof(unsigned), 0u);   // accepted, unused
        hipStream_t st = c.other_stream ? second : (hipStream_t)0;
        if (!nervana_hgemm(a, b, d, c.a_t != 0, c.b_t != 0, c.m, c.n, c.k, lda, ldb, c.n, 1.0f, 0.0f, rand_state.data(),
                           true, c.relu != 0, st)) {
            std::fprintf(stderr, "nervana_hgemm failed\n");
            return 1;
        }
        HIP_OK(hipStreamSynchronize(st));
        HIP_OK(hipMemcpy(hc.data(), d, 2 * nc, hipMemcpyDeviceToHost));
        const int head[6] = {c.m, c.n, c.k, c.a_t, c.b_t, c.relu};
        std::fwrite(head, sizeof(int), 6, f);
        std::fwrite(ha.data(), 2, na, f);
        std::fwrite(hb.data(), 2, nb, f);
        std::fwrite(hc.data(), 2, nc, f);
        HIP_OK(hipFree(a)); HIP_OK(hipFree(b)); HIP_OK(hipFree(d));
    }
    HIP_OK(hipStreamDestroy(second));
    std::fclose(f);
    std::printf("stochastic cases written to %s\n", path);
    return 0;
}

int main(int argc, char** argv)
{
    HIP_OK(hipFree(0));
    if (!nervana_loadKernels("../cubin/")) {
        std::fprintf(stderr, "Couldn't load all kernels\n");
        return 1;
    }
    int rc;
    if (argc >= 3 && std::strcmp(argv[1], "sr") == 0) rc = stochastic_cases(argv[2]);
    else rc = known_answers();
    nervana_unloadKernels();
    return rc;
}
