// Measurement probe: a loop of back-to-back MFMA instructions with no memory
// traffic.  What it reaches on random operands is the practical ceiling of the
// matrix pipes at the clock the power limit allows, the yardstick the GEMM and
// convolution kernels are compared with besides the nameplate peak.
#include "ng_internal.h"

namespace ng {

typedef _Float16 probe_half8_t   __attribute__((ext_vector_type(8)));
typedef float    probe_float16_t __attribute__((ext_vector_type(16)));

// 256 threads = one wavefront per SIMD; 16 independent 32x32 accumulators per
// wavefront, so the pipe never waits on a dependency
__global__ __launch_bounds__(256)
void mfma_loop_kernel(float* out, int iters, int random_data)
{
    probe_half8_t a, b;
    unsigned h = (blockIdx.x * 256u + threadIdx.x) * 2654435761u + 12345u;
#pragma unroll
    for (int i = 0; i < 8; i++) {
        h ^= h >> 15; h *= 0x2c1b3c6du; h ^= h >> 12; h *= 0x297a2d39u; h ^= h >> 15;
        a[i] = random_data ? (_Float16)(((int)(h & 2047) - 1024) * (1.0f / 1024)) : (_Float16)1.0f;
        b[i] = random_data ? (_Float16)(((int)((h >> 11) & 2047) - 1024) * (1.0f / 1024)) : (_Float16)0.5f;
    }
    probe_float16_t acc[16];
#pragma unroll
    for (int j = 0; j < 16; j++)
#pragma unroll
        for (int v = 0; v < 16; v++) acc[j][v] = 0.0f;
    for (int it = 0; it < iters; it++) {
#pragma unroll
        for (int j = 0; j < 16; j++) acc[j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, acc[j], 0, 0, 0);
    }
    float s = 0.0f;
#pragma unroll
    for (int j = 0; j < 16; j++)
#pragma unroll
        for (int v = 0; v < 16; v++) s += acc[j][v];
    out[blockIdx.x * 256u + threadIdx.x] = s;
}

}  // namespace ng

using namespace ng;

// out: blocks * 256 floats.  Flops of one launch: blocks * 4 * iters * 16 * 32768.
extern "C" int ng_probe_mfma_loop(int blocks, int iters, int random_data, float* out, void* stream)
{
    if (blocks <= 0 || iters < 0) return fail(-80, "ng_probe_mfma_loop: bad extent");
    if (!out) return fail(-81, "ng_probe_mfma_loop: null output");
    hipLaunchKernelGGL(mfma_loop_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, out, iters, random_data);
    NG_CHECK_LAUNCH("mfma loop probe");
    return 0;
}
