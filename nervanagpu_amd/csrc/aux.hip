// Small data-movement kernels: 2-D transpose, filter dimension shuffle and the
// fp32 -> storage-type convert, counterparts of nervanagpu/float_ew.py:1325-1428.
// The convolution entry points no longer need them (filter re-layout and the
// update rounding are fused into those launches); they stay exported because
// callers of the reference could reach the same helpers.
#include "ng_internal.h"
#include "ng_device_common.h"

#include <algorithm>

namespace ng {

// out[c][r] = in[r][c] through a padded 64x64 LDS tile (one wavefront row per
// 64 contiguous elements on both the load and the store side)
template <typename T>
__global__ __launch_bounds__(256)
void transpose_kernel(const T* __restrict__ in, T* __restrict__ out, int rows, int cols)
{
    __shared__ T tile[64][65];
    const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
    const int c0 = blockIdx.x * 64, r0 = blockIdx.y * 64;
    for (int j = ty; j < 64; j += 4) {
        const int r = r0 + j, c = c0 + tx;
        if (r < rows && c < cols) tile[j][tx] = in[(long)r * cols + c];
    }
    __syncthreads();
    for (int j = ty; j < 64; j += 4) {
        const int c = c0 + j, r = r0 + tx;
        if (c < cols && r < rows) out[(long)c * rows + r] = tile[tx][j];
    }
}

// out[k][trs][c] = in[c][trs][k]
template <typename T>
__global__ __launch_bounds__(256)
void dimshuffle_kernel(const T* __restrict__ in, T* __restrict__ out, int C, int TRS, int K)
{
    __shared__ T tile[64][65];
    const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
    const int k0 = blockIdx.x * 64, c0 = blockIdx.y * 64, trs = blockIdx.z;
    for (int j = ty; j < 64; j += 4) {
        const int c = c0 + j, k = k0 + tx;
        if (c < C && k < K) tile[j][tx] = in[((long)c * TRS + trs) * K + k];
    }
    __syncthreads();
    for (int j = ty; j < 64; j += 4) {
        const int k = k0 + j, c = c0 + tx;
        if (k < K && c < C) out[((long)k * TRS + trs) * C + c] = tile[tx][j];
    }
}

template <typename T> __device__ __forceinline__ T convert_from_f32(float v);
template <> __device__ __forceinline__ _Float16 convert_from_f32<_Float16>(float v) { return (_Float16)v; }
template <> __device__ __forceinline__ float convert_from_f32<float>(float v) { return v; }
template <> __device__ __forceinline__ unsigned char convert_from_f32<unsigned char>(float v) { return (unsigned char)ng_rint_sat(v, 0.0f, 255.0f); }
template <> __device__ __forceinline__ signed char convert_from_f32<signed char>(float v) { return (signed char)ng_rint_sat(v, -128.0f, 127.0f); }

template <typename T>
__global__ void fp32_convert_kernel(const float* __restrict__ src, T* __restrict__ dst, size_t count)
{
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (; i < count; i += stride) dst[i] = convert_from_f32<T>(src[i]);
}

}  // namespace ng

using namespace ng;

extern "C" {

int ng_transpose(int dtype, const void* in, void* out, int rows, int cols, void* stream)
{
    if (rows <= 0 || cols <= 0) return 0;
    if (!in || !out) return fail(-70, "ng_transpose: null tensor");
    dim3 grid((cols + 63) / 64, (rows + 63) / 64), block(256);
    hipStream_t st = (hipStream_t)stream;
    switch (dtype_size(dtype)) {
    case 2: hipLaunchKernelGGL(transpose_kernel<unsigned short>, grid, block, 0, st, (const unsigned short*)in, (unsigned short*)out, rows, cols); break;
    case 4: hipLaunchKernelGGL(transpose_kernel<unsigned>, grid, block, 0, st, (const unsigned*)in, (unsigned*)out, rows, cols); break;
    default: hipLaunchKernelGGL(transpose_kernel<unsigned char>, grid, block, 0, st, (const unsigned char*)in, (unsigned char*)out, rows, cols); break;
    }
    NG_CHECK_LAUNCH("transpose");
    return 0;
}

int ng_dimshuffle(int dtype, const void* in, void* out, int C, int TRS, int K, void* stream)
{
    if (C <= 0 || TRS <= 0 || K <= 0) return 0;
    if (!in || !out) return fail(-71, "ng_dimshuffle: null tensor");
    if (TRS > 65535) return fail(-72, "ng_dimshuffle: T*R*S too large");
    dim3 grid((K + 63) / 64, (C + 63) / 64, TRS), block(256);
    hipStream_t st = (hipStream_t)stream;
    switch (dtype_size(dtype)) {
    case 2: hipLaunchKernelGGL(dimshuffle_kernel<unsigned short>, grid, block, 0, st, (const unsigned short*)in, (unsigned short*)out, C, TRS, K); break;
    case 4: hipLaunchKernelGGL(dimshuffle_kernel<unsigned>, grid, block, 0, st, (const unsigned*)in, (unsigned*)out, C, TRS, K); break;
    default: hipLaunchKernelGGL(dimshuffle_kernel<unsigned char>, grid, block, 0, st, (const unsigned char*)in, (unsigned char*)out, C, TRS, K); break;
    }
    NG_CHECK_LAUNCH("dimshuffle");
    return 0;
}

int ng_fp32_convert(int dtype, const float* src, void* dst, size_t count, void* stream)
{
    if (count == 0) return 0;
    if (!src || !dst) return fail(-73, "ng_fp32_convert: null tensor");
    const unsigned blocks = (unsigned)std::min<size_t>((count + 255) / 256, 16384);
    hipStream_t st = (hipStream_t)stream;
    switch (dtype) {
    case NG_F16: hipLaunchKernelGGL(fp32_convert_kernel<_Float16>, dim3(blocks), dim3(256), 0, st, src, (_Float16*)dst, count); break;
    case NG_F32: hipLaunchKernelGGL(fp32_convert_kernel<float>, dim3(blocks), dim3(256), 0, st, src, (float*)dst, count); break;
    case NG_U8:  hipLaunchKernelGGL(fp32_convert_kernel<unsigned char>, dim3(blocks), dim3(256), 0, st, src, (unsigned char*)dst, count); break;
    case NG_I8:  hipLaunchKernelGGL(fp32_convert_kernel<signed char>, dim3(blocks), dim3(256), 0, st, src, (signed char*)dst, count); break;
    default: return fail(-74, "ng_fp32_convert: unknown dtype %d", dtype);
    }
    NG_CHECK_LAUNCH("fp32_convert");
    return 0;
}

}  // extern "C"
