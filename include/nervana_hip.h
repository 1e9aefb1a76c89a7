/*
 * nervana_hip.h -- C ABI of libnervana_hip.so (MI355X / gfx950).
 *
 * This is the device boundary of the Python host package: everything the
 * reference obtained from pycuda (nervanagpu/nervanagpu.py:18-21) and from its
 * prebuilt cubins is reached through these entry points instead.  Plain
 * pointers and sizes only; every call returns 0 on success or a non-zero code,
 * and ng_last_error() returns a thread-local message for the last failure
 * (the reference's C API returns false and prints to stderr,
 * kernels/C_interface/nervana_c_api.cu:91-94, 286-289).
 *
 * All launches are asynchronous on the given stream (NULL = default stream).
 */
#ifndef NERVANA_HIP_H
#define NERVANA_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#else
#include <stdbool.h>
#endif

/* element types (numpy dtype.str[1:] of the reference: nervanagpu/nervanagpu.py:44) */
enum ng_dtype { NG_F16 = 0, NG_F32 = 1, NG_U8 = 2, NG_I8 = 3 };

/* op flags: same bit meaning as the reference's kernel `flags` argument
 * (nervanagpu/nervanagpu.py:1071-1073): bit0 stochastic round, bit1 relu,
 * bits 16+ mantissa bits to keep when stochastic rounding. */
#define NG_FLAG_SR    1u
#define NG_FLAG_RELU  2u

/* ---- runtime primitives (replace pycuda.driver) ------------------------- */

/* pycuda.autoinit / drv.Context: select the device, create nothing else. */
int ng_init(int device);
int ng_device_count(int* count);
/* drv.Context.get_device().get_attributes() (nervanagpu/layers.py:775-778).
 * attr: 0 compute units, 1 LDS bytes per workgroup, 2 wavefront size,
 *       3 clock kHz, 4 memory clock kHz, 5 L2 bytes */
int ng_device_attr(int attr, int* value);
int ng_device_name(char* buf, size_t cap);
const char* ng_last_error(void);

/* drv.mem_alloc / DeviceAllocation.free (nervanagpu/nervanagpu.py:34, 83) */
int ng_malloc(void** ptr, size_t bytes);
int ng_free(void* ptr);
int ng_mem_info(size_t* free_bytes, size_t* total_bytes);
/* drv.memcpy_htod_async / dtoh_async / dtod_async (nervanagpu.py:133, 145, 311).
 * d2h synchronises the stream before returning (pageable host memory). */
int ng_memcpy_h2d(void* dst, const void* src, size_t bytes, void* stream);
int ng_memcpy_d2h(void* dst, const void* src, size_t bytes, void* stream);
int ng_memcpy_d2d(void* dst, const void* src, size_t bytes, void* stream);
/* drv.memset_d8/d16/d32_async (nervanagpu.py:298-302, 716); count in elements */
int ng_memset8(void* dst, unsigned value, size_t count, void* stream);
int ng_memset16(void* dst, unsigned value, size_t count, void* stream);
int ng_memset32(void* dst, unsigned value, size_t count, void* stream);

int ng_stream_create(void** stream);
int ng_stream_sync(void* stream);
int ng_stream_destroy(void* stream);
/* drv.Event record/synchronize/time_since (nervanagpu.py:712, 727-729) */
int ng_event_create(void** event);
int ng_event_record(void* event, void* stream);
int ng_event_sync(void* event);
int ng_event_elapsed_ms(float* ms, void* start, void* end);
int ng_event_destroy(void* event);

/* pycuda.compiler.SourceModule + get_function + prepared_async_call
 * (nervanagpu/float_ew.py:1030-1033, 1314): run-time compilation of the
 * generated elementwise kernels with hiprtc for the current device. */
int ng_rtc_compile(const char* source, const char* name,
                   const char** options, int n_options,
                   void** module, char* log, size_t log_cap);
int ng_module_get_function(void** function, void* module, const char* name);
int ng_module_unload(void* module);
int ng_launch(void* function, const unsigned grid[3], const unsigned block[3],
              unsigned shared_bytes, void* stream, void** args);

/* ---- GEMM ---------------------------------------------------------------
 * C = round(beta*C + relu(alpha * op(A).op(B))), row-major, fp32 accumulate.
 * Replaces the {h,s}gemm_{nn,nt,tn}* kernels launched by NervanaGPU.dot and
 * batched_dot (nervanagpu/nervanagpu.py:820-957, 959-1105).
 *   trans_a: A is stored (k,m) row-major; trans_b: B is stored (n,k).
 *   lda/ldb/ldc: row pitch in elements.  "tt" is rejected like the reference.
 *   batch_grid independent GEMMs with batch strides ldaz/ldbz/ldcz (0 =
 *   broadcast); batch_loops > 1 sums batch_loops products into one C.
 *   flags: NG_FLAG_*; stochastic rounding draws element (b*m*n + i*n + j) of
 *   the stream (seed, rng_stream).
 *   workspace: fp32 scratch of workspace_bytes for the split-K partial sums;
 *   may be NULL (then no split is used). */
int ng_gemm(int dtype, int trans_a, int trans_b, int m, int n, int k,
            const void* A, int lda, const void* B, int ldb, void* C, int ldc,
            float alpha, float beta, unsigned flags,
            unsigned seed, unsigned rng_stream,
            int batch_grid, long ldaz, long ldbz, long ldcz, int batch_loops,
            void* workspace, size_t workspace_bytes, void* stream);
/* bytes of workspace ng_gemm would like for this problem (0 = none) */
size_t ng_gemm_workspace_bytes(int dtype, int trans_a, int trans_b, int m, int n, int k,
                               int batch_grid, int batch_loops);

/* ng_gemm for callers that cannot allocate device memory or carry a workspace
 * (code under stream capture, tight serving loops, harnesses that forbid
 * hipMalloc).  No counterpart in the reference.  Same arguments and results as
 * ng_gemm given a workspace of ng_gemm_workspace_bytes(): the split partial
 * sums go to a fixed array of NG_GEMM_STATIC_SCRATCH_BYTES that is part of the
 * library image on every device (ng_init looks up its address).  A problem that
 * wants more is refused with an error.  The call allocates and frees nothing.
 * All calls on one device share the array: calls that overlap in time on one
 * device (different streams or threads) race; calls on one stream do not. */
#define NG_GEMM_STATIC_SCRATCH_BYTES (32u << 20)
size_t ng_gemm_static_scratch_bytes(void);
int ng_gemm_noalloc(int dtype, int trans_a, int trans_b, int m, int n, int k,
                    const void* A, int lda, const void* B, int ldb, void* C, int ldc,
                    float alpha, float beta, unsigned flags,
                    unsigned seed, unsigned rng_stream,
                    int batch_grid, long ldaz, long ldbz, long ldcz, int batch_loops,
                    void* stream);

/* GEMM-only C entry compatible with kernels/C_interface/nervana_c_api.h:31-128
 * (CUstream -> hipStream_t passed as void*; rand_state is unused because the
 * random stream is counter based: seed 0, one stream per stochastic call,
 * numbered from 1 in call order; `grid` is accepted and ignored, and defaults
 * to -1 for C++ callers as at nervana_c_api.h:74,107,117,127, so the 17-argument
 * calls of kernels/C_interface/test.cu:28,43 compile unchanged).  Shapes that
 * fill the chip only with a sliced contraction keep their partial sums in the
 * static array of ng_gemm_noalloc; calls on different streams that use it are
 * ordered among themselves with an event. */
#ifdef __cplusplus
#define NG_GRID_DEFAULT = -1
#else
#define NG_GRID_DEFAULT
#endif
bool nervana_loadKernels(const char* base_path);
bool nervana_unloadKernels(void);
size_t nervana_randStateSizeBytes(void);
bool nervana_sgemm(float* A, float* B, float* C, bool a_t, bool b_t,
                   int m, int n, int k, int lda, int ldb, int ldc,
                   float alpha, float beta, unsigned int* rand_state,
                   bool stochastic_round, bool apply_relu, void* stream, int grid NG_GRID_DEFAULT);
bool nervana_hgemm(short* A, short* B, short* C, bool a_t, bool b_t,
                   int m, int n, int k, int lda, int ldb, int ldc,
                   float alpha, float beta, unsigned int* rand_state,
                   bool stochastic_round, bool apply_relu, void* stream, int grid NG_GRID_DEFAULT);
bool nervana_sgemm_colmajor(float* A, float* B, float* C, bool a_t, bool b_t,
                            int m, int n, int k, int lda, int ldb, int ldc,
                            float alpha, float beta, unsigned int* rand_state,
                            bool stochastic_round, bool apply_relu, void* stream, int grid NG_GRID_DEFAULT);
bool nervana_hgemm_colmajor(short* A, short* B, short* C, bool a_t, bool b_t,
                            int m, int n, int k, int lda, int ldb, int ldc,
                            float alpha, float beta, unsigned int* rand_state,
                            bool stochastic_round, bool apply_relu, void* stream, int grid NG_GRID_DEFAULT);

/* ---- convolution ----------------------------------------------------------
 * Direct convolution in CHWN layout: I (C,D,H,W,N), F (C,T,R,S,K),
 * O/E (K,M,P,Q,N), all row-major with N innermost.  Replaces
 * {h,s}conv_{fprop,bprop,updat}_* launched by NervanaGPU._execute_conv
 * (nervanagpu/nervanagpu.py:642-734) and the dimShuffle / transpose / fp32
 * convert helper launches that surround them (nervanagpu/float_ew.py:1325-1428).
 * Geometry mirrors ConvLayer (nervanagpu/layers.py:279-326). */
typedef struct ng_conv_params {
    int N, C, K;
    int D, H, W;
    int T, R, S;
    int M, P, Q;
    int pad_d, pad_h, pad_w;
    int str_d, str_h, str_w;
} ng_conv_params;

/* ConvLayer.__init__ precomputes every launch constant once per layer
 * (nervanagpu/layers.py:281-481); the plan is the counterpart: it owns the small
 * device-side tap tables of one geometry.  dtype is the storage type of the
 * filters and of the fprop/bprop outputs (NG_F16 or NG_F32). */
int ng_conv_plan_create(const ng_conv_params* p, int dtype, void** plan);
int ng_conv_plan_destroy(void* plan);
/* scratch bytes the three conv ops may use for this plan (filter re-layout for
 * the bprop of layers with few channels or output maps, split partial sums for
 * update and for fprop / bprop grids much smaller than the chip; may be 0); the
 * reference keeps one shared scratch buffer for the first two purposes
 * (nervanagpu/nervanagpu.py:686-698).  fprop, and bprop when it needs no filter
 * re-layout, also run without a workspace (unsliced). */
size_t ng_conv_plan_workspace_bytes(const void* plan);
/* O = round(relu?(alpha * conv(I, F))).  in_dtype may be NG_U8/NG_I8 with
 * NG_F16 filters and output: the bytes are converted exactly on load (declared
 * at README.md:37, stubs kernels/cu/hconv_fprop_u8_K64_N64.cu:19-40). */
int ng_conv_fprop(const void* plan, int in_dtype,
                  const void* I, const void* F, void* O, float alpha, unsigned flags,
                  void* workspace, size_t workspace_bytes, void* stream);
/* gradI = round(alpha * conv_transpose(E, F)); deterministic gather form, every
 * element of gradI is written (no zero fill needed).  relu_mask: NULL, or (unit
 * strides only) the activations of the layer below, a tensor shaped like gradI:
 * gradI is additionally multiplied by (relu_mask > 0), the derivative step that
 * layer would apply next (`bprop_in *= fprop_out > 0`, nervanagpu/layers.py:89-91),
 * for one read of the activations instead of an elementwise pass over both. */
int ng_conv_bprop(const void* plan,
                  const void* F, const void* E, void* gradI, float alpha, const void* relu_mask,
                  void* workspace, size_t workspace_bytes, void* stream);
/* gradF = round(alpha * sum_{pixels,n} I x E); out_dtype NG_F32 or NG_F16;
 * fp32 accumulation with a fixed-order reduction of the split partial sums */
int ng_conv_update(const void* plan, int in_dtype, int out_dtype,
                   const void* I, const void* E, void* gradF, float alpha,
                   void* workspace, size_t workspace_bytes, void* stream);

/* ---- pooling ----------------------------------------------------------------
 * Replaces {h,s}pool_max launched by NervanaGPU._execute_pool
 * (nervanagpu/nervanagpu.py:789-818); geometry mirrors PoolLayer
 * (nervanagpu/layers.py:540-626).  op: 0 max, 1 avg, 2 l2 (square root of the sum of squares,
 * benchmarks/pool_test.py:145-146; forward only). */
typedef struct ng_pool_params {
    int N, C, D, H, W;
    int J, T, R, S;
    int K, M, P, Q;
    int pad_j, pad_d, pad_h, pad_w;
    int str_j, str_d, str_h, str_w;
} ng_pool_params;

int ng_pool_fprop(const ng_pool_params* p, int dtype, int op,
                  const void* I, void* O, void* stream);
/* gradI is fully written (no zero fill needed); window overlap is resolved by a
 * gather over the windows touching each input element, so the result does not
 * depend on execution order.  Overlapping max pooling keeps one byte per output
 * element (the argmax slot) in `workspace`. */
size_t ng_pool_workspace_bytes(const ng_pool_params* p, int dtype, int op);
/* flags: 0, or NG_FLAG_RELU for max pooling over at most 255 elements when I is
 * the output of a rectifier: gradI is additionally multiplied by (I > 0), the
 * derivative step the layer below would apply next (`bprop_in *= fprop_out > 0`,
 * nervanagpu/layers.py:89-91), at no extra memory traffic. */
int ng_pool_bprop(const ng_pool_params* p, int dtype, int op,
                  const void* I, const void* E, void* gradI, unsigned flags,
                  void* workspace, size_t workspace_bytes, void* stream);

/* ---- small data-movement helpers ---------------------------------------------
 * transpose / dimShuffle / fp32 convert kernels of nervanagpu/float_ew.py:1325-1428 */
int ng_transpose(int dtype, const void* in, void* out, int rows, int cols, void* stream);
/* out[k,t,r,s,c] = in[c,t,r,s,k] with TRS = T*R*S */
int ng_dimshuffle(int dtype, const void* in, void* out, int C, int TRS, int K, void* stream);
/* dst (dtype, nearest rounding) = src (fp32) */
int ng_fp32_convert(int dtype, const float* src, void* dst, size_t count, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* NERVANA_HIP_H */
