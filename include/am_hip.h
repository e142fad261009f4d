/*
 * am_hip.h — C ABI of libam_hip.so, the MI355X (gfx950) backend for Arraymancer's
 * GEMM + broadcast/map hot path.
 *
 * Everything here is plain C: device pointers are `void*`/`T*` obtained from
 * am_hip_malloc, sizes and strides are int64_t counted in ELEMENTS (as in the
 * reference's Tensor metadata, src/arraymancer/laser/tensor/datatypes.nim:19-48),
 * and every entry point returns an int status (0 = AM_OK, negative = error; the text of
 * the last error of the calling thread is available from am_hip_last_error()).
 *
 * All work is enqueued on one library-owned HIP stream; results are visible to the host
 * after am_hip_sync() or any am_hip_memcpy_d2h(). The library keeps no caller pointer
 * after a call returns. One host thread at a time may call into the library (the
 * reference's GPU backends have the same contract:
 * src/arraymancer/tensor/backend/cuda_global_state.nim:21-39).
 *
 * "Reference" citations below are paths under the Arraymancer source tree.
 */
#ifndef AM_HIP_H
#define AM_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---------------------------------------------------------------- status codes */
#define AM_OK          0
#define AM_E_ARG      (-1)  /* null pointer, negative size, rank outside 0..6, unknown op      */
#define AM_E_SHAPE    (-2)  /* shapes/strides that the operation cannot accept                  */
#define AM_E_DTYPE    (-3)  /* op not defined for this element type (e.g. tanh on int32)        */
#define AM_E_ALLOC    (-4)  /* device allocation failed                                         */
#define AM_E_HIP      (-5)  /* a HIP runtime call failed; see am_hip_last_error()               */
#define AM_E_NODEVICE (-6)  /* no usable gfx950 device                                          */

#define AM_MAXRANK 6        /* LASER_MAXRANK, src/arraymancer/laser/dynamic_stack_arrays.nim:6  */

/* ---------------------------------------------------------------- runtime
 * Replaces the CUDA backend's global state + memory glue:
 *   src/arraymancer/tensor/backend/cuda_global_state.nim:21-39 (stream/handle creation)
 *   src/arraymancer/tensor/backend/cuda.nim:23-57            (cudaMalloc / deallocCuda)
 *   src/arraymancer/tensor/init_cuda.nim:23-59               (H2D async copy, D2H blocking copy)
 */
const char* am_hip_last_error(void);
const char* am_hip_version(void);

/* Select and initialise `device` (>= 0). Idempotent; called lazily with device 0 by every
 * other entry point if the caller never calls it. */
int am_hip_init(int device);
int am_hip_device_count(int* count);
/* name: caller buffer of name_cap bytes (NUL terminated on return); any out pointer may be NULL. */
int am_hip_device_info(char* name, size_t name_cap, int* compute_units, int* clock_khz,
                       size_t* hbm_bytes, int* lds_bytes_per_cu);

/* Device memory (newCudaStorage / deallocCuda, src/arraymancer/tensor/backend/cuda.nim:23-57). Freed
 * blocks are cached per size and reused: freeing does not synchronise the device, and a block may be
 * handed out again while earlier work on the library stream still uses it (whatever touches it next
 * goes through that stream too). am_hip_free only accepts pointers from am_hip_malloc. */
int am_hip_malloc(size_t bytes, void** out);   /* bytes == 0 -> *out = NULL, AM_OK */
int am_hip_free(void* dptr);                   /* NULL is a no-op. While a graph is being captured the block is not
                                                  released but kept for that graph (its kernels may use it) until
                                                  am_hip_graph_destroy; it counts as live meanwhile. */
/* No counterpart in the reference (it cudaMallocs / cudaFrees per tensor): returns every cached
 * block to the driver (drains the stream first); byte counts of the blocks in use and in the cache.
 * Cache size limit: environment variable AM_HIP_CACHE_LIMIT_MB (default 32768; 0 = no caching). */
int am_hip_empty_cache(void);
int am_hip_memory_stats(size_t* live_bytes, size_t* cached_bytes);
/* Free and total device memory as the driver reports them (hipMemGetInfo): unlike am_hip_memory_stats this sees
 * every allocation of the process, the library's own workspaces included. No counterpart in the reference. */
int am_hip_device_free_bytes(size_t* free_bytes, size_t* total_bytes);
int am_hip_memcpy_h2d(void* dst, const void* src, size_t bytes);  /* host buffer reusable on return */
int am_hip_memcpy_d2h(void* dst, const void* src, size_t bytes);  /* blocking, ordered after prior work */
int am_hip_memcpy_d2d(void* dst, const void* src, size_t bytes);  /* stream ordered */
int am_hip_memset(void* dst, int byte_value, size_t bytes);       /* stream ordered */
int am_hip_sync(void);
/* The library's hipStream_t as an opaque pointer (for callers that enqueue their own work). */
void* am_hip_stream(void);

/* Timing on the library stream (HIP events). */
int am_hip_event_create(void** ev);
int am_hip_event_record(void* ev);
int am_hip_event_elapsed_ms(void* start, void* stop, float* ms); /* synchronises on `stop` */
int am_hip_event_destroy(void* ev);

/* HIP graphs on the library stream: between begin and end, GEMM / element-wise calls are recorded
 * instead of executed (copies, memset and sync are refused meanwhile, allocation is served from the cache: see
 * am_hip_alloc_hold); the returned
 * executable graph replays the whole sequence with one launch. For launch-bound chains of small
 * kernels such as the reference's per-layer gemm + `+.=` + relu sequence
 * (src/arraymancer/nn_primitives/nnp_linear.nim:28-29, fallback/conv.nim:99-106). The reference
 * has no counterpart (one launch per operator, backend/cuda.nim). Buffers recorded in a graph must
 * stay allocated while it is replayed: a block freed DURING the capture is kept alive by the graph itself,
 * one freed after am_hip_graph_end is the caller's responsibility. */
int am_hip_graph_begin(void);
/* Memory for a capture. am_hip_malloc during a capture is served from the library's cache of freed blocks only (the
 * driver cannot be asked for memory while the stream records) and fails with AM_E_ALLOC when the cache has no block of
 * that size. am_hip_alloc_hold(1) ... am_hip_alloc_hold(0) around one ordinary run of the sequence prepares that cache:
 * while the hold is on, freed blocks are set aside instead of being handed out again, so that every allocation of the
 * sequence gets a block of its own, and switching it off puts them all into the cache. The same sequence recorded right
 * afterwards then finds one block per allocation (and the library workspace at its final size). No counterpart in the
 * reference. */
int am_hip_alloc_hold(int on);
int am_hip_graph_end(void** graph_exec);
/* Both accept only a graph that am_hip_graph_end returned and am_hip_graph_destroy has not taken back yet: any other
 * pointer (stale, destroyed twice, foreign) is refused with AM_E_ARG instead of reaching the runtime. NULL: launch
 * refuses it, destroy ignores it. */
int am_hip_graph_launch(void* graph_exec);
int am_hip_graph_destroy(void* graph_exec);

/* ---------------------------------------------------------------- GEMM
 * C[M x N] <- alpha * A[M x K] * B[K x N] + beta * C, element X[r,c] = X[r*rsX + c*csX].
 *
 * Replaces laser `gemm_strided`
 *   src/arraymancer/laser/primitives/matrix_multiplication/gemm.nim:192-201 (signature)
 *   gemm.nim:117-184 (loop nest), gemm_ukernel_generic.nim:53-125 (epilogues)
 * and what reaches it through the Tensor API:
 *   src/arraymancer/tensor/operators_blas_l2l3.nim:58-100 (`*`, gemm)
 *   src/arraymancer/tensor/private/p_operator_blas_l2l3.nim:110-215.
 *
 * Semantics kept from the reference:
 *   - pointers already include the tensor offset; strides are in elements and may be
 *     zero or negative for A and B (views, broadcast, reversed slices). No host copy is made.
 *   - beta == 0 overwrites C (old NaN/Inf in C never propagate); beta is applied once.
 *   - alpha == 0 is not special-cased (NaN/Inf in A or B propagate).
 *   - K == 0 (or M == 0 or N == 0) leaves C untouched, beta is NOT applied.
 *   - integer types wrap modulo 2^32 / 2^64.
 * C must not overlap itself (no zero stride on a dimension of extent > 1) nor A or B.
 *
 * Large integer products run on the int8 matrix cores (the operands are split into base-256
 * digit planes in scratch device memory taken from the block cache behind am_hip_malloc; ring
 * arithmetic, so the bits are those of the vector-ALU kernel); small ones, batched ones and
 * calls made while a graph is being captured use the vector-ALU kernel and allocate nothing.
 */
int am_hip_gemm_f32(int64_t M, int64_t N, int64_t K, float alpha,
                    const float* A, int64_t rsA, int64_t csA,
                    const float* B, int64_t rsB, int64_t csB,
                    float beta, float* C, int64_t rsC, int64_t csC);
int am_hip_gemm_f64(int64_t M, int64_t N, int64_t K, double alpha,
                    const double* A, int64_t rsA, int64_t csA,
                    const double* B, int64_t rsB, int64_t csB,
                    double beta, double* C, int64_t rsC, int64_t csC);
int am_hip_gemm_i32(int64_t M, int64_t N, int64_t K, int32_t alpha,
                    const int32_t* A, int64_t rsA, int64_t csA,
                    const int32_t* B, int64_t rsB, int64_t csB,
                    int32_t beta, int32_t* C, int64_t rsC, int64_t csC);
int am_hip_gemm_i64(int64_t M, int64_t N, int64_t K, int64_t alpha,
                    const int64_t* A, int64_t rsA, int64_t csA,
                    const int64_t* B, int64_t rsB, int64_t csB,
                    int64_t beta, int64_t* C, int64_t rsC, int64_t csC);

/* Integer products whose operand is reused (a weight matrix that enters many products): large int32 / int64 products
 * run on the int8 matrix cores after both operands have been split into base-256 digit planes, two passes over every
 * operand in every call. am_hip_digits_prepare_* makes those planes once for one operand and returns a handle;
 * am_hip_gemm_prepared_* is am_hip_gemm_i32 / _i64 with such a handle beside either operand (NULL = split that operand
 * in the call, as always). Same result bits as am_hip_gemm_* (ring arithmetic). No counterpart in the reference, whose
 * gemm_strided packs both operands in every call (gemm_packing.nim:24-99).
 *   side 0: X is the left operand [rows x cols] = [M x K]; side 1: the right operand [K x N]; element [r, c] at
 *   X[r * rs + c * cs], any strides. Blocking (it reports which planes came out empty). The planes take
 *   sizeof(T) x roundup(M or N, 256) x roundup(K, 256) bytes from am_hip_malloc until am_hip_digits_release.
 * The planes are a snapshot: after the operand's elements change, release the handle and prepare again. The original
 * operand is still passed to am_hip_gemm_prepared_*: products that cannot take the matrix-core path (a long int64 k,
 * one operand unprepared while a graph is being captured) are computed from it. A handle whose extents do not match
 * the product is refused with AM_E_SHAPE, a pointer that is no live handle with AM_E_ARG. */
int am_hip_digits_prepare_i32(int side, int64_t rows, int64_t cols, const int32_t* X, int64_t rs, int64_t cs, void** handle);
int am_hip_digits_prepare_i64(int side, int64_t rows, int64_t cols, const int64_t* X, int64_t rs, int64_t cs, void** handle);
int am_hip_digits_release(void* handle);   /* NULL is a no-op; a released or foreign pointer is AM_E_ARG */
int am_hip_gemm_prepared_i32(int64_t M, int64_t N, int64_t K, int32_t alpha,
                             const int32_t* A, int64_t rsA, int64_t csA, const void* A_digits,
                             const int32_t* B, int64_t rsB, int64_t csB, const void* B_digits,
                             int32_t beta, int32_t* C, int64_t rsC, int64_t csC);
int am_hip_gemm_prepared_i64(int64_t M, int64_t N, int64_t K, int64_t alpha,
                             const int64_t* A, int64_t rsA, int64_t csA, const void* A_digits,
                             const int64_t* B, int64_t rsB, int64_t csB, const void* B_digits,
                             int64_t beta, int64_t* C, int64_t rsC, int64_t csC);

/* am_hip_gemm_f32 for callers that cannot allocate device memory (code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc). No counterpart in the reference. Same
 * arguments and kernels as am_hip_gemm_f32, and the same tile and split of K - hence the same result
 * bits - wherever am_hip_gemm_f32's own plan keeps its partial tiles within 16 MiB and cuts no strips
 * off (it runs extents of 512 or more that lie 1..16 above a multiple of 64 as an aligned block plus
 * strips; this entry point runs them whole). Outside those cases this entry point takes the best plan
 * that fits its array: both results meet the float32 bar, the last bits may differ. The difference is
 * where the split-K partial tiles go (products with few output tiles and a long K are cut along K
 * over several workgroups):
 * am_hip_gemm_f32 takes a workspace from hipMalloc on first use, this entry point uses a 16 MiB
 * array that is part of the library's device code and calls no hipMalloc / hipFree nor any routine
 * that allocates. Each device the library runs on holds that array until the process ends.
 * Limit: a product whose plan needs more than 16 MiB of partials (splits * M * N * 4 bytes, splits
 * <= 32; only products of fewer than 512 wavefront tiles are split at all, so M * N <= 131072 always
 * fits and large products need none) is refused with AM_E_SHAPE and a message that says so.
 * All calls on a device share the array, which keeps the last call's contents (every partial is
 * written before it is read, so nothing has to be cleared). Calls that overlap on one device would
 * race on it; the library's contract (one calling thread at a time, one stream) rules that out. */
int am_hip_gemm_noalloc_f32(int64_t M, int64_t N, int64_t K, float alpha,
                            const float* A, int64_t rsA, int64_t csA,
                            const float* B, int64_t rsB, int64_t csB,
                            float beta, float* C, int64_t rsC, int64_t csC);

/* GEMM with a fused element-wise epilogue:
 *   C <- act( alpha*A*B + beta*C + bias ),  bias[r,c] = bias[r*bias_rs + c*bias_cs]
 * (bias_rs = 0, bias_cs = 1 is the [1,N] row vector of `linear`).
 * Fuses the three passes of the reference's dense layer
 *   src/arraymancer/nn_primitives/nnp_linear.nim:20-29 (gemm, then `+.=` bias)
 *   src/arraymancer/nn_primitives/nnp_activation.nim:35-36 (relu = max(0, x))
 * at the spot the reference marks for it (gemm_ukernel_generic.nim:50-51,78-79; gemm.nim:204).
 */
#define AM_EPI_NONE      0
#define AM_EPI_BIAS      1   /* + bias                      */
#define AM_EPI_RELU      2   /* (0 >= x) ? 0 : x            */
#define AM_EPI_BIAS_RELU 3   /* relu(x + bias)              */
int am_hip_gemm_ex_f32(int64_t M, int64_t N, int64_t K, float alpha,
                       const float* A, int64_t rsA, int64_t csA,
                       const float* B, int64_t rsB, int64_t csB,
                       float beta, float* C, int64_t rsC, int64_t csC,
                       int epilogue, const float* bias, int64_t bias_rs, int64_t bias_cs);
int am_hip_gemm_ex_f64(int64_t M, int64_t N, int64_t K, double alpha,
                       const double* A, int64_t rsA, int64_t csA,
                       const double* B, int64_t rsB, int64_t csB,
                       double beta, double* C, int64_t rsC, int64_t csC,
                       int epilogue, const double* bias, int64_t bias_rs, int64_t bias_cs);

/* Strided-batched GEMM: for z in 0..batch-1, C + z*batch_stride_C <- alpha * (A + z*batch_stride_A)
 * * (B + z*batch_stride_B) + beta * C_z, one launch. A batch stride of 0 shares the operand (the
 * convolution kernel matrix). The bias is shared by the batch. Integer types: epilogue must be
 * AM_EPI_NONE. Replaces the per-image GEMM loop of the reference's convolution
 * (src/arraymancer/nn_primitives/fallback/conv.nim:99-103, "TODO: batch matmul"); the CUDA backend
 * wraps cublas gemmStridedBatched for the same purpose (backend/cublas.nim:172-208). */
int am_hip_gemm_batched_f32(int64_t batch, int64_t M, int64_t N, int64_t K, float alpha,
                            const float* A, int64_t rsA, int64_t csA, int64_t batch_stride_A,
                            const float* B, int64_t rsB, int64_t csB, int64_t batch_stride_B,
                            float beta, float* C, int64_t rsC, int64_t csC, int64_t batch_stride_C,
                            int epilogue, const float* bias, int64_t bias_rs, int64_t bias_cs);
int am_hip_gemm_batched_f64(int64_t batch, int64_t M, int64_t N, int64_t K, double alpha,
                            const double* A, int64_t rsA, int64_t csA, int64_t batch_stride_A,
                            const double* B, int64_t rsB, int64_t csB, int64_t batch_stride_B,
                            double beta, double* C, int64_t rsC, int64_t csC, int64_t batch_stride_C,
                            int epilogue, const double* bias, int64_t bias_rs, int64_t bias_cs);
int am_hip_gemm_batched_i32(int64_t batch, int64_t M, int64_t N, int64_t K, int32_t alpha,
                            const int32_t* A, int64_t rsA, int64_t csA, int64_t batch_stride_A,
                            const int32_t* B, int64_t rsB, int64_t csB, int64_t batch_stride_B,
                            int32_t beta, int32_t* C, int64_t rsC, int64_t csC, int64_t batch_stride_C,
                            int epilogue, const int32_t* bias, int64_t bias_rs, int64_t bias_cs);
int am_hip_gemm_batched_i64(int64_t batch, int64_t M, int64_t N, int64_t K, int64_t alpha,
                            const int64_t* A, int64_t rsA, int64_t csA, int64_t batch_stride_A,
                            const int64_t* B, int64_t rsB, int64_t csB, int64_t batch_stride_B,
                            int64_t beta, int64_t* C, int64_t rsC, int64_t csC, int64_t batch_stride_C,
                            int epilogue, const int64_t* bias, int64_t bias_rs, int64_t bias_cs);

/* col[n][c*kH*kW + kh*kW + kw][h*W_out + w] <- padded input patch element, for the whole batch in
 * one launch; `in` is addressed through its four NCHW strides (elements), `col` is a contiguous
 * [N, C*kH*kW, H_out*W_out] buffer. H_out = (H + 2 padH - kH) / strideH + 1, W_out alike.
 * Replaces im2col (src/arraymancer/nn_primitives/fallback/conv.nim:18-54). */
int am_hip_im2col_f32(int64_t N, int C, int H, int W, int kH, int kW, int padH, int padW, int strideH, int strideW,
                      const float* in, int64_t in_n, int64_t in_c, int64_t in_h, int64_t in_w, float* col);
int am_hip_im2col_f64(int64_t N, int C, int H, int W, int kH, int kW, int padH, int padW, int strideH, int strideW,
                      const double* in, int64_t in_n, int64_t in_c, int64_t in_h, int64_t in_w, double* col);
int am_hip_im2col_i32(int64_t N, int C, int H, int W, int kH, int kW, int padH, int padW, int strideH, int strideW,
                      const int32_t* in, int64_t in_n, int64_t in_c, int64_t in_h, int64_t in_w, int32_t* col);
int am_hip_im2col_i64(int64_t N, int C, int H, int W, int kH, int kW, int padH, int padW, int strideH, int strideW,
                      const int64_t* in, int64_t in_n, int64_t in_c, int64_t in_h, int64_t in_w, int64_t* col);

/* The same column matrix with image n's row r at col + n*col_n + r*col_c (unit stride along a row; col_c and col_n at
 * least H_out*W_out). col_n = H_out*W_out, col_c = N*H_out*W_out folds the batch into the columns
 * ([C*kH*kW][N*H_out*W_out]): the layout in which the backward pass of the convolution is two plain products.
 * Replaces im2col (src/arraymancer/nn_primitives/fallback/conv.nim:18-54) inside the per-image loop of
 * im2colgemm_conv2d_gradient (fallback/conv.nim:134-145). */
int am_hip_im2col_strided_f32(int64_t N, int C, int H, int W, int kH, int kW, int padH, int padW, int strideH, int strideW,
                              const float* in, int64_t in_n, int64_t in_c, int64_t in_h, int64_t in_w,
                              float* col, int64_t col_n, int64_t col_c);
int am_hip_im2col_strided_f64(int64_t N, int C, int H, int W, int kH, int kW, int padH, int padW, int strideH, int strideW,
                              const double* in, int64_t in_n, int64_t in_c, int64_t in_h, int64_t in_w,
                              double* col, int64_t col_n, int64_t col_c);
int am_hip_im2col_strided_i32(int64_t N, int C, int H, int W, int kH, int kW, int padH, int padW, int strideH, int strideW,
                              const int32_t* in, int64_t in_n, int64_t in_c, int64_t in_h, int64_t in_w,
                              int32_t* col, int64_t col_n, int64_t col_c);
int am_hip_im2col_strided_i64(int64_t N, int C, int H, int W, int kH, int kW, int padH, int padW, int strideH, int strideW,
                              const int64_t* in, int64_t in_n, int64_t in_c, int64_t in_h, int64_t in_w,
                              int64_t* col, int64_t col_n, int64_t col_c);

/* out[n][c][y][x] <- sum over (kh, kw), in increasing order, of the entry of row c*kH*kW + kh*kW + kw of image n's
 * column matrix that covers pixel (y, x), if any: the reverse of im2col, overlapping patches summed (integers wrap).
 * `col` is addressed like am_hip_im2col_strided_*'s, `out` through its four NCHW strides (elements); every pixel of
 * `out` is written. Replaces col2im (src/arraymancer/nn_primitives/fallback/conv.nim:55-79), whose scatter loop
 * adds the same entries to a pixel in the same order. */
int am_hip_col2im_f32(int64_t N, int C, int H, int W, int kH, int kW, int padH, int padW, int strideH, int strideW,
                      const float* col, int64_t col_n, int64_t col_c,
                      float* out, int64_t out_n, int64_t out_c, int64_t out_h, int64_t out_w);
int am_hip_col2im_f64(int64_t N, int C, int H, int W, int kH, int kW, int padH, int padW, int strideH, int strideW,
                      const double* col, int64_t col_n, int64_t col_c,
                      double* out, int64_t out_n, int64_t out_c, int64_t out_h, int64_t out_w);
int am_hip_col2im_i32(int64_t N, int C, int H, int W, int kH, int kW, int padH, int padW, int strideH, int strideW,
                      const int32_t* col, int64_t col_n, int64_t col_c,
                      int32_t* out, int64_t out_n, int64_t out_c, int64_t out_h, int64_t out_w);
int am_hip_col2im_i64(int64_t N, int C, int H, int W, int kH, int kW, int padH, int padW, int strideH, int strideW,
                      const int64_t* col, int64_t col_n, int64_t col_c,
                      int64_t* out, int64_t out_n, int64_t out_c, int64_t out_h, int64_t out_w);

/* out[n][co][h*W_out + w] <- sum over (c, kh, kw) of kernel[co][c*kH*kW + kh*kW + kw] * (padded input patch element)
 * (+ bias[co]) (then ReLU), for the whole batch in ONE launch: the column matrix of im2col is never written, the
 * GEMM's B loader gathers it from the images. `in` is addressed through its four NCHW strides (elements); `kernel` is
 * the [C_out, C*kH*kW] matrix of a [C_out, C, kH, kW] tensor, rows `kernel_rs` apart, unit stride within a row;
 * `bias` (epilogue AM_EPI_BIAS / AM_EPI_BIAS_RELU) has C_out elements `bias_s` apart; `out` is a contiguous
 * [N, C_out, H_out, W_out] tensor. Float types; N <= 65535; C*kH*kW must hold one 16-byte vector at least
 * (AM_E_SHAPE otherwise: run am_hip_im2col_* + am_hip_gemm_batched_* then).
 * Replaces im2colgemm_conv2d (src/arraymancer/nn_primitives/fallback/conv.nim:81-106: per image im2col, gemm,
 * then the bias broadcast added) followed by relu (nnp_activation.nim:35-36) where asked for. */
int am_hip_conv2d_f32(int64_t N, int C, int H, int W, int Cout, int kH, int kW, int padH, int padW, int strideH, int strideW,
                      const float* in, int64_t in_n, int64_t in_c, int64_t in_h, int64_t in_w,
                      const float* kernel, int64_t kernel_rs, int epilogue, const float* bias, int64_t bias_s, float* out);
int am_hip_conv2d_f64(int64_t N, int C, int H, int W, int Cout, int kH, int kW, int padH, int padW, int strideH, int strideW,
                      const double* in, int64_t in_n, int64_t in_c, int64_t in_h, int64_t in_w,
                      const double* kernel, int64_t kernel_rs, int epilogue, const double* bias, int64_t bias_s, double* out);

/* grad_weight[co][c*kH*kW + kh*kW + kw] <- sum over the images n and their output pixels (oh, ow) of
 * grad_output[co][n*P + oh*W_out + ow] * (padded input patch element of image n), P = H_out * W_out: the weight
 * gradient of the whole batch as ONE product with k = N * P whose second operand, the transposed column matrices of
 * the images side by side, is never written: the GEMM's B loader gathers it from the images in 16-byte pieces.
 * `in` is addressed through its four NCHW strides (elements); `grad_output` is the [C_out][N * P] matrix (grad_output
 * with its first two axes swapped), rows `gout_rs` apart, unit stride within a row; `out` is a contiguous
 * [C_out, C, kH, kW] tensor, overwritten (left as it is when N = 0). Float types. Takes: unit stride of the window
 * and of the image along the width, W_out a multiple of the elements in 16 bytes, W at least that many, N * P < 2^31
 * (AM_E_SHAPE otherwise: run am_hip_im2col_strided_* + am_hip_gemm_* then). The sum over k is split over workgroups
 * and folded in a fixed order: results do not change from run to run.
 * Replaces the weight-gradient half of im2colgemm_conv2d_gradient
 * (src/arraymancer/nn_primitives/fallback/conv.nim:135-143: per image im2col, then gemm_nt accumulated into grad_weight). */
int am_hip_conv2d_grad_weight_f32(int64_t N, int C, int H, int W, int Cout, int kH, int kW, int padH, int padW, int strideH,
                                  int strideW, const float* in, int64_t in_n, int64_t in_c, int64_t in_h, int64_t in_w,
                                  const float* grad_output, int64_t gout_rs, float* out);
int am_hip_conv2d_grad_weight_f64(int64_t N, int C, int H, int W, int Cout, int kH, int kW, int padH, int padW, int strideH,
                                  int strideW, const double* in, int64_t in_n, int64_t in_c, int64_t in_h, int64_t in_w,
                                  const double* grad_output, int64_t gout_rs, double* out);

/* ---------------------------------------------------------------- GEMV and dot
 * y[M] <- alpha * A[M x N] * x[N] + beta * y, any strides (elements).
 * Replaces gemv (src/arraymancer/tensor/operators_blas_l2l3.nim:24-56; integer fallback
 * fallback/naive_l2_gemv.nim:24-57; CUDA: operators_blas_l2l3_cuda.nim:20-41, which requires a
 * contiguous A). N == 0 leaves y untouched, like K == 0 in GEMM. Integers wrap. */
int am_hip_gemv_f32(int64_t M, int64_t N, float alpha, const float* A, int64_t rsA, int64_t csA,
                    const float* x, int64_t incx, float beta, float* y, int64_t incy);
int am_hip_gemv_f64(int64_t M, int64_t N, double alpha, const double* A, int64_t rsA, int64_t csA,
                    const double* x, int64_t incx, double beta, double* y, int64_t incy);
int am_hip_gemv_i32(int64_t M, int64_t N, int32_t alpha, const int32_t* A, int64_t rsA, int64_t csA,
                    const int32_t* x, int64_t incx, int32_t beta, int32_t* y, int64_t incy);
int am_hip_gemv_i64(int64_t M, int64_t N, int64_t alpha, const int64_t* A, int64_t rsA, int64_t csA,
                    const int64_t* x, int64_t incx, int64_t beta, int64_t* y, int64_t incy);
/* *result (HOST pointer) <- sum_i x[i * incx] * y[i * incy]; blocking.
 * Replaces dot (src/arraymancer/tensor/operators_blas_l1.nim:27-38; CUDA: operators_blas_l1_cuda.nim:28-34). */
int am_hip_dot_f32(int64_t n, const float* x, int64_t incx, const float* y, int64_t incy, float* result);
int am_hip_dot_f64(int64_t n, const double* x, int64_t incx, const double* y, int64_t incy, double* result);
int am_hip_dot_i32(int64_t n, const int32_t* x, int64_t incx, const int32_t* y, int64_t incy, int32_t* result);
int am_hip_dot_i64(int64_t n, const int64_t* x, int64_t incx, const int64_t* y, int64_t incy, int64_t* result);

/* ---------------------------------------------------------------- element-wise / broadcast / map
 * dst[i] = op(a[i], b[i]) over a common `shape` of `rank` dims (0 <= rank <= 6); each operand
 * is traversed in C order through its own strides (elements; 0 = broadcast, negative allowed
 * for inputs). `shape` and the stride arrays are HOST arrays of `rank` entries, passed to the
 * kernel by value (the CUDA backend cudaMallocs them on every call:
 * src/arraymancer/tensor/backend/cuda.nim:102-132).
 *
 * One entry point covers both reference families:
 *   map2_inline  (src/arraymancer/tensor/higher_order_applymap.nim:92-120): dst = fresh
 *                contiguous tensor; behind `+` `-` (operators_blas_l1.nim:44-51) and
 *                `+.` `-.` `*.` `/.` `mod` (operators_broadcasted.nim:28-60) after
 *                broadcast2 (private/p_shapeshifting.nim:96-134);
 *   apply2_inline (higher_order_applymap.nim:40-47): dst == a with a's own strides; behind
 *                `+=` `-=` (operators_blas_l1.nim:53-61) and `+.=` `-.=` `*.=` `/.=`
 *                (operators_broadcasted.nim:65-102).
 * GPU precedent: cuda_apply3 / cuda_apply2
 *   (src/arraymancer/tensor/private/incl_higher_order_cuda.nim:31-119).
 * dst may alias a or b exactly (same pointer, same strides); any other overlap is undefined.
 * dst must not have a zero stride on a dimension of extent > 1.
 */
#define AM_OP_ADD         0
#define AM_OP_SUB         1
#define AM_OP_MUL         2
#define AM_OP_DIV         3   /* floats: IEEE /; integers: truncating `div`; x div 0 -> 0 on device */
#define AM_OP_MOD         4   /* integers: C `%` (sign of dividend), x mod 0 -> 0 on device; floats: C fmod */
#define AM_OP_ADD_RELU    5   /* t = a + b; (0 >= t) ? 0 : t        (fused bias + ReLU)              */
#define AM_OP_ADD_SIGMOID 6   /* floats: 1 / (1 + exp(-(a + b)))    (GRU gates, nnp_gru.nim:78)      */
#define AM_OP_ADD_TANH    7   /* floats: tanh(a + b)                                                */
#define AM_OP_RELU_BWD    8   /* (a <= 0) ? 0 : b                   (nnp_activation.nim:65-70)       */
#define AM_OP_MAX         9
#define AM_OP_MIN        10
#define AM_OP_SIGMOID_BWD 11  /* a * (1 - a) * b   a = cached sigmoid output (nnp_activation.nim:61-63)  */
#define AM_OP_TANH_BWD   12   /* b * (1 - a * a)   a = cached tanh output    (nnp_activation.nim:72-74)  */
#define AM_OP_SQDIFF     13   /* (a - b) * (a - b): the fold body of variance (tensor/aggregate.nim:115-146) */
#define AM_OP_POW        14   /* floats only: pow(a, b); `^.` and `^.=` (operators_broadcasted.nim:153-161, 178-182) */
#define AM_OP_FLOORMOD   15   /* Nim's floorMod: r = a mod b, plus b when r and b have opposite signs
                                 (tensor/math_functions.nim:134-144; std/math floorMod). Integers: b == 0 -> 0 */
#define AM_OP_COPYSIGN   16   /* floats only: magnitude of a, sign of b (copySign / mcopySign, math_functions.nim:119-132) */
#define AM_OP_BINARY_COUNT 17

int am_hip_ew_binary_f32(int op, int rank, const int64_t* shape,
                         float* dst, const int64_t* dst_strides,
                         const float* a, const int64_t* a_strides,
                         const float* b, const int64_t* b_strides);
int am_hip_ew_binary_f64(int op, int rank, const int64_t* shape,
                         double* dst, const int64_t* dst_strides,
                         const double* a, const int64_t* a_strides,
                         const double* b, const int64_t* b_strides);
int am_hip_ew_binary_i32(int op, int rank, const int64_t* shape,
                         int32_t* dst, const int64_t* dst_strides,
                         const int32_t* a, const int64_t* a_strides,
                         const int32_t* b, const int64_t* b_strides);
int am_hip_ew_binary_i64(int op, int rank, const int64_t* shape,
                         int64_t* dst, const int64_t* dst_strides,
                         const int64_t* a, const int64_t* a_strides,
                         const int64_t* b, const int64_t* b_strides);

/* dst[i] = scalar_on_left ? op(scalar, a[i]) : op(a[i], scalar); ops AM_OP_ADD..AM_OP_MOD,
 * AM_OP_MAX, AM_OP_MIN, AM_OP_POW (`t ^. exponent`, `base ^. t`). Replaces the tensor-scalar forms
 *   src/arraymancer/tensor/operators_broadcasted.nim:107-194, operators_blas_l1.nim:66-136
 * (GPU precedent: cuda_apply_rscal / _lscal / _scal, incl_higher_order_cuda.nim:121-229).
 * dst may alias a exactly (the in-place `+.=`, `*=` ... forms). */
int am_hip_ew_scalar_f32(int op, int scalar_on_left, int rank, const int64_t* shape,
                         float* dst, const int64_t* dst_strides,
                         const float* a, const int64_t* a_strides, float scalar);
int am_hip_ew_scalar_f64(int op, int scalar_on_left, int rank, const int64_t* shape,
                         double* dst, const int64_t* dst_strides,
                         const double* a, const int64_t* a_strides, double scalar);
int am_hip_ew_scalar_i32(int op, int scalar_on_left, int rank, const int64_t* shape,
                         int32_t* dst, const int64_t* dst_strides,
                         const int32_t* a, const int64_t* a_strides, int32_t scalar);
int am_hip_ew_scalar_i64(int op, int scalar_on_left, int rank, const int64_t* shape,
                         int64_t* dst, const int64_t* dst_strides,
                         const int64_t* a, const int64_t* a_strides, int64_t scalar);

/* dst[i] = op(a[i]). AM_UOP_COPY is the strided gather behind `clone` / `asContiguous`
 * (src/arraymancer/tensor/shapeshifting.nim:38-57; CUDA: shapeshifting_cuda.nim:34-66).
 * map_inline / apply_inline: src/arraymancer/tensor/higher_order_applymap.nim:27-32,69-90;
 * relu: nn_primitives/nnp_activation.nim:35-36; sigmoid: nn_primitives/private/p_activation.nim:17-18. */
#define AM_UOP_COPY    0
#define AM_UOP_NEG     1
#define AM_UOP_RELU    2   /* (0 >= x) ? 0 : x */
#define AM_UOP_SIGMOID 3   /* floats only      */
#define AM_UOP_TANH    4   /* floats only      */
#define AM_UOP_EXP     5   /* floats only      */
#define AM_UOP_ABS     6
#define AM_UOP_SQRT    7   /* floats only: IEEE square root (tensor/ufunc.nim:91)        */
#define AM_UOP_SQUARE  8   /* x * x (tensor/math_functions.nim:218-222); integers wrap   */
/* The universal functions of tensor/ufunc.nim:82-130 (map_inline of the C math library's
 * function of the same name) and `reciprocal` (tensor/math_functions.nim:52-58). Floats only.
 * The device math library evaluates the transcendental ones: a few units in the last place from
 * the host's libm, not the same bits. floor / ceil / trunc / round (half away from zero) and
 * reciprocal (one IEEE division) are exact. */
#define AM_UOP_LN          9
#define AM_UOP_LOG10      10
#define AM_UOP_LOG2       11
#define AM_UOP_SIN        12
#define AM_UOP_COS        13
#define AM_UOP_TAN        14
#define AM_UOP_SINH       15
#define AM_UOP_COSH       16
#define AM_UOP_ARCSIN     17
#define AM_UOP_ARCCOS     18
#define AM_UOP_ARCTAN     19
#define AM_UOP_ARCSINH    20
#define AM_UOP_ARCCOSH    21
#define AM_UOP_ARCTANH    22
#define AM_UOP_CBRT       23
#define AM_UOP_ERF        24
#define AM_UOP_ERFC       25
#define AM_UOP_GAMMA      26   /* the gamma function itself (C tgamma) */
#define AM_UOP_LGAMMA     27
#define AM_UOP_FLOOR      28
#define AM_UOP_CEIL       29
#define AM_UOP_TRUNC      30
#define AM_UOP_ROUND      31   /* halfway cases away from zero (C round) */
#define AM_UOP_RECIPROCAL 32   /* 1 / x */
#define AM_UOP_DEGTORAD   33   /* x * (PI / 180), the constant rounded to the element type (Nim's degToRad, ufunc.nim:129) */
#define AM_UOP_RADTODEG   34   /* x / (PI / 180)                                           (Nim's radToDeg, ufunc.nim:130) */
#define AM_UOP_FAC        35   /* integers only: n! for 0 <= n <= 20 (Nim's fac, mapped by tensor/ufunc.nim:84-85), wrapped into the
                                   element type; 0 outside that range (Nim raises there: the host layers check first) */
#define AM_UOP_COUNT      36
int am_hip_ew_unary_f32(int op, int rank, const int64_t* shape,
                        float* dst, const int64_t* dst_strides,
                        const float* a, const int64_t* a_strides);
int am_hip_ew_unary_f64(int op, int rank, const int64_t* shape,
                        double* dst, const int64_t* dst_strides,
                        const double* a, const int64_t* a_strides);
int am_hip_ew_unary_i32(int op, int rank, const int64_t* shape,
                        int32_t* dst, const int64_t* dst_strides,
                        const int32_t* a, const int64_t* a_strides);
int am_hip_ew_unary_i64(int op, int rank, const int64_t* shape,
                        int64_t* dst, const int64_t* dst_strides,
                        const int64_t* a, const int64_t* a_strides);

/* Map bodies whose result type differs from the operands': the reference's map templates infer the
 * type of the result (src/arraymancer/tensor/higher_order_applymap.nim:69-120, its own fixture:
 * tests/tensor/test_higherorder.nim:103-112, `x mod y == 0` -> Tensor[bool]).
 *
 * dst[i] (one byte per element, 0 or 1: Nim's bool) = a[i] cmp b[i]. Replaces the broadcast comparison
 * family `==.` `!=.` `<.` `<=.` `>.` `>=.` (src/arraymancer/tensor/operators_comparison.nim:41-94:
 * broadcast2 then map2_inline) and, in the scalar form, :111-146 (map_inline of `x cmp value`; the
 * reversed forms `value cmp t` are the mirrored comparison of `t`, :150-185). Same traversal, strides
 * and dimension collapsing as am_hip_ew_binary_*; dst strides count bytes = elements. Floats compare
 * like IEEE (every comparison with a NaN is false except `!=`). */
#define AM_CMP_EQ 0
#define AM_CMP_NE 1
#define AM_CMP_LT 2
#define AM_CMP_LE 3
#define AM_CMP_GT 4
#define AM_CMP_GE 5
#define AM_CMP_MOD_IS_ZERO 6   /* (a mod b) == 0 with AM_OP_MOD's `mod` */
#define AM_CMP_COUNT 7
int am_hip_ew_compare_f32(int op, int rank, const int64_t* shape, uint8_t* dst, const int64_t* dst_strides,
                          const float* a, const int64_t* a_strides, const float* b, const int64_t* b_strides);
int am_hip_ew_compare_f64(int op, int rank, const int64_t* shape, uint8_t* dst, const int64_t* dst_strides,
                          const double* a, const int64_t* a_strides, const double* b, const int64_t* b_strides);
int am_hip_ew_compare_i32(int op, int rank, const int64_t* shape, uint8_t* dst, const int64_t* dst_strides,
                          const int32_t* a, const int64_t* a_strides, const int32_t* b, const int64_t* b_strides);
int am_hip_ew_compare_i64(int op, int rank, const int64_t* shape, uint8_t* dst, const int64_t* dst_strides,
                          const int64_t* a, const int64_t* a_strides, const int64_t* b, const int64_t* b_strides);
int am_hip_ew_compare_scalar_f32(int op, int rank, const int64_t* shape, uint8_t* dst, const int64_t* dst_strides,
                                 const float* a, const int64_t* a_strides, float scalar);
int am_hip_ew_compare_scalar_f64(int op, int rank, const int64_t* shape, uint8_t* dst, const int64_t* dst_strides,
                                 const double* a, const int64_t* a_strides, double scalar);
int am_hip_ew_compare_scalar_i32(int op, int rank, const int64_t* shape, uint8_t* dst, const int64_t* dst_strides,
                                 const int32_t* a, const int64_t* a_strides, int32_t scalar);
int am_hip_ew_compare_scalar_i64(int op, int rank, const int64_t* shape, uint8_t* dst, const int64_t* dst_strides,
                                 const int64_t* a, const int64_t* a_strides, int64_t scalar);

/* dst[i] (one byte) = predicate(a[i]) for float tensors: isNaN (x != x) and isNotNaN (x == x),
 * src/arraymancer/tensor/operators_comparison.nim:192-206; classify, src/arraymancer/tensor/
 * math_functions.nim:264-276, as the ordinal of Nim's FloatClass: 0 fcNormal, 1 fcSubnormal, 2 fcZero,
 * 3 fcNegZero, 4 fcNan, 5 fcInf, 6 fcNegInf. */
#define AM_PRED_ISNAN    0
#define AM_PRED_ISNOTNAN 1
#define AM_PRED_CLASSIFY 2
#define AM_PRED_SGN      3   /* only through am_hip_ew_sgn_*: its destination is int64 */
int am_hip_ew_predicate_f32(int op, int rank, const int64_t* shape, uint8_t* dst, const int64_t* dst_strides,
                            const float* a, const int64_t* a_strides);
int am_hip_ew_predicate_f64(int op, int rank, const int64_t* shape, uint8_t* dst, const int64_t* dst_strides,
                            const double* a, const int64_t* a_strides);
/* dst[i] (int64: the reference's Tensor[int]) = -1, 0 or 1, the sign of a[i]; zeros of either sign and
 * NaN give 0 (sgn, src/arraymancer/tensor/math_functions.nim:110-117). */
int am_hip_ew_sgn_f32(int rank, const int64_t* shape, int64_t* dst, const int64_t* dst_strides, const float* a, const int64_t* a_strides);
int am_hip_ew_sgn_f64(int rank, const int64_t* shape, int64_t* dst, const int64_t* dst_strides, const double* a, const int64_t* a_strides);
int am_hip_ew_sgn_i32(int rank, const int64_t* shape, int64_t* dst, const int64_t* dst_strides, const int32_t* a, const int64_t* a_strides);
int am_hip_ew_sgn_i64(int rank, const int64_t* shape, int64_t* dst, const int64_t* dst_strides, const int64_t* a, const int64_t* a_strides);

/* dst[i] = op(a[i], b[i], c[i]): map3_inline / apply3_inline
 * (src/arraymancer/tensor/higher_order_applymap.nim:58-67, 122-150) with the enumerated bodies the
 * reference itself uses on this path (GRU gates over column slices of [batch, 3H] buffers,
 * src/arraymancer/nn_primitives/nnp_gru.nim:80-88). Every arithmetic step is rounded on its own.
 * dst may alias any operand exactly. Float tensors: all ops; integer tensors: AM_OP3_MULADD and AM_OP3_ADDMUL (wrapping), AM_OP3_CLAMP. */
#define AM_OP3_MULADD        0   /* x * y + z                                                  */
#define AM_OP3_GRU_CANDIDATE 1   /* tanh(x + y * z)              apply3_inline(n, r, Uh)       */
#define AM_OP3_GRU_BLEND     2   /* (1 - y) * z + y * x          apply3_inline(hidden, z, n)   */
#define AM_OP3_ADDMUL        3   /* (x + y) * z: `(X +. b) *. s` in one pass, each step rounded   */
#define AM_OP3_CLAMP         4   /* (x < y) ? y : (x > z) ? z : x: clamp(x, min, max), any element type
                                    (tensor/math_functions.nim:146-152); min and max as one-element operands
                                    with all strides 0 */
#define AM_OP3_COUNT         5
int am_hip_ew_ternary_f32(int op, int rank, const int64_t* shape, float* dst, const int64_t* dst_strides,
                          const float* a, const int64_t* a_strides, const float* b, const int64_t* b_strides,
                          const float* c, const int64_t* c_strides);
int am_hip_ew_ternary_f64(int op, int rank, const int64_t* shape, double* dst, const int64_t* dst_strides,
                          const double* a, const int64_t* a_strides, const double* b, const int64_t* b_strides,
                          const double* c, const int64_t* c_strides);
int am_hip_ew_ternary_i32(int op, int rank, const int64_t* shape, int32_t* dst, const int64_t* dst_strides,
                          const int32_t* a, const int64_t* a_strides, const int32_t* b, const int64_t* b_strides,
                          const int32_t* c, const int64_t* c_strides);
int am_hip_ew_ternary_i64(int op, int rank, const int64_t* shape, int64_t* dst, const int64_t* dst_strides,
                          const int64_t* a, const int64_t* a_strides, const int64_t* b, const int64_t* b_strides,
                          const int64_t* c, const int64_t* c_strides);

/* dst[i] = (a[i] < lo) ? lo : (a[i] > hi) ? hi : a[i] with both bounds passed by value: clamp / mclamp
 * (src/arraymancer/tensor/math_functions.nim:146-152, map_inline / apply_inline of Nim's clamp). One
 * pass, no device memory for the bounds, no copy, so it can be recorded into a graph like every other
 * element-wise call. dst may alias a exactly. A NaN element stays NaN. */
int am_hip_ew_clamp_f32(int rank, const int64_t* shape, float* dst, const int64_t* dst_strides,
                        const float* a, const int64_t* a_strides, float lo, float hi);
int am_hip_ew_clamp_f64(int rank, const int64_t* shape, double* dst, const int64_t* dst_strides,
                        const double* a, const int64_t* a_strides, double lo, double hi);
int am_hip_ew_clamp_i32(int rank, const int64_t* shape, int32_t* dst, const int64_t* dst_strides,
                        const int32_t* a, const int64_t* a_strides, int32_t lo, int32_t hi);
int am_hip_ew_clamp_i64(int rank, const int64_t* shape, int64_t* dst, const int64_t* dst_strides,
                        const int64_t* a, const int64_t* a_strides, int64_t lo, int64_t hi);

/* ---------------------------------------------------------------- reductions, softmax, pooling
 * dst <- fold of `a` along `axis` with op (AM_RED_*). `shape` / `a_strides` describe `a` (rank
 * 1..AM_MAXRANK, element strides, any sign); dst has the same rank with extent 1 along `axis`
 * (dst_strides[axis] is ignored), exactly what reduce_axis_inline returns
 * (src/arraymancer/tensor/higher_order_foldreduce.nim:46-61; sum/product/min/max(axis),
 * src/arraymancer/tensor/aggregate.nim:38-113). The fold starts from the first slice and takes the
 * following ones in order. Integer sums/products wrap; min/max are Nim's (`if x <= y: x else: y`).
 * An empty tensor returns AM_OK without touching dst (returnEmptyIfEmpty); axis outside the rank:
 * AM_E_SHAPE (the reference's IndexDefect). Float sums along a unit-stride axis are reassociated
 * (tree over a wavefront, chunked for very long axes): equal to a serial fold up to rounding. */
#define AM_RED_SUM  0
#define AM_RED_PROD 1
#define AM_RED_MIN  2
#define AM_RED_MAX  3
int am_hip_reduce_axis_f32(int op, int rank, const int64_t* shape, int axis, float* dst, const int64_t* dst_strides,
                           const float* a, const int64_t* a_strides);
int am_hip_reduce_axis_f64(int op, int rank, const int64_t* shape, int axis, double* dst, const int64_t* dst_strides,
                           const double* a, const int64_t* a_strides);
int am_hip_reduce_axis_i32(int op, int rank, const int64_t* shape, int axis, int32_t* dst, const int64_t* dst_strides,
                           const int32_t* a, const int64_t* a_strides);
int am_hip_reduce_axis_i64(int op, int rank, const int64_t* shape, int axis, int64_t* dst, const int64_t* dst_strides,
                           const int64_t* a, const int64_t* a_strides);

/* idx, val <- position along `axis` and value of the first maximum (op = AM_RED_MAX) or minimum
 * (AM_RED_MIN) of `a` along that axis; both outputs have a's rank with extent 1 along `axis`
 * (their strides along it are ignored); idx is the reference's Tensor[int] (int64). Replaces
 * argmax_max / argmin_min (src/arraymancer/tensor/aggregate.nim:159-193, 216-250; argmax / argmin
 * :195-214, 252-271 keep the indices only): the walk starts from slice 0 and moves on a strict
 * `>` / `<` only, so ties keep the lowest position, a NaN in slice 0 stays and a NaN elsewhere
 * is never taken. An empty tensor returns AM_OK without touching the outputs. */
int am_hip_argreduce_f32(int op, int rank, const int64_t* shape, int axis, int64_t* idx, const int64_t* idx_strides,
                         float* val, const int64_t* val_strides, const float* a, const int64_t* a_strides);
int am_hip_argreduce_f64(int op, int rank, const int64_t* shape, int axis, int64_t* idx, const int64_t* idx_strides,
                         double* val, const int64_t* val_strides, const double* a, const int64_t* a_strides);
int am_hip_argreduce_i32(int op, int rank, const int64_t* shape, int axis, int64_t* idx, const int64_t* idx_strides,
                         int32_t* val, const int64_t* val_strides, const int32_t* a, const int64_t* a_strides);
int am_hip_argreduce_i64(int op, int rank, const int64_t* shape, int axis, int64_t* idx, const int64_t* idx_strides,
                         int64_t* val, const int64_t* val_strides, const int64_t* a, const int64_t* a_strides);

/* *result (HOST pointer) <- fold of every element of `a` (rank 0..AM_MAXRANK); blocks until the
 * value has arrived; not allowed during graph capture. Replaces reduce_inline and sum / product /
 * min / max without axis (higher_order_foldreduce.nim:22-31, aggregate.nim:33-36,46-49,89-106).
 * An empty tensor has no first element to start from: AM_E_SHAPE. */
int am_hip_reduce_all_f32(int op, int rank, const int64_t* shape, const float* a, const int64_t* a_strides, float* result);
int am_hip_reduce_all_f64(int op, int rank, const int64_t* shape, const double* a, const int64_t* a_strides, double* result);
int am_hip_reduce_all_i32(int op, int rank, const int64_t* shape, const int32_t* a, const int64_t* a_strides, int32_t* result);
int am_hip_reduce_all_i64(int op, int rank, const int64_t* shape, const int64_t* a, const int64_t* a_strides, int64_t* result);

/* dst[i, j] <- exp(src[i, j] - max_i) / sum_j exp(src[i, j] - max_i) for a [rows, cols] matrix
 * with element strides (rs, cs) on both sides; dst may be src. Replaces softmax
 * (src/arraymancer/nn_primitives/nnp_softmax.nim:18-38: streaming_max_sumexp + stable_softmax,
 * private/p_logsumexp.nim:30-62); the row sum is accumulated in a different order than the
 * reference's streaming pass, the result agrees to rounding. */
int am_hip_softmax_rows_f32(int64_t rows, int64_t cols, float* dst, int64_t dst_rs, int64_t dst_cs,
                            const float* src, int64_t src_rs, int64_t src_cs);
int am_hip_softmax_rows_f64(int64_t rows, int64_t cols, double* dst, int64_t dst_rs, int64_t dst_cs,
                            const double* src, int64_t src_rs, int64_t src_cs);

/* The gate arithmetic of a GRU cell in one pass over the two [batch, 3H] products w3x = W3 x + bW3 and u3h = U3 h + bU3
 * (rows ldw resp. ldu apart, unit stride within a row; columns [0, H) reset, [H, 2H) update, [2H, 3H) candidate):
 *   r = sigmoid(w3x_r + u3h_r), z = sigmoid(w3x_z + u3h_z), n = tanh(w3x_n + r * u3h_n), hidden <- (1 - z) * n + z * hidden
 * with `hidden` [batch, H] (rows ldh apart) updated in place. When r, z, n and uh are not NULL (all four or none; [batch, H]
 * each, rows lds apart) they receive r, z, n and u3h_n for the backward pass. Replaces steps 2-4 of gru_cell_inference and
 * gru_cell_forward (src/arraymancer/nn_primitives/nnp_gru.nim:72-88, 125-146: three apply2 / apply3 passes over column
 * slices); same expressions, each step rounded on its own. */
int am_hip_gru_gates_f32(int64_t batch, int64_t H, const float* w3x, int64_t ldw, const float* u3h, int64_t ldu,
                         float* hidden, int64_t ldh, float* r, float* z, float* n, float* uh, int64_t lds);
int am_hip_gru_gates_f64(int64_t batch, int64_t H, const double* w3x, int64_t ldw, const double* u3h, int64_t ldu,
                         double* hidden, int64_t ldh, double* r, double* z, double* n, double* uh, int64_t lds);

/* The element-wise part of the cell's backward pass in one launch: from dnext (the gradient of the next hidden state), h
 * (the hidden state BEFORE the step) and r, z, n, uh as kept by am_hip_gru_gates_* (all [batch, H], rows ld_in apart), the
 * gradients of the two products, dw3x = [dWrx | dWzx | dWx] and du3h = [dWrx | dWzx | dUh] ([batch, 3H], rows ldw resp. ldu
 * apart). Replaces the `-.` / `*.` / tanh_backward / sigmoid_backward passes and the two `concat`s of gru_cell_backward
 * (src/arraymancer/nn_primitives/nnp_gru.nim:165-186); the two linear_backward calls and the final dh + dnext * z stay
 * with the caller. */
int am_hip_gru_gates_backward_f32(int64_t batch, int64_t H, const float* dnext, const float* h, const float* r, const float* z,
                                  const float* n, const float* uh, int64_t ld_in, float* dw3x, int64_t ldw, float* du3h, int64_t ldu);
int am_hip_gru_gates_backward_f64(int64_t batch, int64_t H, const double* dnext, const double* h, const double* r, const double* z,
                                  const double* n, const double* uh, int64_t ld_in, double* dw3x, int64_t ldw, double* du3h, int64_t ldu);

/* values[t][i] <- values[t][i] - learning_rate * grads[t][i] for `count` contiguous tensors of sizes[t] elements in ONE
 * launch (64 tensors per launch beyond that). Replaces the SGD optimizer's update, one apply2_inline per parameter
 * (src/arraymancer/nn/optimizers/optimizers.nim:35-51); same expression, the product rounded before the subtraction. */
int am_hip_sgd_update_f32(int count, float* const* values, const float* const* grads, const int64_t* sizes, float learning_rate);
int am_hip_sgd_update_f64(int count, double* const* values, const double* const* grads, const int64_t* sizes, double learning_rate);

/* *loss (host) <- (1 / rows) * sum over the rows i of  ln(sum_j exp(input[i, j])) - sum_j input[i, j] * target[i, j]:
 * softmax and cross-entropy in one pass over `input` [rows, cols] and `target` [rows, cols] (probabilities), element
 * strides (rs, cs). Blocking; 0 for an empty batch. Replaces softmax_cross_entropy
 * (src/arraymancer/nn_primitives/nnp_softmax_cross_entropy.nim:17-86); the rows' losses are added in a fixed order
 * (the reference adds them with an atomic under OpenMP), the result agrees to rounding. */
int am_hip_softmax_cross_entropy_f32(int64_t rows, int64_t cols, const float* input, int64_t in_rs, int64_t in_cs,
                                     const float* target, int64_t t_rs, int64_t t_cs, float* loss);
int am_hip_softmax_cross_entropy_f64(int64_t rows, int64_t cols, const double* input, int64_t in_rs, int64_t in_cs,
                                     const double* target, int64_t t_rs, int64_t t_cs, double* loss);
/* The same with one class index per row instead of probabilities: labels[i * labels_s] in [0, cols); the row's term is
 * ln(sum_j exp(input[i, j])) - input[i, label]. A label outside [0, cols) makes the loss NaN (the reference reads out
 * of bounds or raises an IndexDefect). Replaces sparse_softmax_cross_entropy (nnp_softmax_cross_entropy.nim:88-177). */
int am_hip_sparse_softmax_cross_entropy_f32(int64_t rows, int64_t cols, const float* input, int64_t in_rs, int64_t in_cs,
                                            const int64_t* labels, int64_t labels_s, float* loss);
int am_hip_sparse_softmax_cross_entropy_f64(int64_t rows, int64_t cols, const double* input, int64_t in_rs, int64_t in_cs,
                                            const int64_t* labels, int64_t labels_s, double* loss);
/* result[i, j] <- gradient * (softmax(input[i, :])[j] - target[i, j]) / rows: the gradient of the loss above with respect
 * to `input`, one launch. Replaces softmax_cross_entropy_backward (nnp_softmax_cross_entropy.nim:186-214) with a scalar
 * gradient (a one-element gradient tensor is read by the host layer). */
int am_hip_softmax_cross_entropy_backward_f32(int64_t rows, int64_t cols, float gradient, const float* input, int64_t in_rs,
                                              int64_t in_cs, const float* target, int64_t t_rs, int64_t t_cs,
                                              float* result, int64_t r_rs, int64_t r_cs);
int am_hip_softmax_cross_entropy_backward_f64(int64_t rows, int64_t cols, double gradient, const double* input, int64_t in_rs,
                                              int64_t in_cs, const double* target, int64_t t_rs, int64_t t_cs,
                                              double* result, int64_t r_rs, int64_t r_cs);
/* result[i, j] <- gradient * (softmax(input[i, :])[j] - (j == labels[i] ? 1 : 0)) / rows. A label outside [0, cols)
 * makes its row of the result NaN (the forward pass makes the loss NaN for the same input). Replaces sparse_softmax_cross_entropy_backward
 * (nnp_softmax_cross_entropy.nim:217-256). */
int am_hip_sparse_softmax_cross_entropy_backward_f32(int64_t rows, int64_t cols, float gradient, const float* input,
                                                     int64_t in_rs, int64_t in_cs, const int64_t* labels, int64_t labels_s,
                                                     float* result, int64_t r_rs, int64_t r_cs);
int am_hip_sparse_softmax_cross_entropy_backward_f64(int64_t rows, int64_t cols, double gradient, const double* input,
                                                     int64_t in_rs, int64_t in_cs, const int64_t* labels, int64_t labels_s,
                                                     double* result, int64_t r_rs, int64_t r_cs);

/* *loss (host) <- (1 / rows) * sum over all elements of  -target * input + max(input, 0) + ln1p(exp(-|input|)): sigmoid and
 * binary cross-entropy in one pass over `input` and `target` [rows, cols] (element strides rs, cs), the terms added in a
 * fixed order. Blocking. Replaces sigmoid_cross_entropy (src/arraymancer/nn_primitives/nnp_sigmoid_cross_entropy.nim:23-45:
 * a map2_inline followed by sum). */
int am_hip_sigmoid_cross_entropy_f32(int64_t rows, int64_t cols, const float* input, int64_t in_rs, int64_t in_cs,
                                     const float* target, int64_t t_rs, int64_t t_cs, float* loss);
int am_hip_sigmoid_cross_entropy_f64(int64_t rows, int64_t cols, const double* input, int64_t in_rs, int64_t in_cs,
                                     const double* target, int64_t t_rs, int64_t t_cs, double* loss);
/* result[i, j] <- gradient * (sigmoid(input[i, j]) - target[i, j]) / rows. Replaces sigmoid_cross_entropy_backward
 * (nnp_sigmoid_cross_entropy.nim:47-62) with a scalar gradient. */
int am_hip_sigmoid_cross_entropy_backward_f32(int64_t rows, int64_t cols, float gradient, const float* input, int64_t in_rs,
                                              int64_t in_cs, const float* target, int64_t t_rs, int64_t t_cs,
                                              float* result, int64_t r_rs, int64_t r_cs);
int am_hip_sigmoid_cross_entropy_backward_f64(int64_t rows, int64_t cols, double gradient, const double* input, int64_t in_rs,
                                              int64_t in_cs, const double* target, int64_t t_rs, int64_t t_cs,
                                              double* result, int64_t r_rs, int64_t r_cs);

/* Max pooling of a C-contiguous [N, C, H, W] input into a C-contiguous [N, C, outH, outW] output,
 * outH = (H + 2 padH - kH) / strideH + 1 (outW alike), plus, when argmax != NULL, the flat input
 * index of each maximum (what maxpool2d_backward scatters through). Same window scan order,
 * strict `>` and starting values as maxpool2d
 * (src/arraymancer/nn_primitives/nnp_maxpooling.nim:19-66): identical values and indices. */
int am_hip_maxpool2d_f32(int64_t N, int C, int H, int W, int kH, int kW, int padH, int padW, int strideH, int strideW,
                         const float* input, float* output, int64_t* argmax);
int am_hip_maxpool2d_f64(int64_t N, int C, int H, int W, int kH, int kW, int padH, int padW, int strideH, int strideW,
                         const double* input, double* output, int64_t* argmax);
int am_hip_maxpool2d_i32(int64_t N, int C, int H, int W, int kH, int kW, int padH, int padW, int strideH, int strideW,
                         const int32_t* input, int32_t* output, int64_t* argmax);
int am_hip_maxpool2d_i64(int64_t N, int C, int H, int W, int kH, int kW, int padH, int padW, int strideH, int strideW,
                         const int64_t* input, int64_t* output, int64_t* argmax);

/* grad_input[N, C, H, W] <- zeros, then grad_input[argmax[i]] = grad_output[i] for the outputs i in
 * ascending order (where overlapping windows recorded the same input element, the last one wins):
 * maxpool2d_backward (src/arraymancer/nn_primitives/nnp_maxpooling.nim:68-83; the reference runs this
 * loop under OpenMP, so its own result for such duplicates depends on thread timing; the serial order
 * is reproduced here). argmax is what am_hip_maxpool2d_* wrote for the same geometry, which the
 * reference's signature does not carry and this one needs: the scatter is run as a race-free gather,
 * every input element looking through the windows that contain it. All tensors C-contiguous. */
int am_hip_maxpool2d_backward_f32(int64_t N, int C, int H, int W, int kH, int kW, int padH, int padW, int strideH,
                                  int strideW, const int64_t* argmax, const float* grad_output, float* grad_input);
int am_hip_maxpool2d_backward_f64(int64_t N, int C, int H, int W, int kH, int kW, int padH, int padW, int strideH,
                                  int strideW, const int64_t* argmax, const double* grad_output, double* grad_input);
int am_hip_maxpool2d_backward_i32(int64_t N, int C, int H, int W, int kH, int kW, int padH, int padW, int strideH,
                                  int strideW, const int64_t* argmax, const int32_t* grad_output, int32_t* grad_input);
int am_hip_maxpool2d_backward_i64(int64_t N, int C, int H, int W, int kH, int kW, int padH, int padW, int strideH,
                                  int strideW, const int64_t* argmax, const int64_t* grad_output, int64_t* grad_input);

/* ---------------------------------------------------------------- measurement aid
 * No counterpart in the reference. Register-only micro-benchmarks of the issue ceilings the GEMM
 * kernels are compared with (used by bench.py: 32/64-bit integers have no matrix instruction and no
 * published VALU multiply-add peak, so the integer GEMM is priced against a measured one).
 *   kind 0: MFMA f32 32x32x2 (FLOP/s)      kind 1: MFMA f64 16x16x4 (FLOP/s)
 *   kind 2: VALU int32 wrapping multiply-add, 8x8 register tile (integer op/s, 2 per MAC)
 *   kind 3: VALU int64 multiply-add
 *   kind 4: MFMA int8 32x32x32 (integer op/s), the instruction of the digit-sliced integer GEMM
 *   kind 5: LDS reads of 16 bytes per lane, no bank conflicts (bytes/s over the whole device)
 *   kind 6: v_mad_u64_u32 alone (the int32 GEMM's multiply-accumulate instruction; integer op/s, 2 per lane and
 *           instruction), written in assembly with constant operands; between am_hip_diag_clock_begin and _end it
 *           also reads the shader clock, which turns the rate into cycles per instruction
 * waves_per_simd wavefronts are resident on every SIMD (1..8); iters loop trips each. */
int am_hip_diag_peak(int kind, int iters, int waves_per_simd, double* ops_per_second);
/* What HBM delivers to a kernel that only streams: kind 0 reads, 1 writes, 2 copies `bytes` (a multiple of
 * 32 KiB) per launch (kind 3: the same copy made by the runtime's own hipMemcpyAsync, device to device, as a
 * figure that no kernel of this library is part of; blocks_per_cu, unroll and flags are ignored) with 16-byte accesses, `unroll` (1, 2, 4, 8) of them in flight per lane, from
 * blocks_per_cu x CUs workgroups of 256 lanes. Launches rotate through `windows` disjoint buffers of `bytes`
 * each (allocated and freed inside the call), so that with windows * bytes several times the 256 MB
 * memory-side cache every byte comes from HBM. flags: bit 0 non-temporal loads, bit 1 non-temporal stores,
 * bit 2 one contiguous run of tiles per workgroup instead of every n-th tile. Result: bytes read plus bytes
 * written per second, averaged over `launches` launches. The HBM-bound kernels are priced against the
 * published 8 TB/s; this is the measured ceiling shown beside it. */
int am_hip_diag_hbm(int kind, size_t bytes, int windows, int blocks_per_cu, int unroll, int flags, int launches,
                    double* bytes_per_second);
/* The shader clock the device sustains under the matrix-core GEMM kernels: between _begin and _end the first
 * lane of workgroup 0 of every gemm_mfma / gemm_i8_digits / gemm_valu launch (and of the kind-6 chain above) compares the shader-cycle counter with the
 * constant-rate counter over the kernel's own lifetime; _end (blocking) returns cycles / ticks as MHz, averaged
 * over those launches (0 if none ran). The matrix peaks are quoted at 2.4 GHz; a power-limited kernel settles
 * lower, and its fraction of peak is read against that. */
int am_hip_diag_clock_begin(void);
int am_hip_diag_clock_end(double* shader_mhz);
/* Where the time of a small-product launch (min(M, N) <= 64: the kernels without LDS staging) goes, read inside the
 * kernel between am_hip_diag_phases_begin and am_hip_diag_phases (which closes the window; blocking) by the first lane
 * of every workgroup (up to 8192 of them), in microseconds: out6[0]
 * workgroups that reported; out6[1..4] the mean time from the first instruction to the first loads issued, from there
 * until they have arrived, from there to the last matrix instruction and the fold of the wavefronts' partial tiles,
 * and from there until the stores are done; out6[5] from the earliest first instruction to the latest store over the
 * whole launch (what the launch's duration on a profiler's timeline exceeds by the dispatch and end-of-kernel work).
 * One launch per window. No counterpart in the reference. */
int am_hip_diag_phases_begin(void);
int am_hip_diag_phases(double* out6);

#ifdef __cplusplus
}
#endif
#endif /* AM_HIP_H */
