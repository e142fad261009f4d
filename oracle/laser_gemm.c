/*
 * TEST INFRASTRUCTURE — not part of the product. Only tests, the smoke check and the
 * benchmark's CPU-baseline leg may load this library; the HIP path never does.
 *
 * CPU restatement of Arraymancer's laser GEMM, `gemm_strided`, for float32, float64, int32
 * and int64. It follows, function by function (paths under
 * src/arraymancer/laser/primitives/matrix_multiplication/):
 *   gemm.nim:192-273            gemm_strided (entry, views)        -> am_oracle_gemm_strided_*
 *   gemm.nim:117-184            gemm_impl (pc / ic loop nest, beta only on first K panel)
 *   gemm.nim:57-109             gebp_mkernel (jr / ir loops, full vs edge tiles)
 *   gemm_tiling.nim:282-348     partitionMNK / newTiles (mc = 768/sizeof, kc = 2048/sizeof, nc = N)
 *   gemm_tiling.nim:147-219     register tiles for the AVX2+FMA dispatch the reference picks on
 *                               this class of CPU: f32 6x16, f64 6x8, i32 6x16, i64 6x4 (SSE2)
 *   gemm_packing.nim:24-99      pack_A_mc_kc / pack_B_kc_nc with zero padding
 *   gemm_ukernel_generator.nim:143-253  k-loop of the micro-kernel
 *   gemm_ukernel_generic.nim:53-125     epilogues (beta == 0 overwrites C)
 *
 * Pinned by tests/test_oracle_gemm.py against the reference's own known-answer vectors
 * (gemm.nim:315-567, tests/tensor/test_operators_blas.nim) and against closed forms
 * (NumPy modular integer products, float64 / long-double products, exact rationals).
 * The reference itself (Nim) cannot be compiled in this environment.
 *
 * Build: see Makefile (gcc -O3 -fopenmp -mavx2 -mfma -fwrapv).
 */
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

typedef float    v8f32 __attribute__((vector_size(32)));
typedef double   v4f64 __attribute__((vector_size(32)));
typedef uint32_t v8u32 __attribute__((vector_size(32)));
typedef uint64_t v2u64 __attribute__((vector_size(16)));

#define T float
#define UT float
#define VT v8f32
#define NV 8
#define MR 6
#define SFX f32
#include "laser_gemm_impl.inc"
#undef T
#undef UT
#undef VT
#undef NV
#undef MR
#undef SFX

#define T double
#define UT double
#define VT v4f64
#define NV 4
#define MR 6
#define SFX f64
#include "laser_gemm_impl.inc"
#undef T
#undef UT
#undef VT
#undef NV
#undef MR
#undef SFX

#define T int32_t
#define UT uint32_t
#define VT v8u32
#define NV 8
#define MR 6
#define SFX i32
#include "laser_gemm_impl.inc"
#undef T
#undef UT
#undef VT
#undef NV
#undef MR
#undef SFX

#define T int64_t
#define UT uint64_t
#define VT v2u64
#define NV 2
#define MR 6
#define SFX i64
#include "laser_gemm_impl.inc"
#undef T
#undef UT
#undef VT
#undef NV
#undef MR
#undef SFX

#ifdef _OPENMP
#include <omp.h>
int am_oracle_num_threads(void) { return omp_get_max_threads(); }
void am_oracle_set_num_threads(int n) { if (n > 0) omp_set_num_threads(n); }
#else
int am_oracle_num_threads(void) { return 1; }
void am_oracle_set_num_threads(int n) { (void)n; }
#endif
