/*
 * TEST INFRASTRUCTURE — not part of the product. Only tests, the smoke check and the
 * benchmark's CPU-baseline leg may load this library; the HIP path never does.
 *
 * CPU restatement of Arraymancer's element-wise map / apply machinery (paths under
 * src/arraymancer/tensor/):
 *   higher_order_applymap.nim:27-120   apply_inline, apply2_inline, map_inline, map2_inline
 *   backend/openmp.nim:51-73           omp_parallel_blocks: n < 1000 serial, else
 *                                      min(threads, n) contiguous blocks, last takes the rest
 *   private/p_accessors.nim:181-208    initStridedIteration / advanceStridedIteration
 *                                      (coordinates + backstrides, C order, any strides)
 *   private/p_accessors.nim:378-413    dualStridedIteration (the per-operand walk)
 *   operators_broadcasted.nim:28-194, operators_blas_l1.nim:44-136   the operator bodies
 *   nn_primitives/nnp_activation.nim:35-36, private/p_activation.nim:17-18   relu, sigmoid
 *   nn_primitives/nnp_activation.nim:61-74   relu / sigmoid / tanh backward bodies
 *   ufunc.nim:91, math_functions.nim:218-222, aggregate.nim:115-146   sqrt, square, square(y - mean)
 *   ufunc.nim:82-130, math_functions.nim:52-58, operators_broadcasted.nim:153-182
 *                                      the universal functions (this host's libm), reciprocal, `^.`
 * Op codes are those of include/am_hip.h (AM_OP_*, AM_UOP_*).
 *
 * Pinned by tests/test_oracle_map.py against the reference's literal vectors
 * (tests/tensor/test_broadcasting.nim, test_operators_blas.nim:294-303, test_higherorder.nim)
 * and against NumPy broadcasting / as_strided on random shapes and strides. The backward bodies, sqrt,
 * square and the squared difference have no vector in the reference's tests: each is a short sequence of
 * separately rounded IEEE (or ring) operations and is held bit for bit to NumPy evaluating the same sequence.
 * The universal functions and pow are this host's libm, which is what the reference's map_inline bodies call:
 * pinned on the reference's literals (test_ufunc.nim:38-44 cos / ln, test_broadcasting.nim:130-146 `^.`,
 * test_math_functions.nim:20-30 reciprocal), on NumPy's own evaluation within 2 units in the last place, and
 * on closed forms (floor / ceil / trunc / round on halves and integers, gamma at integers, erf + erfc = 1).
 * Unpinned (no run of the reference possible, Nim stdlib absent): NaN / -0 behaviour of
 * Nim's `max` inside relu; the (0 >= x) ? 0 : x form is adopted.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
static int am_oracle_max_threads(void) { return omp_get_max_threads(); }
#else
static int am_oracle_max_threads(void) { return 1; }
#endif

#define AM_MAXRANK 6
#define OMP_FOR_THRESHOLD 1000   /* src/arraymancer/tensor/backend/global_config.nim:32 */

typedef struct {
  int rank;
  int64_t shape[AM_MAXRANK], strides[AM_MAXRANK], backstrides[AM_MAXRANK], coord[AM_MAXRANK];
  int64_t pos;
} strided_iter;

/* p_accessors.nim:181-198 */
static inline void iter_init(strided_iter* it, int rank, const int64_t* shape,
                             const int64_t* strides, int64_t iter_offset) {
  it->rank = rank;
  it->pos = 0;
  for (int i = 0; i < rank; i++) {
    it->shape[i] = shape[i];
    it->strides[i] = strides[i];
    it->backstrides[i] = strides[i] * (shape[i] - 1);
    it->coord[i] = 0;
  }
  if (iter_offset != 0) {
    int64_t z = 1;
    for (int i = rank - 1; i >= 0; i--) {
      it->coord[i] = (iter_offset / z) % shape[i];
      it->pos += it->coord[i] * strides[i];
      z *= shape[i];
    }
  }
}

/* p_accessors.nim:200-208 */
static inline void iter_advance(strided_iter* it) {
  for (int k = it->rank - 1; k >= 0; k--) {
    if (it->coord[k] < it->shape[k] - 1) {
      it->coord[k] += 1;
      it->pos += it->strides[k];
      break;
    } else {
      it->coord[k] = 0;
      it->pos -= it->backstrides[k];
    }
  }
}

#define T float
#define UT float
#define SFX f32
#define IS_FLOAT 1
#define F_EXP expf
#define F_TANH tanhf
#define F_SQRT sqrtf
#define F_M(name) name##f
#include "strided_map_impl.inc"
#undef T
#undef UT
#undef SFX
#undef IS_FLOAT
#undef F_EXP
#undef F_TANH
#undef F_SQRT
#undef F_M

#define T double
#define UT double
#define SFX f64
#define IS_FLOAT 1
#define F_EXP exp
#define F_TANH tanh
#define F_SQRT sqrt
#define F_M(name) name
#include "strided_map_impl.inc"
#undef T
#undef UT
#undef SFX
#undef IS_FLOAT
#undef F_EXP
#undef F_TANH
#undef F_SQRT
#undef F_M

#define T int32_t
#define UT uint32_t
#define SFX i32
#define IS_FLOAT 0
#include "strided_map_impl.inc"
#undef T
#undef UT
#undef SFX
#undef IS_FLOAT

#define T int64_t
#define UT uint64_t
#define SFX i64
#define IS_FLOAT 0
#include "strided_map_impl.inc"
#undef T
#undef UT
#undef SFX
#undef IS_FLOAT
