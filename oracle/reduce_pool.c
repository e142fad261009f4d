/*
 * TEST INFRASTRUCTURE — not part of the product. Only tests, the smoke check and the
 * benchmark's CPU-baseline leg may load this library; the HIP path never does.
 *
 * CPU restatement of Arraymancer's reductions, row softmax and 2-D max pooling:
 *   tensor/higher_order_foldreduce.nim:22-31   reduce_inline: start from the first element (C order),
 *                                              fold the following ones in order (serial build:
 *                                              omp_parallel_reduce_blocks degenerates to one block)
 *   tensor/higher_order_foldreduce.nim:46-61   reduce_axis_inline: start from a clone of the first
 *                                              slice along the axis, fold slices 1 .. n-1 in order;
 *                                              the result keeps the axis with extent 1
 *   tensor/aggregate.nim:33-113                sum, product, min, max (+ mean = sum div / n)
 *   tensor/aggregate.nim:159-271               argmax_max / argmin_min: first strict maximum / minimum
 *   nn_primitives/private/p_logsumexp.nim:30-62   streaming_max_sumexp, stable_softmax
 *   nn_primitives/nnp_softmax.nim:18-38        softmax over the rows of a [batch, classes] matrix
 *   nn_primitives/nnp_maxpooling.nim:19-66     maxpool2d (values + flat argmax indices)
 *   nn_primitives/nnp_maxpooling.nim:68-83     maxpool2d_backward (scatter through the indices)
 * Op codes are AM_RED_* of include/am_hip.h.
 *
 * Pinned by tests/test_oracle_reduce.py against the reference's literal vectors
 * (tests/tensor/test_aggregate.nim:20-215, tests/nn_primitives/test_nnp_maxpool.nim:20-45) and
 * against NumPy / exact rational arithmetic on random strided inputs. Softmax has no vector in the
 * reference's tests: it is pinned on the closed form exp(x) / sum(exp(x)) in extended precision,
 * on shift invariance and on rows summing to one.
 */
#include <math.h>
#include <stdint.h>
#include <string.h>

#define AM_MAXRANK 6
enum { RED_SUM = 0, RED_PROD = 1, RED_MIN = 2, RED_MAX = 3 };

#define DEFINE_FOLD(T, U, SFX, WRAP)                                                                 \
  static inline T fold_##SFX(int op, T x, T y) {                                                     \
    switch (op) {                                                                                    \
      case RED_SUM: return WRAP ? (T)((U)x + (U)y) : (T)(x + y);                                     \
      case RED_PROD: return WRAP ? (T)((U)x * (U)y) : (T)(x * y);                                    \
      case RED_MIN: return (x <= y) ? x : y;   /* system.min: if x <= y: x else: y */                \
      default: return (y <= x) ? x : y;        /* system.max: if y <= x: x else: y */                \
    }                                                                                                \
  }                                                                                                  \
  /* reduce_axis_inline: dst has extent 1 along `axis` */                                            \
  int am_oracle_reduce_axis_##SFX(int op, int rank, const int64_t* shape, int axis, T* dst,             \
                               const int64_t* sd, const T* a, const int64_t* sa) {                   \
    if (rank < 1 || rank > AM_MAXRANK || axis < 0 || axis >= rank) return -2;                        \
    int64_t outputs = 1;                                                                             \
    for (int d = 0; d < rank; d++) { if (shape[d] == 0) return 0; if (d != axis) outputs *= shape[d]; } \
    int64_t coord[AM_MAXRANK] = {0};                                                                 \
    for (int64_t o = 0; o < outputs; o++) {                                                          \
      int64_t a_off = 0, d_off = 0;                                                                  \
      for (int d = 0; d < rank; d++) if (d != axis) { a_off += coord[d] * sa[d]; d_off += coord[d] * sd[d]; } \
      T acc = a[a_off];                                                                              \
      for (int64_t l = 1; l < shape[axis]; l++) acc = fold_##SFX(op, acc, a[a_off + l * sa[axis]]);  \
      dst[d_off] = acc;                                                                              \
      for (int d = rank - 1; d >= 0; d--) {                                                          \
        if (d == axis) continue;                                                                     \
        if (++coord[d] < shape[d]) break;                                                            \
        coord[d] = 0;                                                                                \
      }                                                                                              \
    }                                                                                                \
    return 0;                                                                                        \
  }                                                                                                  \
  /* argmax_max / argmin_min (tensor/aggregate.nim:159-193, 216-250): values start as slice 0,      \
     positions as 0; slices 1 .. n-1 in order replace them on a strict > (op RED_MAX) or < */        \
  int am_oracle_argreduce_##SFX(int op, int rank, const int64_t* shape, int axis, int64_t* idx,         \
                             const int64_t* si, T* val, const int64_t* sv, const T* a,               \
                             const int64_t* sa) {                                                    \
    if (rank < 1 || rank > AM_MAXRANK || axis < 0 || axis >= rank) return -2;                        \
    if (op != RED_MAX && op != RED_MIN) return -2;                                                   \
    int64_t outputs = 1;                                                                             \
    for (int d = 0; d < rank; d++) { if (shape[d] == 0) return 0; if (d != axis) outputs *= shape[d]; } \
    int64_t coord[AM_MAXRANK] = {0};                                                                 \
    for (int64_t o = 0; o < outputs; o++) {                                                          \
      int64_t a_off = 0, v_off = 0, i_off = 0;                                                       \
      for (int d = 0; d < rank; d++)                                                                 \
        if (d != axis) { a_off += coord[d] * sa[d]; v_off += coord[d] * sv[d]; i_off += coord[d] * si[d]; } \
      T best = a[a_off];                                                                             \
      int64_t at = 0;                                                                                \
      for (int64_t l = 1; l < shape[axis]; l++) {                                                    \
        const T v = a[a_off + l * sa[axis]];                                                         \
        if (op == RED_MAX ? (v > best) : (v < best)) { best = v; at = l; }                           \
      }                                                                                              \
      val[v_off] = best;                                                                             \
      idx[i_off] = at;                                                                               \
      for (int d = rank - 1; d >= 0; d--) {                                                          \
        if (d == axis) continue;                                                                     \
        if (++coord[d] < shape[d]) break;                                                            \
        coord[d] = 0;                                                                                \
      }                                                                                              \
    }                                                                                                \
    return 0;                                                                                        \
  }                                                                                                  \
  /* reduce_inline: C-order fold from the first element */                                           \
  int am_oracle_reduce_all_##SFX(int op, int rank, const int64_t* shape, const T* a, const int64_t* sa, \
                              T* result) {                                                           \
    if (rank < 0 || rank > AM_MAXRANK) return -2;                                                    \
    int64_t size = 1;                                                                                \
    for (int d = 0; d < rank; d++) size *= shape[d];                                                 \
    if (size == 0) return -2;                                                                        \
    int64_t coord[AM_MAXRANK] = {0};                                                                 \
    T acc = a[0];                                                                                    \
    for (int64_t i = 1; i < size; i++) {                                                             \
      for (int d = rank - 1; d >= 0; d--) {                                                          \
        if (++coord[d] < shape[d]) break;                                                            \
        coord[d] = 0;                                                                                \
      }                                                                                              \
      int64_t off = 0;                                                                               \
      for (int d = 0; d < rank; d++) off += coord[d] * sa[d];                                        \
      acc = fold_##SFX(op, acc, a[off]);                                                             \
    }                                                                                                \
    *result = acc;                                                                                   \
    return 0;                                                                                        \
  }                                                                                                  \
  /* nnp_maxpooling.nim:47-66 */                                                                     \
  int am_oracle_maxpool2d_##SFX(int64_t N, int C, int H, int W, int kH, int kW, int padH, int padW,     \
                             int sH, int sW, const T* in, T* out, int64_t* argmax, T lowest) {       \
    const int64_t outH = ((int64_t)H + 2 * padH - kH) / sH + 1, outW = ((int64_t)W + 2 * padW - kW) / sW + 1; \
    for (int64_t n = 0; n < N; n++)                                                                  \
      for (int c = 0; c < C; c++)                                                                    \
        for (int64_t h = 0; h < outH; h++)                                                           \
          for (int64_t w = 0; w < outW; w++) {                                                       \
            T mx = lowest;                                                                           \
            int64_t arg = INT64_MIN;                                                                 \
            for (int ph = 0; ph < kH; ph++) {                                                        \
              const int64_t row = h * sH + ph - padH;                                                \
              if (0 <= row && row < H)                                                               \
                for (int pw = 0; pw < kW; pw++) {                                                    \
                  const int64_t col = w * sW + pw - padW;                                            \
                  if (0 <= col && col < W) {                                                         \
                    const int64_t iidx = col + W * (row + H * (c + n * C));                          \
                    const T val = in[iidx];                                                          \
                    if (val > mx) { mx = val; arg = iidx; }                                          \
                  }                                                                                  \
                }                                                                                    \
            }                                                                                        \
            const int64_t oidx = w + outW * (h + outH * (c + n * C));                                \
            out[oidx] = mx;                                                                          \
            if (argmax) argmax[oidx] = arg;                                                          \
          }                                                                                          \
    return 0;                                                                                        \
  }

/* maxpool2d_backward (nnp_maxpooling.nim:68-83), serial: zeros, then rdata[cmidata[i]] = godata[i] in order */
#define DEFINE_POOL_BACKWARD(T, SFX)                                                                 \
  int am_oracle_maxpool2d_backward_##SFX(int64_t n_in, int64_t n_out, const int64_t* argmax,            \
                                      const T* grad_out, T* grad_in) {                               \
    memset(grad_in, 0, (size_t)n_in * sizeof(T));                                                    \
    for (int64_t i = 0; i < n_out; i++) {                                                            \
      if (argmax[i] < 0 || argmax[i] >= n_in) continue;   /* a window made of padding only */          \
      grad_in[argmax[i]] = grad_out[i];                                                              \
    }                                                                                                \
    return 0;                                                                                        \
  }
DEFINE_POOL_BACKWARD(float, f32)
DEFINE_POOL_BACKWARD(double, f64)
DEFINE_POOL_BACKWARD(int32_t, i32)
DEFINE_POOL_BACKWARD(int64_t, i64)

DEFINE_FOLD(float, float, f32, 0)
DEFINE_FOLD(double, double, f64, 0)
DEFINE_FOLD(int32_t, uint32_t, i32, 1)
DEFINE_FOLD(int64_t, uint64_t, i64, 1)

#define DEFINE_SOFTMAX(T, SFX, EXP)                                                                  \
  /* p_logsumexp.nim:30-40 over one row, then stable_softmax (:57-59) per element */                 \
  int am_oracle_softmax_rows_##SFX(int64_t rows, int64_t cols, T* dst, int64_t d_rs, int64_t d_cs,      \
                                const T* src, int64_t s_rs, int64_t s_cs) {                          \
    for (int64_t i = 0; i < rows; i++) {                                                             \
      T mx = -INFINITY, sumexp = 0;                                                                  \
      for (int64_t j = 0; j < cols; j++) {                                                           \
        const T x = src[i * s_rs + j * s_cs];                                                        \
        if (x <= mx) sumexp += EXP(x - mx);                                                          \
        else { sumexp = sumexp * EXP(mx - x) + 1; mx = x; }                                          \
      }                                                                                              \
      for (int64_t j = 0; j < cols; j++) dst[i * d_rs + j * d_cs] = EXP(src[i * s_rs + j * s_cs] - mx) / sumexp; \
    }                                                                                                \
    return 0;                                                                                        \
  }

DEFINE_SOFTMAX(float, f32, expf)
DEFINE_SOFTMAX(double, f64, exp)
