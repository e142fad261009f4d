// Element-wise / broadcast / map kernels for gfx950 and their host-side dispatch, generic over
// the element type. Each elementwise_<dtype>.hip includes this header and instantiates the
// C-ABI entry points for one type.
//
// Two kernel families:
//   ew_rows     the HBM-streaming path. After dimension collapsing the operands are seen as
//               `rows` x `L` with a unit (or zero) innermost stride; every lane moves 16-byte
//               vectors (dwordx4) with non-temporal loads/stores, several in flight per lane.
//               Broadcast operands are either a vector re-read per row (row vector, stays in
//               L2) or one scalar per row (column vector, read through the scalar path).
//   ew_generic  any strides (transposed, negative, non-unit inner): C-order index -> offsets by
//               per-dimension div/mod on the collapsed shape.
// The reference walks every operand in C order through its own strides
// (src/arraymancer/tensor/private/p_accessors.nim:181-208, 378-413); both kernels compute the
// same element correspondence in closed form instead of carrying coordinates.
#pragma once
#include <stdlib.h>
#include <type_traits>
#include "common.h"

namespace am {
namespace ew {

constexpr int kThreads = 256;
constexpr int kUnroll = 4;  // 16-byte vectors in flight per lane per operand

template <typename T> struct Traits;
template <> struct Traits<float> {
  typedef float U; typedef float V __attribute__((ext_vector_type(4)));
  static constexpr int kVec = 4; static constexpr bool kFloat = true;
};
template <> struct Traits<double> {
  typedef double U; typedef double V __attribute__((ext_vector_type(2)));
  static constexpr int kVec = 2; static constexpr bool kFloat = true;
};
template <> struct Traits<int32_t> {
  typedef uint32_t U; typedef int32_t V __attribute__((ext_vector_type(4)));
  static constexpr int kVec = 4; static constexpr bool kFloat = false;
};
template <> struct Traits<int64_t> {
  typedef uint64_t U; typedef int64_t V __attribute__((ext_vector_type(2)));
  static constexpr int kVec = 2; static constexpr bool kFloat = false;
};

__device__ __forceinline__ float dev_exp(float x) { return expf(x); }
__device__ __forceinline__ double dev_exp(double x) { return exp(x); }
__device__ __forceinline__ float dev_sqrt(float x) { return sqrtf(x); }
__device__ __forceinline__ double dev_sqrt(double x) { return sqrt(x); }
__device__ __forceinline__ float dev_tanh(float x) { return tanhf(x); }
__device__ __forceinline__ double dev_tanh(double x) { return tanh(x); }

// The reference's tests compare `^.` results with == (tests/tensor/test_broadcasting.nim:130-146), and the
// host's powf is correctly rounded in all but rare cases while the device's is not exact even for 2^19.
// Evaluated in double and rounded once, the float result is the correctly rounded one except where the
// exact value lies within 2^-52 (relative) of a rounding boundary.
__device__ __forceinline__ float dev_pow(float x, float y) { return (float)pow((double)x, (double)y); }
__device__ __forceinline__ double dev_pow(double x, double y) { return pow(x, y); }

// The C math library's function for a universal-function op code (tensor/ufunc.nim:82-130), in
// the precision of T. Only instantiated for float and double.
template <int UOP, typename T> __device__ __forceinline__ T dev_math(T x) {
#define AM_MATH1(code, fn) \
  if constexpr (UOP == code) { if constexpr (std::is_same<T, float>::value) return fn##f(x); else return fn(x); } else
  AM_MATH1(AM_UOP_LN, log) AM_MATH1(AM_UOP_LOG10, log10) AM_MATH1(AM_UOP_LOG2, log2)
  AM_MATH1(AM_UOP_SIN, sin) AM_MATH1(AM_UOP_COS, cos) AM_MATH1(AM_UOP_TAN, tan)
  AM_MATH1(AM_UOP_SINH, sinh) AM_MATH1(AM_UOP_COSH, cosh)
  AM_MATH1(AM_UOP_ARCSIN, asin) AM_MATH1(AM_UOP_ARCCOS, acos) AM_MATH1(AM_UOP_ARCTAN, atan)
  AM_MATH1(AM_UOP_ARCSINH, asinh) AM_MATH1(AM_UOP_ARCCOSH, acosh) AM_MATH1(AM_UOP_ARCTANH, atanh)
  AM_MATH1(AM_UOP_CBRT, cbrt) AM_MATH1(AM_UOP_ERF, erf) AM_MATH1(AM_UOP_ERFC, erfc)
  AM_MATH1(AM_UOP_GAMMA, tgamma) AM_MATH1(AM_UOP_LGAMMA, lgamma)
  AM_MATH1(AM_UOP_FLOOR, floor) AM_MATH1(AM_UOP_CEIL, ceil) AM_MATH1(AM_UOP_TRUNC, trunc)
  AM_MATH1(AM_UOP_ROUND, round)
  { static_assert(UOP == AM_UOP_RECIPROCAL, "not a universal-function op code"); return (T)1 / x; }
#undef AM_MATH1
}

// ---- binary op bodies. Integer arithmetic is carried out in the unsigned twin so that it wraps.
template <typename T, int OP> struct BinOp {
  typedef typename Traits<T>::U U;
  static __device__ __forceinline__ T apply(T x, T y) {
    if constexpr (OP == AM_OP_ADD) return (T)((U)x + (U)y);
    else if constexpr (OP == AM_OP_SUB) return (T)((U)x - (U)y);
    else if constexpr (OP == AM_OP_MUL) return (T)((U)x * (U)y);
    else if constexpr (OP == AM_OP_DIV) {
      if constexpr (Traits<T>::kFloat) return x / y;
      else {
        if (y == 0) return 0;
        if (y == (T)-1) return (T)((U)0 - (U)x);
        return x / y;
      }
    } else if constexpr (OP == AM_OP_MOD) {
      if constexpr (std::is_same<T, float>::value) return fmodf(x, y);      // Nim's float `mod` is C fmod: exact
      else if constexpr (std::is_same<T, double>::value) return fmod(x, y);
      else {
        if (y == 0 || y == (T)-1) return 0;
        return x % y;
      }
    } else if constexpr (OP == AM_OP_ADD_RELU) {
      T t = (T)((U)x + (U)y);
      return ((T)0 >= t) ? (T)0 : t;
    } else if constexpr (OP == AM_OP_ADD_SIGMOID) {
      T t = x + y;
      return (T)1 / ((T)1 + dev_exp(-t));
    } else if constexpr (OP == AM_OP_ADD_TANH) {
      return dev_tanh(x + y);
    } else if constexpr (OP == AM_OP_RELU_BWD) {
      return (x <= (T)0) ? (T)0 : y;
    } else if constexpr (OP == AM_OP_MAX) {
      return (y <= x) ? x : y;
    } else if constexpr (OP == AM_OP_MIN) {
      return (x <= y) ? x : y;
    } else if constexpr (OP == AM_OP_SIGMOID_BWD) {
      if constexpr (Traits<T>::kFloat) return x * ((T)1 - x) * y;
      else return (T)((U)x * ((U)1 - (U)x) * (U)y);
    } else if constexpr (OP == AM_OP_TANH_BWD) {
      if constexpr (Traits<T>::kFloat) return y * ((T)1 - x * x);
      else return (T)((U)y * ((U)1 - (U)x * (U)x));
    } else if constexpr (OP == AM_OP_POW) {
      if constexpr (Traits<T>::kFloat) return dev_pow(x, y); else return x;   // never dispatched for integers
    } else if constexpr (OP == AM_OP_FLOORMOD) {
      // Nim's floorMod: r = x mod y, moved by y when r and y have opposite signs (a zero r stays, -0.0 included)
      T r;
      if constexpr (std::is_same<T, float>::value) r = fmodf(x, y);
      else if constexpr (std::is_same<T, double>::value) r = fmod(x, y);
      else r = (y == 0 || y == (T)-1) ? (T)0 : (T)(x % y);
      if ((r > (T)0 && y < (T)0) || (r < (T)0 && y > (T)0)) {
        if constexpr (Traits<T>::kFloat) r = r + y; else r = (T)((U)r + (U)y);
      }
      return r;
    } else if constexpr (OP == AM_OP_COPYSIGN) {
      if constexpr (std::is_same<T, float>::value) return copysignf(x, y);
      else if constexpr (std::is_same<T, double>::value) return copysign(x, y);
      else return x;   // never dispatched for integers
    } else {  // AM_OP_SQDIFF
      if constexpr (Traits<T>::kFloat) { const T d = x - y; return d * d; }
      else { const U d = (U)x - (U)y; return (T)(d * d); }
    }
  }
};

// Unary ops ride the same kernels with the second operand ignored.
constexpr int kUnaryBase = 100;
template <typename T, int UOP> struct UnOp {
  typedef typename Traits<T>::U U;
  static __device__ __forceinline__ T apply(T x, T) {
    if constexpr (UOP == AM_UOP_COPY) return x;
    else if constexpr (UOP == AM_UOP_NEG) {
      if constexpr (Traits<T>::kFloat) return -x; else return (T)((U)0 - (U)x);
    } else if constexpr (UOP == AM_UOP_RELU) return ((T)0 >= x) ? (T)0 : x;
    else if constexpr (UOP == AM_UOP_SIGMOID) return (T)1 / ((T)1 + dev_exp(-x));
    else if constexpr (UOP == AM_UOP_TANH) return dev_tanh(x);
    else if constexpr (UOP == AM_UOP_EXP) return dev_exp(x);
    else if constexpr (UOP == AM_UOP_SQRT) {
      if constexpr (Traits<T>::kFloat) return dev_sqrt(x); else return x;   // never dispatched for integers
    } else if constexpr (UOP == AM_UOP_SQUARE) {
      if constexpr (Traits<T>::kFloat) return x * x; else return (T)((U)x * (U)x);
    }
    else if constexpr (UOP == AM_UOP_DEGTORAD) {   // Nim: d * RadPerDeg, RadPerDeg = PI / 180 rounded to T
      if constexpr (Traits<T>::kFloat) return x * (T)(3.14159265358979323846 / 180.0); else return x;
    } else if constexpr (UOP == AM_UOP_RADTODEG) {   // Nim: d / RadPerDeg
      if constexpr (Traits<T>::kFloat) return x / (T)(3.14159265358979323846 / 180.0); else return x;
    }
    else if constexpr (UOP == AM_UOP_FAC) {   // n! from 0! to 20! (what fits 64 bits, the extent of Nim's table)
      if constexpr (Traits<T>::kFloat) return x;   // never dispatched for floats
      else {
        uint64_t f = 1;
        const bool in_range = x >= 0 && x <= 20;
        for (int i = 2; i <= 20; ++i) f *= (i <= (int)(in_range ? x : 0)) ? (uint64_t)i : 1u;
        return in_range ? (T)f : (T)0;
      }
    }
    else if constexpr (UOP >= AM_UOP_LN) {
      if constexpr (Traits<T>::kFloat) return dev_math<UOP>(x); else return x;   // never dispatched for integers
    }
    else {  // ABS
      if constexpr (Traits<T>::kFloat) return __builtin_fabs(x);
      else return (x < 0) ? (T)((U)0 - (U)x) : x;
    }
  }
};

// Bodies whose result type differs from the operands' (the reference's map templates infer it:
// src/arraymancer/tensor/higher_order_applymap.nim:92-120). Comparisons give Nim's bool as one byte
// (0 / 1): `==.` `!=.` `<.` `<=.` `>.` `>=.` (src/arraymancer/tensor/operators_comparison.nim:41-146)
// and `x mod y == 0`, the body of the reference's own fixture (tests/tensor/test_higherorder.nim:103-112).
constexpr int kCmpBase = 200;
template <typename T, int CMP> struct CmpOp {
  static __device__ __forceinline__ uint8_t apply(T x, T y) {
    if constexpr (CMP == AM_CMP_EQ) return x == y;
    else if constexpr (CMP == AM_CMP_NE) return x != y;
    else if constexpr (CMP == AM_CMP_LT) return x < y;
    else if constexpr (CMP == AM_CMP_LE) return x <= y;
    else if constexpr (CMP == AM_CMP_GT) return x > y;
    else if constexpr (CMP == AM_CMP_GE) return x >= y;
    else return BinOp<T, AM_OP_MOD>::apply(x, y) == (T)0;   // AM_CMP_MOD_IS_ZERO
  }
};

// Predicates and classifiers of one operand: isNaN / isNotNaN (operators_comparison.nim:192-206: x != x,
// x == x), classify (tensor/math_functions.nim:264-276, the ordinal of Nim's FloatClass in one byte) and
// sgn (math_functions.nim:110-117: Tensor[int], i.e. int64; -1, 0, 1, a NaN gives 0).
constexpr int kPredBase = 300;
template <typename T, int PRED> struct PredOp {
  static __device__ __forceinline__ auto apply(T x, T) {
    if constexpr (PRED == AM_PRED_ISNAN) return (uint8_t)(x != x);
    else if constexpr (PRED == AM_PRED_ISNOTNAN) return (uint8_t)(x == x);
    else if constexpr (PRED == AM_PRED_SGN) return (int64_t)((T)0 < x) - (int64_t)(x < (T)0);
    else {   // AM_PRED_CLASSIFY: fcNormal, fcSubnormal, fcZero, fcNegZero, fcNan, fcInf, fcNegInf = 0..6
      if constexpr (Traits<T>::kFloat) {
        if (x != x) return (uint8_t)4;
        if (x == (T)0) return (uint8_t)(__builtin_signbit(x) ? 3 : 2);
        const T ax = __builtin_fabs(x);
        if (ax == (T)__builtin_inf()) return (uint8_t)(x > (T)0 ? 5 : 6);
        constexpr T tiny = std::is_same<T, float>::value ? (T)1.17549435e-38f : (T)2.2250738585072014e-308;
        return (uint8_t)(ax < tiny ? 1 : 0);
      } else return (uint8_t)0;   // never dispatched for integers
    }
  }
};

template <typename T, int CODE> struct OpSel {
  typedef typename std::conditional<(CODE >= kPredBase), PredOp<T, CODE - kPredBase>,
          typename std::conditional<(CODE >= kCmpBase), CmpOp<T, CODE - kCmpBase>,
          typename std::conditional<(CODE >= kUnaryBase), UnOp<T, CODE - kUnaryBase>, BinOp<T, CODE>>::type>::type>::type type;
};

// ---- layouts passed to kernels by value
constexpr int kMaxOuter = AM_MAXRANK - 1;

// How ew_rows sees an operand: a vector stream with its own row offset (kVecOperand), one row re-used for
// every output row (kRowVector: all outer strides zero, loaded once per workgroup and kept in registers), one
// value per row (kRowScalar: inner stride zero) or the scalar argument (kConst).
enum Kind : int { kVecOperand = 0, kRowScalar = 1, kConst = 2, kRowVector = 3 };

// T: element type of the operands, D: of the destination (the same except for comparisons and predicates).
template <typename T, typename D = T> struct RowsArgs {
  D* dst; const T* a; const T* b;
  T scalar;               // the kConst operand
  int a_stream, b_stream; // 1: operand is read once (non-temporal loads); 0: re-read per row, keep cached
  int64_t L;              // inner extent (elements)
  uint32_t tiles_per_row; // ceil(L / tile)
  uint32_t rows;          // product of the outer extents
  uint32_t col_blocks;    // workgroups side by side along a row: workgroup (c, g) = blockIdx.x % col_blocks, / col_blocks
                          // takes the column tiles c, c + col_blocks, ... of the rows g, g + gridDim.x / col_blocks, ...
  int outer_rank;         // 0..5 collapsed outer dims (row-major over them = row index)
  int64_t oshape[kMaxOuter];
  int64_t od[kMaxOuter], oa[kMaxOuter], ob[kMaxOuter];  // outer strides per operand (elements)
};

template <typename T, typename D = T> struct GenericArgs {
  D* dst; const T* a; const T* b;
  T scalar;
  int64_t n;
  int rank;
  int64_t shape[AM_MAXRANK];
  int64_t sd[AM_MAXRANK], sa[AM_MAXRANK], sb[AM_MAXRANK];
};

// Hides a pointer's origin from the optimiser (no instruction is emitted); the result is typed as a pointer to
// global memory, which the optimiser can no longer infer for it.
template <typename P> __device__ __forceinline__ const __attribute__((address_space(1))) P* launder(const P* ptr) {
  auto g = (const __attribute__((address_space(1))) P*)ptr;
  asm("" : "+v"(g));
  return g;
}

// An ordinary or a non-temporal 16-byte load, as two branches (see ew_rows).
template <typename V> __device__ __forceinline__ V load_as(bool keep, const V* ptr) {
  if (keep) return *ptr;
  return __builtin_nontemporal_load(launder(ptr));
}

template <typename T, typename D, int CODE, int AK, int BK, bool SWAP>
__global__ __launch_bounds__(kThreads) void ew_rows(RowsArgs<T, D> p) {
  typedef typename Traits<T>::V V;
  typedef D DV __attribute__((ext_vector_type(Traits<T>::kVec)));   // one result per operand element of a 16-byte vector
  typedef typename OpSel<T, CODE>::type Op;
  constexpr int VEC = Traits<T>::kVec;
  constexpr int64_t TILE = (int64_t)kThreads * VEC * kUnroll;
  constexpr bool A_ROW = AK == kVecOperand || AK == kRowVector, B_ROW = BK == kVecOperand || BK == kRowVector;

  const uint32_t cb = blockIdx.x % p.col_blocks, g0 = blockIdx.x / p.col_blocks, gstep = gridDim.x / p.col_blocks;
  // A workgroup keeps its column tile while it walks down the rows: the column offsets and a row vector that
  // every output row re-uses (the bias of `X +. b`) are computed / loaded once per column tile instead of once
  // per row. WHOLE: the tile lies wholly inside the row (every column tile but a ragged last one), so that
  // the loop body is straight-line code: loads under a branch are waited for one by one.
  auto column_tile = [&](auto whole_tag, uint32_t ct) {
    constexpr bool WHOLE = decltype(whole_tag)::value;
    const int64_t col0 = (int64_t)ct * TILE + (int64_t)threadIdx.x * VEC;
    // Ragged tile: every lane still loads all its vectors, those past the end of the row from the row's first
    // vector instead (the host sends rows shorter than one vector elsewhere), and only the stores are
    // conditional. Loads under a branch would be waited for one at a time.
    bool full[kUnroll];
    int64_t lcol[kUnroll];
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
      const int64_t col = col0 + (int64_t)u * kThreads * VEC;
      full[u] = WHOLE || (col + VEC <= p.L);
      lcol[u] = full[u] ? col : 0;
    }
    V av[kUnroll], bv[kUnroll];
    if constexpr (AK == kRowVector) {
#pragma unroll
      for (int u = 0; u < kUnroll; ++u) av[u] = *(const V*)(p.a + lcol[u]);
    }
    if constexpr (BK == kRowVector) {
#pragma unroll
      for (int u = 0; u < kUnroll; ++u) bv[u] = *(const V*)(p.b + lcol[u]);
    }
    for (uint32_t row = g0; row < p.rows; row += gstep) {
      int64_t offd = 0, offa = 0, offb = 0;
      {
        uint32_t rem = row;
        for (int d = p.outer_rank - 1; d >= 0; --d) {
          const uint32_t ext = (uint32_t)p.oshape[d];
          const uint32_t q = rem / ext;
          const int64_t c = (int64_t)(rem - q * ext);
          rem = q;
          offd += c * p.od[d];
          if constexpr (AK != kRowVector) offa += c * p.oa[d];
          if constexpr (BK != kConst && BK != kRowVector) offb += c * p.ob[d];
        }
      }
      D* __restrict__ drow = p.dst + offd;
      const T* __restrict__ arow = p.a + offa;
      const T* __restrict__ brow = (BK != kConst) ? p.b + offb : nullptr;
      T asc = (T)0, bsc = p.scalar;
      if constexpr (AK == kRowScalar) asc = arow[0];
      if constexpr (BK == kRowScalar) bsc = brow[0];

      // One branch per operand around its loads: a select between a non-temporal and an ordinary load of the
      // same address is merged into an ordinary load by the compiler, hence also the laundered pointer.
      if constexpr (AK == kVecOperand) {
        if (p.a_stream) {
#pragma unroll
          for (int u = 0; u < kUnroll; ++u) av[u] = __builtin_nontemporal_load(launder((const V*)(arow + lcol[u])));
        } else {
#pragma unroll
          for (int u = 0; u < kUnroll; ++u) av[u] = *(const V*)(arow + lcol[u]);
        }
      }
      if constexpr (BK == kVecOperand) {
        if (p.b_stream) {
#pragma unroll
          for (int u = 0; u < kUnroll; ++u) bv[u] = __builtin_nontemporal_load(launder((const V*)(brow + lcol[u])));
        } else {
#pragma unroll
          for (int u = 0; u < kUnroll; ++u) bv[u] = *(const V*)(brow + lcol[u]);
        }
      }
#pragma unroll
      for (int u = 0; u < kUnroll; ++u) {
        DV r;
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
          const T x = A_ROW ? av[u][e] : asc;
          const T y = B_ROW ? bv[u][e] : bsc;
          r[e] = (D)(SWAP ? Op::apply(y, x) : Op::apply(x, y));
        }
        if (full[u]) __builtin_nontemporal_store(r, (DV*)(drow + lcol[u]));
      }
      if constexpr (!WHOLE) {   // the row's last L mod VEC elements, one lane
        const int64_t tail = p.L - p.L % VEC;
        if (threadIdx.x == 0 && tail < p.L && tail >= (int64_t)ct * TILE) {
          for (int64_t c = tail; c < p.L; ++c) {
            const T x = A_ROW ? (AK == kRowVector ? p.a[c] : arow[c]) : asc;
            const T y = B_ROW ? (BK == kRowVector ? p.b[c] : brow[c]) : bsc;
            drow[c] = (D)(SWAP ? Op::apply(y, x) : Op::apply(x, y));
          }
        }
      }
    }
  };
  for (uint32_t ct = cb; ct < p.tiles_per_row; ct += p.col_blocks) {
    if ((int64_t)(ct + 1) * TILE <= p.L) column_tile(std::true_type(), ct);
    else column_tile(std::false_type(), ct);
  }
}

// Rows shorter than half a column tile (a [batch x features] activation plus its bias with a few hundred
// features, per-pixel or per-row factors on images) would leave most of ew_rows' lanes idle. Same operand kinds, other
// decomposition: the problem is the flat sequence of its rows x L / VEC vectors, consecutive lanes take consecutive
// vectors (so a wavefront's access is one contiguous run wherever the rows themselves are contiguous), and every
// vector finds its row, hence its operands' row offsets, by division: a handful of integer instructions per 16 bytes
// moved, where the generic kernel spends them per element and moves 4 bytes per lane and instruction.
// Measured, f32 [65536 x 512] +. [1 x 512]: generic kernel 67.6 us (3.97 TB/s), this one 6.0 TB/s.
// Requires L % VEC == 0; rows x L / VEC < 2^31.
template <typename T, typename D, int CODE, int AK, int BK, bool SWAP>
__global__ __launch_bounds__(kThreads) void ew_short_rows(RowsArgs<T, D> p, uint32_t lv, uint32_t total) {
  typedef typename Traits<T>::V V;
  typedef D DV __attribute__((ext_vector_type(Traits<T>::kVec)));
  typedef typename OpSel<T, CODE>::type Op;
  constexpr int VEC = Traits<T>::kVec;
  const uint32_t v0 = blockIdx.x * (uint32_t)(kThreads * kUnroll) + threadIdx.x;
  bool live[kUnroll];
  int64_t offd[kUnroll], offa[kUnroll], offb[kUnroll];
#pragma unroll
  for (int u = 0; u < kUnroll; ++u) {
    const uint32_t v = v0 + (uint32_t)u * kThreads;
    live[u] = v < total;
    const uint32_t vv = live[u] ? v : 0;     // every lane loads; a vector past the end reads the first one instead
    const uint32_t row = vv / lv;
    const int64_t col = (int64_t)(vv - row * lv) * VEC;
    int64_t od = col, oa = AK == kVecOperand ? col : 0, ob = BK == kVecOperand ? col : 0;
    uint32_t rem = row;
#pragma unroll
    for (int d = kMaxOuter - 1; d >= 0; --d) {
      if (d < p.outer_rank) {
        const uint32_t ext = (uint32_t)p.oshape[d];
        const uint32_t q = rem / ext;
        const int64_t c = (int64_t)(rem - q * ext);
        rem = q;
        od += c * p.od[d];
        oa += c * p.oa[d];
        if constexpr (BK != kConst) ob += c * p.ob[d];
      }
    }
    offd[u] = od; offa[u] = oa; offb[u] = ob;
  }
  V av[kUnroll], bv[kUnroll];
  T asc[kUnroll], bsc[kUnroll];
  if constexpr (AK == kVecOperand) {
    if (p.a_stream) {
#pragma unroll
      for (int u = 0; u < kUnroll; ++u) av[u] = __builtin_nontemporal_load(launder((const V*)(p.a + offa[u])));
    } else {
#pragma unroll
      for (int u = 0; u < kUnroll; ++u) av[u] = *(const V*)(p.a + offa[u]);
    }
  } else {
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) asc[u] = p.a[offa[u]];
  }
  if constexpr (BK == kVecOperand) {
    if (p.b_stream) {
#pragma unroll
      for (int u = 0; u < kUnroll; ++u) bv[u] = __builtin_nontemporal_load(launder((const V*)(p.b + offb[u])));
    } else {
#pragma unroll
      for (int u = 0; u < kUnroll; ++u) bv[u] = *(const V*)(p.b + offb[u]);
    }
  } else if constexpr (BK == kRowScalar) {
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) bsc[u] = p.b[offb[u]];
  } else {
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) bsc[u] = p.scalar;
  }
#pragma unroll
  for (int u = 0; u < kUnroll; ++u) {
    DV r;
#pragma unroll
    for (int e = 0; e < VEC; ++e) {
      const T x = AK == kVecOperand ? av[u][e] : asc[u];
      const T y = BK == kVecOperand ? bv[u][e] : bsc[u];
      r[e] = (D)(SWAP ? Op::apply(y, x) : Op::apply(x, y));
    }
    if (live[u]) __builtin_nontemporal_store(r, (DV*)(p.dst + offd[u]));
  }
}

template <typename T, typename D, int CODE, bool BCONST, bool SWAP, typename IDX>
__global__ __launch_bounds__(kThreads) void ew_generic(GenericArgs<T, D> p) {
  typedef typename OpSel<T, CODE>::type Op;
  const IDX n = (IDX)p.n;
  const IDX step = (IDX)gridDim.x * kThreads;
  for (IDX i = (IDX)blockIdx.x * kThreads + threadIdx.x; i < n; i += step) {
    IDX rem = i;
    int64_t offd = 0, offa = 0, offb = 0;
    for (int d = p.rank - 1; d >= 0; --d) {
      const IDX ext = (IDX)p.shape[d];
      const IDX q = rem / ext;
      const int64_t c = (int64_t)(rem - q * ext);
      rem = q;
      offd += c * p.sd[d];
      offa += c * p.sa[d];
      if constexpr (!BCONST) offb += c * p.sb[d];
    }
    const T x = p.a[offa];
    const T y = BCONST ? p.scalar : p.b[offb];
    p.dst[offd] = (D)(SWAP ? Op::apply(y, x) : Op::apply(x, y));
  }
}

// ---- 2-D tiled kernel: operands whose unit stride runs along the OTHER axis than dst's ------------
// (a + b.transpose, clone of a transposed view, in-place update of a transposed tensor ...).
// After normalisation dst has unit stride along axis 1. An operand with unit stride along axis 0 is
// read in ITS contiguous direction (coalesced) into a padded 64 x 64 LDS tile and consumed
// transposed; operands laid out like dst (or broadcast) are read directly. Every global access of
// a wavefront is therefore a contiguous run, which ew_generic cannot offer for these layouts.
constexpr int kTile2d = 64;

template <typename T, typename D = T> struct TiledArgs {
  D* dst; const T* a; const T* b;
  T scalar;
  int64_t R, C;                 // extents of axis 0 and axis 1
  int64_t d0;                   // dst stride along axis 0 (axis 1 is unit)
  int64_t a0, a1, b0, b1;       // operand strides
  int a_t, b_t;                 // operand has unit stride along axis 0: go through LDS
  int tiles_c;
  int tiles_r, stream;          // vector kernel: tile rows; non-temporal loads (operands beyond what the caches hold)
};

template <typename T, typename D, int CODE, bool BCONST, bool SWAP>
__global__ __launch_bounds__(256) void ew_tiled(TiledArgs<T, D> p) {
  typedef typename OpSel<T, CODE>::type Op;
  __shared__ T ta[kTile2d][kTile2d + 1];
  __shared__ T tb[BCONST ? 1 : kTile2d][kTile2d + 1];
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
  const int tile_r = blockIdx.x / p.tiles_c, tile_c = blockIdx.x - tile_r * p.tiles_c;
  const int64_t r0 = (int64_t)tile_r * kTile2d, c0 = (int64_t)tile_c * kTile2d;
  if (p.a_t) {
#pragma unroll 4
    for (int i = 0; i < kTile2d / 4; ++i) {
      const int cl = ty + 4 * i;                       // local column; lanes run along axis 0
      const int64_t r = r0 + tx, c = c0 + cl;
      if (r < p.R && c < p.C) ta[cl][tx] = p.a[r * p.a0 + c * p.a1];
    }
  }
  if constexpr (!BCONST) {
    if (p.b_t) {
#pragma unroll 4
      for (int i = 0; i < kTile2d / 4; ++i) {
        const int cl = ty + 4 * i;
        const int64_t r = r0 + tx, c = c0 + cl;
        if (r < p.R && c < p.C) tb[cl][tx] = p.b[r * p.b0 + c * p.b1];
      }
    }
  }
  __syncthreads();
#pragma unroll 4
  for (int i = 0; i < kTile2d / 4; ++i) {
    const int rl = ty + 4 * i;
    const int64_t r = r0 + rl, c = c0 + tx;
    if (r < p.R && c < p.C) {
      const T x = p.a_t ? ta[tx][rl] : p.a[r * p.a0 + c * p.a1];
      T y;
      if constexpr (BCONST) y = p.scalar;
      else y = p.b_t ? tb[tx][rl] : p.b[r * p.b0 + c * p.b1];
      p.dst[r * p.d0 + c] = (D)(SWAP ? Op::apply(y, x) : Op::apply(x, y));
    }
  }
}

// The same scheme for operands and results of one width whose runs are 16-byte aligned, at full memory speed:
// tiles of 512 bytes x 512 bytes (128 x 128 four-byte, 64 x 64 eight-byte elements: a wavefront's access is then two
// whole 512-byte runs instead of one of 256 bytes), 16-byte global loads and stores, all of a tile's loads issued before
// the first is needed, non-temporal stores (and loads, beyond what the caches hold), and tiles numbered in bands of
// eight tile rows walked column by column, so that the workgroups running at the same time read and write neighbouring
// runs (4 KiB of every touched row of the transposed operand together, instead of 512 bytes each 8192 columns apart).
// Measured, clone of a transposed 8192 x 8192 float32 view, every byte from HBM: 64 x 64 tiles with element accesses
// 125 us, this form 95 us = 5.6 TB/s against 86 us for a plain copy. A tile that reaches over the edge takes the
// element-wise path of the same layout. LDS rows are padded by one vector: rows stay 16-byte aligned for the
// output's vector reads; the transposing writes then conflict on banks, which costs nothing measurable here
// (an XOR swizzle without conflicts ran at the same speed).
// Bodies whose library code keeps a table in private memory (the argument reduction of sin / cos / tan, gamma) stay on
// the element kernel: there the table lives in registers; here, beside a tile's worth of loads, it goes to scratch.
constexpr bool tiled_vec_body(int code) {
  return !(code == kUnaryBase + AM_UOP_SIN || code == kUnaryBase + AM_UOP_COS || code == kUnaryBase + AM_UOP_TAN ||
           code == kUnaryBase + AM_UOP_GAMMA);
}

template <typename T> struct Tile2dVec {
  static constexpr int TS = 512 / (int)sizeof(T), VEC = 16 / (int)sizeof(T), LD = TS + VEC;
  static constexpr int Q = TS / VEC, RPP = 256 / Q, PASSES = TS / RPP;
  static constexpr size_t kTileBytes = (size_t)TS * LD * sizeof(T);
};

template <typename T, int CODE, bool BCONST, bool SWAP>
__global__ __launch_bounds__(256) void ew_tiled_vec(TiledArgs<T, T> p) {
  typedef typename OpSel<T, CODE>::type Op;
  typedef Tile2dVec<T> G;
  constexpr int TS = G::TS, VEC = G::VEC, LD = G::LD, Q = G::Q, RPP = G::RPP, PASSES = G::PASSES;
  typedef T V __attribute__((ext_vector_type(VEC)));
  extern __shared__ __attribute__((aligned(16))) unsigned char tile_mem[];
  T* ta = reinterpret_cast<T*>(tile_mem);
  T* tb = ta + (p.a_t ? TS * LD : 0);
  const int band = blockIdx.x / (8 * p.tiles_c), in = blockIdx.x - band * 8 * p.tiles_c;
  const int h = p.tiles_r - 8 * band < 8 ? p.tiles_r - 8 * band : 8;
  const int tile_r = 8 * band + in % h, tile_c = in / h;
  const int64_t r0 = (int64_t)tile_r * TS, c0 = (int64_t)tile_c * TS;
  const bool b_t = !BCONST && p.b_t;

  if (r0 + TS > p.R || c0 + TS > p.C) {   // a tile over the edge: one element at a time, same layout
    const int tx = threadIdx.x % TS, ty = threadIdx.x / TS;
    constexpr int STEP = 256 / TS;
    for (int cl = ty; cl < TS; cl += STEP) {
      const int64_t r = r0 + tx, c = c0 + cl;
      if (r < p.R && c < p.C) {
        if (p.a_t) ta[tx * LD + cl] = p.a[r + c * p.a1];
        if (b_t) tb[tx * LD + cl] = p.b[r + c * p.b1];
      }
    }
    __syncthreads();
    for (int rl = ty; rl < TS; rl += STEP) {
      const int64_t r = r0 + rl, c = c0 + tx;
      if (r < p.R && c < p.C) {
        const T x = p.a_t ? ta[rl * LD + tx] : p.a[r * p.a0 + c * p.a1];
        T y;
        if constexpr (BCONST) y = p.scalar;
        else y = b_t ? tb[rl * LD + tx] : p.b[r * p.b0 + c * p.b1];
        p.dst[r * p.d0 + c] = SWAP ? Op::apply(y, x) : Op::apply(x, y);
      }
    }
    return;
  }

  const int q = threadIdx.x % Q, rr = threadIdx.x / Q;
  V va[PASSES], vb[BCONST ? 1 : PASSES];
  // the transposed operands: lane (q, rr) reads VEC elements along axis 0 of column c0 + rr + RPP pass
  if (p.a_t) {
    const T* src = p.a + r0 + VEC * q + (c0 + rr) * p.a1;
    if (p.stream) {
#pragma unroll
      for (int i = 0; i < PASSES; ++i) va[i] = __builtin_nontemporal_load(launder((const V*)(src + (int64_t)i * RPP * p.a1)));
    } else {
#pragma unroll
      for (int i = 0; i < PASSES; ++i) va[i] = *(const V*)(src + (int64_t)i * RPP * p.a1);
    }
  }
  if constexpr (!BCONST) {
    if (b_t) {
      const T* src = p.b + r0 + VEC * q + (c0 + rr) * p.b1;
      if (p.stream) {
#pragma unroll
        for (int i = 0; i < PASSES; ++i) vb[i] = __builtin_nontemporal_load(launder((const V*)(src + (int64_t)i * RPP * p.b1)));
      } else {
#pragma unroll
        for (int i = 0; i < PASSES; ++i) vb[i] = *(const V*)(src + (int64_t)i * RPP * p.b1);
      }
    }
  }
  if (p.a_t) {
#pragma unroll
    for (int i = 0; i < PASSES; ++i)
#pragma unroll
      for (int j = 0; j < VEC; ++j) ta[(VEC * q + j) * LD + rr + i * RPP] = va[i][j];
  }
  if constexpr (!BCONST) {
    if (b_t) {
#pragma unroll
      for (int i = 0; i < PASSES; ++i)
#pragma unroll
        for (int j = 0; j < VEC; ++j) tb[(VEC * q + j) * LD + rr + i * RPP] = vb[i][j];
    }
  }
  __syncthreads();
  // output: lane (q, rr) owns VEC consecutive columns of row r0 + rr + RPP pass; operands laid out like the result are
  // read here (unit stride along axis 1: a vector; stride 0: one value for the row)
  const int64_t col = c0 + VEC * q;
  if (!p.a_t) {
    if (p.a1 == 1) {
      const T* src = p.a + (r0 + rr) * p.a0 + col;
      if (p.stream) {
#pragma unroll
        for (int i = 0; i < PASSES; ++i) va[i] = __builtin_nontemporal_load(launder((const V*)(src + (int64_t)i * RPP * p.a0)));
      } else {
#pragma unroll
        for (int i = 0; i < PASSES; ++i) va[i] = *(const V*)(src + (int64_t)i * RPP * p.a0);
      }
    } else {
#pragma unroll
      for (int i = 0; i < PASSES; ++i) {
        const T x = p.a[(r0 + rr + i * RPP) * p.a0];
#pragma unroll
        for (int j = 0; j < VEC; ++j) va[i][j] = x;
      }
    }
  }
  if constexpr (!BCONST) {
    if (!b_t) {
      if (p.b1 == 1) {
        const T* src = p.b + (r0 + rr) * p.b0 + col;
        if (p.stream) {
#pragma unroll
          for (int i = 0; i < PASSES; ++i) vb[i] = __builtin_nontemporal_load(launder((const V*)(src + (int64_t)i * RPP * p.b0)));
        } else {
#pragma unroll
          for (int i = 0; i < PASSES; ++i) vb[i] = *(const V*)(src + (int64_t)i * RPP * p.b0);
        }
      } else {
#pragma unroll
        for (int i = 0; i < PASSES; ++i) {
          const T y = p.b[(r0 + rr + i * RPP) * p.b0];
#pragma unroll
          for (int j = 0; j < VEC; ++j) vb[i][j] = y;
        }
      }
    }
  }
  T* out = p.dst + (r0 + rr) * p.d0 + col;
#pragma unroll
  for (int i = 0; i < PASSES; ++i) {
    const int rl = rr + i * RPP;
    const V x = p.a_t ? *(const V*)&ta[rl * LD + VEC * q] : va[i];
    V y;
    if constexpr (BCONST) {
#pragma unroll
      for (int j = 0; j < VEC; ++j) y[j] = p.scalar;
    } else {
      y = b_t ? *(const V*)&tb[rl * LD + VEC * q] : vb[i];
    }
    V res;
#pragma unroll
    for (int j = 0; j < VEC; ++j) res[j] = SWAP ? Op::apply(y[j], x[j]) : Op::apply(x[j], y[j]);
    __builtin_nontemporal_store(res, (V*)(out + (int64_t)i * RPP * p.d0));
  }
}

// ---- ternary bodies and kernels (map3_inline / apply3_inline) -----------------------------------
template <typename T, int OP> struct TriOp {
  typedef typename Traits<T>::U U;
  static __device__ __forceinline__ T apply(T x, T y, T z) {
    if constexpr (OP == AM_OP3_MULADD) return (T)((U)x * (U)y + (U)z);
    else if constexpr (OP == AM_OP3_ADDMUL) return (T)(((U)x + (U)y) * (U)z);
    else if constexpr (OP == AM_OP3_GRU_CANDIDATE) return dev_tanh(x + y * z);
    else if constexpr (OP == AM_OP3_CLAMP) return (x < y) ? y : ((x > z) ? z : x);   // a NaN x stays, like Nim's clamp
    else return ((T)1 - y) * z + y * x;
  }
};

template <typename T> struct TriArgs {
  T* dst; const T* a; const T* b; const T* c;
  int64_t n;          // generic kernel: total elements
  int64_t L;          // rows kernel: inner extent
  uint32_t tiles_per_row, rows, col_blocks;   // rows kernel: see RowsArgs
  int rank;           // collapsed rank (generic) / number of outer dims (rows)
  int a_mode, b_mode, c_mode;      // rows kernel: how each operand is read (kTriVec ... kTriImm)
  int bc_imm;                      // operands b and c are the values b_imm and c_imm (clamp bounds passed by value)
  T b_imm, c_imm;
  int64_t shape[AM_MAXRANK];
  int64_t sd[AM_MAXRANK], sa[AM_MAXRANK], sb[AM_MAXRANK], sc[AM_MAXRANK];
};

// Every operand has unit innermost stride and 16-byte aligned rows (the GRU column slices, plain
// contiguous tensors, row vectors broadcast over the rows) or innermost stride 0 (a column vector
// broadcast along the rows: one scalar per row): same streaming structure as ew_rows. A workgroup keeps
// its column tile while it walks down the rows; an operand that is one row for every output row is
// loaded once per column tile and kept in registers; the loads of a row are unconditional (from
// addresses clamped into the row) and sit in one workgroup-uniform branch per operand and kind of load.
// How each operand is read: kTriVec (16-byte loads), kTriVecNt (non-temporal ones), kTriRowVector (one row
// for all output rows), kTriRowScalar (one value per row), kTriImm (a value in the kernel arguments).
enum { kTriVec = 0, kTriVecNt = 1, kTriRowVector = 2, kTriRowScalar = 3, kTriImm = 4 };

template <typename T, int OP>
__global__ __launch_bounds__(kThreads) void ew3_rows(TriArgs<T> p) {
  typedef typename Traits<T>::V V;
  constexpr int VEC = Traits<T>::kVec;
  constexpr int64_t TILE = (int64_t)kThreads * VEC * kUnroll;
  const uint32_t cb = blockIdx.x % p.col_blocks, g0 = blockIdx.x / p.col_blocks, gstep = gridDim.x / p.col_blocks;
  const int am = p.a_mode, bm = p.b_mode, cm = p.c_mode;
  auto column_tile = [&](auto whole_tag, uint32_t ct) {
    constexpr bool WHOLE = decltype(whole_tag)::value;
    const int64_t col0 = (int64_t)ct * TILE + (int64_t)threadIdx.x * VEC;
    bool full[kUnroll];
    int64_t lcol[kUnroll];
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
      const int64_t col = col0 + (int64_t)u * kThreads * VEC;
      full[u] = WHOLE || (col + VEC <= p.L);
      lcol[u] = full[u] ? col : 0;   // (the host sends rows shorter than one vector elsewhere)
    }
    V av[kUnroll], bv[kUnroll], cv[kUnroll];
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) { av[u] = V{}; bv[u] = V{}; cv[u] = V{}; }
    if (am == kTriRowVector) {
#pragma unroll
      for (int u = 0; u < kUnroll; ++u) av[u] = *(const V*)(p.a + lcol[u]);
    }
    if (bm == kTriRowVector) {
#pragma unroll
      for (int u = 0; u < kUnroll; ++u) bv[u] = *(const V*)(p.b + lcol[u]);
    }
    if (cm == kTriRowVector) {
#pragma unroll
      for (int u = 0; u < kUnroll; ++u) cv[u] = *(const V*)(p.c + lcol[u]);
    }
    for (uint32_t row = g0; row < p.rows; row += gstep) {
      int64_t od = 0, oa = 0, ob = 0, oc = 0;
      uint32_t rem = row;
      // constant indices into the argument arrays (a loop with a run-time bound would move them to scratch memory)
#pragma unroll
      for (int d = AM_MAXRANK - 2; d >= 0; --d) {
        if (d < p.rank) {
          const uint32_t ext = (uint32_t)p.shape[d];
          const uint32_t q = rem / ext;
          const int64_t cidx = (int64_t)(rem - q * ext);
          rem = q;
          od += cidx * p.sd[d]; oa += cidx * p.sa[d]; ob += cidx * p.sb[d]; oc += cidx * p.sc[d];
        }
      }
      T* __restrict__ drow = p.dst + od;
      const T* __restrict__ arow = p.a + oa;
      const T* __restrict__ brow = p.b + ob;
      const T* __restrict__ crow = p.c + oc;
      const T asc = am == kTriRowScalar ? arow[0] : (T)0;
      const T bsc = bm == kTriRowScalar ? brow[0] : p.b_imm;
      const T csc = cm == kTriRowScalar ? crow[0] : p.c_imm;
#define AM_TRI_LOADS(mode, vec, rowptr)                                                                                  \
      if (mode == kTriVecNt) {                                                                                            \
        _Pragma("unroll") for (int u = 0; u < kUnroll; ++u) vec[u] = __builtin_nontemporal_load(launder((const V*)(rowptr + lcol[u]))); \
      } else if (mode == kTriVec) {                                                                                       \
        _Pragma("unroll") for (int u = 0; u < kUnroll; ++u) vec[u] = *(const V*)(rowptr + lcol[u]);                       \
      }
      AM_TRI_LOADS(am, av, arow)
      AM_TRI_LOADS(bm, bv, brow)
      AM_TRI_LOADS(cm, cv, crow)
#undef AM_TRI_LOADS
#pragma unroll
      for (int u = 0; u < kUnroll; ++u) {
        V r;
#pragma unroll
        for (int e = 0; e < VEC; ++e)
          r[e] = TriOp<T, OP>::apply(am >= kTriRowScalar ? asc : av[u][e], bm >= kTriRowScalar ? bsc : bv[u][e],
                                     cm >= kTriRowScalar ? csc : cv[u][e]);
        if (full[u]) __builtin_nontemporal_store(r, (V*)(drow + lcol[u]));
      }
      if constexpr (!WHOLE) {   // the row's last L mod VEC elements, one lane
        const int64_t tail = p.L - p.L % VEC;
        if (threadIdx.x == 0 && tail < p.L && tail >= (int64_t)ct * TILE) {
          for (int64_t cc = tail; cc < p.L; ++cc)
            drow[cc] = TriOp<T, OP>::apply(am >= kTriRowScalar ? asc : (am == kTriRowVector ? p.a[cc] : arow[cc]),
                                           bm >= kTriRowScalar ? bsc : (bm == kTriRowVector ? p.b[cc] : brow[cc]),
                                           cm >= kTriRowScalar ? csc : (cm == kTriRowVector ? p.c[cc] : crow[cc]));
        }
      }
    }
  };
  for (uint32_t ct = cb; ct < p.tiles_per_row; ct += p.col_blocks) {
    if ((int64_t)(ct + 1) * TILE <= p.L) column_tile(std::true_type(), ct);
    else column_tile(std::false_type(), ct);
  }
}

// The three-operand bodies on rows shorter than half a column tile (the gate arithmetic of a GRU cell on column slices
// [_, a ..< b] of [batch x 3 hidden] buffers with a few hundred hidden units, nnp_gru.nim:73-88): the flat form, as
// ew_short_rows — consecutive lanes take consecutive 16-byte vectors of the rows x L / VEC of them, each vector finds its row
// and from it every operand's row offset by division. Operand modes as in ew3_rows (a row vector is an ordinary vector
// operand here: its outer strides are zero). Requires L % VEC == 0; rows x L / VEC < 2^31.
template <typename T, int OP>
__global__ __launch_bounds__(kThreads) void ew3_short_rows(TriArgs<T> p, uint32_t lv, uint32_t total) {
  typedef typename Traits<T>::V V;
  constexpr int VEC = Traits<T>::kVec;
  const int am = p.a_mode, bm = p.b_mode, cm = p.c_mode;
  const uint32_t v0 = blockIdx.x * (uint32_t)(kThreads * kUnroll) + threadIdx.x;
  bool live[kUnroll];
  int64_t offd[kUnroll], offa[kUnroll], offb[kUnroll], offc[kUnroll];
#pragma unroll
  for (int u = 0; u < kUnroll; ++u) {
    const uint32_t v = v0 + (uint32_t)u * kThreads;
    live[u] = v < total;
    const uint32_t vv = live[u] ? v : 0;
    const uint32_t row = vv / lv;
    const int64_t col = (int64_t)(vv - row * lv) * VEC;
    int64_t od = col, oa = am >= kTriRowScalar ? 0 : col, ob = bm >= kTriRowScalar ? 0 : col, oc = cm >= kTriRowScalar ? 0 : col;
    uint32_t rem = row;
#pragma unroll
    for (int d = AM_MAXRANK - 2; d >= 0; --d) {
      if (d < p.rank) {
        const uint32_t ext = (uint32_t)p.shape[d];
        const uint32_t q = rem / ext;
        const int64_t cidx = (int64_t)(rem - q * ext);
        rem = q;
        od += cidx * p.sd[d]; oa += cidx * p.sa[d]; ob += cidx * p.sb[d]; oc += cidx * p.sc[d];
      }
    }
    offd[u] = od; offa[u] = oa; offb[u] = ob; offc[u] = oc;
  }
  V av[kUnroll], bv[kUnroll], cv[kUnroll];
  T asc[kUnroll], bsc[kUnroll], csc[kUnroll];
#pragma unroll
  for (int u = 0; u < kUnroll; ++u) { av[u] = V{}; bv[u] = V{}; cv[u] = V{}; asc[u] = (T)0; bsc[u] = p.b_imm; csc[u] = p.c_imm; }
#define AM_TRI_FLAT_LOADS(mode, vec, sc, base, off)                                                                       \
  if (mode == kTriVecNt) {                                                                                                \
    _Pragma("unroll") for (int u = 0; u < kUnroll; ++u) vec[u] = __builtin_nontemporal_load(launder((const V*)(base + off[u]))); \
  } else if (mode == kTriVec || mode == kTriRowVector) {                                                                  \
    _Pragma("unroll") for (int u = 0; u < kUnroll; ++u) vec[u] = *(const V*)(base + off[u]);                              \
  } else if (mode == kTriRowScalar) {                                                                                     \
    _Pragma("unroll") for (int u = 0; u < kUnroll; ++u) sc[u] = base[off[u]];                                             \
  }
  AM_TRI_FLAT_LOADS(am, av, asc, p.a, offa)
  AM_TRI_FLAT_LOADS(bm, bv, bsc, p.b, offb)
  AM_TRI_FLAT_LOADS(cm, cv, csc, p.c, offc)
#undef AM_TRI_FLAT_LOADS
#pragma unroll
  for (int u = 0; u < kUnroll; ++u) {
    V r;
#pragma unroll
    for (int e = 0; e < VEC; ++e)
      r[e] = TriOp<T, OP>::apply(am >= kTriRowScalar ? asc[u] : av[u][e], bm >= kTriRowScalar ? bsc[u] : bv[u][e],
                                 cm >= kTriRowScalar ? csc[u] : cv[u][e]);
    if (live[u]) __builtin_nontemporal_store(r, (V*)(p.dst + offd[u]));
  }
}

template <typename T, int OP, typename IDX>
__global__ __launch_bounds__(kThreads) void ew3_generic(TriArgs<T> p) {
  const IDX n = (IDX)p.n;
  const IDX step = (IDX)gridDim.x * kThreads;
  for (IDX i = (IDX)blockIdx.x * kThreads + threadIdx.x; i < n; i += step) {
    IDX rem = i;
    int64_t od = 0, oa = 0, ob = 0, oc = 0;
    for (int d = p.rank - 1; d >= 0; --d) {
      const IDX ext = (IDX)p.shape[d];
      const IDX q = rem / ext;
      const int64_t cidx = (int64_t)(rem - q * ext);
      rem = q;
      od += cidx * p.sd[d]; oa += cidx * p.sa[d]; ob += cidx * p.sb[d]; oc += cidx * p.sc[d];
    }
    p.dst[od] = TriOp<T, OP>::apply(p.a[oa], p.bc_imm ? p.b_imm : p.b[ob], p.bc_imm ? p.c_imm : p.c[oc]);
  }
}

// ---- host side ------------------------------------------------------------------------------
struct Collapsed {
  int rank;
  int64_t shape[AM_MAXRANK];
  int64_t sd[AM_MAXRANK], sa[AM_MAXRANK], sb[AM_MAXRANK];
  int64_t n;
};

// Drops extent-1 dims and merges neighbours that every operand walks as one run
// (stride[i] == shape[i+1] * stride[i+1] for dst, a and b alike).
static inline int collapse(int rank, const int64_t* shape, const int64_t* sd, const int64_t* sa,
                           const int64_t* sb, Collapsed* out) {
  out->rank = 0;
  out->n = 1;
  for (int i = 0; i < rank; ++i) {
    if (shape[i] < 0) return fail(AM_E_ARG, "negative extent %lld in dimension %d", (long long)shape[i], i);
    out->n *= shape[i];
  }
  if (out->n == 0) return AM_OK;
  for (int i = 0; i < rank; ++i) {
    if (shape[i] == 1) continue;
    const int64_t d = sd[i], a = sa[i], b = sb ? sb[i] : 0;
    if (d == 0) return fail(AM_E_SHAPE, "destination has stride 0 on dimension %d of extent %lld", i, (long long)shape[i]);
    const int r = out->rank;
    if (r > 0 && out->sd[r - 1] == shape[i] * d && out->sa[r - 1] == shape[i] * a &&
        out->sb[r - 1] == shape[i] * b) {
      out->shape[r - 1] *= shape[i];
      out->sd[r - 1] = d; out->sa[r - 1] = a; out->sb[r - 1] = b;
    } else {
      out->shape[r] = shape[i];
      out->sd[r] = d; out->sa[r] = a; out->sb[r] = b;
      out->rank = r + 1;
    }
  }
  if (out->rank == 0) {  // a single element
    out->rank = 1; out->shape[0] = 1; out->sd[0] = 1; out->sa[0] = 1; out->sb[0] = 1;
  }
  return AM_OK;
}

static inline bool aligned16(const void* p) { return ((uintptr_t)p & 15u) == 0; }

template <typename T, int CODE, bool BCONST, bool SWAP, typename D = T>
static int launch_generic(const Collapsed& c, D* dst, const T* a, const T* b, T scalar) {
  GenericArgs<T, D> g;
  g.dst = dst; g.a = a; g.b = b; g.scalar = scalar; g.n = c.n; g.rank = c.rank;
  for (int i = 0; i < AM_MAXRANK; ++i) {
    g.shape[i] = i < c.rank ? c.shape[i] : 1;
    g.sd[i] = i < c.rank ? c.sd[i] : 0;
    g.sa[i] = i < c.rank ? c.sa[i] : 0;
    g.sb[i] = i < c.rank ? c.sb[i] : 0;
  }
  int64_t blocks = (c.n + kThreads - 1) / kThreads;
  const int64_t cap = (int64_t)num_cus() * 16;
  if (blocks > cap) blocks = cap;
  if (c.n < ((int64_t)1 << 31)) {
    hipLaunchKernelGGL((ew_generic<T, D, CODE, BCONST, SWAP, uint32_t>), dim3((unsigned)blocks), dim3(kThreads), 0, stream(), g);
  } else {
    hipLaunchKernelGGL((ew_generic<T, D, CODE, BCONST, SWAP, uint64_t>), dim3((unsigned)blocks), dim3(kThreads), 0, stream(), g);
  }
  return check_launch("ew_generic");
}

// Runs dst = op(a, b) (BCONST: b is `scalar`). Chooses the streaming kernel when every
// operand's innermost collapsed stride is 1 (or 0 for a/b) and rows start 16-byte aligned.
template <typename T, int CODE, bool BCONST, bool SWAP, typename D = T>
static int run(int rank, const int64_t* shape, D* dst, const int64_t* sd, const T* a,
               const int64_t* sa, const T* b, const int64_t* sb, T scalar) {
  constexpr int VEC = Traits<T>::kVec;
  constexpr uintptr_t kDstAlign = VEC * sizeof(D) < 16 ? VEC * sizeof(D) : 16;   // one vector store of VEC results
  Collapsed c;
  AM_TRY(collapse(rank, shape, sd, sa, BCONST ? nullptr : sb, &c));
  if (c.n == 0) return AM_OK;
  AM_TRY(ensure_init());

  const int in = c.rank - 1;
  const int64_t L = c.shape[in];
  const int64_t id = c.sd[in], ia = c.sa[in], ib = BCONST ? 0 : c.sb[in];
  bool ok = (id == 1) && (ia == 0 || ia == 1) && (ib == 0 || ib == 1) && !(ia == 0 && ib == 0 && !BCONST);
  if (BCONST && ia == 0) ok = false;
  if (ok) {
    ok = ((uintptr_t)dst % kDstAlign == 0) && (ia == 0 || aligned16(a)) && (BCONST || ib == 0 || aligned16(b));
    for (int d = 0; d < in && ok; ++d) {
      if (c.sd[d] % VEC != 0) ok = false;
      if (ia == 1 && c.sa[d] % VEC != 0) ok = false;
      if (!BCONST && ib == 1 && c.sb[d] % VEC != 0) ok = false;
    }
  }
  int64_t rows = 1;
  for (int d = 0; d < in; ++d) rows *= c.shape[d];
  const int64_t tile = (int64_t)kThreads * VEC * kUnroll;
  const int64_t tiles_per_row = (L + tile - 1) / tile;
  // Short rows would leave most lanes of a tile idle: whole vectors per row -> the flat form of the kernel, else the
  // generic kernel (and so does a row shorter than one 16-byte vector, which the clamped loads would overrun).
  const bool short_rows = ok && rows > 1 && L < tile / 2 && L >= VEC && L % VEC == 0 && rows * (L / VEC) < ((int64_t)1 << 31);
  if (ok && !short_rows && ((rows > 1 && L < tile / 2) || L < VEC)) ok = false;
  if (ok && (tiles_per_row * rows >= ((int64_t)1 << 31) || rows >= ((int64_t)1 << 31))) ok = false;
  if (!ok) {
    // Two collapsed dims with unit strides on different axes: the LDS-tiled kernel.
    if (c.rank == 2 && c.shape[0] < ((int64_t)1 << 31) && c.shape[1] < ((int64_t)1 << 31)) {
      int ax = -1;                      // axis along which dst has unit stride
      if (c.sd[1] == 1) ax = 1; else if (c.sd[0] == 1) ax = 0;
      if (ax >= 0) {
        const int o = 1 - ax;
        TiledArgs<T, D> t;
        t.dst = dst; t.a = a; t.b = b; t.scalar = scalar;
        t.R = c.shape[o]; t.C = c.shape[ax]; t.d0 = c.sd[o];
        t.a0 = c.sa[o]; t.a1 = c.sa[ax]; t.b0 = BCONST ? 0 : c.sb[o]; t.b1 = BCONST ? 0 : c.sb[ax];
        auto direct = [](int64_t s1) { return s1 == 0 || s1 == 1; };
        t.a_t = (!direct(t.a1) && t.a0 == 1) ? 1 : 0;
        t.b_t = (!BCONST && !direct(t.b1) && t.b0 == 1) ? 1 : 0;
        const bool a_ok = direct(t.a1) || t.a_t, b_ok = BCONST || direct(t.b1) || t.b_t;
        const int64_t tr = (t.R + kTile2d - 1) / kTile2d, tc = (t.C + kTile2d - 1) / kTile2d;
        if (a_ok && b_ok && (t.a_t || t.b_t || ax == 0) && tr * tc < ((int64_t)1 << 31) && t.R >= 16 && t.C >= 16) {
          if constexpr (std::is_same_v<T, D> && tiled_vec_body(CODE)) {
            // 16-byte runs everywhere and at least one whole tile each way: the vector form
            typedef Tile2dVec<T> G;
            auto vec_ok = [&](const void* base, int64_t s_axis0, int64_t s_axis1, bool transposed) {
              if (transposed) return aligned16(base) && s_axis1 % VEC == 0;
              if (s_axis1 == 1) return aligned16(base) && s_axis0 % VEC == 0;
              return s_axis1 == 0;
            };
            static const bool tiled_vec_on = [] { const char* e = getenv("AM_HIP_EW_TILED_VEC"); return !(e && *e == '0'); }();
            if (tiled_vec_on && t.R >= G::TS && t.C >= G::TS && aligned16(dst) && t.d0 % VEC == 0 && vec_ok(a, t.a0, t.a1, t.a_t != 0) &&
                (BCONST || vec_ok(b, t.b0, t.b1, t.b_t != 0))) {
              const int64_t vr = (t.R + G::TS - 1) / G::TS, vc = (t.C + G::TS - 1) / G::TS;
              t.tiles_r = (int)vr; t.tiles_c = (int)vc;
              const double bytes = (double)t.R * (double)t.C * sizeof(T) * (BCONST ? 1.0 : 2.0);
              t.stream = bytes > nt_threshold_bytes() ? 1 : 0;
              const size_t lds = G::kTileBytes * (size_t)((t.a_t ? 1 : 0) + (t.b_t ? 1 : 0));
              auto kernel = ew_tiled_vec<T, CODE, BCONST, SWAP>;
              static bool lds_set = false;   // one flag per instantiation: more than 64 KiB of dynamic LDS has to be asked for
              if (!lds_set) {
                if (hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)(2 * G::kTileBytes)) != hipSuccess)
                  return fail(AM_E_HIP, "hipFuncSetAttribute(ew_tiled_vec) failed");
                lds_set = true;
              }
              hipLaunchKernelGGL(kernel, dim3((unsigned)(vr * vc)), dim3(256), lds, stream(), t);
              return check_launch("ew_tiled_vec");
            }
          }
          t.tiles_c = (int)tc;
          hipLaunchKernelGGL((ew_tiled<T, D, CODE, BCONST, SWAP>), dim3((unsigned)(tr * tc)), dim3(256), 0, stream(), t);
          return check_launch("ew_tiled");
        }
      }
    }
    return launch_generic<T, CODE, BCONST, SWAP, D>(c, dst, a, b, scalar);
  }

  RowsArgs<T, D> r;
  r.dst = dst; r.a = a; r.b = b; r.scalar = scalar; r.L = L;
  r.tiles_per_row = (uint32_t)tiles_per_row;
  r.rows = (uint32_t)rows;
  r.outer_rank = in;
  // An operand whose outer strides are all zero is one row re-read `rows` times: keep it cached.
  r.a_stream = 0; r.b_stream = 0;
  for (int d = 0; d < in; ++d) {
    if (c.sa[d] != 0) r.a_stream = 1;
    if (c.sb[d] != 0) r.b_stream = 1;
  }
  if (in == 0) { r.a_stream = 1; r.b_stream = 1; }
  // Operands that are read once are loaded non-temporally unless they are small enough to be served by the
  // XCDs' L2 (32 MB together). What a previous kernel wrote with non-temporal stores is not in the memory-side
  // cache, so a chain of passes reads every byte from HBM, and from HBM non-temporal loads are the faster ones:
  // f32 8192 x 8192, X +. b then *. s over rotating buffers 183 -> 175 us (the second pass in place: 198 -> 174),
  // one pass 88 -> 86.5 us. (Ordinary loads win only where the same input is read again and again with nothing in
  // between, 77 us: the memory-side cache then still holds part of it.) AM_HIP_EW_NT = 0 | 1 forces the kind.
  {
    const double operand_bytes = (double)rows * (double)L * sizeof(T);
    const int streamed = (ia == 1 ? r.a_stream : 0) + (!BCONST && ib == 1 ? r.b_stream : 0);
    if (!(streamed * operand_bytes > 32.0 * 1024 * 1024)) { r.a_stream = 0; r.b_stream = 0; }
    if (const char* e = getenv("AM_HIP_EW_NT")) { if (*e == '1') { r.a_stream = (ia == 1); r.b_stream = (ib == 1); } else if (*e == '0') { r.a_stream = r.b_stream = 0; } }
  }
  for (int d = 0; d < kMaxOuter; ++d) {
    r.oshape[d] = d < in ? c.shape[d] : 1;
    r.od[d] = d < in ? c.sd[d] : 0;
    r.oa[d] = d < in ? c.sa[d] : 0;
    r.ob[d] = d < in ? c.sb[d] : 0;
  }
  if (short_rows) {
    const uint32_t lv = (uint32_t)(L / VEC), total = (uint32_t)(rows * (L / VEC));
    const dim3 grid((total + kThreads * kUnroll - 1) / (kThreads * kUnroll)), block(kThreads);
    if constexpr (BCONST) {
      hipLaunchKernelGGL((ew_short_rows<T, D, CODE, kVecOperand, kConst, SWAP>), grid, block, 0, stream(), r, lv, total);
    } else {
      if (ia == 1 && ib == 1) hipLaunchKernelGGL((ew_short_rows<T, D, CODE, kVecOperand, kVecOperand, false>), grid, block, 0, stream(), r, lv, total);
      else if (ia == 1) hipLaunchKernelGGL((ew_short_rows<T, D, CODE, kVecOperand, kRowScalar, false>), grid, block, 0, stream(), r, lv, total);
      else hipLaunchKernelGGL((ew_short_rows<T, D, CODE, kRowScalar, kVecOperand, false>), grid, block, 0, stream(), r, lv, total);
    }
    return check_launch("ew_short_rows");
  }
  const int64_t cap = (int64_t)num_cus() * 32;
  const int64_t col_blocks = tiles_per_row < cap ? tiles_per_row : cap;
  int64_t row_groups = cap / col_blocks;
  if (row_groups > rows) row_groups = rows;
  if (row_groups < 1) row_groups = 1;
  r.col_blocks = (uint32_t)col_blocks;
  const dim3 grid((unsigned)(col_blocks * row_groups)), block(kThreads);
  // a vector operand whose outer strides are all zero is the same row for every output row: kept in registers
  bool a_rowvec = ia == 1 && in > 0, b_rowvec = !BCONST && ib == 1 && in > 0;
  for (int d = 0; d < in; ++d) {
    if (c.sa[d] != 0) a_rowvec = false;
    if (BCONST || c.sb[d] != 0) b_rowvec = false;
  }
  if constexpr (BCONST) {
    hipLaunchKernelGGL((ew_rows<T, D, CODE, kVecOperand, kConst, SWAP>), grid, block, 0, stream(), r);
  } else {
    if (ia == 1 && ib == 1) {
      if (b_rowvec && !a_rowvec) hipLaunchKernelGGL((ew_rows<T, D, CODE, kVecOperand, kRowVector, false>), grid, block, 0, stream(), r);
      else if (a_rowvec && !b_rowvec) hipLaunchKernelGGL((ew_rows<T, D, CODE, kRowVector, kVecOperand, false>), grid, block, 0, stream(), r);
      else hipLaunchKernelGGL((ew_rows<T, D, CODE, kVecOperand, kVecOperand, false>), grid, block, 0, stream(), r);
    }
    else if (ia == 1) hipLaunchKernelGGL((ew_rows<T, D, CODE, kVecOperand, kRowScalar, false>), grid, block, 0, stream(), r);
    else hipLaunchKernelGGL((ew_rows<T, D, CODE, kRowScalar, kVecOperand, false>), grid, block, 0, stream(), r);
  }
  return check_launch("ew_rows");
}

static inline int check_common(const char* fn, int rank, const int64_t* shape, const void* dst,
                               const int64_t* sd, const void* a, const int64_t* sa) {
  if (rank < 0 || rank > AM_MAXRANK) return fail(AM_E_ARG, "%s: rank %d outside 0..%d", fn, rank, AM_MAXRANK);
  if (rank > 0 && (!shape || !sd || !sa)) return fail(AM_E_ARG, "%s: null shape/stride array", fn);
  if (!dst || !a) {
    // empty tensors may carry null pointers
    int64_t n = 1;
    for (int i = 0; i < rank; ++i) n *= shape[i];
    if (n != 0) return fail(AM_E_ARG, "%s: null data pointer", fn);
  }
  return AM_OK;
}

template <typename T>
static int binary(const char* fn, int op, int rank, const int64_t* shape, T* dst, const int64_t* sd,
                  const T* a, const int64_t* sa, const T* b, const int64_t* sb) {
  AM_TRY(check_common(fn, rank, shape, dst, sd, a, sa));
  if (rank > 0 && !sb) return fail(AM_E_ARG, "%s: null stride array", fn);
  {
    int64_t n = 1;
    for (int i = 0; i < rank; ++i) n *= shape[i];
    if (n != 0 && !b) return fail(AM_E_ARG, "%s: null data pointer", fn);
  }
  constexpr bool F = Traits<T>::kFloat;
  switch (op) {
#define AM_CASE(code) case code: return run<T, code, false, false>(rank, shape, dst, sd, a, sa, b, sb, (T)0)
    AM_CASE(AM_OP_ADD); AM_CASE(AM_OP_SUB); AM_CASE(AM_OP_MUL); AM_CASE(AM_OP_DIV);
    AM_CASE(AM_OP_ADD_RELU); AM_CASE(AM_OP_RELU_BWD); AM_CASE(AM_OP_MAX); AM_CASE(AM_OP_MIN);
    AM_CASE(AM_OP_SIGMOID_BWD); AM_CASE(AM_OP_TANH_BWD); AM_CASE(AM_OP_SQDIFF); AM_CASE(AM_OP_MOD);
#undef AM_CASE
    case AM_OP_ADD_SIGMOID:
      if constexpr (F) return run<T, AM_OP_ADD_SIGMOID, false, false>(rank, shape, dst, sd, a, sa, b, sb, (T)0);
      else return fail(AM_E_DTYPE, "%s: add_sigmoid is defined for float tensors only", fn);
    case AM_OP_ADD_TANH:
      if constexpr (F) return run<T, AM_OP_ADD_TANH, false, false>(rank, shape, dst, sd, a, sa, b, sb, (T)0);
      else return fail(AM_E_DTYPE, "%s: add_tanh is defined for float tensors only", fn);
    case AM_OP_POW:
      if constexpr (F) return run<T, AM_OP_POW, false, false>(rank, shape, dst, sd, a, sa, b, sb, (T)0);
      else return fail(AM_E_DTYPE, "%s: pow is defined for float tensors only", fn);
    case AM_OP_FLOORMOD: return run<T, AM_OP_FLOORMOD, false, false>(rank, shape, dst, sd, a, sa, b, sb, (T)0);
    case AM_OP_COPYSIGN:
      if constexpr (F) return run<T, AM_OP_COPYSIGN, false, false>(rank, shape, dst, sd, a, sa, b, sb, (T)0);
      else return fail(AM_E_DTYPE, "%s: copySign is defined for float tensors only", fn);
    default:
      return fail(AM_E_ARG, "%s: unknown op %d", fn, op);
  }
}

template <typename T, int CODE>
static int scalar_lr(bool left, int rank, const int64_t* shape, T* dst, const int64_t* sd,
                     const T* a, const int64_t* sa, T s) {
  if (left) return run<T, CODE, true, true>(rank, shape, dst, sd, a, sa, nullptr, nullptr, s);
  return run<T, CODE, true, false>(rank, shape, dst, sd, a, sa, nullptr, nullptr, s);
}

template <typename T>
static int scalar(const char* fn, int op, int left, int rank, const int64_t* shape, T* dst,
                  const int64_t* sd, const T* a, const int64_t* sa, T s) {
  AM_TRY(check_common(fn, rank, shape, dst, sd, a, sa));
  constexpr bool F = Traits<T>::kFloat;
  switch (op) {
#define AM_CASE(code) case code: return scalar_lr<T, code>(left != 0, rank, shape, dst, sd, a, sa, s)
    AM_CASE(AM_OP_ADD); AM_CASE(AM_OP_SUB); AM_CASE(AM_OP_MUL); AM_CASE(AM_OP_DIV);
    AM_CASE(AM_OP_MAX); AM_CASE(AM_OP_MIN); AM_CASE(AM_OP_MOD); AM_CASE(AM_OP_FLOORMOD);
#undef AM_CASE
    case AM_OP_POW:
      if constexpr (F) return scalar_lr<T, AM_OP_POW>(left != 0, rank, shape, dst, sd, a, sa, s);
      else return fail(AM_E_DTYPE, "%s: pow is defined for float tensors only", fn);
    default:
      return fail(AM_E_ARG, "%s: op %d has no tensor-scalar form", fn, op);
  }
}

template <typename T>
static int unary(const char* fn, int op, int rank, const int64_t* shape, T* dst, const int64_t* sd,
                 const T* a, const int64_t* sa) {
  AM_TRY(check_common(fn, rank, shape, dst, sd, a, sa));
  constexpr bool F = Traits<T>::kFloat;
  switch (op) {
#define AM_CASE(code) case code: return run<T, kUnaryBase + code, true, false>(rank, shape, dst, sd, a, sa, nullptr, nullptr, (T)0)
    AM_CASE(AM_UOP_COPY); AM_CASE(AM_UOP_NEG); AM_CASE(AM_UOP_RELU); AM_CASE(AM_UOP_ABS); AM_CASE(AM_UOP_SQUARE);
#undef AM_CASE
    case AM_UOP_SIGMOID:
      if constexpr (F) return run<T, kUnaryBase + AM_UOP_SIGMOID, true, false>(rank, shape, dst, sd, a, sa, nullptr, nullptr, (T)0);
      else return fail(AM_E_DTYPE, "%s: sigmoid is defined for float tensors only", fn);
    case AM_UOP_TANH:
      if constexpr (F) return run<T, kUnaryBase + AM_UOP_TANH, true, false>(rank, shape, dst, sd, a, sa, nullptr, nullptr, (T)0);
      else return fail(AM_E_DTYPE, "%s: tanh is defined for float tensors only", fn);
    case AM_UOP_EXP:
      if constexpr (F) return run<T, kUnaryBase + AM_UOP_EXP, true, false>(rank, shape, dst, sd, a, sa, nullptr, nullptr, (T)0);
      else return fail(AM_E_DTYPE, "%s: exp is defined for float tensors only", fn);
    case AM_UOP_SQRT:
      if constexpr (F) return run<T, kUnaryBase + AM_UOP_SQRT, true, false>(rank, shape, dst, sd, a, sa, nullptr, nullptr, (T)0);
      else return fail(AM_E_DTYPE, "%s: sqrt is defined for float tensors only", fn);
#define AM_CASE(code) \
    case code: \
      if constexpr (F) return run<T, kUnaryBase + code, true, false>(rank, shape, dst, sd, a, sa, nullptr, nullptr, (T)0); \
      else return fail(AM_E_DTYPE, "%s: unary op %d is defined for float tensors only", fn, op)
    AM_CASE(AM_UOP_LN); AM_CASE(AM_UOP_LOG10); AM_CASE(AM_UOP_LOG2); AM_CASE(AM_UOP_SIN); AM_CASE(AM_UOP_COS);
    AM_CASE(AM_UOP_TAN); AM_CASE(AM_UOP_SINH); AM_CASE(AM_UOP_COSH); AM_CASE(AM_UOP_ARCSIN); AM_CASE(AM_UOP_ARCCOS);
    AM_CASE(AM_UOP_ARCTAN); AM_CASE(AM_UOP_ARCSINH); AM_CASE(AM_UOP_ARCCOSH); AM_CASE(AM_UOP_ARCTANH);
    AM_CASE(AM_UOP_CBRT); AM_CASE(AM_UOP_ERF); AM_CASE(AM_UOP_ERFC); AM_CASE(AM_UOP_GAMMA); AM_CASE(AM_UOP_LGAMMA);
    AM_CASE(AM_UOP_FLOOR); AM_CASE(AM_UOP_CEIL); AM_CASE(AM_UOP_TRUNC); AM_CASE(AM_UOP_ROUND); AM_CASE(AM_UOP_RECIPROCAL);
    AM_CASE(AM_UOP_DEGTORAD); AM_CASE(AM_UOP_RADTODEG);
#undef AM_CASE
    case AM_UOP_FAC:
      if constexpr (!F) return run<T, kUnaryBase + AM_UOP_FAC, true, false>(rank, shape, dst, sd, a, sa, nullptr, nullptr, (T)0);
      else return fail(AM_E_DTYPE, "%s: fac is defined for integer tensors only", fn);
    default:
      return fail(AM_E_ARG, "%s: unknown unary op %d", fn, op);
  }
}

// dst (one byte per element, 0 / 1) = cmp(a, b): the broadcast comparison family and any other
// map2 body with a bool result.
template <typename T>
static int compare(const char* fn, int op, int rank, const int64_t* shape, uint8_t* dst, const int64_t* sd,
                   const T* a, const int64_t* sa, const T* b, const int64_t* sb) {
  AM_TRY(check_common(fn, rank, shape, dst, sd, a, sa));
  if (rank > 0 && !sb) return fail(AM_E_ARG, "%s: null stride array", fn);
  {
    int64_t n = 1;
    for (int i = 0; i < rank; ++i) n *= shape[i];
    if (n != 0 && !b) return fail(AM_E_ARG, "%s: null data pointer", fn);
  }
  switch (op) {
#define AM_CASE(code) case code: return run<T, kCmpBase + code, false, false, uint8_t>(rank, shape, dst, sd, a, sa, b, sb, (T)0)
    AM_CASE(AM_CMP_EQ); AM_CASE(AM_CMP_NE); AM_CASE(AM_CMP_LT); AM_CASE(AM_CMP_LE); AM_CASE(AM_CMP_GT); AM_CASE(AM_CMP_GE);
    AM_CASE(AM_CMP_MOD_IS_ZERO);
#undef AM_CASE
    default: return fail(AM_E_ARG, "%s: unknown comparison %d", fn, op);
  }
}

template <typename T>
static int compare_scalar(const char* fn, int op, int rank, const int64_t* shape, uint8_t* dst, const int64_t* sd,
                          const T* a, const int64_t* sa, T s) {
  AM_TRY(check_common(fn, rank, shape, dst, sd, a, sa));
  switch (op) {
#define AM_CASE(code) case code: return run<T, kCmpBase + code, true, false, uint8_t>(rank, shape, dst, sd, a, sa, nullptr, nullptr, s)
    AM_CASE(AM_CMP_EQ); AM_CASE(AM_CMP_NE); AM_CASE(AM_CMP_LT); AM_CASE(AM_CMP_LE); AM_CASE(AM_CMP_GT); AM_CASE(AM_CMP_GE);
    AM_CASE(AM_CMP_MOD_IS_ZERO);
#undef AM_CASE
    default: return fail(AM_E_ARG, "%s: unknown comparison %d", fn, op);
  }
}

template <typename T>
static int predicate(const char* fn, int op, int rank, const int64_t* shape, uint8_t* dst, const int64_t* sd,
                     const T* a, const int64_t* sa) {
  AM_TRY(check_common(fn, rank, shape, dst, sd, a, sa));
  if constexpr (!Traits<T>::kFloat) return fail(AM_E_DTYPE, "%s: defined for float tensors only", fn);
  else switch (op) {
#define AM_CASE(code) case code: return run<T, kPredBase + code, true, false, uint8_t>(rank, shape, dst, sd, a, sa, nullptr, nullptr, (T)0)
    AM_CASE(AM_PRED_ISNAN); AM_CASE(AM_PRED_ISNOTNAN); AM_CASE(AM_PRED_CLASSIFY);
#undef AM_CASE
    default: return fail(AM_E_ARG, "%s: unknown predicate %d", fn, op);
  }
}

template <typename T>
static int sgn(const char* fn, int rank, const int64_t* shape, int64_t* dst, const int64_t* sd, const T* a, const int64_t* sa) {
  AM_TRY(check_common(fn, rank, shape, dst, sd, a, sa));
  return run<T, kPredBase + AM_PRED_SGN, true, false, int64_t>(rank, shape, dst, sd, a, sa, nullptr, nullptr, (T)0);
}

template <typename T, int OP>
static int run3(int rank, const int64_t* shape, T* dst, const int64_t* sd, const T* a, const int64_t* sa,
                const T* b, const int64_t* sb, const T* c, const int64_t* sc, const T* imm = nullptr) {
  constexpr int VEC = Traits<T>::kVec;
  // joint collapse over the four operands
  TriArgs<T> g;
  g.dst = dst; g.a = a; g.b = b; g.c = c;
  g.bc_imm = imm != nullptr; g.b_imm = imm ? imm[0] : (T)0; g.c_imm = imm ? imm[1] : (T)0;
  static const int64_t zero_strides[AM_MAXRANK] = {0, 0, 0, 0, 0, 0};
  if (imm) { sb = zero_strides; sc = zero_strides; }
  int r = 0;
  int64_t n = 1;
  for (int i = 0; i < rank; ++i) {
    if (shape[i] < 0) return fail(AM_E_ARG, "negative extent in dimension %d", i);
    n *= shape[i];
  }
  if (n == 0) return AM_OK;
  for (int i = 0; i < rank; ++i) {
    if (shape[i] == 1) continue;
    if (sd[i] == 0) return fail(AM_E_SHAPE, "destination has stride 0 on dimension %d of extent %lld", i, (long long)shape[i]);
    if (r > 0 && g.sd[r - 1] == shape[i] * sd[i] && g.sa[r - 1] == shape[i] * sa[i] &&
        g.sb[r - 1] == shape[i] * sb[i] && g.sc[r - 1] == shape[i] * sc[i]) {
      g.shape[r - 1] *= shape[i];
      g.sd[r - 1] = sd[i]; g.sa[r - 1] = sa[i]; g.sb[r - 1] = sb[i]; g.sc[r - 1] = sc[i];
    } else {
      g.shape[r] = shape[i]; g.sd[r] = sd[i]; g.sa[r] = sa[i]; g.sb[r] = sb[i]; g.sc[r] = sc[i];
      ++r;
    }
  }
  if (r == 0) { g.shape[0] = 1; g.sd[0] = g.sa[0] = g.sb[0] = g.sc[0] = 1; r = 1; }
  for (int i = r; i < AM_MAXRANK; ++i) { g.shape[i] = 1; g.sd[i] = g.sa[i] = g.sb[i] = g.sc[i] = 0; }
  AM_TRY(ensure_init());
  const int in = r - 1;
  const int64_t L = g.shape[in];
  const bool a_const = g.sa[in] == 0, b_const = g.sb[in] == 0, c_const = g.sc[in] == 0;
  // an operand whose outer strides are all zero is one row for every output row
  bool a_rowvec = in > 0 && !a_const, b_rowvec = in > 0 && !b_const, c_rowvec = in > 0 && !c_const;
  for (int d = 0; d < in; ++d) { a_rowvec &= g.sa[d] == 0; b_rowvec &= g.sb[d] == 0; c_rowvec &= g.sc[d] == 0; }
  bool ok = g.sd[in] == 1 && (g.sa[in] == 1 || a_const) && (g.sb[in] == 1 || b_const) && (g.sc[in] == 1 || c_const) &&
            aligned16(dst) && (a_const || aligned16(a)) && (b_const || aligned16(b)) && (c_const || aligned16(c));
  for (int d = 0; d < in && ok; ++d)
    if (g.sd[d] % VEC || (!a_const && g.sa[d] % VEC) || (!b_const && g.sb[d] % VEC) || (!c_const && g.sc[d] % VEC)) ok = false;
  int64_t rows = 1;
  for (int d = 0; d < in; ++d) rows *= g.shape[d];
  const int64_t tile = (int64_t)kThreads * VEC * kUnroll;
  const int64_t tiles_per_row = (L + tile - 1) / tile;
  // (rows shorter than one vector: the streaming kernel's clamped loads would overrun them)
  // rows shorter than half a column tile would leave most lanes idle (a quarter used: 2.7 TB/s): the flat form when a row is
  // whole vectors, else the generic kernel
  const bool short_rows = ok && rows > 1 && L < tile / 2 && L >= VEC && L % VEC == 0 && rows * (L / VEC) < ((int64_t)1 << 31);
  if (ok && !short_rows && ((rows > 1 && L < tile / 2) || L < VEC)) ok = false;
  if (ok && (tiles_per_row * rows >= ((int64_t)1 << 31) || rows >= ((int64_t)1 << 31))) ok = false;
  g.n = n; g.L = L;
  if (ok) {
    // same rule as the two-operand kernel: non-temporal loads once the operands read once exceed what the L2s hold
    const int streamed = (!a_const && !a_rowvec) + (!imm && !b_const && !b_rowvec) + (!imm && !c_const && !c_rowvec);
    bool nt = streamed * (double)rows * (double)L * sizeof(T) > 32.0 * 1024 * 1024;
    if (const char* e = getenv("AM_HIP_EW_NT")) { if (*e == '1') nt = true; else if (*e == '0') nt = false; }
    auto mode = [&](bool is_const, bool rowvec) { return is_const ? kTriRowScalar : rowvec ? kTriRowVector : nt ? kTriVecNt : kTriVec; };
    g.a_mode = mode(a_const, a_rowvec);
    g.b_mode = imm ? kTriImm : mode(b_const, b_rowvec);
    g.c_mode = imm ? kTriImm : mode(c_const, c_rowvec);
    g.rank = in;
    g.tiles_per_row = (uint32_t)tiles_per_row;
    g.rows = (uint32_t)rows;
    if (short_rows) {
      const uint32_t lv = (uint32_t)(L / VEC), total = (uint32_t)(rows * (L / VEC));
      hipLaunchKernelGGL((ew3_short_rows<T, OP>), dim3((total + kThreads * kUnroll - 1) / (kThreads * kUnroll)), dim3(kThreads), 0, stream(), g, lv, total);
      return check_launch("ew3_short_rows");
    }
    const int64_t cap = (int64_t)num_cus() * 32;
    const int64_t col_blocks = tiles_per_row < cap ? tiles_per_row : cap;
    int64_t row_groups = cap / col_blocks;
    if (row_groups > rows) row_groups = rows;
    if (row_groups < 1) row_groups = 1;
    g.col_blocks = (uint32_t)col_blocks;
    hipLaunchKernelGGL((ew3_rows<T, OP>), dim3((unsigned)(col_blocks * row_groups)), dim3(kThreads), 0, stream(), g);
    return check_launch("ew3_rows");
  }
  g.rank = r;
  int64_t blocks = (n + kThreads - 1) / kThreads;
  const int64_t cap = (int64_t)num_cus() * 16;
  if (blocks > cap) blocks = cap;
  if (n < ((int64_t)1 << 31)) hipLaunchKernelGGL((ew3_generic<T, OP, uint32_t>), dim3((unsigned)blocks), dim3(kThreads), 0, stream(), g);
  else hipLaunchKernelGGL((ew3_generic<T, OP, uint64_t>), dim3((unsigned)blocks), dim3(kThreads), 0, stream(), g);
  return check_launch("ew3_generic");
}

template <typename T>
static int clamp(const char* fn, int rank, const int64_t* shape, T* dst, const int64_t* sd, const T* a, const int64_t* sa, T lo, T hi) {
  AM_TRY(check_common(fn, rank, shape, dst, sd, a, sa));
  const T imm[2] = {lo, hi};
  return run3<T, AM_OP3_CLAMP>(rank, shape, dst, sd, a, sa, nullptr, nullptr, nullptr, nullptr, imm);
}

template <typename T>
static int ternary(const char* fn, int op, int rank, const int64_t* shape, T* dst, const int64_t* sd, const T* a,
                   const int64_t* sa, const T* b, const int64_t* sb, const T* c, const int64_t* sc) {
  AM_TRY(check_common(fn, rank, shape, dst, sd, a, sa));
  if (rank > 0 && (!sb || !sc)) return fail(AM_E_ARG, "%s: null stride array", fn);
  {
    int64_t n = 1;
    for (int i = 0; i < rank; ++i) n *= shape[i];
    if (n != 0 && (!b || !c)) return fail(AM_E_ARG, "%s: null data pointer", fn);
  }
  constexpr bool F = Traits<T>::kFloat;
  switch (op) {
    case AM_OP3_MULADD: return run3<T, AM_OP3_MULADD>(rank, shape, dst, sd, a, sa, b, sb, c, sc);
    case AM_OP3_ADDMUL: return run3<T, AM_OP3_ADDMUL>(rank, shape, dst, sd, a, sa, b, sb, c, sc);
    case AM_OP3_CLAMP: return run3<T, AM_OP3_CLAMP>(rank, shape, dst, sd, a, sa, b, sb, c, sc);
    case AM_OP3_GRU_CANDIDATE:
      if constexpr (F) return run3<T, AM_OP3_GRU_CANDIDATE>(rank, shape, dst, sd, a, sa, b, sb, c, sc);
      else return fail(AM_E_DTYPE, "%s: tanh(x + y * z) is defined for float tensors only", fn);
    case AM_OP3_GRU_BLEND:
      if constexpr (F) return run3<T, AM_OP3_GRU_BLEND>(rank, shape, dst, sd, a, sa, b, sb, c, sc);
      else return fail(AM_E_DTYPE, "%s: (1 - y) * z + y * x is defined for float tensors only", fn);
    default: return fail(AM_E_ARG, "%s: unknown ternary op %d", fn, op);
  }
}

}  // namespace ew
}  // namespace am

#define AM_EW_DEFINE_ENTRY_POINTS(T, SFX)                                                              \
  extern "C" int am_hip_ew_binary_##SFX(int op, int rank, const int64_t* shape, T* dst,                \
                                        const int64_t* ds, const T* a, const int64_t* as_,             \
                                        const T* b, const int64_t* bs) {                               \
    return ::am::ew::binary<T>("am_hip_ew_binary_" #SFX, op, rank, shape, dst, ds, a, as_, b, bs);     \
  }                                                                                                    \
  extern "C" int am_hip_ew_scalar_##SFX(int op, int left, int rank, const int64_t* shape, T* dst,      \
                                        const int64_t* ds, const T* a, const int64_t* as_, T s) {      \
    return ::am::ew::scalar<T>("am_hip_ew_scalar_" #SFX, op, left, rank, shape, dst, ds, a, as_, s);   \
  }                                                                                                    \
  extern "C" int am_hip_ew_ternary_##SFX(int op, int rank, const int64_t* shape, T* dst,               \
                                         const int64_t* ds, const T* a, const int64_t* as_, const T* b, \
                                         const int64_t* bs, const T* c, const int64_t* cs) {           \
    return ::am::ew::ternary<T>("am_hip_ew_ternary_" #SFX, op, rank, shape, dst, ds, a, as_, b, bs, c, \
                                cs);                                                                   \
  }                                                                                                    \
  extern "C" int am_hip_ew_unary_##SFX(int op, int rank, const int64_t* shape, T* dst,                 \
                                       const int64_t* ds, const T* a, const int64_t* as_) {            \
    return ::am::ew::unary<T>("am_hip_ew_unary_" #SFX, op, rank, shape, dst, ds, a, as_);              \
  }                                                                                                    \
  extern "C" int am_hip_ew_compare_##SFX(int op, int rank, const int64_t* shape, uint8_t* dst,         \
                                         const int64_t* ds, const T* a, const int64_t* as_,            \
                                         const T* b, const int64_t* bs) {                              \
    return ::am::ew::compare<T>("am_hip_ew_compare_" #SFX, op, rank, shape, dst, ds, a, as_, b, bs);   \
  }                                                                                                    \
  extern "C" int am_hip_ew_compare_scalar_##SFX(int op, int rank, const int64_t* shape, uint8_t* dst,  \
                                                const int64_t* ds, const T* a, const int64_t* as_, T s) { \
    return ::am::ew::compare_scalar<T>("am_hip_ew_compare_scalar_" #SFX, op, rank, shape, dst, ds, a, as_, s); \
  }                                                                                                    \
  extern "C" int am_hip_ew_clamp_##SFX(int rank, const int64_t* shape, T* dst, const int64_t* ds,      \
                                       const T* a, const int64_t* as_, T lo, T hi) {                   \
    return ::am::ew::clamp<T>("am_hip_ew_clamp_" #SFX, rank, shape, dst, ds, a, as_, lo, hi);          \
  }                                                                                                    \
  extern "C" int am_hip_ew_sgn_##SFX(int rank, const int64_t* shape, int64_t* dst, const int64_t* ds,  \
                                     const T* a, const int64_t* as_) {                                 \
    return ::am::ew::sgn<T>("am_hip_ew_sgn_" #SFX, rank, shape, dst, ds, a, as_);                      \
  }

#define AM_EW_DEFINE_FLOAT_ENTRY_POINTS(T, SFX)                                                        \
  extern "C" int am_hip_ew_predicate_##SFX(int op, int rank, const int64_t* shape, uint8_t* dst,       \
                                           const int64_t* ds, const T* a, const int64_t* as_) {        \
    return ::am::ew::predicate<T>("am_hip_ew_predicate_" #SFX, op, rank, shape, dst, ds, a, as_);      \
  }
