// am_hip_tensor.hpp — header-only C++ host layer over the C ABI of am_hip.h.
//
// The reference is written in Nim (a compiled language whose toolchain is not available where this
// repository is built), so the compiled host-side mirror of its GPU tensor backend is given in
// C++: `am::HipTensor<T>` has the fields and operator set of `CudaTensor`
// (src/arraymancer/tensor/data_structure.nim:29-67; operators_blas_l2l3_cuda.nim,
// operators_blas_l1_cuda.nim, operators_broadcasted_cuda.nim, shapeshifting_cuda.nim,
// init_cuda.nim) for float, double, int32_t and int64_t, row-major by default, any strides.
// Every operation is exactly one call into libam_hip.so; nothing is computed on the host.
//
//   reference                         here
//   t.cuda / t.cpu                    am::toHip(ptr, shape) / t.toCpu()
//   a * b, gemm(alpha, A, B, beta, C) a * b, am::gemm(alpha, A, B, beta, C)
//   a + b, a - b, a += b, a -= b      same
//   s * t, t * s, t / s               same
//   a +. b, a -. b, a *. b, a /. b    am::bc_add / bc_sub / bc_mul / bc_div   (also tensor-scalar)
//   a +.= b ...                       a.bc_iadd(b) / bc_isub / bc_imul / bc_idiv
//   t ^. e, b ^. t, t ^.= e           am::bc_pow(t, e), am::bc_pow(b, t), t.bc_ipow(e)
//   a ==. b, a <. b, t >=. s ...      am::bc_eq / bc_ne / bc_lt / bc_le / bc_gt / bc_ge  -> HipTensor<uint8_t> (bool)
//   map2_inline(a, b, x mod y == 0)   am::map2_bool(AM_CMP_MOD_IS_ZERO, a, b)
//   isNaN, classify, sgn, clamp       am::isNaN, am::classify, am::sgn, am::clamp / t.mclamp(lo, hi)
//   echo t, t.pretty(precision)       std::cout << t, am::pretty(t, precision, specifier)
//   ln(t), cos(t), floor(t) ...       am::ln(t), am::cos(t), am::floor(t) ...
//   t.transpose, t[a..b|s, ...]       t.transpose(), t.slice(axis, first, last, step)
//   t.broadcast(shape)                t.broadcast(shape)
// Errors: std::invalid_argument where the reference raises ValueError, std::out_of_range where it
// raises IndexDefect, am::HipError for device failures.
#pragma once
#include <cstdint>
#include <cstdlib>
#include <cstring>
#include <algorithm>
#include <cstdio>
#include <fstream>
#include <memory>
#include <ostream>
#include <stdexcept>
#include <string>
#include <type_traits>
#include <vector>

#include "am_hip.h"

namespace am {

struct HipError : std::runtime_error {
  using std::runtime_error::runtime_error;
};

inline void check(int rc) {
  if (rc == AM_OK) return;
  const std::string msg = am_hip_last_error();
  if (rc == AM_E_ARG || rc == AM_E_SHAPE || rc == AM_E_DTYPE) throw std::invalid_argument(msg);
  if (rc == AM_E_ALLOC) throw std::bad_alloc();
  throw HipError(msg);
}

using Shape = std::vector<int64_t>;

namespace detail {
// One overload set per element type keeps the templates below free of dispatch code.
#define AM_HPP_BIND(T, SFX)                                                                              \
  inline int gemm_(int64_t M, int64_t N, int64_t K, T al, const T* A, int64_t ra, int64_t ca, const T* B, \
                   int64_t rb, int64_t cb, T be, T* C, int64_t rc, int64_t cc) {                         \
    return am_hip_gemm_##SFX(M, N, K, al, A, ra, ca, B, rb, cb, be, C, rc, cc);                           \
  }                                                                                                      \
  inline int binary_(int op, int rank, const int64_t* sh, T* d, const int64_t* sd, const T* a,           \
                     const int64_t* sa, const T* b, const int64_t* sb) {                                 \
    return am_hip_ew_binary_##SFX(op, rank, sh, d, sd, a, sa, b, sb);                                     \
  }                                                                                                      \
  inline int scalar_(int op, int left, int rank, const int64_t* sh, T* d, const int64_t* sd, const T* a, \
                     const int64_t* sa, T s) {                                                           \
    return am_hip_ew_scalar_##SFX(op, left, rank, sh, d, sd, a, sa, s);                                   \
  }                                                                                                      \
  inline int unary_(int op, int rank, const int64_t* sh, T* d, const int64_t* sd, const T* a,            \
                    const int64_t* sa) {                                                                 \
    return am_hip_ew_unary_##SFX(op, rank, sh, d, sd, a, sa);                                             \
  }                                                                                                      \
  inline int compare_(int op, int rank, const int64_t* sh, uint8_t* d, const int64_t* sd, const T* a,    \
                      const int64_t* sa, const T* b, const int64_t* sb) {                                \
    return am_hip_ew_compare_##SFX(op, rank, sh, d, sd, a, sa, b, sb);                                    \
  }                                                                                                      \
  inline int compare_scalar_(int op, int rank, const int64_t* sh, uint8_t* d, const int64_t* sd,         \
                             const T* a, const int64_t* sa, T s) {                                       \
    return am_hip_ew_compare_scalar_##SFX(op, rank, sh, d, sd, a, sa, s);                                 \
  }                                                                                                      \
  inline int sgn_(int rank, const int64_t* sh, int64_t* d, const int64_t* sd, const T* a,                \
                  const int64_t* sa) {                                                                   \
    return am_hip_ew_sgn_##SFX(rank, sh, d, sd, a, sa);                                                   \
  }                                                                                                      \
  inline int clamp_(int rank, const int64_t* sh, T* d, const int64_t* sd, const T* a, const int64_t* sa, \
                    T lo, T hi) {                                                                        \
    return am_hip_ew_clamp_##SFX(rank, sh, d, sd, a, sa, lo, hi);                                         \
  }
#define AM_HPP_BIND2(T, SFX)                                                                             \
  inline int gemv_(int64_t M, int64_t N, T al, const T* A, int64_t ra, int64_t ca, const T* x, int64_t ix, \
                   T be, T* y, int64_t iy) {                                                              \
    return am_hip_gemv_##SFX(M, N, al, A, ra, ca, x, ix, be, y, iy);                                      \
  }                                                                                                      \
  inline int dot_(int64_t n, const T* x, int64_t ix, const T* y, int64_t iy, T* r) {                     \
    return am_hip_dot_##SFX(n, x, ix, y, iy, r);                                                          \
  }                                                                                                      \
  inline int reduce_axis_(int op, int rank, const int64_t* sh, int axis, T* d, const int64_t* sd, const T* a, \
                          const int64_t* sa) {                                                            \
    return am_hip_reduce_axis_##SFX(op, rank, sh, axis, d, sd, a, sa);                                    \
  }                                                                                                      \
  inline int argreduce_(int op, int rank, const int64_t* sh, int axis, int64_t* i, const int64_t* si, T* v, \
                        const int64_t* sv, const T* a, const int64_t* sa) {                                \
    return am_hip_argreduce_##SFX(op, rank, sh, axis, i, si, v, sv, a, sa);                               \
  }                                                                                                      \
  inline int reduce_all_(int op, int rank, const int64_t* sh, const T* a, const int64_t* sa, T* r) {      \
    return am_hip_reduce_all_##SFX(op, rank, sh, a, sa, r);                                               \
  }                                                                                                      \
  inline int maxpool2d_backward_(int64_t N, int C, int H, int W, int kH, int kW, int pH, int pW, int sH, int sW, \
                                 const int64_t* idx, const T* go, T* gi) {                                \
    return am_hip_maxpool2d_backward_##SFX(N, C, H, W, kH, kW, pH, pW, sH, sW, idx, go, gi);              \
  }                                                                                                      \
  inline int maxpool2d_(int64_t N, int C, int H, int W, int kH, int kW, int pH, int pW, int sH, int sW,    \
                        const T* in, T* out, int64_t* idx) {                                              \
    return am_hip_maxpool2d_##SFX(N, C, H, W, kH, kW, pH, pW, sH, sW, in, out, idx);                      \
  }                                                                                                      \
  inline int im2col_(int64_t N, int C, int H, int W, int kH, int kW, int pH, int pW, int sH, int sW, const T* in, \
                     int64_t in_n, int64_t in_c, int64_t in_h, int64_t in_w, T* col) {                     \
    return am_hip_im2col_##SFX(N, C, H, W, kH, kW, pH, pW, sH, sW, in, in_n, in_c, in_h, in_w, col);      \
  }                                                                                                      \
  inline int im2col_strided_(int64_t N, int C, int H, int W, int kH, int kW, int pH, int pW, int sH, int sW, const T* in, \
                             int64_t in_n, int64_t in_c, int64_t in_h, int64_t in_w, T* col, int64_t col_n, int64_t col_c) { \
    return am_hip_im2col_strided_##SFX(N, C, H, W, kH, kW, pH, pW, sH, sW, in, in_n, in_c, in_h, in_w, col, col_n, col_c); \
  }                                                                                                      \
  inline int col2im_(int64_t N, int C, int H, int W, int kH, int kW, int pH, int pW, int sH, int sW, const T* col, \
                     int64_t col_n, int64_t col_c, T* out, int64_t on, int64_t oc, int64_t oh, int64_t ow) { \
    return am_hip_col2im_##SFX(N, C, H, W, kH, kW, pH, pW, sH, sW, col, col_n, col_c, out, on, oc, oh, ow); \
  }                                                                                                      \
  inline int gemm_batched_(int64_t batch, int64_t M, int64_t N, int64_t K, T al, const T* A, int64_t ra, int64_t ca, \
                           int64_t ba, const T* B, int64_t rb, int64_t cb, int64_t bb, T be, T* C, int64_t rc,     \
                           int64_t cc, int64_t bc, int epi, const T* bias, int64_t brs, int64_t bcs) {            \
    return am_hip_gemm_batched_##SFX(batch, M, N, K, al, A, ra, ca, ba, B, rb, cb, bb, be, C, rc, cc, bc, epi,    \
                                     bias, brs, bcs);                                                      \
  }
AM_HPP_BIND2(float, f32)
AM_HPP_BIND2(double, f64)
AM_HPP_BIND2(int32_t, i32)
AM_HPP_BIND2(int64_t, i64)
#undef AM_HPP_BIND2
AM_HPP_BIND(float, f32)
AM_HPP_BIND(double, f64)
AM_HPP_BIND(int32_t, i32)
AM_HPP_BIND(int64_t, i64)
#undef AM_HPP_BIND
// Unsigned element types ride the kernels of their signed twins, like the reference's GEMM overload for
// uint32 | uint64 | uint | int (laser/primitives/matrix_multiplication/gemm.nim:275-307: the pointers are cast onto the
// int32 / int64 kernels). In the rings Z/2^32 and Z/2^64 the bits of + - * (hence of matrix products, dot, sums and
// products of elements) do not depend on how the operands are read. Whatever reads the sign (division, remainder,
// comparisons, min / max, clamp, sgn) has no overload for these types and does not compile; the run-time codes of
// the generic entry points are checked here.
inline void ring_only_(bool ok, const char* what) {
  if (!ok) throw std::invalid_argument(std::string(what) + " reads the sign of its operands: not defined on unsigned tensors");
}
#define AM_HPP_UNSIGNED(U, S)                                                                            \
  inline int gemm_(int64_t M, int64_t N, int64_t K, U al, const U* A, int64_t ra, int64_t ca, const U* B, \
                   int64_t rb, int64_t cb, U be, U* C, int64_t rc, int64_t cc) {                         \
    return gemm_(M, N, K, (S)al, (const S*)A, ra, ca, (const S*)B, rb, cb, (S)be, (S*)C, rc, cc);         \
  }                                                                                                      \
  inline int gemv_(int64_t M, int64_t N, U al, const U* A, int64_t ra, int64_t ca, const U* x, int64_t ix, \
                   U be, U* y, int64_t iy) {                                                              \
    return gemv_(M, N, (S)al, (const S*)A, ra, ca, (const S*)x, ix, (S)be, (S*)y, iy);                    \
  }                                                                                                      \
  inline int dot_(int64_t n, const U* x, int64_t ix, const U* y, int64_t iy, U* r) {                     \
    return dot_(n, (const S*)x, ix, (const S*)y, iy, (S*)r);                                              \
  }                                                                                                      \
  inline int binary_(int op, int rank, const int64_t* sh, U* d, const int64_t* sd, const U* a,           \
                     const int64_t* sa, const U* b, const int64_t* sb) {                                 \
    ring_only_(op == AM_OP_ADD || op == AM_OP_SUB || op == AM_OP_MUL, "this map2 body");                  \
    return binary_(op, rank, sh, (S*)d, sd, (const S*)a, sa, (const S*)b, sb);                            \
  }                                                                                                      \
  inline int scalar_(int op, int left, int rank, const int64_t* sh, U* d, const int64_t* sd, const U* a, \
                     const int64_t* sa, U s) {                                                           \
    ring_only_(op == AM_OP_ADD || op == AM_OP_SUB || op == AM_OP_MUL, "this scalar operation");           \
    return scalar_(op, left, rank, sh, (S*)d, sd, (const S*)a, sa, (S)s);                                 \
  }                                                                                                      \
  inline int unary_(int op, int rank, const int64_t* sh, U* d, const int64_t* sd, const U* a,            \
                    const int64_t* sa) {                                                                 \
    ring_only_(op == AM_UOP_COPY || op == AM_UOP_NEG, "this map body");                                   \
    return unary_(op, rank, sh, (S*)d, sd, (const S*)a, sa);                                              \
  }                                                                                                      \
  inline int reduce_axis_(int op, int rank, const int64_t* sh, int axis, U* d, const int64_t* sd, const U* a, \
                          const int64_t* sa) {                                                            \
    ring_only_(op == AM_RED_SUM || op == AM_RED_PROD, "min / max");                                       \
    return reduce_axis_(op, rank, sh, axis, (S*)d, sd, (const S*)a, sa);                                  \
  }                                                                                                      \
  inline int reduce_all_(int op, int rank, const int64_t* sh, const U* a, const int64_t* sa, U* r) {      \
    ring_only_(op == AM_RED_SUM || op == AM_RED_PROD, "min / max");                                       \
    return reduce_all_(op, rank, sh, (const S*)a, sa, (S*)r);                                             \
  }
AM_HPP_UNSIGNED(uint32_t, int32_t)
AM_HPP_UNSIGNED(uint64_t, int64_t)
#undef AM_HPP_UNSIGNED
inline int gemm_ex_(int64_t M, int64_t N, int64_t K, float al, const float* A, int64_t ra, int64_t ca,
                    const float* B, int64_t rb, int64_t cb, float be, float* C, int64_t rc, int64_t cc, int epi,
                    const float* bias, int64_t brs, int64_t bcs) {
  return am_hip_gemm_ex_f32(M, N, K, al, A, ra, ca, B, rb, cb, be, C, rc, cc, epi, bias, brs, bcs);
}
inline int gemm_ex_(int64_t M, int64_t N, int64_t K, double al, const double* A, int64_t ra, int64_t ca,
                    const double* B, int64_t rb, int64_t cb, double be, double* C, int64_t rc, int64_t cc, int epi,
                    const double* bias, int64_t brs, int64_t bcs) {
  return am_hip_gemm_ex_f64(M, N, K, al, A, ra, ca, B, rb, cb, be, C, rc, cc, epi, bias, brs, bcs);
}

inline int conv2d_grad_weight_(int64_t N, int C, int H, int W, int Co, int kH, int kW, int pH, int pW, int sH, int sW, const float* in,
                               int64_t in_n, int64_t in_c, int64_t in_h, int64_t in_w, const float* g, int64_t g_rs, float* out) {
  return am_hip_conv2d_grad_weight_f32(N, C, H, W, Co, kH, kW, pH, pW, sH, sW, in, in_n, in_c, in_h, in_w, g, g_rs, out);
}
inline int conv2d_grad_weight_(int64_t N, int C, int H, int W, int Co, int kH, int kW, int pH, int pW, int sH, int sW, const double* in,
                               int64_t in_n, int64_t in_c, int64_t in_h, int64_t in_w, const double* g, int64_t g_rs, double* out) {
  return am_hip_conv2d_grad_weight_f64(N, C, H, W, Co, kH, kW, pH, pW, sH, sW, in, in_n, in_c, in_h, in_w, g, g_rs, out);
}
inline int conv2d_(int64_t N, int C, int H, int W, int Co, int kH, int kW, int pH, int pW, int sH, int sW, const float* in,
                   int64_t in_n, int64_t in_c, int64_t in_h, int64_t in_w, const float* k, int64_t k_rs, int epi,
                   const float* bias, int64_t bias_s, float* out) {
  return am_hip_conv2d_f32(N, C, H, W, Co, kH, kW, pH, pW, sH, sW, in, in_n, in_c, in_h, in_w, k, k_rs, epi, bias, bias_s, out);
}
inline int conv2d_(int64_t N, int C, int H, int W, int Co, int kH, int kW, int pH, int pW, int sH, int sW, const double* in,
                   int64_t in_n, int64_t in_c, int64_t in_h, int64_t in_w, const double* k, int64_t k_rs, int epi,
                   const double* bias, int64_t bias_s, double* out) {
  return am_hip_conv2d_f64(N, C, H, W, Co, kH, kW, pH, pW, sH, sW, in, in_n, in_c, in_h, in_w, k, k_rs, epi, bias, bias_s, out);
}
inline int predicate_(int op, int rank, const int64_t* sh, uint8_t* d, const int64_t* sd, const float* a, const int64_t* sa) {
  return am_hip_ew_predicate_f32(op, rank, sh, d, sd, a, sa);
}
inline int predicate_(int op, int rank, const int64_t* sh, uint8_t* d, const int64_t* sd, const double* a, const int64_t* sa) {
  return am_hip_ew_predicate_f64(op, rank, sh, d, sd, a, sa);
}

inline int softmax_(int64_t r, int64_t c, float* d, int64_t drs, int64_t dcs, const float* s, int64_t srs, int64_t scs) {
  return am_hip_softmax_rows_f32(r, c, d, drs, dcs, s, srs, scs);
}
inline int softmax_(int64_t r, int64_t c, double* d, int64_t drs, int64_t dcs, const double* s, int64_t srs, int64_t scs) {
  return am_hip_softmax_rows_f64(r, c, d, drs, dcs, s, srs, scs);
}

inline std::string str(const Shape& s) {
  std::string r = "[";
  for (size_t i = 0; i < s.size(); ++i) r += (i ? ", " : "") + std::to_string(s[i]);
  return r + "]";
}
}  // namespace detail

// Device allocation shared by every view of it; freed with the last view
// (the role of CudaTensorRefTracker, data_structure.nim:29-67).
template <typename T>
struct HipStorage {
  T* data = nullptr;
  int64_t len = 0;
  explicit HipStorage(int64_t n) : len(n) {
    void* p = nullptr;
    check(am_hip_malloc((size_t)n * sizeof(T), &p));
    data = static_cast<T*>(p);
  }
  // am_hip_free does not fail for a block of am_hip_malloc (inside a graph capture the library keeps the
  // block for the graph instead of releasing it); a destructor could not report it anyway.
  ~HipStorage() { (void)am_hip_free(data); }
  HipStorage(const HipStorage&) = delete;
  HipStorage& operator=(const HipStorage&) = delete;
};

template <typename T>
class HipTensor {
  // uint8_t holds the result of a map whose body changes the type: Tensor[bool] of the comparisons (one
  // byte per element, 0 / 1) and classify's FloatClass ordinals. Such a tensor can be viewed and copied to
  // the host; no arithmetic is defined on it.
  static_assert(std::is_same<T, float>::value || std::is_same<T, double>::value ||
                    std::is_same<T, int32_t>::value || std::is_same<T, int64_t>::value || std::is_same<T, uint8_t>::value ||
                    std::is_same<T, uint32_t>::value || std::is_same<T, uint64_t>::value,
                "HipTensor supports float, double, int32_t and int64_t (uint32_t and uint64_t for + - * and products, "
                "uint8_t as a result type)");

 public:
  Shape shape, strides;     // elements
  int64_t offset = 0;
  std::shared_ptr<HipStorage<T>> storage;

  HipTensor() = default;
  // newTensorUninit: row-major, uninitialised.
  explicit HipTensor(const Shape& shp) : shape(shp), strides(shp.size()) {
    if (shp.size() > AM_MAXRANK) throw std::invalid_argument("rank exceeds " + std::to_string(AM_MAXRANK));
    int64_t acc = 1;
    for (int i = (int)shp.size() - 1; i >= 0; --i) { strides[i] = acc; acc *= shp[i]; }
    storage = std::make_shared<HipStorage<T>>(acc);
  }

  int rank() const { return (int)shape.size(); }
  int64_t size() const { int64_t n = 1; for (auto s : shape) n *= s; return n; }
  T* ptr() const { return storage->data + offset; }   // get_offset_ptr

  bool is_C_contiguous() const {
    int64_t cur = 1;
    for (int i = rank() - 1; i >= 0; --i) {
      if (shape[i] != 1 && strides[i] != cur) return false;
      cur *= shape[i];
    }
    return true;
  }
  bool is_F_contiguous() const {
    int64_t cur = 1;
    for (int i = 0; i < rank(); ++i) {
      if (shape[i] != 1 && strides[i] != cur) return false;
      cur *= shape[i];
    }
    return true;
  }

  // ---- views: metadata only, storage shared -------------------------------------------------
  HipTensor transpose() const {   // shapeshifting.nim:27-36
    HipTensor r = *this;
    r.shape.assign(shape.rbegin(), shape.rend());
    r.strides.assign(strides.rbegin(), strides.rend());
    return r;
  }
  // t[.., first..last|step, ..] on one axis, inclusive ends (p_accessors_macros_read.nim:39-58).
  HipTensor slice(int axis, int64_t first, int64_t last, int64_t step = 1) const {
    if (axis < 0 || axis >= rank()) throw std::out_of_range("slice: axis out of range");
    if (first < 0 || first >= shape[axis] || last < 0 || last >= shape[axis] || step == 0 ||
        (first < last && step < 0) || (first > last && step > 0))
      throw std::out_of_range("slice " + std::to_string(first) + ".." + std::to_string(last) + "|" +
                              std::to_string(step) + " invalid for extent " + std::to_string(shape[axis]));
    HipTensor r = *this;
    r.offset += first * strides[axis];
    r.strides[axis] *= step;
    r.shape[axis] = std::llabs(last - first) / std::llabs(step) + 1;
    return r;
  }
  HipTensor broadcast(const Shape& shp) const {   // p_shapeshifting.nim:76-94
    if ((int)shp.size() != rank()) throw std::invalid_argument("broadcast: ranks differ");
    HipTensor r = *this;
    for (int i = 0; i < rank(); ++i) {
      if (shape[i] == 1) {
        if (shp[i] != 1) { r.shape[i] = shp[i]; r.strides[i] = 0; }
      } else if (shape[i] != shp[i]) {
        throw std::invalid_argument("The broadcasted size of the tensor " + detail::str(shp) +
                                    ", must match existing size " + detail::str(shape) +
                                    " for non-singleton dimension");
      }
    }
    return r;
  }

  // ---- transfers ----------------------------------------------------------------------------
  // Blocking copy of the logical contents in C order (a device-side gather first if strided).
  std::vector<T> toCpu() const {
    if (std::is_same<T, uint8_t>::value && !is_C_contiguous())
      throw std::invalid_argument("toCpu: a strided view of a bool / uint8 tensor cannot be gathered on the device");
    const HipTensor c = is_C_contiguous() ? *this : clone();
    std::vector<T> host((size_t)size());
    if (!host.empty()) check(am_hip_memcpy_d2h(host.data(), c.ptr(), host.size() * sizeof(T)));
    return host;
  }
  HipTensor clone() const {
    HipTensor r(shape);
    if constexpr (std::is_same<T, uint8_t>::value) {
      if (!is_C_contiguous()) throw std::invalid_argument("clone: a strided view of a bool / uint8 tensor cannot be gathered on the device");
      if (size() > 0) check(am_hip_memcpy_d2d(r.ptr(), ptr(), (size_t)size()));
    } else {
      if (size() > 0) check(detail::unary_(AM_UOP_COPY, rank(), shape.data(), r.ptr(), r.strides.data(), ptr(), strides.data()));
    }
    return r;
  }
  // In-place clamp to [lo, hi] (mclamp, math_functions.nim:150-152); the bounds travel by value.
  HipTensor& mclamp(T lo, T hi) {
    if (size() > 0) check(detail::clamp_(rank(), shape.data(), ptr(), strides.data(), ptr(), strides.data(), lo, hi));
    return *this;
  }

  // ---- in-place forms -------------------------------------------------------------------------
  HipTensor& operator+=(const HipTensor& b) { return apply2(AM_OP_ADD, b); }
  HipTensor& operator-=(const HipTensor& b) { return apply2(AM_OP_SUB, b); }
  HipTensor& operator*=(T s) { return apply_scalar(AM_OP_MUL, s); }
  HipTensor& operator/=(T s) { return apply_scalar(AM_OP_DIV, s); }
  // only the right-hand side may be broadcast (operators_broadcasted.nim:65-102)
  HipTensor& bc_iadd(const HipTensor& b) { return apply2(AM_OP_ADD, b.broadcast(shape)); }
  HipTensor& bc_isub(const HipTensor& b) { return apply2(AM_OP_SUB, b.broadcast(shape)); }
  HipTensor& bc_imul(const HipTensor& b) { return apply2(AM_OP_MUL, b.broadcast(shape)); }
  HipTensor& bc_idiv(const HipTensor& b) { return apply2(AM_OP_DIV, b.broadcast(shape)); }
  // `^.=`: pow(x, exponent) in place, float tensors (operators_broadcasted.nim:178-182)
  HipTensor& bc_ipow(T exponent) { return apply_scalar(AM_OP_POW, exponent); }

  // apply2_inline (higher_order_applymap.nim:40-47) with an enumerated body.
  HipTensor& apply2(int op, const HipTensor& src) {
    if (shape != src.shape)
      throw std::invalid_argument("Both Tensors should have the same shape. Left-hand side has shape " +
                                  detail::str(shape) + " while right-hand side has shape " + detail::str(src.shape));
    if (size() > 0)
      check(detail::binary_(op, rank(), shape.data(), ptr(), strides.data(), ptr(), strides.data(), src.ptr(), src.strides.data()));
    return *this;
  }
  // Element-wise copy of a tensor of the same shape into this one's memory, through both tensors' strides
  // (the reference's copyFrom / slice assignment; a device-side pass, recordable into a graph).
  HipTensor& copy_from(const HipTensor& src) {
    if (shape != src.shape)
      throw std::invalid_argument("copy_from: shapes " + detail::str(shape) + " and " + detail::str(src.shape) + " differ");
    if (size() > 0) check(detail::unary_(AM_UOP_COPY, rank(), shape.data(), ptr(), strides.data(), src.ptr(), src.strides.data()));
    return *this;
  }
  HipTensor& apply_scalar(int op, T s) {
    if (size() > 0) check(detail::scalar_(op, 0, rank(), shape.data(), ptr(), strides.data(), ptr(), strides.data(), s));
    return *this;
  }
};

// ---- construction -----------------------------------------------------------------------------
template <typename T>
HipTensor<T> toHip(const T* host, const Shape& shape) {   // init_cuda.nim:23-41, row-major here
  HipTensor<T> t(shape);
  if (t.size() > 0) check(am_hip_memcpy_h2d(t.ptr(), host, (size_t)t.size() * sizeof(T)));
  return t;
}
template <typename T>
HipTensor<T> toHip(const std::vector<T>& host, const Shape& shape) {
  HipTensor<T> probe;   // shape check without allocating
  int64_t n = 1;
  for (auto s : shape) n *= s;
  if ((int64_t)host.size() != n) throw std::invalid_argument("toHip: " + std::to_string(host.size()) + " values for shape " + detail::str(shape));
  return toHip(host.data(), shape);
}

// broadcast(val, shape) (shapeshifting.nim:136-176): a tensor of `shape` whose every element is `val` - ONE element of
// storage, every stride 0. Not to be written through (all positions share the element); clone() materialises it.
template <typename T>
HipTensor<T> broadcast(T val, const Shape& shape) {
  if (shape.size() > AM_MAXRANK) throw std::invalid_argument("rank exceeds " + std::to_string(AM_MAXRANK));
  const HipTensor<T> one = toHip(&val, Shape{1});
  HipTensor<T> r;
  r.shape = shape;
  r.strides.assign(shape.size(), 0);
  r.storage = one.storage;
  return r;
}

// ---- map2 / operators ---------------------------------------------------------------------------
template <typename T>
HipTensor<T> map2(int op, const HipTensor<T>& a, const HipTensor<T>& b) {   // map2_inline, :92-120
  if (a.shape != b.shape)
    throw std::invalid_argument("Both Tensors should have the same shape. Left-hand side has shape " +
                                detail::str(a.shape) + " while right-hand side has shape " + detail::str(b.shape));
  HipTensor<T> r(a.shape);
  if (r.size() > 0)
    check(detail::binary_(op, r.rank(), r.shape.data(), r.ptr(), r.strides.data(), a.ptr(), a.strides.data(), b.ptr(), b.strides.data()));
  return r;
}
template <typename T>
HipTensor<T> scalar_op(int op, const HipTensor<T>& t, T s, bool scalar_on_left = false) {
  HipTensor<T> r(t.shape);
  if (r.size() > 0)
    check(detail::scalar_(op, scalar_on_left ? 1 : 0, r.rank(), r.shape.data(), r.ptr(), r.strides.data(), t.ptr(), t.strides.data(), s));
  return r;
}
template <typename T>
HipTensor<T> unary(int op, const HipTensor<T>& t) {
  HipTensor<T> r(t.shape);
  if (r.size() > 0) check(detail::unary_(op, r.rank(), r.shape.data(), r.ptr(), r.strides.data(), t.ptr(), t.strides.data()));
  return r;
}

template <typename T> HipTensor<T> operator+(const HipTensor<T>& a, const HipTensor<T>& b) { return map2(AM_OP_ADD, a, b); }
template <typename T> HipTensor<T> operator-(const HipTensor<T>& a, const HipTensor<T>& b) { return map2(AM_OP_SUB, a, b); }
template <typename T> HipTensor<T> operator*(const HipTensor<T>& t, T s) { return scalar_op(AM_OP_MUL, t, s); }
template <typename T> HipTensor<T> operator*(T s, const HipTensor<T>& t) { return scalar_op(AM_OP_MUL, t, s, true); }
template <typename T> HipTensor<T> operator/(const HipTensor<T>& t, T s) { return scalar_op(AM_OP_DIV, t, s); }
template <typename T> HipTensor<T> relu(const HipTensor<T>& t) { return unary(AM_UOP_RELU, t); }

// broadcast2Impl, p_shapeshifting.nim:96-134
template <typename T>
std::pair<HipTensor<T>, HipTensor<T>> broadcast2(const HipTensor<T>& a, const HipTensor<T>& b) {
  if (a.rank() != b.rank()) throw std::invalid_argument("Broadcasting error: ranks differ");
  HipTensor<T> ra = a, rb = b;
  for (int i = 0; i < a.rank(); ++i) {
    if (a.shape[i] == b.shape[i]) continue;
    if (a.shape[i] == 1) { ra.shape[i] = b.shape[i]; ra.strides[i] = 0; }
    else if (b.shape[i] == 1) { rb.shape[i] = a.shape[i]; rb.strides[i] = 0; }
    else
      throw std::invalid_argument("Broadcasting error: non-singleton dimensions must be the same in both tensors. "
                                  "Tensors' shapes were: " + detail::str(a.shape) + " and " + detail::str(b.shape));
  }
  return {ra, rb};
}
template <typename T> HipTensor<T> bc(int op, const HipTensor<T>& a, const HipTensor<T>& b) {
  auto p = broadcast2(a, b);
  return map2(op, p.first, p.second);
}
template <typename T> HipTensor<T> bc_add(const HipTensor<T>& a, const HipTensor<T>& b) { return bc(AM_OP_ADD, a, b); }   // +.
template <typename T> HipTensor<T> bc_sub(const HipTensor<T>& a, const HipTensor<T>& b) { return bc(AM_OP_SUB, a, b); }   // -.
template <typename T> HipTensor<T> bc_mul(const HipTensor<T>& a, const HipTensor<T>& b) { return bc(AM_OP_MUL, a, b); }   // *.
template <typename T> HipTensor<T> bc_div(const HipTensor<T>& a, const HipTensor<T>& b) { return bc(AM_OP_DIV, a, b); }   // /.
template <typename T> HipTensor<T> bc_mod(const HipTensor<T>& a, const HipTensor<T>& b) { return bc(AM_OP_MOD, a, b); }   // mod
template <typename T> HipTensor<T> bc_add(const HipTensor<T>& t, T s) { return scalar_op(AM_OP_ADD, t, s); }
template <typename T> HipTensor<T> bc_add(T s, const HipTensor<T>& t) { return scalar_op(AM_OP_ADD, t, s, true); }
template <typename T> HipTensor<T> bc_sub(const HipTensor<T>& t, T s) { return scalar_op(AM_OP_SUB, t, s); }
template <typename T> HipTensor<T> bc_sub(T s, const HipTensor<T>& t) { return scalar_op(AM_OP_SUB, t, s, true); }
template <typename T> HipTensor<T> bc_mul(const HipTensor<T>& t, T s) { return scalar_op(AM_OP_MUL, t, s); }
template <typename T> HipTensor<T> bc_mul(T s, const HipTensor<T>& t) { return scalar_op(AM_OP_MUL, t, s, true); }
template <typename T> HipTensor<T> bc_div(const HipTensor<T>& t, T s) { return scalar_op(AM_OP_DIV, t, s); }
template <typename T> HipTensor<T> bc_div(T s, const HipTensor<T>& t) { return scalar_op(AM_OP_DIV, t, s, true); }
// `^.`: tensor ^. exponent and base ^. tensor, float tensors (operators_broadcasted.nim:153-161)
template <typename T> HipTensor<T> bc_pow(const HipTensor<T>& t, T exponent) { return scalar_op(AM_OP_POW, t, exponent); }
template <typename T> HipTensor<T> bc_pow(T base, const HipTensor<T>& t) { return scalar_op(AM_OP_POW, t, base, true); }
// ---- map bodies whose result type differs from the operands' --------------------------------------
// The reference's map templates infer the result type (higher_order_applymap.nim:69-120); a bool result
// is a HipTensor<uint8_t> here (one byte per element, 0 / 1).
template <typename T>
HipTensor<uint8_t> map2_bool(int cmp, const HipTensor<T>& a, const HipTensor<T>& b) {
  if (a.shape != b.shape)
    throw std::invalid_argument("Both Tensors should have the same shape. Left-hand side has shape " +
                                detail::str(a.shape) + " while right-hand side has shape " + detail::str(b.shape));
  HipTensor<uint8_t> r(a.shape);
  if (r.size() > 0)
    check(detail::compare_(cmp, r.rank(), r.shape.data(), r.ptr(), r.strides.data(), a.ptr(), a.strides.data(), b.ptr(), b.strides.data()));
  return r;
}
template <typename T>
HipTensor<uint8_t> compare_scalar(int cmp, const HipTensor<T>& t, T value) {
  HipTensor<uint8_t> r(t.shape);   // returnEmptyIfEmpty: an empty tensor comes back empty
  if (r.size() > 0)
    check(detail::compare_scalar_(cmp, r.rank(), r.shape.data(), r.ptr(), r.strides.data(), t.ptr(), t.strides.data(), value));
  return r;
}
// `==.` `!=.` `<.` `<=.` `>.` `>=.` (operators_comparison.nim:41-185): tensor-tensor with implicit
// broadcasting, tensor-scalar, and scalar-tensor (the mirrored tensor-scalar comparison, as in the reference).
#define AM_HIP_COMPARISON(name, code, mirrored)                                                                  \
  template <typename T> HipTensor<uint8_t> name(const HipTensor<T>& a, const HipTensor<T>& b) {                  \
    auto p = broadcast2(a, b);                                                                                   \
    return map2_bool(code, p.first, p.second);                                                                   \
  }                                                                                                              \
  template <typename T> HipTensor<uint8_t> name(const HipTensor<T>& t, T value) { return compare_scalar(code, t, value); } \
  template <typename T> HipTensor<uint8_t> name(T value, const HipTensor<T>& t) { return compare_scalar(mirrored, t, value); }
AM_HIP_COMPARISON(bc_eq, AM_CMP_EQ, AM_CMP_EQ) AM_HIP_COMPARISON(bc_ne, AM_CMP_NE, AM_CMP_NE)
AM_HIP_COMPARISON(bc_lt, AM_CMP_LT, AM_CMP_GT) AM_HIP_COMPARISON(bc_le, AM_CMP_LE, AM_CMP_GE)
AM_HIP_COMPARISON(bc_gt, AM_CMP_GT, AM_CMP_LT) AM_HIP_COMPARISON(bc_ge, AM_CMP_GE, AM_CMP_LE)
#undef AM_HIP_COMPARISON
template <typename T> HipTensor<uint8_t> predicate(int op, const HipTensor<T>& t) {
  static_assert(std::is_floating_point<T>::value, "isNaN / isNotNaN / classify are defined for float tensors");
  HipTensor<uint8_t> r(t.shape);
  if (r.size() > 0) check(detail::predicate_(op, r.rank(), r.shape.data(), r.ptr(), r.strides.data(), t.ptr(), t.strides.data()));
  return r;
}
template <typename T> HipTensor<uint8_t> isNaN(const HipTensor<T>& t) { return predicate(AM_PRED_ISNAN, t); }        // operators_comparison.nim:192-198
template <typename T> HipTensor<uint8_t> isNotNaN(const HipTensor<T>& t) { return predicate(AM_PRED_ISNOTNAN, t); }  // :200-206
// Ordinals of Nim's FloatClass: 0 fcNormal, 1 fcSubnormal, 2 fcZero, 3 fcNegZero, 4 fcNan, 5 fcInf, 6 fcNegInf (math_functions.nim:264-276)
template <typename T> HipTensor<uint8_t> classify(const HipTensor<T>& t) { return predicate(AM_PRED_CLASSIFY, t); }
// -1 / 0 / 1 as the reference's Tensor[int]; zeros and NaN give 0 (math_functions.nim:110-117)
template <typename T> HipTensor<int64_t> sgn(const HipTensor<T>& t) {
  HipTensor<int64_t> r(t.shape);
  if (r.size() > 0) check(detail::sgn_(r.rank(), r.shape.data(), r.ptr(), r.strides.data(), t.ptr(), t.strides.data()));
  return r;
}
// clamp (math_functions.nim:146-148): one pass, bounds by value
template <typename T> HipTensor<T> clamp(const HipTensor<T>& t, T lo, T hi) {
  HipTensor<T> r(t.shape);
  if (r.size() > 0) check(detail::clamp_(r.rank(), r.shape.data(), r.ptr(), r.strides.data(), t.ptr(), t.strides.data(), lo, hi));
  return r;
}
// floorMod (math_functions.nim:134-144) and copySign (:119-125)
template <typename T> HipTensor<T> floorMod(const HipTensor<T>& a, const HipTensor<T>& b) { return map2(AM_OP_FLOORMOD, a, b); }
template <typename T> HipTensor<T> floorMod(const HipTensor<T>& t, T value) { return scalar_op(AM_OP_FLOORMOD, t, value); }
template <typename T> HipTensor<T> floorMod(T value, const HipTensor<T>& t) { return scalar_op(AM_OP_FLOORMOD, t, value, true); }
template <typename T> HipTensor<T> copySign(const HipTensor<T>& a, const HipTensor<T>& b) { return map2(AM_OP_COPYSIGN, a, b); }

// The universal functions (ufunc.nim:82-130) and reciprocal (math_functions.nim:52-58), float tensors.
#define AM_HIP_UFUNC(name, code) \
  template <typename T> HipTensor<T> name(const HipTensor<T>& t) { return unary(code, t); }
AM_HIP_UFUNC(ln, AM_UOP_LN) AM_HIP_UFUNC(log10, AM_UOP_LOG10) AM_HIP_UFUNC(log2, AM_UOP_LOG2) AM_HIP_UFUNC(exp, AM_UOP_EXP)
AM_HIP_UFUNC(sin, AM_UOP_SIN) AM_HIP_UFUNC(cos, AM_UOP_COS) AM_HIP_UFUNC(tan, AM_UOP_TAN)
AM_HIP_UFUNC(sinh, AM_UOP_SINH) AM_HIP_UFUNC(cosh, AM_UOP_COSH) AM_HIP_UFUNC(tanh, AM_UOP_TANH)
AM_HIP_UFUNC(arcsin, AM_UOP_ARCSIN) AM_HIP_UFUNC(arccos, AM_UOP_ARCCOS) AM_HIP_UFUNC(arctan, AM_UOP_ARCTAN)
AM_HIP_UFUNC(arcsinh, AM_UOP_ARCSINH) AM_HIP_UFUNC(arccosh, AM_UOP_ARCCOSH) AM_HIP_UFUNC(arctanh, AM_UOP_ARCTANH)
AM_HIP_UFUNC(cbrt, AM_UOP_CBRT) AM_HIP_UFUNC(erf, AM_UOP_ERF) AM_HIP_UFUNC(erfc, AM_UOP_ERFC)
AM_HIP_UFUNC(gamma, AM_UOP_GAMMA) AM_HIP_UFUNC(lgamma, AM_UOP_LGAMMA)
AM_HIP_UFUNC(floor, AM_UOP_FLOOR) AM_HIP_UFUNC(ceil, AM_UOP_CEIL) AM_HIP_UFUNC(trunc, AM_UOP_TRUNC)
AM_HIP_UFUNC(round, AM_UOP_ROUND) AM_HIP_UFUNC(reciprocal, AM_UOP_RECIPROCAL)
AM_HIP_UFUNC(degToRad, AM_UOP_DEGTORAD) AM_HIP_UFUNC(radToDeg, AM_UOP_RADTODEG)
#undef AM_HIP_UFUNC
// fac (ufunc.nim:84-85): n! of every element of an integer tensor; Nim's table covers 0 .. 20 and asserts outside it.
template <typename T> HipTensor<T> fac(const HipTensor<T>& t) {
  static_assert(std::is_integral<T>::value, "fac is defined for integer tensors");
  if (t.size() > 0 && (min(t) < T(0) || max(t) > T(20))) throw std::out_of_range("fac: every element must lie in 0 .. 20");
  return unary(AM_UOP_FAC, t);
}
// map2_inline(x, b.broadcast(x.shape), max(0, x + y)) in one pass
template <typename T> HipTensor<T> bias_relu(const HipTensor<T>& x, const HipTensor<T>& b) { return map2(AM_OP_ADD_RELU, x, b.broadcast(x.shape)); }
// Activation backward passes: map2_inline(cached_tensor, gradient) bodies of nnp_activation.nim:61-74.
template <typename T> HipTensor<T> relu_backward(const HipTensor<T>& gradient, const HipTensor<T>& cached) { return map2(AM_OP_RELU_BWD, cached, gradient); }
template <typename T> HipTensor<T> sigmoid_backward(const HipTensor<T>& gradient, const HipTensor<T>& cached) { return map2(AM_OP_SIGMOID_BWD, cached, gradient); }
template <typename T> HipTensor<T> tanh_backward(const HipTensor<T>& gradient, const HipTensor<T>& cached) { return map2(AM_OP_TANH_BWD, cached, gradient); }

// ---- GEMM -----------------------------------------------------------------------------------------
// C <- alpha A B + beta C (operators_blas_l2l3.nim:58-81); any strides on A, B and C.
template <typename T>
void gemm(T alpha, const HipTensor<T>& A, const HipTensor<T>& B, T beta, HipTensor<T>& C) {
  if (A.rank() != 2 || B.rank() != 2 || C.rank() != 2) throw std::invalid_argument("gemm: A, B and C must be matrices");
  if (A.shape[1] != B.shape[0])   // check_matmat -> IndexDefect (p_checks.nim:159-167)
    throw std::out_of_range("Number of columns in the first matrix: " + std::to_string(A.shape[1]) +
                            ", must be the same as the number of rows in the second matrix: " + std::to_string(B.shape[0]));
  if (C.shape[0] != A.shape[0] || C.shape[1] != B.shape[1]) throw std::out_of_range("gemm: C has the wrong shape " + detail::str(C.shape));
  check(detail::gemm_(A.shape[0], B.shape[1], A.shape[1], alpha, A.ptr(), A.strides[0], A.strides[1], B.ptr(),
                      B.strides[0], B.strides[1], beta, C.ptr(), C.strides[0], C.strides[1]));
}

// y <- alpha A x + beta y (operators_blas_l2l3.nim:24-56)
// Digit planes of an integer matrix split once for products that reuse it (a weight matrix). No counterpart in the
// reference, whose gemm_strided packs both operands in every call (gemm_packing.nim:24-99). A snapshot of the matrix.
class DigitPlanes {
 public:
  DigitPlanes() = default;
  template <typename T>
  DigitPlanes(const HipTensor<T>& t, bool right_operand) {
    static_assert(std::is_same<T, int32_t>::value || std::is_same<T, int64_t>::value, "digit planes belong to int32_t / int64_t matrices");
    if (t.rank() != 2) throw std::invalid_argument("DigitPlanes: the operand must be a matrix");
    if constexpr (std::is_same<T, int32_t>::value)
      check(am_hip_digits_prepare_i32(right_operand ? 1 : 0, t.shape[0], t.shape[1], t.ptr(), t.strides[0], t.strides[1], &handle_));
    else
      check(am_hip_digits_prepare_i64(right_operand ? 1 : 0, t.shape[0], t.shape[1], t.ptr(), t.strides[0], t.strides[1], &handle_));
  }
  ~DigitPlanes() { (void)am_hip_digits_release(handle_); }
  DigitPlanes(const DigitPlanes&) = delete;
  DigitPlanes& operator=(const DigitPlanes&) = delete;
  DigitPlanes(DigitPlanes&& o) noexcept : handle_(o.handle_) { o.handle_ = nullptr; }
  DigitPlanes& operator=(DigitPlanes&& o) noexcept {
    if (this != &o) { (void)am_hip_digits_release(handle_); handle_ = o.handle_; o.handle_ = nullptr; }
    return *this;
  }
  void* handle() const { return handle_; }

 private:
  void* handle_ = nullptr;
};

// gemm with the digit planes of A and / or B split ahead of time (nullptr: split that operand in the call).
inline void gemm(int32_t alpha, const HipTensor<int32_t>& A, const HipTensor<int32_t>& B, int32_t beta, HipTensor<int32_t>& C,
                 const DigitPlanes* a_digits, const DigitPlanes* b_digits) {
  if (A.rank() != 2 || B.rank() != 2 || C.rank() != 2) throw std::invalid_argument("gemm: A, B and C must be matrices");
  if (A.shape[1] != B.shape[0] || C.shape[0] != A.shape[0] || C.shape[1] != B.shape[1]) throw std::out_of_range("gemm: shapes do not agree");
  check(am_hip_gemm_prepared_i32(A.shape[0], B.shape[1], A.shape[1], alpha, A.ptr(), A.strides[0], A.strides[1],
                                 a_digits ? a_digits->handle() : nullptr, B.ptr(), B.strides[0], B.strides[1],
                                 b_digits ? b_digits->handle() : nullptr, beta, C.ptr(), C.strides[0], C.strides[1]));
}
inline void gemm(int64_t alpha, const HipTensor<int64_t>& A, const HipTensor<int64_t>& B, int64_t beta, HipTensor<int64_t>& C,
                 const DigitPlanes* a_digits, const DigitPlanes* b_digits) {
  if (A.rank() != 2 || B.rank() != 2 || C.rank() != 2) throw std::invalid_argument("gemm: A, B and C must be matrices");
  if (A.shape[1] != B.shape[0] || C.shape[0] != A.shape[0] || C.shape[1] != B.shape[1]) throw std::out_of_range("gemm: shapes do not agree");
  check(am_hip_gemm_prepared_i64(A.shape[0], B.shape[1], A.shape[1], alpha, A.ptr(), A.strides[0], A.strides[1],
                                 a_digits ? a_digits->handle() : nullptr, B.ptr(), B.strides[0], B.strides[1],
                                 b_digits ? b_digits->handle() : nullptr, beta, C.ptr(), C.strides[0], C.strides[1]));
}

template <typename T>
void gemv(T alpha, const HipTensor<T>& A, const HipTensor<T>& x, T beta, HipTensor<T>& y) {
  if (A.rank() != 2 || x.rank() != 1 || y.rank() != 1) throw std::invalid_argument("gemv: A must be a matrix, x and y vectors");
  if (A.shape[1] != x.shape[0] || A.shape[0] != y.shape[0])
    throw std::out_of_range("Number of columns in the matrix: " + std::to_string(A.shape[1]) +
                            ", must be the same as the number of rows in the vector: " + std::to_string(x.shape[0]));
  check(detail::gemv_(A.shape[0], A.shape[1], alpha, A.ptr(), A.strides[0], A.strides[1], x.ptr(), x.strides[0], beta,
                      y.ptr(), y.strides[0]));
}

// Scalar product, returned to the host (operators_blas_l1.nim:27-38).
template <typename T>
T dot(const HipTensor<T>& a, const HipTensor<T>& b) {
  if (a.rank() != 1 || b.rank() != 1 || a.shape != b.shape) throw std::invalid_argument("dot: vectors of equal length expected");
  T r{};
  check(detail::dot_(a.shape[0], a.ptr(), a.strides[0], b.ptr(), b.strides[0], &r));
  return r;
}

// `*` (operators_blas_l2l3.nim:88-100): matrix-matrix, or matrix-vector.
template <typename T>
HipTensor<T> operator*(const HipTensor<T>& a, const HipTensor<T>& b) {
  if (a.rank() == 2 && b.rank() == 2) {
    if (a.shape[1] != b.shape[0])
      throw std::out_of_range("Number of columns in the first matrix: " + std::to_string(a.shape[1]) +
                              ", must be the same as the number of rows in the second matrix: " + std::to_string(b.shape[0]));
    HipTensor<T> r(Shape{a.shape[0], b.shape[1]});
    gemm(T(1), a, b, T(0), r);
    return r;
  }
  if (a.rank() == 2 && b.rank() == 1) {
    HipTensor<T> r(Shape{a.shape[0]});
    gemv(T(1), a, b, T(0), r);
    return r;
  }
  throw std::invalid_argument("Matrix-Matrix or Matrix-Vector multiplication valid only if first Tensor is a Matrix "
                              "and second is a Matrix or Vector");
}

// out = x * weight^T +. bias (then ReLU) as ONE kernel: nnp_linear.nim:20-29 + nnp_activation.nim:35-36.
template <typename T>
HipTensor<T> linear(const HipTensor<T>& x, const HipTensor<T>& weight, const HipTensor<T>& bias, bool with_relu = false) {
  static_assert(std::is_floating_point<T>::value, "linear is defined for float tensors");
  HipTensor<T> r(Shape{x.shape[0], weight.shape[0]});
  const HipTensor<T> wt = weight.transpose(), bb = bias.broadcast(r.shape);
  if (x.shape[1] != wt.shape[0]) throw std::out_of_range("linear: inner dimensions differ");
  check(detail::gemm_ex_(x.shape[0], wt.shape[1], x.shape[1], T(1), x.ptr(), x.strides[0], x.strides[1], wt.ptr(),
                         wt.strides[0], wt.strides[1], T(0), r.ptr(), r.strides[0], r.strides[1],
                         with_relu ? AM_EPI_BIAS_RELU : AM_EPI_BIAS, bb.ptr(), bb.strides[0], bb.strides[1]));
  return r;
}

// gru_cell_inference (nn_primitives/nnp_gru.nim:40-88): h(t) -> h'(t) in place. Two dense layers with their bias in the
// GEMM epilogue, then steps 2-4 (three apply2 / apply3 passes over column slices in the reference) as one launch.
// `saved`, when given, receives {r, z, n, Uh} for the backward pass (gru_cell_forward, nnp_gru.nim:90-146).
namespace detail {
inline int gru_gates_(int64_t b, int64_t h, const float* w, int64_t lw, const float* u, int64_t lu, float* hid, int64_t lh, float* r,
                      float* z, float* n, float* uh, int64_t ls) {
  return am_hip_gru_gates_f32(b, h, w, lw, u, lu, hid, lh, r, z, n, uh, ls);
}
inline int gru_gates_(int64_t b, int64_t h, const double* w, int64_t lw, const double* u, int64_t lu, double* hid, int64_t lh, double* r,
                      double* z, double* n, double* uh, int64_t ls) {
  return am_hip_gru_gates_f64(b, h, w, lw, u, lu, hid, lh, r, z, n, uh, ls);
}
}  // namespace detail
template <typename T>
void gru_cell_inference(const HipTensor<T>& input, const HipTensor<T>& W3, const HipTensor<T>& U3, const HipTensor<T>& bW3,
                        const HipTensor<T>& bU3, HipTensor<T>& hidden, std::vector<HipTensor<T>>* saved = nullptr) {
  if (hidden.rank() != 2 || hidden.strides[1] != 1) throw std::invalid_argument("gru_cell_inference: hidden must be [batch, H] with unit-stride rows");
  const int64_t B = hidden.shape[0], H = hidden.shape[1];
  if (W3.shape[0] != 3 * H || U3.shape[0] != 3 * H || U3.shape[1] != H) throw std::invalid_argument("gru_cell_inference: weights must be [3H, features] and [3H, H]");
  const HipTensor<T> W3x = linear(input, W3, bW3), U3h = linear(hidden, U3, bU3);
  T *r = nullptr, *z = nullptr, *n = nullptr, *uh = nullptr;
  if (saved) {
    saved->assign(4, HipTensor<T>());
    for (auto& t : *saved) t = HipTensor<T>(Shape{B, H});
    r = (*saved)[0].ptr(); z = (*saved)[1].ptr(); n = (*saved)[2].ptr(); uh = (*saved)[3].ptr();
  }
  check(detail::gru_gates_(B, H, W3x.ptr(), W3x.strides[0], U3h.ptr(), U3h.strides[0], hidden.ptr(), hidden.strides[0], r, z, n, uh, H));
}

// Fold along `axis`; the result keeps the axis with extent 1 (reduce_axis_inline,
// higher_order_foldreduce.nim:46-61). op: AM_RED_SUM / PROD / MIN / MAX.
template <typename T>
HipTensor<T> reduce_axis(int op, const HipTensor<T>& t, int axis) {
  if (axis < 0 || axis >= t.rank())
    throw std::out_of_range("Input tensor rank (" + std::to_string(t.rank()) + ") must be greater than reduction axis (" +
                            std::to_string(axis) + ")");
  if (t.size() == 0) return HipTensor<T>(t.shape);   // returnEmptyIfEmpty
  Shape sh = t.shape;
  sh[axis] = 1;
  HipTensor<T> r(sh);
  check(detail::reduce_axis_(op, t.rank(), t.shape.data(), axis, r.ptr(), r.strides.data(), t.ptr(), t.strides.data()));
  return r;
}

// Fold of every element, returned to the host (reduce_inline, higher_order_foldreduce.nim:22-31).
template <typename T>
T reduce_all(int op, const HipTensor<T>& t) {
  T r{};
  check(detail::reduce_all_(op, t.rank(), t.shape.data(), t.ptr(), t.strides.data(), &r));
  return r;
}

// aggregate.nim:33-113
template <typename T> T sum(const HipTensor<T>& t) { return reduce_all(AM_RED_SUM, t); }
template <typename T> HipTensor<T> sum(const HipTensor<T>& t, int axis) { return reduce_axis(AM_RED_SUM, t, axis); }
template <typename T> T product(const HipTensor<T>& t) { return reduce_all(AM_RED_PROD, t); }
template <typename T> HipTensor<T> product(const HipTensor<T>& t, int axis) { return reduce_axis(AM_RED_PROD, t, axis); }
template <typename T> T min(const HipTensor<T>& t) { return reduce_all(AM_RED_MIN, t); }
template <typename T> HipTensor<T> min(const HipTensor<T>& t, int axis) { return reduce_axis(AM_RED_MIN, t, axis); }
template <typename T> T max(const HipTensor<T>& t) { return reduce_all(AM_RED_MAX, t); }
template <typename T> HipTensor<T> max(const HipTensor<T>& t, int axis) { return reduce_axis(AM_RED_MAX, t, axis); }

// gradInput = gradOutput * weight, gradWeight = gradOutput^T * input (the transposed view reaches
// the GEMM as strides), gradBias = sum(gradOutput, axis 0): nnp_linear.nim:39-66.
template <typename T> struct LinearGrads { HipTensor<T> input, weight, bias; };
template <typename T>
LinearGrads<T> linear_backward(const HipTensor<T>& input, const HipTensor<T>& weight, const HipTensor<T>& grad_output) {
  return {grad_output * weight, grad_output.transpose() * input, sum(grad_output, 0)};
}
// integers: C++ `/` truncates towards zero like Nim's `div`
template <typename T> T mean(const HipTensor<T>& t) { return sum(t) / static_cast<T>(t.size()); }
template <typename T> HipTensor<T> mean(const HipTensor<T>& t, int axis) {
  HipTensor<T> s = sum(t, axis);
  if (s.size() == 0) return s;
  return scalar_op(AM_OP_DIV, s, static_cast<T>(t.shape[axis]));
}

// (indices, values) of the first maximum / minimum along an axis (argmax_max / argmin_min,
// aggregate.nim:159-193, 216-250); indices are int64, both keep the axis with extent 1.
template <typename T>
std::pair<HipTensor<int64_t>, HipTensor<T>> argreduce(int op, const HipTensor<T>& t, int axis) {
  if (axis < 0 || axis >= t.rank())
    throw std::out_of_range("Input tensor rank (" + std::to_string(t.rank()) + ") must be greater than reduction axis (" +
                            std::to_string(axis) + ")");
  Shape shape = t.shape;
  if (t.size() != 0) shape[axis] = 1;
  HipTensor<int64_t> idx(shape);
  HipTensor<T> val(shape);
  if (t.size() != 0)
    check(detail::argreduce_(op, t.rank(), t.shape.data(), axis, idx.ptr(), idx.strides.data(), val.ptr(), val.strides.data(),
                             t.ptr(), t.strides.data()));
  return {idx, val};
}
template <typename T> std::pair<HipTensor<int64_t>, HipTensor<T>> argmax_max(const HipTensor<T>& t, int axis) { return argreduce(AM_RED_MAX, t, axis); }
template <typename T> std::pair<HipTensor<int64_t>, HipTensor<T>> argmin_min(const HipTensor<T>& t, int axis) { return argreduce(AM_RED_MIN, t, axis); }
template <typename T> HipTensor<int64_t> argmax(const HipTensor<T>& t, int axis) { return argreduce(AM_RED_MAX, t, axis).first; }
template <typename T> HipTensor<int64_t> argmin(const HipTensor<T>& t, int axis) { return argreduce(AM_RED_MIN, t, axis).first; }

template <typename T> HipTensor<T> sqrt(const HipTensor<T>& t) { return unary(AM_UOP_SQRT, t); }      // ufunc.nim:91
template <typename T> HipTensor<T> square(const HipTensor<T>& t) { return unary(AM_UOP_SQUARE, t); }  // math_functions.nim:218-222
// Sample variance, normalised by n - 1, and its square root (aggregate.nim:115-158): the mean, then the
// sum of square(y - mean).
template <typename T> T variance(const HipTensor<T>& t) {
  static_assert(std::is_floating_point<T>::value, "variance is defined for float tensors");
  return sum(square(scalar_op(AM_OP_SUB, t, mean(t)))) / static_cast<T>(t.size() - 1);
}
template <typename T> HipTensor<T> variance(const HipTensor<T>& t, int axis) {
  static_assert(std::is_floating_point<T>::value, "variance is defined for float tensors");
  HipTensor<T> m = mean(t, axis);
  if (m.size() == 0) return m;
  return scalar_op(AM_OP_DIV, sum(map2(AM_OP_SQDIFF, t, m.broadcast(t.shape)), axis), static_cast<T>(t.shape[axis] - 1));
}
template <typename T> T stddev(const HipTensor<T>& t) { return std::sqrt(variance(t)); }
template <typename T> HipTensor<T> stddev(const HipTensor<T>& t, int axis) {
  HipTensor<T> v = variance(t, axis);
  return v.size() == 0 ? v : sqrt(v);
}

// Row softmax of a [batch_size, number_of_classes] matrix (nnp_softmax.nim:18-38).
template <typename T>
HipTensor<T> softmax(const HipTensor<T>& t) {
  static_assert(std::is_floating_point<T>::value, "softmax is defined for float tensors");
  if (t.rank() != 2) throw std::invalid_argument("softmax: input must be [batch_size, number_of_classes]");
  HipTensor<T> r(t.shape);
  check(detail::softmax_(t.shape[0], t.shape[1], r.ptr(), r.strides[0], r.strides[1], t.ptr(), t.strides[0], t.strides[1]));
  return r;
}

// Softmax + cross-entropy in one pass, averaged over the batch, and its gradient
// (nn_primitives/nnp_softmax_cross_entropy.nim:17-86, 88-177, 186-214, 217-256). The dense forms take probabilities
// [batch_size, classes], the sparse forms one int64 class index per row.
namespace detail {
#define AM_HPP_LOSS(T, SFX)                                                                                                   \
  inline int sce_(int64_t r, int64_t c, const T* x, int64_t xr, int64_t xc, const T* t, int64_t tr, int64_t tc, T* loss) {    \
    return am_hip_softmax_cross_entropy_##SFX(r, c, x, xr, xc, t, tr, tc, loss);                                              \
  }                                                                                                                           \
  inline int sparse_sce_(int64_t r, int64_t c, const T* x, int64_t xr, int64_t xc, const int64_t* l, int64_t ls, T* loss) {   \
    return am_hip_sparse_softmax_cross_entropy_##SFX(r, c, x, xr, xc, l, ls, loss);                                           \
  }                                                                                                                           \
  inline int sce_bwd_(int64_t r, int64_t c, T g, const T* x, int64_t xr, int64_t xc, const T* t, int64_t tr, int64_t tc,      \
                      T* o, int64_t orr, int64_t oc) {                                                                        \
    return am_hip_softmax_cross_entropy_backward_##SFX(r, c, g, x, xr, xc, t, tr, tc, o, orr, oc);                            \
  }                                                                                                                           \
  inline int sparse_sce_bwd_(int64_t r, int64_t c, T g, const T* x, int64_t xr, int64_t xc, const int64_t* l, int64_t ls,     \
                             T* o, int64_t orr, int64_t oc) {                                                                 \
    return am_hip_sparse_softmax_cross_entropy_backward_##SFX(r, c, g, x, xr, xc, l, ls, o, orr, oc);                         \
  }
AM_HPP_LOSS(float, f32)
AM_HPP_LOSS(double, f64)
#undef AM_HPP_LOSS
}  // namespace detail

template <typename T>
T softmax_cross_entropy(const HipTensor<T>& input, const HipTensor<T>& target) {
  if (input.rank() != 2 || input.shape != target.shape)
    throw std::invalid_argument("softmax_cross_entropy: input " + detail::str(input.shape) + " and target " + detail::str(target.shape) +
                                " must be matrices of the same shape");
  T loss = T(0);
  check(detail::sce_(input.shape[0], input.shape[1], input.ptr(), input.strides[0], input.strides[1], target.ptr(), target.strides[0],
                     target.strides[1], &loss));
  return loss;
}
template <typename T>
T sparse_softmax_cross_entropy(const HipTensor<T>& input, const HipTensor<int64_t>& target) {
  if (input.rank() != 2 || target.rank() != 1 || target.shape[0] != input.shape[0])
    throw std::invalid_argument("sparse_softmax_cross_entropy: one label per row of the input is needed");
  T loss = T(0);
  check(detail::sparse_sce_(input.shape[0], input.shape[1], input.ptr(), input.strides[0], input.strides[1], target.ptr(),
                            target.strides[0], &loss));
  return loss;
}
template <typename T>
HipTensor<T> softmax_cross_entropy_backward(T gradient, const HipTensor<T>& cached_tensor, const HipTensor<T>& target) {
  if (cached_tensor.rank() != 2 || cached_tensor.shape != target.shape)
    throw std::invalid_argument("softmax_cross_entropy_backward: input and target must be matrices of the same shape");
  HipTensor<T> r(cached_tensor.shape);
  check(detail::sce_bwd_(cached_tensor.shape[0], cached_tensor.shape[1], gradient, cached_tensor.ptr(), cached_tensor.strides[0],
                         cached_tensor.strides[1], target.ptr(), target.strides[0], target.strides[1], r.ptr(), r.strides[0], r.strides[1]));
  return r;
}
template <typename T>
HipTensor<T> sparse_softmax_cross_entropy_backward(T gradient, const HipTensor<T>& cached_tensor, const HipTensor<int64_t>& target) {
  if (cached_tensor.rank() != 2 || target.rank() != 1 || target.shape[0] != cached_tensor.shape[0])
    throw std::invalid_argument("sparse_softmax_cross_entropy_backward: one label per row of the input is needed");
  HipTensor<T> r(cached_tensor.shape);
  check(detail::sparse_sce_bwd_(cached_tensor.shape[0], cached_tensor.shape[1], gradient, cached_tensor.ptr(), cached_tensor.strides[0],
                                cached_tensor.strides[1], target.ptr(), target.strides[0], r.ptr(), r.strides[0], r.strides[1]));
  return r;
}

// Sigmoid + binary cross-entropy averaged over the batch, and its gradient (nnp_sigmoid_cross_entropy.nim:23-62).
namespace detail {
inline int sigmoid_ce_(int64_t r, int64_t c, const float* x, int64_t xr, int64_t xc, const float* t, int64_t tr, int64_t tc, float* l) {
  return am_hip_sigmoid_cross_entropy_f32(r, c, x, xr, xc, t, tr, tc, l);
}
inline int sigmoid_ce_(int64_t r, int64_t c, const double* x, int64_t xr, int64_t xc, const double* t, int64_t tr, int64_t tc, double* l) {
  return am_hip_sigmoid_cross_entropy_f64(r, c, x, xr, xc, t, tr, tc, l);
}
inline int sigmoid_ce_bwd_(int64_t r, int64_t c, float g, const float* x, int64_t xr, int64_t xc, const float* t, int64_t tr, int64_t tc,
                           float* o, int64_t orr, int64_t oc) {
  return am_hip_sigmoid_cross_entropy_backward_f32(r, c, g, x, xr, xc, t, tr, tc, o, orr, oc);
}
inline int sigmoid_ce_bwd_(int64_t r, int64_t c, double g, const double* x, int64_t xr, int64_t xc, const double* t, int64_t tr, int64_t tc,
                           double* o, int64_t orr, int64_t oc) {
  return am_hip_sigmoid_cross_entropy_backward_f64(r, c, g, x, xr, xc, t, tr, tc, o, orr, oc);
}
inline int sgd_(int n, float* const* v, const float* const* g, const int64_t* s, float lr) { return am_hip_sgd_update_f32(n, v, g, s, lr); }
inline int sgd_(int n, double* const* v, const double* const* g, const int64_t* s, double lr) { return am_hip_sgd_update_f64(n, v, g, s, lr); }
}  // namespace detail
template <typename T>
T sigmoid_cross_entropy(const HipTensor<T>& input, const HipTensor<T>& target) {
  if (input.rank() != 2 || input.shape != target.shape || input.shape[0] == 0)
    throw std::invalid_argument("sigmoid_cross_entropy: input and target must be non-empty matrices of the same shape");
  T loss = T(0);
  check(detail::sigmoid_ce_(input.shape[0], input.shape[1], input.ptr(), input.strides[0], input.strides[1], target.ptr(),
                            target.strides[0], target.strides[1], &loss));
  return loss;
}
template <typename T>
HipTensor<T> sigmoid_cross_entropy_backward(T gradient, const HipTensor<T>& cached_tensor, const HipTensor<T>& target) {
  if (cached_tensor.rank() != 2 || cached_tensor.shape != target.shape)
    throw std::invalid_argument("sigmoid_cross_entropy_backward: input and target must be matrices of the same shape");
  HipTensor<T> r(cached_tensor.shape);
  check(detail::sigmoid_ce_bwd_(cached_tensor.shape[0], cached_tensor.shape[1], gradient, cached_tensor.ptr(), cached_tensor.strides[0],
                                cached_tensor.strides[1], target.ptr(), target.strides[0], target.strides[1], r.ptr(), r.strides[0], r.strides[1]));
  return r;
}

// value -= learning_rate * gradient for every pair in ONE launch: the SGD optimizer's update
// (nn/optimizers/optimizers.nim:35-51 runs one apply2_inline per parameter). C-contiguous tensors.
template <typename T>
void sgd_update(const std::vector<HipTensor<T>*>& values, const std::vector<const HipTensor<T>*>& gradients, T learning_rate) {
  if (values.size() != gradients.size()) throw std::invalid_argument("sgd_update: one gradient per value");
  std::vector<T*> v;
  std::vector<const T*> g;
  std::vector<int64_t> n;
  for (size_t i = 0; i < values.size(); ++i) {
    if (values[i]->shape != gradients[i]->shape || !values[i]->is_C_contiguous() || !gradients[i]->is_C_contiguous())
      throw std::invalid_argument("sgd_update: each gradient must have its value's shape, both C-contiguous");
    v.push_back(values[i]->ptr()); g.push_back(gradients[i]->ptr()); n.push_back(values[i]->size());
  }
  if (!v.empty()) check(detail::sgd_((int)v.size(), v.data(), g.data(), n.data(), learning_rate));
}

// conv2d = im2colgemm_conv2d (nn_primitives/fallback/conv.nim:81-106), bias [C_out] or [C_out, 1, 1], optionally
// followed by relu. Float tensors with `fused`: one launch, the GEMM's B loader gathers the column matrix from the
// images. Otherwise (integer tensors, or asked for): device im2col of the batch, then one strided-batched GEMM
// written straight into the NCHW result.
template <typename T>
HipTensor<T> conv2d(const HipTensor<T>& x, const HipTensor<T>& kernel, const HipTensor<T>* bias = nullptr, int padH = 0,
                    int padW = 0, int strideH = 1, int strideW = 1, bool with_relu = false, bool fused = true) {
  if (x.rank() != 4 || kernel.rank() != 4) throw std::invalid_argument("conv2d: input must be [N, C, H, W], kernel [C_out, C, kH, kW]");
  if (kernel.shape[1] != x.shape[1])
    throw std::invalid_argument("conv2d: kernel expects " + std::to_string(kernel.shape[1]) + " input channels, input has " + std::to_string(x.shape[1]));
  const int64_t N = x.shape[0], C = x.shape[1], H = x.shape[2], W = x.shape[3];
  const int64_t co = kernel.shape[0], kH = kernel.shape[2], kW = kernel.shape[3], K = C * kH * kW;
  const int64_t oh = (H + 2 * padH - kH) / strideH + 1, ow = (W + 2 * padW - kW) / strideW + 1, P = oh * ow;
  if (bias && bias->size() != co) throw std::invalid_argument("conv2d: bias must have one element per output channel");
  const HipTensor<T> kc = kernel.is_C_contiguous() ? kernel : kernel.clone();
  int64_t bias_s = 0;
  if (bias) for (int d = 0; d < bias->rank(); ++d) if (bias->shape[d] == co) { bias_s = bias->strides[d]; break; }
  constexpr bool F = std::is_floating_point<T>::value;
  const int epi = F ? ((bias ? AM_EPI_BIAS : 0) | (with_relu ? AM_EPI_RELU : 0)) : AM_EPI_NONE;
  HipTensor<T> out(Shape{N, co, oh, ow});
  if (out.size() == 0) return out;
  if constexpr (F) {
    if (fused && K * (int64_t)sizeof(T) >= 16 && N <= 65535) {
      check(detail::conv2d_(N, (int)C, (int)H, (int)W, (int)co, (int)kH, (int)kW, padH, padW, strideH, strideW, x.ptr(), x.strides[0],
                            x.strides[1], x.strides[2], x.strides[3], kc.ptr(), K, epi, bias ? bias->ptr() : nullptr, bias_s, out.ptr()));
      return out;
    }
  }
  HipTensor<T> col(Shape{N, K, P});
  check(detail::im2col_(N, (int)C, (int)H, (int)W, (int)kH, (int)kW, padH, padW, strideH, strideW, x.ptr(), x.strides[0], x.strides[1],
                        x.strides[2], x.strides[3], col.ptr()));
  check(detail::gemm_batched_(N, co, P, K, T(1), kc.ptr(), K, 1, 0, col.ptr(), P, 1, K * P, T(0), out.ptr(), P, 1, co * P, epi,
                              (F && bias) ? bias->ptr() : nullptr, bias_s, 0));
  if constexpr (!F) {   // integer tensors have no fused epilogue: result +.= bias.unsqueeze(0), then relu
    if (bias) {
      HipTensor<T> b3 = *bias;
      b3.shape = Shape{1, co, 1, 1};
      b3.strides = Shape{0, bias_s, 0, 0};
      out.bc_iadd(b3);
    }
    if (with_relu) out = unary(AM_UOP_RELU, out);
  }
  return out;
}

// col2im (nn_primitives/fallback/conv.nim:55-79) for a batch: [N, C*kH*kW, H_out*W_out] -> [N, C, H, W], pixels
// covered by several columns summed in the order of the reference's loop.
template <typename T>
HipTensor<T> col2im(const HipTensor<T>& col, int64_t C, int64_t H, int64_t W, int kH, int kW, int padH = 0, int padW = 0,
                    int strideH = 1, int strideW = 1) {
  const int64_t oh = (H + 2 * padH - kH) / strideH + 1, ow = (W + 2 * padW - kW) / strideW + 1;
  if (col.rank() != 3 || col.shape[1] != C * kH * kW || col.shape[2] != oh * ow)
    throw std::invalid_argument("col2im: column matrix of shape " + detail::str(col.shape) + " does not match the geometry");
  const HipTensor<T> c = col.strides[2] == 1 ? col : col.clone();
  HipTensor<T> out(Shape{col.shape[0], C, H, W});
  check(detail::col2im_(col.shape[0], (int)C, (int)H, (int)W, kH, kW, padH, padW, strideH, strideW, c.ptr(), c.strides[0], c.strides[1],
                        out.ptr(), out.strides[0], out.strides[1], out.strides[2], out.strides[3]));
  return out;
}

// conv2d_backward (nn_primitives/nnp_convolution.nim:65-107) over im2colgemm_conv2d_gradient (fallback/conv.nim:107-145).
// The reference loops over the images; here the batch is folded into the columns: g [C_out, N*P] is grad_output with
// its first two axes swapped, col [C*kH*kW, N*P] the column matrices side by side, and the pass is
// grad_bias = row sums of g, grad_weight = g * col^T, grad_input = col2im(kernel_col^T * g). `bias` of the result has
// shape [C_out, 1, 1]; without with_bias it stays a rank-0 tensor without storage (the reference's "bias.rank == 0").
template <typename T> struct Conv2dGrads { HipTensor<T> input, weight, bias; };
template <typename T>
Conv2dGrads<T> conv2d_backward(const HipTensor<T>& x, const HipTensor<T>& weight, bool with_bias, int padH, int padW, int strideH,
                               int strideW, const HipTensor<T>& grad_output) {
  if (x.rank() != 4 || weight.rank() != 4 || weight.shape[1] != x.shape[1])
    throw std::invalid_argument("conv2d_backward: input must be [N, C, H, W], kernel [C_out, C, kH, kW]");
  const int64_t N = x.shape[0], C = x.shape[1], H = x.shape[2], W = x.shape[3];
  const int64_t co = weight.shape[0], kH = weight.shape[2], kW = weight.shape[3], K = C * kH * kW;
  const int64_t oh = (H + 2 * padH - kH) / strideH + 1, ow = (W + 2 * padW - kW) / strideW + 1, P = oh * ow;
  if (grad_output.shape != Shape{N, co, oh, ow})
    throw std::invalid_argument("conv2d_backward: grad_output is " + detail::str(grad_output.shape) + ", the convolution's result is " +
                                detail::str(Shape{N, co, oh, ow}));
  const HipTensor<T> go = grad_output.is_C_contiguous() ? grad_output : grad_output.clone();
  HipTensor<T> gview = go;                       // g[co, n, p] = grad_output[n, co, p]
  gview.shape = Shape{co, N, P};
  gview.strides = Shape{P, co * P, 1};
  HipTensor<T> g = gview.clone();
  g.shape = Shape{co, N * P};
  g.strides = Shape{N * P, 1};
  Conv2dGrads<T> r;
  if (with_bias) {
    r.bias = sum(g, 1);
    r.bias.shape = Shape{co, 1, 1};
    r.bias.strides = Shape{1, 1, 1};
  }
  HipTensor<T> kcol = weight.is_C_contiguous() ? weight : weight.clone();
  kcol.shape = Shape{co, K};
  kcol.strides = Shape{K, 1};
  bool gathered = false;
  if constexpr (std::is_floating_point<T>::value) {
    // one launch where the library's loader can gather col^T from the images in 16-byte pieces: col is never written
    constexpr int64_t VK = 16 / (int64_t)sizeof(T);
    if (strideW == 1 && x.strides[3] == 1 && ow % VK == 0 && W >= VK && N >= 1 && P >= 1 && N * P < ((int64_t)1 << 31) &&
        K * kH * kW < ((int64_t)1 << 32) && co * K < 1000000) {   // (larger gradients: the plain product's larger tiles win)
      r.weight = HipTensor<T>(Shape{co, C, kH, kW});
      check(detail::conv2d_grad_weight_(N, (int)C, (int)H, (int)W, (int)co, (int)kH, (int)kW, padH, padW, strideH, strideW, x.ptr(),
                                        x.strides[0], x.strides[1], x.strides[2], x.strides[3], g.ptr(), g.strides[0], r.weight.ptr()));
      gathered = true;
    }
  }
  if (!gathered) {
    HipTensor<T> col(Shape{K, N * P});
    check(detail::im2col_strided_(N, (int)C, (int)H, (int)W, (int)kH, (int)kW, padH, padW, strideH, strideW, x.ptr(), x.strides[0],
                                  x.strides[1], x.strides[2], x.strides[3], col.ptr(), P, N * P));
    r.weight = g * col.transpose();
    r.weight.shape = Shape{co, C, kH, kW};
    r.weight.strides = Shape{K, kH * kW, kW, 1};
  }
  const HipTensor<T> gcol = kcol.transpose() * g;
  r.input = HipTensor<T>(Shape{N, C, H, W});
  check(detail::col2im_(N, (int)C, (int)H, (int)W, (int)kH, (int)kW, padH, padW, strideH, strideW, gcol.ptr(), P, N * P, r.input.ptr(),
                        r.input.strides[0], r.input.strides[1], r.input.strides[2], r.input.strides[3]));
  return r;
}

// maxpool2d (nnp_maxpooling.nim:19-66): values and the flat input index of each maximum.
template <typename T> struct MaxPooled { HipTensor<int64_t> max_indices; HipTensor<T> maxpooled; };
template <typename T>
MaxPooled<T> maxpool2d(const HipTensor<T>& x, int kH, int kW, int padH = 0, int padW = 0, int strideH = 1, int strideW = 1) {
  if (x.rank() != 4 || !x.is_C_contiguous()) throw std::invalid_argument("maxpool2d: input must be a C-contiguous [N, C, H, W] tensor");
  const int64_t N = x.shape[0], C = x.shape[1], H = x.shape[2], W = x.shape[3];
  const int64_t oh = (H + 2 * padH - kH) / strideH + 1, ow = (W + 2 * padW - kW) / strideW + 1;
  MaxPooled<T> r{HipTensor<int64_t>(Shape{N * C * oh * ow}), HipTensor<T>(Shape{N, C, oh, ow})};
  check(detail::maxpool2d_(N, (int)C, (int)H, (int)W, kH, kW, padH, padW, strideH, strideW, x.ptr(), r.maxpooled.ptr(),
                           r.max_indices.ptr()));
  return r;
}

// maxpool2d_backward (nnp_maxpooling.nim:68-83): zeros of the cached input shape with
// gradInput[max_indices[i]] = gradOutput[i]. The device runs the scatter as a gather over the pooling
// windows, so the geometry of the forward pass is passed again.
template <typename T>
HipTensor<T> maxpool2d_backward(const Shape& cached_input_shape, const HipTensor<int64_t>& cached_max_indices,
                                const HipTensor<T>& grad_output, int kH, int kW, int padH = 0, int padW = 0,
                                int strideH = 1, int strideW = 1) {
  if (cached_input_shape.size() != 4) throw std::invalid_argument("maxpool2d_backward: cached_input_shape must be [N, C, H, W]");
  const int64_t N = cached_input_shape[0], C = cached_input_shape[1], H = cached_input_shape[2], W = cached_input_shape[3];
  const int64_t oh = (H + 2 * padH - kH) / strideH + 1, ow = (W + 2 * padW - kW) / strideW + 1;
  if (grad_output.size() != cached_max_indices.size() || grad_output.size() != N * C * oh * ow ||
      !grad_output.is_C_contiguous() || !cached_max_indices.is_C_contiguous())
    throw std::invalid_argument("maxpool2d_backward: gradOutput, the indices and the pooling geometry do not match");
  HipTensor<T> r(cached_input_shape);
  check(detail::maxpool2d_backward_(N, (int)C, (int)H, (int)W, kH, kW, padH, padW, strideH, strideW, cached_max_indices.ptr(),
                                    grad_output.ptr(), r.ptr()));
  return r;
}

// ---- HIP graphs ---------------------------------------------------------------------------------
// A recorded sequence of device operations, replayed with one launch. Graph::record(fn) runs fn twice: once as a
// rehearsal with the allocator holding back every block that is freed (afterwards its cache has one block per
// allocation fn makes, and the library workspace its final size), then under capture, where allocation is served from
// that cache - so fn may create temporaries freely. fn must only issue device work (no toCpu / toHip) on tensors that
// outlive the graph. The reference has no counterpart (one launch per operator).
class Graph {
 public:
  Graph() = default;
  Graph(const Graph&) = delete;
  Graph& operator=(const Graph&) = delete;
  Graph(Graph&& o) noexcept : exec_(o.exec_) { o.exec_ = nullptr; }
  Graph& operator=(Graph&& o) noexcept {
    if (this != &o) { reset(); exec_ = o.exec_; o.exec_ = nullptr; }
    return *this;
  }
  ~Graph() { reset(); }

  template <typename F> static Graph record(F&& fn) {
    check(am_hip_alloc_hold(1));
    try { fn(); } catch (...) { (void)am_hip_alloc_hold(0); throw; }
    check(am_hip_alloc_hold(0));
    check(am_hip_graph_begin());
    Graph g;
    try { fn(); } catch (...) { void* dead = nullptr; (void)am_hip_graph_end(&dead); if (dead) (void)am_hip_graph_destroy(dead); throw; }
    check(am_hip_graph_end(&g.exec_));
    return g;
  }
  void launch() const { check(am_hip_graph_launch(exec_)); }
  explicit operator bool() const { return exec_ != nullptr; }

 private:
  void reset() { if (exec_) { (void)am_hip_graph_destroy(exec_); exec_ = nullptr; } }
  void* exec_ = nullptr;
};

// ---- .npy files (src/arraymancer/io/io_npy.nim:64-183) -----------------------------------------
namespace detail {
template <typename S, typename T>
inline void npy_convert(const unsigned char* raw, size_t n, bool big_endian, std::vector<T>& out) {
  out.resize(n);
  for (size_t i = 0; i < n; ++i) {
    unsigned char b[sizeof(S)];
    for (size_t k = 0; k < sizeof(S); ++k) b[k] = raw[i * sizeof(S) + (big_endian ? sizeof(S) - 1 - k : k)];   // to little endian
    S v;
    std::memcpy(&v, b, sizeof(S));
    out[i] = static_cast<T>(v);   // `stream.readXxx.T`: float -> integer truncates
  }
}
}  // namespace detail

// read_npy[T](path): versions 1.0 / 2.0; <f4 >f4 <f8 >f8 <i4 >i4 <i8 >i8 <u4 >u4 <u8 >u8 converted
// element by element to T; a Fortran-ordered file gives a column-major tensor.
template <typename T>
HipTensor<T> read_npy(const std::string& path) {
  std::ifstream f(path, std::ios::binary);
  if (!f) throw std::ios_base::failure(".npy file \"" + path + "\" does not exist");
  char magic[8];
  f.read(magic, 8);
  if (f.gcount() != 8 || std::memcmp(magic, "\x93NUMPY", 6) != 0) throw std::invalid_argument("This file is not a Numpy file");
  const int major = (unsigned char)magic[6], minor = (unsigned char)magic[7];
  if (!((major == 1 || major == 2) && minor == 0)) throw std::invalid_argument("Unsupported .npy format: only 1.0 or 2.0 files can be loaded");
  unsigned char lb[4] = {0, 0, 0, 0};
  f.read((char*)lb, major == 1 ? 2 : 4);
  const size_t header_len = (size_t)lb[0] | ((size_t)lb[1] << 8) | ((size_t)lb[2] << 16) | ((size_t)lb[3] << 24);
  std::string header(header_len, '\0');
  f.read(&header[0], (std::streamsize)header_len);
  auto field = [&](const std::string& key, const std::string& until) {
    const size_t a = header.find(key);
    if (a == std::string::npos) throw std::invalid_argument("Error while parsing .npy header " + header);
    const size_t b = header.find(until, a + key.size());
    if (b == std::string::npos) throw std::invalid_argument("Error while parsing .npy header " + header);
    return header.substr(a + key.size(), b - a - key.size());
  };
  const std::string descr = field("'descr': '", "'"), fortran = field("'fortran_order': ", ","), shp = field("'shape': (", ")");
  if (fortran != "False" && fortran != "True") throw std::invalid_argument("Invalid token '" + fortran + "' in numpy description " + header);
  Shape shape;
  for (size_t i = 0; i < shp.size();) {
    if (shp[i] == ' ' || shp[i] == ',') { ++i; continue; }
    if (shp[i] < '0' || shp[i] > '9') throw std::invalid_argument(std::string("Invalid token '") + shp[i] + "' in numpy shape (" + shp + ")");
    int64_t v = 0;
    while (i < shp.size() && shp[i] >= '0' && shp[i] <= '9') v = v * 10 + (shp[i++] - '0');
    shape.push_back(v);
  }
  if (descr.size() != 3 || (descr[0] != '<' && descr[0] != '>') || std::string("fiu").find(descr[1]) == std::string::npos ||
      (descr[2] != '4' && descr[2] != '8'))
    throw std::invalid_argument("Numpy type not supported: " + descr + " in file.");
  size_t n = 1;
  for (auto e : shape) n *= (size_t)e;
  const size_t width = (size_t)(descr[2] - '0');
  std::vector<unsigned char> raw(n * width);
  f.read((char*)raw.data(), (std::streamsize)raw.size());
  if ((size_t)f.gcount() != raw.size()) throw std::invalid_argument("truncated .npy file " + path);
  const bool be = descr[0] == '>';
  std::vector<T> host;
  if (descr[1] == 'f' && width == 4) detail::npy_convert<float, T>(raw.data(), n, be, host);
  else if (descr[1] == 'f') detail::npy_convert<double, T>(raw.data(), n, be, host);
  else if (descr[1] == 'i' && width == 4) detail::npy_convert<int32_t, T>(raw.data(), n, be, host);
  else if (descr[1] == 'i') detail::npy_convert<int64_t, T>(raw.data(), n, be, host);
  else if (width == 4) detail::npy_convert<uint32_t, T>(raw.data(), n, be, host);
  else detail::npy_convert<uint64_t, T>(raw.data(), n, be, host);
  if (fortran == "False") return toHip(host, shape);
  // column-major sequence in the file: upload as is, describe with column-major strides
  HipTensor<T> t = toHip(host, Shape{(int64_t)n});
  t.shape = shape;
  t.strides.assign(shape.size(), 0);
  int64_t acc = 1;
  for (size_t i = 0; i < shape.size(); ++i) { t.strides[i] = acc; acc *= shape[i]; }
  return t;
}

// t.write_npy(path): a contiguous copy, in Fortran order when the tensor is column-major, version
// 1.0 header (2.0 past 16 bits) padded so that the data starts on a 16-byte boundary: the same
// bytes NumPy's own writer produced for the reference's test files. Little-endian hosts.
template <typename T>
void write_npy(const HipTensor<T>& t, const std::string& path) {
  if (t.rank() == 0) throw std::invalid_argument("write_npy: rank-0 tensors are not supported");
  const bool fortran = t.rank() > 1 && t.is_F_contiguous() && !t.is_C_contiguous();
  const std::vector<T> host = fortran ? t.transpose().toCpu() : t.toCpu();   // column-major sequence = C order of the transpose
  std::string header = std::string("{'descr': '<") + (std::is_floating_point<T>::value ? "f" : "i") + std::to_string(sizeof(T)) +
                       "', 'fortran_order': " + (fortran ? "True" : "False") + ", 'shape': (";
  for (int i = 0; i < t.rank(); ++i) header += (i ? ", " : "") + std::to_string(t.shape[i]);
  header += t.rank() == 1 ? ",), }" : "), }";
  size_t meta = 6 + 4 + header.size() + 1;
  const bool v1 = meta <= 0xFFFF;
  if (!v1) meta += 2;
  header += std::string((16 - (meta & 15)) & 15, ' ') + "\n";
  std::ofstream f(path, std::ios::binary | std::ios::trunc);
  if (!f) throw std::ios_base::failure("cannot open " + path + " for writing");
  f.write("\x93NUMPY", 6);
  const size_t hl = header.size();
  if (v1) { const unsigned char b[4] = {1, 0, (unsigned char)(hl & 255), (unsigned char)(hl >> 8)}; f.write((const char*)b, 4); }
  else { const unsigned char b[6] = {2, 0, (unsigned char)(hl & 255), (unsigned char)((hl >> 8) & 255), (unsigned char)((hl >> 16) & 255), (unsigned char)(hl >> 24)}; f.write((const char*)b, 6); }
  f.write(header.data(), (std::streamsize)hl);
  f.write((const char*)host.data(), (std::streamsize)(host.size() * sizeof(T)));
}

// ---- display (src/arraymancer/tensor/display_cuda.nim:19-36 over display.nim:19-115, private/p_display.nim:152-485) ----
// A device tensor prints as its host copy laid out by the reference's CPU printer: table mode (specifier ""
// or "||" / "<|>" / "<>||": last two dimensions as rows between `|`, odd dimensions side by side under their
// index, even dimensions stacked with their index on the left), or array modes ("[]" one line, "[:]" one row
// per line; "<>" / "<:>" / "<>[]" / "<>[:]" with a compact header). Floats print like printf's %g
// (precision -1) or %#.{precision}g. Everything below formats host data; nothing runs on the device.
namespace detail {
inline std::string nim_type_name(float) { return "float32"; }
inline std::string nim_type_name(double) { return "float"; }     // Nim's float is the 64-bit one
inline std::string nim_type_name(int32_t) { return "int32"; }
inline std::string nim_type_name(int64_t) { return "int"; }      // Nim's int is the 64-bit one here
inline std::string nim_type_name(uint8_t) { return "bool"; }

template <typename T> std::string disp_element(T v, int precision) {
  char buf[64];
  if constexpr (std::is_floating_point<T>::value) {
    if (v != v) return "nan";
    if (precision >= 0) std::snprintf(buf, sizeof(buf), "%#.*g", precision, (double)v);
    else std::snprintf(buf, sizeof(buf), "%g", (double)v);
    return buf;
  } else if constexpr (std::is_same<T, uint8_t>::value) {
    return v ? "true" : "false";
  } else {
    return std::to_string((long long)v);
  }
}
inline std::vector<std::string> split_lines(const std::string& s) {   // "a\nb\n" -> {"a", "b", ""}
  std::vector<std::string> out(1);
  for (char c : s) { if (c == '\n') out.emplace_back(); else out.back() += c; }
  return out;
}
inline std::string center(const std::string& s, size_t width) {       // the smaller padding on the left
  if (width <= s.size()) return s;
  const size_t left = (width - s.size()) / 2;
  return std::string(left, ' ') + s + std::string(width - s.size() - left, ' ');
}
inline std::string strip(const std::string& s) {
  const char* ws = " \t\n\r";
  const size_t a = s.find_first_not_of(ws);
  if (a == std::string::npos) return "";
  return s.substr(a, s.find_last_not_of(ws) - a + 1);
}
inline std::string zip_strings(const std::string& s1, const std::string& s2, const std::string& sep, bool allow_empty) {
  const auto a = split_lines(s1), b = split_lines(s2);
  if (a.size() == 1) return s2;
  if (b.size() == 1) return s1;
  std::string out;
  for (size_t i = 0; i < std::min(a.size(), b.size()); ++i) {
    if (!allow_empty && a[i].empty() && b[i].empty()) continue;
    out += a[i] + sep + b[i] + "\n";
  }
  return out;
}
inline std::string gen_sep(int rank, size_t line_len = 0, bool xaxis = false) {
  std::string out;
  for (int i = 2; i < rank; ++i) {
    if (i % 2 == 0) out += xaxis ? std::string(line_len, '-') : std::string(" ");
    else out += xaxis ? std::string(line_len, ' ') : std::string(" | ");
    if (xaxis) out += "\n";
  }
  return out;
}
inline std::string left_idx(const std::string& ax, const std::string& s) {
  const std::string c = center(ax + " ", split_lines(s).size());
  std::vector<std::string> tmp(1);
  for (char ch : c) { if (ch == ' ') tmp.emplace_back(); else tmp.back() += ch; }
  std::string out;
  const size_t high = tmp.size() - 1;
  for (size_t i = 0; i < high; ++i) {
    out += tmp[i].empty() ? std::string(ax.size(), ' ') + " " : tmp[i] + " ";
    if (i + 1 < high) out += "\n";
  }
  return out;
}
inline std::string pad_left(const std::string& v, int w) { return (int)v.size() >= w ? v : std::string(w - v.size(), ' ') + v; }
inline std::string pad_right(const std::string& v, int w) { return (int)v.size() >= w ? v : v + std::string(w - v.size(), ' '); }

// `data` holds the elements of a tensor of `shape` in C order.
template <typename T>
std::string disp_table(const T* data, Shape shape, int input_rank, int align_by, int precision) {
  const int align_spacing = 4;
  int64_t n = 1;
  for (auto e : shape) n *= e;
  if (input_rank == 0) {
    input_rank = (int)shape.size();
    size_t largest = 0;
    for (int64_t i = 0; i < n; ++i) largest = std::max(largest, disp_element(data[i], precision).size());
    align_by = std::max(6, (int)largest + align_spacing);
  }
  if (shape.size() <= 2) {
    std::string out;
    const int64_t cols = shape.size() == 2 ? shape[1] : 0;
    for (int64_t idx = 1; idx <= n; ++idx) {
      const std::string val = disp_element(data[idx - 1], precision);
      if (cols == 0) out += pad_left(val, align_by);
      else if (idx % cols == 0) out += cols == 1 ? "|" + pad_left(val, align_by - align_spacing) + "|\n" : pad_left(val, align_by) + "|\n";
      else if (idx % cols == 1) out += "|" + pad_right(val, align_by - align_spacing);
      else out += pad_left(val, align_by);
    }
    return strip(out);
  }
  const int rank = (int)shape.size();
  const bool odd = rank % 2 != 0;
  Shape sub(shape.begin() + 1, shape.end());
  sub.erase(std::remove(sub.begin(), sub.end(), (int64_t)1), sub.end());   // squeeze
  if (sub.empty()) sub.push_back(1);
  const int64_t sub_n = n / shape[0];
  std::string res;
  for (int64_t ax = 0; ax < shape[0]; ++ax) {
    std::string part = disp_table(data + ax * sub_n, sub, input_rank, align_by, precision);
    if (odd) {
      part = center(std::to_string(ax), split_lines(part)[0].size()) + "\n" + part;
      res = zip_strings(res, part, gen_sep(rank), false);
    } else {
      res += zip_strings(left_idx(std::to_string(ax), part), part, "", true);
    }
  }
  if (odd && rank != input_rank) res += gen_sep(rank, split_lines(res)[0].size(), true);
  return res;
}

template <typename T>
std::string disp_array(const T* data, Shape shape, int precision, const std::string& row_sep) {
  if (shape.size() <= 1) {
    const int64_t n = shape.empty() ? 1 : shape[0];
    std::string out = "[";
    for (int64_t i = 0; i < n; ++i) out += (i ? ", " : "") + disp_element(data[i], precision);
    return out + "]";
  }
  int64_t sub_n = 1;
  for (size_t i = 1; i < shape.size(); ++i) sub_n *= shape[i];
  const Shape sub(shape.begin() + 1, shape.end());
  std::string out = "[";
  for (int64_t i = 0; i < shape[0]; ++i) {
    if (i) out += ", " + row_sep;
    out += disp_array(data + i * sub_n, sub, precision, row_sep);
  }
  return out + "]";
}
}  // namespace detail

// prettyImpl for host data of `shape` in C order; `type_name` / `backend` go into the header.
template <typename T>
std::string pretty_host(const std::vector<T>& host, const Shape& shape, const std::string& type_name, const std::string& backend,
                        int precision = -1, const std::string& specifier = "") {
  int mode;      // 0 table, 1 single line, 2 one row per line
  bool header;
  if (specifier == "" || specifier == "<|>" || specifier == "<>||") { mode = 0; header = true; }
  else if (specifier == "||") { mode = 0; header = false; }
  else if (specifier == "[]") { mode = 1; header = false; }
  else if (specifier == "<>[]" || specifier == "<>") { mode = 1; header = true; }
  else if (specifier == "[:]") { mode = 2; header = false; }
  else if (specifier == "<>[:]" || specifier == "<:>") { mode = 2; header = true; }
  else throw std::invalid_argument("Invalid tensor format specifier (" + specifier + ")");
  const std::string elem = detail::nim_type_name(T());
  if (mode != 0) {
    std::string compact = type_name + "[" + elem + "]<";
    for (size_t i = 0; i < shape.size(); ++i) compact += (i ? "," : "") + std::to_string(shape[i]);
    compact += ">";
    if (mode == 1) return (header ? compact + ":" : "") + detail::disp_array(host.data(), shape, precision, "");
    std::string body;
    for (const std::string& line : detail::split_lines(detail::disp_array(host.data(), shape, precision, "\n"))) {
      const size_t brackets = line.find_first_not_of('[') == std::string::npos ? line.size() : line.find_first_not_of('[');
      body += (line.empty() ? "" : std::string(shape.size() > brackets ? shape.size() - brackets : 0, ' ')) + line + "\n";
    }
    while (!body.empty() && (body.back() == '\n' || body.back() == ' ')) body.pop_back();
    return (header ? compact + ":\n" : "") + body;
  }
  const std::string desc = header ? type_name + "[system." + elem + "] of shape \"" + detail::str(shape) + "\" on backend \"" + backend + "\"\n" : "";
  if (host.empty()) return desc + "    [] (empty)";
  if (shape.size() == 1) return desc + "    " + detail::disp_table(host.data(), shape, 0, 0, precision);
  return desc + detail::disp_table(host.data(), shape, 0, 0, precision);
}

// t.pretty(precision) / `$t` for a device tensor.
template <typename T>
std::string pretty(const HipTensor<T>& t, int precision = -1, const std::string& specifier = "") {
  return pretty_host(t.toCpu(), t.shape, "HipTensor", "Hip", precision, specifier);
}
template <typename T>
std::ostream& operator<<(std::ostream& os, const HipTensor<T>& t) { return os << pretty(t); }

inline void sync() { check(am_hip_sync()); }

}  // namespace am
