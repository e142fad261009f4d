// Matrix-vector product and dot product for gfx950 (HBM-bound): am_hip_gemv_*, am_hip_dot_*.
//
// y[M] <- alpha * A[M x N] * x[N] + beta * y      (src/arraymancer/tensor/operators_blas_l2l3.nim:24-56,
//                                                 integer fallback fallback/naive_l2_gemv.nim:24-57)
// dot(x, y)                                       (src/arraymancer/tensor/operators_blas_l1.nim:27-38)
//
// Every byte of A is needed once, so the kernels are shaped around the unit-stride direction of A:
//   gemv_rows  A has unit column stride: one wavefront per row, lanes stride along the row with
//              16-byte loads of A and x, 64-lane shuffle reduction at the end.
//   gemv_cols  A has unit row stride (a transposed view): a lane owns VEC consecutive rows and
//              walks the columns with 16-byte loads (coalesced along m), UN of them in flight; x[j] is
//              one scalar load.
//              The column range is cut over gridDim.y so the chip fills for short, wide matrices;
//              partial vectors go through the split-K workspace and the shared reduce kernel.
// Anything else (both strides non-unit, tiny M) runs as an N = 1 GEMM, which handles all strides.
// Integer arithmetic wraps (unsigned twin); float partial sums are combined in a fixed order.
#include "gemm_common.h"
#include "gemm_loader.h"

using namespace am;
using namespace am::gemm;

extern "C" int am_hip_gemm_f32(int64_t, int64_t, int64_t, float, const float*, int64_t, int64_t, const float*, int64_t, int64_t, float, float*, int64_t, int64_t);
extern "C" int am_hip_gemm_f64(int64_t, int64_t, int64_t, double, const double*, int64_t, int64_t, const double*, int64_t, int64_t, double, double*, int64_t, int64_t);
extern "C" int am_hip_gemm_i32(int64_t, int64_t, int64_t, int32_t, const int32_t*, int64_t, int64_t, const int32_t*, int64_t, int64_t, int32_t, int32_t*, int64_t, int64_t);
extern "C" int am_hip_gemm_i64(int64_t, int64_t, int64_t, int64_t, const int64_t*, int64_t, int64_t, const int64_t*, int64_t, int64_t, int64_t, int64_t*, int64_t, int64_t);

namespace {

template <typename T> struct Acc { typedef T type; };
template <> struct Acc<int32_t> { typedef uint32_t type; };
template <> struct Acc<int64_t> { typedef uint64_t type; };

template <typename U> __device__ __forceinline__ U wave_sum(U v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_down(v, off, 64);
  return v;   // lane 0 holds the total
}
template <> __device__ __forceinline__ uint32_t wave_sum<uint32_t>(uint32_t v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += (uint32_t)__shfl_down((int)v, off, 64);
  return v;
}
template <> __device__ __forceinline__ uint64_t wave_sum<uint64_t>(uint64_t v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += (uint64_t)__shfl_down((long long)v, off, 64);
  return v;
}

template <typename U> __device__ __forceinline__ U xor_lane(U v, int d) { return __shfl_xor(v, d, 64); }
template <> __device__ __forceinline__ uint32_t xor_lane<uint32_t>(uint32_t v, int d) { return (uint32_t)__shfl_xor((int)v, d, 64); }
template <> __device__ __forceinline__ uint64_t xor_lane<uint64_t>(uint64_t v, int d) { return (uint64_t)__shfl_xor((long long)v, d, 64); }

template <typename T> struct GemvArgs {
  int64_t M, N;
  T alpha, beta;
  const T* A; int64_t rsA, csA;
  const T* x; int64_t incx;
  T* y; int64_t incy;
  T* ws; int splits; int64_t n_chunk;
};

template <typename T, typename U>
__device__ __forceinline__ void store_y(const GemvArgs<T>& p, int64_t row, U sum) {
  T* yp = p.y + row * p.incy;
  U v = (U)p.alpha * sum;
  if (p.beta != (T)0) v += (U)p.beta * (U)*yp;
  *yp = (T)v;
}

// A row-contiguous. VECLOAD: rows and x are 16-byte aligned and x has unit stride. With p.splits > 1 (few, long
// rows: a wavefront per row would leave most of the chip idle) a wavefront takes one chunk of one row, columns
// [chunk * n_chunk, ...), and its sum goes to ws[chunk][row] for the split-K reduce kernel.
template <typename T, bool VECLOAD>
__global__ __launch_bounds__(256) void gemv_rows(GemvArgs<T> p) {
  typedef typename Acc<T>::type U;
  typedef typename VecTraits<T>::vec_t vec_t;
  constexpr int VEC = VecTraits<T>::VK;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int64_t units = p.M * p.splits;
  for (int64_t unit = (int64_t)blockIdx.x * 4 + wave; unit < units; unit += (int64_t)gridDim.x * 4) {
    const int64_t chunk = unit / p.M, row = unit - chunk * p.M;
    const int64_t c0 = chunk * p.n_chunk;
    const int64_t len = (c0 + p.n_chunk < p.N) ? p.n_chunk : p.N - c0;
    const T* __restrict__ a = p.A + row * p.rsA + c0;
    const T* __restrict__ xs = p.x + c0 * p.incx;
    U acc0 = 0, acc1 = 0;
    if constexpr (VECLOAD) {
      const int64_t nvec = len / VEC;
      int64_t j = lane;
      for (; j + 192 < nvec; j += 256) {   // four 16-byte loads of A in flight per lane
        const vec_t a0 = __builtin_nontemporal_load((const vec_t*)a + j), a1 = __builtin_nontemporal_load((const vec_t*)a + j + 64);
        const vec_t a2 = __builtin_nontemporal_load((const vec_t*)a + j + 128), a3 = __builtin_nontemporal_load((const vec_t*)a + j + 192);
        const vec_t x0 = *((const vec_t*)xs + j), x1 = *((const vec_t*)xs + j + 64), x2 = *((const vec_t*)xs + j + 128), x3 = *((const vec_t*)xs + j + 192);
#pragma unroll
        for (int e = 0; e < VEC; ++e) { acc0 += (U)a0[e] * (U)x0[e]; acc1 += (U)a1[e] * (U)x1[e]; }
#pragma unroll
        for (int e = 0; e < VEC; ++e) { acc0 += (U)a2[e] * (U)x2[e]; acc1 += (U)a3[e] * (U)x3[e]; }
      }
      for (; j < nvec; j += 64) {
        const vec_t a0 = __builtin_nontemporal_load((const vec_t*)a + j);
        const vec_t x0 = *((const vec_t*)xs + j);
#pragma unroll
        for (int e = 0; e < VEC; ++e) acc0 += (U)a0[e] * (U)x0[e];
      }
      for (int64_t c = nvec * VEC + lane; c < len; c += 64) acc1 += (U)a[c] * (U)xs[c];
    } else {
      for (int64_t c = lane; c < len; c += 64) acc0 += (U)a[c] * (U)xs[c * p.incx];
    }
    const U total = wave_sum<U>(acc0 + acc1);
    if (lane == 0) {
      if (p.splits > 1) p.ws[chunk * p.M + row] = (T)total;
      else store_y<T, U>(p, row, total);
    }
  }
}

// Many SHORT rows (a [batch x features] matrix times a weight vector, 4 ... 128 features): `lanes` lanes (a power of
// two <= 32) share a row, one 16-byte vector of A each and their piece of x in registers, so a wavefront's load is one
// contiguous run of 64 / lanes rows; four row groups in flight; the lanes of a row are summed by a butterfly.
// Requires unit strides of A's columns and of x, N % VEC == 0, 16-byte aligned rows.
template <typename T>
__global__ __launch_bounds__(256) void gemv_rows_short(GemvArgs<T> p, int lanes) {
  typedef typename Acc<T>::type U;
  typedef typename VecTraits<T>::vec_t vec_t;
  constexpr int VEC = VecTraits<T>::VK;
  constexpr int UNR = 4;
  const int lane = threadIdx.x & 63;
  const int j = lane & (lanes - 1), sub = lane / lanes, rows_per_step = 64 / lanes;
  const int64_t nvec = p.N / VEC;
  const bool mine = j < nvec;
  const vec_t xv = *((const vec_t*)p.x + (mine ? j : 0));
  const int64_t wave = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  const int64_t row0 = wave * (int64_t)(UNR * rows_per_step) + sub;
  vec_t av[UNR];
#pragma unroll
  for (int u = 0; u < UNR; ++u) {
    const int64_t row = row0 + (int64_t)u * rows_per_step;
    av[u] = __builtin_nontemporal_load((const vec_t*)(p.A + (row < p.M ? row : 0) * p.rsA) + (mine ? j : 0));
  }
#pragma unroll
  for (int u = 0; u < UNR; ++u) {
    const int64_t row = row0 + (int64_t)u * rows_per_step;
    U acc = 0;
    if (mine) {
#pragma unroll
      for (int e = 0; e < VEC; ++e) acc += (U)av[u][e] * (U)xv[e];
    }
    for (int d = lanes >> 1; d >= 1; d >>= 1) acc += xor_lane<U>(acc, d);
    if (j == 0 && row < p.M) store_y<T, U>(p, row, acc);
  }
}

// A column-contiguous with FEW rows (y = A^T r for a tall [batch x features] matrix: the outputs are the features):
// the 256 lanes of a workgroup are laid over cxw lanes along the unit-stride direction x 256 / cxw columns, each lane
// walks every (256 / cxw)-th column of the workgroup's chunk with eight loads in flight, and the column classes are
// summed through LDS in a fixed order. grid = (chunks of the walk, blocks of cxw lanes along m). With chunks, the
// partials ws[chunk][M] are folded by a second launch of this kernel over the partials themselves (x == nullptr: every
// factor is one; 8 lanes wide, so that it spreads over many workgroups), which applies alpha and beta.
template <typename T>
__global__ __launch_bounds__(256) void gemv_cols_narrow(GemvArgs<T> p, int cxw) {
  typedef typename Acc<T>::type U;
  typedef typename VecTraits<T>::vec_t vec_t;
  constexpr int VEC = VecTraits<T>::VK;
  constexpr int UN = 8;
  __shared__ U part[256][VEC];
  const int ry = 256 / cxw;
  const int xq = (int)threadIdx.x % cxw, yq = (int)threadIdx.x / cxw;
  const int64_t m = ((int64_t)blockIdx.y * cxw + xq) * VEC;
  const bool active = yq < ry && m < p.M;
  const bool ones = p.x == nullptr;
  const int64_t j0 = (int64_t)blockIdx.x * p.n_chunk;
  const int64_t j1 = (j0 + p.n_chunk < p.N) ? j0 + p.n_chunk : p.N;
  U acc[VEC];
#pragma unroll
  for (int e = 0; e < VEC; ++e) acc[e] = 0;
  if (active) {
    const T* __restrict__ a = p.A + m;
    int64_t j = j0 + yq;
    for (; j + (int64_t)(UN - 1) * ry < j1; j += (int64_t)UN * ry) {
      vec_t v[UN];
      U xs[UN];
#pragma unroll
      for (int u = 0; u < UN; ++u) {
        v[u] = __builtin_nontemporal_load((const vec_t*)(a + (j + (int64_t)u * ry) * p.csA));
        xs[u] = ones ? (U)1 : (U)p.x[(j + (int64_t)u * ry) * p.incx];
      }
#pragma unroll
      for (int u = 0; u < UN; ++u)
#pragma unroll
        for (int e = 0; e < VEC; ++e) acc[e] += (U)v[u][e] * xs[u];
    }
    for (; j < j1; j += ry) {
      const vec_t v = *(const vec_t*)(a + j * p.csA);
      const U xj = ones ? (U)1 : (U)p.x[j * p.incx];
#pragma unroll
      for (int e = 0; e < VEC; ++e) acc[e] += (U)v[e] * xj;
    }
  }
#pragma unroll
  for (int e = 0; e < VEC; ++e) part[threadIdx.x][e] = acc[e];
  __syncthreads();
  if (active && yq == 0) {
    for (int yy = 1; yy < ry; ++yy)
#pragma unroll
      for (int e = 0; e < VEC; ++e) acc[e] += part[yy * cxw + xq][e];
    if (p.splits > 1) {
      T* ws = p.ws + (int64_t)blockIdx.x * p.M + m;
#pragma unroll
      for (int e = 0; e < VEC; ++e) ws[e] = (T)acc[e];
    } else {
#pragma unroll
      for (int e = 0; e < VEC; ++e) store_y<T, U>(p, m + e, acc[e]);
    }
  }
}

// A column-contiguous (unit row stride), rows and column starts 16-byte aligned, M % VEC == 0.
template <typename T, int UN>
__global__ __launch_bounds__(256) void gemv_cols(GemvArgs<T> p) {
  typedef typename Acc<T>::type U;
  typedef typename VecTraits<T>::vec_t vec_t;
  constexpr int VEC = VecTraits<T>::VK;
  const int64_t m = ((int64_t)blockIdx.x * 256 + threadIdx.x) * VEC;
  if (m >= p.M) return;
  const int64_t j0 = (int64_t)blockIdx.y * p.n_chunk;
  const int64_t j1 = (j0 + p.n_chunk < p.N) ? j0 + p.n_chunk : p.N;
  U acc[VEC];
#pragma unroll
  for (int e = 0; e < VEC; ++e) acc[e] = 0;
  const T* __restrict__ a = p.A + m;
  int64_t j = j0;
  for (; j + UN <= j1; j += UN) {
    vec_t v[UN];
    U xs[UN];
#pragma unroll
    for (int u = 0; u < UN; ++u) {
      v[u] = __builtin_nontemporal_load((const vec_t*)(a + (j + u) * p.csA));
      xs[u] = (U)p.x[(j + u) * p.incx];
    }
#pragma unroll
    for (int u = 0; u < UN; ++u)
#pragma unroll
      for (int e = 0; e < VEC; ++e) acc[e] += (U)v[u][e] * xs[u];
  }
  for (; j < j1; ++j) {
    const vec_t v = *(const vec_t*)(a + j * p.csA);
    const U xj = (U)p.x[j * p.incx];
#pragma unroll
    for (int e = 0; e < VEC; ++e) acc[e] += (U)v[e] * xj;
  }
  if (p.splits > 1) {
    T* ws = p.ws + (int64_t)blockIdx.y * p.M + m;
#pragma unroll
    for (int e = 0; e < VEC; ++e) ws[e] = (T)acc[e];
  } else {
#pragma unroll
    for (int e = 0; e < VEC; ++e) store_y<T, U>(p, m + e, acc[e]);
  }
}

// Per-workgroup partial dot products, one slot each, in the workspace.
template <typename T, bool VECLOAD, bool STREAM>
__global__ __launch_bounds__(256) void dot_partial(int64_t n, const T* x, int64_t incx, const T* y, int64_t incy, T* ws) {
  typedef typename Acc<T>::type U;
  typedef typename VecTraits<T>::vec_t vec_t;
  constexpr int VEC = VecTraits<T>::VK;
  __shared__ U part[4];
  U acc = 0;
  if constexpr (VECLOAD) {   // unit strides, 16-byte aligned: two 16-byte loads per vector and lane, two vectors in flight
    const int64_t nvec = n / VEC, stride = (int64_t)gridDim.x * 256;
    U acc1 = 0;
    int64_t v = (int64_t)blockIdx.x * 256 + threadIdx.x;
    for (; v + stride < nvec; v += 2 * stride) {
      vec_t x0, y0, x1, y1;
      if constexpr (STREAM) {   // vectors beyond the memory-side cache
        x0 = __builtin_nontemporal_load((const vec_t*)x + v); y0 = __builtin_nontemporal_load((const vec_t*)y + v);
        x1 = __builtin_nontemporal_load((const vec_t*)x + v + stride); y1 = __builtin_nontemporal_load((const vec_t*)y + v + stride);
      } else {
        x0 = *((const vec_t*)x + v); y0 = *((const vec_t*)y + v);
        x1 = *((const vec_t*)x + v + stride); y1 = *((const vec_t*)y + v + stride);
      }
#pragma unroll
      for (int e = 0; e < VEC; ++e) { acc += (U)x0[e] * (U)y0[e]; acc1 += (U)x1[e] * (U)y1[e]; }
    }
    for (; v < nvec; v += stride) {
      const vec_t x0 = *((const vec_t*)x + v), y0 = *((const vec_t*)y + v);
#pragma unroll
      for (int e = 0; e < VEC; ++e) acc += (U)x0[e] * (U)y0[e];
    }
    acc += acc1;
    for (int64_t i = nvec * VEC + (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += stride) acc += (U)x[i] * (U)y[i];
  } else {
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (int64_t)gridDim.x * 256)
      acc += (U)x[i * incx] * (U)y[i * incy];
  }
  acc = wave_sum<U>(acc);
  if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = acc;
  __syncthreads();
  if (threadIdx.x == 0) ws[blockIdx.x] = (T)(part[0] + part[1] + part[2] + part[3]);
}

// The per-workgroup partials into one value: a lane adds every 256th partial, then the lanes are combined
// in a fixed order (one thread walking a thousand partials costs 20 us of dependent loads).
template <typename T>
__global__ __launch_bounds__(256) void dot_final(int count, const T* ws, T* out) {
  typedef typename Acc<T>::type U;
  __shared__ U part[4];
  U acc = 0;
  for (int i = threadIdx.x; i < count; i += 256) acc += (U)ws[i];
  acc = wave_sum<U>(acc);
  if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = acc;
  __syncthreads();
  if (threadIdx.x == 0) *out = (T)(part[0] + part[1] + part[2] + part[3]);
}

template <typename T>
int gemm_fallback(int64_t M, int64_t N, T alpha, const T* A, int64_t rsA, int64_t csA, const T* x, int64_t incx, T beta, T* y, int64_t incy);
#define AM_GEMV_FALLBACK(T, SFX)                                                                                   \
  template <> int gemm_fallback<T>(int64_t M, int64_t N, T alpha, const T* A, int64_t rsA, int64_t csA, const T* x, \
                                   int64_t incx, T beta, T* y, int64_t incy) {                                     \
    return am_hip_gemm_##SFX(M, 1, N, alpha, A, rsA, csA, x, incx, 1, beta, y, incy, 1);                            \
  }
AM_GEMV_FALLBACK(float, f32)
AM_GEMV_FALLBACK(double, f64)
AM_GEMV_FALLBACK(int32_t, i32)
AM_GEMV_FALLBACK(int64_t, i64)

template <typename T>
int gemv(const char* fn, int64_t M, int64_t N, T alpha, const T* A, int64_t rsA, int64_t csA, const T* x,
         int64_t incx, T beta, T* y, int64_t incy) {
  typedef typename Acc<T>::type U;
  constexpr int VEC = VecTraits<T>::VK;
  if (M < 0 || N < 0) return fail(AM_E_ARG, "%s: negative dimension", fn);
  if (M == 0) return AM_OK;
  if (!y || (N > 0 && (!A || !x))) return fail(AM_E_ARG, "%s: null pointer", fn);
  if (M > 1 && incy == 0) return fail(AM_E_SHAPE, "%s: y has stride 0", fn);
  if (N == 0) return AM_OK;   // same convention as GEMM with K == 0: nothing runs, y untouched
  AM_TRY(ensure_init());
  GemvArgs<T> g;
  g.M = M; g.N = N; g.alpha = alpha; g.beta = beta; g.A = A; g.rsA = rsA; g.csA = csA;
  g.x = x; g.incx = incx; g.y = y; g.incy = incy; g.ws = nullptr; g.splits = 1; g.n_chunk = N;

  // y seen as one row of M columns: the split-K reduce kernel adds the partials ws[split][M] in ascending order
  auto fold_partials = [&]() {
    Args<T> r;
    memset(&r, 0, sizeof(r));
    r.M = 1; r.N = M; r.K = N; r.alpha = alpha; r.beta = beta; r.C = y; r.c_m = 0; r.c_n = incy;
    r.epilogue = AM_EPI_NONE; r.splits = g.splits; r.ws = g.ws;
    return launch_splitk_reduce<T, U>(r);
  };
  if (csA == 1 && (M >= 64 || N >= 16384)) {
    const bool vec = aligned16(A) && aligned16(x) && incx == 1 && (rsA % VEC == 0);
    // short rows: several per wavefront
    if (vec && N % VEC == 0 && N / VEC <= 32 && M >= 4096) {
      int lanes = 1;
      while (lanes < N / VEC) lanes *= 2;
      const int64_t rows_per_wg = 4 * 4 * (64 / lanes);
      const int64_t blocks = (M + rows_per_wg - 1) / rows_per_wg;
      if (blocks < ((int64_t)1 << 31)) {
        hipLaunchKernelGGL((gemv_rows_short<T>), dim3((unsigned)blocks), dim3(256), 0, stream(), g, lanes);
        return check_launch("gemv_rows_short");
      }
    }
    // few long rows: chunks of a row over several wavefronts (16 wavefronts per CU over the chip, at least 4096 columns each)
    const int64_t want_waves = (int64_t)num_cus() * 16;
    if (M < want_waves / 2 && N >= 8192) {
      int64_t splits = (want_waves + M - 1) / M;
      if (splits > N / 4096) splits = N / 4096;
      if (splits > 256) splits = 256;
      if (splits >= 2) {
        int64_t chunk = (N + splits - 1) / splits;
        chunk = (chunk + 255) / 256 * 256;                      // chunk starts stay 16-byte aligned
        splits = (N + chunk - 1) / chunk;
        T* ws = splits >= 2 ? (T*)splitk_workspace((size_t)splits * M * sizeof(T)) : nullptr;
        if (ws) { g.ws = ws; g.splits = (int)splits; g.n_chunk = chunk; }
      }
    }
    int64_t blocks = (M * g.splits + 3) / 4;
    const int64_t cap = (int64_t)num_cus() * 16;
    if (blocks > cap) blocks = cap;
    if (vec) hipLaunchKernelGGL((gemv_rows<T, true>), dim3((unsigned)blocks), dim3(256), 0, stream(), g);
    else hipLaunchKernelGGL((gemv_rows<T, false>), dim3((unsigned)blocks), dim3(256), 0, stream(), g);
    AM_TRY(check_launch("gemv_rows"));
    return g.splits > 1 ? fold_partials() : AM_OK;
  }
  if (rsA == 1 && M % VEC == 0 && M / VEC <= 128 && csA % VEC == 0 && csA >= M && aligned16(A) && N >= 512) {
    // few outputs, a long walk: the workgroup-wide form, the walk cut into chunks (4 workgroups per CU)
    const int cx = (int)(M / VEC);
    int64_t splits = (int64_t)num_cus() * 4;
    if (splits > N / 256) splits = N / 256;
    if (splits >= 2) {
      const int64_t chunk = (N + splits - 1) / splits;
      splits = (N + chunk - 1) / chunk;
      T* ws = splits >= 2 ? (T*)splitk_workspace((size_t)splits * M * sizeof(T)) : nullptr;
      if (ws) { g.ws = ws; g.splits = (int)splits; g.n_chunk = chunk; }
    }
    hipLaunchKernelGGL((gemv_cols_narrow<T>), dim3((unsigned)g.splits, 1), dim3(256), 0, stream(), g, cx);
    AM_TRY(check_launch("gemv_cols_narrow"));
    if (g.splits > 1) {
      GemvArgs<T> r = g;
      r.A = g.ws; r.rsA = 1; r.csA = M; r.N = g.splits; r.x = nullptr; r.incx = 0;
      r.ws = nullptr; r.splits = 1; r.n_chunk = r.N;
      const int cxw = cx < 8 ? cx : 8;
      hipLaunchKernelGGL((gemv_cols_narrow<T>), dim3(1, (unsigned)((cx + cxw - 1) / cxw)), dim3(256), 0, stream(), r, cxw);
      AM_TRY(check_launch("gemv_cols_narrow (second pass)"));
    }
    return AM_OK;
  }
  if (rsA == 1 && M % VEC == 0 && csA % VEC == 0 && csA >= 0 && aligned16(A) && M >= 256) {
    const int64_t blocks_m = (M / VEC + 255) / 256;
    // one workgroup per CU: fewer, longer column walks (and fewer partial vectors) measured fastest
    int64_t splits = ((int64_t)num_cus() + blocks_m - 1) / blocks_m;
    if (splits > N / 32) splits = N / 32;
    if (splits > 64) splits = 64;
    if (splits >= 2) {
      const int64_t chunk = (N + splits - 1) / splits;
      splits = (N + chunk - 1) / chunk;
      T* ws = (T*)splitk_workspace((size_t)splits * M * sizeof(T));
      if (ws && splits >= 2) { g.ws = ws; g.splits = (int)splits; g.n_chunk = chunk; }
    }
    hipLaunchKernelGGL((gemv_cols<T, 8>), dim3((unsigned)blocks_m, (unsigned)g.splits), dim3(256), 0, stream(), g);
    AM_TRY(check_launch("gemv_cols"));
    return g.splits > 1 ? fold_partials() : AM_OK;
  }
  return gemm_fallback<T>(M, N, alpha, A, rsA, csA, x, incx, beta, y, incy);
}

template <typename T>
int dot(const char* fn, int64_t n, const T* x, int64_t incx, const T* y, int64_t incy, T* result) {
  typedef typename Acc<T>::type U;
  if (!result) return fail(AM_E_ARG, "%s: null result pointer", fn);
  *result = (T)0;
  if (n < 0) return fail(AM_E_ARG, "%s: negative length", fn);
  if (n == 0) return AM_OK;
  if (!x || !y) return fail(AM_E_ARG, "%s: null pointer", fn);
  AM_TRY(ensure_init());
  if (capturing()) return fail(AM_E_ARG, "%s: returns a value to the host, not allowed while a graph is being captured", fn);
  int64_t blocks = (n + 1023) / 1024;
  const int64_t cap = (int64_t)num_cus() * 4;
  if (blocks > cap) blocks = cap;
  const bool vec = incx == 1 && incy == 1 && aligned16(x) && aligned16(y);
  const bool stream_loads = 2.0 * (double)n * sizeof(T) > nt_threshold_bytes();
  T* ws = (T*)splitk_workspace((size_t)(blocks + 1) * sizeof(T));
  if (!ws) return fail(AM_E_ALLOC, "%s: workspace unavailable", fn);
  const dim3 grid((unsigned)blocks), block(256);
  if (vec && stream_loads) hipLaunchKernelGGL((dot_partial<T, true, true>), grid, block, 0, stream(), n, x, incx, y, incy, ws);
  else if (vec) hipLaunchKernelGGL((dot_partial<T, true, false>), grid, block, 0, stream(), n, x, incx, y, incy, ws);
  else hipLaunchKernelGGL((dot_partial<T, false, false>), grid, block, 0, stream(), n, x, incx, y, incy, ws);
  AM_TRY(check_launch("dot_partial"));
  hipLaunchKernelGGL((dot_final<T>), dim3(1), block, 0, stream(), (int)blocks, ws, ws + blocks);
  AM_TRY(check_launch("dot_final"));
  return fetch_result(result, ws + blocks, sizeof(T));
}

}  // namespace

#define AM_GEMV_ENTRY(T, SFX)                                                                                      \
  extern "C" int am_hip_gemv_##SFX(int64_t M, int64_t N, T alpha, const T* A, int64_t rsA, int64_t csA, const T* x, \
                                   int64_t incx, T beta, T* y, int64_t incy) {                                     \
    return gemv<T>("am_hip_gemv_" #SFX, M, N, alpha, A, rsA, csA, x, incx, beta, y, incy);                         \
  }                                                                                                                \
  extern "C" int am_hip_dot_##SFX(int64_t n, const T* x, int64_t incx, const T* y, int64_t incy, T* result) {      \
    return dot<T>("am_hip_dot_" #SFX, n, x, incx, y, incy, result);                                                \
  }
AM_GEMV_ENTRY(float, f32)
AM_GEMV_ENTRY(double, f64)
AM_GEMV_ENTRY(int32_t, i32)
AM_GEMV_ENTRY(int64_t, i64)
