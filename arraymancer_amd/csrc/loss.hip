// Softmax + cross-entropy fused, forward and backward: am_hip_softmax_cross_entropy_*,
// am_hip_sparse_softmax_cross_entropy_* and their _backward forms; sigmoid + cross-entropy likewise
// (am_hip_sigmoid_cross_entropy_*, src/arraymancer/nn_primitives/nnp_sigmoid_cross_entropy.nim:23-62)
// (src/arraymancer/nn_primitives/nnp_softmax_cross_entropy.nim:17-86, 88-177, 186-214, 217-256).
//
// The reference walks each row once with a running maximum and a sum of exp(x - maximum) that is rescaled whenever
// the maximum moves (private/p_logsumexp.nim:20-31), rows in parallel under OpenMP, and adds the rows' losses with an
// atomic. Here `lanes` lanes (a power of two up to 64) share a row: each runs the same recurrence over every lanes-th
// element, the lanes' maxima and then their sums, each rescaled once to the row's maximum, are folded in fixed butterflies,
// so a wavefront covers 64 / lanes rows and a load instruction of the wavefront reads neighbouring elements of them.
// The rows' losses go to the library workspace and are added there in a fixed order (slices of 8192, then the slices'
// sums): the result does not depend on timing, unlike the reference's atomic sum. The backward kernels recompute (M, S) the same way and write
// grad * (exp(x - M) / S - target) / batch_size in a second walk over the row, which the caches still hold.
#include <limits>
#include "common.h"

namespace am {
namespace gemm { void* splitk_workspace(size_t bytes); }
namespace loss {

template <typename T> struct Args {
  const T* x; int64_t x_rs, x_cs;
  const T* target; int64_t t_rs, t_cs;       // dense form: probabilities [rows, cols]
  const int64_t* labels; int64_t l_s;        // sparse form: one class index per row
  int64_t rows, cols;
  T* row_loss;                               // forward: one loss per row (workspace)
  T* out; int64_t o_rs, o_cs;                // backward: the gradient with respect to x
  T grad, batch;                             // backward: grad * (...) / batch
};

template <typename T> __device__ __forceinline__ T dev_exp(T v);
template <> __device__ __forceinline__ float dev_exp<float>(float v) { return expf(v); }
template <> __device__ __forceinline__ double dev_exp<double>(double v) { return exp(v); }
template <typename T> __device__ __forceinline__ T dev_log(T v);
template <> __device__ __forceinline__ float dev_log<float>(float v) { return logf(v); }
template <> __device__ __forceinline__ double dev_log<double>(double v) { return log(v); }

// Running maximum m and sum s of exp(x - m) of one lane's share of its row, then merged over the row's lanes: every
// lane of the row ends with the same (m, s). `dot` (DENSE only) likewise becomes the row's sum of x * target.
// A lane takes U units at a time (VEC: 16-byte vectors of a unit-stride row, else single elements; all loads issued
// before the first is used), raises the maximum to that of the group with one rescaling of the sum, then adds the
// group's exponentials: one exp per element and one per group instead of the reference's data-dependent branch per
// element.
template <typename T, bool DENSE, bool VEC, bool SHORT>
__device__ __forceinline__ void row_max_sumexp(const Args<T>& p, const T* x, const T* t, int j0, int lanes, T& m, T& s, T& dot) {
  constexpr int V = VEC ? 16 / (int)sizeof(T) : 1;
  constexpr int U = SHORT ? 1 : (VEC ? 4 : 8);   // SHORT: the row has at most one unit per lane
  typedef T vec_t __attribute__((ext_vector_type(V)));
  const T ninf = -std::numeric_limits<T>::infinity();
  m = ninf;
  s = (T)0;
  dot = (T)0;
  const int64_t units = p.cols / V;
  for (int64_t u0 = j0; u0 < units; u0 += (int64_t)lanes * U) {
    T v[U][V], w[U][V];
    bool live[U];
#pragma unroll
    for (int k = 0; k < U; ++k) {
      const int64_t u = u0 + (int64_t)k * lanes;
      live[k] = u < units;
      if constexpr (VEC) {
        const vec_t xv = live[k] ? *(const vec_t*)(x + u * V) : (vec_t)(ninf);
#pragma unroll
        for (int e = 0; e < V; ++e) v[k][e] = xv[e];
        if constexpr (DENSE) {
          const vec_t tv = live[k] ? *(const vec_t*)(t + u * V) : (vec_t)((T)0);
#pragma unroll
          for (int e = 0; e < V; ++e) w[k][e] = tv[e];
        }
      } else {
        v[k][0] = live[k] ? x[u * p.x_cs] : ninf;
        if constexpr (DENSE) w[k][0] = live[k] ? t[u * p.t_cs] : (T)0;
      }
    }
    T gm = m;
#pragma unroll
    for (int k = 0; k < U; ++k)
#pragma unroll
      for (int e = 0; e < V; ++e) gm = (v[k][e] <= gm) ? gm : v[k][e];
    if (!(gm <= m)) { s = (s == (T)0) ? (T)0 : s * dev_exp<T>(m - gm); m = gm; }   // also taken when gm is NaN: it propagates
    T add = (T)0;
#pragma unroll
    for (int k = 0; k < U; ++k)
#pragma unroll
      for (int e = 0; e < V; ++e) {
        if (live[k]) {
          add += dev_exp<T>(v[k][e] - m);
          if constexpr (DENSE) dot += v[k][e] * w[k][e];
        }
      }
    s += add;
  }
  // The lanes of the row: first their maxima (a butterfly of comparisons), then every lane's sum rescaled once to the
  // row's maximum, then the sums (a butterfly of additions). One exp per lane instead of two per butterfly step, which
  // on rows of a few vectors was most of the kernel's arithmetic.
  T M = m;
  for (int d = lanes >> 1; d >= 1; d >>= 1) {
    const T om = __shfl_xor(M, d, 64);
    M = (om <= M) ? M : om;
  }
  // a lane without elements holds (-inf, 0): its share is 0 whatever M is (exp(-inf - -inf) would be NaN)
  s = (s == (T)0) ? (T)0 : s * dev_exp<T>(m - M);
  m = M;
  for (int d = lanes >> 1; d >= 1; d >>= 1) {
    s += __shfl_xor(s, d, 64);
    if constexpr (DENSE) dot += __shfl_xor(dot, d, 64);
  }
}

template <typename T, bool DENSE, bool VEC, bool SHORT>
__global__ __launch_bounds__(256) void sce_forward(Args<T> p, int lanes) {
  const int lane = threadIdx.x & 63;
  const int j0 = lane & (lanes - 1);
  const int rows_per_wave = 64 / lanes;
  const int64_t groups = (p.rows + rows_per_wave - 1) / rows_per_wave;
  // a wavefront walks over groups of 64 / lanes rows: with short rows and very many of them (a loss per pixel) a
  // wavefront per group would live for a kilobyte of input
  for (int64_t grp = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6); grp < groups; grp += (int64_t)gridDim.x * 4) {
    const int64_t row = grp * rows_per_wave + lane / lanes;
    const bool ok = row < p.rows;
    const int64_t r = ok ? row : 0;
    const T* x = p.x + r * p.x_rs;
    const T* t = DENSE ? p.target + r * p.t_rs : nullptr;
    T m, s, dot;
    row_max_sumexp<T, DENSE, VEC, SHORT>(p, x, t, j0, lanes, m, s, dot);
    if (!ok || j0 != 0) continue;
    const T lse = dev_log<T>(s) + m;
    if constexpr (DENSE) {
      p.row_loss[row] = lse - dot;
    } else {
      const int64_t label = p.labels[row * p.l_s];
      // a label outside the row cannot be read: the loss says so
      p.row_loss[row] = (label >= 0 && label < p.cols) ? lse - x[label * p.x_cs] : std::numeric_limits<T>::quiet_NaN();
    }
  }
}

// Sum of v[0 .. n) in a fixed order, in up to three levels. sum_slices: workgroup b adds the slice
// [b * per, (b + 1) * per) (each lane every 256th value, eight loads in flight, then the lanes pairwise through LDS)
// into out[b], divided by `divisor`; the host runs it over the rows' losses, then over the slices' sums if there are
// many (divisor 1), and last with one workgroup and the batch size as divisor, as the reference divides its sum.
template <typename T>
__global__ __launch_bounds__(256) void sum_slices(const T* __restrict__ v, int64_t n, int64_t per, T divisor, T* __restrict__ out) {
  __shared__ T part[256];
  const int64_t lo = (int64_t)blockIdx.x * per, hi = (lo + per < n) ? lo + per : n;
  T acc = (T)0;
  int64_t i = lo + threadIdx.x;
  for (; i + 7 * 256 < hi; i += 8 * 256) {
    T a[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) a[u] = v[i + u * 256];
#pragma unroll
    for (int u = 0; u < 8; ++u) acc += a[u];
  }
  for (; i < hi; i += 256) acc += v[i];
  part[threadIdx.x] = acc;
  __syncthreads();
  for (int d = 128; d >= 1; d >>= 1) {
    if ((int)threadIdx.x < d) part[threadIdx.x] += part[threadIdx.x + d];
    __syncthreads();
  }
  if (threadIdx.x == 0) out[blockIdx.x] = part[0] / divisor;
}

template <typename T, bool DENSE, bool VEC, bool SHORT>
__global__ __launch_bounds__(256) void sce_backward(Args<T> p, int lanes) {
  constexpr int V = VEC ? 16 / (int)sizeof(T) : 1;
  constexpr int U = SHORT ? 1 : (VEC ? 2 : 4);
  typedef T vec_t __attribute__((ext_vector_type(V)));
  const int lane = threadIdx.x & 63;
  const int j0 = lane & (lanes - 1);
  const int rows_per_wave = 64 / lanes;
  const int64_t groups = (p.rows + rows_per_wave - 1) / rows_per_wave;
  for (int64_t grp = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6); grp < groups; grp += (int64_t)gridDim.x * 4) {
  const int64_t row = grp * rows_per_wave + lane / lanes;
  const bool ok = row < p.rows;
  const int64_t r = ok ? row : 0;
  const T* x = p.x + r * p.x_rs;
  const T* t = DENSE ? p.target + r * p.t_rs : nullptr;
  T m, s, dot;
  row_max_sumexp<T, false, VEC, SHORT>(p, x, t, j0, lanes, m, s, dot);
  if (!ok) continue;
  int64_t label = -1;
  if constexpr (!DENSE) label = p.labels[row * p.l_s];
  // A label outside the row cannot raise on the device: its gradient row becomes NaN, as the forward pass makes the
  // loss NaN, so that a bad label shows instead of training on silently.
  const bool bad_label = !DENSE && (label < 0 || label >= p.cols);
  T* out = p.out + row * p.o_rs;
  const int64_t units = p.cols / V;
  for (int64_t u0 = j0; u0 < units; u0 += (int64_t)lanes * U) {
    vec_t xv[U], tv[U];
#pragma unroll
    for (int k = 0; k < U; ++k) {
      const int64_t u = u0 + (int64_t)k * lanes;
      if (u < units) {
        if constexpr (VEC) {
          xv[k] = *(const vec_t*)(x + u * V);
          if constexpr (DENSE) tv[k] = *(const vec_t*)(t + u * V);
        } else {
          xv[k][0] = x[u * p.x_cs];
          if constexpr (DENSE) tv[k][0] = t[u * p.t_cs];
        }
      }
    }
#pragma unroll
    for (int k = 0; k < U; ++k) {
      const int64_t u = u0 + (int64_t)k * lanes;
      if (u >= units) continue;
      vec_t y;
#pragma unroll
      for (int e = 0; e < V; ++e) {
        const T sm = dev_exp<T>(xv[k][e] - m) / s;
        // dense: softmax - target; sparse: softmax + (-1 at the label, 0 elsewhere)
        const T inner = DENSE ? sm - tv[k][e] : sm + ((u * V + e == label) ? (T)-1 : (T)0);
        y[e] = bad_label ? (T)NAN : p.grad * inner / p.batch;
      }
      if constexpr (VEC) __builtin_nontemporal_store(y, (vec_t*)(out + u * V));
      else out[u * p.o_cs] = y[0];
    }
  }
  }
}

// Sigmoid + cross-entropy (nnp_sigmoid_cross_entropy.nim:23-45): the map2 body -y * x + max(x, 0) + ln1p(exp(-|x|)) summed
// over every element, divided by the batch size. One lane per 8 elements of the C-order traversal (any strides), the
// workgroup's 2048 terms folded through LDS into one partial; the partials are then added like the rows' losses above.
template <typename T> __device__ __forceinline__ T dev_log1p(T v);
template <> __device__ __forceinline__ float dev_log1p<float>(float v) { return log1pf(v); }
template <> __device__ __forceinline__ double dev_log1p<double>(double v) { return log1p(v); }

template <typename T>
__global__ __launch_bounds__(256) void sigmoid_ce_partial(Args<T> p, T* __restrict__ partial) {
  __shared__ T part[256];
  const int64_t total = p.rows * p.cols;
  T acc = (T)0;
  const int64_t base = (int64_t)blockIdx.x * 2048 + threadIdx.x;
#pragma unroll
  for (int u = 0; u < 8; ++u) {
    const int64_t i = base + (int64_t)u * 256;
    if (i < total) {
      const int64_t r = i / p.cols, c = i - r * p.cols;
      const T x = p.x[r * p.x_rs + c * p.x_cs], y = p.target[r * p.t_rs + c * p.t_cs];
      const T ax = x < (T)0 ? -x : x;
      acc += -y * x + (x > (T)0 ? x : (T)0) + dev_log1p<T>(dev_exp<T>(-ax));
    }
  }
  part[threadIdx.x] = acc;
  __syncthreads();
  for (int d = 128; d >= 1; d >>= 1) {
    if ((int)threadIdx.x < d) part[threadIdx.x] += part[threadIdx.x + d];
    __syncthreads();
  }
  if (threadIdx.x == 0) partial[blockIdx.x] = part[0];
}

// grad * (sigmoid(x) - y) / batch_size (nnp_sigmoid_cross_entropy.nim:47-62), sigmoid = 1 / (1 + exp(-x)).
template <typename T>
__global__ __launch_bounds__(256) void sigmoid_ce_backward(Args<T> p) {
  const int64_t total = p.rows * p.cols;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
    const int64_t r = i / p.cols, c = i - r * p.cols;
    const T x = p.x[r * p.x_rs + c * p.x_cs], y = p.target[r * p.t_rs + c * p.t_cs];
    const T sg = (T)1 / ((T)1 + dev_exp<T>(-x));
    p.out[r * p.o_rs + c * p.o_cs] = p.grad * (sg - y) / p.batch;
  }
}

// Whether the rows can be walked in 16-byte vectors: unit stride along the row, whole vectors, aligned row starts.
template <typename T>
static bool vec_ok(const Args<T>& p, bool dense, bool with_out) {
  constexpr int64_t V = 16 / (int64_t)sizeof(T);
  auto fits = [&](const void* base, int64_t rs, int64_t cs) {
    return cs == 1 && (uintptr_t)base % 16 == 0 && (p.rows == 1 || rs % V == 0);
  };
  if (p.cols % V != 0 || !fits(p.x, p.x_rs, p.x_cs)) return false;
  if (dense && !fits(p.target, p.t_rs, p.t_cs)) return false;
  if (with_out && !fits(p.out, p.o_rs, p.o_cs)) return false;
  return true;
}

static int lanes_for(int64_t cols) {
  int lanes = 1;
  while (lanes < cols && lanes < 64) lanes *= 2;
  return lanes;
}

template <typename T>
static int check_common(const char* fn, int64_t rows, int64_t cols, const void* x, const void* second) {
  if (rows < 0 || cols < 0) return fail(AM_E_SHAPE, "%s: negative extent", fn);
  if (rows > 0 && cols == 0) return fail(AM_E_SHAPE, "%s: rows without classes", fn);
  if (rows >= ((int64_t)1 << 31)) return fail(AM_E_SHAPE, "%s: too many rows", fn);
  if (rows > 0 && (!x || !second)) return fail(AM_E_ARG, "%s: null tensor pointer", fn);
  return AM_OK;
}

template <typename T, bool DENSE>
static int forward(const char* fn, int64_t rows, int64_t cols, const T* x, int64_t x_rs, int64_t x_cs, const T* target,
                   int64_t t_rs, int64_t t_cs, const int64_t* labels, int64_t l_s, T* loss) {
  if (!loss) return fail(AM_E_ARG, "%s: null result pointer", fn);
  AM_TRY(check_common<T>(fn, rows, cols, x, DENSE ? (const void*)target : (const void*)labels));
  if (rows == 0) { *loss = (T)0; return AM_OK; }   // the reference's early return for an empty batch
  AM_TRY(ensure_init());
  if (capturing()) return fail(AM_E_ARG, "%s: returns a value to the host, not allowed while a graph is being captured", fn);
  // [0, 256) the result; then one loss per row; then the sums of slices of 8192 of them, and of slices of those
  char* ws = (char*)gemm::splitk_workspace(256 + ((size_t)rows + (size_t)rows / 4096 + 16) * sizeof(T));
  if (!ws) return fail(AM_E_ALLOC, "%s: workspace unavailable", fn);
  Args<T> p = {};
  p.x = x; p.x_rs = x_rs; p.x_cs = x_cs; p.target = target; p.t_rs = t_rs; p.t_cs = t_cs; p.labels = labels; p.l_s = l_s;
  p.rows = rows; p.cols = cols; p.row_loss = (T*)(ws + 256);
  const bool vec = vec_ok<T>(p, DENSE, false);
  const int lanes = lanes_for(vec ? cols / (16 / (int64_t)sizeof(T)) : cols);
  const int64_t rows_per_wg = 4 * (64 / lanes);
  int64_t wgs = (rows + rows_per_wg - 1) / rows_per_wg;
  if (wgs > (int64_t)num_cus() * 16) wgs = (int64_t)num_cus() * 16;
  const dim3 grid((unsigned)wgs);
  const bool short_rows = (vec ? cols / (16 / (int64_t)sizeof(T)) : cols) <= lanes;   // one unit per lane at most
  if (vec && short_rows) hipLaunchKernelGGL((sce_forward<T, DENSE, true, true>), grid, dim3(256), 0, stream(), p, lanes);
  else if (vec) hipLaunchKernelGGL((sce_forward<T, DENSE, true, false>), grid, dim3(256), 0, stream(), p, lanes);
  else if (short_rows) hipLaunchKernelGGL((sce_forward<T, DENSE, false, true>), grid, dim3(256), 0, stream(), p, lanes);
  else hipLaunchKernelGGL((sce_forward<T, DENSE, false, false>), grid, dim3(256), 0, stream(), p, lanes);
  AM_TRY(check_launch("sce_forward"));
  // the rows' losses -> their mean at ws[0]: slices of 8192 (and of 8192 slices) while there are many
  const T* v = p.row_loss;
  int64_t n = rows;
  T* spare = (T*)(ws + 256) + rows;
  while (n > 8192) {
    const int64_t slices = (n + 8191) / 8192;
    hipLaunchKernelGGL((sum_slices<T>), dim3((unsigned)slices), dim3(256), 0, stream(), v, n, (int64_t)8192, (T)1, spare);
    AM_TRY(check_launch("sum_slices"));
    v = spare; n = slices; spare += slices;
  }
  hipLaunchKernelGGL((sum_slices<T>), dim3(1), dim3(256), 0, stream(), v, n, n, (T)rows, (T*)ws);
  AM_TRY(check_launch("sum_slices"));
  return fetch_result(loss, ws, sizeof(T));
}

template <typename T, bool DENSE>
static int backward(const char* fn, int64_t rows, int64_t cols, T gradient, const T* x, int64_t x_rs, int64_t x_cs,
                    const T* target, int64_t t_rs, int64_t t_cs, const int64_t* labels, int64_t l_s, T* out, int64_t o_rs,
                    int64_t o_cs) {
  AM_TRY(check_common<T>(fn, rows, cols, x, DENSE ? (const void*)target : (const void*)labels));
  if (rows == 0 || cols == 0) return AM_OK;
  if (!out) return fail(AM_E_ARG, "%s: null result pointer", fn);
  AM_TRY(ensure_init());
  Args<T> p = {};
  p.x = x; p.x_rs = x_rs; p.x_cs = x_cs; p.target = target; p.t_rs = t_rs; p.t_cs = t_cs; p.labels = labels; p.l_s = l_s;
  p.rows = rows; p.cols = cols; p.out = out; p.o_rs = o_rs; p.o_cs = o_cs; p.grad = gradient; p.batch = (T)rows;
  const bool vec = vec_ok<T>(p, DENSE, true);
  const int lanes = lanes_for(vec ? cols / (16 / (int64_t)sizeof(T)) : cols);
  const int64_t rows_per_wg = 4 * (64 / lanes);
  int64_t wgs = (rows + rows_per_wg - 1) / rows_per_wg;
  if (wgs > (int64_t)num_cus() * 16) wgs = (int64_t)num_cus() * 16;
  const dim3 grid((unsigned)wgs);
  const bool short_rows = (vec ? cols / (16 / (int64_t)sizeof(T)) : cols) <= lanes;
  if (vec && short_rows) hipLaunchKernelGGL((sce_backward<T, DENSE, true, true>), grid, dim3(256), 0, stream(), p, lanes);
  else if (vec) hipLaunchKernelGGL((sce_backward<T, DENSE, true, false>), grid, dim3(256), 0, stream(), p, lanes);
  else if (short_rows) hipLaunchKernelGGL((sce_backward<T, DENSE, false, true>), grid, dim3(256), 0, stream(), p, lanes);
  else hipLaunchKernelGGL((sce_backward<T, DENSE, false, false>), grid, dim3(256), 0, stream(), p, lanes);
  return check_launch("sce_backward");
}

template <typename T>
static int sigmoid_forward(const char* fn, int64_t rows, int64_t cols, const T* x, int64_t x_rs, int64_t x_cs, const T* target,
                           int64_t t_rs, int64_t t_cs, T* loss) {
  if (!loss) return fail(AM_E_ARG, "%s: null result pointer", fn);
  if (rows < 0 || cols < 0) return fail(AM_E_SHAPE, "%s: negative extent", fn);
  if (rows == 0) return fail(AM_E_SHAPE, "%s: empty batch (the reference divides by the batch size)", fn);
  if (cols == 0) { *loss = (T)0; return AM_OK; }
  if (!x || !target) return fail(AM_E_ARG, "%s: null tensor pointer", fn);
  AM_TRY(ensure_init());
  if (capturing()) return fail(AM_E_ARG, "%s: returns a value to the host, not allowed while a graph is being captured", fn);
  const int64_t total = rows * cols, blocks = (total + 2047) / 2048;
  if (blocks >= ((int64_t)1 << 31)) return fail(AM_E_SHAPE, "%s: too many elements", fn);
  char* ws = (char*)gemm::splitk_workspace(256 + ((size_t)blocks + (size_t)blocks / 4096 + 16) * sizeof(T));
  if (!ws) return fail(AM_E_ALLOC, "%s: workspace unavailable", fn);
  Args<T> p = {};
  p.x = x; p.x_rs = x_rs; p.x_cs = x_cs; p.target = target; p.t_rs = t_rs; p.t_cs = t_cs; p.rows = rows; p.cols = cols;
  T* partial = (T*)(ws + 256);
  hipLaunchKernelGGL((sigmoid_ce_partial<T>), dim3((unsigned)blocks), dim3(256), 0, stream(), p, partial);
  AM_TRY(check_launch("sigmoid_ce_partial"));
  const T* v = partial;
  int64_t n = blocks;
  T* spare = partial + blocks;
  while (n > 8192) {
    const int64_t slices = (n + 8191) / 8192;
    hipLaunchKernelGGL((sum_slices<T>), dim3((unsigned)slices), dim3(256), 0, stream(), v, n, (int64_t)8192, (T)1, spare);
    AM_TRY(check_launch("sum_slices"));
    v = spare; n = slices; spare += slices;
  }
  hipLaunchKernelGGL((sum_slices<T>), dim3(1), dim3(256), 0, stream(), v, n, n, (T)rows, (T*)ws);
  AM_TRY(check_launch("sum_slices"));
  return fetch_result(loss, ws, sizeof(T));
}

template <typename T>
static int sigmoid_backward(const char* fn, int64_t rows, int64_t cols, T gradient, const T* x, int64_t x_rs, int64_t x_cs,
                            const T* target, int64_t t_rs, int64_t t_cs, T* out, int64_t o_rs, int64_t o_cs) {
  if (rows < 0 || cols < 0) return fail(AM_E_SHAPE, "%s: negative extent", fn);
  if (rows == 0 || cols == 0) return AM_OK;
  if (!x || !target || !out) return fail(AM_E_ARG, "%s: null tensor pointer", fn);
  AM_TRY(ensure_init());
  Args<T> p = {};
  p.x = x; p.x_rs = x_rs; p.x_cs = x_cs; p.target = target; p.t_rs = t_rs; p.t_cs = t_cs; p.rows = rows; p.cols = cols;
  p.out = out; p.o_rs = o_rs; p.o_cs = o_cs; p.grad = gradient; p.batch = (T)rows;
  int64_t blocks = (rows * cols + 255) / 256;
  const int64_t cap = (int64_t)num_cus() * 32;
  if (blocks > cap) blocks = cap;
  hipLaunchKernelGGL((sigmoid_ce_backward<T>), dim3((unsigned)blocks), dim3(256), 0, stream(), p);
  return check_launch("sigmoid_ce_backward");
}

}  // namespace loss
}  // namespace am

using namespace am;

#define AM_LOSS_ENTRY_POINTS(T, SFX)                                                                                          \
  extern "C" int am_hip_softmax_cross_entropy_##SFX(int64_t rows, int64_t cols, const T* input, int64_t in_rs, int64_t in_cs, \
                                                    const T* target, int64_t t_rs, int64_t t_cs, T* loss) {                 \
    return loss::forward<T, true>("am_hip_softmax_cross_entropy_" #SFX, rows, cols, input, in_rs, in_cs, target, t_rs, t_cs, \
                                  nullptr, 0, loss);                                                                        \
  }                                                                                                                         \
  extern "C" int am_hip_sparse_softmax_cross_entropy_##SFX(int64_t rows, int64_t cols, const T* input, int64_t in_rs,       \
                                                           int64_t in_cs, const int64_t* labels, int64_t labels_s, T* loss) { \
    return loss::forward<T, false>("am_hip_sparse_softmax_cross_entropy_" #SFX, rows, cols, input, in_rs, in_cs, nullptr, 0, 0, \
                                   labels, labels_s, loss);                                                                 \
  }                                                                                                                         \
  extern "C" int am_hip_softmax_cross_entropy_backward_##SFX(int64_t rows, int64_t cols, T gradient, const T* input,        \
                                                             int64_t in_rs, int64_t in_cs, const T* target, int64_t t_rs,   \
                                                             int64_t t_cs, T* result, int64_t r_rs, int64_t r_cs) {        \
    return loss::backward<T, true>("am_hip_softmax_cross_entropy_backward_" #SFX, rows, cols, gradient, input, in_rs, in_cs, \
                                   target, t_rs, t_cs, nullptr, 0, result, r_rs, r_cs);                                     \
  }                                                                                                                         \
  extern "C" int am_hip_sparse_softmax_cross_entropy_backward_##SFX(int64_t rows, int64_t cols, T gradient, const T* input, \
                                                                    int64_t in_rs, int64_t in_cs, const int64_t* labels,    \
                                                                    int64_t labels_s, T* result, int64_t r_rs, int64_t r_cs) { \
    return loss::backward<T, false>("am_hip_sparse_softmax_cross_entropy_backward_" #SFX, rows, cols, gradient, input, in_rs, \
                                    in_cs, nullptr, 0, 0, labels, labels_s, result, r_rs, r_cs);                            \
  }
#define AM_SIGMOID_CE_ENTRY_POINTS(T, SFX)                                                                                   \
  extern "C" int am_hip_sigmoid_cross_entropy_##SFX(int64_t rows, int64_t cols, const T* input, int64_t in_rs, int64_t in_cs, \
                                                    const T* target, int64_t t_rs, int64_t t_cs, T* loss) {                 \
    return loss::sigmoid_forward<T>("am_hip_sigmoid_cross_entropy_" #SFX, rows, cols, input, in_rs, in_cs, target, t_rs, t_cs, loss); \
  }                                                                                                                         \
  extern "C" int am_hip_sigmoid_cross_entropy_backward_##SFX(int64_t rows, int64_t cols, T gradient, const T* input,        \
                                                             int64_t in_rs, int64_t in_cs, const T* target, int64_t t_rs,   \
                                                             int64_t t_cs, T* result, int64_t r_rs, int64_t r_cs) {        \
    return loss::sigmoid_backward<T>("am_hip_sigmoid_cross_entropy_backward_" #SFX, rows, cols, gradient, input, in_rs, in_cs, \
                                     target, t_rs, t_cs, result, r_rs, r_cs);                                               \
  }
AM_SIGMOID_CE_ENTRY_POINTS(float, f32)
AM_SIGMOID_CE_ENTRY_POINTS(double, f64)
AM_LOSS_ENTRY_POINTS(float, f32)
AM_LOSS_ENTRY_POINTS(double, f64)
