// Reductions, row softmax and 2-D max pooling on device memory.
//
//   am_hip_reduce_axis_*   sum / product / min / max along one axis of a strided tensor
//                          (reduce_axis_inline, src/arraymancer/tensor/higher_order_foldreduce.nim:46-61,
//                           used by sum/product/min/max(axis), src/arraymancer/tensor/aggregate.nim:38-113)
//   am_hip_reduce_all_*    the same over every element, result to the host
//                          (reduce_inline, higher_order_foldreduce.nim:22-31; aggregate.nim:33-36,46-49,89-106)
//   am_hip_softmax_rows_*  exp(x - max) / sum(exp(x - max)) per row
//                          (src/arraymancer/nn_primitives/nnp_softmax.nim:18-38, private/p_logsumexp.nim:30-62)
//   am_hip_maxpool2d_*     NCHW max pooling with the flat argmax indices the backward pass needs
//                          (src/arraymancer/nn_primitives/nnp_maxpooling.nim:19-66)
//
// All of it is HBM-bound. Two kernels cover the axis reductions:
//   * reduce_seq  one lane per output element, walking the axis front to back: consecutive lanes
//                 read consecutive outputs, so it streams whenever some other dimension has unit
//                 stride (e.g. sum over the rows of a row-major matrix). The fold order is the
//                 reference's (first slice, then each following slice), so float sums agree with a
//                 serial CPU fold bit for bit as long as the axis is not cut into chunks (below).
//   * reduce_row  one wavefront per output element, lanes striding along the axis (16-byte loads
//                 when it has unit stride), then a butterfly over the wavefront. Used when the
//                 axis itself is the unit-stride dimension. Float results differ from a serial fold
//                 by reassociation only.
// When there are too few outputs to fill the chip, the axis is cut into chunks whose partial
// results go to the library's workspace and are folded by a second pass.
#include <limits>
#include <string.h>
#include "common.h"
#include "fastdiv.h"

namespace am {
namespace gemm { void* splitk_workspace(size_t bytes); }
namespace red {

constexpr int kMaxDims = AM_MAXRANK;

template <typename T, int OP> struct Fold;
template <typename T> struct Fold<T, AM_RED_SUM> { static __device__ __forceinline__ T apply(T x, T y) { return x + y; } };
template <typename T> struct Fold<T, AM_RED_PROD> { static __device__ __forceinline__ T apply(T x, T y) { return x * y; } };
// Nim's min / max on ordered types: `if x <= y: x else: y` / `if y <= x: x else: y`.
template <typename T> struct Fold<T, AM_RED_MIN> { static __device__ __forceinline__ T apply(T x, T y) { return (x <= y) ? x : y; } };
template <typename T> struct Fold<T, AM_RED_MAX> { static __device__ __forceinline__ T apply(T x, T y) { return (y <= x) ? x : y; } };

// Integer sums and products wrap (two's complement), like the reference's `+=` / `*=` compiled
// without overflow checks (-d:danger) and like the integer GEMM: fold in the unsigned twin.
template <> struct Fold<int32_t, AM_RED_SUM> { static __device__ __forceinline__ int32_t apply(int32_t x, int32_t y) { return (int32_t)((uint32_t)x + (uint32_t)y); } };
template <> struct Fold<int64_t, AM_RED_SUM> { static __device__ __forceinline__ int64_t apply(int64_t x, int64_t y) { return (int64_t)((uint64_t)x + (uint64_t)y); } };
template <> struct Fold<int32_t, AM_RED_PROD> { static __device__ __forceinline__ int32_t apply(int32_t x, int32_t y) { return (int32_t)((uint32_t)x * (uint32_t)y); } };
template <> struct Fold<int64_t, AM_RED_PROD> { static __device__ __forceinline__ int64_t apply(int64_t x, int64_t y) { return (int64_t)((uint64_t)x * (uint64_t)y); } };

// The output elements: up to kMaxDims collapsed dimensions, slowest first.
template <typename T> struct Args {
  const T* a;
  T* dst;            // final destination (strided)
  T* ws;             // partial results [chunk][outputs] when chunks > 1
  int ndim;
  int64_t extent[kMaxDims], a_stride[kMaxDims], d_stride[kMaxDims];
  int64_t outputs;   // product of the extents
  int64_t L, a_axis_stride;   // reduced axis
  int chunks;
  int64_t chunk_len;
};

template <typename T>
__device__ __forceinline__ void decode(const Args<T>& p, int64_t o, int64_t& a_off, int64_t& d_off) {
  a_off = 0; d_off = 0;
#pragma unroll
  for (int d = kMaxDims - 1; d >= 0; --d) {
    if (d < p.ndim) {
      const int64_t q = o / p.extent[d], r = o - q * p.extent[d];
      a_off += r * p.a_stride[d];
      d_off += r * p.d_stride[d];
      o = q;
    }
  }
}

template <typename T, int OP>
__global__ __launch_bounds__(256) void reduce_seq(Args<T> p) {
  const int64_t o = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (o >= p.outputs) return;
  int64_t a_off, d_off;
  decode(p, o, a_off, d_off);
  const int64_t l0 = (int64_t)blockIdx.y * p.chunk_len;
  const int64_t l1 = (l0 + p.chunk_len < p.L) ? l0 + p.chunk_len : p.L;
  const T* src = p.a + a_off + l0 * p.a_axis_stride;
  T acc = *src;
  int64_t l = l0 + 1;
  // four loads in flight, folded in axis order
  for (; l + 4 <= l1; l += 4) {
    const T v0 = __builtin_nontemporal_load(p.a + a_off + l * p.a_axis_stride), v1 = __builtin_nontemporal_load(p.a + a_off + (l + 1) * p.a_axis_stride);
    const T v2 = __builtin_nontemporal_load(p.a + a_off + (l + 2) * p.a_axis_stride), v3 = __builtin_nontemporal_load(p.a + a_off + (l + 3) * p.a_axis_stride);
    acc = Fold<T, OP>::apply(acc, v0);
    acc = Fold<T, OP>::apply(acc, v1);
    acc = Fold<T, OP>::apply(acc, v2);
    acc = Fold<T, OP>::apply(acc, v3);
  }
  for (; l < l1; ++l) acc = Fold<T, OP>::apply(acc, p.a[a_off + l * p.a_axis_stride]);
  if (p.chunks > 1) p.ws[(int64_t)blockIdx.y * p.outputs + o] = acc;
  else p.dst[d_off] = acc;
}

// (Column walks load non-temporally: measured 10 % faster, also when the tensor would fit the memory-side
// cache; the wavefront-per-output kernels are faster with ordinary loads.)
// The same walk with one lane per 16 bytes of adjacent outputs (the innermost output dimension has
// unit stride in the source and the destination): 16-byte loads, eight in flight, every output
// still folded front to back along the axis, so the results are those of reduce_seq bit for bit.
template <typename T, int OP>
__global__ __launch_bounds__(256) void reduce_seq_vec(Args<T> p) {
  constexpr int V = 16 / (int)sizeof(T);
  constexpr int U = 8;
  typedef T vec_t __attribute__((ext_vector_type(V)));
  const int64_t ov = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (ov * V >= p.outputs) return;
  int64_t a_off, d_off;
  decode(p, ov * V, a_off, d_off);
  const int64_t l0 = (int64_t)blockIdx.y * p.chunk_len;
  const int64_t l1 = (l0 + p.chunk_len < p.L) ? l0 + p.chunk_len : p.L;
  const T* src = p.a + a_off;
  vec_t acc = *(const vec_t*)(src + l0 * p.a_axis_stride);
  int64_t l = l0 + 1;
  auto fold = [&](const vec_t& x) {
#pragma unroll
    for (int e = 0; e < V; ++e) acc[e] = Fold<T, OP>::apply(acc[e], x[e]);
  };
  for (; l + U <= l1; l += U) {
    vec_t x[U];
#pragma unroll
    for (int u = 0; u < U; ++u) x[u] = __builtin_nontemporal_load((const vec_t*)(src + (l + u) * p.a_axis_stride));
#pragma unroll
    for (int u = 0; u < U; ++u) fold(x[u]);
  }
  for (; l < l1; ++l) fold(*(const vec_t*)(src + l * p.a_axis_stride));
  if (p.chunks > 1) *(vec_t*)(p.ws + (int64_t)blockIdx.y * p.outputs + ov * V) = acc;
  else *(vec_t*)(p.dst + d_off) = acc;
}

// Butterfly over the 64 lanes; lanes without an element (has == false) are skipped, so no
// identity value is ever mixed in (a sum of negative zeros stays a negative zero).
template <typename T, int OP>
__device__ __forceinline__ void wave_fold(T& acc, bool& has) {
#pragma unroll
  for (int d = 32; d >= 1; d >>= 1) {
    const T other = __shfl_xor(acc, d, 64);
    const int other_has = __shfl_xor((int)has, d, 64);
    // a fixed pairing and operand order: the result is the same on every run
    const bool low = ((threadIdx.x & 63) & d) == 0;
    if (other_has) {
      if (has) acc = low ? Fold<T, OP>::apply(acc, other) : Fold<T, OP>::apply(other, acc);
      else acc = other;
      has = true;
    }
  }
}

template <typename T, int OP, bool VEC, bool STREAM>
__global__ __launch_bounds__(256) void reduce_row(Args<T> p) {
  constexpr int V = 16 / (int)sizeof(T);
  typedef T vec_t __attribute__((ext_vector_type(V)));
  const int lane = threadIdx.x & 63;
  // one wavefront per (output, chunk) pair
  const int64_t unit = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (unit >= p.outputs * p.chunks) return;
  const int64_t chunk = unit / p.outputs, o = unit - chunk * p.outputs;
  int64_t a_off, d_off;
  decode(p, o, a_off, d_off);
  const int64_t l0 = chunk * p.chunk_len;
  const int64_t l1 = (l0 + p.chunk_len < p.L) ? l0 + p.chunk_len : p.L;
  T acc = (T)0;
  bool has = false;
  auto take = [&](T x) { acc = has ? Fold<T, OP>::apply(acc, x) : x; has = true; };
  auto take_vec = [&](vec_t x) {
    T part = x[0];
#pragma unroll
    for (int e = 1; e < V; ++e) part = Fold<T, OP>::apply(part, x[e]);
    take(part);
  };
  if constexpr (VEC) {   // unit stride along the axis, every chunk start 16-byte aligned
    const vec_t* src = (const vec_t*)(p.a + a_off + l0);
    const int64_t nvec = (l1 - l0) / V;
    int64_t v = lane;
    for (; v + 192 < nvec; v += 256) {   // four 16-byte loads in flight per lane
      vec_t x0, x1, x2, x3;
      if constexpr (STREAM) {   // a template parameter: a run-time branch is merged back into ordinary loads
        x0 = __builtin_nontemporal_load(src + v); x1 = __builtin_nontemporal_load(src + v + 64);
        x2 = __builtin_nontemporal_load(src + v + 128); x3 = __builtin_nontemporal_load(src + v + 192);
      } else {
        x0 = src[v]; x1 = src[v + 64]; x2 = src[v + 128]; x3 = src[v + 192];
      }
      take_vec(x0); take_vec(x1); take_vec(x2); take_vec(x3);
    }
    for (; v < nvec; v += 64) take_vec(src[v]);
    for (int64_t l = l0 + nvec * V + lane; l < l1; l += 64) take(p.a[a_off + l]);
  } else {
    for (int64_t l = l0 + lane; l < l1; l += 64) take(p.a[a_off + l * p.a_axis_stride]);
  }
  wave_fold<T, OP>(acc, has);
  if (lane == 0) {
    if (p.chunks > 1) p.ws[chunk * p.outputs + o] = acc;
    else p.dst[d_off] = acc;
  }
}

// A walk down the rows of a matrix with FEW columns (the bias gradient of a dense layer, sum(gradOutput, axis = 0) over
// [batch x features], nnp_linear.nim:55): one lane per 16 bytes of outputs leaves most of a workgroup idle, and a
// wavefront per output reads one element per row, a cache line apart. Here the 256 lanes of a workgroup are laid over
// cxw lanes along the columns x 256 / cxw rows: a load instruction of the workgroup covers whole rows side by side (one
// contiguous run when the matrix is), each lane walks every (256 / cxw)-th row of the workgroup's chunk of the axis with
// eight loads in flight, and the row classes are folded through LDS in a fixed order. grid = (column blocks, chunks of
// the axis); chunk partials go to the workspace and a second launch of the same kernel folds them, this time cut along
// the columns (8 lanes wide), so that it is as parallel as the first.
// Measured, f32 sum over axis 0: [65536 x 512] 198 us before (a wavefront per column) -> 27 us; [1048576 x 64] 373 -> 48 us.
template <typename T, int OP>
__global__ __launch_bounds__(256) void reduce_cols_narrow(Args<T> p, int cxw) {
  constexpr int V = 16 / (int)sizeof(T);
  constexpr int U = 8;
  typedef T vec_t __attribute__((ext_vector_type(V)));
  __shared__ vec_t part[256];
  __shared__ int part_has[256];
  const int ry = 256 / cxw;
  const int x = (int)threadIdx.x % cxw, y = (int)threadIdx.x / cxw;
  const int64_t col = ((int64_t)blockIdx.x * cxw + x) * V;
  const bool active = y < ry && col < p.outputs;
  const int64_t l0 = (int64_t)blockIdx.y * p.chunk_len;
  const int64_t l1 = (l0 + p.chunk_len < p.L) ? l0 + p.chunk_len : p.L;
  vec_t acc;
#pragma unroll
  for (int e = 0; e < V; ++e) acc[e] = (T)0;
  bool has = false;
  auto fold = [&](const vec_t& v) {
    if (has) {
#pragma unroll
      for (int e = 0; e < V; ++e) acc[e] = Fold<T, OP>::apply(acc[e], v[e]);
    } else {
      acc = v; has = true;
    }
  };
  if (active) {
    const T* src = p.a + col;
    int64_t l = l0 + y;
    for (; l + (int64_t)(U - 1) * ry < l1; l += (int64_t)U * ry) {
      vec_t v[U];
#pragma unroll
      for (int u = 0; u < U; ++u) v[u] = __builtin_nontemporal_load((const vec_t*)(src + (l + (int64_t)u * ry) * p.a_axis_stride));
#pragma unroll
      for (int u = 0; u < U; ++u) fold(v[u]);
    }
    for (; l < l1; l += ry) fold(*(const vec_t*)(src + l * p.a_axis_stride));
  }
  part[threadIdx.x] = acc;
  part_has[threadIdx.x] = has ? 1 : 0;
  __syncthreads();
  if (active && y == 0) {
    for (int yy = 1; yy < ry; ++yy)
      if (part_has[yy * cxw + x]) fold(part[yy * cxw + x]);
    if (p.chunks > 1) *(vec_t*)(p.ws + (int64_t)blockIdx.y * p.outputs + col) = acc;
    else *(vec_t*)(p.dst + col) = acc;
  }
}

// Whether reduce_cols_narrow applies: the outputs are one unit-stride run in the source and the destination, at most
// half a workgroup of 16-byte lanes wide, everything 16-byte aligned, and the axis is not the unit-stride direction.
template <typename T>
static bool cols_narrow_ok(const Args<T>& g) {
  constexpr int64_t V = 16 / (int64_t)sizeof(T);
  if (g.ndim != 1 || g.a_stride[0] != 1 || g.d_stride[0] != 1) return false;
  if (g.outputs % V != 0 || g.outputs / V > 128 || g.L < 512) return false;
  if (g.a_axis_stride < g.outputs || g.a_axis_stride % V != 0) return false;
  return (uintptr_t)g.a % 16 == 0 && (uintptr_t)g.dst % 16 == 0;
}

template <typename T, int OP>
static int launch_cols_narrow(Args<T>& g) {
  constexpr int64_t V = 16 / (int64_t)sizeof(T);
  const int cx = (int)(g.outputs / V);
  int64_t chunks = (int64_t)num_cus() * 4;
  if (chunks > g.L / 256) chunks = g.L / 256;
  if (chunks < 1) chunks = 1;
  int64_t len = (g.L + chunks - 1) / chunks;
  chunks = (g.L + len - 1) / len;
  g.chunks = 1; g.chunk_len = g.L; g.ws = nullptr;
  if (chunks > 1) {
    char* base = (char*)gemm::splitk_workspace((size_t)chunks * (size_t)g.outputs * sizeof(T));
    if (base) { g.chunks = (int)chunks; g.chunk_len = len; g.ws = (T*)base; }
  }
  hipLaunchKernelGGL((reduce_cols_narrow<T, OP>), dim3(1, (unsigned)g.chunks), dim3(256), 0, stream(), g, cx);
  AM_TRY(check_launch("reduce_cols_narrow"));
  if (g.chunks > 1) {
    Args<T> r = g;
    r.a = g.ws; r.L = g.chunks; r.a_axis_stride = g.outputs;
    r.chunks = 1; r.chunk_len = r.L; r.ws = nullptr;
    const int cxw = cx < 8 ? cx : 8;
    hipLaunchKernelGGL((reduce_cols_narrow<T, OP>), dim3((unsigned)((cx + cxw - 1) / cxw), 1), dim3(256), 0, stream(), r, cxw);
    AM_TRY(check_launch("reduce_cols_narrow (second pass)"));
  }
  return AM_OK;
}

template <typename T>
static int dispatch_cols_narrow(int op, Args<T>& g) {
  switch (op) {
    case AM_RED_SUM: return launch_cols_narrow<T, AM_RED_SUM>(g);
    case AM_RED_PROD: return launch_cols_narrow<T, AM_RED_PROD>(g);
    case AM_RED_MIN: return launch_cols_narrow<T, AM_RED_MIN>(g);
    default: return launch_cols_narrow<T, AM_RED_MAX>(g);
  }
}

// Many SHORT rows folded along their unit-stride axis (row sums of [rows x 4 ... 1024] tensors): a wavefront per
// row would move 16 ... 4096 bytes per six-step butterfly, a lane per row reads 16 bytes of every cache line it touches
// per instruction. Here `lanes` lanes (a power of two <= 64) share a row, VPL 16-byte vectors each (1, 2 or 4: rows
// of up to 256 vectors), so that a wavefront's load instruction is one contiguous run of 64 / lanes rows; each lane folds
// its vectors in element order, then the lanes of a row fold in a fixed butterfly. Several row groups per wavefront are
// in flight (eight loads per lane).
// Measured, f32 sum over axis 1: [1048576 x 64] 260 us before (a wavefront per row) -> 48 us; [4194304 x 16] 154 -> 51 us.
template <typename T, int OP, bool STREAM, int VPL>
__global__ __launch_bounds__(256) void reduce_rows_short(Args<T> p, int lanes) {
  constexpr int V = 16 / (int)sizeof(T);
  constexpr int U = VPL >= 4 ? 2 : 4;
  typedef T vec_t __attribute__((ext_vector_type(V)));
  const int lane = threadIdx.x & 63;
  const int j = lane & (lanes - 1), sub = lane / lanes, rows_per_step = 64 / lanes;
  const int64_t wave = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  const int64_t row0 = wave * (int64_t)(U * rows_per_step) + sub;
  const int64_t nvec = p.L / V;
  vec_t x[U][VPL];
  bool ok[U];
  int64_t d_off[U];
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const int64_t o = row0 + (int64_t)u * rows_per_step;
    ok[u] = o < p.outputs;
    int64_t a_off;
    decode(p, ok[u] ? o : 0, a_off, d_off[u]);
    const vec_t* row = (const vec_t*)(p.a + a_off);
#pragma unroll
    for (int w = 0; w < VPL; ++w) {
      const int64_t v = j + (int64_t)w * lanes;
      const vec_t* at = row + (v < nvec ? v : 0);   // every lane loads, from inside its row
      if constexpr (STREAM) x[u][w] = __builtin_nontemporal_load(at); else x[u][w] = *at;
    }
  }
#pragma unroll
  for (int u = 0; u < U; ++u) {
    T acc = (T)0;
    bool has = false;
#pragma unroll
    for (int w = 0; w < VPL; ++w) {
      if (j + (int64_t)w * lanes < nvec) {
        T part = x[u][w][0];
#pragma unroll
        for (int e = 1; e < V; ++e) part = Fold<T, OP>::apply(part, x[u][w][e]);
        acc = has ? Fold<T, OP>::apply(acc, part) : part;
        has = true;
      }
    }
    has = has && ok[u];
    for (int d = lanes >> 1; d >= 1; d >>= 1) {
      const T other = __shfl_xor(acc, d, 64);
      const int other_has = __shfl_xor((int)has, d, 64);
      const bool low = (lane & d) == 0;
      if (other_has) {
        if (has) acc = low ? Fold<T, OP>::apply(acc, other) : Fold<T, OP>::apply(other, acc);
        else acc = other;
        has = true;
      }
    }
    if (j == 0 && ok[u]) p.dst[d_off[u]] = acc;
  }
}

// Whether reduce_rows_short applies, and with how many lanes per row (*vpl: 16-byte vectors per lane, 1, 2 or 4).
template <typename T>
static int rows_short_lanes(const Args<T>& g, int* vpl) {
  constexpr int64_t V = 16 / (int64_t)sizeof(T);
  if (g.a_axis_stride != 1 || g.L % V != 0 || g.L / V > 256 || g.outputs < 4096) return 0;
  if ((uintptr_t)g.a % 16 != 0) return 0;
  for (int d = 0; d < g.ndim; ++d)
    if (g.a_stride[d] % V != 0) return 0;
  int lanes = 1;
  while (lanes < g.L / V && lanes < 64) lanes *= 2;
  const int64_t per_lane = (g.L / V + lanes - 1) / lanes;
  *vpl = per_lane <= 1 ? 1 : per_lane <= 2 ? 2 : 4;
  return lanes;
}

template <typename T, int VPL>
static int dispatch_rows_short_vpl(int op, Args<T>& g, int lanes) {
  constexpr int U = VPL >= 4 ? 2 : 4;
  const int64_t rows_per_wg = 4 * U * (64 / lanes);
  const int64_t bx = (g.outputs + rows_per_wg - 1) / rows_per_wg;
  if (bx >= ((int64_t)1 << 31)) return fail(AM_E_SHAPE, "reduce: too many output elements");
  g.chunks = 1; g.chunk_len = g.L; g.ws = nullptr;
  const bool stream_loads = (double)g.outputs * (double)g.L * sizeof(T) > nt_threshold_bytes();
  const dim3 grid((unsigned)bx), block(256);
#define AM_ROWS_SHORT(OPC)                                                                                               \
  do {                                                                                                                   \
    if (stream_loads) hipLaunchKernelGGL((reduce_rows_short<T, OPC, true, VPL>), grid, block, 0, stream(), g, lanes);    \
    else hipLaunchKernelGGL((reduce_rows_short<T, OPC, false, VPL>), grid, block, 0, stream(), g, lanes);                \
  } while (0)
  switch (op) {
    case AM_RED_SUM: AM_ROWS_SHORT(AM_RED_SUM); break;
    case AM_RED_PROD: AM_ROWS_SHORT(AM_RED_PROD); break;
    case AM_RED_MIN: AM_ROWS_SHORT(AM_RED_MIN); break;
    default: AM_ROWS_SHORT(AM_RED_MAX); break;
  }
#undef AM_ROWS_SHORT
  return check_launch("reduce_rows_short");
}

template <typename T>
static int dispatch_rows_short(int op, Args<T>& g, int lanes, int vpl) {
  if (vpl == 1) return dispatch_rows_short_vpl<T, 1>(op, g, lanes);
  if (vpl == 2) return dispatch_rows_short_vpl<T, 2>(op, g, lanes);
  return dispatch_rows_short_vpl<T, 4>(op, g, lanes);
}

// Whether reduce_seq_vec applies: the innermost output dimension is a unit-stride run in the source
// and the destination whose length, like every other stride, is a multiple of the 16-byte vector,
// and both base pointers are 16-byte aligned.
// Workgroups per CU the axis is cut for: fewer, longer column walks measured fastest (f64 8192 x 8192:
// 97 us with 1 or 2, 114-125 us with 4 to 16; 4-byte types do not care).
constexpr int64_t kSeqVecUnits = 1;
template <typename T>
static bool seq_vec_ok(const Args<T>& g) {
  constexpr int64_t V = 16 / (int64_t)sizeof(T);
  if (g.ndim < 1 || g.outputs < 256 * V) return false;
  const int last = g.ndim - 1;
  if (g.a_stride[last] != 1 || g.d_stride[last] != 1 || g.extent[last] % V != 0) return false;
  if ((uintptr_t)g.a % 16 != 0 || (uintptr_t)g.dst % 16 != 0 || g.a_axis_stride % V != 0) return false;
  for (int d = 0; d < last; ++d)
    if (g.a_stride[d] % V != 0 || g.d_stride[d] % V != 0) return false;
  return true;
}

// ws_off: bytes at the start of the library workspace that the caller keeps for itself (the
// chunk partials of this call go after them).
template <typename T, int OP>
static int launch(Args<T>& g, bool row_kernel, size_t ws_off) {
  constexpr int64_t V = 16 / (int64_t)sizeof(T);
  const int64_t cus = num_cus();
  // Enough independent work for the whole chip: if the outputs alone do not supply it, cut the axis.
  const bool seq_vec = !row_kernel && seq_vec_ok(g);
  const int64_t units = row_kernel ? g.outputs : seq_vec ? (g.outputs / V + 255) / 256 : (g.outputs + 255) / 256;   // wavefronts resp. workgroups
  const int64_t want_units = row_kernel ? cus * 32 : seq_vec ? cus * kSeqVecUnits : cus * 8;
  const int64_t min_chunk = row_kernel ? 4096 : 64;
  int64_t chunks = 1;
  if (units < want_units && g.L >= 2 * min_chunk) {
    chunks = (want_units + units - 1) / units;
    if (chunks > g.L / min_chunk) chunks = g.L / min_chunk;
    if (chunks > 8192) chunks = 8192;
  }
  g.chunks = 1; g.chunk_len = g.L; g.ws = nullptr;
  // Inputs beyond what the L2s hold are read with non-temporal loads: 8192 x 8192 f32 row sums over rotating
  // buffers (every byte from HBM) 47.2 -> 42.8 us; the same buffer every launch, which the memory-side cache
  // partly holds, 40.4 -> 41.7 us.
  bool stream_loads = (double)g.outputs * (double)g.L * sizeof(T) > nt_threshold_bytes();
  if (chunks > 1) {
    int64_t len = (g.L + chunks - 1) / chunks;
    len = (len + V - 1) / V * V;                    // chunk starts stay 16-byte aligned
    chunks = (g.L + len - 1) / len;
    char* base = (chunks > 1) ? (char*)gemm::splitk_workspace(ws_off + (size_t)chunks * (size_t)g.outputs * sizeof(T)) : nullptr;
    if (base) { g.chunks = (int)chunks; g.chunk_len = len; g.ws = (T*)(base + ws_off); }
  }
  if (row_kernel) {
    bool vec = g.a_axis_stride == 1 && ((uintptr_t)g.a % 16 == 0);
    for (int d = 0; d < g.ndim && vec; ++d) vec = (g.a_stride[d] % V == 0) || g.extent[d] == 1;
    const int64_t bx = (g.outputs * g.chunks + 3) / 4;
    if (bx >= ((int64_t)1 << 31)) return fail(AM_E_SHAPE, "reduce: too many output elements");
    const dim3 grid((unsigned)bx), block(256);
    if (vec && stream_loads) hipLaunchKernelGGL((reduce_row<T, OP, true, true>), grid, block, 0, stream(), g);
    else if (vec) hipLaunchKernelGGL((reduce_row<T, OP, true, false>), grid, block, 0, stream(), g);
    else hipLaunchKernelGGL((reduce_row<T, OP, false, false>), grid, block, 0, stream(), g);
  } else if (seq_vec) {
    const int64_t bx = (g.outputs / V + 255) / 256;
    hipLaunchKernelGGL((reduce_seq_vec<T, OP>), dim3((unsigned)bx, (unsigned)g.chunks), dim3(256), 0, stream(), g);
  } else {
    const int64_t bx = (g.outputs + 255) / 256;
    if (bx >= ((int64_t)1 << 31)) return fail(AM_E_SHAPE, "reduce: too many output elements");
    hipLaunchKernelGGL((reduce_seq<T, OP>), dim3((unsigned)bx, (unsigned)g.chunks), dim3(256), 0, stream(), g);
  }
  AM_TRY(check_launch("reduce"));
  if (g.chunks > 1) {   // fold the partials [chunk][outputs] front to back into dst
    Args<T> r = g;
    r.a = g.ws;
    r.L = g.chunks; r.a_axis_stride = g.outputs;
    int64_t s = 1;
    for (int d = g.ndim - 1; d >= 0; --d) { r.a_stride[d] = s; s *= g.extent[d]; }
    r.chunks = 1; r.chunk_len = r.L; r.ws = nullptr;
    if (g.outputs < 1024 && g.chunks >= 64) {   // few outputs, many partials: a wavefront per output
      const int64_t bx = (g.outputs + 3) / 4;
      // a single output: its partials are one run of memory, read 16 bytes per lane
      if (g.outputs == 1 && (uintptr_t)r.a % 16 == 0) hipLaunchKernelGGL((reduce_row<T, OP, true, false>), dim3((unsigned)bx), dim3(256), 0, stream(), r);
      else hipLaunchKernelGGL((reduce_row<T, OP, false, false>), dim3((unsigned)bx), dim3(256), 0, stream(), r);
    } else if (seq_vec) {   // the partials are laid out like the outputs, so the same test holds for them
      const int64_t bx = (g.outputs / V + 255) / 256;
      hipLaunchKernelGGL((reduce_seq_vec<T, OP>), dim3((unsigned)bx, 1), dim3(256), 0, stream(), r);
    } else {
      const int64_t bx = (g.outputs + 255) / 256;
      hipLaunchKernelGGL((reduce_seq<T, OP>), dim3((unsigned)bx, 1), dim3(256), 0, stream(), r);
    }
    AM_TRY(check_launch("reduce (second pass)"));
  }
  return AM_OK;
}

template <typename T>
static int dispatch(int op, Args<T>& g, bool row_kernel, size_t ws_off) {
  switch (op) {
    case AM_RED_SUM: return launch<T, AM_RED_SUM>(g, row_kernel, ws_off);
    case AM_RED_PROD: return launch<T, AM_RED_PROD>(g, row_kernel, ws_off);
    case AM_RED_MIN: return launch<T, AM_RED_MIN>(g, row_kernel, ws_off);
    default: return launch<T, AM_RED_MAX>(g, row_kernel, ws_off);
  }
}

// Fills the output dimensions of `g` from every dimension but `axis`, merging neighbours that are
// contiguous with each other in both the source and the destination.
template <typename T>
static void set_outputs(Args<T>& g, int rank, const int64_t* shape, int axis, const int64_t* sa, const int64_t* sd) {
  g.ndim = 0; g.outputs = 1;
  for (int d = 0; d < rank; ++d) {
    if (d == axis || shape[d] == 1) continue;
    const int64_t ds = sd ? sd[d] : 0;
    if (g.ndim > 0 && g.a_stride[g.ndim - 1] == sa[d] * shape[d] && (!sd || g.d_stride[g.ndim - 1] == ds * shape[d])) {
      g.extent[g.ndim - 1] *= shape[d];
      g.a_stride[g.ndim - 1] = sa[d];
      g.d_stride[g.ndim - 1] = ds;
    } else {
      g.extent[g.ndim] = shape[d]; g.a_stride[g.ndim] = sa[d]; g.d_stride[g.ndim] = ds;
      ++g.ndim;
    }
    g.outputs *= shape[d];
  }
  for (int d = g.ndim; d < kMaxDims; ++d) { g.extent[d] = 1; g.a_stride[d] = 0; g.d_stride[d] = 0; }
}

static inline int64_t iabs64(int64_t v) { return v < 0 ? -v : v; }

template <typename T>
static int reduce_axis(const char* fn, int op, int rank, const int64_t* shape, int axis, T* dst, const int64_t* sd,
                       const T* a, const int64_t* sa) {
  if (op < AM_RED_SUM || op > AM_RED_MAX) return fail(AM_E_ARG, "%s: unknown reduction %d", fn, op);
  if (rank < 1 || rank > AM_MAXRANK) return fail(AM_E_SHAPE, "%s: rank %d outside 1..%d", fn, rank, AM_MAXRANK);
  if (!shape || !sd || !sa) return fail(AM_E_ARG, "%s: null shape or strides", fn);
  // IndexDefect of reduce_axis_inline (higher_order_foldreduce.nim:50-54)
  if (axis < 0 || axis >= rank) return fail(AM_E_SHAPE, "%s: axis %d outside the tensor's rank %d", fn, axis, rank);
  int64_t size = 1;
  for (int d = 0; d < rank; ++d) {
    if (shape[d] < 0) return fail(AM_E_SHAPE, "%s: negative extent", fn);
    size *= shape[d];
  }
  if (size == 0) return AM_OK;   // returnEmptyIfEmpty (aggregate.nim:40)
  if (!dst || !a) return fail(AM_E_ARG, "%s: null tensor pointer", fn);
  AM_TRY(ensure_init());
  Args<T> g;
  memset(&g, 0, sizeof(g));
  g.a = a; g.dst = dst;
  set_outputs(g, rank, shape, axis, sa, sd);
  g.L = shape[axis]; g.a_axis_stride = sa[axis];
  // The wavefront-per-output kernel when the axis is the cheapest direction to walk and long
  // enough to feed 64 lanes; else one lane per output.
  int64_t best_other = -1;
  for (int d = 0; d < g.ndim; ++d) if (best_other < 0 || iabs64(g.a_stride[d]) < best_other) best_other = iabs64(g.a_stride[d]);
  if (best_other >= 0 && iabs64(g.a_axis_stride) > best_other && cols_narrow_ok(g)) return dispatch_cols_narrow<T>(op, g);
  {
    int vpl = 1;
    if (const int lanes = rows_short_lanes(g, &vpl)) return dispatch_rows_short<T>(op, g, lanes, vpl);
  }
  const bool row_kernel = g.L >= 64 && (best_other < 0 || iabs64(g.a_axis_stride) < best_other || g.outputs < 1024);
  return dispatch<T>(op, g, row_kernel, 0);
}

template <typename T>
static int reduce_all(const char* fn, int op, int rank, const int64_t* shape, const T* a, const int64_t* sa, T* result) {
  if (!result) return fail(AM_E_ARG, "%s: null result pointer", fn);
  if (op < AM_RED_SUM || op > AM_RED_MAX) return fail(AM_E_ARG, "%s: unknown reduction %d", fn, op);
  if (rank < 0 || rank > AM_MAXRANK) return fail(AM_E_SHAPE, "%s: rank %d outside 0..%d", fn, rank, AM_MAXRANK);
  if (rank > 0 && (!shape || !sa)) return fail(AM_E_ARG, "%s: null shape or strides", fn);
  int64_t size = 1;
  for (int d = 0; d < rank; ++d) {
    if (shape[d] < 0) return fail(AM_E_SHAPE, "%s: negative extent", fn);
    size *= shape[d];
  }
  // reduce_inline starts from the first element: nothing to start from in an empty tensor
  if (size == 0) return fail(AM_E_SHAPE, "%s: reduction of an empty tensor", fn);
  if (!a) return fail(AM_E_ARG, "%s: null tensor pointer", fn);
  AM_TRY(ensure_init());
  if (capturing()) return fail(AM_E_ARG, "%s: returns a value to the host, not allowed while a graph is being captured", fn);
  // Dimensions merged where contiguous; a tensor that is one run of memory is a single "row".
  Args<T> g;
  memset(&g, 0, sizeof(g));
  set_outputs(g, rank, shape, -1, sa, nullptr);
  // workspace layout: [0, 256) the result; [256, 256 + tmp) one partial per run of a strided
  // tensor; then the chunk partials of whichever step is running
  T* out = (T*)gemm::splitk_workspace(256);
  if (!out) return fail(AM_E_ALLOC, "%s: workspace unavailable", fn);
  Args<T> r;
  memset(&r, 0, sizeof(r));
  r.dst = out; r.ndim = 0; r.outputs = 1;
  for (int d = 0; d < kMaxDims; ++d) r.extent[d] = 1;
  if (g.ndim <= 1) {
    r.a = a;
    r.L = g.ndim == 1 ? g.extent[0] : 1;
    r.a_axis_stride = g.ndim == 1 ? g.a_stride[0] : 1;
    AM_TRY(dispatch<T>(op, r, r.L >= 64, 256));
  } else {
    // several runs of memory: fold the last (collapsed) dimension of each run into a temporary in
    // the workspace, then fold that contiguous temporary
    const int last = g.ndim - 1;
    const int64_t rows = g.outputs / g.extent[last];
    const size_t tmp_bytes = ((size_t)rows * sizeof(T) + 255) / 256 * 256;
    // The per-run partials live in the workspace while they fit beside the chunk partials; a tensor of very
    // many short runs (a stepped slice [4M, k], a tall transposed view) takes them from the block cache
    // instead and gives them back once the value is on the host.
    const bool in_ws = tmp_bytes <= (size_t)16 * 1024 * 1024;
    void* big = nullptr;
    T* tmp;
    if (in_ws) {
      char* base = (char*)gemm::splitk_workspace(256 + tmp_bytes);
      if (!base) return fail(AM_E_ALLOC, "%s: workspace unavailable", fn);
      tmp = (T*)(base + 256);
    } else {
      AM_TRY(am_hip_malloc(tmp_bytes, &big));
      tmp = (T*)big;
    }
    const size_t ws_off = in_ws ? 256 + tmp_bytes : 256;
    Args<T> s;
    memset(&s, 0, sizeof(s));
    s.a = a; s.dst = tmp;
    s.ndim = last; s.outputs = rows;
    int64_t cs = 1;
    for (int d = last - 1; d >= 0; --d) { s.extent[d] = g.extent[d]; s.a_stride[d] = g.a_stride[d]; s.d_stride[d] = cs; cs *= g.extent[d]; }
    for (int d = last; d < kMaxDims; ++d) { s.extent[d] = 1; s.a_stride[d] = 0; s.d_stride[d] = 0; }
    s.L = g.extent[last]; s.a_axis_stride = g.a_stride[last];
    int rc = dispatch<T>(op, s, s.L >= 64, ws_off);
    if (rc == AM_OK) {
      r.a = tmp; r.L = rows; r.a_axis_stride = 1;
      rc = dispatch<T>(op, r, r.L >= 64, ws_off);
    }
    if (rc == AM_OK) rc = fetch_result(result, out, sizeof(T));   // blocking: the partials are no longer in use afterwards
    if (big) (void)am_hip_free(big);
    return rc;
  }
  return fetch_result(result, out, sizeof(T));
}

// ------------------------------------------------------------------------------------------------
// Index and value of the first maximum (or minimum) along an axis: argmax_max / argmin_min of the
// reference (src/arraymancer/tensor/aggregate.nim:159-193, 216-250). It starts from slice 0 and
// replaces the running value only on a strict `>` (`<`), so ties keep the lowest index, a NaN in
// slice 0 stays (nothing compares greater than it) and a NaN elsewhere is never taken.
template <typename T> struct ArgArgs {
  const T* a; T* val; int64_t* idx;
  int ndim;
  int64_t extent[kMaxDims], a_stride[kMaxDims], v_stride[kMaxDims], i_stride[kMaxDims];
  int64_t outputs, L, a_axis_stride;
  // the axis cut into chunks (one-lane-per-output kernel, too few outputs to fill the chip): partial
  // values and positions [chunk][output] in the workspace, position -1 = nothing but NaN in the chunk
  int chunks; int64_t chunk_len; T* ws_val; int64_t* ws_idx;
};

template <typename T>
__device__ __forceinline__ void decode3(const ArgArgs<T>& p, int64_t o, int64_t& a_off, int64_t& v_off, int64_t& i_off) {
  a_off = 0; v_off = 0; i_off = 0;
#pragma unroll
  for (int d = kMaxDims - 1; d >= 0; --d) {
    if (d < p.ndim) {
      const int64_t q = o / p.extent[d], r = o - q * p.extent[d];
      a_off += r * p.a_stride[d];
      v_off += r * p.v_stride[d];
      i_off += r * p.i_stride[d];
      o = q;
    }
  }
}

template <typename T, bool MAXOP> __device__ __forceinline__ bool beats(T x, T cur) { return MAXOP ? (x > cur) : (x < cur); }

// One lane per output element walks the axis (or its chunk of it) front to back. The chunk that holds
// slice 0 starts from that slice whatever it is; later chunks skip NaN, which the serial walk never takes.
template <typename T, bool MAXOP>
__global__ __launch_bounds__(256) void argreduce_seq(ArgArgs<T> p) {
  const int64_t o = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (o >= p.outputs) return;
  int64_t a_off, v_off, i_off;
  decode3(p, o, a_off, v_off, i_off);
  const T* src = p.a + a_off;
  const int64_t l0 = (int64_t)blockIdx.y * p.chunk_len;
  const int64_t l1 = (l0 + p.chunk_len < p.L) ? l0 + p.chunk_len : p.L;
  T best = src[l0 * p.a_axis_stride];
  int64_t at = l0;
  bool has = (blockIdx.y == 0) || (best == best);
  auto take = [&](T v, int64_t l) {
    if (has ? beats<T, MAXOP>(v, best) : (v == v)) { best = v; at = l; has = true; }
  };
  int64_t l = l0 + 1;
  for (; l + 4 <= l1; l += 4) {   // four loads in flight, compared in axis order
    const T v0 = __builtin_nontemporal_load(src + l * p.a_axis_stride), v1 = __builtin_nontemporal_load(src + (l + 1) * p.a_axis_stride);
    const T v2 = __builtin_nontemporal_load(src + (l + 2) * p.a_axis_stride), v3 = __builtin_nontemporal_load(src + (l + 3) * p.a_axis_stride);
    take(v0, l); take(v1, l + 1); take(v2, l + 2); take(v3, l + 3);
  }
  for (; l < l1; ++l) take(src[l * p.a_axis_stride], l);
  if (p.chunks > 1) {
    p.ws_val[(int64_t)blockIdx.y * p.outputs + o] = best;
    p.ws_idx[(int64_t)blockIdx.y * p.outputs + o] = has ? at : -1;
  } else {
    p.val[v_off] = best;
    p.idx[i_off] = at;
  }
}

// Second pass of the chunked walk: the chunks' results in axis order under the same strict comparison.
template <typename T, bool MAXOP>
__global__ __launch_bounds__(256) void argreduce_merge(ArgArgs<T> p) {
  const int64_t o = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (o >= p.outputs) return;
  int64_t a_off, v_off, i_off;
  decode3(p, o, a_off, v_off, i_off);
  T best = p.ws_val[o];
  int64_t at = p.ws_idx[o];       // chunk 0 always has a position
  for (int c = 1; c < p.chunks; ++c) {
    const T v = p.ws_val[(int64_t)c * p.outputs + o];
    const int64_t i = p.ws_idx[(int64_t)c * p.outputs + o];
    if (i >= 0 && beats<T, MAXOP>(v, best)) { best = v; at = i; }
  }
  p.val[v_off] = best;
  p.idx[i_off] = at;
}

// One wavefront per output element, lanes striding along the axis (16-byte loads when it has unit
// stride). A lane keeps the first best of its own positions among the values that are not NaN; the
// butterfly keeps the better value and, between equal values, the lower position; slice 0 holding a
// NaN overrides everything, as in the serial walk.
template <typename T, bool MAXOP, bool VEC>
__global__ __launch_bounds__(256) void argreduce_row(ArgArgs<T> p) {
  constexpr int V = 16 / (int)sizeof(T);
  typedef T vec_t __attribute__((ext_vector_type(V)));
  const int lane = threadIdx.x & 63;
  // one wavefront per (output, chunk of the axis): with few outputs and a long axis the axis is cut (chunk starts are
  // multiples of the vector) and the chunks' results go to the workspace for argreduce_merge
  const int64_t unit = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (unit >= p.outputs * p.chunks) return;
  const int64_t chunk = unit / p.outputs, o = unit - chunk * p.outputs;
  int64_t a_off, v_off, i_off;
  decode3(p, o, a_off, v_off, i_off);
  const int64_t l0 = chunk * p.chunk_len;
  const int64_t len = (l0 + p.chunk_len < p.L) ? p.chunk_len : p.L - l0;
  const T* row = p.a + a_off;
  const T* src = row + l0 * p.a_axis_stride;
  T best = (T)0;
  int64_t at = 0;
  bool has = false;
  auto take = [&](T v, int64_t l) {
    if (v == v && (!has || beats<T, MAXOP>(v, best))) { best = v; at = l0 + l; has = true; }
  };
  if constexpr (VEC) {
    const vec_t* vs = (const vec_t*)src;
    const int64_t nvec = len / V;
    int64_t v = lane;
    for (; v + 192 < nvec; v += 256) {   // four 16-byte loads in flight per lane, taken in position order
      const vec_t x0 = vs[v], x1 = vs[v + 64], x2 = vs[v + 128], x3 = vs[v + 192];
#pragma unroll
      for (int e = 0; e < V; ++e) take(x0[e], v * V + e);
#pragma unroll
      for (int e = 0; e < V; ++e) take(x1[e], (v + 64) * V + e);
#pragma unroll
      for (int e = 0; e < V; ++e) take(x2[e], (v + 128) * V + e);
#pragma unroll
      for (int e = 0; e < V; ++e) take(x3[e], (v + 192) * V + e);
    }
    for (; v < nvec; v += 64) {
      const vec_t x0 = vs[v];
#pragma unroll
      for (int e = 0; e < V; ++e) take(x0[e], v * V + e);
    }
    for (int64_t l = nvec * V + lane; l < len; l += 64) take(src[l], l);
  } else {
    for (int64_t l = lane; l < len; l += 64) take(src[l * p.a_axis_stride], l);
  }
#pragma unroll
  for (int d = 32; d >= 1; d >>= 1) {
    const T ov = __shfl_xor(best, d, 64);
    const int64_t oa = (int64_t)__shfl_xor((long long)at, d, 64);
    const bool oh = __shfl_xor((int)has, d, 64) != 0;
    if (oh && (!has || beats<T, MAXOP>(ov, best) || (ov == best && oa < at))) { best = ov; at = oa; has = true; }
  }
  if (lane == 0) {
    if (chunk == 0) {
      const T first = row[0];
      if (!(first == first) || !has) { best = first; at = 0; has = true; }
    }
    if (p.chunks > 1) {
      p.ws_val[chunk * p.outputs + o] = best;
      p.ws_idx[chunk * p.outputs + o] = has ? at : -1;
    } else {
      p.val[v_off] = best;
      p.idx[i_off] = at;
    }
  }
}

// Many SHORT rows along their unit-stride axis (the class of each row of a [batch x classes] matrix): `lanes` lanes (a
// power of two <= 32) share a row, one 16-byte vector each; a lane keeps the first best of its elements that are not
// NaN, the lanes of a row merge by (better value, lower position), and a NaN in position 0 overrides, as above.
template <typename T, bool MAXOP>
__global__ __launch_bounds__(256) void argreduce_rows_short(ArgArgs<T> p, int lanes) {
  constexpr int V = 16 / (int)sizeof(T);
  constexpr int U = 4;
  typedef T vec_t __attribute__((ext_vector_type(V)));
  const int lane = threadIdx.x & 63;
  const int j = lane & (lanes - 1), sub = lane / lanes, rows_per_step = 64 / lanes;
  const int64_t wave = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  const int64_t row0 = wave * (int64_t)(U * rows_per_step) + sub;
  const int64_t nvec = p.L / V;
  vec_t x[U];
  int64_t v_off[U], i_off[U];
  bool ok[U];
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const int64_t o = row0 + (int64_t)u * rows_per_step;
    ok[u] = o < p.outputs && j < nvec;
    int64_t a_off;
    decode3(p, o < p.outputs ? o : 0, a_off, v_off[u], i_off[u]);
    x[u] = *((const vec_t*)(p.a + a_off) + (j < nvec ? j : 0));
  }
#pragma unroll
  for (int u = 0; u < U; ++u) {
    T best = (T)0;
    int64_t at = 0;
    bool has = false;
    if (ok[u]) {
#pragma unroll
      for (int e = 0; e < V; ++e) {
        const T v = x[u][e];
        if (v == v && (!has || beats<T, MAXOP>(v, best))) { best = v; at = (int64_t)j * V + e; has = true; }
      }
    }
    const T first = __shfl(x[u][0], lane - j, 64);   // element 0 of the row sits in the group's first lane
    for (int d = lanes >> 1; d >= 1; d >>= 1) {
      const T ov = __shfl_xor(best, d, 64);
      const int64_t oa = (int64_t)__shfl_xor((long long)at, d, 64);
      const bool oh = __shfl_xor((int)has, d, 64) != 0;
      if (oh && (!has || beats<T, MAXOP>(ov, best) || (ov == best && oa < at))) { best = ov; at = oa; has = true; }
    }
    if (j == 0 && ok[u]) {
      if (!(first == first) || !has) { best = first; at = 0; }
      p.val[v_off[u]] = best;
      p.idx[i_off[u]] = at;
    }
  }
}

// A walk down the rows of a matrix with FEW columns (the outputs are one unit-stride run of at most half a workgroup of
// 16-byte lanes): lanes over the columns x 256 / cx row classes as in reduce_cols_narrow, every lane VEC outputs with
// their own (value, position), row classes merged through LDS by (better value, lower position), so any merge order
// gives the serial walk's answer; NaN is never taken except from row 0 (the chunk that holds it checks). Chunks of the
// axis over the grid; their results go to the workspace in axis order for argreduce_merge.
template <typename T, bool MAXOP>
__global__ __launch_bounds__(256) void argreduce_cols_narrow(ArgArgs<T> p, int cx) {
  constexpr int V = 16 / (int)sizeof(T);
  constexpr int U = 4;
  typedef T vec_t __attribute__((ext_vector_type(V)));
  __shared__ T s_val[256][V];
  __shared__ int64_t s_idx[256][V];
  const int ry = 256 / cx;
  const int xq = (int)threadIdx.x % cx, yq = (int)threadIdx.x / cx;
  const int64_t col = (int64_t)xq * V;
  const bool active = yq < ry;
  const int64_t l0 = (int64_t)blockIdx.x * p.chunk_len;
  const int64_t l1 = (l0 + p.chunk_len < p.L) ? l0 + p.chunk_len : p.L;
  T best[V];
  int64_t at[V];
#pragma unroll
  for (int e = 0; e < V; ++e) { best[e] = (T)0; at[e] = -1; }
  auto take = [&](const vec_t& v, int64_t l) {
#pragma unroll
    for (int e = 0; e < V; ++e)
      if (v[e] == v[e] && (at[e] < 0 || beats<T, MAXOP>(v[e], best[e]))) { best[e] = v[e]; at[e] = l; }
  };
  const T* src = p.a + col;
  if (active) {
    int64_t l = l0 + yq;
    for (; l + (int64_t)(U - 1) * ry < l1; l += (int64_t)U * ry) {
      vec_t v[U];
#pragma unroll
      for (int u = 0; u < U; ++u) v[u] = __builtin_nontemporal_load((const vec_t*)(src + (l + (int64_t)u * ry) * p.a_axis_stride));
#pragma unroll
      for (int u = 0; u < U; ++u) take(v[u], l + (int64_t)u * ry);
    }
    for (; l < l1; l += ry) take(*(const vec_t*)(src + l * p.a_axis_stride), l);
  }
#pragma unroll
  for (int e = 0; e < V; ++e) { s_val[threadIdx.x][e] = best[e]; s_idx[threadIdx.x][e] = at[e]; }
  __syncthreads();
  if (active && yq == 0) {
    for (int yy = 1; yy < ry; ++yy)
#pragma unroll
      for (int e = 0; e < V; ++e) {
        const T ov = s_val[yy * cx + xq][e];
        const int64_t oa = s_idx[yy * cx + xq][e];
        if (oa >= 0 && (at[e] < 0 || beats<T, MAXOP>(ov, best[e]) || (ov == best[e] && oa < at[e]))) { best[e] = ov; at[e] = oa; }
      }
    if (blockIdx.x == 0) {   // row 0 holding a NaN overrides; a column of nothing but NaN reports row 0 as well
      const vec_t first = *(const vec_t*)src;
#pragma unroll
      for (int e = 0; e < V; ++e)
        if (!(first[e] == first[e]) || at[e] < 0) { best[e] = first[e]; at[e] = 0; }
    }
#pragma unroll
    for (int e = 0; e < V; ++e) {
      if (p.chunks > 1) {
        p.ws_val[(int64_t)blockIdx.x * p.outputs + col + e] = best[e];
        p.ws_idx[(int64_t)blockIdx.x * p.outputs + col + e] = at[e];
      } else {
        p.val[(col + e) * p.v_stride[0]] = best[e];
        p.idx[(col + e) * p.i_stride[0]] = at[e];
      }
    }
  }
}

template <typename T>
static int argreduce(const char* fn, int op, int rank, const int64_t* shape, int axis, int64_t* idx, const int64_t* si,
                     T* val, const int64_t* sv, const T* a, const int64_t* sa) {
  if (op != AM_RED_MAX && op != AM_RED_MIN) return fail(AM_E_ARG, "%s: op must be AM_RED_MAX or AM_RED_MIN", fn);
  if (rank < 1 || rank > AM_MAXRANK) return fail(AM_E_SHAPE, "%s: rank %d outside 1..%d", fn, rank, AM_MAXRANK);
  if (!shape || !si || !sv || !sa) return fail(AM_E_ARG, "%s: null shape or strides", fn);
  if (axis < 0 || axis >= rank) return fail(AM_E_SHAPE, "%s: axis %d outside the tensor's rank %d", fn, axis, rank);
  int64_t size = 1;
  for (int d = 0; d < rank; ++d) {
    if (shape[d] < 0) return fail(AM_E_SHAPE, "%s: negative extent", fn);
    size *= shape[d];
  }
  if (size == 0) return AM_OK;
  if (!idx || !val || !a) return fail(AM_E_ARG, "%s: null tensor pointer", fn);
  AM_TRY(ensure_init());
  ArgArgs<T> g;
  memset(&g, 0, sizeof(g));
  g.a = a; g.val = val; g.idx = idx;
  g.outputs = 1;
  int64_t best_other = -1;
  for (int d = 0; d < rank; ++d) {
    if (d == axis || shape[d] == 1) continue;
    g.extent[g.ndim] = shape[d]; g.a_stride[g.ndim] = sa[d]; g.v_stride[g.ndim] = sv[d]; g.i_stride[g.ndim] = si[d];
    ++g.ndim;
    g.outputs *= shape[d];
    if (best_other < 0 || iabs64(sa[d]) < best_other) best_other = iabs64(sa[d]);
  }
  for (int d = g.ndim; d < kMaxDims; ++d) g.extent[d] = 1;
  g.L = shape[axis]; g.a_axis_stride = sa[axis];
  const bool row_kernel = g.L >= 64 && (best_other < 0 || iabs64(g.a_axis_stride) < best_other || g.outputs < 1024);
  const int64_t bx = row_kernel ? (g.outputs + 3) / 4 : (g.outputs + 255) / 256;
  if (bx >= ((int64_t)1 << 31)) return fail(AM_E_SHAPE, "%s: too many output elements", fn);
  g.chunks = 1; g.chunk_len = g.L; g.ws_val = nullptr; g.ws_idx = nullptr;
  const dim3 block(256);
  constexpr int64_t V = 16 / (int64_t)sizeof(T);
  // chunk partials [chunk][output]: values, then positions
  auto chunk_workspace = [&](int64_t chunks, int64_t len) {
    const size_t val_bytes = ((size_t)chunks * (size_t)g.outputs * sizeof(T) + 255) / 256 * 256;
    char* base = chunks > 1 ? (char*)gemm::splitk_workspace(val_bytes + (size_t)chunks * (size_t)g.outputs * sizeof(int64_t)) : nullptr;
    if (base) { g.chunks = (int)chunks; g.chunk_len = len; g.ws_val = (T*)base; g.ws_idx = (int64_t*)(base + val_bytes); }
  };
  auto merge_chunks = [&]() {
    AM_TRY(check_launch("argreduce"));
    const dim3 mgrid((unsigned)((g.outputs + 255) / 256));
    if (op == AM_RED_MAX) hipLaunchKernelGGL((argreduce_merge<T, true>), mgrid, block, 0, stream(), g);
    else hipLaunchKernelGGL((argreduce_merge<T, false>), mgrid, block, 0, stream(), g);
    return check_launch("argreduce_merge");
  };
  const bool aligned = (uintptr_t)g.a % 16 == 0;
  // few columns, a walk down many rows
  if (g.ndim == 1 && g.a_stride[0] == 1 && iabs64(g.a_axis_stride) > 1 && g.outputs % V == 0 && g.outputs / V <= 128 && g.L >= 512 &&
      g.a_axis_stride >= g.outputs && g.a_axis_stride % V == 0 && aligned) {
    int64_t chunks = (int64_t)num_cus() * 2;
    if (chunks > g.L / 256) chunks = g.L / 256;
    if (chunks >= 2) {
      const int64_t len = (g.L + chunks - 1) / chunks;
      chunk_workspace((g.L + len - 1) / len, len);
    }
    const dim3 grid((unsigned)g.chunks);
    const int cx = (int)(g.outputs / V);
    if (op == AM_RED_MAX) hipLaunchKernelGGL((argreduce_cols_narrow<T, true>), grid, block, 0, stream(), g, cx);
    else hipLaunchKernelGGL((argreduce_cols_narrow<T, false>), grid, block, 0, stream(), g, cx);
    return g.chunks > 1 ? merge_chunks() : check_launch("argreduce_cols_narrow");
  }
  // many short rows along their unit-stride axis
  if (g.a_axis_stride == 1 && g.L % V == 0 && g.L / V <= 32 && g.outputs >= 4096 && aligned) {
    bool rows_aligned = true;
    for (int d = 0; d < g.ndim; ++d) rows_aligned = rows_aligned && g.a_stride[d] % V == 0;
    if (rows_aligned) {
      int lanes = 1;
      while (lanes < g.L / V) lanes *= 2;
      const int64_t rows_per_wg = 4 * 4 * (64 / lanes);
      const int64_t sb = (g.outputs + rows_per_wg - 1) / rows_per_wg;
      if (sb < ((int64_t)1 << 31)) {
        if (op == AM_RED_MAX) hipLaunchKernelGGL((argreduce_rows_short<T, true>), dim3((unsigned)sb), block, 0, stream(), g, lanes);
        else hipLaunchKernelGGL((argreduce_rows_short<T, false>), dim3((unsigned)sb), block, 0, stream(), g, lanes);
        return check_launch("argreduce_rows_short");
      }
    }
  }
  if (row_kernel) {
    bool vec = g.a_axis_stride == 1 && aligned;
    for (int d = 0; d < g.ndim && vec; ++d) vec = g.a_stride[d] % V == 0;
    // few outputs, a long axis: chunks of the axis over several wavefronts (16 per CU over the chip, 4096 elements or more each)
    const int64_t want_waves = (int64_t)num_cus() * 16;
    if (g.outputs < want_waves / 2 && g.L >= 8192) {
      int64_t chunks = (want_waves + g.outputs - 1) / g.outputs;
      if (chunks > g.L / 4096) chunks = g.L / 4096;
      if (chunks > 1024) chunks = 1024;
      if (chunks >= 2) {
        int64_t len = (g.L + chunks - 1) / chunks;
        len = (len + 255) / 256 * 256;
        chunk_workspace((g.L + len - 1) / len, len);
      }
    }
    const int64_t rb = (g.outputs * g.chunks + 3) / 4;
    const dim3 grid((unsigned)rb);
    if (op == AM_RED_MAX) {
      if (vec) hipLaunchKernelGGL((argreduce_row<T, true, true>), grid, block, 0, stream(), g);
      else hipLaunchKernelGGL((argreduce_row<T, true, false>), grid, block, 0, stream(), g);
    } else {
      if (vec) hipLaunchKernelGGL((argreduce_row<T, false, true>), grid, block, 0, stream(), g);
      else hipLaunchKernelGGL((argreduce_row<T, false, false>), grid, block, 0, stream(), g);
    }
    if (g.chunks > 1) return merge_chunks();
  } else {
    // too few outputs to fill the chip: cut the axis (eight workgroups per CU, at least 64 slices per chunk)
    const int64_t want = (int64_t)num_cus() * 8;
    if (bx < want && g.L >= 128) {
      int64_t chunks = (want + bx - 1) / bx;
      if (chunks > g.L / 64) chunks = g.L / 64;
      if (chunks > 1024) chunks = 1024;
      const int64_t len = (g.L + chunks - 1) / chunks;
      chunk_workspace((g.L + len - 1) / len, len);
    }
    const dim3 grid((unsigned)bx, (unsigned)g.chunks);
    if (op == AM_RED_MAX) hipLaunchKernelGGL((argreduce_seq<T, true>), grid, block, 0, stream(), g);
    else hipLaunchKernelGGL((argreduce_seq<T, false>), grid, block, 0, stream(), g);
    if (g.chunks > 1) return merge_chunks();
  }
  return check_launch("argreduce");
}

// ------------------------------------------------------------------------------------------------
// Row softmax. One wavefront per row up to 4096 columns, one workgroup per row beyond. The row is
// read three times (maximum, sum of exponentials, output); the second and third reads come from
// cache. max and sum are what the reference's streaming pass arrives at, up to rounding of the sum.
template <typename T> struct SoftmaxArgs {
  const T* src; T* dst;
  int64_t rows, cols, s_rs, s_cs, d_rs, d_cs;
};

template <typename T> __device__ __forceinline__ T dev_exp(T x);
template <> __device__ __forceinline__ float dev_exp<float>(float x) { return expf(x); }
template <> __device__ __forceinline__ double dev_exp<double>(double x) { return exp(x); }

template <typename T, bool BLOCK>
__global__ __launch_bounds__(256) void softmax_rows(SoftmaxArgs<T> p) {
  constexpr int W = BLOCK ? 256 : 64;            // lanes working on one row
  __shared__ T part[4];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int64_t row = BLOCK ? (int64_t)blockIdx.x : (int64_t)blockIdx.x * 4 + wave;
  const bool active = row < p.rows;
  const int me = BLOCK ? (int)threadIdx.x : lane;
  const T* src = p.src + (active ? row : 0) * p.s_rs;
  // `x <= max` is false for the first element against -Inf only if x is NaN; NaN rows give NaN
  T mx = -std::numeric_limits<T>::infinity();
  if (active) for (int64_t c = me; c < p.cols; c += W) { const T x = src[c * p.s_cs]; mx = (x <= mx) ? mx : x; }
#pragma unroll
  for (int d = 32; d >= 1; d >>= 1) { const T o = __shfl_xor(mx, d, 64); mx = (o <= mx) ? mx : o; }
  if constexpr (BLOCK) {
    if (lane == 0) part[wave] = mx;
    __syncthreads();
    mx = part[0];
#pragma unroll
    for (int w = 1; w < 4; ++w) mx = (part[w] <= mx) ? mx : part[w];
    __syncthreads();
  }
  T sum = (T)0;
  if (active) for (int64_t c = me; c < p.cols; c += W) sum += dev_exp<T>(src[c * p.s_cs] - mx);
#pragma unroll
  for (int d = 32; d >= 1; d >>= 1) sum += __shfl_xor(sum, d, 64);
  if constexpr (BLOCK) {
    if (lane == 0) part[wave] = sum;
    __syncthreads();
    sum = ((part[0] + part[1]) + part[2]) + part[3];
  }
  if (!active) return;
  T* dst = p.dst + row * p.d_rs;
  const T inv = (T)1 / sum;
  for (int64_t c = me; c < p.cols; c += W) dst[c * p.d_cs] = dev_exp<T>(src[c * p.s_cs] - mx) * inv;   // stable_softmax
}

// Contiguous rows that fit in registers: each lane keeps NV 16-byte vectors of its row, so the
// row is read from memory once and written once. W lanes per row (64: four rows per workgroup;
// 256: one row per workgroup). Requires unit column strides, cols a multiple of the vector width
// and 16-byte aligned rows; cols <= W * NV * VEC.
template <typename T, int W, int NV, bool STREAM>
__global__ __launch_bounds__(W == 64 ? 256 : W) void softmax_rows_reg(SoftmaxArgs<T> p) {
  constexpr int V = 16 / (int)sizeof(T);
  constexpr int NW = W == 64 ? 4 : W / 64;   // wavefronts per workgroup (W == 64: four rows per workgroup)
  typedef T vec_t __attribute__((ext_vector_type(V)));
  __shared__ T part[NW];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int64_t row = (W != 64) ? (int64_t)blockIdx.x : (int64_t)blockIdx.x * 4 + wave;
  const bool active = row < p.rows;
  const int me = (W != 64) ? (int)threadIdx.x : lane;
  const int64_t nvec = p.cols / V;
  const vec_t* src = (const vec_t*)(p.src + (active ? row : 0) * p.s_rs);
  const T ninf = -std::numeric_limits<T>::infinity();
  vec_t x[NV];
  T mx = ninf;
  // every load of the row is issued before the first use, unconditionally (vectors past the end of the row read
  // its first one): loads under a per-lane test are waited for one by one
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int64_t v = (int64_t)i * W + me;
    const vec_t* at = src + (v < nvec ? v : 0);
    if constexpr (STREAM) x[i] = __builtin_nontemporal_load(at); else x[i] = *at;
  }
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int64_t v = (int64_t)i * W + me;
    if (active && v < nvec) {
#pragma unroll
      for (int e = 0; e < V; ++e) mx = (x[i][e] <= mx) ? mx : x[i][e];
    }
  }
#pragma unroll
  for (int d = 32; d >= 1; d >>= 1) { const T o = __shfl_xor(mx, d, 64); mx = (o <= mx) ? mx : o; }
  if constexpr (W != 64) {
    if (lane == 0) part[wave] = mx;
    __syncthreads();
    mx = part[0];
#pragma unroll
    for (int w = 1; w < NW; ++w) mx = (part[w] <= mx) ? mx : part[w];
    __syncthreads();
  }
  T sum = (T)0;
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int64_t v = (int64_t)i * W + me;
    if (active && v < nvec) {
#pragma unroll
      for (int e = 0; e < V; ++e) { x[i][e] = dev_exp<T>(x[i][e] - mx); sum += x[i][e]; }
    }
  }
#pragma unroll
  for (int d = 32; d >= 1; d >>= 1) sum += __shfl_xor(sum, d, 64);
  if constexpr (W != 64) {
    if (lane == 0) part[wave] = sum;
    __syncthreads();
    sum = part[0];
#pragma unroll
    for (int w = 1; w < NW; ++w) sum += part[w];   // front to back: ((p0 + p1) + p2) + ...
  }
  if (!active) return;
  vec_t* dst = (vec_t*)(p.dst + row * p.d_rs);
  const T inv = (T)1 / sum;   // one division per row; every element is then within 1.5 ulp of exp / sum
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int64_t v = (int64_t)i * W + me;
    if (v < nvec) {
      vec_t y;
#pragma unroll
      for (int e = 0; e < V; ++e) y[e] = x[i][e] * inv;
      __builtin_nontemporal_store(y, dst + v);
    }
  }
}

// Short contiguous rows (a [batch x classes] matrix with 4 ... 128 classes): `lanes` lanes (a power of two <= 32)
// share a row, one 16-byte vector each, so a wavefront handles 64 / lanes rows at once and its loads and stores are
// contiguous runs; maximum and sum go through a butterfly inside the lane group. Same arithmetic per element as
// softmax_rows_reg.
template <typename T, bool STREAM>
__global__ __launch_bounds__(256) void softmax_rows_short(SoftmaxArgs<T> p, int lanes) {
  constexpr int V = 16 / (int)sizeof(T);
  typedef T vec_t __attribute__((ext_vector_type(V)));
  const int lane = threadIdx.x & 63;
  const int j = lane & (lanes - 1), rows_per_wave = 64 / lanes;
  const int64_t row = ((int64_t)blockIdx.x * 4 + (threadIdx.x >> 6)) * rows_per_wave + lane / lanes;
  const int64_t nvec = p.cols / V;
  const bool ok = row < p.rows && j < nvec;
  const vec_t* at = (const vec_t*)(p.src + (row < p.rows ? row : 0) * p.s_rs) + (j < nvec ? j : 0);
  vec_t x;
  if constexpr (STREAM) x = __builtin_nontemporal_load(at); else x = *at;
  T mx = -std::numeric_limits<T>::infinity();
  if (ok) {
#pragma unroll
    for (int e = 0; e < V; ++e) mx = (x[e] <= mx) ? mx : x[e];
  }
  for (int d = lanes >> 1; d >= 1; d >>= 1) { const T o = __shfl_xor(mx, d, 64); mx = (o <= mx) ? mx : o; }
  T sum = (T)0;
  if (ok) {
#pragma unroll
    for (int e = 0; e < V; ++e) { x[e] = dev_exp<T>(x[e] - mx); sum += x[e]; }
  }
  for (int d = lanes >> 1; d >= 1; d >>= 1) sum += __shfl_xor(sum, d, 64);
  if (!ok) return;
  const T inv = (T)1 / sum;
  vec_t y;
#pragma unroll
  for (int e = 0; e < V; ++e) y[e] = x[e] * inv;
  __builtin_nontemporal_store(y, (vec_t*)(p.dst + row * p.d_rs) + j);
}

// Rows of at most 64 elements with any strides and lengths (ten classes): one lane per row, three walks over the row
// (maximum, sum, output); a wavefront's rows are neighbours, so the second and third walk hit the vector cache.
template <typename T>
__global__ __launch_bounds__(256) void softmax_rows_lane(SoftmaxArgs<T> p) {
  const int64_t row = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (row >= p.rows) return;
  const T* src = p.src + row * p.s_rs;
  T mx = -std::numeric_limits<T>::infinity();
  for (int64_t c = 0; c < p.cols; ++c) { const T x = src[c * p.s_cs]; mx = (x <= mx) ? mx : x; }
  T sum = (T)0;
  for (int64_t c = 0; c < p.cols; ++c) sum += dev_exp<T>(src[c * p.s_cs] - mx);
  const T inv = (T)1 / sum;
  T* dst = p.dst + row * p.d_rs;
  for (int64_t c = 0; c < p.cols; ++c) dst[c * p.d_cs] = dev_exp<T>(src[c * p.s_cs] - mx) * inv;
}

// Rows too long for one workgroup's registers (beyond 65536 four-byte elements: vocabulary-sized rows, or a handful of
// very long ones that would leave most CUs without work): the row is cut into chunks over several workgroups.
// softmax_long_partial: maximum m and sum of exp(x - m) of one chunk -> ws[row][chunk] = (m, s).
// softmax_long_write: every workgroup folds its row's partials (M = max m, S = sum s exp(m - M), front to back) and
// writes exp(x - M) / S for its chunk. The input is read twice, the second time largely from the caches.
template <typename T>
__global__ __launch_bounds__(256) void softmax_long_partial(SoftmaxArgs<T> p, T* ws, int chunks, int64_t chunk_vecs) {
  constexpr int V = 16 / (int)sizeof(T);
  typedef T vec_t __attribute__((ext_vector_type(V)));
  __shared__ T part[4];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int64_t row = blockIdx.y, chunk = blockIdx.x;
  const int64_t nvec = p.cols / V, v0 = chunk * chunk_vecs, v1 = (v0 + chunk_vecs < nvec) ? v0 + chunk_vecs : nvec;
  const vec_t* src = (const vec_t*)(p.src + row * p.s_rs);
  const T ninf = -std::numeric_limits<T>::infinity();
  T mx = ninf;
  int64_t v = v0 + threadIdx.x;
  for (; v + 768 < v1; v += 1024) {
    const vec_t a = src[v], b = src[v + 256], c = src[v + 512], d = src[v + 768];
#pragma unroll
    for (int e = 0; e < V; ++e) {
      mx = (a[e] <= mx) ? mx : a[e]; mx = (b[e] <= mx) ? mx : b[e]; mx = (c[e] <= mx) ? mx : c[e]; mx = (d[e] <= mx) ? mx : d[e];
    }
  }
  for (; v < v1; v += 256) {
    const vec_t a = src[v];
#pragma unroll
    for (int e = 0; e < V; ++e) mx = (a[e] <= mx) ? mx : a[e];
  }
#pragma unroll
  for (int d = 32; d >= 1; d >>= 1) { const T o = __shfl_xor(mx, d, 64); mx = (o <= mx) ? mx : o; }
  if (lane == 0) part[wave] = mx;
  __syncthreads();
  mx = part[0];
#pragma unroll
  for (int w = 1; w < 4; ++w) mx = (part[w] <= mx) ? mx : part[w];
  __syncthreads();
  T sum = (T)0;
  for (v = v0 + threadIdx.x; v < v1; v += 256) {   // second walk over the chunk: from cache
    const vec_t a = src[v];
#pragma unroll
    for (int e = 0; e < V; ++e) sum += dev_exp<T>(a[e] - mx);
  }
#pragma unroll
  for (int d = 32; d >= 1; d >>= 1) sum += __shfl_xor(sum, d, 64);
  if (lane == 0) part[wave] = sum;
  __syncthreads();
  if (threadIdx.x == 0) {
    T* out = ws + 2 * (row * chunks + chunk);
    out[0] = mx;
    out[1] = ((part[0] + part[1]) + part[2]) + part[3];
  }
}

template <typename T>
__global__ __launch_bounds__(256) void softmax_long_write(SoftmaxArgs<T> p, const T* ws, int chunks, int64_t chunk_vecs) {
  constexpr int V = 16 / (int)sizeof(T);
  typedef T vec_t __attribute__((ext_vector_type(V)));
  const int64_t row = blockIdx.y, chunk = blockIdx.x;
  const T* mine = ws + 2 * row * chunks;
  T mx = mine[0];
  for (int c = 1; c < chunks; ++c) mx = (mine[2 * c] <= mx) ? mx : mine[2 * c];
  T sum = (T)0;
  for (int c = 0; c < chunks; ++c) sum += mine[2 * c + 1] * dev_exp<T>(mine[2 * c] - mx);
  const T inv = (T)1 / sum;
  const int64_t nvec = p.cols / V, v0 = chunk * chunk_vecs, v1 = (v0 + chunk_vecs < nvec) ? v0 + chunk_vecs : nvec;
  const vec_t* src = (const vec_t*)(p.src + row * p.s_rs);
  vec_t* dst = (vec_t*)(p.dst + row * p.d_rs);
  for (int64_t v = v0 + threadIdx.x; v < v1; v += 256) {
    const vec_t a = src[v];
    vec_t y;
#pragma unroll
    for (int e = 0; e < V; ++e) y[e] = dev_exp<T>(a[e] - mx) * inv;
    __builtin_nontemporal_store(y, dst + v);
  }
}

template <typename T, int W, bool STREAM>
static void launch_softmax_reg(const SoftmaxArgs<T>& p, int nv, dim3 grid) {
  switch (nv) {
    case 1: hipLaunchKernelGGL((softmax_rows_reg<T, W, 1, STREAM>), grid, dim3(W == 64 ? 256 : W), 0, stream(), p); break;
    case 2: hipLaunchKernelGGL((softmax_rows_reg<T, W, 2, STREAM>), grid, dim3(W == 64 ? 256 : W), 0, stream(), p); break;
    case 4: hipLaunchKernelGGL((softmax_rows_reg<T, W, 4, STREAM>), grid, dim3(W == 64 ? 256 : W), 0, stream(), p); break;
    case 8: hipLaunchKernelGGL((softmax_rows_reg<T, W, 8, STREAM>), grid, dim3(W == 64 ? 256 : W), 0, stream(), p); break;
    default: hipLaunchKernelGGL((softmax_rows_reg<T, W, 16, STREAM>), grid, dim3(W == 64 ? 256 : W), 0, stream(), p); break;
  }
}

template <typename T>
static int softmax(const char* fn, int64_t rows, int64_t cols, T* dst, int64_t d_rs, int64_t d_cs, const T* src,
                   int64_t s_rs, int64_t s_cs) {
  constexpr int64_t V = 16 / (int64_t)sizeof(T);
  if (rows < 0 || cols < 0) return fail(AM_E_SHAPE, "%s: negative extent", fn);
  if (rows == 0 || cols == 0) return AM_OK;
  if (!dst || !src) return fail(AM_E_ARG, "%s: null tensor pointer", fn);
  if (rows >= ((int64_t)1 << 31)) return fail(AM_E_SHAPE, "%s: too many rows", fn);
  AM_TRY(ensure_init());
  SoftmaxArgs<T> p = {src, dst, rows, cols, s_rs, s_cs, d_rs, d_cs};
  const bool vec = s_cs == 1 && d_cs == 1 && cols % V == 0 && (rows == 1 || (s_rs % V == 0 && d_rs % V == 0)) &&
                   (uintptr_t)src % 16 == 0 && (uintptr_t)dst % 16 == 0;
  const int64_t nvec = cols / V;
  const bool stream_loads = (double)rows * (double)cols * sizeof(T) > nt_threshold_bytes();
  if (vec && nvec <= 32 && rows >= 1024) {   // several rows per wavefront
    int lanes = 1;
    while (lanes < nvec) lanes *= 2;
    const dim3 grid((unsigned)((rows + 4 * (64 / lanes) - 1) / (4 * (64 / lanes))));
    if (stream_loads) hipLaunchKernelGGL((softmax_rows_short<T, true>), grid, dim3(256), 0, stream(), p, lanes);
    else hipLaunchKernelGGL((softmax_rows_short<T, false>), grid, dim3(256), 0, stream(), p, lanes);
  } else if (!vec && cols <= 64 && rows >= 1024) {   // a lane per row
    hipLaunchKernelGGL((softmax_rows_lane<T>), dim3((unsigned)((rows + 255) / 256)), dim3(256), 0, stream(), p);
  } else if (vec && nvec <= 64 * 8) {          // a wavefront per row
    int nv = 1;
    while (64 * nv < nvec) nv *= 2;
    launch_softmax_reg<T, 64, false>(p, nv, dim3((unsigned)((rows + 3) / 4)));
  } else if (vec && nvec <= 256 * 16) {  // a workgroup per row (up to 64 registers of row per lane)
    int nv = 1;
    while (256 * nv < nvec) nv *= 2;
    // rows this long make an input beyond the L2s at a few thousand rows: read it with non-temporal loads then
    if (stream_loads) launch_softmax_reg<T, 256, true>(p, nv, dim3((unsigned)rows));
    else launch_softmax_reg<T, 256, false>(p, nv, dim3((unsigned)rows));
  } else if (vec && nvec <= 1024 * 16) {  // sixteen wavefronts per row: rows of up to 65536 four-byte elements stay in registers
    int nv = 1;
    while (1024 * nv < nvec) nv *= 2;
    if (stream_loads) launch_softmax_reg<T, 1024, true>(p, nv, dim3((unsigned)rows));
    else launch_softmax_reg<T, 1024, false>(p, nv, dim3((unsigned)rows));
  } else if (vec && rows < 65536) {   // longer rows still: chunks of a row over several workgroups
    int64_t chunks = ((int64_t)num_cus() * 8 + rows - 1) / rows;
    if (chunks > nvec / 1024) chunks = nvec / 1024;
    if (chunks > 1024) chunks = 1024;
    if (chunks < 1) chunks = 1;
    const int64_t chunk_vecs = (nvec + chunks - 1) / chunks;
    chunks = (nvec + chunk_vecs - 1) / chunk_vecs;
    T* ws = (T*)gemm::splitk_workspace((size_t)rows * (size_t)chunks * 2 * sizeof(T));
    if (!ws) return fail(AM_E_ALLOC, "%s: no workspace for the partial maxima and sums of %lld rows", fn, (long long)rows);
    const dim3 grid((unsigned)chunks, (unsigned)rows);
    hipLaunchKernelGGL((softmax_long_partial<T>), grid, dim3(256), 0, stream(), p, ws, (int)chunks, chunk_vecs);
    AM_TRY(check_launch("softmax_long_partial"));
    hipLaunchKernelGGL((softmax_long_write<T>), grid, dim3(256), 0, stream(), p, (const T*)ws, (int)chunks, chunk_vecs);
  } else if (cols > 4096) {
    hipLaunchKernelGGL((softmax_rows<T, true>), dim3((unsigned)rows), dim3(256), 0, stream(), p);
  } else {
    hipLaunchKernelGGL((softmax_rows<T, false>), dim3((unsigned)((rows + 3) / 4)), dim3(256), 0, stream(), p);
  }
  return check_launch("softmax_rows");
}

// ------------------------------------------------------------------------------------------------
// Max pooling, one lane per output element; same scan order, strict `>` and starting values as
// the reference, so values and argmax indices are identical (first maximum wins; a window that
// lies wholly in the padding yields lowest(T) and the lowest index).
template <typename T> struct Lowest { static __device__ __forceinline__ T value() { return std::numeric_limits<T>::lowest(); } };
// low(float) in Nim is -Inf
template <> struct Lowest<float> { static __device__ __forceinline__ float value() { return -std::numeric_limits<float>::infinity(); } };
template <> struct Lowest<double> { static __device__ __forceinline__ double value() { return -std::numeric_limits<double>::infinity(); } };

// IDX: uint32_t when both tensors have fewer than 2^32 elements (64-bit division is slow).
template <typename T, typename IDX>
__global__ __launch_bounds__(256) void maxpool2d(const T* in, T* out, int64_t* argmax, int64_t total, int C, int H, int W,
                                                 int kH, int kW, int padH, int padW, int sH, int sW, int outH, int outW) {
  const int64_t oidx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (oidx >= total) return;
  const IDX oi = (IDX)oidx;
  const int w = (int)(oi % (IDX)outW);
  const IDX t = oi / (IDX)outW;
  const int h = (int)(t % (IDX)outH);
  const int64_t nc = (int64_t)(t / (IDX)outH);   // n * C + c
  T mx = Lowest<T>::value();
  int64_t arg = std::numeric_limits<int64_t>::lowest();
  for (int ph = 0; ph < kH; ++ph) {
    const int row = h * sH + ph - padH;
    if (row < 0 || row >= H) continue;
    for (int pw = 0; pw < kW; ++pw) {
      const int col = w * sW + pw - padW;
      if (col < 0 || col >= W) continue;
      const int64_t iidx = col + (int64_t)W * (row + (int64_t)H * nc);
      const T v = in[iidx];
      if (v > mx) { mx = v; arg = iidx; }
    }
  }
  out[oidx] = mx;
  if (argmax) argmax[oidx] = arg;
}

// The common 2-wide, stride-2, unpadded-in-width pooling with 16-byte aligned rows: one lane makes
// V = 16 / sizeof(T) neighbouring outputs from two 16-byte loads per window row, and stores them
// (and their indices) as vectors. Window scan order and comparisons as in the kernel above.
// Windows of a few elements (KH x KW known at compile time, any stride and padding): the KH * KW loads of a window are
// issued together, from a clamped address where the window reaches into the padding, and compared afterwards in the
// reference's scan order with its strict `>`; the output index is taken apart with launch-constant dividers. 3 x 3
// windows with stride 2 and padding 1 on [64, 64, 112, 112] f32: 2.6 -> see the measurement beside the host function.
template <typename T, int KH, int KW>
__global__ __launch_bounds__(256) void maxpool2d_small(const T* __restrict__ in, T* __restrict__ out, int64_t* __restrict__ argmax,
                                                       uint32_t total, int H, int W, int padH, int padW, int sH, int sW,
                                                       FastDiv by_outw, FastDiv by_outh) {
  const uint32_t oidx = blockIdx.x * 256u + threadIdx.x;
  if (oidx >= total) return;
  uint32_t w, h;
  const uint32_t nc = by_outh.divmod(by_outw.divmod(oidx, w), h);   // n * C + c
  const int row0 = (int)h * sH - padH, col0 = (int)w * sW - padW;
  const int64_t base = (int64_t)nc * H * W;
  const T* __restrict__ plane = in + base;
  T v[KH][KW];
  int off[KH][KW];
#pragma unroll
  for (int ph = 0; ph < KH; ++ph)
#pragma unroll
    for (int pw = 0; pw < KW; ++pw) {
      const int row = row0 + ph, col = col0 + pw;
      const bool ok = (unsigned)row < (unsigned)H && (unsigned)col < (unsigned)W;
      off[ph][pw] = ok ? row * W + col : -1;
      v[ph][pw] = plane[ok ? row * W + col : 0];
    }
  T mx = Lowest<T>::value();
  int best = -1;
#pragma unroll
  for (int ph = 0; ph < KH; ++ph)
#pragma unroll
    for (int pw = 0; pw < KW; ++pw)
      if (off[ph][pw] >= 0 && v[ph][pw] > mx) { mx = v[ph][pw]; best = off[ph][pw]; }
  out[oidx] = mx;
  if (argmax) argmax[oidx] = best >= 0 ? base + best : std::numeric_limits<int64_t>::lowest();
}

template <typename T>
__global__ __launch_bounds__(256) void maxpool2d_w2(const T* in, T* out, int64_t* argmax, int64_t total_vec, int H, int W,
                                                    int kH, int padH, int sH, int outH, int outWv) {
  constexpr int V = 16 / (int)sizeof(T);
  typedef T vec_t __attribute__((ext_vector_type(V)));
  typedef int64_t idx2_t __attribute__((ext_vector_type(2)));
  const int64_t ov = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (ov >= total_vec) return;
  const uint32_t o32 = (uint32_t)ov;           // the launcher guarantees total_vec < 2^32
  const int wv = (int)(o32 % (uint32_t)outWv);
  const uint32_t t = o32 / (uint32_t)outWv;
  const int h = (int)(t % (uint32_t)outH);
  const int64_t nc = (int64_t)(t / (uint32_t)outH);
  T mx[V];
  int64_t arg[V];
#pragma unroll
  for (int j = 0; j < V; ++j) { mx[j] = Lowest<T>::value(); arg[j] = std::numeric_limits<int64_t>::lowest(); }
  for (int ph = 0; ph < kH; ++ph) {
    const int row = h * sH + ph - padH;
    if (row < 0 || row >= H) continue;
    const int64_t base = (int64_t)W * (row + (int64_t)H * nc) + (int64_t)wv * 2 * V;
    const vec_t lo = *(const vec_t*)(in + base), hi = *(const vec_t*)(in + base + V);
#pragma unroll
    for (int j = 0; j < V; ++j) {
#pragma unroll
      for (int pw = 0; pw < 2; ++pw) {
        const int e = 2 * j + pw;
        const T v = (e < V) ? lo[e] : hi[e - V];
        if (v > mx[j]) { mx[j] = v; arg[j] = base + e; }
      }
    }
  }
  vec_t r;
#pragma unroll
  for (int j = 0; j < V; ++j) r[j] = mx[j];
  __builtin_nontemporal_store(r, (vec_t*)(out + ov * V));
  if (argmax) {
#pragma unroll
    for (int j = 0; j < V; j += 2) {
      idx2_t a2 = {arg[j], arg[j + 1]};
      __builtin_nontemporal_store(a2, (idx2_t*)(argmax + ov * V + j));
    }
  }
}

template <typename T>
static int maxpool(const char* fn, int64_t N, int C, int H, int W, int kH, int kW, int padH, int padW, int sH, int sW,
                   const T* in, T* out, int64_t* argmax) {
  if (N < 0 || C < 0 || H < 0 || W < 0) return fail(AM_E_SHAPE, "%s: negative extent", fn);
  if (kH < 1 || kW < 1 || sH < 1 || sW < 1 || padH < 0 || padW < 0) return fail(AM_E_ARG, "%s: kernel and stride must be >= 1, padding >= 0", fn);
  const int64_t outH = ((int64_t)H + 2 * padH - kH) / sH + 1, outW = ((int64_t)W + 2 * padW - kW) / sW + 1;
  if ((int64_t)H + 2 * padH < kH || (int64_t)W + 2 * padW < kW) return fail(AM_E_SHAPE, "%s: kernel larger than the padded input", fn);
  const int64_t total = N * C * outH * outW;
  if (total == 0) return AM_OK;
  if (!in || !out) return fail(AM_E_ARG, "%s: null tensor pointer", fn);
  AM_TRY(ensure_init());
  constexpr int64_t V = 16 / (int64_t)sizeof(T);
  if (kW == 2 && sW == 2 && padW == 0 && W % (2 * V) == 0 && total / V < ((int64_t)1 << 32) && (uintptr_t)in % 16 == 0 &&
      (uintptr_t)out % 16 == 0 && (uintptr_t)argmax % 16 == 0) {
    const int64_t total_vec = total / V;
    hipLaunchKernelGGL((maxpool2d_w2<T>), dim3((unsigned)((total_vec + 255) / 256)), dim3(256), 0, stream(), in, out, argmax,
                       total_vec, H, W, kH, padH, sH, (int)outH, (int)(outW / V));
    return check_launch("maxpool2d_w2");
  }
  const int64_t bx = (total + 255) / 256;
  if (bx >= ((int64_t)1 << 31)) return fail(AM_E_SHAPE, "%s: too many output elements", fn);
  if (total < ((int64_t)1 << 32) && (int64_t)H * W < ((int64_t)1 << 31) && kH == kW && (kH == 2 || kH == 3)) {
    const FastDiv by_outw((uint32_t)outW), by_outh((uint32_t)outH);
    if (kH == 2)
      hipLaunchKernelGGL((maxpool2d_small<T, 2, 2>), dim3((unsigned)bx), dim3(256), 0, stream(), in, out, argmax, (uint32_t)total, H, W,
                         padH, padW, sH, sW, by_outw, by_outh);
    else
      hipLaunchKernelGGL((maxpool2d_small<T, 3, 3>), dim3((unsigned)bx), dim3(256), 0, stream(), in, out, argmax, (uint32_t)total, H, W,
                         padH, padW, sH, sW, by_outw, by_outh);
    return check_launch("maxpool2d_small");
  }
  if (total < ((int64_t)1 << 32))
    hipLaunchKernelGGL((maxpool2d<T, uint32_t>), dim3((unsigned)bx), dim3(256), 0, stream(), in, out, argmax, total, C, H, W,
                       kH, kW, padH, padW, sH, sW, (int)outH, (int)outW);
  else
    hipLaunchKernelGGL((maxpool2d<T, uint64_t>), dim3((unsigned)bx), dim3(256), 0, stream(), in, out, argmax, total, C, H, W,
                       kH, kW, padH, padW, sH, sW, (int)outH, (int)outW);
  return check_launch("maxpool2d");
}

// Backward pass of max pooling: grad_in[argmax[i]] = grad_out[i] over zeros, the LAST i winning where
// overlapping windows picked the same input element (the serial order of
// src/arraymancer/nn_primitives/nnp_maxpooling.nim:68-83). Run as a gather so that nothing races: one
// lane per input element looks through the windows that contain it, highest output index first, and
// takes the first whose recorded maximum is this element.
template <typename T, typename IDX>
__global__ __launch_bounds__(256) void maxpool2d_backward(const int64_t* argmax, const T* grad_out, T* grad_in, int64_t total,
                                                          int H, int W, int kH, int kW, int padH, int padW, int sH, int sW,
                                                          int outH, int outW) {
  const int64_t p64 = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (p64 >= total) return;
  const IDX p = (IDX)p64;             // 32-bit index arithmetic whenever the tensor allows it
  const int col = (int)(p % (IDX)W);
  const IDX t = p / (IDX)W;
  const int row = (int)(t % (IDX)H);
  const IDX nc = t / (IDX)H;
  // windows h with h * sH - padH <= row < h * sH - padH + kH
  const int rh = row + padH, rw = col + padW;
  int h_hi = rh / sH, w_hi = rw / sW;
  int h_lo = rh - kH + 1 <= 0 ? 0 : (rh - kH + sH) / sH, w_lo = rw - kW + 1 <= 0 ? 0 : (rw - kW + sW) / sW;
  if (h_hi > outH - 1) h_hi = outH - 1;
  if (w_hi > outW - 1) w_hi = outW - 1;
  T g = (T)0;
  bool found = false;
  for (int h = h_hi; h >= h_lo && !found; --h)
    for (int w = w_hi; w >= w_lo; --w) {
      const int64_t o = w + (int64_t)outW * (h + (int64_t)outH * nc);
      if (argmax[o] == p64) { g = grad_out[o]; found = true; break; }
    }
  grad_in[p64] = g;
}

// Windows two wide with stride two and no padding in width (W a multiple of the 16-byte vector): a lane
// owns V consecutive input columns, i.e. V / 2 windows per candidate row of windows, read and written
// as vectors.
// At most NH x NW windows contain an input element (NH = ceil(kH / sH), NW likewise, known at compile time): their recorded
// indices and gradients are loaded together (from a clamped position where a window does not exist) and the first match
// in the order "highest output index first" decides.
template <typename T, int NH, int NW>
__global__ __launch_bounds__(256) void maxpool2d_backward_small(const int64_t* __restrict__ argmax, const T* __restrict__ grad_out,
                                                                T* __restrict__ grad_in, uint32_t total, int H, int W, int kH, int kW,
                                                                int padH, int padW, int sH, int sW, int outH, int outW,
                                                                FastDiv by_w, FastDiv by_h, FastDiv by_sh, FastDiv by_sw) {
  const uint32_t p = blockIdx.x * 256u + threadIdx.x;
  if (p >= total) return;
  uint32_t col, row;
  const uint32_t nc = by_h.divmod(by_w.divmod(p, col), row);
  const int rh = (int)row + padH, rw = (int)col + padW;
  int h_hi = (int)by_sh.div((uint32_t)rh), w_hi = (int)by_sw.div((uint32_t)rw);
  const int h_lo = rh - kH + 1 <= 0 ? 0 : (int)by_sh.div((uint32_t)(rh - kH + sH));
  const int w_lo = rw - kW + 1 <= 0 ? 0 : (int)by_sw.div((uint32_t)(rw - kW + sW));
  if (h_hi > outH - 1) h_hi = outH - 1;
  if (w_hi > outW - 1) w_hi = outW - 1;
  const int64_t obase = (int64_t)nc * outH * outW;
  constexpr bool EAGER = NH * NW <= 4;
  int64_t rec[NH][NW];
  T gv[NH][NW];
  bool ok[NH][NW];
#pragma unroll
  for (int i = 0; i < NH; ++i)
#pragma unroll
    for (int j = 0; j < NW; ++j) {
      const int h = h_hi - i, w = w_hi - j;
      ok[i][j] = h >= h_lo && w >= w_lo;
      const int64_t o = obase + (ok[i][j] ? h * outW + w : 0);
      rec[i][j] = argmax[o];
      // up to four candidates: the gradients are read with the indices, not after the comparison (one memory round
      // trip per element: 14 x 14 maps, 2 x 2 / 2: 180 -> 152 us); with nine that costs more than it saves
      if constexpr (EAGER) gv[i][j] = grad_out[o];
    }
  T g = (T)0;
  int64_t hit = -1;
#pragma unroll
  for (int i = 0; i < NH; ++i)
#pragma unroll
    for (int j = 0; j < NW; ++j)
      if (hit < 0 && ok[i][j] && rec[i][j] == (int64_t)p) {
        hit = obase + (h_hi - i) * outW + (w_hi - j);
        if constexpr (EAGER) g = gv[i][j];
      }
  if constexpr (!EAGER) { if (hit >= 0) g = grad_out[hit]; }
  grad_in[p] = g;
}

template <typename T>
__global__ __launch_bounds__(256) void maxpool2d_backward_w2(const int64_t* argmax, const T* grad_out, T* grad_in,
                                                             uint32_t total_vec, int H, int Wv, int kH, int padH, int sH,
                                                             int outH) {
  constexpr int V = 16 / (int)sizeof(T), NO = V / 2;
  typedef T vec_t __attribute__((ext_vector_type(V)));
  typedef T go_t __attribute__((ext_vector_type(NO)));
  typedef int64_t ix_t __attribute__((ext_vector_type(NO)));
  const uint32_t q = blockIdx.x * 256u + threadIdx.x;
  if (q >= total_vec) return;
  const uint32_t cv = q % (uint32_t)Wv, t = q / (uint32_t)Wv;
  const int row = (int)(t % (uint32_t)H);
  const uint32_t nc = t / (uint32_t)H;
  const int64_t p0 = (int64_t)q * V;               // flat index of the lane's first input element
  const int outW = Wv * NO;
  const int rh = row + padH;
  int h_hi = rh / sH;
  const int h_lo = rh - kH + 1 <= 0 ? 0 : (rh - kH + sH) / sH;
  if (h_hi > outH - 1) h_hi = outH - 1;
  vec_t g;
  bool found[V];
#pragma unroll
  for (int e = 0; e < V; ++e) { g[e] = (T)0; found[e] = false; }
  for (int h = h_hi; h >= h_lo; --h) {
    const int64_t o = (int64_t)cv * NO + (int64_t)outW * (h + (int64_t)outH * nc);
    const ix_t ix = *(const ix_t*)(argmax + o);
    const go_t go = *(const go_t*)(grad_out + o);
#pragma unroll
    for (int e = 0; e < V; ++e) {
      if (!found[e] && ix[e / 2] == p0 + e) { g[e] = go[e / 2]; found[e] = true; }
    }
  }
  *(vec_t*)(grad_in + p0) = g;
}

template <typename T>
static int maxpool_backward(const char* fn, int64_t N, int C, int H, int W, int kH, int kW, int padH, int padW, int sH, int sW,
                            const int64_t* argmax, const T* grad_out, T* grad_in) {
  if (N < 0 || C < 0 || H < 0 || W < 0) return fail(AM_E_SHAPE, "%s: negative extent", fn);
  if (kH < 1 || kW < 1 || sH < 1 || sW < 1 || padH < 0 || padW < 0) return fail(AM_E_ARG, "%s: kernel and stride must be >= 1, padding >= 0", fn);
  if ((int64_t)H + 2 * padH < kH || (int64_t)W + 2 * padW < kW) return fail(AM_E_SHAPE, "%s: kernel larger than the padded input", fn);
  const int64_t outH = ((int64_t)H + 2 * padH - kH) / sH + 1, outW = ((int64_t)W + 2 * padW - kW) / sW + 1;
  const int64_t total = N * C * (int64_t)H * W;
  if (total == 0) return AM_OK;
  if (!argmax || !grad_out || !grad_in) return fail(AM_E_ARG, "%s: null tensor pointer", fn);
  AM_TRY(ensure_init());
  constexpr int64_t V = 16 / (int64_t)sizeof(T);
  if (kW == 2 && sW == 2 && padW == 0 && W % (2 * V) == 0 && total / V < ((int64_t)1 << 32) && (uintptr_t)argmax % 16 == 0 &&
      (uintptr_t)grad_out % 16 == 0 && (uintptr_t)grad_in % 16 == 0) {
    const int64_t total_vec = total / V;
    hipLaunchKernelGGL((maxpool2d_backward_w2<T>), dim3((unsigned)((total_vec + 255) / 256)), dim3(256), 0, stream(), argmax,
                       grad_out, grad_in, (uint32_t)total_vec, H, (int)(W / V), kH, padH, sH, (int)outH);
    return check_launch("maxpool2d_backward_w2");
  }
  const int64_t bx = (total + 255) / 256;
  if (bx >= ((int64_t)1 << 31)) return fail(AM_E_SHAPE, "%s: too many input elements", fn);
  {
    const int nh = (kH + sH - 1) / sH, nw = (kW + sW - 1) / sW;   // windows that can contain one element
    const int64_t outH_ = ((int64_t)H + 2 * padH - kH) / sH + 1, outW_ = ((int64_t)W + 2 * padW - kW) / sW + 1;
    if (total < ((int64_t)1 << 31) && nh == nw && nh <= 3 && outH_ * outW_ < ((int64_t)1 << 31) &&
        (int64_t)H + padH < ((int64_t)1 << 30) && (int64_t)W + padW < ((int64_t)1 << 30)) {
      const FastDiv by_w((uint32_t)W), by_h((uint32_t)H), by_sh((uint32_t)sH), by_sw((uint32_t)sW);
      if (nh == 1)   // windows that do not overlap (the stride is the window or more): one candidate
        hipLaunchKernelGGL((maxpool2d_backward_small<T, 1, 1>), dim3((unsigned)bx), dim3(256), 0, stream(), argmax, grad_out, grad_in,
                           (uint32_t)total, H, W, kH, kW, padH, padW, sH, sW, (int)outH_, (int)outW_, by_w, by_h, by_sh, by_sw);
      else if (nh == 2)
        hipLaunchKernelGGL((maxpool2d_backward_small<T, 2, 2>), dim3((unsigned)bx), dim3(256), 0, stream(), argmax, grad_out, grad_in,
                           (uint32_t)total, H, W, kH, kW, padH, padW, sH, sW, (int)outH_, (int)outW_, by_w, by_h, by_sh, by_sw);
      else
        hipLaunchKernelGGL((maxpool2d_backward_small<T, 3, 3>), dim3((unsigned)bx), dim3(256), 0, stream(), argmax, grad_out, grad_in,
                           (uint32_t)total, H, W, kH, kW, padH, padW, sH, sW, (int)outH_, (int)outW_, by_w, by_h, by_sh, by_sw);
      return check_launch("maxpool2d_backward_small");
    }
  }
  if (total < ((int64_t)1 << 32))
    hipLaunchKernelGGL((maxpool2d_backward<T, uint32_t>), dim3((unsigned)bx), dim3(256), 0, stream(), argmax, grad_out, grad_in,
                       total, H, W, kH, kW, padH, padW, sH, sW, (int)outH, (int)outW);
  else
    hipLaunchKernelGGL((maxpool2d_backward<T, uint64_t>), dim3((unsigned)bx), dim3(256), 0, stream(), argmax, grad_out, grad_in,
                       total, H, W, kH, kW, padH, padW, sH, sW, (int)outH, (int)outW);
  return check_launch("maxpool2d_backward");
}

}  // namespace red
}  // namespace am

using namespace am;

#define AM_RED_ENTRY_POINTS(T, SFX)                                                                                    \
  extern "C" int am_hip_reduce_axis_##SFX(int op, int rank, const int64_t* shape, int axis, T* dst,                    \
                                          const int64_t* dst_strides, const T* a, const int64_t* a_strides) {          \
    return red::reduce_axis<T>("am_hip_reduce_axis_" #SFX, op, rank, shape, axis, dst, dst_strides, a, a_strides);     \
  }                                                                                                                    \
  extern "C" int am_hip_reduce_all_##SFX(int op, int rank, const int64_t* shape, const T* a, const int64_t* a_strides, \
                                         T* result) {                                                                  \
    return red::reduce_all<T>("am_hip_reduce_all_" #SFX, op, rank, shape, a, a_strides, result);                       \
  }                                                                                                                    \
  extern "C" int am_hip_argreduce_##SFX(int op, int rank, const int64_t* shape, int axis, int64_t* idx,                \
                                        const int64_t* idx_strides, T* val, const int64_t* val_strides, const T* a,    \
                                        const int64_t* a_strides) {                                                    \
    return red::argreduce<T>("am_hip_argreduce_" #SFX, op, rank, shape, axis, idx, idx_strides, val, val_strides, a,   \
                             a_strides);                                                                               \
  }                                                                                                                    \
  extern "C" int am_hip_maxpool2d_##SFX(int64_t N, int C, int H, int W, int kH, int kW, int padH, int padW,            \
                                        int strideH, int strideW, const T* input, T* output, int64_t* argmax) {        \
    return red::maxpool<T>("am_hip_maxpool2d_" #SFX, N, C, H, W, kH, kW, padH, padW, strideH, strideW, input, output,  \
                           argmax);                                                                                    \
  }                                                                                                                    \
  extern "C" int am_hip_maxpool2d_backward_##SFX(int64_t N, int C, int H, int W, int kH, int kW, int padH, int padW,   \
                                                 int strideH, int strideW, const int64_t* argmax, const T* grad_output, \
                                                 T* grad_input) {                                                      \
    return red::maxpool_backward<T>("am_hip_maxpool2d_backward_" #SFX, N, C, H, W, kH, kW, padH, padW, strideH,        \
                                    strideW, argmax, grad_output, grad_input);                                         \
  }

AM_RED_ENTRY_POINTS(float, f32)
AM_RED_ENTRY_POINTS(double, f64)
AM_RED_ENTRY_POINTS(int32_t, i32)
AM_RED_ENTRY_POINTS(int64_t, i64)

extern "C" int am_hip_softmax_rows_f32(int64_t rows, int64_t cols, float* dst, int64_t dst_rs, int64_t dst_cs,
                                       const float* src, int64_t src_rs, int64_t src_cs) {
  return red::softmax<float>("am_hip_softmax_rows_f32", rows, cols, dst, dst_rs, dst_cs, src, src_rs, src_cs);
}
extern "C" int am_hip_softmax_rows_f64(int64_t rows, int64_t cols, double* dst, int64_t dst_rs, int64_t dst_cs,
                                       const double* src, int64_t src_rs, int64_t src_cs) {
  return red::softmax<double>("am_hip_softmax_rows_f64", rows, cols, dst, dst_rs, dst_cs, src, src_rs, src_cs);
}
