// The SGD update of ALL parameters of a model in one launch: am_hip_sgd_update_*.
//
// The reference's optimizer walks the parameters and runs one apply2_inline per tensor, value <- value - lr * grad
// (src/arraymancer/nn/optimizers/optimizers.nim:35-51). A model has a handful to a few hundred parameter tensors, many
// of them biases of a few hundred elements: one launch each is all launch latency. Here up to 64 (value, gradient)
// pairs travel in the kernel's argument block; a workgroup takes one 4096-element piece of one tensor (found by a scan
// over the tensors' piece counts), so the launch is as wide as the parameters are large. Same expression, the product
// rounded before the subtraction, so the bits are those of the per-tensor passes. Contiguous tensors.
#include "common.h"

namespace am {
namespace optim {

constexpr int kMaxTensors = 64;
constexpr int kPiece = 4096;

template <typename T> struct Args {
  T* value[kMaxTensors];
  const T* grad[kMaxTensors];
  int64_t size[kMaxTensors];
  uint32_t first_piece[kMaxTensors + 1];   // running sum of the tensors' piece counts
  int count;
  T lr;
};

template <typename T>
__global__ __launch_bounds__(256) void sgd_update(Args<T> p) {
  constexpr int V = 16 / (int)sizeof(T);
  typedef T vec_t __attribute__((ext_vector_type(V)));
  int t = 0;
  while (t + 1 < p.count && blockIdx.x >= p.first_piece[t + 1]) ++t;
  const int64_t lo = (int64_t)(blockIdx.x - p.first_piece[t]) * kPiece;
  const int64_t hi = (lo + kPiece < p.size[t]) ? lo + kPiece : p.size[t];
  T* __restrict__ x = p.value[t];
  const T* __restrict__ g = p.grad[t];
  const bool vec = ((uintptr_t)x % 16 == 0) && ((uintptr_t)g % 16 == 0);
  if (vec) {
    int64_t i = lo + (int64_t)threadIdx.x * V;
    for (; i + V <= hi; i += 256 * V) {
      vec_t xv = *(vec_t*)(x + i);
      const vec_t gv = *(const vec_t*)(g + i);
#pragma unroll
      for (int e = 0; e < V; ++e) xv[e] = xv[e] - p.lr * gv[e];
      *(vec_t*)(x + i) = xv;
    }
    // the last, partial vector of the tensor (pieces are whole vectors except at the tensor's end)
    const int64_t tail = lo + (hi - lo) / V * V;
    if (threadIdx.x < (unsigned)(hi - tail)) x[tail + threadIdx.x] = x[tail + threadIdx.x] - p.lr * g[tail + threadIdx.x];
  } else {
    for (int64_t i = lo + threadIdx.x; i < hi; i += 256) x[i] = x[i] - p.lr * g[i];
  }
}

template <typename T>
static int update(const char* fn, int count, T* const* values, const T* const* grads, const int64_t* sizes, T lr) {
  if (count < 0) return fail(AM_E_ARG, "%s: negative tensor count", fn);
  if (count == 0) return AM_OK;
  if (!values || !grads || !sizes) return fail(AM_E_ARG, "%s: null array", fn);
  AM_TRY(ensure_init());
  int i = 0;
  while (i < count) {   // at most kMaxTensors tensors per launch
    Args<T> p;
    p.count = 0; p.lr = lr;
    uint32_t pieces = 0;
    for (; i < count && p.count < kMaxTensors; ++i) {
      if (sizes[i] < 0) return fail(AM_E_SHAPE, "%s: negative size", fn);
      if (sizes[i] == 0) continue;
      if (!values[i] || !grads[i]) return fail(AM_E_ARG, "%s: null tensor pointer", fn);
      const int64_t n = (sizes[i] + kPiece - 1) / kPiece;
      if (n + pieces >= ((int64_t)1 << 31)) {
        if (p.count == 0) return fail(AM_E_SHAPE, "%s: a tensor with too many elements for one launch", fn);
        break;   // this tensor starts the next launch
      }
      p.value[p.count] = values[i]; p.grad[p.count] = grads[i]; p.size[p.count] = sizes[i];
      p.first_piece[p.count] = pieces;
      pieces += (uint32_t)n;
      ++p.count;
    }
    if (p.count == 0) continue;
    p.first_piece[p.count] = pieces;
    hipLaunchKernelGGL((sgd_update<T>), dim3(pieces), dim3(256), 0, stream(), p);
    AM_TRY(check_launch("sgd_update"));
  }
  return AM_OK;
}

}  // namespace optim
}  // namespace am

using namespace am;

extern "C" int am_hip_sgd_update_f32(int count, float* const* values, const float* const* grads, const int64_t* sizes, float learning_rate) {
  return optim::update<float>("am_hip_sgd_update_f32", count, values, grads, sizes, learning_rate);
}
extern "C" int am_hip_sgd_update_f64(int count, double* const* values, const double* const* grads, const int64_t* sizes, double learning_rate) {
  return optim::update<double>("am_hip_sgd_update_f64", count, values, grads, sizes, learning_rate);
}
