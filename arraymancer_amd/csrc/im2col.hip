// im2col on the device for a whole NCHW batch: am_hip_im2col_*.
//
// The reference unrolls one image at a time on the host and multiplies per image
// (src/arraymancer/nn_primitives/fallback/conv.nim:18-54 im2col, :99-103 per-image loop with a
// "TODO: batch matmul"). Here one launch writes col[n][c * kH * kW + kh * kW + kw][h * W_out + w]
// for every image n, so that a single strided-batched GEMM  out[n] = kernel_col * col[n] (+ bias)
// finishes the convolution. Same index arithmetic as the reference, zero padding included.
#include "common.h"

using namespace am;

namespace {

struct Im2colArgs {
  int64_t total;       // N * C*kH*kW * H_out * W_out
  int C, H, W, kH, kW, padH, padW, strideH, strideW, Hout, Wout;
  int64_t in_n, in_c, in_h, in_w;   // input strides (elements)
};

template <typename T>
__global__ __launch_bounds__(256) void im2col_kernel(Im2colArgs p, const T* __restrict__ in, T* __restrict__ col) {
  const int64_t P = (int64_t)p.Hout * p.Wout;
  const int64_t CK = (int64_t)p.C * p.kH * p.kW;
  for (int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x; idx < p.total; idx += (int64_t)gridDim.x * 256) {
    const int64_t n = idx / (CK * P);
    const int64_t r = idx - n * CK * P;
    const int c = (int)(r / P);                 // row of the column matrix
    const int pix = (int)(r - (int64_t)c * P);
    const int h = pix / p.Wout, w = pix - h * p.Wout;
    const int w_off = c % p.kW - p.padW;
    const int h_off = (c / p.kW) % p.kH - p.padH;
    const int c_off = (c / p.kW) / p.kH;
    const int row = h_off + h * p.strideH, cc = w_off + w * p.strideW;
    T v = (T)0;
    if (row >= 0 && cc >= 0 && row < p.H && cc < p.W) v = in[n * p.in_n + c_off * p.in_c + row * p.in_h + cc * p.in_w];
    col[idx] = v;
  }
}

// One lane per 16 bytes of one row of the column matrix (V consecutive output pixels of one (n, c)):
// 32-bit index arithmetic, five divisions per lane instead of seven 64-bit ones per element, one
// 16-byte store. Needs H_out * W_out to be a multiple of V and fewer than 2^32 vectors.
template <typename T, bool STREAM>
__global__ __launch_bounds__(256) void im2col_vec(Im2colArgs p, const T* __restrict__ in, T* __restrict__ col, uint32_t total_vec) {
  constexpr int V = 16 / (int)sizeof(T);
  typedef T vec_t __attribute__((ext_vector_type(V)));
  const uint32_t Pv = (uint32_t)(p.Hout * p.Wout) / V;
  const uint32_t CK = (uint32_t)(p.C * p.kH * p.kW);
  for (uint32_t q = blockIdx.x * 256u + threadIdx.x; q < total_vec; q += gridDim.x * 256u) {
    const uint32_t rid = q / Pv, pv = q - rid * Pv;          // row of the column matrix over all images, vector in it
    const uint32_t n = rid / CK, c = rid - n * CK;
    const uint32_t ck = c / (uint32_t)p.kW;
    const int w_off = (int)(c - ck * (uint32_t)p.kW) - p.padW;
    const uint32_t c_off = ck / (uint32_t)p.kH;
    const int h_off = (int)(ck - c_off * (uint32_t)p.kH) - p.padH;
    const uint32_t pix0 = pv * V;
    int h = (int)(pix0 / (uint32_t)p.Wout), w = (int)(pix0 - (uint32_t)h * (uint32_t)p.Wout);
    const T* __restrict__ base = in + (int64_t)n * p.in_n + (int64_t)c_off * p.in_c;
    vec_t v;
#pragma unroll
    for (int e = 0; e < V; ++e) {
      const int row = h_off + h * p.strideH, cc = w_off + w * p.strideW;
      v[e] = (row >= 0 && cc >= 0 && row < p.H && cc < p.W) ? base[(int64_t)row * p.in_h + (int64_t)cc * p.in_w] : (T)0;
      if (++w == p.Wout) { w = 0; ++h; }
    }
    // a column matrix beyond the memory-side cache is written past it; a smaller one stays there for the GEMM
    if constexpr (STREAM) __builtin_nontemporal_store(v, (vec_t*)(col + (int64_t)q * V));
    else *(vec_t*)(col + (int64_t)q * V) = v;
  }
}

template <typename T>
int im2col(const char* fn, int64_t N, int C, int H, int W, int kH, int kW, int padH, int padW, int strideH,
           int strideW, const T* in, int64_t in_n, int64_t in_c, int64_t in_h, int64_t in_w, T* col) {
  if (N < 0 || C <= 0 || H <= 0 || W <= 0 || kH <= 0 || kW <= 0 || padH < 0 || padW < 0 || strideH <= 0 || strideW <= 0)
    return fail(AM_E_ARG, "%s: bad geometry", fn);
  const int Hout = (H + 2 * padH - kH) / strideH + 1, Wout = (W + 2 * padW - kW) / strideW + 1;
  if (Hout <= 0 || Wout <= 0) return fail(AM_E_SHAPE, "%s: kernel larger than the padded image", fn);
  Im2colArgs a;
  a.total = N * (int64_t)C * kH * kW * Hout * Wout;
  if (a.total == 0) return AM_OK;
  if (!in || !col) return fail(AM_E_ARG, "%s: null pointer", fn);
  AM_TRY(ensure_init());
  a.C = C; a.H = H; a.W = W; a.kH = kH; a.kW = kW; a.padH = padH; a.padW = padW;
  a.strideH = strideH; a.strideW = strideW; a.Hout = Hout; a.Wout = Wout;
  a.in_n = in_n; a.in_c = in_c; a.in_h = in_h; a.in_w = in_w;
  constexpr int64_t V = 16 / (int64_t)sizeof(T);
  const int64_t cap = (int64_t)num_cus() * 32;
  if (((int64_t)Hout * Wout) % V == 0 && a.total / V < ((int64_t)1 << 32) && (int64_t)C * kH * kW < ((int64_t)1 << 31) &&
      (uintptr_t)col % 16 == 0) {
    int64_t blocks = (a.total / V + 255) / 256;
    if (blocks > cap) blocks = cap;
    if ((double)a.total * sizeof(T) > 384.0 * 1024 * 1024)
      hipLaunchKernelGGL((im2col_vec<T, true>), dim3((unsigned)blocks), dim3(256), 0, stream(), a, in, col, (uint32_t)(a.total / V));
    else
      hipLaunchKernelGGL((im2col_vec<T, false>), dim3((unsigned)blocks), dim3(256), 0, stream(), a, in, col, (uint32_t)(a.total / V));
    return check_launch("im2col");
  }
  int64_t blocks = (a.total + 255) / 256;
  if (blocks > cap) blocks = cap;
  hipLaunchKernelGGL((im2col_kernel<T>), dim3((unsigned)blocks), dim3(256), 0, stream(), a, in, col);
  return check_launch("im2col");
}

}  // namespace

#define AM_IM2COL_ENTRY(T, SFX)                                                                                  \
  extern "C" int am_hip_im2col_##SFX(int64_t N, int C, int H, int W, int kH, int kW, int padH, int padW,         \
                                     int strideH, int strideW, const T* in, int64_t in_n, int64_t in_c,          \
                                     int64_t in_h, int64_t in_w, T* col) {                                       \
    return im2col<T>("am_hip_im2col_" #SFX, N, C, H, W, kH, kW, padH, padW, strideH, strideW, in, in_n, in_c,    \
                     in_h, in_w, col);                                                                           \
  }
AM_IM2COL_ENTRY(float, f32)
AM_IM2COL_ENTRY(double, f64)
AM_IM2COL_ENTRY(int32_t, i32)
AM_IM2COL_ENTRY(int64_t, i64)
