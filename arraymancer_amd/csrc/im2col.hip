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
  int64_t blocks = (a.total + 255) / 256;
  const int64_t cap = (int64_t)num_cus() * 32;
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
