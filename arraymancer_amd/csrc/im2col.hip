// im2col on the device for a whole NCHW batch: am_hip_im2col_*.
//
// The reference unrolls one image at a time on the host and multiplies per image
// (src/arraymancer/nn_primitives/fallback/conv.nim:18-54 im2col, :99-103 per-image loop with a
// "TODO: batch matmul"). Here one launch writes col[n][c * kH * kW + kh * kW + kw][h * W_out + w]
// for every image n, so that a single strided-batched GEMM  out[n] = kernel_col * col[n] (+ bias)
// finishes the convolution. Same index arithmetic as the reference, zero padding included.
// am_hip_im2col_strided_* places image n's row c at col + n * col_n + c * col_c (unit stride along a row), so that the
// batch can also be folded into the columns ([C*kH*kW][N * H_out*W_out]: col_n = H_out*W_out, col_c = N * col_n), the
// layout in which the backward pass of the convolution is two plain products. am_hip_col2im_* is the reverse
// (fallback/conv.nim:55-79): every pixel sums the column entries that cover it.
#include "common.h"
#include "fastdiv.h"
#include <type_traits>

using namespace am;

namespace {

struct Im2colArgs {
  int64_t total;       // N * C*kH*kW * H_out * W_out
  int C, H, W, kH, kW, padH, padW, strideH, strideW, Hout, Wout;
  int64_t in_n, in_c, in_h, in_w;   // input strides (elements)
  int64_t col_n, col_c;             // image and row strides of the column matrix (elements); unit stride along a row
  FastDiv by_pv, by_ck, by_kw, by_kh, by_wout;   // vectors per row, rows per image, kernel extents, output width
  FastDiv by_ckp, by_p;                          // element-wise kernel: elements per image, per row
};

// One lane per element. FAST: fewer than 2^32 elements and fewer than 2^31 per image, the index is taken apart with
// the launch-constant dividers; otherwise with 64-bit divisions.
template <typename T, bool FAST>
__global__ __launch_bounds__(256) void im2col_kernel(Im2colArgs p, const T* __restrict__ in, T* __restrict__ col) {
  const int64_t P = (int64_t)p.Hout * p.Wout;
  const int64_t CK = (int64_t)p.C * p.kH * p.kW;
  for (int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x; idx < p.total; idx += (int64_t)gridDim.x * 256) {
    int64_t n;
    int c, pix, h, w, w_off, h_off, c_off;
    if constexpr (FAST) {
      uint32_t r, upix, uw, kw, kh;
      n = p.by_ckp.divmod((uint32_t)idx, r);
      c = (int)p.by_p.divmod(r, upix);
      pix = (int)upix;
      h = (int)p.by_wout.divmod(upix, uw);
      w = (int)uw;
      c_off = (int)p.by_kh.divmod(p.by_kw.divmod((uint32_t)c, kw), kh);
      w_off = (int)kw - p.padW; h_off = (int)kh - p.padH;
    } else {
      n = idx / (CK * P);
      const int64_t r = idx - n * CK * P;
      c = (int)(r / P);                 // row of the column matrix
      pix = (int)(r - (int64_t)c * P);
      h = pix / p.Wout; w = pix - h * p.Wout;
      w_off = c % p.kW - p.padW;
      h_off = (c / p.kW) % p.kH - p.padH;
      c_off = (c / p.kW) / p.kH;
    }
    const int row = h_off + h * p.strideH, cc = w_off + w * p.strideW;
    T v = (T)0;
    if (row >= 0 && cc >= 0 && row < p.H && cc < p.W) v = in[n * p.in_n + c_off * p.in_c + row * p.in_h + cc * p.in_w];
    col[n * p.col_n + (int64_t)c * p.col_c + pix] = v;
  }
}

// One lane per 16 bytes of one row of the column matrix (V consecutive output pixels of one (n, c)):
// 32-bit index arithmetic with the launch-constant dividers, one 16-byte load where the pixels are V neighbours of
// one image row inside the image (unit stride along the width), element loads at the borders, one 16-byte store. Needs H_out * W_out to be a multiple of V and fewer than 2^32 vectors.
template <typename T, bool STREAM, bool UNITW>
__global__ __launch_bounds__(256) void im2col_vec(Im2colArgs p, const T* __restrict__ in, T* __restrict__ col, uint32_t total_vec) {
  constexpr int V = 16 / (int)sizeof(T);
  typedef T vec_t __attribute__((ext_vector_type(V)));
  typedef vec_t gvec_t __attribute__((aligned(sizeof(T))));
  const uint64_t step = (uint64_t)gridDim.x * 256u;
  for (uint64_t q64 = (uint64_t)blockIdx.x * 256u + threadIdx.x; q64 < total_vec; q64 += step) {
    const uint32_t q = (uint32_t)q64;
    uint32_t pv, c, kw, kh, w_;
    const uint32_t rid = p.by_pv.divmod(q, pv);              // row of the column matrix over all images, vector in it
    const uint32_t n = p.by_ck.divmod(rid, c);
    const uint32_t ck = p.by_kw.divmod(c, kw);
    const uint32_t c_off = p.by_kh.divmod(ck, kh);
    const int w_off = (int)kw - p.padW, h_off = (int)kh - p.padH;
    const uint32_t pix0 = pv * V;
    int h = (int)p.by_wout.divmod(pix0, w_), w = (int)w_;
    const T* __restrict__ base = in + (int64_t)n * p.in_n + (int64_t)c_off * p.in_c;
    vec_t v;
    const int row0 = h_off + h * p.strideH, cc0 = w_off + w * p.strideW;
    if (UNITW && w + V <= p.Wout && row0 >= 0 && row0 < p.H && cc0 >= 0 && cc0 + V <= p.W) {
      // V neighbouring pixels of one image row, all inside the image: one load (from any element-aligned address)
      v = *(const gvec_t*)(base + (int64_t)row0 * p.in_h + cc0);
    } else {
#pragma unroll
      for (int e = 0; e < V; ++e) {
        const int row = h_off + h * p.strideH, cc = w_off + w * p.strideW;
        v[e] = (row >= 0 && cc >= 0 && row < p.H && cc < p.W) ? base[(int64_t)row * p.in_h + (int64_t)cc * p.in_w] : (T)0;
        if (++w == p.Wout) { w = 0; ++h; }
      }
    }
    // a column matrix beyond the memory-side cache is written past it; a smaller one stays there for the GEMM
    T* at = col + (int64_t)n * p.col_n + (int64_t)c * p.col_c + (int64_t)pix0;
    if constexpr (STREAM) __builtin_nontemporal_store(v, (vec_t*)at);
    else *(vec_t*)at = v;
  }
}

template <typename T>
int im2col(const char* fn, int64_t N, int C, int H, int W, int kH, int kW, int padH, int padW, int strideH,
           int strideW, const T* in, int64_t in_n, int64_t in_c, int64_t in_h, int64_t in_w, T* col, int64_t col_n, int64_t col_c) {
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
  const int64_t P = (int64_t)Hout * Wout;
  if (col_n == 0 && col_c == 0) { col_c = P; col_n = (int64_t)C * kH * kW * P; }   // [N][C*kH*kW][P]
  if (col_c < P || col_n < P) return fail(AM_E_ARG, "%s: rows of the column matrix overlap", fn);
  a.col_n = col_n; a.col_c = col_c;
  constexpr int64_t V = 16 / (int64_t)sizeof(T);
  a.by_pv = FastDiv((uint32_t)(P / V > 0 ? P / V : 1)); a.by_ck = FastDiv((uint32_t)((int64_t)C * kH * kW));
  a.by_kw = FastDiv((uint32_t)kW); a.by_kh = FastDiv((uint32_t)kH); a.by_wout = FastDiv((uint32_t)Wout);
  const int64_t cap = (int64_t)num_cus() * 32;
  if (((int64_t)Hout * Wout) % V == 0 && a.total / V < ((int64_t)1 << 32) && (int64_t)C * kH * kW < ((int64_t)1 << 31) &&
      (uintptr_t)col % 16 == 0 && col_n % V == 0 && col_c % V == 0) {
    int64_t blocks = (a.total / V + 255) / 256;
    if (blocks > cap) blocks = cap;
    const bool stream_out = (double)a.total * sizeof(T) > 384.0 * 1024 * 1024;
    const bool unit_w = strideW == 1 && in_w == 1;   // UNITW: neighbouring output pixels are neighbouring input elements
    const dim3 grid((unsigned)blocks), block(256);
    const uint32_t nv = (uint32_t)(a.total / V);
    if (stream_out && unit_w) hipLaunchKernelGGL((im2col_vec<T, true, true>), grid, block, 0, stream(), a, in, col, nv);
    else if (stream_out) hipLaunchKernelGGL((im2col_vec<T, true, false>), grid, block, 0, stream(), a, in, col, nv);
    else if (unit_w) hipLaunchKernelGGL((im2col_vec<T, false, true>), grid, block, 0, stream(), a, in, col, nv);
    else hipLaunchKernelGGL((im2col_vec<T, false, false>), grid, block, 0, stream(), a, in, col, nv);
    return check_launch("im2col");
  }
  int64_t blocks = (a.total + 255) / 256;
  if (blocks > cap) blocks = cap;
  const int64_t per_image = (int64_t)C * kH * kW * P;
  if (a.total < ((int64_t)1 << 32) && per_image < ((int64_t)1 << 31)) {
    a.by_ckp = FastDiv((uint32_t)per_image); a.by_p = FastDiv((uint32_t)P);
    hipLaunchKernelGGL((im2col_kernel<T, true>), dim3((unsigned)blocks), dim3(256), 0, stream(), a, in, col);
  } else {
    hipLaunchKernelGGL((im2col_kernel<T, false>), dim3((unsigned)blocks), dim3(256), 0, stream(), a, in, col);
  }
  return check_launch("im2col");
}


struct Col2imArgs {
  int64_t total;       // N * C * H * W
  int C, H, W, kH, kW, padH, padW, strideH, strideW, Hout, Wout;
  int64_t col_n, col_c;                   // image and row strides of the column matrix (elements)
  int64_t out_n, out_c, out_h, out_w;     // strides of the image batch that is written (elements)
  FastDiv by_w, by_h, by_c;               // for fewer than 2^31 pixels
};

template <typename T> __device__ __forceinline__ T wrap_add(T x, T y) {
  if constexpr (std::is_integral_v<T>) return (T)((std::make_unsigned_t<T>)x + (std::make_unsigned_t<T>)y);
  else return x + y;
}

// The reference scatters: row by row of the column matrix it adds each entry to the pixel that it covers. Here one
// lane per pixel gathers instead: for every kernel offset (kh, kw) at most one column entry covers the pixel, and
// walking the offsets in increasing order adds them in the order in which the reference's loop meets them (a row of
// the column matrix is one (c, kh, kw)), starting from the same zero, so float results have the reference's bits.
// Lanes that are neighbours along x read neighbouring entries of one row (stride 1 / strideW): every entry of the
// column matrix is read once, the kernel is bound by that read.
// KW > 0: unit strides and a kernel KW wide, known at compile time: the KW loads of a kernel row are issued together
// (from a clamped address where no entry covers the pixel) and added afterwards, in order; KW == 0: any geometry.
template <typename T, typename IDX, int KW>
__global__ __launch_bounds__(256) void col2im_kernel(Col2imArgs p, const T* __restrict__ col, T* __restrict__ out) {
  const IDX total = (IDX)p.total;
  for (IDX idx = (IDX)blockIdx.x * 256 + threadIdx.x; idx < total; idx += (IDX)gridDim.x * 256) {
    int x, y, c;
    IDX n;
    if constexpr (sizeof(IDX) == 4) {
      uint32_t ux, uy, uc;
      n = p.by_c.divmod(p.by_h.divmod(p.by_w.divmod((uint32_t)idx, ux), uy), uc);
      x = (int)ux; y = (int)uy; c = (int)uc;
    } else {
      const IDX q1 = idx / (IDX)p.W;
      x = (int)(idx - q1 * (IDX)p.W);
      const IDX q2 = q1 / (IDX)p.H;
      y = (int)(q1 - q2 * (IDX)p.H);
      n = q2 / (IDX)p.C;
      c = (int)(q2 - n * (IDX)p.C);
    }
    const T* __restrict__ rows = col + (int64_t)n * p.col_n + (int64_t)c * p.kH * p.kW * p.col_c;
    T acc = (T)0;
    if constexpr (KW > 0) {
      const int wx0 = x + p.padW;
      for (int kh = 0; kh < p.kH; ++kh) {
        const int h = y + p.padH - kh;
        if (h < 0) break;
        if (h >= p.Hout) continue;
        const T* __restrict__ row = rows + (int64_t)kh * KW * p.col_c + (int64_t)h * p.Wout;
        T v[KW];
        bool ok[KW];
#pragma unroll
        for (int kw = 0; kw < KW; ++kw) {
          const int w = wx0 - kw;
          ok[kw] = w >= 0 && w < p.Wout;
          v[kw] = row[(int64_t)kw * p.col_c + (ok[kw] ? w : 0)];
        }
#pragma unroll
        for (int kw = 0; kw < KW; ++kw)
          if (ok[kw]) acc = wrap_add(acc, v[kw]);
      }
    } else {
      // only every strideH-th kernel row (strideW-th column) can cover the pixel: kh = (y + padH) mod strideH, then
      // in steps of strideH, with the output row going down by one each time
      const int hy0 = y + p.padH, wx0 = x + p.padW;
      const int qh = hy0 / p.strideH, qw = wx0 / p.strideW;
      const int kh0 = hy0 - qh * p.strideH, kw0 = wx0 - qw * p.strideW;
      for (int kh = kh0, h = qh; kh < p.kH && h >= 0; kh += p.strideH, --h) {
        if (h >= p.Hout) continue;
        const T* __restrict__ row = rows + (int64_t)kh * p.kW * p.col_c + (int64_t)h * p.Wout;
        for (int kw = kw0, w = qw; kw < p.kW && w >= 0; kw += p.strideW, --w) {
          if (w >= p.Wout) continue;
          acc = wrap_add(acc, row[(int64_t)kw * p.col_c + w]);
        }
      }
    }
    out[(int64_t)n * p.out_n + (int64_t)c * p.out_c + (int64_t)y * p.out_h + (int64_t)x * p.out_w] = acc;
  }
}

template <typename T>
int col2im(const char* fn, int64_t N, int C, int H, int W, int kH, int kW, int padH, int padW, int strideH, int strideW,
           const T* col, int64_t col_n, int64_t col_c, T* out, int64_t out_n, int64_t out_c, int64_t out_h, int64_t out_w) {
  if (N < 0 || C <= 0 || H <= 0 || W <= 0 || kH <= 0 || kW <= 0 || padH < 0 || padW < 0 || strideH <= 0 || strideW <= 0)
    return fail(AM_E_ARG, "%s: bad geometry", fn);
  const int Hout = (H + 2 * padH - kH) / strideH + 1, Wout = (W + 2 * padW - kW) / strideW + 1;
  if (Hout <= 0 || Wout <= 0) return fail(AM_E_SHAPE, "%s: kernel larger than the padded image", fn);
  if ((int64_t)C * kH * kW >= ((int64_t)1 << 31)) return fail(AM_E_SHAPE, "%s: column matrix with 2^31 rows or more", fn);
  Col2imArgs a;
  a.total = N * (int64_t)C * H * W;
  if (a.total == 0) return AM_OK;
  if (!col || !out) return fail(AM_E_ARG, "%s: null pointer", fn);
  if (col_n < 0 || col_c < 0) return fail(AM_E_ARG, "%s: negative stride of the column matrix", fn);
  AM_TRY(ensure_init());
  a.C = C; a.H = H; a.W = W; a.kH = kH; a.kW = kW; a.padH = padH; a.padW = padW;
  a.strideH = strideH; a.strideW = strideW; a.Hout = Hout; a.Wout = Wout;
  a.col_n = col_n; a.col_c = col_c; a.out_n = out_n; a.out_c = out_c; a.out_h = out_h; a.out_w = out_w;
  a.by_w = FastDiv((uint32_t)W); a.by_h = FastDiv((uint32_t)H); a.by_c = FastDiv((uint32_t)C);
  int64_t blocks = (a.total + 255) / 256;
  const int64_t cap = (int64_t)num_cus() * 32;
  if (blocks > cap) blocks = cap;
  const dim3 grid((unsigned)blocks), block(256);
  if (a.total >= ((int64_t)1 << 31)) {
    hipLaunchKernelGGL((col2im_kernel<T, int64_t, 0>), grid, block, 0, stream(), a, col, out);
  } else if (strideH == 1 && strideW == 1 && kW <= 7) {
    switch (kW) {
      case 1: hipLaunchKernelGGL((col2im_kernel<T, uint32_t, 1>), grid, block, 0, stream(), a, col, out); break;
      case 2: hipLaunchKernelGGL((col2im_kernel<T, uint32_t, 2>), grid, block, 0, stream(), a, col, out); break;
      case 3: hipLaunchKernelGGL((col2im_kernel<T, uint32_t, 3>), grid, block, 0, stream(), a, col, out); break;
      case 4: hipLaunchKernelGGL((col2im_kernel<T, uint32_t, 4>), grid, block, 0, stream(), a, col, out); break;
      case 5: hipLaunchKernelGGL((col2im_kernel<T, uint32_t, 5>), grid, block, 0, stream(), a, col, out); break;
      case 6: hipLaunchKernelGGL((col2im_kernel<T, uint32_t, 6>), grid, block, 0, stream(), a, col, out); break;
      default: hipLaunchKernelGGL((col2im_kernel<T, uint32_t, 7>), grid, block, 0, stream(), a, col, out); break;
    }
  } else {
    hipLaunchKernelGGL((col2im_kernel<T, uint32_t, 0>), grid, block, 0, stream(), a, col, out);
  }
  return check_launch("col2im");
}

}  // namespace

#define AM_IM2COL_ENTRY(T, SFX)                                                                                  \
  extern "C" int am_hip_im2col_##SFX(int64_t N, int C, int H, int W, int kH, int kW, int padH, int padW,         \
                                     int strideH, int strideW, const T* in, int64_t in_n, int64_t in_c,          \
                                     int64_t in_h, int64_t in_w, T* col) {                                       \
    return im2col<T>("am_hip_im2col_" #SFX, N, C, H, W, kH, kW, padH, padW, strideH, strideW, in, in_n, in_c,    \
                     in_h, in_w, col, 0, 0);                                                                     \
  }                                                                                                              \
  extern "C" int am_hip_im2col_strided_##SFX(int64_t N, int C, int H, int W, int kH, int kW, int padH, int padW, \
                                             int strideH, int strideW, const T* in, int64_t in_n, int64_t in_c,  \
                                             int64_t in_h, int64_t in_w, T* col, int64_t col_n, int64_t col_c) { \
    if (col_n <= 0 || col_c <= 0) return fail(AM_E_ARG, "am_hip_im2col_strided_" #SFX ": strides must be positive"); \
    return im2col<T>("am_hip_im2col_strided_" #SFX, N, C, H, W, kH, kW, padH, padW, strideH, strideW, in, in_n,  \
                     in_c, in_h, in_w, col, col_n, col_c);                                                       \
  }                                                                                                              \
  extern "C" int am_hip_col2im_##SFX(int64_t N, int C, int H, int W, int kH, int kW, int padH, int padW,         \
                                     int strideH, int strideW, const T* col, int64_t col_n, int64_t col_c,       \
                                     T* out, int64_t out_n, int64_t out_c, int64_t out_h, int64_t out_w) {       \
    return col2im<T>("am_hip_col2im_" #SFX, N, C, H, W, kH, kW, padH, padW, strideH, strideW, col, col_n, col_c, \
                     out, out_n, out_c, out_h, out_w);                                                           \
  }
AM_IM2COL_ENTRY(float, f32)
AM_IM2COL_ENTRY(double, f64)
AM_IM2COL_ENTRY(int32_t, i32)
AM_IM2COL_ENTRY(int64_t, i64)
