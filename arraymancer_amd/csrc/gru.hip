// The gate arithmetic of a GRU cell as ONE pass, forward and backward: am_hip_gru_gates_*, am_hip_gru_gates_backward_*.
//
// The reference runs steps 2 - 4 of gru_cell_inference / gru_cell_forward
// (src/arraymancer/nn_primitives/nnp_gru.nim:72-88, 125-146) as three element-wise passes over column slices of the
// two [batch, 3H] products W3x = W3 * x + bW3 and U3h = U3 * h + bU3:
//     r = sigmoid(W3x[:, 0:H] + U3h[:, 0:H])     z = sigmoid(W3x[:, H:2H] + U3h[:, H:2H])
//     n = tanh(W3x[:, 2H:3H] + r * U3h[:, 2H:3H])
//     h' = (1 - z) * n + z * h
// Every output element depends on the same (row, column) of its seven inputs only, so one lane computes all four
// values from registers: seven reads and one write per element (five writes when r, z, n and the candidate's U3h
// slice are kept for the backward pass) instead of ten reads and four writes over three launches. The expressions and
// the device math functions are those of the separate bodies (AM_OP_ADD_SIGMOID, AM_OP3_GRU_CANDIDATE,
// AM_OP3_GRU_BLEND), each step rounded on its own, so the bits are those of the three-pass form.
#include "common.h"

namespace am {
namespace gru {

template <typename T> struct Args {
  const T* w3x; int64_t ldw;     // [batch, 3H], rows ldw apart, unit stride within a row
  const T* u3h; int64_t ldu;
  T* hidden; int64_t ldh;        // [batch, H], read and written
  T* r; T* z; T* n; T* uh;       // [batch, H] each, rows lds apart; all null when nothing is kept
  int64_t lds;
  int64_t batch, H;
};

__device__ __forceinline__ float dev_exp(float x) { return expf(x); }
__device__ __forceinline__ double dev_exp(double x) { return exp(x); }
__device__ __forceinline__ float dev_tanh(float x) { return tanhf(x); }
__device__ __forceinline__ double dev_tanh(double x) { return tanh(x); }

template <typename T>
__device__ __forceinline__ T cell(T wr, T wz, T wn, T ur, T uz, T un, T h, T& r, T& z, T& n) {
  const T tr = wr + ur, tz = wz + uz;
  r = (T)1 / ((T)1 + dev_exp(-tr));
  z = (T)1 / ((T)1 + dev_exp(-tz));
  n = dev_tanh(wn + r * un);
  return ((T)1 - z) * n + z * h;
}

// One lane per V consecutive columns of one row (V = 16 bytes when VEC, else one element).
template <typename T, bool VEC, bool SAVE>
__global__ __launch_bounds__(256) void gru_gates(Args<T> p) {
  constexpr int V = VEC ? 16 / (int)sizeof(T) : 1;
  typedef T vec_t __attribute__((ext_vector_type(V)));
  const int64_t per_row = p.H / V, total = p.batch * per_row;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
    const int64_t b = i / per_row, j = (i - b * per_row) * V;
    const T* w = p.w3x + b * p.ldw + j;
    const T* u = p.u3h + b * p.ldu + j;
    T* h = p.hidden + b * p.ldh + j;
    const vec_t wr = *(const vec_t*)w, wz = *(const vec_t*)(w + p.H), wn = *(const vec_t*)(w + 2 * p.H);
    const vec_t ur = *(const vec_t*)u, uz = *(const vec_t*)(u + p.H), un = *(const vec_t*)(u + 2 * p.H);
    const vec_t hv = *(const vec_t*)h;
    vec_t r, z, n, out;
#pragma unroll
    for (int e = 0; e < V; ++e) {
      T re, ze, ne;
      out[e] = cell<T>(wr[e], wz[e], wn[e], ur[e], uz[e], un[e], hv[e], re, ze, ne);
      r[e] = re; z[e] = ze; n[e] = ne;
    }
    *(vec_t*)h = out;
    if constexpr (SAVE) {
      const int64_t at = b * p.lds + j;
      *(vec_t*)(p.r + at) = r;
      *(vec_t*)(p.z + at) = z;
      *(vec_t*)(p.n + at) = n;
      *(vec_t*)(p.uh + at) = un;
    }
  }
}

template <typename T>
static int gates(const char* fn, int64_t batch, int64_t H, const T* w3x, int64_t ldw, const T* u3h, int64_t ldu, T* hidden,
                 int64_t ldh, T* r, T* z, T* n, T* uh, int64_t lds) {
  if (batch < 0 || H < 0) return fail(AM_E_SHAPE, "%s: negative extent", fn);
  if (batch == 0 || H == 0) return AM_OK;
  if (!w3x || !u3h || !hidden) return fail(AM_E_ARG, "%s: null tensor pointer", fn);
  const bool save = r || z || n || uh;
  if (save && !(r && z && n && uh)) return fail(AM_E_ARG, "%s: r, z, n and Uh are kept together or not at all", fn);
  if (ldw < 3 * H || ldu < 3 * H || ldh < H || (save && lds < H)) return fail(AM_E_ARG, "%s: a row stride is shorter than its row", fn);
  AM_TRY(ensure_init());
  Args<T> p = {w3x, ldw, u3h, ldu, hidden, ldh, r, z, n, uh, lds, batch, H};
  constexpr int64_t V = 16 / (int64_t)sizeof(T);
  auto fits = [&](const void* base, int64_t ld) { return (uintptr_t)base % 16 == 0 && ld % V == 0; };
  bool vec = H % V == 0 && fits(w3x, ldw) && fits(u3h, ldu) && fits(hidden, ldh);
  if (save) vec = vec && fits(r, lds) && fits(z, lds) && fits(n, lds) && fits(uh, lds);
  const int64_t total = batch * (vec ? H / V : H);
  int64_t blocks = (total + 255) / 256;
  const int64_t cap = (int64_t)num_cus() * 16;
  if (blocks > cap) blocks = cap;
  const dim3 grid((unsigned)blocks), block(256);
  if (vec && save) hipLaunchKernelGGL((gru_gates<T, true, true>), grid, block, 0, stream(), p);
  else if (vec) hipLaunchKernelGGL((gru_gates<T, true, false>), grid, block, 0, stream(), p);
  else if (save) hipLaunchKernelGGL((gru_gates<T, false, true>), grid, block, 0, stream(), p);
  else hipLaunchKernelGGL((gru_gates<T, false, false>), grid, block, 0, stream(), p);
  return check_launch("gru_gates");
}

// The element-wise part of gru_cell_backward (nnp_gru.nim:165-186) as one pass: from the gradient of the next hidden
// state and what the forward pass kept, the gradients of the two [batch, 3H] products,
//     dz = (h - n) * dnext            dn = (1 - z) * dnext
//     dWx = dn * (1 - n * n)          dr = Uh * dWx           dUh = r * dWx
//     dWzx = z * (1 - z) * dz         dWrx = r * (1 - r) * dr
//     dW3x = [dWrx | dWzx | dWx]      dU3h = [dWrx | dWzx | dUh]
// written straight into the column slices that the reference builds with two `concat`s: six reads and six writes per
// element instead of nine launches. Same expressions and association as the separate bodies (`-.`, `*.`,
// tanh_backward, sigmoid_backward), each step rounded on its own.
template <typename T> struct BwdArgs {
  const T* dnext; const T* h; const T* r; const T* z; const T* n; const T* uh;   // [batch, H], rows ld_in apart
  int64_t ld_in;
  T* dw3x; int64_t ldw;          // [batch, 3H]
  T* du3h; int64_t ldu;
  int64_t batch, H;
};

template <typename T, bool VEC>
__global__ __launch_bounds__(256) void gru_gates_backward(BwdArgs<T> p) {
  constexpr int V = VEC ? 16 / (int)sizeof(T) : 1;
  typedef T vec_t __attribute__((ext_vector_type(V)));
  const int64_t per_row = p.H / V, total = p.batch * per_row;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
    const int64_t b = i / per_row, j = (i - b * per_row) * V;
    const int64_t at = b * p.ld_in + j;
    const vec_t dnext = *(const vec_t*)(p.dnext + at), h = *(const vec_t*)(p.h + at), r = *(const vec_t*)(p.r + at);
    const vec_t z = *(const vec_t*)(p.z + at), n = *(const vec_t*)(p.n + at), uh = *(const vec_t*)(p.uh + at);
    vec_t dwr, dwz, dwx, duh;
#pragma unroll
    for (int e = 0; e < V; ++e) {
      const T dz = (h[e] - n[e]) * dnext[e];
      const T dn = ((T)1 - z[e]) * dnext[e];
      dwx[e] = dn * ((T)1 - n[e] * n[e]);
      const T dr = uh[e] * dwx[e];
      duh[e] = r[e] * dwx[e];
      dwz[e] = z[e] * ((T)1 - z[e]) * dz;
      dwr[e] = r[e] * ((T)1 - r[e]) * dr;
    }
    T* w = p.dw3x + b * p.ldw + j;
    T* u = p.du3h + b * p.ldu + j;
    *(vec_t*)w = dwr; *(vec_t*)(w + p.H) = dwz; *(vec_t*)(w + 2 * p.H) = dwx;
    *(vec_t*)u = dwr; *(vec_t*)(u + p.H) = dwz; *(vec_t*)(u + 2 * p.H) = duh;
  }
}

template <typename T>
static int gates_backward(const char* fn, int64_t batch, int64_t H, const T* dnext, const T* h, const T* r, const T* z, const T* n,
                          const T* uh, int64_t ld_in, T* dw3x, int64_t ldw, T* du3h, int64_t ldu) {
  if (batch < 0 || H < 0) return fail(AM_E_SHAPE, "%s: negative extent", fn);
  if (batch == 0 || H == 0) return AM_OK;
  if (!dnext || !h || !r || !z || !n || !uh || !dw3x || !du3h) return fail(AM_E_ARG, "%s: null tensor pointer", fn);
  if (ld_in < H || ldw < 3 * H || ldu < 3 * H) return fail(AM_E_ARG, "%s: a row stride is shorter than its row", fn);
  AM_TRY(ensure_init());
  BwdArgs<T> p = {dnext, h, r, z, n, uh, ld_in, dw3x, ldw, du3h, ldu, batch, H};
  constexpr int64_t V = 16 / (int64_t)sizeof(T);
  auto fits = [&](const void* base, int64_t ld) { return (uintptr_t)base % 16 == 0 && ld % V == 0; };
  const bool vec = H % V == 0 && fits(dnext, ld_in) && fits(h, ld_in) && fits(r, ld_in) && fits(z, ld_in) && fits(n, ld_in) &&
                   fits(uh, ld_in) && fits(dw3x, ldw) && fits(du3h, ldu);
  const int64_t total = batch * (vec ? H / V : H);
  int64_t blocks = (total + 255) / 256;
  const int64_t cap = (int64_t)num_cus() * 16;
  if (blocks > cap) blocks = cap;
  if (vec) hipLaunchKernelGGL((gru_gates_backward<T, true>), dim3((unsigned)blocks), dim3(256), 0, stream(), p);
  else hipLaunchKernelGGL((gru_gates_backward<T, false>), dim3((unsigned)blocks), dim3(256), 0, stream(), p);
  return check_launch("gru_gates_backward");
}

}  // namespace gru
}  // namespace am

using namespace am;

extern "C" int am_hip_gru_gates_f32(int64_t batch, int64_t H, const float* w3x, int64_t ldw, const float* u3h, int64_t ldu,
                                    float* hidden, int64_t ldh, float* r, float* z, float* n, float* uh, int64_t lds) {
  return gru::gates<float>("am_hip_gru_gates_f32", batch, H, w3x, ldw, u3h, ldu, hidden, ldh, r, z, n, uh, lds);
}
extern "C" int am_hip_gru_gates_f64(int64_t batch, int64_t H, const double* w3x, int64_t ldw, const double* u3h, int64_t ldu,
                                    double* hidden, int64_t ldh, double* r, double* z, double* n, double* uh, int64_t lds) {
  return gru::gates<double>("am_hip_gru_gates_f64", batch, H, w3x, ldw, u3h, ldu, hidden, ldh, r, z, n, uh, lds);
}
extern "C" int am_hip_gru_gates_backward_f32(int64_t batch, int64_t H, const float* dnext, const float* h, const float* r,
                                             const float* z, const float* n, const float* uh, int64_t ld_in, float* dw3x,
                                             int64_t ldw, float* du3h, int64_t ldu) {
  return gru::gates_backward<float>("am_hip_gru_gates_backward_f32", batch, H, dnext, h, r, z, n, uh, ld_in, dw3x, ldw, du3h, ldu);
}
extern "C" int am_hip_gru_gates_backward_f64(int64_t batch, int64_t H, const double* dnext, const double* h, const double* r,
                                             const double* z, const double* n, const double* uh, int64_t ld_in, double* dw3x,
                                             int64_t ldw, double* du3h, int64_t ldu) {
  return gru::gates_backward<double>("am_hip_gru_gates_backward_f64", batch, H, dnext, h, r, z, n, uh, ld_in, dw3x, ldw, du3h, ldu);
}
