// Host-side pieces shared by the MFMA (f32/f64) and VALU (i32/i64) GEMM families: the kernel
// argument block, argument validation, operand classification and the tile-shape choice.
#pragma once
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <type_traits>
#include "common.h"
#include "fastdiv.h"

namespace am {
namespace gemm {

// How the loader may fetch an operand tile X(mn, k) = X[mn * ld_mn + k * ld_k].
enum LoadKind : int {
  kKContig = 0,   // ld_k == 1: 16-byte vectors along k
  kMNContig = 1,  // ld_mn == 1: 16-byte vectors along m (A) or n (B)
  kGeneric = 2,   // any strides (zero, negative, non-unit): scalar gathers
  kGather = 3,    // B only: the column matrix of a convolution, read straight from the image (ConvGeom)
  kGatherVec = 4, // kGather in 16-byte pieces: unit stride along the image's and the window's width, whole vectors per output row
  kGatherVecT = 5 // B only: the TRANSPOSED column matrices of a batch side by side, B(n, k) with n = (c, kh, kw) and
                  // k = image * P + output pixel, in 16-byte pieces along k (the weight gradient's operand); k-group LDS layout
};
// Kinds whose slab sits in LDS as k-groups (16-byte slots of VK consecutive k per row / column).
constexpr bool k_grouped(int kind) { return kind == kKContig || kind == kGatherVecT; }

// Geometry of a convolution whose column matrix col(k, j) = image[c, oh * sh - ph + kh, ow * sw - pw + kw]
// (k = (c * kH + kh) * kW + kw, j = oh * Wo + ow; zero where the window leaves the image) is the B operand of
// a GEMM without ever being written to memory (fallback/conv.nim:18-54 writes it, one image at a time).
// k is decoded with two multiply-high divisions by kH * kW and kW (multipliers from the host, exact while
// K * kH * kW < 2^32).
struct ConvGeom {
  int H, W, kH, kW, Wo, ph, pw, sh, sw;
  uint32_t magic_khw, magic_kw;   // ceil(2^32 / (kH * kW)), ceil(2^32 / kW); 0 where the divisor is 1
  // Strides of the image in BYTES, and the distance in bytes from the lowest address any of its elements has to
  // its element (0, 0, 0): every element's offset from that lowest address is then a non-negative 32-bit number
  // (the host refuses images that span 4 GiB or more), which is what a load with a scalar base and a 32-bit
  // vector offset takes. The image pointer is the GEMM's B.
  int in_c, in_h, in_w;
  uint32_t origin;
  // kGatherVecT only: output pixels per image, the distance between images in bytes, dividers by P and by Wo
  int P;
  int64_t in_n;
  FastDiv by_p, by_wo;
};

template <typename T> struct Args {
  int64_t M, N, K;
  T alpha, beta;
  const T* A; int64_t a_mn, a_k;   // strides of A along m and along k (elements)
  const T* B; int64_t b_mn, b_k;   // strides of B along n and along k
  T* C; int64_t c_m, c_n;
  int epilogue;
  const T* bias; int64_t bias_m, bias_n;
  int tiles_m, tiles_n;
  int a_kfast, b_kfast;            // generic loader: 1 = walk k fastest across lanes
  // Split-K: workgroup (tile, split) multiplies the k range [split * k_chunk, (split + 1) * k_chunk)
  // and stores its raw partial tile to ws[split][M][N]; splitk_reduce adds the partials in a fixed
  // order and applies alpha / beta / epilogue. splits == 1: the kernel writes C itself.
  int splits;
  int64_t k_chunk;
  T* ws;
  int want_splits;                 // > 0: the split factor the tile chooser decided on (plan_splitk then takes it as is)
  // Strided batch: workgroups with blockIdx.y = z work on A + z * batch_a, B + z * batch_b,
  // C + z * batch_c (elements); the bias is shared by the whole batch.
  int batch;
  int64_t batch_a, batch_b, batch_c;
  bool swapped;                    // prepare() exchanged the roles of A and B (column-major C)
  // Integer products launched behind the digit-sliced path as its alternative: when gate_flags is
  // set, the vector-ALU kernels leave at once if the operands have at most gate_max_pairs non-empty
  // digit pairs (the digit-sliced kernel, launched just before with the same limit, has then
  // written C); otherwise the digit-sliced kernel has left and they do the work.
  const uint32_t* gate_flags;
  uint32_t gate_gen;
  int gate_max_pairs;
  // Allocation-free entry point: split-K partials go to the library's static device array instead
  // of the hipMalloc'ed workspace; a plan that needs more than the array holds is recorded in
  // static_ws_short (bytes it would have needed) and the call is refused.
  bool static_ws;
  size_t static_ws_short;
  long long* clock_out;            // where the matrix-core kernels add their cycle counts while a clock window is open
  long long* phase_out;            // the small-product kernels' phase marks while a phase window is open (PhaseProbe)
  int phase_cap;
  ConvGeom conv;                   // read by the kGather loader only
};

// Digit pairs (i, j), i + j < ND, whose planes are both marked non-empty: flags[i] == gen for A's
// plane i, flags[ND + j] == gen for B's plane j. Uniform over the workgroup.
template <int ND>
__device__ __forceinline__ int live_digit_pairs(const uint32_t* flags, uint32_t gen) {
  int n = 0, live_b = 0;
#pragma unroll
  for (int i = ND - 1; i >= 0; --i) {          // live_b counts B's live planes j <= ND - 1 - i
    live_b += flags[ND + (ND - 1 - i)] == gen ? 1 : 0;
    n += flags[i] == gen ? live_b : 0;
  }
  return n;
}

static inline bool aligned16(const void* p) { return ((uintptr_t)p & 15u) == 0; }

// An operand with a unit stride is moved in 16-byte vectors whatever its row pitch, extent or base address
// (the loaders take care of vectors that straddle an edge); a row shorter than one vector, a negative pitch
// along the vectors' direction... everything else is gathered element by element.
template <typename T>
static inline int classify(const T* X, int64_t ld_mn, int64_t ld_k, int64_t MN, int64_t K) {
  constexpr int64_t VK = 16 / (int64_t)sizeof(T);
  (void)X;
  if (ld_k == 1 && K >= VK && ld_mn >= 0) return kKContig;
  if (ld_mn == 1 && MN >= VK && (MN % VK == 0 ? ld_k >= 0 : ld_k >= MN)) return kMNContig;   // ragged rows must not overlap
  return kGeneric;
}

static inline int64_t iabs64(int64_t v) { return v < 0 ? -v : v; }

// Validates the caller's arguments and normalises them into `out`. Returns 1 (positive) when
// there is nothing to do (an empty extent: the reference's loops never run and C stays as is).
template <typename T>
static int prepare(const char* fn, int64_t M, int64_t N, int64_t K, T alpha, const T* A, int64_t rsA,
                   int64_t csA, const T* B, int64_t rsB, int64_t csB, T beta, T* C, int64_t rsC,
                   int64_t csC, int epilogue, const T* bias, int64_t bias_rs, int64_t bias_cs,
                   Args<T>* out) {
  if (M < 0 || N < 0 || K < 0) return fail(AM_E_ARG, "%s: negative dimension (M=%lld N=%lld K=%lld)", fn, (long long)M, (long long)N, (long long)K);
  if (M == 0 || N == 0 || K == 0) return 1;
  if (!A || !B || !C) return fail(AM_E_ARG, "%s: null matrix pointer", fn);
  if (epilogue < AM_EPI_NONE || epilogue > AM_EPI_BIAS_RELU) return fail(AM_E_ARG, "%s: unknown epilogue %d", fn, epilogue);
  if ((epilogue & AM_EPI_BIAS) && !bias) return fail(AM_E_ARG, "%s: bias epilogue without a bias pointer", fn);
  if ((M > 1 && rsC == 0) || (N > 1 && csC == 0))
    return fail(AM_E_SHAPE, "%s: C has a zero stride on a dimension of extent > 1", fn);
  if (M > 1 && N > 1 && iabs64(rsC) == iabs64(csC))
    return fail(AM_E_SHAPE, "%s: C's row and column strides coincide (%lld): elements overlap", fn, (long long)rsC);
  if (M >= ((int64_t)1 << 31) || N >= ((int64_t)1 << 31) || K >= ((int64_t)1 << 31))
    return fail(AM_E_SHAPE, "%s: dimensions of 2^31 or more are not supported", fn);

  Args<T>& g = *out;
  // Writes along n should be the unit-stride direction: for a column-major C compute
  // C^T = B^T * A^T instead (same kernel, operands swapped, no data movement).
  const bool swap = (iabs64(csC) != 1 && iabs64(rsC) == 1);
  if (!swap) {
    g.M = M; g.N = N;
    g.A = A; g.a_mn = rsA; g.a_k = csA;
    g.B = B; g.b_mn = csB; g.b_k = rsB;
    g.c_m = rsC; g.c_n = csC;
    g.bias_m = bias_rs; g.bias_n = bias_cs;
  } else {
    g.M = N; g.N = M;
    g.A = B; g.a_mn = csB; g.a_k = rsB;
    g.B = A; g.b_mn = rsA; g.b_k = csA;
    g.c_m = csC; g.c_n = rsC;
    g.bias_m = bias_cs; g.bias_n = bias_rs;
  }
  g.K = K; g.alpha = alpha; g.beta = beta; g.C = C;
  g.epilogue = epilogue; g.bias = bias;
  g.batch = 1; g.batch_a = g.batch_b = g.batch_c = 0;
  g.gate_flags = nullptr; g.gate_gen = 0; g.gate_max_pairs = 0;
  g.static_ws = false; g.static_ws_short = 0;
  g.want_splits = 0;
  g.clock_out = clock_probe_buffer();
  g.phase_out = phase_probe_buffer(&g.phase_cap);
  g.swapped = swap;
  g.a_kfast = iabs64(g.a_k) <= iabs64(g.a_mn);
  g.b_kfast = iabs64(g.b_k) < iabs64(g.b_mn);
  return AM_OK;
}

// AM_HIP_GEMM_TRACE=1 in the environment: every GEMM call prints the tile / split it chose to stderr.
static inline bool trace_choices() {
  static const bool on = [] { const char* e = getenv("AM_HIP_GEMM_TRACE"); return e && *e && *e != '0'; }();
  return on;
}

// One candidate tile shape and the relative speed of a CU that runs it; bk / waves (slab width, wavefronts per
// workgroup; 0 = 16 / 4) are what the split-K estimate of choose_tile_and_split needs.
struct TileChoice { int bm, bn; double eff; int bk, waves; };

// Picks the candidate with the least estimated time: rounds of one block per CU, each round
// costing bm*bn/eff. Ragged edges and under-filled rounds are priced by construction.
static inline int choose_tile(const TileChoice* cand, int ncand, int64_t M, int64_t N, const char* env, int64_t batch = 1,
                              double* cost_out = nullptr) {
  const char* forced = getenv(env);
  if (forced && *forced && !cost_out) {
    int idx = atoi(forced);
    if (idx >= 0 && idx < ncand) return idx;
  }
  const int64_t cus = num_cus();
  int best = 0;
  double best_cost = 0;
  for (int i = 0; i < ncand; ++i) {
    if (cand[i].eff <= 0) continue;   // experimental shape: only when forced
    const int64_t tiles = ((M + cand[i].bm - 1) / cand[i].bm) * ((N + cand[i].bn - 1) / cand[i].bn) * batch;
    const int64_t rounds = (tiles + cus - 1) / cus;
    const double cost = (double)rounds * cand[i].bm * cand[i].bn / cand[i].eff;
    if (i == 0 || cost < best_cost) { best = i; best_cost = cost; }
  }
  if (cost_out) *cost_out = best_cost;
  return best;
}

// Fills the GEMM view of a convolution (fallback/conv.nim:81-106: out[n] = kernel_col * col[n] + bias) whose column
// matrix is gathered by the kGather loader: M = C_out, N = H_out * W_out, K = C * kH * kW, one batch member per image.
// Returns 1 when there is nothing to do, a negative code on bad arguments.
template <typename T>
static int prepare_conv(const char* fn, int64_t N, int C, int H, int W, int Cout, int kH, int kW, int padH, int padW, int strideH,
                        int strideW, const T* in, int64_t in_n, int64_t in_c, int64_t in_h, int64_t in_w, const T* kernel,
                        int64_t kernel_rs, int epilogue, const T* bias, int64_t bias_s, T* out, Args<T>* g_out) {
  if (N < 0 || C < 0 || H < 0 || W < 0 || Cout < 0 || kH <= 0 || kW <= 0 || padH < 0 || padW < 0 || strideH <= 0 || strideW <= 0)
    return fail(AM_E_ARG, "%s: bad geometry", fn);
  if (N > 65535) return fail(AM_E_SHAPE, "%s: more than 65535 images in one call", fn);
  const int64_t Ho = ((int64_t)H + 2 * padH - kH) / strideH + 1, Wo = ((int64_t)W + 2 * padW - kW) / strideW + 1;
  if ((int64_t)H + 2 * padH < kH || (int64_t)W + 2 * padW < kW) return fail(AM_E_SHAPE, "%s: kernel larger than the padded image", fn);
  if (N == 0 || C == 0 || Cout == 0 || Ho <= 0 || Wo <= 0) return 1;
  const int64_t K = (int64_t)C * kH * kW, P = Ho * Wo;
  if (K < 16 / (int64_t)sizeof(T) || K * kH * kW >= ((int64_t)1 << 32) || P >= ((int64_t)1 << 31))
    return fail(AM_E_SHAPE, "%s: C * kH * kW = %lld outside what the fused kernel takes (use im2col + gemm_batched)", fn, (long long)K);
  if (!in || !kernel || !out) return fail(AM_E_ARG, "%s: null tensor pointer", fn);
  const int rc = prepare<T>(fn, Cout, P, K, (T)1, kernel, kernel_rs, 1, in, 0, 1, (T)0, out, P, 1, epilogue, bias, bias_s, 0, g_out);
  if (rc != AM_OK) return rc;
  Args<T>& g = *g_out;
  g.batch = (int)N; g.batch_a = 0; g.batch_b = in_n; g.batch_c = (int64_t)Cout * P;
  ConvGeom& cg = g.conv;
  cg.H = H; cg.W = W; cg.kH = kH; cg.kW = kW; cg.Wo = (int)Wo; cg.ph = padH; cg.pw = padW; cg.sh = strideH; cg.sw = strideW;
  {
    const int64_t sz = (int64_t)sizeof(T);
    const int64_t ext[3] = {C, H, W}, str[3] = {in_c, in_h, in_w};
    int64_t lowest = 0, highest = 0;     // element offsets of the image's lowest and highest address
    for (int d = 0; d < 3; ++d) {
      if (str[d] < 0) lowest += str[d] * (ext[d] - 1); else highest += str[d] * (ext[d] - 1);
    }
    if ((highest - lowest + 1) * sz >= ((int64_t)1 << 32))
      return fail(AM_E_SHAPE, "%s: one image spans 4 GiB or more (use im2col + gemm_batched)", fn);
    cg.in_c = (int)(in_c * sz); cg.in_h = (int)(in_h * sz); cg.in_w = (int)(in_w * sz);
    cg.origin = (uint32_t)(-lowest * sz);
  }
  auto magic = [](int d) { return d == 1 ? 0u : (uint32_t)((((uint64_t)1 << 32) + (uint64_t)d - 1) / (uint64_t)d); };
  cg.magic_khw = magic(kH * kW); cg.magic_kw = magic(kW);
  return AM_OK;
}

// Fills the GEMM view of a convolution's weight gradient (fallback/conv.nim:135-143 adds grad_output_col * input_col^T image
// by image): M = C_out, N = C * kH * kW, K = images * P with the images' column matrices side by side, gathered by the
// kGatherVecT loader. gout is grad_output as [C_out][images * P] with unit stride along its rows. Returns 1 when there is
// nothing to do (no images or no outputs: the result is left as it is), a negative code on bad arguments, AM_E_SHAPE for geometries the gathered form does not take.
template <typename T>
static int prepare_conv_grad_weight(const char* fn, int64_t N, int C, int H, int W, int Cout, int kH, int kW, int padH, int padW,
                                    int strideH, int strideW, const T* in, int64_t in_n, int64_t in_c, int64_t in_h, int64_t in_w,
                                    const T* gout, int64_t gout_rs, T* out, Args<T>* g_out) {
  constexpr int VK = 16 / (int)sizeof(T);
  if (N < 0 || C < 0 || H < 0 || W < 0 || Cout < 0 || kH <= 0 || kW <= 0 || padH < 0 || padW < 0 || strideH <= 0 || strideW <= 0)
    return fail(AM_E_ARG, "%s: bad geometry", fn);
  const int64_t Ho = ((int64_t)H + 2 * padH - kH) / strideH + 1, Wo = ((int64_t)W + 2 * padW - kW) / strideW + 1;
  if ((int64_t)H + 2 * padH < kH || (int64_t)W + 2 * padW < kW) return fail(AM_E_SHAPE, "%s: kernel larger than the padded image", fn);
  if (C == 0 || Cout == 0) return 1;
  const int64_t CKK = (int64_t)C * kH * kW, P = Ho * Wo, K = N * P;
  if (strideW != 1 || in_w != 1 || Wo % VK != 0 || W < VK)
    return fail(AM_E_SHAPE, "%s: needs unit stride along the width (image and window) and output rows of whole 16-byte vectors "
                "(use im2col_strided + gemm)", fn);
  if (CKK * kH * kW >= ((int64_t)1 << 32) || K >= ((int64_t)1 << 31))
    return fail(AM_E_SHAPE, "%s: C * kH * kW = %lld or images * outputs = %lld outside what the fused kernel takes (use im2col_strided + gemm)",
                fn, (long long)CKK, (long long)K);
  if (N == 0 || P <= 0) return 1;     // no column at all: the sum over none is the caller's zero
  if (!out || !in || !gout) return fail(AM_E_ARG, "%s: null tensor pointer", fn);
  const int rc = prepare<T>(fn, Cout, CKK, K, (T)1, gout, gout_rs, 1, in, 0, 1, (T)0, out, CKK, 1, 0, (const T*)nullptr, 0, 0, g_out);
  if (rc != AM_OK) return rc;
  Args<T>& g = *g_out;
  ConvGeom& cg = g.conv;
  cg.H = H; cg.W = W; cg.kH = kH; cg.kW = kW; cg.Wo = (int)Wo; cg.ph = padH; cg.pw = padW; cg.sh = strideH; cg.sw = strideW;
  {
    const int64_t sz = (int64_t)sizeof(T);
    const int64_t ext[3] = {C, H, W}, str[3] = {in_c, in_h, in_w};
    int64_t lowest = 0, highest = 0;
    for (int d = 0; d < 3; ++d) {
      if (str[d] < 0) lowest += str[d] * (ext[d] - 1); else highest += str[d] * (ext[d] - 1);
    }
    if ((highest - lowest + 1) * sz >= ((int64_t)1 << 32))
      return fail(AM_E_SHAPE, "%s: one image spans 4 GiB or more (use im2col_strided + gemm)", fn);
    cg.in_c = (int)(in_c * sz); cg.in_h = (int)(in_h * sz); cg.in_w = (int)(in_w * sz);
    cg.origin = (uint32_t)(-lowest * sz);
    cg.in_n = in_n * sz;
  }
  auto magic = [](int d) { return d == 1 ? 0u : (uint32_t)((((uint64_t)1 << 32) + (uint64_t)d - 1) / (uint64_t)d); };
  cg.magic_khw = magic(kH * kW); cg.magic_kw = magic(kW);
  cg.P = (int)P;
  cg.by_p = FastDiv((uint32_t)P); cg.by_wo = FastDiv((uint32_t)Wo);
  return AM_OK;
}

// The sub-problem C[r0:r1, c0:c1] of g (rows of A, columns of B, the block of C and of the bias).
template <typename T>
static inline Args<T> sub_problem(const Args<T>& g, int64_t r0, int64_t r1, int64_t c0, int64_t c1) {
  Args<T> s = g;
  s.M = r1 - r0; s.N = c1 - c0;
  s.A = g.A + r0 * g.a_mn;
  s.B = g.B + c0 * g.b_mn;
  s.C = g.C + r0 * g.c_m + c0 * g.c_n;
  if (g.bias) s.bias = g.bias + r0 * g.bias_m + c0 * g.bias_n;
  return s;
}

// A matrix whose extent is a few rows or columns more than a multiple of the tile edge costs a whole extra
// round of tiles for those few (4097^2 outputs: 289 tiles of 256 x 256 on 256 CUs, two rounds for what is
// 1.0005 rounds of work). Such a product is cut into the aligned block, run by the tiled kernel, and strips of
// at most 16 rows / columns, run as the skinny products they are (they stream the other operand once).
// Returns the number of rows (*rm) and columns (*rn) to cut off, both 0 when the product is better left whole:
// the estimate compares rounds x tile area (choose_tile's cost) with and without the cut, and prices a strip
// by the bytes it streams.
template <typename T>
static inline void plan_peel(const Args<T>& g, const TileChoice* cand, int ncand, const char* env, double flops_per_cu_us,
                             int64_t* rm, int64_t* rn) {
  *rm = *rn = 0;
  if (g.batch > 1 || g.static_ws) return;   // (the allocation-free entry point refuses a product as a whole or not at all)
  const char* e = getenv("AM_HIP_GEMM_PEEL");   // "0": never cut; "1": cut whenever the shape allows it (tests)
  if (e && *e == '0') return;
  const int64_t pm = g.M % 64, pn = g.N % 64;
  const bool cm = pm > 0 && pm <= 16 && g.M >= 512, cn = pn > 0 && pn <= 16 && g.N >= 512;
  if (!cm && !cn) return;
  double whole = 0, cut = 0;
  (void)choose_tile(cand, ncand, g.M, g.N, env, 1, &whole);
  const int64_t M0 = cm ? g.M - pm : g.M, N0 = cn ? g.N - pn : g.N;
  (void)choose_tile(cand, ncand, M0, N0, env, 1, &cut);
  const double us_per_cost = 2.0 * (double)g.K / flops_per_cu_us;          // time of one output element's K loop on one CU
  // a strip: one launch, and the other operand streamed once at ~3 TB/s
  const double strips = (cm ? 6.0 + (double)g.K * (double)g.N * sizeof(T) / 3.0e6 : 0.0) +
                        (cn ? 6.0 + (double)g.K * (double)M0 * sizeof(T) / 3.0e6 : 0.0);
  if ((e && *e == '1') || cut * us_per_cost + strips < 0.92 * whole * us_per_cost) { *rm = cm ? pm : 0; *rn = cn ? pn : 0; }
}

// Persistent device workspace for split-K partial sums (runtime.hip): allocated once, on first use
// outside graph capture; nullptr when `bytes` exceeds its capacity or it cannot be allocated now.
void* splitk_workspace(size_t bytes);
// The static device array behind the allocation-free entry point (runtime.hip): its device address
// (looked up once when the library initialised the device) and its size. Never allocates.
void* static_scratch(size_t* capacity);

// Decides the split-K factor for a problem that would otherwise leave most SIMDs idle: small M x N
// (few tiles) with a long K runs as one serial MFMA / MAC chain per wave, so K is cut into
// `splits` ranges handled by different workgroups. bk = slab width, waves = wavefronts per tile.
// The split factors worth considering for `tiles` workgroup tiles of `waves` wavefronts and `slabs` slabs of k:
// *base = one wavefront per SIMD over the chip, at least two slabs per split, at most 32 (1 when the tiles already
// fill half the chip or k is short); *deep = up to four wavefronts per SIMD while every split keeps eight slabs, at most
// 128: worth it for a very long k on tiles large enough that the matrix cores, not the round trips of a slab, set
// a split's time (0 when it offers nothing beyond *base).
static inline void splitk_factors(int64_t tiles, int waves, int64_t slabs, int64_t* base, int64_t* deep) {
  *base = 1; *deep = 0;
  const int64_t simds = (int64_t)num_cus() * 4;
  if (tiles * waves * 2 > simds || slabs < 4) return;
  int64_t want = simds / (tiles * waves);
  if (want > slabs / 2) want = slabs / 2;
  if (want > 32) want = 32;
  if (want >= 2) *base = want;
  int64_t d = 4 * simds / (tiles * waves);
  if (d > slabs / 8) d = slabs / 8;
  if (d > 128) d = 128;
  if (d > *base) *deep = d;
}

template <typename T>
static inline void plan_splitk(Args<T>& g, int bk, int waves_per_tile) {
  g.splits = 1; g.k_chunk = g.K; g.ws = nullptr;
  if (g.batch > 1) return;   // a batch already supplies the parallelism
  const int64_t tiles = (int64_t)g.tiles_m * g.tiles_n;
  const int64_t slabs = (g.K + bk - 1) / bk;
  int64_t splits, deep;
  splitk_factors(tiles, waves_per_tile, slabs, &splits, &deep);
  if (g.want_splits > 0) splits = g.want_splits;
  if (splits > slabs) splits = slabs;
  if (splits < 2) return;
  const int64_t chunk_slabs = (slabs + splits - 1) / splits;
  splits = (slabs + chunk_slabs - 1) / chunk_slabs;           // no empty split
  if (splits < 2) return;
  const size_t bytes = (size_t)splits * (size_t)g.M * (size_t)g.N * sizeof(T);
  T* ws;
  if (g.static_ws) {
    size_t cap = 0;
    ws = (T*)static_scratch(&cap);
    if (!ws || bytes > cap) { g.static_ws_short = bytes; return; }
  } else {
    ws = (T*)splitk_workspace(bytes);
  }
  if (!ws) return;
  g.splits = (int)splits; g.k_chunk = chunk_slabs * bk; g.ws = ws;
}

// Tile AND split factor of a float product together. Where the tiles alone fill the chip this is choose_tile (rounds of
// one workgroup per CU x tile area / efficiency). Where they do not, choose_tile's answer is the smallest tile (most
// workgroups), whose matrix instructions wait on LDS and whose operands cross L2 most often, although a split of k can
// supply the workgroups instead: [500 x 65536] * [65536 x 800] as 32 x 32 tiles 630 us, as 128 x 128 tiles x 9 splits
// 440 us. So every candidate is priced with its own split factor (both kinds, see splitk_factors):
//   rounds x slabs per split x time of a slab  +  the second pass (launch, and the partials read eight at a time by
//   however many lanes the result offers)  +  a workgroup's fixed cost.
// flops_per_cu_us: what one CU sustains (peak / CUs). Sets g.want_splits.
template <typename T>
static inline int choose_tile_and_split(Args<T>& g, const TileChoice* cand, int ncand, const char* env, double flops_per_cu_us) {
  g.want_splits = 0;
  const int by_rounds = choose_tile(cand, ncand, g.M, g.N, env, g.batch);
  const char* forced = getenv(env);
  if ((forced && *forced) || g.batch > 1) return by_rounds;
  // what the partial tiles of a plan may take: the workspace's share, or the whole static array of the allocation-free
  // entry point (which therefore runs the same plan as the allocating one wherever that plan fits its array)
  double partials_limit = 48.0 * 1024 * 1024;
  if (g.static_ws) { size_t cap = 0; (void)static_scratch(&cap); partials_limit = (double)cap; }
  static const bool joint = [] { const char* e = getenv("AM_HIP_GEMM_JOINT"); return !(e && *e == '0'); }();
  if (!joint) return by_rounds;
  const int64_t cus = num_cus();
  // choose_tile's answer priced the same way is the bar; the other tiles enter with their split factors only (without
  // a split they have lost against it already), and one of them has to beat the bar by a tenth.
  auto price = [&](int i, int64_t sp_in, int64_t* sp_out) {
    const TileChoice& c = cand[i];
    const int bk = c.bk ? c.bk : 16;
    const int64_t tiles = ((g.M + c.bm - 1) / c.bm) * ((g.N + c.bn - 1) / c.bn);
    const int64_t slabs = (g.K + bk - 1) / bk;
    const int64_t chunk = (slabs + sp_in - 1) / sp_in;
    const int64_t sp = (slabs + chunk - 1) / chunk;
    *sp_out = sp;
    if (sp > 1 && (double)sp * g.M * g.N * sizeof(T) > partials_limit) return -1.0;
    // a slab's time: the matrix instructions; a workgroup alone on its CU cannot go below what its chain of LDS and
    // barrier waits allows (measured on the 32 x 32 tile: 0.23 us per slab of 32 k)
    double slab_us = 2.0 * c.bm * c.bn * bk / (flops_per_cu_us * c.eff);
    if ((sp > 1 || tiles < cus) && slab_us < 0.22) slab_us = 0.22;
    const int64_t rounds = (tiles * sp + cus - 1) / cus;
    double us = 4.0 + (double)rounds * (double)chunk * slab_us;
    if (sp > 1) {
      const double lanes = (double)g.M * (double)g.N / (16.0 / sizeof(T));
      const double passes = (double)((sp + (sp >= 32 ? 31 : 7)) / (sp >= 32 ? 32 : 8));   // 8 partials in flight per lane, x 4 wavefronts
      const double latency = passes * 1.0, bandwidth = (double)(sp + 1) * g.M * g.N * sizeof(T) / 4.0e6;
      us += 5.0 + (lanes >= (double)cus * 1024 ? bandwidth : (latency > bandwidth ? latency : bandwidth));
    }
    return us;
  };
  int best = by_rounds;
  int64_t best_splits = 0;
  double best_us = -1, bar_us = -1;
  for (int i = 0; i < ncand; ++i) {
    const TileChoice& c = cand[i];
    if (c.eff <= 0) continue;
    const int bk = c.bk ? c.bk : 16, waves = c.waves ? c.waves : 4;
    const int64_t tiles = ((g.M + c.bm - 1) / c.bm) * ((g.N + c.bn - 1) / c.bn);
    // choose_tile's tile also without any split: a second launch for a product of a few microseconds costs more than
    // the idle SIMDs it fills (256^3: 8.4 us as 4 ranges of k + second pass, 5.5 us whole)
    int64_t opt[3] = {0, 0, i == by_rounds ? 1 : 0};
    splitk_factors(tiles, waves, (g.K + bk - 1) / bk, &opt[0], &opt[1]);
    for (int o = 0; o < 3; ++o) {
      if (opt[o] < 1 || (opt[o] < 2 && i != by_rounds)) continue;
      int64_t sp;
      const double us = price(i, opt[o], &sp);
      if (us < 0) continue;
      if (i == by_rounds && (bar_us < 0 || us < bar_us)) bar_us = us;
      if (best_us < 0 || us < best_us) { best_us = us; best = i; best_splits = sp; }
    }
  }
  if (best != by_rounds && bar_us >= 0 && best_us > 0.85 * bar_us) {   // not convincingly better: choose_tile's tile, at its own best split
    best = by_rounds; best_us = -1;
    const TileChoice& c = cand[best];
    const int bk = c.bk ? c.bk : 16, waves = c.waves ? c.waves : 4;
    int64_t opt[3] = {0, 0, 1};
    splitk_factors(((g.M + c.bm - 1) / c.bm) * ((g.N + c.bn - 1) / c.bn), waves, (g.K + bk - 1) / bk, &opt[0], &opt[1]);
    for (int o = 0; o < 3; ++o) {
      if (opt[o] < 1) continue;
      int64_t sp;
      const double us = price(best, opt[o], &sp);
      if (us >= 0 && (best_us < 0 || us < best_us)) { best_us = us; best_splits = sp; }
    }
  }
  g.want_splits = (int)best_splits;
  if (trace_choices())
    fprintf(stderr, "am_hip gemm: M=%lld N=%lld K=%lld tile %dx%d with %lld splits of k, est %.1f us (by rounds alone: %dx%d)\n", (long long)g.M,
            (long long)g.N, (long long)g.K, cand[best].bm, cand[best].bn, (long long)best_splits, best_us, cand[by_rounds].bm, cand[by_rounds].bn);
  return best;
}

// Cuts K into `want` ranges (fewer if K has too few slabs or the workspace is too small / cannot
// be allocated now). want <= 1 leaves the problem whole.
template <typename T>
static inline void apply_splitk(Args<T>& g, int bk, int64_t want) {
  g.splits = 1; g.k_chunk = g.K; g.ws = nullptr;
  if (want <= 1 || g.batch > 1) return;
  const int64_t slabs = (g.K + bk - 1) / bk;
  if (want > slabs) want = slabs;
  const int64_t chunk_slabs = (slabs + want - 1) / want;
  const int64_t splits = (slabs + chunk_slabs - 1) / chunk_slabs;   // no empty split
  if (splits < 2) return;
  const size_t bytes = (size_t)splits * (size_t)g.M * (size_t)g.N * sizeof(T);
  T* ws = (T*)splitk_workspace(bytes);
  if (!ws) return;
  g.splits = (int)splits; g.k_chunk = chunk_slabs * bk; g.ws = ws;
}

// Joint choice of workgroup tile and split-K factor for the exact (ring arithmetic) integer
// products, where cutting K changes no bit of the result. Estimated time of a candidate =
// rounds of two workgroups per CU x time of one workgroup, plus the second pass that adds the
// partial sums (its launch and its HBM traffic). mac_per_us: multiply-adds one CU sustains.
struct TileSplit { int tile; int splits; double est_us; };
template <typename T>
static inline TileSplit choose_tile_split(const TileChoice* cand, int ncand, int64_t M, int64_t N, int64_t K, int bk,
                                          double mac_per_us, const char* env, int64_t batch) {
  TileSplit best = {0, 1, 0.0};
  int forced_tile = -1;
  const char* forced = getenv(env);
  if (forced && *forced) { const int idx = atoi(forced); if (idx >= 0 && idx < ncand) forced_tile = idx; }
  int forced_splits = 0;
  const char* fs = getenv("AM_HIP_GEMM_SPLITK");
  if (fs && *fs) forced_splits = atoi(fs);
  const int64_t cus = num_cus();
  const int64_t slabs = (K + bk - 1) / bk;
  double best_cost = -1;
  for (int i = 0; i < ncand; ++i) {
    if (cand[i].eff <= 0 || (forced_tile >= 0 && i != forced_tile)) continue;
    const int64_t tiles = ((M + cand[i].bm - 1) / cand[i].bm) * ((N + cand[i].bn - 1) / cand[i].bn) * batch;
    const double slab_us = (double)cand[i].bm * cand[i].bn * bk / (mac_per_us * cand[i].eff);
    for (int64_t want = 1; want <= 16; ++want) {
      if (forced_splits > 0 && want != forced_splits) continue;
      if (want > 1 && (batch > 1 || want > slabs / 2)) break;
      const int64_t chunk = (slabs + want - 1) / want;
      const int64_t sp = (slabs + chunk - 1) / chunk;
      if (sp != want) continue;
      if (sp > 1 && (double)sp * M * N * sizeof(T) > 64.0 * 1024 * 1024) break;
      // Two workgroups fit on a CU and share it at full speed; a workgroup alone on its CU runs
      // at about two thirds of the CU's rate (one wavefront per SIMD: latencies are exposed).
      const int64_t wgs = tiles * sp, slots = 2 * cus;
      const int64_t full = wgs / slots, rem = wgs - full * slots;
      const double wg_us = (double)chunk * slab_us;
      double cost = (double)full * 2.0 * wg_us + (rem == 0 ? 0.0 : rem <= cus ? wg_us / 0.66 : 2.0 * wg_us);
      if (sp > 1) cost += 3.0 + (2.0 * sp + 1.0) * (double)M * N * sizeof(T) / 4.0e6;   // second pass at ~4 TB/s
      if (best_cost < 0 || cost < best_cost) { best_cost = cost; best.tile = i; best.splits = (int)sp; }
    }
  }
  if (trace_choices()) fprintf(stderr, "am_hip gemm: M=%lld N=%lld K=%lld tile %d (%dx%d) splits %d est %.1f us\n", (long long)M, (long long)N, (long long)K, best.tile, cand[best.tile].bm, cand[best.tile].bn, best.splits, best_cost);
  best.est_us = best_cost;
  return best;
}

// Second pass of split-K: C <- epilogue(alpha * sum_s ws[s] + beta * C), partials added in
// ascending s (deterministic). ACC is the type the partials were stored in. One thread per group
// of VEC consecutive columns of one row (blockIdx.y walks the rows): VEC = 16 bytes / element when
// N is a multiple of it (the partials are then read as 16-byte vectors), else 1.
// SY = 4 (many partials, few outputs: the pass is then a chain of memory round trips per lane, not bandwidth): the four
// wavefronts of a workgroup share 64 column groups and take the partials s = w, w + 4, w + 8, ... each; their four sums
// are added through LDS in the order ((w0 + w1) + w2) + w3 and the first wavefront writes. Needs splits >= 4.
template <typename T, typename ACC, int VEC, int SY = 1>
__global__ __launch_bounds__(256) void splitk_reduce(Args<T> p) {
  typedef ACC vec_t __attribute__((ext_vector_type(VEC)));
  if (std::is_integral<T>::value && p.gate_flags != nullptr && live_digit_pairs<(int)sizeof(T)>(p.gate_flags, p.gate_gen) <= p.gate_max_pairs) return;
  const int64_t total = p.M * p.N;
  const ACC* ws = (const ACC*)p.ws;
  __shared__ ACC cls[SY > 1 ? SY - 1 : 1][SY > 1 ? 64 * VEC : 1];
  const int cl = SY > 1 ? (int)(threadIdx.x >> 6) : 0;
  const int64_t col = SY > 1 ? ((int64_t)blockIdx.x * 64 + (threadIdx.x & 63)) * VEC : ((int64_t)blockIdx.x * 256 + threadIdx.x) * VEC;
  if (SY == 1 && col >= p.N) return;
  const bool in_range = col < p.N;
  for (int64_t row = blockIdx.y; row < p.M; row += gridDim.y) {
    const int64_t idx = row * p.N + (in_range ? col : 0);
    ACC sum[VEC];
    {
      const vec_t v = *(const vec_t*)(ws + (int64_t)cl * total + idx);
#pragma unroll
      for (int e = 0; e < VEC; ++e) sum[e] = v[e];
    }
    // eight partials in flight at a time (the loads are independent; the additions stay in
    // ascending s): with one load per trip the pass is a chain of memory round trips
    int sidx = cl + SY;
    for (; sidx + 7 * SY < p.splits; sidx += 8 * SY) {
      vec_t v[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) v[u] = *(const vec_t*)(ws + (int64_t)(sidx + u * SY) * total + idx);
#pragma unroll
      for (int u = 0; u < 8; ++u)
#pragma unroll
        for (int e = 0; e < VEC; ++e) sum[e] += v[u][e];
    }
    for (; sidx < p.splits; sidx += SY) {
      const vec_t v = *(const vec_t*)(ws + (int64_t)sidx * total + idx);
#pragma unroll
      for (int e = 0; e < VEC; ++e) sum[e] += v[e];
    }
    if constexpr (SY > 1) {
      if (row != (int64_t)blockIdx.y) __syncthreads();   // the previous row's sums have been read
      if (cl > 0) {
#pragma unroll
        for (int e = 0; e < VEC; ++e) cls[cl - 1][(threadIdx.x & 63) * VEC + e] = sum[e];
      }
      __syncthreads();
      if (cl > 0 || !in_range) continue;
#pragma unroll
      for (int w = 0; w < SY - 1; ++w)
#pragma unroll
        for (int e = 0; e < VEC; ++e) sum[e] += cls[w][(threadIdx.x & 63) * VEC + e];
    }
    T* cp = p.C + row * p.c_m + col * p.c_n;
    ACC cold[VEC], bias[VEC];
    if (p.beta != (T)0) {
#pragma unroll
      for (int e = 0; e < VEC; ++e) cold[e] = (ACC)cp[e * p.c_n];
    }
    if (p.epilogue & AM_EPI_BIAS) {
#pragma unroll
      for (int e = 0; e < VEC; ++e) bias[e] = (ACC)p.bias[row * p.bias_m + (col + e) * p.bias_n];
    }
#pragma unroll
    for (int e = 0; e < VEC; ++e) {
      ACC ab = sum[e];
      if (p.alpha != (T)1) ab = (ACC)p.alpha * ab;
      ACC v = ab;
      if (p.beta != (T)0) {
        ACC c = cold[e];
        if (p.beta != (T)1) c = c * (ACC)p.beta;
        v = c + ab;
      }
      if (p.epilogue & AM_EPI_BIAS) v = v + bias[e];
      if (p.epilogue & AM_EPI_RELU) v = ((ACC)0 >= v) ? (ACC)0 : v;
      cp[e * p.c_n] = (T)v;
    }
  }
}

template <typename T, typename ACC>
static int launch_splitk_reduce(const Args<T>& g) {
  constexpr int VEC = 16 / (int)sizeof(ACC);
  const bool vec = (g.N % VEC == 0);   // the workspace itself is 256-byte aligned and row pitch N
  const int64_t cols = vec ? g.N / VEC : g.N;
  // many partials of a small result: four wavefronts per 64 column groups, each a quarter of the partials
  const bool wide = vec && g.splits >= 32 && cols * g.M < (int64_t)num_cus() * 1024;
  const int64_t bx = wide ? (cols + 63) / 64 : (cols + 255) / 256;
  int64_t by = g.M;
  const int64_t cap = (int64_t)num_cus() * 16;
  if (bx * by > cap) by = (cap + bx - 1) / bx;
  if (by > 65535) by = 65535;
  if (by < 1) by = 1;
  const dim3 grid((unsigned)bx, (unsigned)by), block(256);
  if (wide) hipLaunchKernelGGL((splitk_reduce<T, ACC, VEC, 4>), grid, block, 0, stream(), g);
  else if (vec) hipLaunchKernelGGL((splitk_reduce<T, ACC, VEC>), grid, block, 0, stream(), g);
  else hipLaunchKernelGGL((splitk_reduce<T, ACC, 1>), grid, block, 0, stream(), g);
  return check_launch("splitk_reduce");
}

// Workgroup id -> (tile_m, tile_n).
//  1. Hardware deals consecutive workgroup ids round-robin to the 8 XCDs (each with its own L2):
//     id -> (id mod 8) * (n / 8) + id div 8 hands every XCD one contiguous run of tile numbers.
//  2. Tile numbers walk the grid in groups of kGroupM tile rows, column by column inside a group,
//     so the tiles an XCD works on at any moment form a roughly square patch: fewer distinct A and
//     B panels per XCD, hence fewer fetches into its L2.
constexpr int kGroupM = 8;
__device__ __forceinline__ void tile_of_block(int bid, int tiles_m, int tiles_n, int& tile_m, int& tile_n) {
  const int nb = tiles_m * tiles_n;
  if ((nb & 7) == 0) bid = (bid & 7) * (nb >> 3) + (bid >> 3);
  const int in_group = kGroupM * tiles_n;
  const int group = bid / in_group;
  const int first_m = group * kGroupM;
  const int rows = (tiles_m - first_m < kGroupM) ? tiles_m - first_m : kGroupM;
  const int r = bid - group * in_group;
  tile_m = first_m + r % rows;
  tile_n = r / rows;
}

}  // namespace gemm
}  // namespace am
