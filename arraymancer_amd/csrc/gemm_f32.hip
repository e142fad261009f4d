// float32 GEMM entry points (MFMA path): am_hip_gemm_f32, am_hip_gemm_ex_f32.
#include "gemm_mfma_impl.h"
#include "gemm_small_impl.h"

using namespace am;
using namespace am::gemm;

static int run_whole_f32(Args<float>& g);
static const TileChoice* candidates_f32(int* n);

// The product as the caller stated it: whole, or as an aligned block plus strips (plan_peel).
static int run_f32(Args<float>& g) {
  int nc = 0;
  const TileChoice* cand = candidates_f32(&nc);
  int64_t rm = 0, rn = 0;
  if (!small::applicable(g)) plan_peel(g, cand, nc, "AM_HIP_GEMM_TILE_F32", 157.3e6 / 256, &rm, &rn);
  if (rm == 0 && rn == 0) return run_whole_f32(g);
  const int64_t M0 = g.M - rm, N0 = g.N - rn;
  Args<float> part = sub_problem(g, 0, M0, 0, N0);
  AM_TRY(run_whole_f32(part));
  if (rm) { part = sub_problem(g, M0, g.M, 0, g.N); AM_TRY(run_whole_f32(part)); }   // bottom strip, full width
  if (rn) { part = sub_problem(g, 0, M0, N0, g.N); AM_TRY(run_whole_f32(part)); }   // right strip above it
  return AM_OK;
}

static int run_whole_f32(Args<float>& g) {
  if (small::applicable(g)) return small::run(g);   // few rows or columns: no LDS staging, no second kernel
  int ak = classify(g.A, g.a_mn, g.a_k, g.M, g.K);
  int bk = classify(g.B, g.b_mn, g.b_k, g.N, g.K);
  // Candidate workgroup tiles with the relative MFMA efficiency of each (measured on 2048^3 and
  // 4096^3). PF = 2 (two slabs of global loads in flight) on the tiles whose slab is short.
  int nc = 0;
  const TileChoice* cand = candidates_f32(&nc);
  switch (choose_tile_and_split(g, cand, nc, "AM_HIP_GEMM_TILE_F32", 157.3e6 / 256)) {
    case 0: return launch_kinds<float, 256, 256, 16, 2, 4, 1, true, false>(g, ak, bk);   // its loop is long enough: unrolling it over the ring costs 4 %
    case 1: {
      // Eight wavefronts of 32 x 64 (two per SIMD, which cover each other's waits) where no split of k is planned and the
      // four-wavefront form would not split either: 2048^3 127.2 -> 125.6 us, 2560^3 317 -> 302, 3072 x 3072 x 1024 193 ->
      // 187, 2048 x 2048 x 256 23.4 -> 21.9. Eight of 64 x 32 lose (133.5 us at 2048^3). Products that are cut along k keep
      // four wavefronts of 64 x 64: two workgroups, on different ranges of k, then share a CU.
      const int64_t tiles = ((g.M + 127) / 128) * ((g.N + 127) / 128) * (g.batch > 1 ? g.batch : 1);
      if (g.want_splits <= 1 && tiles * 8 > (int64_t)num_cus() * 4) return launch_kinds<float, 128, 128, 16, 4, 2, 2>(g, ak, bk);
      return launch_kinds<float, 128, 128, 16, 2, 2, 2>(g, ak, bk);
    }
    case 2: return launch_kinds<float, 64, 64, 16, 2, 2, 2>(g, ak, bk);
    case 3: return launch_kinds<float, 256, 128, 16, 4, 2>(g, ak, bk);
    case 4: return launch_kinds<float, 128, 64, 16, 2, 2, 2>(g, ak, bk);
    // four wavefronts of 16 x 16 each (one per SIMD) where one of 32 x 32 would run alone on its CU: 64 batched
    // [50 x 500] . [500 x 64] products 13.3 -> 7.2 us
    default: return launch_kinds<float, 32, 32, 32, 2, 2, 2, true, true, MfmaF32x16>(g, ak, bk);
  }
}

static const TileChoice* candidates_f32(int* n) {
  // {rows, columns, efficiency, slab width, wavefronts}
  static const TileChoice cand[] = {{256, 256, 1.0, 16, 8}, {128, 128, 0.94, 16, 4}, {64, 64, 0.88, 16, 4}, {256, 128, 0.97, 16, 8},
                                    {128, 64, 0.92, 16, 4},  {32, 32, 0.74, 32, 4}};
  *n = (int)(sizeof(cand) / sizeof(cand[0]));
  return cand;
}

extern "C" int am_hip_gemm_ex_f32(int64_t M, int64_t N, int64_t K, float alpha, const float* A, int64_t rsA,
                                  int64_t csA, const float* B, int64_t rsB, int64_t csB, float beta, float* C,
                                  int64_t rsC, int64_t csC, int epilogue, const float* bias,
                                  int64_t bias_rs, int64_t bias_cs) {
  Args<float> g;
  const int rc = prepare<float>("am_hip_gemm_f32", M, N, K, alpha, A, rsA, csA, B, rsB, csB, beta, C, rsC, csC,
                            epilogue, bias, bias_rs, bias_cs, &g);
  if (rc > 0) return AM_OK;
  if (rc < 0) return rc;
  AM_TRY(ensure_init());
  return run_f32(g);
}

extern "C" int am_hip_gemm_f32(int64_t M, int64_t N, int64_t K, float alpha, const float* A, int64_t rsA,
                               int64_t csA, const float* B, int64_t rsB, int64_t csB, float beta, float* C,
                               int64_t rsC, int64_t csC) {
  return am_hip_gemm_ex_f32(M, N, K, alpha, A, rsA, csA, B, rsB, csB, beta, C, rsC, csC, AM_EPI_NONE,
                            nullptr, 0, 0);
}

// am_hip_gemm_f32 for callers that cannot allocate: same kernels, split-K partials in the library's
// static device array. Calls no hipMalloc / hipFree and no routine that allocates.
extern "C" int am_hip_gemm_noalloc_f32(int64_t M, int64_t N, int64_t K, float alpha, const float* A, int64_t rsA,
                                       int64_t csA, const float* B, int64_t rsB, int64_t csB, float beta, float* C,
                                       int64_t rsC, int64_t csC) {
  Args<float> g;
  const int rc = prepare<float>("am_hip_gemm_noalloc_f32", M, N, K, alpha, A, rsA, csA, B, rsB, csB, beta, C, rsC, csC,
                                AM_EPI_NONE, nullptr, 0, 0, &g);
  if (rc > 0) return AM_OK;
  if (rc < 0) return rc;
  AM_TRY(ensure_init());
  g.static_ws = true;
  return run_f32(g);
}

extern "C" int am_hip_gemm_batched_f32(int64_t batch, int64_t M, int64_t N, int64_t K, float alpha, const float* A,
                                       int64_t rsA, int64_t csA, int64_t bsA, const float* B, int64_t rsB, int64_t csB,
                                       int64_t bsB, float beta, float* C, int64_t rsC, int64_t csC, int64_t bsC,
                                       int epilogue, const float* bias, int64_t bias_rs, int64_t bias_cs) {
  if (batch < 0 || batch > 65535) return fail(AM_E_ARG, "am_hip_gemm_batched_f32: batch %lld outside 0..65535", (long long)batch);
  if (batch == 0) return AM_OK;
  Args<float> g;
  const int rc = prepare<float>("am_hip_gemm_batched_f32", M, N, K, alpha, A, rsA, csA, B, rsB, csB, beta, C, rsC, csC,
                            epilogue, bias, bias_rs, bias_cs, &g);
  if (rc > 0) return AM_OK;
  if (rc < 0) return rc;
  if (batch > 1 && bsC == 0) return fail(AM_E_SHAPE, "am_hip_gemm_batched_f32: C has batch stride 0");
  g.batch = (int)batch;
  g.batch_a = g.swapped ? bsB : bsA;
  g.batch_b = g.swapped ? bsA : bsB;
  g.batch_c = bsC;
  AM_TRY(ensure_init());
  return run_f32(g);
}

// im2colgemm_conv2d (src/arraymancer/nn_primitives/fallback/conv.nim:81-106) in one launch: the column matrix is never
// written, the GEMM's B loader gathers it from the images; bias and ReLU in the epilogue.
extern "C" int am_hip_conv2d_f32(int64_t N, int C, int H, int W, int Cout, int kH, int kW, int padH, int padW, int strideH,
                                 int strideW, const float* in, int64_t in_n, int64_t in_c, int64_t in_h, int64_t in_w,
                                 const float* kernel, int64_t kernel_rs, int epilogue, const float* bias, int64_t bias_s, float* out) {
  Args<float> g;
  const int rc = prepare_conv<float>("am_hip_conv2d_f32", N, C, H, W, Cout, kH, kW, padH, padW, strideH, strideW, in, in_n, in_c,
                                    in_h, in_w, kernel, kernel_rs, epilogue, bias, bias_s, out, &g);
  if (rc > 0) return AM_OK;
  if (rc < 0) return rc;
  AM_TRY(ensure_init());
  // (128 x 128 and 64 x 128 tiles measured slower than these on every shape tried; 128 x 64 pays from 128 output channels on)
  static const TileChoice cand[] = {{64, 64, 0.88}, {32, 32, 0.60}, {128, 64, 0.92}};
  switch (choose_tile(cand, 3, g.M, g.N, "AM_HIP_CONV_TILE_F32", g.batch)) {
    case 0: return launch_conv<float, 64, 64, 16, 2, 2, 2>(g);
    case 2: return launch_conv<float, 128, 64, 16, 2, 2, 2>(g);
    default: return launch_conv<float, 32, 32, 32, 2, 2, 2, true, true, MfmaF32x16>(g);
  }
}

// The weight gradient of im2colgemm_conv2d_gradient (src/arraymancer/nn_primitives/fallback/conv.nim:135-143) over the whole
// batch as ONE product with k = images * outputs: the column matrices are never written, the GEMM's B loader gathers
// their transposes from the images in 16-byte pieces.
extern "C" int am_hip_conv2d_grad_weight_f32(int64_t N, int C, int H, int W, int Cout, int kH, int kW, int padH, int padW, int strideH,
                                             int strideW, const float* in, int64_t in_n, int64_t in_c, int64_t in_h, int64_t in_w,
                                             const float* gout, int64_t gout_rs, float* out) {
  Args<float> g;
  const int rc = prepare_conv_grad_weight<float>("am_hip_conv2d_grad_weight_f32", N, C, H, W, Cout, kH, kW, padH, padW, strideH, strideW,
                                                in, in_n, in_c, in_h, in_w, gout, gout_rs, out, &g);
  if (rc > 0) return AM_OK;
  if (rc < 0) return rc;
  AM_TRY(ensure_init());
  // the candidates of the plain product that a gathered B takes (few output channels: 64 rows; 128 from 128 on)
  static const TileChoice cand[] = {{64, 64, 0.88, 16, 4}, {32, 32, 0.74, 32, 4}, {128, 64, 0.92, 16, 4}};
  switch (choose_tile_and_split(g, cand, 3, "AM_HIP_CONV_GW_TILE_F32", 157.3e6 / 256)) {
    case 0: return launch_conv_grad_weight<float, 64, 64, 16, 2, 2, 2>(g);
    case 2: return launch_conv_grad_weight<float, 128, 64, 16, 2, 2, 2>(g);
    default: return launch_conv_grad_weight<float, 32, 32, 32, 2, 2, 2, true, true, MfmaF32x16>(g);
  }
}
