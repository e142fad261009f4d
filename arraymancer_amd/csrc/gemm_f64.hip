// float64 GEMM entry points (MFMA path): am_hip_gemm_f64, am_hip_gemm_ex_f64.
#include "gemm_mfma_impl.h"
#include "gemm_small_impl.h"

using namespace am;
using namespace am::gemm;

static int run_whole_f64(Args<double>& g);
static const TileChoice* candidates_f64(int* n);

// The product as the caller stated it: whole, or as an aligned block plus strips (plan_peel).
static int run_f64(Args<double>& g) {
  int nc = 0;
  const TileChoice* cand = candidates_f64(&nc);
  int64_t rm = 0, rn = 0;
  if (!small::applicable(g)) plan_peel(g, cand, nc, "AM_HIP_GEMM_TILE_F64", 78.6e6 / 256, &rm, &rn);
  if (rm == 0 && rn == 0) return run_whole_f64(g);
  const int64_t M0 = g.M - rm, N0 = g.N - rn;
  Args<double> part = sub_problem(g, 0, M0, 0, N0);
  AM_TRY(run_whole_f64(part));
  if (rm) { part = sub_problem(g, M0, g.M, 0, g.N); AM_TRY(run_whole_f64(part)); }   // bottom strip, full width
  if (rn) { part = sub_problem(g, 0, M0, N0, g.N); AM_TRY(run_whole_f64(part)); }   // right strip above it
  return AM_OK;
}

static int run_whole_f64(Args<double>& g) {
  if (small::applicable(g)) return small::run(g);   // few rows or columns: no LDS staging, no second kernel
  int ak = classify(g.A, g.a_mn, g.a_k, g.M, g.K);
  int bk = classify(g.B, g.b_mn, g.b_k, g.N, g.K);
  // Candidate workgroup tiles with the relative MFMA efficiency of each. The 128 x 128 tile runs
  // with 8 wavefronts (64 x 32 each) and the 256 x 128 one without fragment prefetch: a 64 x 64
  // wavefront tile of doubles (128 accumulator registers) leaves no room for a second fragment set.
  // 128 x 192 (8 wavefronts of 64 x 48) exists for shapes that the others cut into a number of
  // tiles just above a multiple of the CU count: 2048 x 3072 is 384 tiles of 128 x 128 (two rounds,
  // the second half empty) but exactly 256 of 128 x 192.
  int nc = 0;
  const TileChoice* cand = candidates_f64(&nc);
  switch (choose_tile_and_split(g, cand, nc, "AM_HIP_GEMM_TILE_F64", 78.6e6 / 256)) {
    case 0: return launch_kinds<double, 128, 128, 16, 2, 4>(g, ak, bk);
    case 1: return launch_kinds<double, 64, 64, 16, 2, 2, 2>(g, ak, bk);
    case 2: return launch_kinds<double, 32, 32, 16, 2, 2, 2>(g, ak, bk);
    case 3: return launch_kinds<double, 256, 128, 16, 4, 2, 1, false>(g, ak, bk);
    case 4: return launch_kinds<double, 128, 64, 16, 2, 2, 2>(g, ak, bk);
    default: return launch_kinds<double, 128, 192, 16, 2, 4, 1, false>(g, ak, bk);
  }
}

static const TileChoice* candidates_f64(int* n) {
  // {rows, columns, efficiency, slab width, wavefronts}
  static const TileChoice cand[] = {{128, 128, 0.97, 16, 8}, {64, 64, 0.93, 16, 4}, {32, 32, 0.76, 16, 4}, {256, 128, 1.0, 16, 8},
                                    {128, 64, 0.96, 16, 4},  {128, 192, 0.98, 16, 8}};
  *n = (int)(sizeof(cand) / sizeof(cand[0]));
  return cand;
}

extern "C" int am_hip_gemm_ex_f64(int64_t M, int64_t N, int64_t K, double alpha, const double* A, int64_t rsA,
                                  int64_t csA, const double* B, int64_t rsB, int64_t csB, double beta, double* C,
                                  int64_t rsC, int64_t csC, int epilogue, const double* bias,
                                  int64_t bias_rs, int64_t bias_cs) {
  Args<double> g;
  const int rc = prepare<double>("am_hip_gemm_f64", M, N, K, alpha, A, rsA, csA, B, rsB, csB, beta, C, rsC, csC,
                            epilogue, bias, bias_rs, bias_cs, &g);
  if (rc > 0) return AM_OK;
  if (rc < 0) return rc;
  AM_TRY(ensure_init());
  return run_f64(g);
}

extern "C" int am_hip_gemm_f64(int64_t M, int64_t N, int64_t K, double alpha, const double* A, int64_t rsA,
                               int64_t csA, const double* B, int64_t rsB, int64_t csB, double beta, double* C,
                               int64_t rsC, int64_t csC) {
  return am_hip_gemm_ex_f64(M, N, K, alpha, A, rsA, csA, B, rsB, csB, beta, C, rsC, csC, AM_EPI_NONE,
                            nullptr, 0, 0);
}

extern "C" int am_hip_gemm_batched_f64(int64_t batch, int64_t M, int64_t N, int64_t K, double alpha, const double* A,
                                       int64_t rsA, int64_t csA, int64_t bsA, const double* B, int64_t rsB, int64_t csB,
                                       int64_t bsB, double beta, double* C, int64_t rsC, int64_t csC, int64_t bsC,
                                       int epilogue, const double* bias, int64_t bias_rs, int64_t bias_cs) {
  if (batch < 0 || batch > 65535) return fail(AM_E_ARG, "am_hip_gemm_batched_f64: batch %lld outside 0..65535", (long long)batch);
  if (batch == 0) return AM_OK;
  Args<double> g;
  const int rc = prepare<double>("am_hip_gemm_batched_f64", M, N, K, alpha, A, rsA, csA, B, rsB, csB, beta, C, rsC, csC,
                            epilogue, bias, bias_rs, bias_cs, &g);
  if (rc > 0) return AM_OK;
  if (rc < 0) return rc;
  if (batch > 1 && bsC == 0) return fail(AM_E_SHAPE, "am_hip_gemm_batched_f64: C has batch stride 0");
  g.batch = (int)batch;
  g.batch_a = g.swapped ? bsB : bsA;
  g.batch_b = g.swapped ? bsA : bsB;
  g.batch_c = bsC;
  AM_TRY(ensure_init());
  return run_f64(g);
}

// im2colgemm_conv2d (src/arraymancer/nn_primitives/fallback/conv.nim:81-106) in one launch: the column matrix is never
// written, the GEMM's B loader gathers it from the images; bias and ReLU in the epilogue.
extern "C" int am_hip_conv2d_f64(int64_t N, int C, int H, int W, int Cout, int kH, int kW, int padH, int padW, int strideH,
                                 int strideW, const double* in, int64_t in_n, int64_t in_c, int64_t in_h, int64_t in_w,
                                 const double* kernel, int64_t kernel_rs, int epilogue, const double* bias, int64_t bias_s, double* out) {
  Args<double> g;
  const int rc = prepare_conv<double>("am_hip_conv2d_f64", N, C, H, W, Cout, kH, kW, padH, padW, strideH, strideW, in, in_n, in_c,
                                    in_h, in_w, kernel, kernel_rs, epilogue, bias, bias_s, out, &g);
  if (rc > 0) return AM_OK;
  if (rc < 0) return rc;
  AM_TRY(ensure_init());
  static const TileChoice cand[] = {{64, 64, 0.93}, {32, 32, 0.62}};
  switch (choose_tile(cand, 2, g.M, g.N, "AM_HIP_CONV_TILE_F64", g.batch)) {
    case 0: return launch_conv<double, 64, 64, 16, 2, 2, 2>(g);
    default: return launch_conv<double, 32, 32, 16, 2, 2, 2>(g);
  }
}

// The weight gradient of im2colgemm_conv2d_gradient (src/arraymancer/nn_primitives/fallback/conv.nim:135-143) over the whole
// batch as ONE product with k = images * outputs: the column matrices are never written, the GEMM's B loader gathers
// their transposes from the images in 16-byte pieces.
extern "C" int am_hip_conv2d_grad_weight_f64(int64_t N, int C, int H, int W, int Cout, int kH, int kW, int padH, int padW, int strideH,
                                             int strideW, const double* in, int64_t in_n, int64_t in_c, int64_t in_h, int64_t in_w,
                                             const double* gout, int64_t gout_rs, double* out) {
  Args<double> g;
  const int rc = prepare_conv_grad_weight<double>("am_hip_conv2d_grad_weight_f64", N, C, H, W, Cout, kH, kW, padH, padW, strideH, strideW,
                                                in, in_n, in_c, in_h, in_w, gout, gout_rs, out, &g);
  if (rc > 0) return AM_OK;
  if (rc < 0) return rc;
  AM_TRY(ensure_init());
  static const TileChoice cand[] = {{64, 64, 0.88, 16, 4}, {32, 32, 0.60, 16, 4}};
  switch (choose_tile_and_split(g, cand, 2, "AM_HIP_CONV_GW_TILE_F64", 78.6e6 / 256)) {
    case 0: return launch_conv_grad_weight<double, 64, 64, 16, 2, 2, 2>(g);
    default: return launch_conv_grad_weight<double, 32, 32, 16, 2, 2, 2>(g);
  }
}
