// int64 GEMM entry points (wraparound arithmetic): large products run on the int8 matrix cores by
// digit slicing, the others on the vector ALU.
#include "gemm_int_impl.h"
#include "gemm_i8_digits.h"

using namespace am;
using namespace am::gemm;

static int run_i64(Args<int64_t>& g) {
  int ak = classify(g.A, g.a_mn, g.a_k, g.M, g.K);
  int bk = classify(g.B, g.b_mn, g.b_k, g.N, g.K);
  // 8 x 8 and 4 x 4 results per lane; the small tile re-reads LDS twice as often per multiply-add.
  static const TileChoice cand[] = {{128, 128, 1.0}, {64, 64, 0.85}};
  // 34.0e3 multiply-adds per microsecond and CU: the measured VALU ceiling of this element type.
  const TileSplit ts = choose_tile_split<int64_t>(cand, 2, g.M, g.N, g.K, 16, 34.0e3, "AM_HIP_GEMM_TILE_I64", g.batch);
  // The same product on the int8 matrix cores (digit slicing) when that is estimated to be faster,
  // or when it would be for operands with few non-empty digit planes (then the data decides on the device).
  int rc = AM_OK;
  if (!i8::try_digits(g, ts.est_us, &rc)) return rc;
  switch (ts.tile) {
    case 0: return launch_valu<int64_t, 8, 8, 16>(g, ak, bk, ts.splits);
    default: return launch_valu<int64_t, 4, 4, 16>(g, ak, bk, ts.splits);
  }
}

extern "C" int am_hip_gemm_i64(int64_t M, int64_t N, int64_t K, int64_t alpha, const int64_t* A, int64_t rsA,
                               int64_t csA, const int64_t* B, int64_t rsB, int64_t csB, int64_t beta, int64_t* C,
                               int64_t rsC, int64_t csC) {
  Args<int64_t> g;
  const int rc = prepare<int64_t>("am_hip_gemm_i64", M, N, K, alpha, A, rsA, csA, B, rsB, csB, beta, C, rsC, csC,
                            AM_EPI_NONE, nullptr, 0, 0, &g);
  if (rc > 0) return AM_OK;
  if (rc < 0) return rc;
  AM_TRY(ensure_init());
  return run_i64(g);
}

extern "C" int am_hip_gemm_prepared_i64(int64_t M, int64_t N, int64_t K, int64_t alpha, const int64_t* A, int64_t rsA,
                                        int64_t csA, const void* A_digits, const int64_t* B, int64_t rsB, int64_t csB,
                                        const void* B_digits, int64_t beta, int64_t* C, int64_t rsC, int64_t csC) {
  const i8::Prepared* ha = A_digits ? i8::lookup_prepared(A_digits) : nullptr;
  const i8::Prepared* hb = B_digits ? i8::lookup_prepared(B_digits) : nullptr;
  if ((A_digits && !ha) || (B_digits && !hb))
    return fail(AM_E_ARG, "am_hip_gemm_prepared_i64: not a live handle of am_hip_digits_prepare_i64");
  Args<int64_t> g;
  const int rc = prepare<int64_t>("am_hip_gemm_prepared_i64", M, N, K, alpha, A, rsA, csA, B, rsB, csB, beta, C, rsC, csC,
                                  AM_EPI_NONE, nullptr, 0, 0, &g);
  if (rc > 0) return AM_OK;
  if (rc < 0) return rc;
  AM_TRY(ensure_init());
  if (ha || hb) {
    int r = AM_OK;
    if (!i8::run_prepared(g, ha, hb, &r)) return r;
  }
  return run_i64(g);
}

// Integer batched product: no fused epilogue (pass AM_EPI_NONE; add a bias with the element-wise ops).
extern "C" int am_hip_gemm_batched_i64(int64_t batch, int64_t M, int64_t N, int64_t K, int64_t alpha, const int64_t* A,
                                       int64_t rsA, int64_t csA, int64_t bsA, const int64_t* B, int64_t rsB, int64_t csB,
                                       int64_t bsB, int64_t beta, int64_t* C, int64_t rsC, int64_t csC, int64_t bsC,
                                       int epilogue, const int64_t* bias, int64_t bias_rs, int64_t bias_cs) {
  (void)bias; (void)bias_rs; (void)bias_cs;
  if (epilogue != AM_EPI_NONE) return fail(AM_E_DTYPE, "am_hip_gemm_batched_i64: fused epilogues are defined for float tensors");
  if (batch < 0 || batch > 65535) return fail(AM_E_ARG, "am_hip_gemm_batched_i64: batch %lld outside 0..65535", (long long)batch);
  if (batch == 0) return AM_OK;
  Args<int64_t> g;
  const int rc = prepare<int64_t>("am_hip_gemm_batched_i64", M, N, K, alpha, A, rsA, csA, B, rsB, csB, beta, C, rsC, csC,
                            AM_EPI_NONE, nullptr, 0, 0, &g);
  if (rc > 0) return AM_OK;
  if (rc < 0) return rc;
  if (batch > 1 && bsC == 0) return fail(AM_E_SHAPE, "am_hip_gemm_batched_i64: C has batch stride 0");
  g.batch = (int)batch;
  g.batch_a = g.swapped ? bsB : bsA;
  g.batch_b = g.swapped ? bsA : bsB;
  g.batch_c = bsC;
  AM_TRY(ensure_init());
  return run_i64(g);
}
