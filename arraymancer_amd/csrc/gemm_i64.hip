// int64 GEMM entry point (VALU path, wraparound arithmetic): am_hip_gemm_i64.
#include "gemm_int_impl.h"

using namespace am;
using namespace am::gemm;

extern "C" int am_hip_gemm_i64(int64_t M, int64_t N, int64_t K, int64_t alpha, const int64_t* A, int64_t rsA,
                               int64_t csA, const int64_t* B, int64_t rsB, int64_t csB, int64_t beta, int64_t* C,
                               int64_t rsC, int64_t csC) {
  Args<int64_t> g;
  const int rc = prepare<int64_t>("am_hip_gemm_i64", M, N, K, alpha, A, rsA, csA, B, rsB, csB, beta, C, rsC, csC,
                            AM_EPI_NONE, nullptr, 0, 0, &g);
  if (rc > 0) return AM_OK;
  if (rc < 0) return rc;
  AM_TRY(ensure_init());
  const int ak = classify(g.A, g.a_mn, g.a_k, g.M, g.K);
  const int bk = classify(g.B, g.b_mn, g.b_k, g.N, g.K);
  static const TileChoice cand[] = {{128, 128, 1.0}, {64, 64, 1.0}};
  switch (choose_tile(cand, 2, g.M, g.N, "AM_HIP_GEMM_TILE_I64")) {
    case 0: return launch_valu<int64_t, 8, 8, 16>(g, ak, bk);
    default: return launch_valu<int64_t, 4, 4, 16>(g, ak, bk);
  }
}
