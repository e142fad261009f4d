// int32 GEMM entry point (VALU path, wraparound arithmetic): am_hip_gemm_i32.
#include "gemm_int_impl.h"

using namespace am;
using namespace am::gemm;

extern "C" int am_hip_gemm_i32(int64_t M, int64_t N, int64_t K, int32_t alpha, const int32_t* A, int64_t rsA,
                               int64_t csA, const int32_t* B, int64_t rsB, int64_t csB, int32_t beta, int32_t* C,
                               int64_t rsC, int64_t csC) {
  Args<int32_t> g;
  const int rc = prepare<int32_t>("am_hip_gemm_i32", M, N, K, alpha, A, rsA, csA, B, rsB, csB, beta, C, rsC, csC,
                            AM_EPI_NONE, nullptr, 0, 0, &g);
  if (rc > 0) return AM_OK;
  if (rc < 0) return rc;
  AM_TRY(ensure_init());
  const int ak = classify(g.A, g.a_mn, g.a_k, g.M, g.K);
  const int bk = classify(g.B, g.b_mn, g.b_k, g.N, g.K);
  static const TileChoice cand[] = {{128, 128, 1.0}, {64, 64, 1.0}};
  switch (choose_tile(cand, 2, g.M, g.N, "AM_HIP_GEMM_TILE_I32")) {
    case 0: return launch_valu<int32_t, 8, 8, 16>(g, ak, bk);
    default: return launch_valu<int32_t, 4, 4, 16>(g, ak, bk);
  }
}
