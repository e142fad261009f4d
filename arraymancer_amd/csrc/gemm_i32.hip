// int32 GEMM entry points (wraparound arithmetic): large products run on the int8 matrix cores by
// digit slicing, the others on the vector ALU.
#include <mutex>
#include <unordered_set>
#include "gemm_int_impl.h"
#include "gemm_i8_digits.h"

using namespace am;
using namespace am::gemm;

namespace am {
namespace gemm {
namespace i8 {
static std::mutex g_prepared_mu;
static std::unordered_set<const Prepared*> g_prepared;
void remember_prepared(const Prepared* p) {
  std::lock_guard<std::mutex> lk(g_prepared_mu);
  g_prepared.insert(p);
}
const Prepared* lookup_prepared(const void* handle) {
  std::lock_guard<std::mutex> lk(g_prepared_mu);
  const Prepared* p = (const Prepared*)handle;
  return g_prepared.count(p) ? p : nullptr;
}
}  // namespace i8
}  // namespace gemm
}  // namespace am

extern "C" int am_hip_digits_release(void* handle) {
  if (!handle) return AM_OK;
  i8::Prepared* p = nullptr;
  {
    std::lock_guard<std::mutex> lk(i8::g_prepared_mu);
    auto it = i8::g_prepared.find((const i8::Prepared*)handle);
    if (it == i8::g_prepared.end())
      return fail(AM_E_ARG, "am_hip_digits_release: %p is not a handle of am_hip_digits_prepare_* (or was released already)", handle);
    p = const_cast<i8::Prepared*>(*it);
    i8::g_prepared.erase(it);
  }
  // (stream ordered: a product that still reads the planes is ahead of whoever receives the block next)
  const int rc = am_hip_free(p->planes);
  p->magic = 0;
  delete p;
  return rc;
}

// side 0: X is the left operand of later products, [rows x cols] = [M x K]; side 1: the right one, [K x N].
template <typename T>
static int digits_prepare(const char* who, int side, int64_t rows, int64_t cols, const T* X, int64_t rs, int64_t cs, void** handle) {
  if (!handle) return fail(AM_E_ARG, "%s: null handle pointer", who);
  *handle = nullptr;
  if (side != 0 && side != 1) return fail(AM_E_ARG, "%s: side must be 0 (left operand) or 1 (right operand)", who);
  if (rows <= 0 || cols <= 0 || !X) return fail(AM_E_SHAPE, "%s: empty operand", who);
  AM_TRY(ensure_init());
  if (capturing()) return fail(AM_E_ARG, "%s: not allowed while a graph is being captured", who);
  i8::Prepared* p = new i8::Prepared();
  const int rc = side == 0 ? i8::prepare_planes<T>(X, rows, cols, rs, cs, p) : i8::prepare_planes<T>(X, cols, rows, cs, rs, p);
  if (rc != AM_OK) { delete p; return rc; }
  i8::remember_prepared(p);
  *handle = p;
  return AM_OK;
}

extern "C" int am_hip_digits_prepare_i32(int side, int64_t rows, int64_t cols, const int32_t* X, int64_t rs, int64_t cs, void** handle) {
  return digits_prepare<int32_t>("am_hip_digits_prepare_i32", side, rows, cols, X, rs, cs, handle);
}
extern "C" int am_hip_digits_prepare_i64(int side, int64_t rows, int64_t cols, const int64_t* X, int64_t rs, int64_t cs, void** handle) {
  return digits_prepare<int64_t>("am_hip_digits_prepare_i64", side, rows, cols, X, rs, cs, handle);
}

static int run_i32(Args<int32_t>& g) {

  int ak = classify(g.A, g.a_mn, g.a_k, g.M, g.K);
  int bk = classify(g.B, g.b_mn, g.b_k, g.N, g.K);
  // 8 x 8 and 4 x 4 results per lane; the small tile re-reads LDS twice as often per multiply-add.
  static const TileChoice cand[] = {{128, 128, 1.0}, {64, 64, 0.85}};
  // 119.0e3 multiply-adds per microsecond and CU: the measured VALU ceiling of this element type.
  const TileSplit ts = choose_tile_split<int32_t>(cand, 2, g.M, g.N, g.K, 16, 119.0e3, "AM_HIP_GEMM_TILE_I32", g.batch);
  // The same product on the int8 matrix cores (digit slicing) when that is estimated to be faster,
  // or when it would be for operands with few non-empty digit planes (then the data decides on the device).
  int rc = AM_OK;
  if (!i8::try_digits(g, ts.est_us, &rc)) return rc;
  switch (ts.tile) {
    case 0: return launch_valu<int32_t, 8, 8, 16>(g, ak, bk, ts.splits);
    default: return launch_valu<int32_t, 4, 4, 16>(g, ak, bk, ts.splits);
  }
}

extern "C" int am_hip_gemm_i32(int64_t M, int64_t N, int64_t K, int32_t alpha, const int32_t* A, int64_t rsA,
                               int64_t csA, const int32_t* B, int64_t rsB, int64_t csB, int32_t beta, int32_t* C,
                               int64_t rsC, int64_t csC) {
  Args<int32_t> g;
  const int rc = prepare<int32_t>("am_hip_gemm_i32", M, N, K, alpha, A, rsA, csA, B, rsB, csB, beta, C, rsC, csC,
                            AM_EPI_NONE, nullptr, 0, 0, &g);
  if (rc > 0) return AM_OK;
  if (rc < 0) return rc;
  AM_TRY(ensure_init());
  return run_i32(g);
}

extern "C" int am_hip_gemm_prepared_i32(int64_t M, int64_t N, int64_t K, int32_t alpha, const int32_t* A, int64_t rsA,
                                        int64_t csA, const void* A_digits, const int32_t* B, int64_t rsB, int64_t csB,
                                        const void* B_digits, int32_t beta, int32_t* C, int64_t rsC, int64_t csC) {
  const i8::Prepared* ha = A_digits ? i8::lookup_prepared(A_digits) : nullptr;
  const i8::Prepared* hb = B_digits ? i8::lookup_prepared(B_digits) : nullptr;
  if ((A_digits && !ha) || (B_digits && !hb))
    return fail(AM_E_ARG, "am_hip_gemm_prepared_i32: not a live handle of am_hip_digits_prepare_i32");
  Args<int32_t> g;
  const int rc = prepare<int32_t>("am_hip_gemm_prepared_i32", M, N, K, alpha, A, rsA, csA, B, rsB, csB, beta, C, rsC, csC,
                                  AM_EPI_NONE, nullptr, 0, 0, &g);
  if (rc > 0) return AM_OK;
  if (rc < 0) return rc;
  AM_TRY(ensure_init());
  if (ha || hb) {
    int r = AM_OK;
    if (!i8::run_prepared(g, ha, hb, &r)) return r;
  }
  return run_i32(g);
}

// Integer batched product: no fused epilogue (pass AM_EPI_NONE; add a bias with the element-wise ops).
extern "C" int am_hip_gemm_batched_i32(int64_t batch, int64_t M, int64_t N, int64_t K, int32_t alpha, const int32_t* A,
                                       int64_t rsA, int64_t csA, int64_t bsA, const int32_t* B, int64_t rsB, int64_t csB,
                                       int64_t bsB, int32_t beta, int32_t* C, int64_t rsC, int64_t csC, int64_t bsC,
                                       int epilogue, const int32_t* bias, int64_t bias_rs, int64_t bias_cs) {
  (void)bias; (void)bias_rs; (void)bias_cs;
  if (epilogue != AM_EPI_NONE) return fail(AM_E_DTYPE, "am_hip_gemm_batched_i32: fused epilogues are defined for float tensors");
  if (batch < 0 || batch > 65535) return fail(AM_E_ARG, "am_hip_gemm_batched_i32: batch %lld outside 0..65535", (long long)batch);
  if (batch == 0) return AM_OK;
  Args<int32_t> g;
  const int rc = prepare<int32_t>("am_hip_gemm_batched_i32", M, N, K, alpha, A, rsA, csA, B, rsB, csB, beta, C, rsC, csC,
                            AM_EPI_NONE, nullptr, 0, 0, &g);
  if (rc > 0) return AM_OK;
  if (rc < 0) return rc;
  if (batch > 1 && bsC == 0) return fail(AM_E_SHAPE, "am_hip_gemm_batched_i32: C has batch stride 0");
  g.batch = (int)batch;
  g.batch_a = g.swapped ? bsB : bsA;
  g.batch_b = g.swapped ? bsA : bsB;
  g.batch_c = bsC;
  AM_TRY(ensure_init());
  return run_i32(g);
}
