// Host-side pieces shared by the MFMA (f32/f64) and VALU (i32/i64) GEMM families: the kernel
// argument block, argument validation, operand classification and the tile-shape choice.
#pragma once
#include <stdlib.h>
#include <string.h>
#include "common.h"

namespace am {
namespace gemm {

// How the loader may fetch an operand tile X(mn, k) = X[mn * ld_mn + k * ld_k].
enum LoadKind : int {
  kKContig = 0,   // ld_k == 1: 16-byte vectors along k
  kMNContig = 1,  // ld_mn == 1: 16-byte vectors along m (A) or n (B)
  kGeneric = 2    // any strides (zero, negative, non-unit): scalar gathers
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
};

static inline bool aligned16(const void* p) { return ((uintptr_t)p & 15u) == 0; }

template <typename T>
static inline int classify(const T* X, int64_t ld_mn, int64_t ld_k, int64_t MN, int64_t K) {
  constexpr int64_t VK = 16 / (int64_t)sizeof(T);
  if (ld_k == 1 && K % VK == 0 && (ld_mn % VK == 0 || MN == 1) && ld_mn >= 0 && aligned16(X)) return kKContig;
  if (ld_mn == 1 && MN % VK == 0 && (ld_k % VK == 0 || K == 1) && ld_k >= 0 && aligned16(X)) return kMNContig;
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
  g.a_kfast = iabs64(g.a_k) <= iabs64(g.a_mn);
  g.b_kfast = iabs64(g.b_k) < iabs64(g.b_mn);
  return AM_OK;
}

// One candidate tile shape and the relative speed of a CU that runs it.
struct TileChoice { int bm, bn; double eff; };

// Picks the candidate with the least estimated time: rounds of one block per CU, each round
// costing bm*bn/eff. Ragged edges and under-filled rounds are priced by construction.
static inline int choose_tile(const TileChoice* cand, int ncand, int64_t M, int64_t N, const char* env) {
  const char* forced = getenv(env);
  if (forced && *forced) {
    int idx = atoi(forced);
    if (idx >= 0 && idx < ncand) return idx;
  }
  const int64_t cus = num_cus();
  int best = 0;
  double best_cost = 0;
  for (int i = 0; i < ncand; ++i) {
    if (cand[i].eff <= 0) continue;   // experimental shape: only when forced
    const int64_t tiles = ((M + cand[i].bm - 1) / cand[i].bm) * ((N + cand[i].bn - 1) / cand[i].bn);
    const int64_t rounds = (tiles + cus - 1) / cus;
    const double cost = (double)rounds * cand[i].bm * cand[i].bn / cand[i].eff;
    if (i == 0 || cost < best_cost) { best = i; best_cost = cost; }
  }
  return best;
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
