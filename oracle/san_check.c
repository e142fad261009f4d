/*
 * TEST INFRASTRUCTURE - sanitizer run of the CPU oracle. Built with -fsanitize=address,undefined (see the
 * Makefile target `san_check`) and run by tests/test_oracle_sanitizers.py: every entry family of the oracle
 * is driven over small, awkward shapes (tile edges of the blocked GEMM, zero and negative strides, ragged
 * block splits) and each result is compared with a brute-force loop written here, so that an out-of-bounds
 * access or undefined operation in the restatement shows up as a sanitizer report and a wrong index as a
 * mismatch. Exit code 0 = clean.
 */
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#define DECL(T, SFX)                                                                                          \
  int am_oracle_gemm_strided_##SFX(int64_t, int64_t, int64_t, T, const T*, int64_t, int64_t, const T*, int64_t, \
                                   int64_t, T, T*, int64_t, int64_t);                                         \
  int am_oracle_map2_##SFX(int, int, const int64_t*, T*, const int64_t*, const T*, const int64_t*, const T*,   \
                           const int64_t*);                                                                    \
  int am_oracle_compare_##SFX(int, int, const int64_t*, uint8_t*, const int64_t*, const T*, const int64_t*,    \
                              const T*, const int64_t*);                                                       \
  int am_oracle_reduce_axis_##SFX(int, int, const int64_t*, int, T*, const int64_t*, const T*, const int64_t*);
DECL(float, f32) DECL(double, f64) DECL(int32_t, i32) DECL(int64_t, i64)

static uint64_t rng_state = 0x9e3779b97f4a7c15ull;
static uint64_t rnd(void) { rng_state ^= rng_state << 13; rng_state ^= rng_state >> 7; rng_state ^= rng_state << 17; return rng_state; }
static int64_t rnd_in(int64_t lo, int64_t hi) { return lo + (int64_t)(rnd() % (uint64_t)(hi - lo + 1)); }

static int failures = 0;
#define EXPECT(cond, ...) do { if (!(cond)) { ++failures; printf("MISMATCH "); printf(__VA_ARGS__); printf("\n"); } } while (0)

/* A [rows x cols] view of geometry `kind` over a freshly allocated parent; returns the view's first element. */
typedef struct { void* parent; int64_t rs, cs; } view_t;
#define MAKE_VIEW(T)                                                                                 \
  static T* view_##T(int kind, int64_t r, int64_t c, view_t* v, int ints) {                          \
    int64_t pr = r, pc = c;                                                                          \
    if (kind == 2) pr = 2 * r;                                                                       \
    if (kind == 3) pc = 2 * c;                                                                       \
    if (kind == 6) { pr = r + 3; pc = c + 5; }                                                       \
    if (kind == 1) { pr = c; pc = r; }                                                               \
    if (kind == 7) pr = 1;                                                                           \
    T* p = (T*)malloc((size_t)(pr * pc) * sizeof(T));                                                \
    for (int64_t i = 0; i < pr * pc; ++i) p[i] = ints ? (T)rnd_in(-100, 100) : (T)((double)rnd_in(-1000, 1000) / 1000.0); \
    v->parent = p;                                                                                   \
    switch (kind) {                                                                                  \
      case 0: v->rs = pc; v->cs = 1; return p;                  /* C order */                        \
      case 1: v->rs = 1; v->cs = pc; return p;                  /* transposed */                     \
      case 2: v->rs = 2 * pc; v->cs = 1; return p;              /* every other row */                \
      case 3: v->rs = pc; v->cs = 2; return p;                  /* every other column */             \
      case 4: v->rs = -pc; v->cs = 1; return p + (pr - 1) * pc; /* rows reversed */                  \
      case 5: v->rs = pc; v->cs = -1; return p + (pc - 1);      /* columns reversed */               \
      case 6: v->rs = pc; v->cs = 1; return p + 2 * pc + 1;     /* inner block */                    \
      default: v->rs = 0; v->cs = 1; return p;                  /* one row broadcast */              \
    }                                                                                                \
  }
MAKE_VIEW(float) MAKE_VIEW(double) MAKE_VIEW(int32_t) MAKE_VIEW(int64_t)

#define GEMM_CASE(T, U, SFX, INTS, TOL)                                                              \
  static void gemm_##SFX(int64_t M, int64_t N, int64_t K, int ka, int kb, int kc) {                  \
    view_t va, vb, vc, vr;                                                                           \
    T* A = view_##T(ka, M, K, &va, INTS);                                                            \
    T* B = view_##T(kb, K, N, &vb, INTS);                                                            \
    T* C = view_##T(kc, M, N, &vc, INTS);                                                            \
    T* R = view_##T(0, M, N, &vr, INTS);                                                             \
    const T alpha = INTS ? (T)3 : (T)1.5, beta = (rnd() & 1) ? (T)0 : (INTS ? (T)-2 : (T)0.5);       \
    for (int64_t i = 0; i < M; ++i)                                                                  \
      for (int64_t j = 0; j < N; ++j) {                                                              \
        if (INTS) {                                                                                  \
          U acc = 0;                                                                                 \
          for (int64_t k = 0; k < K; ++k) acc += (U)A[i * va.rs + k * va.cs] * (U)B[k * vb.rs + j * vb.cs]; \
          R[i * N + j] = (T)((U)alpha * acc + (beta == 0 ? (U)0 : (U)beta * (U)C[i * vc.rs + j * vc.cs])); \
        } else {                                                                                     \
          long double acc = 0;                                                                       \
          for (int64_t k = 0; k < K; ++k) acc += (long double)A[i * va.rs + k * va.cs] * B[k * vb.rs + j * vb.cs]; \
          R[i * N + j] = (T)((long double)alpha * acc + (beta == 0 ? 0 : (long double)beta * C[i * vc.rs + j * vc.cs])); \
        }                                                                                            \
      }                                                                                              \
    const int rc = am_oracle_gemm_strided_##SFX(M, N, K, alpha, A, va.rs, va.cs, B, vb.rs, vb.cs, beta, C, vc.rs, vc.cs); \
    EXPECT(rc == 0, "gemm " #SFX " rc=%d", rc);                                                      \
    for (int64_t i = 0; i < M; ++i)                                                                  \
      for (int64_t j = 0; j < N; ++j) {                                                              \
        const T got = C[i * vc.rs + j * vc.cs], want = R[i * N + j];                                 \
        const int ok = INTS ? (got == want) : (fabs((double)got - (double)want) <= TOL * (1.0 + fabs((double)want) + (double)K)); \
        if (!ok) { EXPECT(0, "gemm " #SFX " %lldx%lldx%lld views %d %d %d at (%lld,%lld)", (long long)M, (long long)N, (long long)K, ka, kb, kc, (long long)i, (long long)j); i = M; break; } \
      }                                                                                              \
    free(va.parent); free(vb.parent); free(vc.parent); free(vr.parent);                              \
  }
GEMM_CASE(float, uint32_t, f32, 0, 2e-6)
GEMM_CASE(double, uint64_t, f64, 0, 1e-14)
GEMM_CASE(int32_t, uint32_t, i32, 1, 0)
GEMM_CASE(int64_t, uint64_t, i64, 1, 0)

/* element offset of C-order index `idx` of a tensor with `shape` / `strides` */
static int64_t offset_of(int rank, const int64_t* shape, const int64_t* strides, int64_t idx) {
  int64_t off = 0;
  for (int d = rank - 1; d >= 0; --d) { off += (idx % shape[d]) * strides[d]; idx /= shape[d]; }
  return off;
}

static void map_cases(void) {
  for (int it = 0; it < 300; ++it) {
    const int rank = (int)rnd_in(1, 6);
    int64_t shape[6], sa[6], sb[6], sd[6], n = 1;
    for (int d = 0; d < rank; ++d) { shape[d] = rnd_in(1, (it % 7 == 0 && rank <= 3) ? 40 : 5); n *= shape[d]; }   /* n <= 64000 */
    /* a: C order over a padded parent, some dims reversed; b: broadcast along some dims; dst: C order */
    int64_t pa = 1, pd = 1, first_a = 0;
    for (int d = rank - 1; d >= 0; --d) {
      const int64_t pad = rnd_in(0, 2);
      sa[d] = pa; pa *= shape[d] + pad;
      sd[d] = pd; pd *= shape[d];
    }
    for (int d = 0; d < rank; ++d) if (rnd() % 4 == 0) { first_a += (shape[d] - 1) * sa[d]; sa[d] = -sa[d]; }
    int64_t pb = 1;
    for (int d = rank - 1; d >= 0; --d) { if (rnd() % 3 == 0) sb[d] = 0; else { sb[d] = pb; pb *= shape[d]; } }
    int64_t* A = (int64_t*)malloc((size_t)pa * 8); int64_t* B = (int64_t*)malloc((size_t)pb * 8);
    int64_t* D = (int64_t*)malloc((size_t)pd * 8); uint8_t* Q = (uint8_t*)malloc((size_t)pd);
    double* Af = (double*)malloc((size_t)pa * 8); double* Bf = (double*)malloc((size_t)pb * 8); double* Df = (double*)malloc((size_t)pd * 8);
    for (int64_t i = 0; i < pa; ++i) { A[i] = rnd_in(-9, 9); Af[i] = (double)A[i] / 4; }
    for (int64_t i = 0; i < pb; ++i) { B[i] = rnd_in(-9, 9); if (B[i] == 0) B[i] = 3; Bf[i] = (double)B[i] / 4; }
    const int ops[] = {0, 1, 2, 3, 4, 9, 10, 15};
    for (unsigned o = 0; o < sizeof(ops) / sizeof(ops[0]); ++o) {
      EXPECT(am_oracle_map2_i64(ops[o], rank, shape, D, sd, A + first_a, sa, B, sb) == 0, "map2 i64 op %d", ops[o]);
      for (int64_t i = 0; i < n; ++i) {
        const int64_t x = A[first_a + offset_of(rank, shape, sa, i)], y = B[offset_of(rank, shape, sb, i)];
        int64_t w = 0;
        switch (ops[o]) {
          case 0: w = x + y; break; case 1: w = x - y; break; case 2: w = x * y; break; case 3: w = x / y; break;
          case 4: w = x % y; break; case 9: w = x > y ? x : y; break; case 10: w = x < y ? x : y; break;
          default: w = x % y; if ((w > 0 && y < 0) || (w < 0 && y > 0)) w += y; break;
        }
        if (D[offset_of(rank, shape, sd, i)] != w) { EXPECT(0, "map2 i64 op %d rank %d element %lld", ops[o], rank, (long long)i); break; }
      }
    }
    EXPECT(am_oracle_map2_f64(0, rank, shape, Df, sd, Af + first_a, sa, Bf, sb) == 0, "map2 f64 add");
    for (int64_t i = 0; i < n; ++i)
      if (Df[offset_of(rank, shape, sd, i)] != Af[first_a + offset_of(rank, shape, sa, i)] + Bf[offset_of(rank, shape, sb, i)]) { EXPECT(0, "map2 f64 add rank %d", rank); break; }
    for (int cmp = 0; cmp < 7; ++cmp) {
      EXPECT(am_oracle_compare_i64(cmp, rank, shape, Q, sd, A + first_a, sa, B, sb) == 0, "compare %d", cmp);
      for (int64_t i = 0; i < n; ++i) {
        const int64_t x = A[first_a + offset_of(rank, shape, sa, i)], y = B[offset_of(rank, shape, sb, i)];
        const int w = cmp == 0 ? x == y : cmp == 1 ? x != y : cmp == 2 ? x < y : cmp == 3 ? x <= y : cmp == 4 ? x > y : cmp == 5 ? x >= y : (x % y == 0);
        if (Q[offset_of(rank, shape, sd, i)] != (uint8_t)w) { EXPECT(0, "compare %d rank %d element %lld", cmp, rank, (long long)i); break; }
      }
    }
    /* sum along a random axis against the direct double loop */
    const int axis = (int)rnd_in(0, rank - 1);
    int64_t rshape[6], rs[6], rp = 1;
    for (int d = rank - 1; d >= 0; --d) { rshape[d] = d == axis ? 1 : shape[d]; rs[d] = rp; rp *= rshape[d]; }
    int64_t* Rd = (int64_t*)malloc((size_t)rp * 8);
    EXPECT(am_oracle_reduce_axis_i64(0, rank, shape, axis, Rd, rs, A + first_a, sa) == 0, "reduce_axis");
    for (int64_t o = 0; o < rp; ++o) {
      int64_t coord[6], rem = o, want = 0;
      for (int d = rank - 1; d >= 0; --d) { coord[d] = rem % rshape[d]; rem /= rshape[d]; }
      for (int64_t k = 0; k < shape[axis]; ++k) {
        int64_t off = first_a;
        for (int d = 0; d < rank; ++d) off += (d == axis ? k : coord[d]) * sa[d];
        want += A[off];
      }
      if (Rd[o] != want) { EXPECT(0, "reduce_axis rank %d axis %d output %lld", rank, axis, (long long)o); break; }
    }
    free(A); free(B); free(D); free(Q); free(Af); free(Bf); free(Df); free(Rd);
  }
}

int main(void) {
  /* tile edges of the blocked kernel: MR = 6, NR = 16 / 8 / 4, mc = 192 / 96, kc = 512 / 256 */
  const int64_t ms[] = {1, 5, 6, 7, 13, 97, 193}, ns[] = {1, 3, 4, 5, 15, 16, 17, 33}, ks[] = {1, 2, 255, 256, 257, 513};
  int cases = 0;
  for (unsigned a = 0; a < sizeof(ms) / sizeof(ms[0]); ++a)
    for (unsigned b = 0; b < sizeof(ns) / sizeof(ns[0]); ++b)
      for (unsigned c = 0; c < sizeof(ks) / sizeof(ks[0]); ++c) {
        const int ka = (int)rnd_in(0, 7), kb = (int)rnd_in(0, 7), kc = (int)rnd_in(0, 6);   /* C: no broadcast */
        switch ((a + b + c) & 3) {
          case 0: gemm_f32(ms[a], ns[b], ks[c], ka, kb, kc); break;
          case 1: gemm_f64(ms[a], ns[b], ks[c], ka, kb, kc); break;
          case 2: gemm_i32(ms[a], ns[b], ks[c], ka, kb, kc); break;
          default: gemm_i64(ms[a], ns[b], ks[c], ka, kb, kc); break;
        }
        ++cases;
      }
  gemm_i32(200, 130, 600, 1, 3, 0);   /* several M blocks and K panels, OpenMP split */
  gemm_f64(130, 70, 300, 4, 5, 1);
  map_cases();
  printf("%d gemm cases + 300 map / compare / reduce cases, %d mismatches\n", cases + 2, failures);
  return failures ? 1 : 0;
}
