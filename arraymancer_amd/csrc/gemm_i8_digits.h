// Exact int32 and int64 GEMM on the int8 matrix cores of gfx950 by digit slicing.
//
// An int32 is written in four balanced base-256 digits, x = d0 + 2^8 d1 + 2^16 d2 + 2^24 d3 (mod 2^32),
// each d in [-128, 127]. Modulo 2^32 the product of two such numbers only needs the ten digit pairs
// with i + j <= 3, so
//     A * B  =  sum_{s=0..3} 2^(8s) * sum_{i+j=s} A_i * B_j          (mod 2^32)
// where every A_i * B_j is an int8 x int8 -> int32 matrix product, which v_mfma_i32_32x32x32_i8
// computes exactly; its accumulator wraps modulo 2^32, and a wrapped partial sum shifted left by 8s
// is still right modulo 2^32. Ring arithmetic: the result has the same bits as the wrapping VALU
// kernel and as the reference's integer micro-kernels
// (src/arraymancer/laser/primitives/matrix_multiplication/gemm_ukernel_avx2.nim:15-16), whatever
// the order of the additions. Ten int8 products cost 10 x 2MNK int8 operations at 5 POP/s of matrix
// throughput against 2MNK multiply-adds at the 61 Top/s the vector ALU sustains.
//
// Three passes:
//   split_digits<first>   reads both operands (any strided view), marks the digit planes that hold a
//                  non-zero digit anywhere and writes plane 0 of each: int8 planes with rows padded to
//                  the tile size and k to the slab size with zeros, stored as 1 KiB blocks of 32 rows x
//                  32 k in the register layout of the matrix instruction (a 32 x 128 tile goes through
//                  LDS so that both the strided read and the block write are coalesced);
//   split_digits<second>  writes the marked planes above plane 0. Entries within +-127 have none (the
//                  pass leaves at once, the operands were read only once, one pair instead of ten runs);
//   gemm_i8_digits one workgroup of eight wavefronts per 256 x 256 (or 256 x 128) tile of C. For
//                  s = 3..0 it walks the pairs (i, s - i) whose planes are not empty and the k slabs
//                  of each pair as one long k loop: blocks go from global memory straight into an
//                  LDS ring (global_load_lds_dwordx4, no register stage, no LDS write instructions),
//                  several slabs ahead; fragments are double-buffered in registers. Between two
//                  values of s the accumulators are shifted left by 8 (Horner form of the sum over
//                  s). Padded planes mean no bounds tests in the loop. Of 72 us for one pair at
//                  4096^3, 31 are the matrix instructions, 10 the store of C, 15 the operand fetch
//                  from L2 that the prefetch does not hide, the rest fragment reads and barriers.
//
// int64 works the same way with eight digits and the 36 pairs i + j <= 7. The matrix cores
// accumulate in 32 bits, which holds one pair's sum over k exactly while k * 2^14 < 2^31; after each
// pair the 32-bit accumulators are sign-extended into a 64-bit set, which takes the Horner shifts.
#pragma once
#include <type_traits>
#include "gemm_common.h"

extern "C" int am_hip_malloc(size_t bytes, void** out);
extern "C" int am_hip_free(void* dptr);

namespace am {
namespace gemm {
namespace i8 {

constexpr int kKPad = 256;     // operand planes are padded to a multiple of the workgroup tile in rows and to this many k
                               // (a whole turn of the LDS ring: four slabs of 64)

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

// All balanced base-256 digits of x at once, one per byte: digit d is ((x + 128 (1 + 2^8 + .. + 2^(8d))) >> 8d)
// mod 256 - 128 (the carry of "x - digit" into the next byte is that of adding 128 to it), and adding
// the higher bytes of the constant does not reach byte d; subtracting 128 from a byte is flipping its top bit.
template <typename T>
__device__ __forceinline__ std::make_unsigned_t<T> balanced_digits(T x) {
  using U = std::make_unsigned_t<T>;
  constexpr U C = (U)0x8080808080808080ull;
  return ((U)x + C) ^ C;
}

// The digits of four neighbouring k, packed as one 32-bit word per plane (a 4 x 4 byte transpose per
// 32 bits of element width; v_perm_b32 picks bytes 0-3 from its second and 4-7 from its first operand).
template <typename T>
__device__ __forceinline__ void digits_of4(const T (&x)[4], uint32_t (&w)[sizeof(T)]) {
  using U = std::make_unsigned_t<T>;
  U y[4];
#pragma unroll
  for (int e = 0; e < 4; ++e) y[e] = balanced_digits<T>(x[e]);
#pragma unroll
  for (int h = 0; h < (int)sizeof(T) / 4; ++h) {
    uint32_t v[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) v[e] = (uint32_t)(y[e] >> (h * 32 % (8 * (int)sizeof(T))));
    const uint32_t a = __builtin_amdgcn_perm(v[1], v[0], 0x05010400u), b = __builtin_amdgcn_perm(v[1], v[0], 0x07030602u);
    const uint32_t c = __builtin_amdgcn_perm(v[3], v[2], 0x05010400u), d = __builtin_amdgcn_perm(v[3], v[2], 0x07030602u);
    w[4 * h + 0] = __builtin_amdgcn_perm(c, a, 0x05040100u);
    w[4 * h + 1] = __builtin_amdgcn_perm(c, a, 0x07060302u);
    w[4 * h + 2] = __builtin_amdgcn_perm(d, b, 0x05040100u);
    w[4 * h + 3] = __builtin_amdgcn_perm(d, b, 0x07060302u);
  }
}

// Both operands of one product, as the two splitting passes see them: X(mn, k) = X[mn * ld_mn + k * ld_k],
// planes P[d][mn][k] (mn < MNp, k < Kp). flags[op * ND + d] == gen says that plane d of operand op
// holds a non-zero digit somewhere; gen is a number that grows with every product, so the flags of
// earlier products read as unset and the flag words never need clearing.
template <typename T>
struct SplitArgs {
  const T* X[2];
  int64_t ld_mn[2], ld_k[2], MN[2], MNp[2];
  int kfast[2];
  int mode[2];      // 0: element loads; 1 / 2: 16-byte loads along k / along mn (unit stride there, 16-byte aligned lines)
  int8_t* P[2];
  int64_t K, Kp;
  uint32_t* flags;
  uint32_t gen;
  int max_pairs;    // the second splitting pass writes nothing when more digit pairs than this are live (the product then runs elsewhere)
};

// The 32 (mn) x 128 (k) tile at (mn0, k0) of operand op, 16 elements per lane of a 256-lane workgroup:
// every load is issued before f(mn, k, value) sees the first element (zeros outside the operand).
template <typename T, bool STREAM, typename F>
__device__ __forceinline__ void visit_tile(const SplitArgs<T>& a, int op, int64_t mn0, int64_t k0, F&& f) {
  constexpr int VEC = 16 / (int)sizeof(T);
  typedef T vec_t __attribute__((ext_vector_type(VEC)));
  const T* X = a.X[op];
  const int64_t ld_mn = a.ld_mn[op], ld_k = a.ld_k[op], MN = a.MN[op], K = a.K;
  const int mode = a.mode[op];
  const int t = (int)threadIdx.x;
  if (mode == 1) {
    constexpr int KV = 128 / VEC, ROWS = 256 / KV, PASSES = 32 / ROWS;
    vec_t v[PASSES];
    const int k = (t % KV) * VEC;
#pragma unroll
    for (int i = 0; i < PASSES; ++i) {
      const int mn = t / KV + i * ROWS;
      const T* src = X + (mn0 + mn) * ld_mn + (k0 + k);
      if ((mn0 + mn) < MN && (k0 + k + VEC) <= K) {
        if constexpr (STREAM) v[i] = __builtin_nontemporal_load((const vec_t*)src); else v[i] = *(const vec_t*)src;
      } else {
#pragma unroll
        for (int e = 0; e < VEC; ++e) v[i][e] = ((mn0 + mn) < MN && (k0 + k + e) < K) ? src[e] : (T)0;
      }
    }
#pragma unroll
    for (int i = 0; i < PASSES; ++i)
#pragma unroll
      for (int e = 0; e < VEC; ++e) f(t / KV + i * ROWS, k + e, v[i][e]);
  } else if (mode == 2) {
    constexpr int MV = 32 / VEC, ROWS = 256 / MV, PASSES = 128 / ROWS;
    vec_t v[PASSES];
    const int mn = (t % MV) * VEC;
#pragma unroll
    for (int i = 0; i < PASSES; ++i) {
      const int k = t / MV + i * ROWS;
      const T* src = X + (mn0 + mn) + (k0 + k) * ld_k;
      if ((k0 + k) < K && (mn0 + mn + VEC) <= MN) {
        if constexpr (STREAM) v[i] = __builtin_nontemporal_load((const vec_t*)src); else v[i] = *(const vec_t*)src;
      } else {
#pragma unroll
        for (int e = 0; e < VEC; ++e) v[i][e] = ((k0 + k) < K && (mn0 + mn + e) < MN) ? src[e] : (T)0;
      }
    }
#pragma unroll
    for (int i = 0; i < PASSES; ++i)
#pragma unroll
      for (int e = 0; e < VEC; ++e) f(mn + e, t / MV + i * ROWS, v[i][e]);
  } else {
    const int kfast = a.kfast[op];
    T x[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int e = t + i * 256;
      int mn, k;
      if (kfast) { k = e & 127; mn = e >> 7; } else { mn = e & 31; k = e >> 5; }
      const bool ok = (mn0 + mn) < MN && (k0 + k) < K;
      x[i] = ok ? X[(mn0 + mn) * ld_mn + (k0 + k) * ld_k] : (T)0;
    }
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int e = t + i * 256;
      int mn, k;
      if (kfast) { k = e & 127; mn = e >> 7; } else { mn = e & 31; k = e >> 5; }
      f(mn, k, x[i]);
    }
  }
}

// The two splitting passes. A workgroup moves one 32 (mn) x 128 (k) tile of an operand at a time through
// LDS: the read walks whichever of the two directions is the faster one in memory, the write is
// 16 bytes per lane and plane into the 1 KiB blocks the product kernel wants (32 rows x 32 k in the
// register layout of the matrix instruction: lane (row % 32) + 32 * ((k % 32) / 16) owns 16 consecutive k).
//   FIRST = true : marks the digit planes that hold anything (flags) and writes plane 0, which
//                  practically every operand needs. Operands with entries within +-127 need nothing else:
//                  the second pass then leaves at once and the operand has been read only once.
//   FIRST = false: writes the marked planes above plane 0 (nothing if there is none, or if the product
//                  has more live digit pairs than max_pairs and therefore runs on the vector ALU).
template <typename T, bool FIRST, bool STREAM_LOADS = false>
__global__ __launch_bounds__(256) void split_digits(SplitArgs<T> a) {
  typedef uint32_t u4 __attribute__((ext_vector_type(4)));
  constexpr int ND = (int)sizeof(T);
  using U = std::make_unsigned_t<T>;
  // the tile in LDS: whole elements for the second pass, only their lowest digit for the first (rows stay 16-byte aligned)
  typedef std::conditional_t<FIRST, int8_t, T> tile_t;
  __shared__ __attribute__((aligned(16))) tile_t tile[32][128 + 16 / sizeof(tile_t)];
  bool live[2][ND];   // second pass: which planes were marked (one round trip for all the flag words)
  bool any_high[2] = {false, false};
  if constexpr (!FIRST) {
    uint32_t fl[2 * ND];
#pragma unroll
    for (int i = 0; i < 2 * ND; ++i) fl[i] = a.flags[i];
    int pairs = 0, live_b = 0;
#pragma unroll
    for (int i = ND - 1; i >= 0; --i) {
      live_b += fl[ND + (ND - 1 - i)] == a.gen ? 1 : 0;
      pairs += fl[i] == a.gen ? live_b : 0;
    }
#pragma unroll
    for (int o = 0; o < 2; ++o)
#pragma unroll
      for (int d = 0; d < ND; ++d) {
        live[o][d] = fl[o * ND + d] == a.gen;
        if (d > 0) any_high[o] |= live[o][d];
      }
    if (pairs > a.max_pairs || !(any_high[0] || any_high[1])) return;
  }
  // a few workgroups per CU walk the tiles of both operands (a second pass with nothing to do ends quickly)
  const int64_t kt = a.Kp >> 7, t0 = (a.MNp[0] >> 5) * kt, t1 = (a.MNp[1] >> 5) * kt;
  for (int64_t t = blockIdx.x; t < t0 + t1; t += gridDim.x) {
  const int op = t < t0 ? 0 : 1;
  const int64_t tt = t - (op ? t0 : 0);
  const int64_t mn0 = (tt / kt) * 32, k0 = (tt % kt) * 128;
  const int64_t MNp = a.MNp[op];
  uint32_t* flags = a.flags + op * ND;
  if constexpr (!FIRST) {
    if (!any_high[op]) {   // nothing above plane 0 in this operand: go to the other one, or leave
      if (op == 1) return;
      t += (t0 - 1 - tt) / gridDim.x * gridDim.x;   // the last tile of this workgroup's walk that is still in operand 0
      continue;
    }
  }
  U seen = 0;   // byte d: OR of the digits d of this lane's elements
  visit_tile<T, FIRST && STREAM_LOADS>(a, op, mn0, k0, [&](int mn, int k, T x) {
    if constexpr (FIRST) {
      const U y = balanced_digits<T>(x);
      seen |= y;
      tile[mn][k] = (int8_t)(y & 0xFFu);
    } else {
      tile[mn][k] = x;
    }
  });
  if constexpr (FIRST) {
#pragma unroll
    for (int d = 0; d < ND; ++d) {   // every writer stores the same value; at most one store per wavefront and plane
      const bool nz = ((uint32_t)(seen >> (8 * d)) & 0xFFu) != 0;
      if (__ballot(nz) != 0 && (threadIdx.x & 63) == 0 && flags[d] != a.gen) flags[d] = a.gen;
    }
  }
  __syncthreads();
  const int64_t plane = MNp * a.Kp;
  const int k16 = threadIdx.x & 7, mn = threadIdx.x >> 3;
  int8_t* dst = a.P[op] + ((((mn0 >> 5) * (a.Kp >> 5) + (k0 >> 5) + (k16 >> 1)) * 64 + (k16 & 1) * 32 + mn) << 4);
  if constexpr (FIRST) {
    *(u4*)dst = *(const u4*)&tile[mn][k16 * 16];
  } else {
    u4 out[ND];
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const T xs[4] = {tile[mn][k16 * 16 + g * 4], tile[mn][k16 * 16 + g * 4 + 1], tile[mn][k16 * 16 + g * 4 + 2],
                       tile[mn][k16 * 16 + g * 4 + 3]};
      uint32_t w[ND];   // one 4-byte word (4 consecutive k) per digit plane
      digits_of4<T>(xs, w);
#pragma unroll
      for (int d = 0; d < ND; ++d) out[d][g] = w[d];
    }
#pragma unroll
    for (int d = 1; d < ND; ++d)
      if (op == 0 ? live[0][d] : live[1][d]) *(u4*)(dst + d * plane) = out[d];
  }
  __syncthreads();   // the tile buffer is reused
  }
}

template <typename T>
struct DigitArgs {
  const int8_t* PA; const int8_t* PB;   // ND = sizeof(T) digit planes each, in 1 KiB fragment blocks [rows/32][Kp/32][64 lanes][16]
  const uint32_t* flags;                // [0..ND-1]: planes of A, [ND..2ND-1]: planes of B; == gen: not all zero
  uint32_t gen;
  int max_pairs;                        // the kernel leaves at once when more digit pairs than this are live
  int64_t Mp, Np, Kp;
  T* C; int64_t c_m, c_n;
  int64_t M, N;
  T alpha, beta;
  int tiles_m, tiles_n;
  long long* clock_out;                 // see ClockProbe (common.h)
  int preset_a, preset_b;               // >= 0: bit d set = plane d of that operand is live (planes split ahead of time,
                                        // Prepared below); < 0: read the flag words
};

// WAVES_M x WAVES_N wavefronts, each with TM x TN accumulator tiles of 32 x 32; BK k (bytes) per slab.
// The digit sums are evaluated in Horner form, the highest s first: after the pairs of one s the
// accumulators are shifted left by 8 and go on accumulating the pairs of s - 1, so one accumulator set
// suffices (int32: everything modulo 2^32, which both the shift and the matrix cores respect; int64:
// the 32-bit accumulators of one pair are exact and are added into 64-bit ones when the pair ends).
template <typename T, int WAVES_M, int WAVES_N, int TM, int TN, int BK, int RING>
__global__ __launch_bounds__(WAVES_M* WAVES_N * 64, 1) void gemm_i8_digits(DigitArgs<T> p) {
  using U = std::make_unsigned_t<T>;
  const ClockProbe probe(p.clock_out);
  constexpr int ND = (int)sizeof(T), NPAIRS = ND * (ND + 1) / 2;
  constexpr bool WIDE = sizeof(T) == 8;
  constexpr int NT = WAVES_M * WAVES_N * 64;
  constexpr int WM = TM * 32, WN = TN * 32, BM = WAVES_M * WM, BN = WAVES_N * WN, NKS = BK / 32, QN = BK / 16;
  // One slab = NKS k-steps of 32; its blocks in LDS: A's (BM / 32) x NKS, then B's (BN / 32) x NKS, 1 KiB each.
  constexpr int NW = WAVES_M * WAVES_N, NBA = BM / 32 * NKS, NBB = BN / 32 * NKS;
  constexpr int LPA = NBA / NW, LPB = NBB / NW;            // block loads per wavefront and slab
  constexpr int SLAB = (NBA + NBB) * 1024;   // RING slabs in LDS: the one being multiplied and RING - 1 on their way
  static_assert(NKS % 2 == 0 && NBA % NW == 0 && NBB % NW == 0 && QN > 0 && RING >= 3 && (RING - 2) * (LPA + LPB) <= 15, "tile shape");
  __shared__ __attribute__((aligned(1024))) int8_t sbuf[RING][SLAB];

  int tile_m, tile_n;
  tile_of_block((int)blockIdx.x, p.tiles_m, p.tiles_n, tile_m, tile_n);
  const int64_t m0 = (int64_t)tile_m * BM, n0 = (int64_t)tile_n * BN;
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int wave_m = wave / WAVES_N, wave_n = wave % WAVES_N;
  const int lrow = lane & 31, kg = lane >> 5;

  // global -> LDS without registers: a wavefront's load instruction moves one block, lane l's 16 bytes to
  // LDS offset 16 l of the block. Wavefront w takes blocks w, w + NW, ... of each operand.
  const int64_t planeA = p.Mp * p.Kp, planeB = p.Np * p.Kp;
  const int64_t kb32 = p.Kp >> 5;
  const int8_t* ga[LPA]; const int8_t* gb[LPB];
  int lds_a[LPA], lds_b[LPB];
#pragma unroll
  for (int i = 0; i < LPA; ++i) {
    const int b = wave + i * NW;
    ga[i] = p.PA + ((((m0 >> 5) + b / NKS) * kb32 + b % NKS) << 10) + lane * 16;
    lds_a[i] = b * 1024;
  }
#pragma unroll
  for (int i = 0; i < LPB; ++i) {
    const int b = wave + i * NW;
    gb[i] = p.PB + ((((n0 >> 5) + b / NKS) * kb32 + b % NKS) << 10) + lane * 16;
    lds_b[i] = (NBA + b) * 1024;
  }
  // The digit pairs to multiply: (s, i) with i + j = s <= ND - 1, the highest s first, restricted to planes
  // that hold something. tab_shift[pr] = how far the accumulators move left before pair pr (the
  // Horner steps between its s and the previous pair's), tab_shift[n_pairs] = the final shift.
  __shared__ int tab_a[NPAIRS], tab_b[NPAIRS], tab_shift[NPAIRS + 1], tab_n;
  if (threadIdx.x == 0) {
    int n = 0, prev_s = -1;
    for (int s = ND - 1; s >= 0; --s)
      for (int i = 0; i <= s; ++i)
        if ((p.preset_a >= 0 ? ((p.preset_a >> i) & 1) != 0 : p.flags[i] == p.gen) &&
            (p.preset_b >= 0 ? ((p.preset_b >> (s - i)) & 1) != 0 : p.flags[ND + s - i] == p.gen)) {
          tab_a[n] = i; tab_b[n] = s - i;
          tab_shift[n] = prev_s < 0 ? 0 : 8 * (prev_s - s);
          prev_s = s;
          ++n;
        }
    tab_shift[n] = prev_s < 0 ? 0 : 8 * prev_s;
    tab_n = n;
  }
  __syncthreads();
  const int n_pairs = tab_n;
  if (n_pairs > p.max_pairs) return;   // uniform: the vector-ALU kernel launched behind this one takes the product
  const int64_t slabs_per_pair = p.Kp / BK;
  const int64_t total = (int64_t)n_pairs * slabs_per_pair;
  // Slabs are fetched in order, RING - 1 ahead of the one being multiplied; (f_oa, f_ob) + f_k are the
  // offsets of the next one's A and B blocks. Fetches past the last slab re-read it (never multiplied).
  int f_pr = 0;
  int64_t f_k = 0;   // in bytes of a block row: 1024 per k-step of 32
  int64_t f_oa = n_pairs > 0 ? tab_a[0] * planeA : 0, f_ob = n_pairs > 0 ? tab_b[0] * planeB : 0;
  // The load is written as inline assembly: the compiler's own wait-count pass would otherwise drain
  // every outstanding load (vmcnt(0)) before the next LDS read, which undoes the prefetch. The waits
  // that order these loads before the reads of their slab are the explicit s_waitcnt before each barrier.
  const uint32_t lds0 = (uint32_t)reinterpret_cast<uintptr_t>(&sbuf[0][0]);
  auto block_to_lds = [&](const int8_t* src, int lds_off) {
    const uint32_t m0 = __builtin_amdgcn_readfirstlane(lds0 + (uint32_t)lds_off);
    asm volatile("s_mov_b32 m0, %1\n\tglobal_load_lds_dwordx4 %0, off" : : "v"(src), "s"(m0) : "memory", "m0");
  };
  auto fetch = [&](int buf) {
#pragma unroll
    for (int i = 0; i < LPA; ++i) block_to_lds(ga[i] + f_oa + f_k, buf * SLAB + lds_a[i]);
#pragma unroll
    for (int i = 0; i < LPB; ++i) block_to_lds(gb[i] + f_ob + f_k, buf * SLAB + lds_b[i]);
    f_k += NKS * 1024;
    if (f_k == (kb32 << 10)) {
      if (f_pr + 1 < n_pairs) {
        ++f_pr;
        f_k = 0;
        f_oa = tab_a[f_pr] * planeA;
        f_ob = tab_b[f_pr] * planeB;
      } else {
        f_k -= NKS * 1024;
      }
    }
  };
  v4i af[2][TM], bf[2][TN];
  auto read_frags = [&](auto parity_tag, int buf, int ks) {
    constexpr int P = decltype(parity_tag)::value;
#pragma unroll
    for (int i = 0; i < TM; ++i) af[P][i] = *(const v4i*)(sbuf[buf] + (((wave_m * TM + i) * NKS + ks) << 10) + lane * 16);
#pragma unroll
    for (int j = 0; j < TN; ++j) bf[P][j] = *(const v4i*)(sbuf[buf] + ((NBA + (wave_n * TN + j) * NKS + ks) << 10) + lane * 16);
  };

  v16i acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0;

  uint64_t wide[WIDE ? TM : 1][WIDE ? TN : 1][WIDE ? 16 : 1];
  if constexpr (WIDE) {
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r) wide[i][j][r] = 0;
  }
  // End of a pair: int64 moves the pair's exact 32-bit sums into the 64-bit accumulators; then the
  // Horner shift (0 when the next pair has the same s).
  auto end_pair = [&](int sh) {
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          if constexpr (WIDE) {
            wide[i][j][r] = (wide[i][j][r] + (uint64_t)(int64_t)acc[i][j][r]) << sh;
            acc[i][j][r] = 0;
          } else {
            acc[i][j][r] = (int)((uint32_t)acc[i][j][r] << sh);
          }
        }
  };

  if (total > 0) {   // (every plane of an operand empty: the product is zero)
  // prologue: slabs 0 and 1 on their way into LDS; slab 0 must have landed
#pragma unroll
  for (int r = 0; r < RING - 1; ++r) fetch(r);
  __builtin_amdgcn_s_waitcnt(0x0F70 | ((RING - 2) * (LPA + LPB)));   // all but the loads of the later slabs: slab 0 is in
  __syncthreads();
  read_frags(std::integral_constant<int, 0>(), 0, 0);

  // One inner loop per pair keeps the end-of-pair arithmetic out of the slab loop's body (as a
  // branch inside one flat loop the compiler turns it into selects executed for every slab). The
  // planes are padded to a whole number of turns of the ring per pair, so the loop can be unrolled over
  // the ring: the ring position is then a compile-time constant and every LDS address a constant offset
  // (the lambda below). That pays for the 256 x 128 tile (int64: 96 -> 90 us per pair at 4096^3); the
  // 256 x 256 tile is faster with the rolled loop further down (69 against 74 us), the same steps with the
  // position in `cur`.
  int cur = 0;   // ring position of the slab being multiplied (rolled loop)
  auto slab = [&](auto cur_tag) {
    constexpr int CUR = decltype(cur_tag)::value;
    constexpr int NXT = CUR == RING - 1 ? 0 : CUR + 1, LAST = CUR == 0 ? RING - 1 : CUR - 1;
    fetch(LAST);   // slab t + RING - 1; its buffer held slab t - 1, which every wavefront left before the last barrier
#pragma unroll
    for (int ks = 0; ks < NKS; ++ks) {
      if (ks + 1 < NKS) {
        if (ks & 1) read_frags(std::integral_constant<int, 0>(), CUR, ks + 1);
        else read_frags(std::integral_constant<int, 1>(), CUR, ks + 1);
      } else {
        // Slab t + 1 was requested RING - 2 slabs ago: wait for this wavefront's part of it (vmcnt <= the
        // loads of the later slabs) and for its own outstanding reads of slab t (lgkmcnt 0: the matrix
        // instructions below need them anyway), then for everyone's. A bare barrier: the fence of
        // __syncthreads would drain the later slabs' loads as well.
        __builtin_amdgcn_s_waitcnt(0x0070 | ((RING - 2) * (LPA + LPB)));
        __builtin_amdgcn_s_barrier();
        read_frags(std::integral_constant<int, 0>(), NXT, 0);   // NKS is even
      }
      // the fragment reads above are for the next k-step: they are spread between this step's matrix
      // instructions (a wavefront issues in order; in front of them they would only delay them)
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[ks & 1][i], bf[ks & 1][j], acc[i][j], 0, 0, 0);
#pragma unroll
      for (int m = 0; m < TM * TN; ++m) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);   // one matrix instruction
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);   // one LDS read
        __builtin_amdgcn_sched_group_barrier(0x006, 4, 0);   // address arithmetic
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  static_assert(RING == 4, "the slab loop below is written out for a ring of four");
  constexpr bool UNROLL_RING = BM * BN < 256 * 256;
  for (int pr = 0; pr < n_pairs; ++pr) {
    if constexpr (UNROLL_RING) {
      for (int64_t t = 0; t < slabs_per_pair; t += RING) {   // slabs_per_pair is a multiple of RING (kKPad)
        slab(std::integral_constant<int, 0>());
        slab(std::integral_constant<int, 1>());
        slab(std::integral_constant<int, 2>());
        slab(std::integral_constant<int, 3>());
      }
    } else {
      for (int64_t t = 0; t < slabs_per_pair; ++t) {
        const int nxt = cur == RING - 1 ? 0 : cur + 1, last = cur == 0 ? RING - 1 : cur - 1;
        fetch(last);
#pragma unroll
        for (int ks = 0; ks < NKS; ++ks) {
          if (ks + 1 < NKS) {
            if (ks & 1) read_frags(std::integral_constant<int, 0>(), cur, ks + 1);
            else read_frags(std::integral_constant<int, 1>(), cur, ks + 1);
          } else {
            __builtin_amdgcn_s_waitcnt(0x0070 | ((RING - 2) * (LPA + LPB)));
            __builtin_amdgcn_s_barrier();
            read_frags(std::integral_constant<int, 0>(), nxt, 0);
          }
#pragma unroll
          for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j)
              acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[ks & 1][i], bf[ks & 1][j], acc[i][j], 0, 0, 0);
#pragma unroll
          for (int m = 0; m < TM * TN; ++m) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x006, 4, 0);
          }
          __builtin_amdgcn_sched_barrier(0);
        }
        cur = nxt;
      }
    }
    // the pair is done: Horner step(s) down to the next pair's s (or to s = 0 after the last one)
    const int sh = tab_shift[pr + 1];
    if (WIDE || sh != 0) end_pair(sh);
  }
  }

  // C <- alpha * AB + beta * C in the ring of integers modulo 2^32 / 2^64 (same case analysis as the other kernels)
  const U alpha = (U)p.alpha, beta = (U)p.beta;
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const int64_t col = n0 + wave_n * WN + j * 32 + lrow;
      U cv[16];
      if (beta != 0) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int64_t row = m0 + wave_m * WM + i * 32 + 8 * (r >> 2) + 4 * kg + (r & 3);
          cv[r] = (row < p.M && col < p.N) ? (U)p.C[row * p.c_m + col * p.c_n] : (U)0;
        }
      }
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int64_t row = m0 + wave_m * WM + i * 32 + 8 * (r >> 2) + 4 * kg + (r & 3);
        if (row < p.M && col < p.N) {
          U v;
          if constexpr (WIDE) v = alpha * (U)wide[i][j][r];
          else v = alpha * (U)(uint32_t)acc[i][j][r];
          if (beta != 0) v += beta * cv[r];
          p.C[row * p.c_m + col * p.c_n] = (T)v;
        }
      }
    }
  probe.finish();
}

// Padded operand extents and the estimated time of the digit-sliced product for both tile shapes
// (rounds of one workgroup per CU x measured time per tile and k, plus the two splitting passes).
// The estimate is for operands that use every digit; the kernel itself skips empty planes.
// Estimated times of the digit path in microseconds: the two splitting passes, the product kernel with
// every digit pair live (main_us, of which fixed_us do not depend on the number of pairs), and their sum.
struct Plan { int64_t Mp, Np, Kp; int tile; double est_us, main_us, fixed_us, first_us, second_us; };

// Workgroup tiles of the product kernel: 256 x 128 (8 wavefronts of 64 x 64), 256 x 256 (8 of 128 x 64: fewest LDS
// reads per matrix instruction; int32 only, the 64-bit accumulators of int64 leave no registers for it), 128 x 128
// (8 of 64 x 32) and 64 x 64 (4 of 32 x 32) for products that the large tiles spread over a fraction of the chip.
constexpr int kTileCount = 4;
constexpr int kTileRows[kTileCount] = {256, 256, 128, 64}, kTileCols[kTileCount] = {128, 256, 128, 64};
static inline const char* tile_name(int t) { static const char* n[kTileCount] = {"256x128", "256x256", "128x128", "64x64"}; return n[t]; }

// Microseconds per k (all digit pairs live) of the product kernel for `tiles` workgroup tiles, fitted to kernel times
// (rocprofv3) at 512^3 ... 4096^3. `slots` workgroups of a tile shape share a CU (LDS: 128 / 64 / 32 KiB per workgroup
// for the two large, the 128 x 128 and the 64 x 64 tile). Whole rounds of slots x CUs tiles take c_full each. A last,
// partial round of r tiles: up to one per CU a tile's time grows with the share of the chip that is busy (the tiles
// compete for L2 and fabric bandwidth), c0 (1 + a (r / CUs)^2); from there to a whole round it grows linearly to c_full.
struct TileFit { double c0, a, c_full; int slots; };
static inline TileFit tile_fit(int tile, bool wide) {
  //                                           256 x 128                256 x 256               128 x 128                64 x 64
  static const TileFit i32[kTileCount] = {{0.048, 0.58, 0.076, 1}, {0.090, 0.34, 0.121, 1}, {0.029, 0.31, 0.0755, 2}, {0.0215, 0.0, 0.059, 4}};
  static const TileFit i64[kTileCount] = {{0.205, 0.42, 0.291, 1}, {0.0, 0.0, 0.0, 1}, {0.118, 0.30, 0.296, 2}, {0.083, 0.0, 0.231, 4}};
  return wide ? i64[tile] : i32[tile];
}
static inline double main_us_per_k(int tile, bool wide, int64_t tiles, int64_t cus) {
  const TileFit f = tile_fit(tile, wide);
  const int64_t round = cus * f.slots, full = tiles / round, r = tiles - full * round;
  double us = (double)full * f.c_full;
  if (r > 0) {
    const double one_per_cu = f.c0 * (1.0 + f.a);
    if (r <= cus) { const double load = (double)r / (double)cus; us += f.c0 * (1.0 + f.a * load * load); }
    else us += one_per_cu + (f.c_full - one_per_cu) * (double)(r - cus) / (double)(round - cus);
  }
  return us;
}
// Launch, prologue (pair table, filling the ring) and the store of the result.
static inline double fixed_us(int tile, bool wide, double c_bytes) {
  static const double base[kTileCount] = {11.0, 13.0, 8.0, 5.5};
  return base[tile] + c_bytes / (wide ? 1.0e7 : 6.0e6);
}

template <typename T>
static inline Plan plan(const Args<T>& g) {
  constexpr bool WIDE = sizeof(T) == 8;
  Plan pl;
  pl.Kp = (g.K + kKPad - 1) / kKPad * kKPad;
  const int64_t cus = num_cus();
  const double c_bytes = (double)g.M * (double)g.N * sizeof(T);
  // rows and columns are padded to the chosen tile only (1280 is 20 tiles of 64, not 24)
  auto padded = [](int64_t x, int64_t to) { return (x + to - 1) / to * to; };
  auto tiles_of = [&](int t) { return (padded(g.M, kTileRows[t]) / kTileRows[t]) * (padded(g.N, kTileCols[t]) / kTileCols[t]); };
  int best = 0;
  double best_us = 0.0;
  for (int t = 0; t < kTileCount; ++t) {
    if (WIDE && t == 1) continue;
    const double us = fixed_us(t, WIDE, c_bytes) + main_us_per_k(t, WIDE, tiles_of(t), cus) * (double)pl.Kp;
    if (t == 0 || us < best_us) { best = t; best_us = us; }
  }
  if (const char* force = getenv("AM_HIP_GEMM_TILE_I8")) {   // tests: 0 ... 3, see kTileRows / kTileCols
    if (*force) { const int t = atoi(force); if (t >= 0 && t < kTileCount && !(WIDE && t == 1)) best = t; }
  }
  pl.tile = best;
  pl.Mp = padded(g.M, kTileRows[best]);
  pl.Np = padded(g.N, kTileCols[best]);
  pl.fixed_us = fixed_us(best, WIDE, c_bytes);
  pl.main_us = pl.fixed_us + main_us_per_k(best, WIDE, tiles_of(best), cus) * (double)pl.Kp;
  // The first pass reads every element and writes its lowest digit; the second reads it again (mostly
  // from the memory-side cache) and writes the other planes.
  const double elems = (double)(pl.Mp + pl.Np) * pl.Kp, sz = (double)sizeof(T);
  pl.first_us = 4.5 + elems * (sz + 1.0) / (WIDE ? 5.5e6 : 6.2e6);
  pl.second_us = 4.5 + elems * (2.0 * sz - 1.0) / 7.0e6;
  pl.est_us = pl.main_us + pl.first_us + pl.second_us;
  return pl;
}

// Whether the digit-sliced path may take this product at all: not part of a batch, not being
// recorded into a graph (it allocates its planes), and for int64 k small enough that one pair's
// sum over k fits the 32-bit accumulators of the matrix cores (k * 2^14 < 2^31).
// AM_HIP_GEMM_I32_PATH / AM_HIP_GEMM_I64_PATH = "valu" / "mfma" forces a path (tests, benchmarks);
// returns 0 = no, 1 = if estimated faster, 2 = forced, 3 = forced as a data-dependent choice.
template <typename T>
static inline int applicable(const Args<T>& g) {
  const char* e = getenv(sizeof(T) == 8 ? "AM_HIP_GEMM_I64_PATH" : "AM_HIP_GEMM_I32_PATH");
  if (e && *e == 'v') return 0;
  if (g.batch > 1 || capturing()) return 0;
  if (sizeof(T) == 8 && g.K > 131071) return 0;
  if (e && *e == 'm') return 2;
  if (e && *e == 's') return 3;   // "spec": both kernels behind the first splitting pass, the data decides (tests)
  return (g.M >= 64 && g.N >= 64 && g.K >= 256) ? 1 : 0;
}

// The digit planes of one operand split ahead of time (am_hip_digits_prepare_*): a weight matrix that enters many
// products is read and split once instead of in every call. Rows are padded to 256, a multiple of every tile edge, so
// the planes serve whatever tile a product chooses and either side of it (the layout does not depend on the side:
// X(mn, k), mn = a row of a left operand or a column of a right one).
struct Prepared {
  uint32_t magic;        // kPreparedMagic while the handle is alive
  int elem_size;         // 4 or 8
  int64_t MN, K, MNp, Kp;
  int8_t* planes;        // elem_size planes of MNp x Kp bytes, from am_hip_malloc
  int mask;              // bit d set: plane d holds a non-zero digit somewhere
};
constexpr uint32_t kPreparedMagic = 0x44504c4eu;
// The handles am_hip_digits_prepare_* has handed out and am_hip_digits_release has not taken back (gemm_i32.hip):
// anything else passed as a handle is refused instead of being dereferenced.
void remember_prepared(const Prepared* p);
const Prepared* lookup_prepared(const void* handle);

// max_pairs < all pairs: the product is left alone when the operands turn out to have more live digit
// pairs; *gate_flags / *gate_gen then tell the caller what to hand to the kernels it launches next.
// pa / pb: planes of the kernel's A / B operand split ahead of time (nullptr: split here, into scratch memory).
template <typename T>
static int run(const Args<T>& g, const Plan& pl, int max_pairs = 1 << 30, const uint32_t** gate_flags = nullptr,
               uint32_t* gate_gen = nullptr, const Prepared* pa = nullptr, const Prepared* pb = nullptr) {
  constexpr int ND = (int)sizeof(T);
  const int64_t Mp = pa ? pa->MNp : pl.Mp, Np = pb ? pb->MNp : pl.Np, Kp = pl.Kp;
  if (Mp / 32 >= ((int64_t)1 << 31) || Np / 32 >= ((int64_t)1 << 31) || Kp / 128 > 65535) return 1;
  const int64_t tiles_m = (g.M + kTileRows[pl.tile] - 1) / kTileRows[pl.tile], tiles_n = (g.N + kTileCols[pl.tile] - 1) / kTileCols[pl.tile];
  if (tiles_m * tiles_n >= ((int64_t)1 << 31)) return 1;
  // Flag words live as long as the process: every product uses a new generation number, so they are
  // cleared only once (and again should the 32-bit counter ever wrap).
  static uint32_t* flags = nullptr;
  static uint32_t gen = 0;
  if (!(pa && pb)) {   // (with both operands split ahead of time nothing reads the flag words: nothing to set up, so
                       // such a product can be recorded into a graph even as the first of the process)
    if (!flags) {
      void* f = nullptr;
      if (am_hip_malloc(256, &f) != AM_OK) return 1;
      flags = (uint32_t*)f;
      gen = 0;
    }
    if (gen == 0 || gen == 0xFFFFFFFFu) {
      if (hipMemsetAsync(flags, 0, 256, stream()) != hipSuccess) { (void)hipGetLastError(); return 1; }
      gen = 0;
    }
    ++gen;
  }
  void* ws = nullptr;
  const size_t plane_bytes = (size_t)ND * (size_t)((pa ? 0 : Mp) + (pb ? 0 : Np)) * (size_t)Kp;
  if (plane_bytes > 0 && am_hip_malloc(plane_bytes, &ws) != AM_OK) return 1;
  int8_t* PA = pa ? pa->planes : (int8_t*)ws;
  int8_t* PB = pb ? pb->planes : (int8_t*)ws + (pa ? 0 : (int64_t)ND * Mp * Kp);
  SplitArgs<T> sp;
  // (an operand split ahead of time has no tiles for the passes to visit: MNp = 0)
  sp.X[0] = g.A; sp.ld_mn[0] = g.a_mn; sp.ld_k[0] = g.a_k; sp.MN[0] = g.M; sp.MNp[0] = pa ? 0 : Mp; sp.kfast[0] = g.a_kfast; sp.P[0] = PA;
  sp.X[1] = g.B; sp.ld_mn[1] = g.b_mn; sp.ld_k[1] = g.b_k; sp.MN[1] = g.N; sp.MNp[1] = pb ? 0 : Np; sp.kfast[1] = g.b_kfast; sp.P[1] = PB;
  sp.K = g.K; sp.Kp = Kp; sp.flags = flags; sp.gen = gen; sp.max_pairs = max_pairs;
  if (gate_flags) *gate_flags = flags;
  if (gate_gen) *gate_gen = gen;
  constexpr int64_t VEC = 16 / (int64_t)sizeof(T);
  for (int op = 0; op < 2; ++op) {
    const bool aligned = ((uintptr_t)sp.X[op] & 15) == 0;
    sp.mode[op] = (aligned && sp.ld_k[op] == 1 && sp.ld_mn[op] % VEC == 0)   ? 1
                  : (aligned && sp.ld_mn[op] == 1 && sp.ld_k[op] % VEC == 0) ? 2
                                                                             : 0;
  }
  const int64_t stiles = (sp.MNp[0] + sp.MNp[1]) / 32 * (Kp / 128), smax = (int64_t)num_cus() * 16;
  if (stiles > 0) {
    const dim3 sgrid((unsigned)(stiles < smax ? stiles : smax));
    // Operands beyond what the memory-side cache may still hold from their producer are read with non-temporal
    // loads (int64 4096^3, 256 MiB of operands: first pass 65 -> 46 us); smaller ones are faster with ordinary loads.
    const bool stream_loads = (double)((pa ? 0 : g.M) + (pb ? 0 : g.N)) * (double)g.K * sizeof(T) > 192.0 * 1024 * 1024;
    if (stream_loads) hipLaunchKernelGGL((split_digits<T, true, true>), sgrid, dim3(256), 0, stream(), sp);
    else hipLaunchKernelGGL((split_digits<T, true>), sgrid, dim3(256), 0, stream(), sp);
    // with at most one live pair allowed there is nothing above plane 0 that could be needed
    if (max_pairs >= 2) hipLaunchKernelGGL((split_digits<T, false>), sgrid, dim3(256), 0, stream(), sp);
  }
  DigitArgs<T> d;
  d.preset_a = pa ? pa->mask : -1; d.preset_b = pb ? pb->mask : -1;
  d.PA = PA; d.PB = PB; d.flags = flags; d.gen = gen; d.max_pairs = max_pairs; d.Mp = Mp; d.Np = Np; d.Kp = Kp;
  d.C = g.C; d.c_m = g.c_m; d.c_n = g.c_n; d.M = g.M; d.N = g.N; d.clock_out = g.clock_out;
  d.alpha = g.alpha; d.beta = g.beta;
  d.tiles_m = (int)tiles_m; d.tiles_n = (int)tiles_n;
  const dim3 grid((unsigned)(tiles_m * tiles_n));
  switch (pl.tile) {
    case 1:
      if constexpr (sizeof(T) == 4) { hipLaunchKernelGGL((gemm_i8_digits<T, 2, 4, 4, 2, 64, 4>), grid, dim3(512), 0, stream(), d); break; }
      [[fallthrough]];   // int64 has no 256 x 256 tile (plan() never picks it)
    default: hipLaunchKernelGGL((gemm_i8_digits<T, 4, 2, 2, 2, 64, 4>), grid, dim3(512), 0, stream(), d); break;
    case 2: hipLaunchKernelGGL((gemm_i8_digits<T, 2, 4, 2, 1, 64, 4>), grid, dim3(512), 0, stream(), d); break;
    case 3: hipLaunchKernelGGL((gemm_i8_digits<T, 2, 2, 1, 1, 64, 4>), grid, dim3(256), 0, stream(), d); break;
  }
  const int rc = check_launch("gemm_i8_digits");
  // The planes go back to the allocator's cache at once: whoever gets the block next reaches it
  // through the same stream, after this product.
  if (ws) (void)am_hip_free(ws);
  return rc;
}

// Splits X(mn, k) = X[mn * ld_mn + k * ld_k] (MN x K) into planes of its own (both passes, then a blocking look at
// which planes came out non-empty). Returns AM_OK and the planes in *out, or an error code.
template <typename T>
static int prepare_planes(const T* X, int64_t MN, int64_t K, int64_t ld_mn, int64_t ld_k, Prepared* out) {
  constexpr int ND = (int)sizeof(T);
  constexpr int64_t VEC = 16 / (int64_t)sizeof(T);
  const int64_t MNp = (MN + 255) / 256 * 256, Kp = (K + kKPad - 1) / kKPad * kKPad;
  if (MNp / 32 >= ((int64_t)1 << 31) || Kp / 128 > 65535) return fail(AM_E_SHAPE, "am_hip_digits_prepare: operand too large");
  void* planes = nullptr;
  void* fl = nullptr;
  AM_TRY(am_hip_malloc((size_t)ND * (size_t)MNp * (size_t)Kp, &planes));
  if (am_hip_malloc(256, &fl) != AM_OK) { (void)am_hip_free(planes); return AM_E_ALLOC; }
  hipError_t e = hipMemsetAsync(fl, 0, 256, stream());
  SplitArgs<T> sp;
  sp.X[0] = X; sp.ld_mn[0] = ld_mn; sp.ld_k[0] = ld_k; sp.MN[0] = MN; sp.MNp[0] = MNp; sp.kfast[0] = iabs64(ld_k) <= iabs64(ld_mn); sp.P[0] = (int8_t*)planes;
  sp.X[1] = X; sp.ld_mn[1] = ld_mn; sp.ld_k[1] = ld_k; sp.MN[1] = 0; sp.MNp[1] = 0; sp.kfast[1] = sp.kfast[0]; sp.P[1] = (int8_t*)planes;
  sp.K = K; sp.Kp = Kp; sp.flags = (uint32_t*)fl; sp.gen = 1; sp.max_pairs = 1 << 30;
  const bool aligned = ((uintptr_t)X & 15) == 0;
  sp.mode[0] = sp.mode[1] = (aligned && ld_k == 1 && ld_mn % VEC == 0) ? 1 : (aligned && ld_mn == 1 && ld_k % VEC == 0) ? 2 : 0;
  const int64_t stiles = MNp / 32 * (Kp / 128), smax = (int64_t)num_cus() * 16;
  const dim3 sgrid((unsigned)(stiles < smax ? stiles : smax));
  if (e == hipSuccess) {
    hipLaunchKernelGGL((split_digits<T, true>), sgrid, dim3(256), 0, stream(), sp);
    hipLaunchKernelGGL((split_digits<T, false>), sgrid, dim3(256), 0, stream(), sp);
    e = hipGetLastError();
  }
  uint32_t host_flags[ND];
  int rc = e == hipSuccess ? fetch_result(host_flags, fl, sizeof(host_flags)) : fail(AM_E_HIP, "am_hip_digits_prepare: %s", hipGetErrorString(e));
  (void)am_hip_free(fl);
  if (rc != AM_OK) { (void)am_hip_free(planes); return rc; }
  out->magic = kPreparedMagic; out->elem_size = ND; out->MN = MN; out->K = K; out->MNp = MNp; out->Kp = Kp;
  out->planes = (int8_t*)planes;
  out->mask = 0;
  for (int d = 0; d < ND; ++d) out->mask |= (host_flags[d] == 1u) ? (1 << d) : 0;
  return AM_OK;
}

// A product whose A and / or B operand (as the caller named them) was split ahead of time. The digit path is taken
// outright (no estimate: the planes exist). Returns 1 when the product cannot run here (a batch member, a long int64
// k, no scratch memory for the other operand): the caller then runs it from the original operands.
template <typename T>
static int run_prepared(const Args<T>& g, const Prepared* user_a, const Prepared* user_b, int* rc) {
  *rc = AM_OK;
  const Prepared* pa = g.swapped ? user_b : user_a;
  const Prepared* pb = g.swapped ? user_a : user_b;
  for (int side = 0; side < 2; ++side) {
    const Prepared* h = side ? pb : pa;
    if (!h) continue;
    if (h->magic != kPreparedMagic || h->elem_size != (int)sizeof(T)) { *rc = fail(AM_E_ARG, "gemm with prepared digits: not a live handle of this element type"); return 0; }
    if (h->MN != (side ? g.N : g.M) || h->K != g.K) {
      *rc = fail(AM_E_SHAPE, "gemm with prepared digits: the handle holds a %lld x %lld operand, the product needs %lld x %lld on that side",
                 (long long)h->MN, (long long)h->K, (long long)(side ? g.N : g.M), (long long)g.K);
      return 0;
    }
  }
  if (g.batch > 1 || (sizeof(T) == 8 && g.K > 131071)) return 1;
  if (capturing() && !(pa && pb)) return 1;      // the other operand's planes would need scratch memory
  const Plan pl = plan(g);
  if (trace_choices()) fprintf(stderr, "am_hip gemm: int8 digit path with planes split ahead of time (%s%s), %s tiles\n", pa ? "A" : "", pb ? "B" : "", tile_name(pl.tile));
  const int r = run(g, pl, 1 << 30, nullptr, nullptr, pa, pb);
  if (r <= 0) { *rc = r; return 0; }
  return 1;
}

// The integer product on the matrix cores, decided in three steps. (1) Estimated faster than the
// vector-ALU kernel even if every digit pair is needed: taken outright. (2) Not, but faster when
// few pairs are live (operands with small entries): the splitting passes and the digit kernel are launched with
// the largest pair count that still wins; the caller then launches the vector-ALU kernel gated on the
// same flags, and whichever of the two the data rules out leaves at once. (3) Otherwise not taken.
// Returns 0 when the product is done or a launch failed (rc), 1 when the caller has to launch the
// vector-ALU kernel (g.gate_* set for case 2).
template <typename T>
static int try_digits(Args<T>& g, double valu_est_us, int* rc) {
  constexpr int ND = (int)sizeof(T), NPAIRS = ND * (ND + 1) / 2;
  *rc = AM_OK;
  const int may = applicable(g);
  if (!may) return 1;
  const Plan pl = plan(g);
  // What the vector-ALU kernel takes in practice: its tile model leaves out launch and tail effects
  // (fitted to the same sizes as the digit path's model).
  const double valu_us = (sizeof(T) == 8 ? 1.15 : 1.3) * valu_est_us + 5.0;
  if (may == 2 || (may == 1 && pl.est_us < 1.1 * valu_us)) {
    if (trace_choices()) fprintf(stderr, "am_hip gemm: int8 digit path, %s tiles, est %.1f us (VALU est %.1f us)\n", tile_name(pl.tile), pl.est_us, valu_us);
    const int r = run(g, pl);
    if (r <= 0) { *rc = r; return 0; }
    return 1;   // no scratch memory for the digit planes
  }
  // When the data says no, the first splitting pass and two kernels that leave at once have been paid
  // for nothing (about 10 us at small sizes): only worth risking on products that take a few times that.
  const double per_pair = (pl.main_us - pl.fixed_us) / NPAIRS, fixed = pl.first_us + 4.5 + 3.0 + pl.fixed_us;   // + a second pass and a product kernel that leave at once
  int max_pairs = (int)((0.85 * valu_us - fixed) / per_pair);
  if (const char* e = getenv("AM_HIP_GEMM_SPEC_PAIRS")) max_pairs = atoi(e);   // tests
  if (max_pairs > NPAIRS) max_pairs = NPAIRS;
  if (may != 3 && (max_pairs < 1 || valu_us < 32.0)) return 1;
  if (max_pairs < 0) max_pairs = 0;
  if (trace_choices()) fprintf(stderr, "am_hip gemm: int8 digit path if at most %d digit pairs are live, else VALU (est %.1f us)\n", max_pairs, valu_us);
  const uint32_t* flags = nullptr;
  uint32_t gen = 0;
  const int r = run(g, pl, max_pairs, &flags, &gen);
  if (r < 0) { *rc = r; return 0; }
  if (r == 0) { g.gate_flags = flags; g.gate_gen = gen; g.gate_max_pairs = max_pairs; }
  return 1;
}

}  // namespace i8
}  // namespace gemm
}  // namespace am
