// MFMA GEMM for gfx950 (CDNA4), float32 (v_mfma_f32_32x32x2_f32) and float64
// (v_mfma_f64_16x16x4_f64). C[MxN] <- alpha * A * B + beta * C with arbitrary element strides
// on every operand and an optional fused bias / ReLU epilogue.
//
// Replaces the reference's CPU blocked GEMM (src/arraymancer/laser/primitives/
// matrix_multiplication/gemm.nim:117-184: pack B panel, pack A block, micro-kernel) with a
// GPU decomposition built for 64-wide wavefronts:
//   * one workgroup per BM x BN tile of C, WAVES_M x WAVES_N wavefronts, each owning a
//     (BM/WAVES_M) x (BN/WAVES_N) sub-tile as TM x TN MFMA accumulators held in registers
//     for the whole K loop;
//   * K is walked in BK-wide slabs, double-buffered in LDS: while the matrix cores work on slab
//     t, the global loads of slab t+1 are in flight into registers and are written to the other
//     LDS buffer afterwards (one barrier per slab);
//   * "packing" (gemm_packing.nim:24-99) becomes the choice of LDS layout per operand, so that
//     both the global->LDS copy and the LDS->register fragment reads are 16-byte accesses when
//     the operand has a unit stride in either direction, with no transpose through registers:
//       - unit stride along k  -> "k-group" layout [k/VK][mn][VK]; a lane reads the VK
//         consecutive k values of its row with one ds_read_b128;
//       - unit stride along mn -> "k-row" layout [k][mn]; a lane reads its VK k values with VK
//         ds_read_b32/b64 (conflict-free: consecutive lanes, consecutive addresses);
//       - anything else (zero / negative / non-unit strides) -> scalar gathers into the k-row
//         layout. No host-side copy is ever made (the reference copies non-contiguous float
//         operands first: src/arraymancer/tensor/private/p_operator_blas_l2l3.nim:151-152).
//     The MFMA k index is a free permutation as long as A and B agree, which is what lets a
//     lane own VK consecutive k values: MFMA step s of a KSTEP = VK * (64/TILE) wide k-step
//     multiplies k = VK*kl + s for lane group kl on both operands.
//   * out-of-range rows/columns/k are zero-filled on load (the reference zero-pads its packed
//     panels the same way, gemm_packing.nim:54-55, 98-99) and masked on store.
#pragma once
#include <type_traits>
#include "gemm_loader.h"

namespace am {
namespace gemm {

template <typename T> struct Mfma;

template <> struct Mfma<float> {
  static constexpr int TILE = 32;  // output tile edge
  static constexpr int KL = 2;     // lane groups along k (64 / TILE)
  static constexpr int VK = 4;     // k values per lane per k-step (16 bytes)
  static constexpr int NACC = 16;  // accumulator registers per lane per tile
  typedef float acc_t __attribute__((ext_vector_type(16)));
  typedef float vec_t __attribute__((ext_vector_type(4)));
  static __device__ __forceinline__ acc_t mma(float a, float b, acc_t c) {
    return __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, 0, 0, 0);
  }
  // Row of the 32x32 tile held in accumulator register r of `lane` (column = lane % 32).
  static __device__ __forceinline__ int acc_row(int r, int lane) { return 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3); }
};

// float32 with the 16 x 16 x 4 instruction (8 passes, the same rate per cycle as 32 x 32 x 2): a quarter of the
// accumulator registers per tile, so a small workgroup tile can be spread over four wavefronts, one per SIMD,
// where the large instruction would leave it to a single one.
struct MfmaF32x16 {
  static constexpr int TILE = 16;
  static constexpr int KL = 4;
  static constexpr int VK = 4;
  static constexpr int NACC = 4;
  typedef float acc_t __attribute__((ext_vector_type(4)));
  typedef float vec_t __attribute__((ext_vector_type(4)));
  static __device__ __forceinline__ acc_t mma(float a, float b, acc_t c) {
    return __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0);
  }
  // Register r of lane group g = lane / 16 holds row 4 * g + r (column = lane % 16).
  static __device__ __forceinline__ int acc_row(int r, int lane) { return 4 * (lane >> 4) + r; }
};

template <> struct Mfma<double> {
  static constexpr int TILE = 16;
  static constexpr int KL = 4;
  static constexpr int VK = 2;
  static constexpr int NACC = 4;
  typedef double acc_t __attribute__((ext_vector_type(4)));
  typedef double vec_t __attribute__((ext_vector_type(2)));
  static __device__ __forceinline__ acc_t mma(double a, double b, acc_t c) {
    return __builtin_amdgcn_mfma_f64_16x16x4f64(a, b, c, 0, 0, 0);
  }
  // v_mfma_f64_16x16x4: register r of lane group g = lane / 16 holds row 4 * r + g (column = lane % 16).
  static __device__ __forceinline__ int acc_row(int r, int lane) { return 4 * r + (lane >> 4); }
};

// Reads the VK k values that `lane` feeds to the MFMA steps of k-step `ks` for row/col `mn`.
template <typename T, typename MF, int KIND, int BMN, int BK>
__device__ __forceinline__ void read_frag(const T* lds, int mn, int ks, int kl, T (&out)[MF::VK]) {
  typedef typename MF::vec_t vec_t;
  constexpr int VK = MF::VK, KL = MF::KL;
  if constexpr (k_grouped(KIND)) {
    constexpr int LD = Slab<T, KIND, BMN, BK>::LDKG;
    const vec_t v = *(const vec_t*)(lds + ((ks * KL + kl) * LD + mn) * VK);
#pragma unroll
    for (int s = 0; s < VK; ++s) out[s] = v[s];
  } else {
    constexpr int LD = Slab<T, KIND, BMN, BK>::LDMN;
#pragma unroll
    for (int s = 0; s < VK; ++s) out[s] = lds[((ks * KL + kl) * VK + s) * LD + mn];
  }
}

// Second __launch_bounds__ argument: two wavefronts per SIMD whatever the workgroup size, i.e. at
// most 256 registers per lane, all of them architectural VGPRs. Allowed more, the compiler spreads
// a large tile's accumulators over VGPRs and AGPRs and copies them back and forth in every loop
// trip (measured: f64 128 x 128 falls from 61 to 48 TFLOP/s).
constexpr int mfma_min_blocks(int nt) { return nt <= 256 ? 2 : 1; }

template <int I, int N, typename F> __device__ __forceinline__ void static_for(F&& f) {
  if constexpr (I < N) {
    f(std::integral_constant<int, I>());
    static_for<I + 1, N>(f);
  }
}

template <typename T, typename MF, int BM, int BN, int BK, int WAVES_M, int WAVES_N, int PF, bool FPF, bool RU, int AK, int BKIND>
__global__ __launch_bounds__(WAVES_M* WAVES_N * 64, (WAVES_M * WAVES_N <= 4 ? 2 : 1))
void gemm_mfma(Args<T> p) {
  typedef typename MF::acc_t acc_t;
  // Every argument the prologue reads is wanted in a scalar register here, so that the argument block's cache lines
  // are requested together and waited for once: left alone, the compiler requests each line where a field of it is
  // first used, behind the branches in between (five dependent round trips to memory in front of the first operand load).
  asm volatile("" ::"s"(p.M), "s"(p.N), "s"(p.K), "s"(p.A), "s"(p.a_mn), "s"(p.a_k), "s"(p.B), "s"(p.b_mn), "s"(p.b_k), "s"(p.C),
               "s"(p.c_m), "s"(p.c_n), "s"(p.tiles_m), "s"(p.tiles_n), "s"(p.splits), "s"(p.k_chunk), "s"(p.batch), "s"(p.clock_out));
  const ClockProbe probe(p.clock_out);
  constexpr int NT = WAVES_M * WAVES_N * 64;
  constexpr int TILE = MF::TILE, VK = MF::VK, KL = MF::KL, KSTEP = VK * KL;
  constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N, TM = WM / TILE, TN = WN / TILE;
  static_assert(BK % KSTEP == 0 && WM % TILE == 0 && WN % TILE == 0, "tile shape");
  constexpr int A_ELEMS = Slab<T, AK, BM, BK>::ELEMS, B_ELEMS = Slab<T, BKIND, BN, BK>::ELEMS;

  static_assert((BK / KSTEP) % 2 == 0, "fragment double buffering needs an even number of k-steps per slab");
  __shared__ __attribute__((aligned(16))) T sA[3][A_ELEMS];
  __shared__ __attribute__((aligned(16))) T sB[3][B_ELEMS];

  int tile_m, tile_n, bid = (int)blockIdx.x, split = 0;
  if (p.splits > 1) {
    const int nt = p.tiles_m * p.tiles_n;
    split = bid / nt;
    bid -= split * nt;
  }
  tile_of_block(bid, p.tiles_m, p.tiles_n, tile_m, tile_n);
  if (p.batch > 1) {
    const int64_t z = blockIdx.y;
    p.A += z * p.batch_a;
    p.B += z * p.batch_b;
    p.C += z * p.batch_c;
  }
  const int64_t m0 = (int64_t)tile_m * BM, n0 = (int64_t)tile_n * BN;
  const int64_t k_begin = (int64_t)split * p.k_chunk;
  const int64_t k_end = (k_begin + p.k_chunk < p.K) ? k_begin + p.k_chunk : p.K;

  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int wave_m = wave / WAVES_N, wave_n = wave % WAVES_N;
  const int lrow = lane % TILE, kl = lane / TILE;

  Loader<T, AK, BM, BK, NT, true, PF> la(p.A, p.a_mn, p.a_k, m0, p.M, k_end, p.a_kfast);
  Loader<T, BKIND, BN, BK, NT, true, PF> lb(p.B, p.b_mn, p.b_k, n0, p.N, k_end, p.b_kfast, &p.conv);

  acc_t acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int r = 0; r < MF::NACC; ++r) acc[i][j][r] = (T)0;

  // Software pipeline over the K slabs; nothing but the barrier itself is left between the MFMA
  // streams of consecutive slabs.
  //   global --fetch--> register stage (PF of them) --commit--> LDS ring of 3 slabs --> fragments
  // Iteration t multiplies slab t out of LDS buffer t % 3. During its last k-step it
  //   * reads the first fragments of slab t + 1 (buffer (t+1) % 3, complete since the barrier that
  //     ended iteration t - 1), so the next iteration starts with its operands in registers
  //     (FPF = true: fragments are double-buffered in registers and always read one k-step ahead;
  //     FPF = false, for shapes whose accumulators leave no room: read at the k-step's start);
  //   * commits slab t + 2 from register stage t % PF to buffer (t+2) % 3 (last read in iteration
  //     t - 1, i.e. before the previous barrier), then refills that stage with slab t + 2 + PF:
  //     a global load has PF whole slabs of MFMA work to arrive.
  // The LDS writes of iteration t are waited for at the barrier that ends it, having had a
  // k-step of MFMAs to drain.
  // The loop body is straight-line code on purpose (no test for "is there a next slab"): only then can
  // the compiler count the loads in flight and wait for the oldest stage alone. The slabs near the end of
  // the k range, whose fetches or commits would pass it, run other instances of the same body (see below).
  constexpr int NKS = BK / KSTEP;
  const int64_t ktiles = (k_end - k_begin + BK - 1) / BK;
  // Slabs that the unmasked (steady-state) loop may fetch: those wholly inside the k range, less the last
  // one when a loader must not run its unmasked fetch on the operand's last k row (see tail_guard).
  const int64_t full_slabs = (k_end - k_begin) / BK - ((la.tail_guard() || lb.tail_guard()) ? 1 : 0);

  T af[2][TM][VK], bf[2][TN][VK];
  auto read_frags = [&](auto parity_tag, const T* a_lds, const T* b_lds, int ks) {
    constexpr int P = decltype(parity_tag)::value;
#pragma unroll
    for (int i = 0; i < TM; ++i) read_frag<T, MF, AK, BM, BK>(a_lds, wave_m * WM + i * TILE + lrow, ks, kl, af[P][i]);
#pragma unroll
    for (int j = 0; j < TN; ++j) read_frag<T, MF, BKIND, BN, BK>(b_lds, wave_n * WN + j * TILE + lrow, ks, kl, bf[P][j]);
  };

  // Prologue: slabs 0 and 1 into LDS, slabs 2 .. 2 + PF - 1 into the register stages (stage s holds slab 2 + s).
  // When all of them lie wholly inside the k range (any but a very short one) the unmasked loads do: a few
  // instructions each, where the masked ones compute clamped addresses per vector.
  auto prologue = [&](auto mask_tag) {
    constexpr bool MASK = decltype(mask_tag)::value;
    if constexpr (PF > 1) {
      la.template fetch<0, MASK>(k_begin);
      lb.template fetch<0, MASK>(k_begin);
      la.template fetch<1, MASK>(k_begin + BK);
      lb.template fetch<1, MASK>(k_begin + BK);
      la.template commit<0, MASK>(sA[0], k_begin);
      lb.template commit<0, MASK>(sB[0], k_begin);
      la.template commit<1, MASK>(sA[1], k_begin + BK);
      lb.template commit<1, MASK>(sB[1], k_begin + BK);
      static_for<0, PF>([&](auto st) {
        la.template fetch<decltype(st)::value, MASK>(k_begin + (2 + decltype(st)::value) * BK);
        lb.template fetch<decltype(st)::value, MASK>(k_begin + (2 + decltype(st)::value) * BK);
      });
    } else {
      la.template fetch<0, MASK>(k_begin);
      lb.template fetch<0, MASK>(k_begin);
      la.template commit<0, MASK>(sA[0], k_begin);
      lb.template commit<0, MASK>(sB[0], k_begin);
      la.template fetch<0, MASK>(k_begin + BK);
      lb.template fetch<0, MASK>(k_begin + BK);
      la.template commit<0, MASK>(sA[1], k_begin + BK);
      lb.template commit<0, MASK>(sB[1], k_begin + BK);
      la.template fetch<0, MASK>(k_begin + 2 * BK);
      lb.template fetch<0, MASK>(k_begin + 2 * BK);
    }
  };
  if (full_slabs >= 2 + PF) prologue(std::false_type());
  else prologue(std::true_type());
  __syncthreads();
  if constexpr (FPF) read_frags(std::integral_constant<int, 0>(), sA[0], sB[0], 0);

  int cur = 0;   // ring position of the slab being multiplied
  // cur_tag >= 0: the ring position is known at compile time (the steady-state loop is unrolled over the
  // ring), so every LDS address of the slab is a constant offset and no address arithmetic stands
  // between the matrix instructions and the fragment reads; -1: taken from `cur` (the last few slabs).
  // What a slab's last k-step moves besides multiplying: kSteady commits slab kt + 2 and fetches slab kt + 2 + PF, both
  // wholly inside the k range (nothing clamped or zeroed); kMasked does the same with clamping and zero fill; kCommit
  // commits a whole slab and fetches nothing (slab kt + 2 + PF does not exist); kIdle moves nothing (slab kt + 2 does
  // not exist either).
  constexpr int kSteady = 0, kMasked = 1, kCommit = 2, kIdle = 3;
  auto slab = [&](auto stage_tag, auto mode_tag, auto cur_tag, int64_t kt) {
    constexpr int S = decltype(stage_tag)::value;
    constexpr int MODE = decltype(mode_tag)::value;
    constexpr bool MASK = MODE == kMasked;
    constexpr int CT = decltype(cur_tag)::value;
    const int here = CT >= 0 ? CT : cur;
    const int nxt = (here == 2) ? 0 : here + 1;
    const int nxt2 = (nxt == 2) ? 0 : nxt + 1;
#pragma unroll
    for (int ks = 0; ks < NKS; ++ks) {
      // fragments for the k-step after this one: next k-step of this slab, or first of the next slab
      if constexpr (!FPF) read_frags(std::integral_constant<int, 0>(), sA[here], sB[here], ks);
      if (ks + 1 < NKS) {
        if constexpr (FPF) {
          if (ks & 1) read_frags(std::integral_constant<int, 0>(), sA[here], sB[here], ks + 1);
          else read_frags(std::integral_constant<int, 1>(), sA[here], sB[here], ks + 1);
        }
      } else {
        if constexpr (FPF) read_frags(std::integral_constant<int, 0>(), sA[nxt], sB[nxt], 0);   // NKS is even
        if constexpr (MODE != kIdle) {
          la.template commit<S, MASK>(sA[nxt2], k_begin + (kt + 2) * BK);
          lb.template commit<S, MASK>(sB[nxt2], k_begin + (kt + 2) * BK);
        }
        if constexpr (MODE == kSteady || MODE == kMasked) {
          la.template fetch<S, MASK>(k_begin + (kt + 2 + PF) * BK);
          lb.template fetch<S, MASK>(k_begin + (kt + 2 + PF) * BK);
        }
      }
      // Left alone, the instruction scheduler sinks the reads and loads above down to their first use.
      // With fragment prefetch (the operands of this k-step are already in registers) they are spread
      // between this k-step's matrix instructions instead: a wavefront issues in order, so whatever
      // stands in front of its matrix instructions delays them (measured: +15 % on 64 x 64 tiles with one
      // wavefront per SIMD, +2 to 7 % on the large ones). Without prefetch they have to come first.
      constexpr bool ILV = FPF;
      if constexpr (ILV) {
#pragma unroll
        for (int s = 0; s < VK; ++s)
#pragma unroll
          for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j) acc[i][j] = MF::mma(af[ks & 1][i][s], bf[ks & 1][j][s], acc[i][j]);
      } else {
        // No prefetch: this k-step's own fragments were requested just above. Row block by row block,
        // so that the matrix instructions of block i can start once the B fragments and A fragment i
        // are in, while the reads of the later A fragments and everything else go on between them.
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
          for (int s = 0; s < VK; ++s)
#pragma unroll
            for (int j = 0; j < TN; ++j) acc[i][j] = MF::mma(af[0][i][s], bf[0][j][s], acc[i][j]);
        constexpr int RA = k_grouped(AK) ? 1 : VK, RB = k_grouped(BKIND) ? 1 : VK;   // LDS reads per fragment
        __builtin_amdgcn_sched_group_barrier(0x100, TN * RB + RA, 0);   // the B fragments and A fragment 0
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
          for (int m = 0; m < VK * TN; ++m) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            if (m == 0 && i + 1 < TM) __builtin_amdgcn_sched_group_barrier(0x100, RA, 0);   // A fragment i + 1
            __builtin_amdgcn_sched_group_barrier(0x200, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x006, 4, 0);
          }
      }
      if constexpr (ILV) {
#pragma unroll
        for (int m = 0; m < VK * TM * TN; ++m) {
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);   // one matrix instruction
          __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);   // LDS reads
          __builtin_amdgcn_sched_group_barrier(0x200, 2, 0);   // LDS writes
          __builtin_amdgcn_sched_group_barrier(0x020, 2, 0);   // global loads
          __builtin_amdgcn_sched_group_barrier(0x006, 8, 0);   // address arithmetic
        }
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    __syncthreads();
    cur = nxt;
  };
  // Steady state: every slab this iteration fetches or commits lies wholly inside the k range,
  // so no clamping or zeroing is compiled in. The last 2 + PF slabs (more when the range ends in a partial slab)
  // run the masked form or, slab by slab, the cheapest form that is correct for them.
  int64_t kt = 0;
  typedef std::integral_constant<int, -1> dyn;
  typedef std::integral_constant<int, kSteady> steady;
  constexpr int UNR = PF % 3 == 0 ? PF : 3 * PF;   // whole turns of the ring, a whole number of register stages
  for (; RU && kt + (UNR - 1) + 2 + PF < full_slabs; kt += UNR)   // starts and ends at ring position 0
    static_for<0, UNR>([&](auto i) {
      constexpr int I = decltype(i)::value;
      slab(std::integral_constant<int, I % PF>(), steady(), std::integral_constant<int, I % 3>(), kt + I);
    });
  for (; kt + (PF - 1) + 2 + PF < full_slabs; kt += PF)
    static_for<0, PF>([&](auto i) { slab(i, steady(), dyn(), kt + decltype(i)::value); });
  // The cheaper forms only where a wavefront owns one or two accumulator tiles: there the last slabs are a
  // visible share of a short K loop. The large tiles, whose registers are all taken, run the masked form throughout
  // (more instances of their loop body cost them spills, and their K loops are long).
  constexpr bool CHEAP_TAIL = TM * TN <= 2;
  const int64_t whole = (k_end - k_begin) / BK;   // slabs wholly inside the k range
  for (; kt < ktiles; kt += PF)
    static_for<0, PF>([&](auto i) {
      const int64_t k = kt + decltype(i)::value;
      if (k >= ktiles) return;                                  // uniform, like every test below
      if (CHEAP_TAIL && k + 2 >= ktiles) slab(i, std::integral_constant<int, CHEAP_TAIL ? kIdle : kMasked>(), dyn(), k);
      else if (CHEAP_TAIL && k + 2 < whole && k + 2 + PF >= ktiles) slab(i, std::integral_constant<int, CHEAP_TAIL ? kCommit : kMasked>(), dyn(), k);
      else slab(i, std::integral_constant<int, kMasked>(), dyn(), k);
    });

  // Epilogue (gemm_ukernel_generic.nim:53-125): beta == 0 never reads C; C *= beta, then
  // C += alpha * AB, each rounded on its own; then the optional fused bias / ReLU.
  if (p.splits > 1) {   // split-K: raw partial tile to the workspace, epilogue in splitk_reduce
    T* ws = p.ws + (int64_t)split * p.M * p.N;
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j) {
        const int64_t col = n0 + wave_n * WN + j * TILE + lrow;
#pragma unroll
        for (int r = 0; r < MF::NACC; ++r) {
          const int64_t row = m0 + wave_m * WM + i * TILE + MF::acc_row(r, lane);
          if (row < p.M && col < p.N) ws[row * p.N + col] = acc[i][j][r];
        }
      }
    probe.finish();
    return;
  }
  const T alpha = p.alpha, beta = p.beta;
  const bool has_bias = (p.epilogue & AM_EPI_BIAS) != 0, relu = (p.epilogue & AM_EPI_RELU) != 0;
  // Accumulator register r of tile (i, j) holds C(row0 + i * TILE + acc_row(r, 0), col0 + j * TILE): one 64-bit
  // address product per lane, every other offset is a compile-time multiple of a stride (scalar arithmetic).
  const int64_t row0 = m0 + wave_m * WM + MF::acc_row(0, lane), col0 = n0 + wave_n * WN + lrow;
  T* const c0 = p.C + row0 * p.c_m + col0 * p.c_n;
  const T* const b0 = has_bias ? p.bias + row0 * p.bias_m + col0 * p.bias_n : nullptr;
  // One accumulator tile at a time: first every load of C and of the bias for that tile is issued,
  // then the arithmetic and the stores follow. Interleaving load / store per element would make
  // each load wait for the store before it (one memory counter orders both), i.e. one round trip
  // to HBM per element. (A whole row of tiles at once needs more registers than the largest tile
  // shapes have left next to their accumulators.) INTERIOR: the workgroup's tile lies wholly inside C,
  // nothing is tested per element. PLAIN: C <- AB (alpha = 1, beta = 0, no fused epilogue), stores only, and those
  // non-temporal: every workgroup of a round writes its tile at the same moment and nothing of C is read again by this
  // kernel (f32 2048^3: 125.4 -> 123.3 - 124.0 us; no change where C is read first, so those stores stay ordinary).
  auto write_out = [&](auto interior_tag, auto plain_tag) {
    constexpr bool INTERIOR = decltype(interior_tag)::value;
    constexpr bool PLAIN = decltype(plain_tag)::value;
#pragma unroll
    for (int i = 0; i < TM; ++i) {
#pragma unroll
      for (int j = 0; j < TN; ++j) {
        const bool col_ok = INTERIOR || col0 + j * TILE < p.N;
        T cv[MF::NACC], bv[MF::NACC];
        if constexpr (PLAIN) {
#pragma unroll
          for (int r = 0; r < MF::NACC; ++r) {
            const int dr = i * TILE + MF::acc_row(r, 0);
            if (INTERIOR || (col_ok && row0 + dr < p.M)) __builtin_nontemporal_store(acc[i][j][r], &c0[dr * p.c_m + j * TILE * p.c_n]);
          }
          continue;
        }
        if (beta != (T)0) {
#pragma unroll
          for (int r = 0; r < MF::NACC; ++r) {
            const int dr = i * TILE + MF::acc_row(r, 0);
            cv[r] = (INTERIOR || (col_ok && row0 + dr < p.M)) ? c0[dr * p.c_m + j * TILE * p.c_n] : (T)0;
          }
        }
        if (has_bias) {
#pragma unroll
          for (int r = 0; r < MF::NACC; ++r) {
            const int dr = i * TILE + MF::acc_row(r, 0);
            bv[r] = (INTERIOR || (col_ok && row0 + dr < p.M)) ? b0[dr * p.bias_m + j * TILE * p.bias_n] : (T)0;
          }
        }
#pragma unroll
        for (int r = 0; r < MF::NACC; ++r) {
          const int dr = i * TILE + MF::acc_row(r, 0);
          if (INTERIOR || (col_ok && row0 + dr < p.M)) {
            T ab = acc[i][j][r];
            if (alpha != (T)1) ab = alpha * ab;
            T v = ab;
            if (beta != (T)0) {
              T c = cv[r];
              if (beta != (T)1) c = c * beta;
              v = c + ab;
            }
            if (has_bias) v = v + bv[r];
            if (relu) v = ((T)0 >= v) ? (T)0 : v;
            c0[dr * p.c_m + j * TILE * p.c_n] = v;
          }
        }
      }
    }
  };
  const bool interior = m0 + BM <= p.M && n0 + BN <= p.N;
  if (alpha == (T)1 && beta == (T)0 && p.epilogue == 0) {
    if (interior) write_out(std::true_type(), std::true_type());
    else write_out(std::false_type(), std::true_type());
  } else {
    if (interior) write_out(std::true_type(), std::false_type());
    else write_out(std::false_type(), std::false_type());
  }
  probe.finish();
}

// PF: register stages of global loads; FPF: fragment prefetch; RU: steady-state loop unrolled over the LDS ring.
// MF: the matrix instruction (Mfma<T>, or MfmaF32x16 for small float tiles).
template <typename T, int BM, int BN, int BK, int WAVES_M, int WAVES_N, int PF = 1, bool FPF = true, bool RU = true, typename MF = Mfma<T>>
static int launch_kinds(Args<T>& g, int ak, int bk) {
  g.tiles_m = (int)((g.M + BM - 1) / BM);
  g.tiles_n = (int)((g.N + BN - 1) / BN);
  const int64_t nb = (int64_t)g.tiles_m * g.tiles_n;
  if (nb >= ((int64_t)1 << 31)) return fail(AM_E_SHAPE, "gemm: too many tiles");
  plan_splitk(g, BK, WAVES_M * WAVES_N);
  if (g.static_ws_short) {
    size_t cap = 0;
    (void)static_scratch(&cap);
    return fail(AM_E_SHAPE, "am_hip_gemm_noalloc_f32: M=%lld N=%lld K=%lld needs %zu bytes of split-K scratch, the static "
                "buffer holds %zu; call am_hip_gemm_f32 for this product", (long long)g.M, (long long)g.N, (long long)g.K,
                g.static_ws_short, cap);
  }
  const dim3 grid((unsigned)(nb * g.splits), (unsigned)g.batch), block(WAVES_M * WAVES_N * 64);
#define AM_LAUNCH(AKIND, BKIND_)                                                                   \
  hipLaunchKernelGGL((gemm_mfma<T, MF, BM, BN, BK, WAVES_M, WAVES_N, PF, FPF, RU, AKIND, BKIND_>), grid, block, 0, \
                     stream(), g)
  switch (ak * 3 + bk) {
    case 0: AM_LAUNCH(kKContig, kKContig); break;
    case 1: AM_LAUNCH(kKContig, kMNContig); break;
    case 2: AM_LAUNCH(kKContig, kGeneric); break;
    case 3: AM_LAUNCH(kMNContig, kKContig); break;
    case 4: AM_LAUNCH(kMNContig, kMNContig); break;
    case 5: AM_LAUNCH(kMNContig, kGeneric); break;
    case 6: AM_LAUNCH(kGeneric, kKContig); break;
    case 7: AM_LAUNCH(kGeneric, kMNContig); break;
    default: AM_LAUNCH(kGeneric, kGeneric); break;
  }
#undef AM_LAUNCH
  AM_TRY(check_launch("gemm_mfma"));
  if (g.splits > 1) return launch_splitk_reduce<T, T>(g);
  return AM_OK;
}

// A convolution as one batched GEMM whose B operand is gathered from the images (kGather): A = the kernel matrix
// [C_out, C * kH * kW] with unit stride along k, one batch member per image.
template <typename T, int BM, int BN, int BK, int WAVES_M, int WAVES_N, int PF = 1, bool FPF = true, bool RU = true, typename MF = Mfma<T>>
static int launch_conv(Args<T>& g) {
  g.tiles_m = (int)((g.M + BM - 1) / BM);
  g.tiles_n = (int)((g.N + BN - 1) / BN);
  const int64_t nb = (int64_t)g.tiles_m * g.tiles_n;
  if (nb >= ((int64_t)1 << 31)) return fail(AM_E_SHAPE, "conv2d: too many tiles");
  plan_splitk(g, BK, WAVES_M * WAVES_N);
  const dim3 grid((unsigned)(nb * g.splits), (unsigned)g.batch), block(WAVES_M * WAVES_N * 64);
  // 16-byte gathers where VK neighbouring output pixels of a row read VK neighbouring image elements
  constexpr int VK = VecTraits<T>::VK;
  const ConvGeom& cg = g.conv;
  static const bool vec_on = [] { const char* e = getenv("AM_HIP_CONV_GATHER"); return !(e && strcmp(e, "scalar") == 0); }();   // tests
  if (vec_on && cg.in_w == (int)sizeof(T) && cg.sw == 1 && cg.Wo % VK == 0 && cg.W >= VK)
    hipLaunchKernelGGL((gemm_mfma<T, MF, BM, BN, BK, WAVES_M, WAVES_N, PF, FPF, RU, kKContig, kGatherVec>), grid, block, 0, stream(), g);
  else
    hipLaunchKernelGGL((gemm_mfma<T, MF, BM, BN, BK, WAVES_M, WAVES_N, PF, FPF, RU, kKContig, kGather>), grid, block, 0, stream(), g);
  AM_TRY(check_launch("gemm_mfma (convolution)"));
  if (g.splits > 1) return launch_splitk_reduce<T, T>(g);
  return AM_OK;
}

// The weight gradient of a convolution as one long-k GEMM whose B operand is gathered from the images (kGatherVecT):
// A = grad_output as [C_out, N * P] with unit stride along k.
template <typename T, int BM, int BN, int BK, int WAVES_M, int WAVES_N, int PF = 1, bool FPF = true, bool RU = true, typename MF = Mfma<T>>
static int launch_conv_grad_weight(Args<T>& g) {
  g.tiles_m = (int)((g.M + BM - 1) / BM);
  g.tiles_n = (int)((g.N + BN - 1) / BN);
  const int64_t nb = (int64_t)g.tiles_m * g.tiles_n;
  if (nb >= ((int64_t)1 << 31)) return fail(AM_E_SHAPE, "conv2d_grad_weight: too many tiles");
  plan_splitk(g, BK, WAVES_M * WAVES_N);
  const dim3 grid((unsigned)(nb * g.splits), 1u), block(WAVES_M * WAVES_N * 64);
  hipLaunchKernelGGL((gemm_mfma<T, MF, BM, BN, BK, WAVES_M, WAVES_N, PF, FPF, RU, kKContig, kGatherVecT>), grid, block, 0, stream(), g);
  AM_TRY(check_launch("gemm_mfma (weight gradient of a convolution)"));
  if (g.splits > 1) return launch_splitk_reduce<T, T>(g);
  return AM_OK;
}

}  // namespace gemm
}  // namespace am
