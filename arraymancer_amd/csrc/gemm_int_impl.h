// Integer GEMM for gfx950: int32 and int64 have no matrix-core instruction, so the product runs
// on the vector ALU as an LDS-tiled register-blocked multiply-accumulate. All arithmetic is
// carried out in the unsigned twin of the element type, i.e. modulo 2^32 / 2^64 — the same
// wraparound the reference's SIMD integer micro-kernels have
// (src/arraymancer/laser/primitives/matrix_multiplication/gemm_ukernel_avx2.nim:15-16,
//  gemm_ukernel_sse2.nim:111-119). Ring arithmetic is order independent, so every bit of C is
// fixed regardless of the tiling.
//
// Decomposition: workgroup of 256 lanes (16 x 16) per BM x BN tile of C; lane (ty, tx) owns a
// TM x TN register tile made of TM/VK row chunks and TN/VK column chunks of VK consecutive
// elements (VK = 16 bytes / sizeof(T)), chunk c at offset c * 16 * VK + t * VK, so that the 16
// lanes of a row read one contiguous 16 * 16-byte run of LDS (no bank conflicts) and lanes that
// share ty read the same A address (broadcast). Both operands sit in LDS as [k][mn] slabs,
// double-buffered exactly like the MFMA kernels; the same three loaders (unit stride along k,
// unit stride along m/n, arbitrary strides) feed them, so views never need a host copy.
#pragma once
#include "gemm_loader.h"

namespace am {
namespace gemm {

template <typename T> struct UnsignedOf;
// `acc` is the accumulator type: for int32 it is 64 bits wide so that every multiply-accumulate is
// ONE v_mad_u64_u32 (its low 32 bits are the wrapped 32-bit MAC; the high half is never used),
// instead of v_mul_lo_u32 + v_add (1.5 instructions per MAC after the compiler pairs the adds).
template <> struct UnsignedOf<int32_t> { typedef uint32_t type; typedef uint64_t acc; };
template <> struct UnsignedOf<int64_t> { typedef uint64_t type; typedef uint64_t acc; };

template <typename T, int TM, int TN, int BK, int AK, int BKIND>
__global__ __launch_bounds__(256, 2) void gemm_valu(Args<T> p) {
  typedef typename UnsignedOf<T>::type U;
  typedef typename UnsignedOf<T>::acc ACC;
  typedef typename VecTraits<T>::vec_t vec_t;
  constexpr int VK = VecTraits<T>::VK;
  constexpr int NT = 256, BM = 16 * TM, BN = 16 * TN;
  constexpr int CM = TM / VK, CN = TN / VK;   // chunks per lane along m / n
  static_assert(TM % VK == 0 && TN % VK == 0, "register tile must be whole 16-byte chunks");
  constexpr int LDA = Slab<T, AK, BM, BK, false>::LDMN, LDB = Slab<T, BKIND, BN, BK, false>::LDMN;

  __shared__ __attribute__((aligned(16))) T sA[2][BK * LDA];
  __shared__ __attribute__((aligned(16))) T sB[2][BK * LDB];

  if (p.gate_flags != nullptr && live_digit_pairs<(int)sizeof(T)>(p.gate_flags, p.gate_gen) <= p.gate_max_pairs) return;
  const ClockProbe probe(p.clock_out);
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
  const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;

  Loader<T, AK, BM, BK, NT, false> la(p.A, p.a_mn, p.a_k, m0, p.M, k_end, p.a_kfast);
  Loader<T, BKIND, BN, BK, NT, false> lb(p.B, p.b_mn, p.b_k, n0, p.N, k_end, p.b_kfast);

  ACC acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j) acc[i][j] = 0;

  const int64_t ktiles = (k_end - k_begin + BK - 1) / BK;
  la.fetch(k_begin);
  lb.fetch(k_begin);
  la.commit(sA[0], k_begin);
  lb.commit(sB[0], k_begin);
  __syncthreads();

  for (int64_t kt = 0; kt < ktiles; ++kt) {
    const int cur = (int)(kt & 1);
    const bool more = (kt + 1) < ktiles;
    if (more) {
      la.fetch(k_begin + (kt + 1) * BK);
      lb.fetch(k_begin + (kt + 1) * BK);
    }
    const T* a_lds = sA[cur];
    const T* b_lds = sB[cur];
#pragma unroll 2
    for (int k = 0; k < BK; ++k) {
      U a[TM], b[TN];
#pragma unroll
      for (int c = 0; c < CM; ++c) {
        const vec_t v = *(const vec_t*)(a_lds + k * LDA + c * 16 * VK + ty * VK);
#pragma unroll
        for (int e = 0; e < VK; ++e) a[c * VK + e] = (U)v[e];
      }
#pragma unroll
      for (int c = 0; c < CN; ++c) {
        const vec_t v = *(const vec_t*)(b_lds + k * LDB + c * 16 * VK + tx * VK);
#pragma unroll
        for (int e = 0; e < VK; ++e) b[c * VK + e] = (U)v[e];
      }
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) acc[i][j] += (ACC)a[i] * (ACC)b[j];
    }
    if (more) {
      la.commit(sA[cur ^ 1], k_begin + (kt + 1) * BK);
      lb.commit(sB[cur ^ 1], k_begin + (kt + 1) * BK);
    }
    __syncthreads();
  }

  // Epilogue: same case analysis as the reference (gemm_ukernel_generic.nim:53-125), mod 2^w.
  if (p.splits > 1) {   // split-K: raw partial sums (mod 2^w) to the workspace
    T* ws = p.ws + (int64_t)split * p.M * p.N;
#pragma unroll
    for (int i = 0; i < TM; ++i) {
      const int64_t row = m0 + (i / VK) * 16 * VK + ty * VK + (i % VK);
      if (row >= p.M) continue;
#pragma unroll
      for (int j = 0; j < TN; ++j) {
        const int64_t col = n0 + (j / VK) * 16 * VK + tx * VK + (j % VK);
        if (col < p.N) ws[row * p.N + col] = (T)(U)acc[i][j];
      }
    }
    probe.finish();
    return;
  }
  const U alpha = (U)p.alpha, beta = (U)p.beta;
#pragma unroll
  for (int i = 0; i < TM; ++i) {
    const int64_t row = m0 + (i / VK) * 16 * VK + ty * VK + (i % VK);
    if (row >= p.M) continue;
    // all loads of this row of C first, then the arithmetic and the stores: a load issued after a
    // store would wait for that store (one memory counter orders both)
    U cv[TN];
    if (beta != 0) {
#pragma unroll
      for (int j = 0; j < TN; ++j) {
        const int64_t col = n0 + (j / VK) * 16 * VK + tx * VK + (j % VK);
        cv[j] = (col < p.N) ? (U)p.C[row * p.c_m + col * p.c_n] : (U)0;
      }
    }
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const int64_t col = n0 + (j / VK) * 16 * VK + tx * VK + (j % VK);
      if (col < p.N) {
        U v = alpha * (U)acc[i][j];
        if (beta != 0) v += beta * cv[j];
        p.C[row * p.c_m + col * p.c_n] = (T)v;
      }
    }
  }
  probe.finish();
}

template <typename T, int TM, int TN, int BK>
static int launch_valu(Args<T>& g, int ak, int bk, int want_splits) {
  constexpr int BM = 16 * TM, BN = 16 * TN;
  g.tiles_m = (int)((g.M + BM - 1) / BM);
  g.tiles_n = (int)((g.N + BN - 1) / BN);
  const int64_t nb = (int64_t)g.tiles_m * g.tiles_n;
  if (nb >= ((int64_t)1 << 31)) return fail(AM_E_SHAPE, "gemm: too many tiles");
  apply_splitk(g, BK, want_splits);
  const dim3 grid((unsigned)(nb * g.splits), (unsigned)g.batch), block(256);
#define AM_LAUNCH(AKIND, BKIND_) \
  hipLaunchKernelGGL((gemm_valu<T, TM, TN, BK, AKIND, BKIND_>), grid, block, 0, stream(), g)
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
  AM_TRY(check_launch("gemm_valu"));
  // ring arithmetic: the reduction runs in the unsigned twin, so it wraps like the main kernel
  if (g.splits > 1) return launch_splitk_reduce<T, typename UnsignedOf<T>::type>(g);
  return AM_OK;
}

}  // namespace gemm
}  // namespace am
