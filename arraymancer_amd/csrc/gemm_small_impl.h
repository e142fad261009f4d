// Float GEMM for products with at most 64 rows (or, through the transposed problem, at most 64
// columns) and a modest amount of work: the dense layers of small-batch inference, e.g.
// [64 x 800] * [800 x 500] (src/arraymancer/nn_primitives/nnp_linear.nim:20-29) or the im2col
// products of a small convolution (nn_primitives/fallback/conv.nim:81-106).
//
// The tiled kernel handles such shapes with 32 x 32 tiles, one wavefront each, a split of k
// over workgroups and a second kernel that adds the partial tiles: a chain of global -> LDS ->
// register round trips whose latency nothing overlaps, 10 to 14 microseconds per product. Here
// there is no LDS staging and no second kernel:
//   - a workgroup of W wavefronts (1..4) owns one 16 x 16 tile of C; wavefront w multiplies a
//     contiguous share of the k range with v_mfma_*_16x16x4, loading its operand elements
//     straight from global memory in the register layout of the instruction (lane (i, g) =
//     (lane % 16, lane / 16) supplies A[m0 + i][k] and B[k][n0 + i] for one k per group g);
//   - within a block of 16 k, group g takes k = 4 g + s for step s = 0..3, so an operand with unit
//     stride along k is read with one 16-byte load per lane and block; any bijection between
//     (step, group) and k is legal as long as A and B use the same one;
//   - the W partial tiles are added in a fixed order through LDS and the first wavefront applies
//     alpha / beta / bias / ReLU exactly as the tiled kernel does.
// A wavefront keeps the loads of the next chunk of k in flight while it multiplies the current one.
#pragma once
#include "gemm_common.h"

namespace am {
namespace gemm {
namespace small {

template <typename T> struct M16;
template <> struct M16<float> {
  typedef float acc_t __attribute__((ext_vector_type(4)));
  static __device__ __forceinline__ acc_t mma(float a, float b, acc_t c) { return __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0); }
  // v_mfma_f32_16x16x4: register r of lane group g = lane / 16 holds row 4 g + r (column = lane % 16).
  static __device__ __forceinline__ int acc_row(int r, int lane) { return 4 * (lane >> 4) + r; }
};
template <> struct M16<double> {
  typedef double acc_t __attribute__((ext_vector_type(4)));
  static __device__ __forceinline__ acc_t mma(double a, double b, acc_t c) { return __builtin_amdgcn_mfma_f64_16x16x4f64(a, b, c, 0, 0, 0); }
  // v_mfma_f64_16x16x4: register r of lane group g holds row 4 r + g.
  static __device__ __forceinline__ int acc_row(int r, int lane) { return 4 * r + (lane >> 4); }
};

constexpr int kMaxWaves = 4;

// What the kernels of this file take: only the fields they read, packed into 160 bytes. A short kernel's first
// instructions wait for its arguments to arrive from memory; the general argument block spreads the fields these
// kernels need over six cache lines, which the compiler fetched in five dependent round trips (0.7 - 1.4 us before
// the first operand load was issued, a fifth of the kernel).
template <typename T> struct SmallArgs {
  const T* A; const T* B; T* C; const T* bias;
  int64_t a_mn, a_k, b_mn, b_k, c_m, c_n, bias_m, bias_n;
  int64_t M, N, K;
  long long* phase_out;            // PhaseProbe (common.h); null outside a phase window
  T alpha, beta;
  int epilogue, nw, phase_cap;     // nw: wavefronts per workgroup (reading blockDim costs another round trip)
  int per;                         // blocks of 16 k per wavefront = ceil(ceil(K / 16) / nw), from the host: a 64-bit division
                                   // by a run-time number is some 130 instructions in front of the kernel's first load
};
// Called first in a kernel: every field that the kernel reads early is wanted in a scalar register HERE, so that the
// compiler requests the three cache lines of the argument block together and waits once (left alone it requests each
// line where a field of it is first used, behind the branches in between: four dependent round trips).
template <typename T>
__device__ __forceinline__ void request_args(const SmallArgs<T>& p) {
  asm volatile("" ::"s"(p.A), "s"(p.B), "s"(p.C), "s"(p.a_mn), "s"(p.a_k), "s"(p.b_mn), "s"(p.b_k), "s"(p.c_m), "s"(p.c_n),
               "s"(p.M), "s"(p.N), "s"(p.K), "s"(p.phase_out), "s"(p.epilogue), "s"(p.nw), "s"(p.per));
}

template <typename T>
static inline SmallArgs<T> small_args(const Args<T>& g, int nw) {
  SmallArgs<T> s;
  s.A = g.A; s.B = g.B; s.C = g.C; s.bias = g.bias;
  s.a_mn = g.a_mn; s.a_k = g.a_k; s.b_mn = g.b_mn; s.b_k = g.b_k; s.c_m = g.c_m; s.c_n = g.c_n; s.bias_m = g.bias_m; s.bias_n = g.bias_n;
  s.M = g.M; s.N = g.N; s.K = g.K;
  s.phase_out = g.phase_out; s.alpha = g.alpha; s.beta = g.beta; s.epilogue = g.epilogue; s.nw = nw; s.phase_cap = g.phase_cap;
  s.per = (int)((((g.K + 15) >> 4) + nw - 1) / nw);
  return s;
}

// The four values lane group g feeds to the four steps of the 16-k block at kb: X[x + (kb + 4 g + s) * ld_k].
template <typename T, bool VEC>
__device__ __forceinline__ void load4(const T* x, int64_t ld_k, int64_t k, T (&out)[4]) {
  if constexpr (VEC) {
    constexpr int VK = 16 / (int)sizeof(T);
    typedef T vec_t __attribute__((ext_vector_type(VK)));
#pragma unroll
    for (int v = 0; v < 4 / VK; ++v) {
      const vec_t t = *(const vec_t*)(x + k + v * VK);
#pragma unroll
      for (int e = 0; e < VK; ++e) out[v * VK + e] = t[e];
    }
  } else {
#pragma unroll
    for (int s = 0; s < 4; ++s) out[s] = x[(k + s) * ld_k];
  }
}

// MAXW: most wavefronts per workgroup this instantiation is launched with (it sets the register budget);
// CHUNK: blocks of 16 k whose loads are issued together. The chunks of a wavefront's share are double
// buffered: the loads of chunk c + 1 are in flight while chunk c is multiplied.
template <typename T, bool AVEC, bool BVEC, int MAXW, int CHUNK>
__global__ __launch_bounds__(MAXW * 64) void gemm_rows16(SmallArgs<T> p) {
  typedef typename M16<T>::acc_t acc_t;
  extern __shared__ __attribute__((aligned(16))) unsigned char red_raw[];   // [W][256] partial tiles, W > 1 only
  T (*red)[256] = reinterpret_cast<T (*)[256]>(red_raw);
  request_args(p);
  // marks: 1 first loads issued, 2 they have arrived, 3 last matrix instruction and fold, 4 stores done
  PhaseProbe probe(p.phase_out, p.phase_cap, (unsigned)((p.N + 15) >> 4));
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = p.nw;
  const int i = lane & 15, g = lane >> 4;
  const int64_t m0 = (int64_t)blockIdx.y * 16, n0 = (int64_t)blockIdx.x * 16;
  // rows / columns past the edge read the last valid one; their results are not stored
  const int64_t arow = (m0 + i < p.M) ? m0 + i : p.M - 1, bcol = (n0 + i < p.N) ? n0 + i : p.N - 1;
  const T* a = p.A + arow * p.a_mn;
  const T* b = p.B + bcol * p.b_mn;

  // blocks of 16 k: nfull whole ones and possibly a partial one; wavefront w takes a contiguous share
  const int64_t nfull = p.K >> 4, nblk = (p.K + 15) >> 4;
  const int64_t per = p.per;
  const int64_t blk0 = (int64_t)wave * per;
  int64_t blk1 = blk0 + per;
  if (blk1 > nblk) blk1 = nblk;
  const int64_t full1 = blk1 < nfull ? blk1 : nfull;   // end of this wavefront's whole blocks

  acc_t acc = {0, 0, 0, 0};
  // The partial last block of the k range (elements past K count as zero), if this wavefront owns it:
  // requested first, multiplied last, so that its round trip to memory runs beside the whole blocks'.
  const bool has_tail = blk0 <= nfull && nfull < blk1;   // nfull is the number of the partial block, if there is one
  // (the values are kept as loaded and zeroed where they are multiplied: a select here would make the wavefront wait
  // for these loads before it has issued those of the whole blocks)
  T tail_a[4] = {0, 0, 0, 0}, tail_b[4] = {0, 0, 0, 0};
  const int64_t tail_k = (nfull << 4) + 4 * g;
  if (has_tail) {
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      const int64_t kk = tail_k + s < p.K ? tail_k + s : p.K - 1;
      tail_a[s] = a[kk * p.a_k];
      tail_b[s] = b[kk * p.b_k];
    }
  }
  T av[2][CHUNK][4], bv[2][CHUNK][4];
  auto load_chunk = [&](int set, int64_t first_blk) {   // set is a constant after unrolling
#pragma unroll
    for (int u = 0; u < CHUNK; ++u) {
      const int64_t k = ((first_blk + u) << 4) + 4 * g;
      load4<T, AVEC>(a, p.a_k, k, av[set][u]);
      load4<T, BVEC>(b, p.b_k, k, bv[set][u]);
    }
  };
  auto mma_chunk = [&](int set) {
#pragma unroll
    for (int u = 0; u < CHUNK; ++u)
#pragma unroll
      for (int s = 0; s < 4; ++s) acc = M16<T>::mma(av[set][u][s], bv[set][u][s], acc);
  };
  const int64_t nchunks = (full1 - blk0) / CHUNK;
  int64_t blk = blk0;
  if (nchunks > 0) {
    load_chunk(0, blk0);
    probe.mark(1);
    probe.settle();
    probe.mark(2);
    int64_t c = 0;
    for (; c + 2 <= nchunks; c += 2) {
      load_chunk(1, blk0 + (c + 1) * CHUNK);
      mma_chunk(0);
      const int64_t nxt = c + 2 < nchunks ? c + 2 : nchunks - 1;   // past the end: a harmless reload
      load_chunk(0, blk0 + nxt * CHUNK);
      mma_chunk(1);
    }
    if (c < nchunks) mma_chunk(0);
    blk = blk0 + nchunks * CHUNK;
  }
  // what is left of the whole blocks (fewer than CHUNK): halving groups, loads before matrix instructions
#pragma unroll
  for (int grp = CHUNK / 2; grp >= 1; grp /= 2) {
    if (blk + grp <= full1) {
#pragma unroll
      for (int u = 0; u < grp; ++u) {
        const int64_t k = ((blk + u) << 4) + 4 * g;
        load4<T, AVEC>(a, p.a_k, k, av[0][u]);
        load4<T, BVEC>(b, p.b_k, k, bv[0][u]);
      }
#pragma unroll
      for (int u = 0; u < grp; ++u)
#pragma unroll
        for (int s = 0; s < 4; ++s) acc = M16<T>::mma(av[0][u][s], bv[0][u][s], acc);
      blk += grp;
    }
  }
  if (has_tail) {
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      const bool ok = tail_k + s < p.K;
      acc = M16<T>::mma(ok ? tail_a[s] : (T)0, ok ? tail_b[s] : (T)0, acc);
    }
  }

  if (nchunks <= 0) { probe.mark(1); probe.settle(); probe.mark(2); }
  if (nw > 1) {
#pragma unroll
    for (int r = 0; r < 4; ++r) red[wave][r * 64 + lane] = acc[r];
    __syncthreads();
    if (wave != 0) return;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      T sum = red[0][r * 64 + lane];
      for (int w = 1; w < nw; ++w) sum += red[w][r * 64 + lane];   // fixed order: the result does not depend on timing
      acc[r] = sum;
    }
  }
  if (probe.out) { acc_t pin = acc; asm volatile("s_nop 0" : "+v"(pin)); acc = pin; }   // the accumulators are final before the mark is read
  probe.mark(3);

  // Epilogue (gemm_ukernel_generic.nim:53-125): beta == 0 never reads C; C *= beta, then
  // C += alpha * AB, each rounded on its own; then the optional fused bias / ReLU.
  const T alpha = p.alpha, beta = p.beta;
  const bool has_bias = (p.epilogue & AM_EPI_BIAS) != 0, relu = (p.epilogue & AM_EPI_RELU) != 0;
  const int64_t col = n0 + i;
  T cv[4], bias[4];
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const int64_t row = m0 + M16<T>::acc_row(r, lane);
    const bool ok = row < p.M && col < p.N;
    cv[r] = (ok && beta != (T)0) ? p.C[row * p.c_m + col * p.c_n] : (T)0;
    bias[r] = (ok && has_bias) ? p.bias[row * p.bias_m + col * p.bias_n] : (T)0;
  }
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const int64_t row = m0 + M16<T>::acc_row(r, lane);
    if (row < p.M && col < p.N) {
      T ab = acc[r];
      if (alpha != (T)1) ab = alpha * ab;
      T v = ab;
      if (beta != (T)0) {
        T c = cv[r];
        if (beta != (T)1) c = c * beta;
        v = c + ab;
      }
      if (has_bias) v = v + bias[r];
      if (relu) v = ((T)0 >= v) ? (T)0 : v;
      p.C[row * p.c_m + col * p.c_n] = v;
    }
  }
  probe.settle();
  probe.mark(4);
  probe.finish();
}

// The same product when B has unit stride along n (a row-major [k x n] operand, e.g. x * W with W stored
// [in x out]): a workgroup owns 16 rows x 16 VN columns (VN = elements per 16 bytes), i.e. VN tiles that share
// one A fragment. Lane (i, g) reads B[k][n0 + VN i .. n0 + VN i + VN - 1] with one 16-byte load per k and gives
// element j to tile j, so tile j holds the columns n0 + VN i + j: a permutation of the block's columns under which
// a lane ends up with VN consecutive columns of each of its rows, stored with one 16-byte store when C has unit
// stride along n. Against gemm_rows16 on the same operand: a quarter of the load instructions (an eighth for A),
// 16-byte instead of 64-byte runs on both B and C, and VN independent accumulator chains per wavefront.
// Requires N % VN == 0 (no vector crosses the end of a row of B).
template <typename T, bool AVEC, int MAXW, int CHUNK>
__global__ __launch_bounds__(MAXW * 64) void gemm_rows16n(SmallArgs<T> p) {
  typedef typename M16<T>::acc_t acc_t;
  constexpr int VN = 16 / (int)sizeof(T);
  typedef T vec_t __attribute__((ext_vector_type(VN)));
  extern __shared__ __attribute__((aligned(16))) unsigned char red_raw[];   // [W][VN][256] partial tiles, W > 1 only
  T (*red)[VN * 256] = reinterpret_cast<T (*)[VN * 256]>(red_raw);
  request_args(p);
  PhaseProbe probe(p.phase_out, p.phase_cap, (unsigned)((p.N + 16 * VN - 1) / (16 * VN)));   // marks as in gemm_rows16
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = p.nw;
  const int i = lane & 15, g = lane >> 4;
  const int64_t m0 = (int64_t)blockIdx.y * 16, n0 = (int64_t)blockIdx.x * (16 * VN);
  // rows / column vectors past the edge read the last valid one; their results are not stored
  const int64_t arow = (m0 + i < p.M) ? m0 + i : p.M - 1;
  const int64_t col0 = n0 + VN * i, bcol = (col0 < p.N) ? col0 : p.N - VN;
  const T* a = p.A + arow * p.a_mn;
  const T* b = p.B + bcol;

  const int64_t nfull = p.K >> 4, nblk = (p.K + 15) >> 4;
  const int64_t per = p.per;
  const int64_t blk0 = (int64_t)wave * per;
  int64_t blk1 = blk0 + per;
  if (blk1 > nblk) blk1 = nblk;
  const int64_t full1 = blk1 < nfull ? blk1 : nfull;

  acc_t acc[VN];
#pragma unroll
  for (int j = 0; j < VN; ++j) acc[j] = acc_t{0, 0, 0, 0};
  const bool has_tail = blk0 <= nfull && nfull < blk1;
  T tail_a[4] = {0, 0, 0, 0};
  vec_t tail_b[4];
#pragma unroll
  for (int s = 0; s < 4; ++s) tail_b[s] = vec_t{};
  const int64_t tail_k = (nfull << 4) + 4 * g;
  if (has_tail) {   // kept as loaded, zeroed where they are multiplied (see gemm_rows16)
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      const int64_t kk = tail_k + s < p.K ? tail_k + s : p.K - 1;
      tail_a[s] = a[kk * p.a_k];
      tail_b[s] = *(const vec_t*)(b + kk * p.b_k);
    }
  }
  T av[2][CHUNK][4];
  vec_t bv[2][CHUNK][4];
  auto load_blocks = [&](int set, int64_t first_blk, int count) {   // set and count are constants after unrolling
#pragma unroll
    for (int u = 0; u < count; ++u) {
      const int64_t k = ((first_blk + u) << 4) + 4 * g;
      load4<T, AVEC>(a, p.a_k, k, av[set][u]);
#pragma unroll
      for (int s = 0; s < 4; ++s) bv[set][u][s] = *(const vec_t*)(b + (k + s) * p.b_k);
    }
  };
  auto mma_blocks = [&](int set, int count) {
#pragma unroll
    for (int u = 0; u < count; ++u)
#pragma unroll
      for (int s = 0; s < 4; ++s)
#pragma unroll
        for (int j = 0; j < VN; ++j) acc[j] = M16<T>::mma(av[set][u][s], bv[set][u][s][j], acc[j]);
  };
  const int64_t nchunks = (full1 - blk0) / CHUNK;
  int64_t blk = blk0;
  if (nchunks > 0) {
    load_blocks(0, blk0, CHUNK);
    probe.mark(1);
    probe.settle();
    probe.mark(2);
    int64_t c = 0;
    for (; c + 2 <= nchunks; c += 2) {
      load_blocks(1, blk0 + (c + 1) * CHUNK, CHUNK);
      mma_blocks(0, CHUNK);
      const int64_t nxt = c + 2 < nchunks ? c + 2 : nchunks - 1;   // past the end: a harmless reload
      load_blocks(0, blk0 + nxt * CHUNK, CHUNK);
      mma_blocks(1, CHUNK);
    }
    if (c < nchunks) mma_blocks(0, CHUNK);
    blk = blk0 + nchunks * CHUNK;
  }
#pragma unroll
  for (int grp = CHUNK / 2; grp >= 1; grp /= 2) {
    if (blk + grp <= full1) {
      load_blocks(0, blk, grp);
      mma_blocks(0, grp);
      blk += grp;
    }
  }
  if (has_tail) {
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      const bool ok = tail_k + s < p.K;
      const T x = ok ? tail_a[s] : (T)0;
#pragma unroll
      for (int j = 0; j < VN; ++j) acc[j] = M16<T>::mma(x, ok ? tail_b[s][j] : (T)0, acc[j]);
    }
  }

  if (nchunks <= 0) { probe.mark(1); probe.settle(); probe.mark(2); }
  if (nw > 1) {
#pragma unroll
    for (int j = 0; j < VN; ++j)
#pragma unroll
      for (int r = 0; r < 4; ++r) red[wave][(j * 4 + r) * 64 + lane] = acc[j][r];
    __syncthreads();
    if (wave != 0) return;
#pragma unroll
    for (int j = 0; j < VN; ++j)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        T sum = red[0][(j * 4 + r) * 64 + lane];
        for (int w = 1; w < nw; ++w) sum += red[w][(j * 4 + r) * 64 + lane];   // fixed order
        acc[j][r] = sum;
      }
  }

  // Epilogue: the same steps, each rounded on its own, as gemm_rows16 (gemm_ukernel_generic.nim:53-125)
  const T alpha = p.alpha, beta = p.beta;
  const bool has_bias = (p.epilogue & AM_EPI_BIAS) != 0, relu = (p.epilogue & AM_EPI_RELU) != 0;
  const bool cvec = p.c_n == 1;
  if (probe.out) { acc_t pin = acc[0]; asm volatile("s_nop 0" : "+v"(pin)); acc[0] = pin; }
  probe.mark(3);
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const int64_t row = m0 + M16<T>::acc_row(r, lane);
    if (row >= p.M || col0 >= p.N) continue;
    T* c = p.C + row * p.c_m + col0 * p.c_n;
    vec_t old = vec_t{};
    if (beta != (T)0) {
      if (cvec) old = *(const vec_t*)c;
      else {
#pragma unroll
        for (int j = 0; j < VN; ++j) old[j] = c[j * p.c_n];
      }
    }
    vec_t out;
#pragma unroll
    for (int j = 0; j < VN; ++j) {
      T ab = acc[j][r];
      if (alpha != (T)1) ab = alpha * ab;
      T v = ab;
      if (beta != (T)0) {
        T cc = old[j];
        if (beta != (T)1) cc = cc * beta;
        v = cc + ab;
      }
      if (has_bias) v = v + p.bias[row * p.bias_m + (col0 + j) * p.bias_n];
      if (relu) v = ((T)0 >= v) ? (T)0 : v;
      out[j] = v;
    }
    if (cvec) *(vec_t*)c = out;
    else {
#pragma unroll
      for (int j = 0; j < VN; ++j) c[j * p.c_n] = out[j];
    }
  }
  probe.settle();
  probe.mark(4);
  probe.finish();
}

// Whether this product belongs here: few rows or few columns, little work, not a batch member.
// AM_HIP_GEMM_SMALL = 0 / 1 in the environment turns the path off / forces it where its limits allow (tests).
template <typename T>
static inline bool applicable(const Args<T>& g) {
  const char* e = getenv("AM_HIP_GEMM_SMALL");
  const int forced = (e && *e) ? atoi(e) : -1;
  if (forced == 0 || g.batch > 1) return false;
  const int64_t mn = g.M < g.N ? g.M : g.N;
  if (mn > 64) return false;
  if (forced == 1) return true;
  const double macs = (double)g.M * (double)g.N * (double)g.K;
  if (!(macs <= 268435456.0 && g.K <= 8192)) return false;
  // Where 32 x 32 tiles of the LDS-staged kernel already give every CU a workgroup without any split of k, that kernel
  // is ahead: its operands cross the vector L1 once per 32 x 32 tile instead of once per 16 x 16 tile, and the number of
  // L1 accesses is what bounds such a product here ([50 x 500] * [500 x 4096]: 7.3 against 8.0 us). A short k is not worth
  // the staging ([20 x 25] * [25 x 36864]: 6.2 against 6.0).
  const int64_t tiles32 = ((g.M + 31) / 32) * ((g.N + 31) / 32);
  return !(tiles32 >= (int64_t)num_cus() && g.K >= 128);
}

template <typename T>
static int run(const Args<T>& g_in) {
  constexpr int64_t VK = 16 / (int64_t)sizeof(T);
  Args<T> g = g_in;
  if (g.M > 64) {   // few columns: the transposed problem C^T = B^T A^T has few rows
    g.M = g_in.N; g.N = g_in.M;
    g.A = g_in.B; g.a_mn = g_in.b_mn; g.a_k = g_in.b_k;
    g.B = g_in.A; g.b_mn = g_in.a_mn; g.b_k = g_in.a_k;
    g.c_m = g_in.c_n; g.c_n = g_in.c_m;
    g.bias_m = g_in.bias_n; g.bias_n = g_in.bias_m;
  }
  // B with unit stride along n (and no unit stride along k): the kernel whose wavefronts own VK tiles side by side
  // Measured: it wins (6.1 -> 5.2 us on [20 x 25] * [25 x 36864], 7.9 -> 5.8 on [16 x 64] * [64 x 65536], float64 15.2 -> 9.1
  // on [64 x 256] * [256 x 8192]) where its fewer, wider tiles still give every SIMD of the chip a wavefront, and loses
  // below that (a wavefront's chain of load round trips is what such a product costs, and fewer wavefronts means longer
  // chains). AM_HIP_GEMM_SMALL_NVEC = 0 / 2 in the environment turns it off / forces it where it is legal (tests).
  const char* nv = getenv("AM_HIP_GEMM_SMALL_NVEC");
  const int nvec_mode = (nv && *nv) ? atoi(nv) : 1;
  const bool nvec_legal = g.b_mn == 1 && g.b_k != 1 && g.N % VK == 0 && g.N >= 8 * VK;
  const bool nvec = nvec_legal && nvec_mode != 0 &&
                    (nvec_mode == 2 || ((g.M + 15) / 16) * ((g.N + 16 * VK - 1) / (16 * VK)) >= (int64_t)num_cus() * 4);
  const int64_t tile_cols = nvec ? 16 * VK : 16;
  const int64_t tiles_m = (g.M + 15) / 16, tiles_n = (g.N + tile_cols - 1) / tile_cols;
  if (tiles_n >= ((int64_t)1 << 31)) return fail(AM_E_SHAPE, "gemm: too many tiles");
  // Wavefronts per tile: about one per SIMD over the chip and at most four (measured: starting more
  // wavefronts costs more than the latency they would hide), every one with at least two blocks of 16 k.
  const int64_t tiles = tiles_m * tiles_n, nblk = (g.K + 15) / 16;
  int64_t want = (int64_t)num_cus() * 4 / tiles;
  if (want > nblk / 2) want = nblk / 2;
  int nw = 1;
  while (nw * 2 <= want && nw * 2 <= kMaxWaves) nw *= 2;
  if (const char* e = getenv("AM_HIP_GEMM_SMALL_W")) { const int w = atoi(e); if (w >= 1 && w <= kMaxWaves) nw = w; }   // tests
  const size_t lds = nw > 1 ? (size_t)nw * 256 * sizeof(T) * (nvec ? VK : 1) : 0;
  const bool avec = g.a_k == 1 && aligned16(g.A) && (g.a_mn % VK == 0 || g.M == 1);
  const bool bvec = g.b_k == 1 && aligned16(g.B) && (g.b_mn % VK == 0 || g.N == 1);
  const dim3 grid((unsigned)tiles_n, (unsigned)tiles_m), block((unsigned)nw * 64);
  const SmallArgs<T> sa = small_args(g, nw);
  if (trace_choices()) fprintf(stderr, "am_hip gemm: small path, %lld x %lld tiles of 16 x 16, %d wavefronts per tile\n", (long long)tiles_m, (long long)tiles_n, nw);
  // Chunks of four (float) or two (double) blocks of 16 k where a wavefront has that many; one block at a
  // time where its share of k is one or two blocks: that instantiation needs a third of the registers,
  // so all the wavefronts of a product with many tiles and a short k are resident at once.
  constexpr int CH = sizeof(T) == 4 ? 4 : 2;
  const bool short_k = (nblk + nw - 1) / nw <= 2;
  if (nvec) {
    if (trace_choices()) fprintf(stderr, "am_hip gemm: small path, B in 16-byte vectors along n\n");
    constexpr int CHN = 2;
    if (short_k) {
      if (avec) hipLaunchKernelGGL((gemm_rows16n<T, true, kMaxWaves, 1>), grid, block, lds, stream(), sa);
      else hipLaunchKernelGGL((gemm_rows16n<T, false, kMaxWaves, 1>), grid, block, lds, stream(), sa);
    } else {
      if (avec) hipLaunchKernelGGL((gemm_rows16n<T, true, kMaxWaves, CHN>), grid, block, lds, stream(), sa);
      else hipLaunchKernelGGL((gemm_rows16n<T, false, kMaxWaves, CHN>), grid, block, lds, stream(), sa);
    }
    return check_launch("gemm_rows16n");
  }
#define AM_SMALL_LAUNCH(AV, BV)                                                                              \
  do {                                                                                                       \
    if (short_k) hipLaunchKernelGGL((gemm_rows16<T, AV, BV, kMaxWaves, 1>), grid, block, lds, stream(), sa);   \
    else hipLaunchKernelGGL((gemm_rows16<T, AV, BV, kMaxWaves, CH>), grid, block, lds, stream(), sa);          \
  } while (0)
  if (avec && bvec) AM_SMALL_LAUNCH(true, true);
  else if (avec) AM_SMALL_LAUNCH(true, false);
  else if (bvec) AM_SMALL_LAUNCH(false, true);
  else AM_SMALL_LAUNCH(false, false);
#undef AM_SMALL_LAUNCH
  return check_launch("gemm_rows16");
}

}  // namespace small
}  // namespace gemm
}  // namespace am
