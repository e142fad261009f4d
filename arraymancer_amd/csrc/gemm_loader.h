// Global -> register -> LDS movers for one operand slab of a GEMM workgroup tile, shared by the
// MFMA (f32/f64) and VALU (i32/i64) kernels. An operand is X(mn, k) = X[mn * ld_mn + k * ld_k];
// a slab is BMN rows/cols by BK k values. Out-of-range elements are zero-filled.
//
// LDS layouts:
//   k-group  [k / VK][mn][VK]   (16-byte slot per (k-group, mn)); only for kKContig with KG = true
//   k-row    [k][mn]            everything else
// VK = 16 bytes / sizeof(T).
#pragma once
#include "gemm_common.h"

namespace am {
namespace gemm {

// vec_t: a 16-byte vector in registers / LDS. gvec_t: the same vector as it sits in global memory, where only
// the element's own alignment is promised (a row of 4095 floats starts 4 bytes off every 16): the hardware
// serves a 16-byte global load from any dword-aligned address, so an operand with a unit stride is moved in
// 16-byte pieces whatever its row pitch, extent or base address.
template <typename T> struct VecTraits;
template <> struct VecTraits<float> { static constexpr int VK = 4; typedef float vec_t __attribute__((ext_vector_type(4))); typedef vec_t gvec_t __attribute__((aligned(4))); };
template <> struct VecTraits<double> { static constexpr int VK = 2; typedef double vec_t __attribute__((ext_vector_type(2))); typedef vec_t gvec_t __attribute__((aligned(8))); };
template <> struct VecTraits<int32_t> { static constexpr int VK = 4; typedef int32_t vec_t __attribute__((ext_vector_type(4))); typedef vec_t gvec_t __attribute__((aligned(4))); };
template <> struct VecTraits<int64_t> { static constexpr int VK = 2; typedef int64_t vec_t __attribute__((ext_vector_type(2))); typedef vec_t gvec_t __attribute__((aligned(8))); };

// LDS geometry of one operand slab (BMN rows/cols x BK k values).
template <typename T, int KIND, int BMN, int BK, bool KG = true> struct Slab {
  static constexpr int VK = VecTraits<T>::VK;
  // Padding of the k-group planes. A 16-byte LDS access is served 8 lanes at a time (8 x 16 B =
  // all 32 banks); the 8 lanes of a global->LDS write step through the BK/VK k-groups of a row
  // first, so consecutive planes must start 8/(BK/VK) slots apart modulo 8 to spread them over
  // the banks (measured on f64: +7 % over a padding that is a multiple of 4).
  static constexpr int QN_ = BK / VK;
  static constexpr int LDKG = BMN + (QN_ >= 8 ? 1 : 8 / QN_);   // 16-byte slots per k-group plane
  static constexpr int LDMN = BMN + 4;   // k-row layout: elements per k row (4 * LDMN mod 32 banks = 16: the
                                         // four k-rows a transposing write touches fall on two bank halves, not one)
  static constexpr int ELEMS = (k_grouped(KIND) && KG) ? (BK / VK) * LDKG * VK : BK * LDMN;
};

// Moves one operand slab global -> registers (fetch) -> LDS (commit). PF register stages let PF
// slabs be in flight at once: fetch<S> fills stage S, commit<S> writes stage S to LDS.
//
// fetch is branch-free and unconditional: every lane always loads, from an address clamped into
// the operand. (Loads under a branch would keep the compiler from counting the loads in flight,
// and every wait would then be a wait for all of them, including those just issued for a later
// slab.) What the clamping brings in is dealt with as follows:
//   * rows / columns past the edge of the operand (edge tiles) repeat the last valid one; they
//     only ever reach rows / columns of C past its edge, which the store masks;
//   * k values past the end of the k range can only occur in a range's last slab; commit zeroes
//     them in both operands, so that 0 * Inf never arises. A slab wholly past the end is not
//     fetched at all (wave-uniform test) and commits as zeros. MASK = false versions of fetch and
//     commit skip the k clamping and zeroing: for slabs known to lie wholly inside the k range.
template <typename T, int KIND, int BMN, int BK, int NT, bool KG = true, int PF = 1> struct Loader;

template <typename T, int BMN, int BK, int NT, bool KG, int PF> struct Loader<T, kKContig, BMN, BK, NT, KG, PF> {
  typedef typename VecTraits<T>::vec_t vec_t;
  typedef typename VecTraits<T>::gvec_t gvec_t;
  static constexpr int VK = VecTraits<T>::VK;
  static constexpr int QN = BK / VK;               // vectors per row
  static constexpr int NV = BMN * QN / NT;         // vectors per thread
  static_assert(BMN * QN % NT == 0 && NV >= 1, "slab must divide evenly over the workgroup");
  const T* ptr[NV];
  int64_t K;
  vec_t reg[PF][NV];
  __device__ __forceinline__ Loader(const T* X, int64_t ld_mn, int64_t, int64_t mn0, int64_t MN, int64_t K_, int, const ConvGeom* = nullptr) : K(K_) {
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int v = threadIdx.x + i * NT;
      const int q = v % QN, mn = v / QN;
      ptr[i] = X + ((mn0 + mn) < MN ? mn0 + mn : MN - 1) * ld_mn + q * VK;
    }
  }
  __device__ __forceinline__ bool tail_guard() const { return false; }
  template <int S = 0, bool MASK = true> __device__ __forceinline__ void fetch(int64_t k0) {
    if (MASK && k0 >= K) return;   // slab wholly past the end: commit writes zeros without these registers
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int q = (threadIdx.x + i * NT) % QN;
      if constexpr (MASK) {
        // A vector that straddles the end of the k range (K not a multiple of VK) is read from where it
        // ends at K instead and moved into place (what lies past K is zeroed): nothing past the last element
        // of a row is ever touched. A vector wholly past the end repeats the row's first one. (The host sends
        // k ranges shorter than one vector to the element-wise loader.)
        const int64_t kv = k0 + q * VK;
        if (K % VK != 0) {   // uniform
          const int64_t over = kv + VK - K;                       // elements past the end, if positive
          const bool straddles = over > 0 && over < VK;
          const vec_t v = *(const gvec_t*)(ptr[i] + (kv >= K ? (int64_t)(-q * VK) : straddles ? k0 - over : k0));
          vec_t r = v;
          if (straddles) {
#pragma unroll
            for (int e = 0; e < VK; ++e) {
              T x = (T)0;
#pragma unroll
              for (int f = 0; f < VK; ++f) x = (e + over == f) ? v[f] : x;
              r[e] = x;
            }
          }
          reg[S][i] = r;
        } else {
          reg[S][i] = *(const gvec_t*)(ptr[i] + (kv >= K ? (int64_t)(-q * VK) : k0));
        }
      } else {
        reg[S][i] = *(const gvec_t*)(ptr[i] + k0);
      }
    }
  }
  template <int S = 0, bool MASK = true> __device__ __forceinline__ void commit(T* lds, int64_t k0) {
    if (MASK && k0 >= K) {   // nothing was fetched: zeros, without waiting for any load
#pragma unroll
      for (int i = 0; i < NV; ++i) { vec_t z = {}; reg[S][i] = z; }
    } else if (MASK && k0 + BK > K) {
#pragma unroll
      for (int i = 0; i < NV; ++i) {
        const int q = (threadIdx.x + i * NT) % QN;
#pragma unroll
        for (int e = 0; e < VK; ++e)
          if ((k0 + q * VK + e) >= K) reg[S][i][e] = (T)0;
      }
    }
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int v = threadIdx.x + i * NT;
      const int q = v % QN, mn = v / QN;
      if constexpr (KG) {
        constexpr int LD = Slab<T, kKContig, BMN, BK, true>::LDKG;
        *(vec_t*)(lds + (q * LD + mn) * VK) = reg[S][i];
      } else {  // k-row layout wanted: scatter the VK k values of this row
        constexpr int LD = Slab<T, kKContig, BMN, BK, false>::LDMN;
#pragma unroll
        for (int s = 0; s < VK; ++s) lds[(q * VK + s) * LD + mn] = reg[S][i][s];
      }
    }
  }
};

template <typename T, int BMN, int BK, int NT, bool KG, int PF> struct Loader<T, kMNContig, BMN, BK, NT, KG, PF> {
  typedef typename VecTraits<T>::vec_t vec_t;
  typedef typename VecTraits<T>::gvec_t gvec_t;
  static constexpr int VK = VecTraits<T>::VK;
  static constexpr int CN = BMN / VK;              // vectors per k row
  static constexpr int NV = CN * BK / NT;
  static_assert(CN * BK % NT == 0 && NV >= 1, "slab must divide evenly over the workgroup");
  const T* ptr[NV];
  int64_t K, ld_k;
  // The one vector per k row that straddles the edge of the operand (MN not a multiple of VK; edge tiles only)
  // reads up to VK - 1 elements past the end of its row. In every k row but the operand's last one those are
  // the first elements of the next row (the host sends operands whose rows overlap elsewhere), and what they
  // hold only reaches columns of C past its edge. The last row must not be overrun: the MASK = true versions,
  // which the kernel runs for the slab that holds it (tail_guard), read that vector from where it ends at MN,
  // `shift` elements back, and move it into place in registers.
  int shift[NV];
  bool shift_any;   // uniform over the workgroup
  vec_t reg[PF][NV];
  __device__ __forceinline__ Loader(const T* X, int64_t, int64_t ld_k_, int64_t mn0, int64_t MN, int64_t K_, int, const ConvGeom* = nullptr) : K(K_), ld_k(ld_k_) {
    shift_any = (MN % VK != 0) && (mn0 + BMN > MN);
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int v = threadIdx.x + i * NT;
      const int c = v % CN, k = v / CN;
      const int64_t col = mn0 + c * VK;
      const int64_t over = col + VK - MN;          // elements past the edge, if positive
      shift[i] = (over > 0 && over < VK) ? (int)over : 0;
      ptr[i] = X + (col < MN ? col : 0) + k * ld_k;
    }
  }
  // True when the unmasked fetch must not be used for the slab that holds the last k row.
  __device__ __forceinline__ bool tail_guard() const { return shift_any; }
  template <int S = 0, bool MASK = true> __device__ __forceinline__ void fetch(int64_t k0) {
    if (MASK && k0 >= K) return;
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int k = (threadIdx.x + i * NT) / CN;
      if constexpr (MASK) {
        const vec_t v = *(const gvec_t*)(ptr[i] - shift[i] + ((k0 + k) < K ? k0 : (int64_t)(-k)) * ld_k);
        vec_t r = v;
        if (shift_any) {
#pragma unroll
          for (int e = 0; e < VK; ++e) {
            T x = v[e];
#pragma unroll
            for (int f = 0; f < VK; ++f) x = (shift[i] != 0 && e + shift[i] == f) ? v[f] : x;
            r[e] = x;
          }
        }
        reg[S][i] = r;
      } else {
        reg[S][i] = *(const gvec_t*)(ptr[i] + k0 * ld_k);
      }
    }
  }
  template <int S = 0, bool MASK = true> __device__ __forceinline__ void commit(T* lds, int64_t k0) {
    constexpr int LD = Slab<T, kMNContig, BMN, BK>::LDMN;
    if (MASK && k0 >= K) {
#pragma unroll
      for (int i = 0; i < NV; ++i) { vec_t z = {}; reg[S][i] = z; }
    } else if (MASK && k0 + BK > K) {
#pragma unroll
      for (int i = 0; i < NV; ++i) {
        const int k = (threadIdx.x + i * NT) / CN;
        vec_t z = {};
        if ((k0 + k) >= K) reg[S][i] = z;
      }
    }
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int v = threadIdx.x + i * NT;
      const int c = v % CN, k = v / CN;
      *(vec_t*)(lds + k * LD + c * VK) = reg[S][i];
    }
  }
};

// Any strides (zero, negative, stepped): one element per load. Each lane keeps the address of its NE
// elements of slab 0 (row / column clamped into the operand); a slab's loads are those addresses plus
// k0 * ld_k, one 64-bit product per slab shared by all of them, instead of two per element.
template <typename T, int BMN, int BK, int NT, bool KG, int PF> struct Loader<T, kGeneric, BMN, BK, NT, KG, PF> {
  static constexpr int NE = BMN * BK / NT;         // elements per thread
  static_assert(BMN * BK % NT == 0 && NE >= 1, "slab must divide evenly over the workgroup");
  const T* ptr[NE];
  int64_t ld_k, K;
  int kfast;
  T reg[PF][NE];
  __device__ __forceinline__ void coords(int i, int& mn, int& k) const {
    const int e = threadIdx.x + i * NT;
    if (kfast) { k = e % BK; mn = e / BK; } else { mn = e % BMN; k = e / BMN; }
  }
  __device__ __forceinline__ Loader(const T* X, int64_t ld_mn, int64_t ld_k_, int64_t mn0, int64_t MN, int64_t K_, int kfast_, const ConvGeom* = nullptr)
      : ld_k(ld_k_), K(K_), kfast(kfast_) {
#pragma unroll
    for (int i = 0; i < NE; ++i) {
      int mn, k;
      coords(i, mn, k);
      const int64_t cm = (mn0 + mn) < MN ? mn0 + mn : MN - 1;
      ptr[i] = X + cm * ld_mn + (int64_t)k * ld_k;
    }
  }
  __device__ __forceinline__ bool tail_guard() const { return false; }
  template <int S = 0, bool MASK = true> __device__ __forceinline__ void fetch(int64_t k0) {
    if (MASK && k0 >= K) return;
    const int64_t step = k0 * ld_k;
#pragma unroll
    for (int i = 0; i < NE; ++i) {
      if constexpr (MASK) {
        int mn, k;
        coords(i, mn, k);
        reg[S][i] = ptr[i][(k0 + k) < K ? step : (K - 1 - k) * ld_k];   // past the end: the last valid k (zeroed at commit)
      } else {
        reg[S][i] = ptr[i][step];
      }
    }
  }
  template <int S = 0, bool MASK = true> __device__ __forceinline__ void commit(T* lds, int64_t k0) {
    constexpr int LD = Slab<T, kGeneric, BMN, BK>::LDMN;
    if (MASK && k0 >= K) {
#pragma unroll
      for (int i = 0; i < NE; ++i) reg[S][i] = (T)0;
    } else if (MASK && k0 + BK > K) {
#pragma unroll
      for (int i = 0; i < NE; ++i) {
        int mn, k;
        coords(i, mn, k);
        if ((k0 + k) >= K) reg[S][i] = (T)0;
      }
    }
#pragma unroll
    for (int i = 0; i < NE; ++i) {
      int mn, k;
      coords(i, mn, k);
      lds[k * LD + mn] = reg[S][i];
    }
  }
};

// The column matrix of a convolution as the B operand, gathered from the image (ConvGeom): element (k, j) is one
// image element or zero. A lane owns one column j (one output pixel: its window origin is decoded once) and NE k
// values per slab, NT / BMN apart. k is decoded into (c, kh, kw) by two multiply-high divisions - scalar arithmetic
// where the slab is 64 columns wide or more, since the lanes of a wavefront then share k; an element's address is a
// uniform base plus a non-negative 32-bit byte offset. Every load is unconditional (what the padding or the end of
// the k range rules out is loaded from the image's lowest address instead) and replaced by zero before the commit.
// The loader is bound by the instructions it issues, not by its loads: each of these choices removes some.
// k-row LDS layout.
template <typename T, int BMN, int BK, int NT, bool KG, int PF> struct Loader<T, kGather, BMN, BK, NT, KG, PF> {
  static constexpr int NE = BMN * BK / NT;         // elements per thread
  static constexpr int KSTRIDE = NT / BMN;         // distance in k between a lane's elements
  static_assert(BMN * BK % NT == 0 && NE >= 1 && NT % BMN == 0, "a lane must own one column of the slab");
  const char* low;       // the image's lowest address
  uint32_t noff;         // byte offset of the window origin from `low` (modulo 2^32: it may lie in the padding)
  int ih0, iw0, kbase;
  int64_t K;
  ConvGeom g;
  T reg[PF][NE];
  bool ok[PF][NE];       // the element is a real image element
  __device__ __forceinline__ Loader(const T* X, int64_t, int64_t, int64_t mn0, int64_t MN, int64_t K_, int, const ConvGeom* geom)
      : K(K_), g(*geom) {
    low = (const char*)X - g.origin;
    const int64_t j = mn0 + (int)(threadIdx.x % BMN);
    const int jj = (int)(j < MN ? j : MN - 1);      // columns past the edge repeat the last one (masked at the store)
    const int oh = jj / g.Wo, ow = jj - oh * g.Wo;
    ih0 = oh * g.sh - g.ph;
    iw0 = ow * g.sw - g.pw;
    noff = g.origin + (uint32_t)(ih0 * g.in_h) + (uint32_t)(iw0 * g.in_w);
    kbase = (int)(threadIdx.x / BMN);
  }
  __device__ __forceinline__ bool tail_guard() const { return false; }
  template <int S = 0, bool MASK = true> __device__ __forceinline__ void fetch(int64_t k0) {
    if (MASK && k0 >= K) return;
    const uint32_t kb = (BMN % 64 == 0) ? (uint32_t)__builtin_amdgcn_readfirstlane(kbase) : (uint32_t)kbase;
#pragma unroll
    for (int i = 0; i < NE; ++i) {
      const uint32_t k = (uint32_t)k0 + kb + (uint32_t)(i * KSTRIDE);
      const uint32_t c = g.magic_khw ? __umulhi(k, g.magic_khw) : k;        // (multiplier 0: the divisor is 1)
      const uint32_t r = k - c * (uint32_t)(g.kH * g.kW);
      const uint32_t kh = g.magic_kw ? __umulhi(r, g.magic_kw) : r;
      const uint32_t kw = r - kh * (uint32_t)g.kW;
      const uint32_t koff = c * (uint32_t)g.in_c + kh * (uint32_t)g.in_h + kw * (uint32_t)g.in_w;   // modulo 2^32, like noff
      const bool valid = (!MASK || (int64_t)k < K) && (uint32_t)(ih0 + (int)kh) < (uint32_t)g.H && (uint32_t)(iw0 + (int)kw) < (uint32_t)g.W;
      ok[S][i] = valid;
      reg[S][i] = *(const T*)(low + (valid ? noff + koff : 0u));
    }
  }
  template <int S = 0, bool MASK = true> __device__ __forceinline__ void commit(T* lds, int64_t k0) {
    constexpr int LD = Slab<T, kGather, BMN, BK>::LDMN;
    const bool none = MASK && k0 >= K;     // nothing was fetched
    const int mn = (int)(threadIdx.x % BMN);
#pragma unroll
    for (int i = 0; i < NE; ++i) lds[(kbase + i * KSTRIDE) * LD + mn] = (!none && ok[S][i]) ? reg[S][i] : (T)0;
  }
};

// The same column matrix where VK neighbouring output pixels of one row read VK neighbouring image elements: unit
// stride along the image's width and along the window's step, output rows that are whole vectors (the host checks).
// A lane owns VK columns (their common window origin is decoded once) and NV k values per slab: one 16-byte load and
// one 16-byte LDS write where the scalar loader issues VK of each, and one decode of k (now per lane: the lanes of a
// wavefront no longer share it). A vector that hangs over the left or right edge of the image row is loaded from
// where it fits inside the row instead and moved into place at the commit, zeros in the padding; a vector whose row
// lies in the padding, or past the end of the k range, is loaded from the image's lowest address and committed as
// zeros. Every load is unconditional. k-row LDS layout.
template <typename T, int BMN, int BK, int NT, bool KG, int PF> struct Loader<T, kGatherVec, BMN, BK, NT, KG, PF> {
  typedef typename VecTraits<T>::vec_t vec_t;
  typedef typename VecTraits<T>::gvec_t gvec_t;
  static constexpr int VK = VecTraits<T>::VK;
  static constexpr int CG = BMN / VK;              // column groups of a slab
  static constexpr int KSTRIDE = NT / CG;          // distance in k between a lane's vectors
  static constexpr int NV = BK / KSTRIDE;          // vectors per thread
  static constexpr int kZero = 127;                // `how`: every element is padding (0: every element is real; else the shift)
  static_assert(BMN % VK == 0 && NT % CG == 0 && BK % KSTRIDE == 0 && NV >= 1, "a lane must own one column group of the slab");
  const char* low;       // the image's lowest address
  uint32_t noff;         // byte offset of the window origin from `low` (modulo 2^32: it may lie in the padding)
  int ih0, iw0, kbase;
  int64_t K;
  ConvGeom g;
  vec_t reg[PF][NV];
  int how[PF][NV];
  __device__ __forceinline__ Loader(const T* X, int64_t, int64_t, int64_t mn0, int64_t MN, int64_t K_, int, const ConvGeom* geom)
      : K(K_), g(*geom) {
    low = (const char*)X - g.origin;
    const int64_t j = mn0 + (int)(threadIdx.x % CG) * VK;
    const int jj = (int)(j < MN ? j : MN - VK);     // column groups past the edge repeat the last one (masked at the store)
    const int oh = jj / g.Wo, ow = jj - oh * g.Wo;
    ih0 = oh * g.sh - g.ph;
    iw0 = ow - g.pw;
    noff = g.origin + (uint32_t)(ih0 * g.in_h) + (uint32_t)(iw0 * g.in_w);
    kbase = (int)(threadIdx.x / CG);
  }
  __device__ __forceinline__ bool tail_guard() const { return false; }
  template <int S = 0, bool MASK = true> __device__ __forceinline__ void fetch(int64_t k0) {
    if (MASK && k0 >= K) return;
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const uint32_t k = (uint32_t)k0 + (uint32_t)(kbase + i * KSTRIDE);
      const uint32_t c = g.magic_khw ? __umulhi(k, g.magic_khw) : k;        // (multiplier 0: the divisor is 1)
      const uint32_t r = k - c * (uint32_t)(g.kH * g.kW);
      const uint32_t kh = g.magic_kw ? __umulhi(r, g.magic_kw) : r;
      const uint32_t kw = r - kh * (uint32_t)g.kW;
      const uint32_t koff = c * (uint32_t)g.in_c + kh * (uint32_t)g.in_h + kw * (uint32_t)g.in_w;   // modulo 2^32, like noff
      const int iws = iw0 + (int)kw;               // image column of the vector's first element
      const bool row_ok = (!MASK || (int64_t)k < K) && (uint32_t)(ih0 + (int)kh) < (uint32_t)g.H;
      const bool some = row_ok && iws > -VK && iws < g.W;
      const int fit = iws < 0 ? 0 : (iws > g.W - VK ? g.W - VK : iws);   // where a vector that hangs over an edge is read from
      const int shift = iws - fit;
      how[S][i] = some ? shift : kZero;
      reg[S][i] = *(const gvec_t*)(low + (some ? noff + koff - (uint32_t)(shift * (int)sizeof(T)) : 0u));
    }
  }
  template <int S = 0, bool MASK = true> __device__ __forceinline__ void commit(T* lds, int64_t k0) {
    constexpr int LD = Slab<T, kGatherVec, BMN, BK>::LDMN;
    const bool none = MASK && k0 >= K;     // nothing was fetched
    const int cgp = (int)(threadIdx.x % CG);
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      vec_t v = {};
      if (!none && how[S][i] != kZero) {
        v = reg[S][i];
        const int d = how[S][i];
        if (d != 0) {        // element e is image column fit + e + d: real while 0 <= e + d < VK
          const vec_t w = v;
#pragma unroll
          for (int e = 0; e < VK; ++e) {
            T x = (T)0;
#pragma unroll
            for (int f = 0; f < VK; ++f) x = (e + d == f) ? w[f] : x;
            v[e] = x;
          }
        }
      }
      *(vec_t*)(lds + (kbase + i * KSTRIDE) * LD + cgp * VK) = v;
    }
  }
};

// The transposed column matrices of a whole batch side by side, as the B operand of the weight gradient
// grad_weight[C_out][C * kH * kW] = g[C_out][N * P] . col^T: B(n, k) with n = (c, kh, kw), k = image * P + pixel. Along k
// neighbouring output pixels of one row read neighbouring image elements (same conditions as kGatherVec, checked by
// the host: unit strides along the width, output rows that are whole vectors - so P and every image's first k are
// multiples of VK too), so the operand moves like a k-contiguous one: a lane owns one n (decoded once) and one 16-byte
// k-group per slab, whose k is decoded into (image, oh, ow) by two launch-constant divisions. Edges as in kGatherVec.
// k-group LDS layout, the one the k-contiguous loader writes.
template <typename T, int BMN, int BK, int NT, bool KG, int PF> struct Loader<T, kGatherVecT, BMN, BK, NT, KG, PF> {
  typedef typename VecTraits<T>::vec_t vec_t;
  typedef typename VecTraits<T>::gvec_t gvec_t;
  static constexpr int VK = VecTraits<T>::VK;
  static constexpr int QN = BK / VK;               // k-groups per row
  static constexpr int NV = BMN * QN / NT;         // vectors per thread
  static constexpr int kZero = 127;
  static_assert(KG && BMN * QN % NT == 0 && NV >= 1, "slab must divide evenly over the workgroup");
  const char* low;       // image 0's lowest address
  uint32_t coff[NV];     // byte offset from `low` of the element that n reads for output pixel (0, 0) (modulo 2^32)
  int dh[NV], dw[NV];    // kh - padH, kw - padW
  int64_t K;
  ConvGeom g;
  vec_t reg[PF][NV];
  int how[PF][NV];
  __device__ __forceinline__ Loader(const T* X, int64_t, int64_t, int64_t mn0, int64_t MN, int64_t K_, int, const ConvGeom* geom)
      : K(K_), g(*geom) {
    low = (const char*)X - g.origin;
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int64_t mn = mn0 + (int)((threadIdx.x + i * NT) / QN);
      const uint32_t n = (uint32_t)(mn < MN ? mn : MN - 1);    // rows past the edge repeat the last one (masked at the store)
      const uint32_t c = g.magic_khw ? __umulhi(n, g.magic_khw) : n;
      const uint32_t r = n - c * (uint32_t)(g.kH * g.kW);
      const uint32_t kh = g.magic_kw ? __umulhi(r, g.magic_kw) : r;
      const uint32_t kw = r - kh * (uint32_t)g.kW;
      dh[i] = (int)kh - g.ph;
      dw[i] = (int)kw - g.pw;
      coff[i] = g.origin + c * (uint32_t)g.in_c + (uint32_t)(dh[i] * g.in_h) + (uint32_t)(dw[i] * g.in_w);
    }
  }
  __device__ __forceinline__ bool tail_guard() const { return false; }
  template <int S = 0, bool MASK = true> __device__ __forceinline__ void fetch(int64_t k0) {
    if (MASK && k0 >= K) return;
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const uint32_t k = (uint32_t)k0 + (uint32_t)(((threadIdx.x + i * NT) % QN) * VK);
      uint32_t pix, ow;
      const uint32_t img = g.by_p.divmod(k, pix);
      const uint32_t oh = g.by_wo.divmod(pix, ow);
      const int ih = (int)oh * g.sh + dh[i];
      const int iws = (int)ow + dw[i];             // image column of the vector's first element
      const bool row_ok = (!MASK || (int64_t)k < K) && (uint32_t)ih < (uint32_t)g.H;
      const bool some = row_ok && iws > -VK && iws < g.W;
      const int fit = iws < 0 ? 0 : (iws > g.W - VK ? g.W - VK : iws);
      const int shift = iws - fit;
      how[S][i] = some ? shift : kZero;
      const uint32_t off = coff[i] + oh * (uint32_t)(g.sh * g.in_h) + (ow - (uint32_t)shift) * (uint32_t)g.in_w;
      reg[S][i] = *(const gvec_t*)(low + (some ? (int64_t)img * g.in_n + (int64_t)off : (int64_t)0));
    }
  }
  template <int S = 0, bool MASK = true> __device__ __forceinline__ void commit(T* lds, int64_t k0) {
    constexpr int LD = Slab<T, kGatherVecT, BMN, BK, true>::LDKG;
    const bool none = MASK && k0 >= K;     // nothing was fetched
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int v_ = threadIdx.x + i * NT;
      const int q = v_ % QN, mn = v_ / QN;
      vec_t v = {};
      if (!none && how[S][i] != kZero) {
        v = reg[S][i];
        const int d = how[S][i];
        if (d != 0) {
          const vec_t w = v;
#pragma unroll
          for (int e = 0; e < VK; ++e) {
            T x = (T)0;
#pragma unroll
            for (int f = 0; f < VK; ++f) x = (e + d == f) ? w[f] : x;
            v[e] = x;
          }
        }
      }
      *(vec_t*)(lds + (q * LD + mn) * VK) = v;
    }
  }
};

}  // namespace gemm
}  // namespace am
