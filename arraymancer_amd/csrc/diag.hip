// Register-only micro-benchmarks that measure the issue ceilings the GEMM kernels are compared
// with: MFMA f32 / f64 and the VALU integer multiply-accumulate. No memory traffic inside the
// timed loops; every wave keeps several independent accumulators so that the pipes stay full.
#include "common.h"

using namespace am;

namespace {

typedef float v16f __attribute__((ext_vector_type(16)));
typedef double v4d __attribute__((ext_vector_type(4)));

constexpr int kMfmaChains = 8;    // independent accumulators per wave

// The accumulators are pinned to VGPRs through inline assembly so that the loop body is nothing
// but the chain of independent MFMAs (the builtin form made the compiler shuttle them through
// AccVGPRs every trip). Chains are kMfmaChains apart, far beyond any MFMA->MFMA wait state.
__global__ __launch_bounds__(256) void peak_mfma_f32(int iters, float* out) {
  v16f acc[kMfmaChains];
  for (int c = 0; c < kMfmaChains; ++c)
    for (int r = 0; r < 16; ++r) acc[c][r] = 0.f;
  const float a = 1.0f + threadIdx.x * 1e-6f, b = 1.0f - threadIdx.x * 1e-6f;
  for (int i = 0; i < iters; ++i) {
#pragma unroll
    for (int c = 0; c < kMfmaChains; ++c)
      asm volatile("v_mfma_f32_32x32x2_f32 %0, %1, %2, %0" : "+v"(acc[c]) : "v"(a), "v"(b));
  }
  asm volatile("s_nop 15\n\ts_nop 15\n\ts_nop 15" ::: "memory");
  float s = 0.f;
  for (int c = 0; c < kMfmaChains; ++c) s += acc[c][0] + acc[c][15];
  if (s == 12345.678f) out[0] = s;   // keeps the loop alive without a store in the common case
}

__global__ __launch_bounds__(256) void peak_mfma_f64(int iters, double* out) {
  v4d acc[kMfmaChains];
  for (int c = 0; c < kMfmaChains; ++c)
    for (int r = 0; r < 4; ++r) acc[c][r] = 0.0;
  const double a = 1.0 + threadIdx.x * 1e-9, b = 1.0 - threadIdx.x * 1e-9;
  for (int i = 0; i < iters; ++i) {
#pragma unroll
    for (int c = 0; c < kMfmaChains; ++c)
      asm volatile("v_mfma_f64_16x16x4_f64 %0, %1, %2, %0" : "+v"(acc[c]) : "v"(a), "v"(b));
  }
  asm volatile("s_nop 15\n\ts_nop 15\n\ts_nop 15" ::: "memory");
  double s = 0.0;
  for (int c = 0; c < kMfmaChains; ++c) s += acc[c][0] + acc[c][3];
  if (s == 12345.678) out[0] = s;
}

// int8 matrix instruction of the digit-sliced integer GEMM; operands with mixed byte values (the power
// drawn, and with it the clock the chip settles at, depends on how many bits toggle).
typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
__global__ __launch_bounds__(256) void peak_mfma_i8(int iters, int* out) {
  v16i acc[4];   // four chains: 64 accumulator registers, 32 cycles apart
  for (int c = 0; c < 4; ++c)
    for (int r = 0; r < 16; ++r) acc[c][r] = 0;
  const int t = (int)threadIdx.x;
  const v4i a = {0x5a3c9671 + t * 0x01010101, 0x1234fedc ^ t, (int)0x9e3779b9 * (t + 1), 0x7f80017f};
  const v4i b = {(int)0x85ebca6b * (t + 3), 0x0badf00d + t, 0x13579bdf ^ (t << 8), (int)0xc2b2ae35};
  for (int i = 0; i < iters; ++i) {
#pragma unroll
    for (int c = 0; c < 4; ++c)
      asm volatile("v_mfma_i32_32x32x32_i8 %0, %1, %2, %0" : "+v"(acc[c]) : "v"(a), "v"(b));
  }
  asm volatile("s_nop 15\n\ts_nop 15\n\ts_nop 15" ::: "memory");
  int s = 0;
  for (int c = 0; c < 4; ++c) s += acc[c][0] + acc[c][15];
  if (s == 0x12345678) out[0] = s;
}

// LDS read rate: every wavefront reads 16 bytes per lane (ds_read_b128, consecutive lanes at consecutive
// addresses: no bank conflicts), eight independent reads in flight per trip, each wavefront from its own 8 KiB.
// Written as inline assembly so that the loop is the eight reads, one wait and the loop counter.
__global__ __launch_bounds__(256) void peak_lds_read(int iters, int* out) {
  __shared__ __attribute__((aligned(16))) int buf[8192];
  for (int i = threadIdx.x; i < 8192; i += 256) buf[i] = i * 0x9e3779b9;
  __syncthreads();
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const uint32_t addr = (uint32_t)reinterpret_cast<uintptr_t>(buf) + (uint32_t)(wave * 8192 + lane * 16);
  v4i v0, v1, v2, v3, v4, v5, v6, v7;
  int s = 0;
  for (int i = 0; i < iters; ++i) {
    asm volatile(
        "ds_read_b128 %0, %8\n\tds_read_b128 %1, %8 offset:1024\n\tds_read_b128 %2, %8 offset:2048\n\t"
        "ds_read_b128 %3, %8 offset:3072\n\tds_read_b128 %4, %8 offset:4096\n\tds_read_b128 %5, %8 offset:5120\n\t"
        "ds_read_b128 %6, %8 offset:6144\n\tds_read_b128 %7, %8 offset:7168\n\ts_waitcnt lgkmcnt(0)"
        : "=&v"(v0), "=&v"(v1), "=&v"(v2), "=&v"(v3), "=&v"(v4), "=&v"(v5), "=&v"(v6), "=&v"(v7)
        : "v"(addr)
        : "memory");
    s ^= v0[0] ^ v7[3];
  }
  s ^= v1[1] ^ v2[2] ^ v3[3] ^ v4[0] ^ v5[1] ^ v6[2];
  if (s == 0x12345678) out[0] = s;
}

// 8 x 8 register tile of wrapping 32-bit multiply-accumulates per step: the inner body of the
// integer GEMM kernel without its LDS reads.
template <typename U>
__global__ __launch_bounds__(256) void peak_valu_mac(int iters, U* out, U seed) {
  U acc[8][8];
  U a[8], b[8];
  for (int i = 0; i < 8; ++i) {
    a[i] = seed + threadIdx.x * 3 + i;
    b[i] = seed * 7 + threadIdx.x + i * 5;
    for (int j = 0; j < 8; ++j) acc[i][j] = 0;
  }
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
      for (int j = 0; j < 8; ++j) acc[i][j] += a[i] * b[j];
#pragma unroll
    for (int i = 0; i < 8; ++i) { a[i] += 1; b[i] ^= a[i]; }   // operands change every step, as in a GEMM
  }
  U s = 0;
  for (int i = 0; i < 8; ++i)
    for (int j = 0; j < 8; ++j) s += acc[i][j];
  if (s == (U)0x1234567) out[0] = s;
}

// The instruction of the int32 GEMM's inner loop alone: v_mad_u64_u32 (the low half of its 64-bit result is the wrapped
// 32-bit multiply-accumulate), 32 independent accumulator pairs per lane, operands that never change, written in
// assembly so that nothing else is in the loop (in C the compiler replaces a loop of constant multiply-adds by its
// closed form). With the clock window open this gives cycles per instruction on the device, not an estimate.
__global__ __launch_bounds__(256) void peak_mad_u64_u32(int iters, unsigned long long* out, unsigned seed, long long* clk) {
  const ClockProbe probe(clk);
  unsigned long long acc[32];
  unsigned a[4], b[8];
  for (int i = 0; i < 4; ++i) a[i] = seed + threadIdx.x * 3u + i;
  for (int j = 0; j < 8; ++j) b[j] = seed * 7u + threadIdx.x + j * 5u;
  for (int i = 0; i < 32; ++i) acc[i] = i;
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 8; ++j)
        asm volatile("v_mad_u64_u32 %0, vcc, %1, %2, %0" : "+v"(acc[i * 8 + j]) : "v"(a[i]), "v"(b[j]) : "vcc");
  }
  unsigned long long s = 0;
  for (int i = 0; i < 32; ++i) s += acc[i];
  if (s == 0x123456789abcull) out[0] = s;
  probe.finish();
}

// ---- HBM streams: what the memory system delivers to a kernel that does nothing else --------------
// One workgroup walks tiles of 256 lanes x UNROLL x 16 bytes (every load instruction of a wavefront
// covers 1 KiB of consecutive addresses, UNROLL of them in flight per lane), grid-stride over the
// buffer. KIND 0 reads (folds into a register, stores nothing), 1 writes a constant, 2 copies.
// NTL / NTS: non-temporal loads / stores. CHUNKED: a workgroup owns one contiguous run of tiles
// instead of every gridDim.x-th tile.
typedef uint32_t v4u __attribute__((ext_vector_type(4)));
template <int KIND, int UNROLL, bool NTL, bool NTS, bool CHUNKED>
__global__ __launch_bounds__(256) void hbm_stream(const v4u* __restrict__ src, v4u* __restrict__ dst, uint64_t ntiles, uint32_t* sink) {
  constexpr uint64_t TILE_V = 256ull * UNROLL;   // 16-byte vectors per tile
  v4u fold = {0u, 0u, 0u, 0u};
  uint64_t first = blockIdx.x, last = ntiles, step = gridDim.x;
  if (CHUNKED) {
    const uint64_t per = (ntiles + gridDim.x - 1) / gridDim.x;
    first = per * blockIdx.x;
    last = first + per < ntiles ? first + per : ntiles;
    step = 1;
  }
  for (uint64_t tile = first; tile < last; tile += step) {
    const uint64_t base = tile * TILE_V + threadIdx.x;
    v4u v[UNROLL];
    if (KIND != 1) {
#pragma unroll
      for (int u = 0; u < UNROLL; ++u) {
        if (NTL) v[u] = __builtin_nontemporal_load(src + base + (uint64_t)u * 256);
        else v[u] = src[base + (uint64_t)u * 256];
      }
    }
    if (KIND == 0) {
#pragma unroll
      for (int u = 0; u < UNROLL; ++u) fold ^= v[u];
    } else {
#pragma unroll
      for (int u = 0; u < UNROLL; ++u) {
        const v4u w = KIND == 1 ? v4u{(uint32_t)tile, 1u, 2u, 3u} : v[u];
        if (NTS) __builtin_nontemporal_store(w, dst + base + (uint64_t)u * 256);
        else dst[base + (uint64_t)u * 256] = w;
      }
    }
  }
  if (KIND == 0 && (fold[0] ^ fold[1] ^ fold[2] ^ fold[3]) == 0x9e3779b9u) sink[0] = fold[0];   // keeps the loads alive
}

template <int KIND, int UNROLL>
static void launch_hbm(bool ntl, bool nts, bool chunked, unsigned blocks, const v4u* src, v4u* dst, uint64_t ntiles, uint32_t* sink) {
#define AM_HBM(L, S, C) hipLaunchKernelGGL((hbm_stream<KIND, UNROLL, L, S, C>), dim3(blocks), dim3(256), 0, stream(), src, dst, ntiles, sink)
  const int sel = (ntl ? 4 : 0) | (nts ? 2 : 0) | (chunked ? 1 : 0);
  switch (sel) {
    case 0: AM_HBM(false, false, false); break;
    case 1: AM_HBM(false, false, true); break;
    case 2: AM_HBM(false, true, false); break;
    case 3: AM_HBM(false, true, true); break;
    case 4: AM_HBM(true, false, false); break;
    case 5: AM_HBM(true, false, true); break;
    case 6: AM_HBM(true, true, false); break;
    default: AM_HBM(true, true, true); break;
  }
#undef AM_HBM
}

template <int KIND>
static void launch_hbm_u(int unroll, bool ntl, bool nts, bool chunked, unsigned blocks, const v4u* src, v4u* dst, uint64_t bytes, uint32_t* sink) {
  switch (unroll) {
    case 1: launch_hbm<KIND, 1>(ntl, nts, chunked, blocks, src, dst, bytes / (4096ull * 1), sink); break;
    case 2: launch_hbm<KIND, 2>(ntl, nts, chunked, blocks, src, dst, bytes / (4096ull * 2), sink); break;
    case 8: launch_hbm<KIND, 8>(ntl, nts, chunked, blocks, src, dst, bytes / (4096ull * 8), sink); break;
    default: launch_hbm<KIND, 4>(ntl, nts, chunked, blocks, src, dst, bytes / (4096ull * 4), sink); break;
  }
}

}  // namespace

// HBM stream ceilings. kind: 0 read, 1 write, 2 copy, 3 copy made by the runtime (hipMemcpyAsync device to device over the
// same windows: not a kernel of this library; blocks_per_cu, unroll and flags do not apply). Each launch moves `bytes` (a multiple of 32 KiB) of
// a window that rotates through `windows` disjoint buffers (windows * bytes should exceed the 256 MB
// memory-side cache several times over, so that no launch finds its input there); blocks_per_cu x CUs
// workgroups; `unroll` (1, 2, 4, 8) 16-byte accesses in flight per lane; flags: bit 0 non-temporal loads,
// bit 1 non-temporal stores, bit 2 a contiguous run of tiles per workgroup. Returns bytes moved per second
// (read + written) averaged over `launches` launches after `windows` untimed ones.
extern "C" int am_hip_diag_hbm(int kind, size_t bytes, int windows, int blocks_per_cu, int unroll, int flags, int launches,
                               double* bytes_per_second) {
  if (!bytes_per_second || kind < 0 || kind > 3 || bytes == 0 || bytes % 32768 != 0 || windows < 1 || windows > 64 ||
      blocks_per_cu < 1 || blocks_per_cu > 64 || (unroll != 1 && unroll != 2 && unroll != 4 && unroll != 8) || launches < 1)
    return fail(AM_E_ARG, "am_hip_diag_hbm: bad argument");
  AM_TRY(ensure_init());
  char *src = nullptr, *dst = nullptr;
  uint32_t* sink = nullptr;
  const size_t total = bytes * (size_t)windows;
  AM_HIP_TRY(hipMalloc((void**)&sink, 256));
  if (kind != 1) {
    if (hipMalloc((void**)&src, total) != hipSuccess) { (void)hipGetLastError(); (void)hipFree(sink); return fail(AM_E_ALLOC, "am_hip_diag_hbm: %zu bytes", total); }
    AM_HIP_TRY(hipMemsetAsync(src, 0x5a, total, stream()));
  }
  if (kind != 0) {
    if (hipMalloc((void**)&dst, total) != hipSuccess) { (void)hipGetLastError(); (void)hipFree(src); (void)hipFree(sink); return fail(AM_E_ALLOC, "am_hip_diag_hbm: %zu bytes", total); }
    AM_HIP_TRY(hipMemsetAsync(dst, 0, total, stream()));
  }
  const unsigned blocks = (unsigned)(num_cus() * blocks_per_cu);
  hipEvent_t e0, e1;
  AM_HIP_TRY(hipEventCreate(&e0));
  AM_HIP_TRY(hipEventCreate(&e1));
  auto one = [&](int i) {
    const size_t off = (size_t)(i % windows) * bytes;
    const v4u* s = (const v4u*)(src ? src + off : nullptr);
    v4u* d = (v4u*)(dst ? dst + off : nullptr);
    const bool ntl = flags & 1, nts = flags & 2, chunked = flags & 4;
    if (kind == 3) { (void)hipMemcpyAsync(d, s, bytes, hipMemcpyDeviceToDevice, stream()); return; }
    if (kind == 0) launch_hbm_u<0>(unroll, ntl, nts, chunked, blocks, s, d, bytes, sink);
    else if (kind == 1) launch_hbm_u<1>(unroll, ntl, nts, chunked, blocks, s, d, bytes, sink);
    else launch_hbm_u<2>(unroll, ntl, nts, chunked, blocks, s, d, bytes, sink);
  };
  for (int i = 0; i < windows; ++i) one(i);
  AM_HIP_TRY(hipEventRecord(e0, stream()));
  for (int i = 0; i < launches; ++i) one(windows + i);
  AM_HIP_TRY(hipEventRecord(e1, stream()));
  AM_HIP_TRY(hipEventSynchronize(e1));
  float ms = 0;
  AM_HIP_TRY(hipEventElapsedTime(&ms, e0, e1));
  AM_HIP_TRY(hipEventDestroy(e0));
  AM_HIP_TRY(hipEventDestroy(e1));
  (void)hipFree(src); (void)hipFree(dst); (void)hipFree(sink);
  AM_TRY(check_launch("hbm_stream"));
  *bytes_per_second = (double)bytes * (kind >= 2 ? 2.0 : 1.0) * launches / (ms * 1e-3);
  return AM_OK;
}

// ---- shader clock sustained by the matrix kernels themselves --------------------------------------
// While armed, the matrix-core GEMM kernels (gemm_mfma, gemm_i8_digits) have the first lane of workgroup 0
// read the shader-cycle counter and the constant-rate counter when it starts and when it ends, and add the
// two differences to this buffer: cycles / ticks x the constant rate is the shader clock averaged over the
// kernels that ran, measured inside them (a second kernel running beside them to watch the clock takes a CU
// from a launch of exactly one workgroup per CU and doubles its time).
namespace {
long long* g_clock_buf = nullptr;   // device: [0] shader cycles, [1] constant-rate ticks
bool g_clock_armed = false;
}  // namespace
namespace am {
long long* clock_probe_buffer() { return g_clock_armed ? g_clock_buf : nullptr; }
}

extern "C" int am_hip_diag_clock_begin(void) {
  AM_TRY(ensure_init());
  if (capturing()) return fail(AM_E_ARG, "am_hip_diag_clock_begin: not allowed while a graph is being captured");
  if (!g_clock_buf) AM_HIP_TRY(hipMalloc((void**)&g_clock_buf, 256));
  AM_HIP_TRY(hipMemsetAsync(g_clock_buf, 0, 256, stream()));
  g_clock_armed = true;
  return AM_OK;
}

extern "C" int am_hip_diag_clock_end(double* shader_mhz) {
  if (!shader_mhz) return fail(AM_E_ARG, "am_hip_diag_clock_end: null pointer");
  if (!g_clock_armed) return fail(AM_E_ARG, "am_hip_diag_clock_end: am_hip_diag_clock_begin was not called");
  g_clock_armed = false;
  long long h[2] = {0, 0};
  AM_TRY(fetch_result(h, g_clock_buf, sizeof(h)));
  int khz = 100000;
  (void)hipDeviceGetAttribute(&khz, hipDeviceAttributeWallClockRate, 0);
  *shader_mhz = h[1] > 0 ? (double)h[0] / (double)h[1] * (khz / 1e3) : 0.0;
  return AM_OK;
}

// ---- phase marks of the small-product kernels (PhaseProbe, common.h) --------------------------------
namespace {
constexpr int kPhaseSlots = 8192;          // workgroups that can record
long long* g_phase_buf = nullptr;          // device: [kPhaseSlots][5] readings of the constant-rate counter
bool g_phase_armed = false;
}  // namespace
namespace am {
long long* phase_probe_buffer(int* capacity) {
  if (capacity) *capacity = kPhaseSlots;
  return g_phase_armed ? g_phase_buf : nullptr;
}
}

extern "C" int am_hip_diag_phases_begin(void) {
  AM_TRY(ensure_init());
  if (capturing()) return fail(AM_E_ARG, "am_hip_diag_phases_begin: not allowed while a graph is being captured");
  if (!g_phase_buf) AM_HIP_TRY(hipMalloc((void**)&g_phase_buf, (size_t)kPhaseSlots * 5 * sizeof(long long)));
  AM_HIP_TRY(hipMemsetAsync(g_phase_buf, 0, (size_t)kPhaseSlots * 5 * sizeof(long long), stream()));
  g_phase_armed = true;
  return AM_OK;
}

// Closes the window (blocking) and summarises it, in microseconds: out[0] workgroups that reported, out[1..4] the mean
// of each of the four intervals (start -> first loads issued -> arrived -> last matrix instruction and fold -> stores
// done), out[5] earliest start to latest end over all of them. Meaningful for ONE launch per window.
extern "C" int am_hip_diag_phases(double* out6) {
  if (!out6) return fail(AM_E_ARG, "am_hip_diag_phases: null pointer");
  if (!g_phase_armed) return fail(AM_E_ARG, "am_hip_diag_phases: am_hip_diag_phases_begin was not called");
  g_phase_armed = false;
  static long long* host = nullptr;
  const size_t bytes = (size_t)kPhaseSlots * 5 * sizeof(long long);
  if (!host) AM_HIP_TRY(hipHostMalloc((void**)&host, bytes, hipHostMallocDefault));
  AM_HIP_TRY(hipMemcpyAsync(host, g_phase_buf, bytes, hipMemcpyDeviceToHost, stream()));
  AM_HIP_TRY(hipStreamSynchronize(stream()));
  int khz = 100000;
  (void)hipDeviceGetAttribute(&khz, hipDeviceAttributeWallClockRate, 0);
  const double us_per_tick = 1e3 / (double)khz;
  double sum[4] = {0, 0, 0, 0};
  long long first = 0, last = 0, n = 0;
  for (int s = 0; s < kPhaseSlots; ++s) {
    const long long* t = host + (size_t)s * 5;
    if (t[0] == 0) continue;
    for (int i = 0; i < 4; ++i) sum[i] += (double)(t[i + 1] - t[i]);
    if (n == 0 || t[0] < first) first = t[0];
    if (n == 0 || t[4] > last) last = t[4];
    ++n;
  }
  out6[0] = (double)n;
  for (int i = 0; i < 4; ++i) out6[1 + i] = n ? sum[i] / (double)n * us_per_tick : 0.0;
  out6[5] = n ? (double)(last - first) * us_per_tick : 0.0;
  return AM_OK;
}

// kind: 0 = MFMA f32 32x32x2 (FLOP/s), 1 = MFMA f64 16x16x4 (FLOP/s),
//       2 = VALU int32 multiply-add (integer op/s, 2 per MAC), 3 = VALU int64 multiply-add,
//       4 = MFMA i32 32x32x32 int8 (integer op/s), 5 = LDS reads of 16 bytes per lane (bytes/s),
//       6 = v_mad_u64_u32 alone, in assembly (integer op/s, 2 per instruction and lane; reads the shader clock when a
//           clock window is open).
// Launches `waves_per_simd` wavefronts on every SIMD of the device, `iters` loop trips each.
extern "C" int am_hip_diag_peak(int kind, int iters, int waves_per_simd, double* ops_per_second) {
  if (!ops_per_second || iters <= 0 || waves_per_simd < 1 || waves_per_simd > 8)
    return fail(AM_E_ARG, "am_hip_diag_peak: bad argument");
  AM_TRY(ensure_init());
  void* scratch = nullptr;
  AM_HIP_TRY(hipMalloc(&scratch, 256));
  const int blocks = num_cus() * waves_per_simd;   // 256 lanes = 4 waves = one per SIMD
  hipEvent_t e0, e1;
  AM_HIP_TRY(hipEventCreate(&e0));
  AM_HIP_TRY(hipEventCreate(&e1));
  double ops_per_launch = 0;
  for (int rep = 0; rep < 2; ++rep) {   // first repetition warms up
    AM_HIP_TRY(hipEventRecord(e0, stream()));
    switch (kind) {
      case 0:
        hipLaunchKernelGGL(peak_mfma_f32, dim3(blocks), dim3(256), 0, stream(), iters, (float*)scratch);
        ops_per_launch = (double)blocks * 4 * iters * kMfmaChains * (32.0 * 32 * 2 * 2);
        break;
      case 1:
        hipLaunchKernelGGL(peak_mfma_f64, dim3(blocks), dim3(256), 0, stream(), iters, (double*)scratch);
        ops_per_launch = (double)blocks * 4 * iters * kMfmaChains * (16.0 * 16 * 4 * 2);
        break;
      case 2:
        hipLaunchKernelGGL(peak_valu_mac<uint32_t>, dim3(blocks), dim3(256), 0, stream(), iters, (uint32_t*)scratch, 12345u);
        ops_per_launch = (double)blocks * 256 * iters * 64 * 2.0;
        break;
      case 3:
        hipLaunchKernelGGL(peak_valu_mac<uint64_t>, dim3(blocks), dim3(256), 0, stream(), iters, (uint64_t*)scratch, (uint64_t)12345);
        ops_per_launch = (double)blocks * 256 * iters * 64 * 2.0;
        break;
      case 4:
        hipLaunchKernelGGL(peak_mfma_i8, dim3(blocks), dim3(256), 0, stream(), iters, (int*)scratch);
        ops_per_launch = (double)blocks * 4 * iters * 4 * (32.0 * 32 * 32 * 2);
        break;
      case 5:
        hipLaunchKernelGGL(peak_lds_read, dim3(blocks), dim3(256), 0, stream(), iters, (int*)scratch);
        ops_per_launch = (double)blocks * 256 * iters * 8 * 16.0;   // bytes
        break;
      case 6:
        hipLaunchKernelGGL(peak_mad_u64_u32, dim3(blocks), dim3(256), 0, stream(), iters, (unsigned long long*)scratch, 12345u,
                           clock_probe_buffer());
        ops_per_launch = (double)blocks * 256 * iters * 32 * 2.0;
        break;
      default:
        (void)hipFree(scratch);
        return fail(AM_E_ARG, "am_hip_diag_peak: unknown kind %d", kind);
    }
    AM_HIP_TRY(hipEventRecord(e1, stream()));
    AM_HIP_TRY(hipEventSynchronize(e1));
  }
  float ms = 0;
  AM_HIP_TRY(hipEventElapsedTime(&ms, e0, e1));
  AM_HIP_TRY(hipEventDestroy(e0));
  AM_HIP_TRY(hipEventDestroy(e1));
  AM_HIP_TRY(hipFree(scratch));
  *ops_per_second = ops_per_launch / (ms * 1e-3);
  return AM_OK;
}
