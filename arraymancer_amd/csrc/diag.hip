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

}  // namespace

// kind: 0 = MFMA f32 32x32x2 (FLOP/s), 1 = MFMA f64 16x16x4 (FLOP/s),
//       2 = VALU int32 multiply-add (integer op/s, 2 per MAC), 3 = VALU int64 multiply-add,
//       4 = MFMA i32 32x32x32 int8 (integer op/s).
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
