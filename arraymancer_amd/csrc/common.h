// Shared host-side helpers of libam_hip.so: status codes, thread-local error text, the
// library stream, and the shape/stride container that kernels take by value.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include "../../include/am_hip.h"

namespace am {

// Records `msg` (printf style) as the calling thread's last error and returns `code`.
int fail(int code, const char* fmt, ...) __attribute__((format(printf, 2, 3)));
// Lazily initialises the device context (device 0 unless am_hip_init chose another).
int ensure_init();
hipStream_t stream();
bool capturing();
// Brings up to 256 bytes of a result from device memory to `host_dst` after everything queued on the
// stream (blocking). Goes through a pinned buffer of the library: a copy straight into pageable
// memory is staged by the runtime and costs about 10 us more.
int fetch_result(void* host_dst, const void* dev_src, size_t bytes);
int num_cus();
// Device buffer the matrix-core kernels add their shader-cycle / constant-rate-tick counts to while
// am_hip_diag_clock_begin .. _end is open; nullptr otherwise (the kernels then read no counter).
long long* clock_probe_buffer();

// Inputs larger than this are read with non-temporal loads by the streaming kernels outside the element-wise
// family (experiments: AM_HIP_NT_MB in the environment, in MiB).
double nt_threshold_bytes();

// In a kernel: reads both counters at construction; finish() has the first lane of workgroup 0 add the
// differences to out[0] (shader cycles) and out[1] (ticks). Does nothing when `out` is null.
struct ClockProbe {
  long long c0, w0;
  long long* out;
  __device__ __forceinline__ explicit ClockProbe(long long* o) : c0(0), w0(0), out(o) {
    if (out) { c0 = clock64(); w0 = wall_clock64(); }
  }
  __device__ __forceinline__ void finish() const {
    if (out && blockIdx.x == 0 && blockIdx.y == 0 && threadIdx.x == 0) {
      out[0] += clock64() - c0;
      out[1] += wall_clock64() - w0;
    }
  }
};

// Where a short kernel's time goes, read inside it. While a phase window is open (am_hip_diag_phases_begin), the first
// lane of every workgroup reads the constant-rate counter when the kernel body starts and at four marks and writes the
// five readings to its own slot of the window's buffer (plain stores: nothing is shared between workgroups; workgroups
// beyond the buffer's capacity record nothing). The host turns them into mean intervals and into the time from the
// earliest start to the latest last mark, which the duration a profiler reports for the launch exceeds by the
// dispatch and end-of-kernel work. settle() drains the wave's memory operations before a mark, only while armed, so
// that a mark means "arrived", not "issued". Does nothing when `out` is null.
struct PhaseProbe {
  long long* out;
  long long t[5];
  // `row_pitch` = workgroups per row of the grid (passed in: reading gridDim costs the prologue another memory round trip)
  __device__ __forceinline__ PhaseProbe(long long* base, int capacity, unsigned row_pitch) : out(nullptr) {
    if (base) {
      const unsigned slot = blockIdx.y * row_pitch + blockIdx.x;
      if (slot < (unsigned)capacity) { out = base + (size_t)slot * 5; t[0] = wall_clock64(); }
    }
  }
  __device__ __forceinline__ void settle() const {
    if (out) asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
  }
  __device__ __forceinline__ void mark(int i) {
    if (out) t[i] = wall_clock64();
  }
  __device__ __forceinline__ void finish() const {
    if (out && threadIdx.x == 0) {
#pragma unroll
      for (int i = 0; i < 5; ++i) out[i] = t[i];
    }
  }
};
// The open phase window's buffer and its capacity in workgroups; nullptr when none is open.
long long* phase_probe_buffer(int* capacity);

#define AM_HIP_TRY(expr)                                                                    \
  do {                                                                                      \
    hipError_t _e = (expr);                                                                 \
    if (_e != hipSuccess)                                                                   \
      return ::am::fail(AM_E_HIP, "%s failed: %s (%s:%d)", #expr, hipGetErrorString(_e),    \
                        __FILE__, __LINE__);                                                \
  } while (0)

#define AM_TRY(expr)                 \
  do {                               \
    int _rc = (expr);                \
    if (_rc != AM_OK) return _rc;    \
  } while (0)

// Checks the launch that was just enqueued.
static inline int check_launch(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(AM_E_HIP, "launch of %s failed: %s", what, hipGetErrorString(e));
  return AM_OK;
}

}  // namespace am
