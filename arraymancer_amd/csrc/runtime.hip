// Device context, stream, memory and timing entry points of the C ABI.
#include <map>
#include <mutex>
#include <stdarg.h>
#include <stdlib.h>
#include <unordered_map>
#include <unordered_set>
#include <vector>
#include <string.h>
#include "common.h"

namespace am {

static thread_local char g_err[512] = "";

double nt_threshold_bytes() {
  static const double mb = [] { const char* e = getenv("AM_HIP_NT_MB"); return (e && *e) ? atof(e) : 32.0; }();
  return mb * 1024.0 * 1024.0;
}

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

// Scratch of the allocation-free entry point (am_hip_gemm_noalloc_f32): the split-K partial tiles go
// here instead of into the workspace that splitk_workspace() takes from hipMalloc. The array lives
// in the code object, so every device the library runs on holds its own copy, at its own address,
// until the process ends. Host code never uses the array's name as an address: init_locked() asks
// the runtime for the device address once, with the device current, and everything afterwards
// (kernel arguments) uses that pointer.
static constexpr size_t kStaticScratchBytes = (size_t)16 << 20;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];
static void* g_scratch_ptr = nullptr;   // device address of `scratch` on g_device (the library binds one device per process)

static std::mutex g_mu;
static bool g_ready = false;
static int g_device = -1;
static hipStream_t g_stream = nullptr;
static hipDeviceProp_t g_prop;
static bool g_capturing = false;   // between am_hip_graph_begin and am_hip_graph_end

static int init_locked(int device) {
  if (g_ready) {
    if (device == g_device) return AM_OK;
    return fail(AM_E_ARG, "am_hip_init(%d): library already initialised on device %d", device, g_device);
  }
  int count = 0;
  hipError_t e = hipGetDeviceCount(&count);
  if (e != hipSuccess || count <= 0)
    return fail(AM_E_NODEVICE, "no HIP device available (%s)", e == hipSuccess ? "count = 0" : hipGetErrorString(e));
  if (device < 0 || device >= count) return fail(AM_E_ARG, "device %d out of range [0, %d)", device, count);
  AM_HIP_TRY(hipSetDevice(device));
  AM_HIP_TRY(hipGetDeviceProperties(&g_prop, device));
  if (strncmp(g_prop.gcnArchName, "gfx950", 6) != 0)
    return fail(AM_E_NODEVICE, "device %d is %s; this library carries gfx950 code only", device, g_prop.gcnArchName);
  AM_HIP_TRY(hipStreamCreateWithFlags(&g_stream, hipStreamNonBlocking));
  AM_HIP_TRY(hipGetSymbolAddress((void**)&g_scratch_ptr, HIP_SYMBOL(scratch)));
  g_device = device;
  g_ready = true;
  return AM_OK;
}

int ensure_init() {
  if (g_ready) return AM_OK;
  std::lock_guard<std::mutex> lk(g_mu);
  return init_locked(0);
}

// Split-K workspace: one allocation for the life of the process (64 MiB of the 288 GB), so that GEMM
// calls never allocate (and can be recorded into graphs once it exists).
static void* g_ws = nullptr;
static const size_t kWorkspaceBytes = (size_t)64 << 20;
namespace gemm {
void* splitk_workspace(size_t bytes) {
  if (bytes > kWorkspaceBytes) return nullptr;
  if (!g_ws) {
    if (g_capturing) return nullptr;
    if (hipMalloc(&g_ws, kWorkspaceBytes) != hipSuccess) { (void)hipGetLastError(); g_ws = nullptr; }
  }
  return g_ws;
}
void* static_scratch(size_t* capacity) {
  if (capacity) *capacity = kStaticScratchBytes;
  return g_ready ? g_scratch_ptr : nullptr;
}
}  // namespace gemm

// ---- caching allocator -------------------------------------------------------------------------
// Every operator of the host layers that returns a tensor allocates its result, and hipFree
// synchronises the device: freed blocks are therefore kept in per-size free lists and handed out
// again. A block freed while kernels still use it may be reused at once, because whoever receives
// it next can only touch it through the library stream, i.e. after those kernels. Blocks go back
// to the driver only from am_hip_empty_cache, when the cache exceeds its limit, or when hipMalloc
// fails (cache emptied, one retry); each of those drains the stream first.
static std::mutex g_alloc_mu;
static std::unordered_map<void*, size_t> g_live;            // blocks handed out -> rounded size
static std::map<size_t, std::vector<void*>> g_free_blocks;   // rounded size -> cached blocks
static size_t g_live_bytes = 0, g_cached_bytes = 0;

static size_t cache_limit() {   // AM_HIP_CACHE_LIMIT_MB (default 32768, 0 disables caching)
  static const size_t limit = [] {
    const char* e = getenv("AM_HIP_CACHE_LIMIT_MB");
    return (size_t)((e && *e) ? strtoull(e, nullptr, 10) : 32768ull) << 20;
  }();
  return limit;
}

// 512-byte granules below 1 MiB, 2 MiB granules above: a freed block fits any later request of
// the same rounded size (no splitting, so no fragmentation inside blocks).
static size_t round_size(size_t bytes) {
  const size_t g = bytes < ((size_t)1 << 20) ? 512 : ((size_t)2 << 20);
  return (bytes + g - 1) / g * g;
}

// Blocks freed while a graph is being captured: the recorded kernels may use them (a temporary that a
// host layer allocated before the capture and dropped inside it), so they stay allocated, owned by the
// graph, and go back to the cache when the graph is destroyed.
static std::vector<void*> g_capture_freed;
// Rehearsal of a sequence that is about to be captured: while the hold is on, freed blocks are not handed out again
// but collected here, so that every allocation of the sequence takes a block of its own; switching the hold off puts
// them all into the cache, where the capture of the same sequence then finds one block per allocation.
static bool g_hold = false;
static std::vector<void*> g_held;
static std::unordered_map<void*, std::vector<void*>> g_graph_blocks;   // executable graph -> blocks it keeps alive
// Every executable graph am_hip_graph_end has handed out and am_hip_graph_destroy has not yet taken back: launch and
// destroy refuse any other pointer (a stale, foreign or twice-destroyed handle would otherwise crash inside the runtime,
// and a second destroy would hand the graph's blocks to the cache twice).
static std::unordered_set<void*> g_graphs;

// Hands a live block back: to the cache, or to the driver when the cache is full. g_alloc_mu held.
static int free_block_locked(void* dptr) {
  auto it = g_live.find(dptr);
  if (it == g_live.end()) return fail(AM_E_ARG, "am_hip_free: %p was not allocated by am_hip_malloc (or freed twice)", dptr);
  const size_t rounded = it->second;
  g_live.erase(it);
  g_live_bytes -= rounded;
  if (g_cached_bytes + rounded <= cache_limit()) {
    g_free_blocks[rounded].push_back(dptr);
    g_cached_bytes += rounded;
    return AM_OK;
  }
  // Work that still reads or writes the buffer is on the library stream: drain it first.
  AM_HIP_TRY(hipStreamSynchronize(g_stream));
  AM_HIP_TRY(hipFree(dptr));
  return AM_OK;
}

static void release_cached_locked() {
  for (auto& kv : g_free_blocks)
    for (void* p : kv.second) (void)hipFree(p);
  g_free_blocks.clear();
  g_cached_bytes = 0;
}

hipStream_t stream() { return g_stream; }
bool capturing() { return g_capturing; }
int num_cus() { return g_ready ? g_prop.multiProcessorCount : 256; }

}  // namespace am

using namespace am;

extern "C" {

const char* am_hip_last_error(void) { return g_err; }
const char* am_hip_version(void) { return "arraymancer-hip 0.1 (gfx950)"; }

int am_hip_init(int device) {
  std::lock_guard<std::mutex> lk(g_mu);
  return init_locked(device);
}

int am_hip_device_count(int* count) {
  if (!count) return fail(AM_E_ARG, "am_hip_device_count: null pointer");
  int c = 0;
  hipError_t e = hipGetDeviceCount(&c);
  *count = (e == hipSuccess) ? c : 0;
  return AM_OK;
}

int am_hip_device_info(char* name, size_t name_cap, int* compute_units, int* clock_khz,
                       size_t* hbm_bytes, int* lds_bytes_per_cu) {
  AM_TRY(ensure_init());
  if (name && name_cap > 0) {
    snprintf(name, name_cap, "%s (%s)", g_prop.name, g_prop.gcnArchName);
  }
  if (compute_units) *compute_units = g_prop.multiProcessorCount;
  if (clock_khz) *clock_khz = g_prop.clockRate;
  if (hbm_bytes) *hbm_bytes = g_prop.totalGlobalMem;
  if (lds_bytes_per_cu) *lds_bytes_per_cu = (int)g_prop.maxSharedMemoryPerMultiProcessor;
  return AM_OK;
}

int am_hip_malloc(size_t bytes, void** out) {
  if (!out) return fail(AM_E_ARG, "am_hip_malloc: null out pointer");
  *out = nullptr;
  if (bytes == 0) return AM_OK;
  AM_TRY(ensure_init());
  const size_t rounded = round_size(bytes);
  std::lock_guard<std::mutex> lk(g_alloc_mu);
  auto it = g_free_blocks.find(rounded);
  if (it != g_free_blocks.end() && !it->second.empty()) {
    *out = it->second.back();
    it->second.pop_back();
    g_cached_bytes -= rounded;
  } else if (g_capturing) {
    // The driver cannot be asked for memory while the stream records: a capture is served from the cache alone.
    return fail(AM_E_ALLOC, "am_hip_malloc: no cached block of %zu bytes while a graph is being captured (run the sequence "
                "once between am_hip_alloc_hold(1) and am_hip_alloc_hold(0) first: that leaves one cached block per allocation)", rounded);
  } else {
    hipError_t e = hipMalloc(out, rounded);
    if (e != hipSuccess && g_cached_bytes > 0) {   // give the cache back and try once more
      (void)hipGetLastError();
      (void)hipStreamSynchronize(g_stream);
      release_cached_locked();
      e = hipMalloc(out, rounded);
    }
    if (e != hipSuccess) {
      *out = nullptr;
      (void)hipGetLastError();
      return fail(AM_E_ALLOC, "hipMalloc(%zu bytes) failed: %s", rounded, hipGetErrorString(e));
    }
  }
  g_live[*out] = rounded;
  g_live_bytes += rounded;
  return AM_OK;
}

int am_hip_free(void* dptr) {
  if (!dptr) return AM_OK;
  AM_TRY(ensure_init());
  std::lock_guard<std::mutex> lk(g_alloc_mu);
  if (g_capturing) {   // kept for the graph being recorded, see g_capture_freed
    if (g_live.find(dptr) == g_live.end())
      return fail(AM_E_ARG, "am_hip_free: %p was not allocated by am_hip_malloc (or freed twice)", dptr);
    for (void* q : g_capture_freed)
      if (q == dptr) return fail(AM_E_ARG, "am_hip_free: %p freed twice", dptr);
    g_capture_freed.push_back(dptr);
    return AM_OK;
  }
  if (g_hold) {   // kept until am_hip_alloc_hold(0), see g_held
    if (g_live.find(dptr) == g_live.end())
      return fail(AM_E_ARG, "am_hip_free: %p was not allocated by am_hip_malloc (or freed twice)", dptr);
    for (void* q : g_held)
      if (q == dptr) return fail(AM_E_ARG, "am_hip_free: %p freed twice", dptr);
    g_held.push_back(dptr);
    return AM_OK;
  }
  return free_block_locked(dptr);
}

int am_hip_alloc_hold(int on) {
  AM_TRY(ensure_init());
  if (g_capturing) return fail(AM_E_ARG, "am_hip_alloc_hold: not allowed while a graph is being captured");
  std::lock_guard<std::mutex> lk(g_alloc_mu);
  if (on) { g_hold = true; return AM_OK; }
  g_hold = false;
  int rc = AM_OK;
  for (void* q : g_held) {
    const int r = free_block_locked(q);
    if (r != AM_OK) rc = r;
  }
  g_held.clear();
  return rc;
}

int am_hip_empty_cache(void) {
  AM_TRY(ensure_init());
  if (g_capturing) return fail(AM_E_ARG, "am_hip_empty_cache: not allowed while a graph is being captured");
  std::lock_guard<std::mutex> lk(g_alloc_mu);
  AM_HIP_TRY(hipStreamSynchronize(g_stream));
  release_cached_locked();
  return AM_OK;
}

int am_hip_memory_stats(size_t* live_bytes, size_t* cached_bytes) {
  std::lock_guard<std::mutex> lk(g_alloc_mu);
  if (live_bytes) *live_bytes = g_live_bytes;
  if (cached_bytes) *cached_bytes = g_cached_bytes;
  return AM_OK;
}

int am_hip_device_free_bytes(size_t* free_bytes, size_t* total_bytes) {
  AM_TRY(ensure_init());
  size_t f = 0, t = 0;
  AM_HIP_TRY(hipMemGetInfo(&f, &t));
  if (free_bytes) *free_bytes = f;
  if (total_bytes) *total_bytes = t;
  return AM_OK;
}

int am_hip_memcpy_h2d(void* dst, const void* src, size_t bytes) {
  if (bytes == 0) return AM_OK;
  if (!dst || !src) return fail(AM_E_ARG, "am_hip_memcpy_h2d: null pointer");
  AM_TRY(ensure_init());
  if (g_capturing) return fail(AM_E_ARG, "am_hip_memcpy_h2d: not allowed while a graph is being captured");
  AM_HIP_TRY(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, g_stream));
  AM_HIP_TRY(hipStreamSynchronize(g_stream));
  return AM_OK;
}

}  // extern "C"

namespace am {
int fetch_result(void* host_dst, const void* dev_src, size_t bytes) {
  static void* pinned = nullptr;
  if (bytes > 256) return fail(AM_E_ARG, "fetch_result: %zu bytes", bytes);
  if (!pinned) AM_HIP_TRY(hipHostMalloc(&pinned, 256, hipHostMallocDefault));
  AM_HIP_TRY(hipMemcpyAsync(pinned, dev_src, bytes, hipMemcpyDeviceToHost, g_stream));
  AM_HIP_TRY(hipStreamSynchronize(g_stream));
  memcpy(host_dst, pinned, bytes);
  return AM_OK;
}
}  // namespace am

extern "C" {
int am_hip_memcpy_d2h(void* dst, const void* src, size_t bytes) {
  if (bytes == 0) return AM_OK;
  if (!dst || !src) return fail(AM_E_ARG, "am_hip_memcpy_d2h: null pointer");
  AM_TRY(ensure_init());
  if (g_capturing) return fail(AM_E_ARG, "am_hip_memcpy_d2h: not allowed while a graph is being captured");
  AM_HIP_TRY(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, g_stream));
  AM_HIP_TRY(hipStreamSynchronize(g_stream));
  return AM_OK;
}

int am_hip_memcpy_d2d(void* dst, const void* src, size_t bytes) {
  if (bytes == 0) return AM_OK;
  if (!dst || !src) return fail(AM_E_ARG, "am_hip_memcpy_d2d: null pointer");
  AM_TRY(ensure_init());
  if (g_capturing) return fail(AM_E_ARG, "am_hip_memcpy_d2d: not allowed while a graph is being captured");
  AM_HIP_TRY(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, g_stream));
  return AM_OK;
}

int am_hip_memset(void* dst, int byte_value, size_t bytes) {
  if (bytes == 0) return AM_OK;
  if (!dst) return fail(AM_E_ARG, "am_hip_memset: null pointer");
  AM_TRY(ensure_init());
  // Memset nodes are kept out of captured graphs (clear memory with an element-wise kernel instead).
  if (g_capturing) return fail(AM_E_ARG, "am_hip_memset: not allowed while a graph is being captured");
  AM_HIP_TRY(hipMemsetAsync(dst, byte_value, bytes, g_stream));
  return AM_OK;
}

int am_hip_sync(void) {
  AM_TRY(ensure_init());
  if (g_capturing) return fail(AM_E_ARG, "am_hip_sync: not allowed while a graph is being captured");
  AM_HIP_TRY(hipStreamSynchronize(g_stream));
  return AM_OK;
}

// ---- HIP graphs: record a sequence of kernel launches once, replay it with one call -------------
int am_hip_graph_begin(void) {
  AM_TRY(ensure_init());
  if (g_capturing) return fail(AM_E_ARG, "am_hip_graph_begin: a capture is already in progress");
  AM_HIP_TRY(hipStreamBeginCapture(g_stream, hipStreamCaptureModeThreadLocal));
  g_capturing = true;
  return AM_OK;
}

int am_hip_graph_end(void** graph_exec) {
  if (!graph_exec) return fail(AM_E_ARG, "am_hip_graph_end: null pointer");
  *graph_exec = nullptr;
  if (!g_capturing) return fail(AM_E_ARG, "am_hip_graph_end: no capture in progress");
  g_capturing = false;
  hipGraph_t graph = nullptr;
  hipGraphExec_t exec = nullptr;
  hipError_t e = hipStreamEndCapture(g_stream, &graph);
  if (e == hipSuccess) {
    e = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0);
    (void)hipGraphDestroy(graph);
  }
  std::lock_guard<std::mutex> lk(g_alloc_mu);
  if (e != hipSuccess) {   // no graph will replay anything: the blocks freed meanwhile go back now
    for (void* q : g_capture_freed) (void)free_block_locked(q);
    g_capture_freed.clear();
    (void)hipGetLastError();
    return fail(AM_E_HIP, "ending the capture failed: %s", hipGetErrorString(e));
  }
  if (!g_capture_freed.empty()) g_graph_blocks[(void*)exec] = std::move(g_capture_freed);
  g_capture_freed.clear();
  g_graphs.insert((void*)exec);
  *graph_exec = (void*)exec;
  return AM_OK;
}

int am_hip_graph_launch(void* graph_exec) {
  if (!graph_exec) return fail(AM_E_ARG, "am_hip_graph_launch: null graph");
  {   // (before anything touches the device: an unknown handle is refused on a machine without one too)
    std::lock_guard<std::mutex> lk(g_alloc_mu);
    if (!g_graphs.count(graph_exec))
      return fail(AM_E_ARG, "am_hip_graph_launch: %p is not a graph of am_hip_graph_end (or was destroyed)", graph_exec);
  }
  AM_TRY(ensure_init());
  if (g_capturing) return fail(AM_E_ARG, "am_hip_graph_launch: not allowed while a graph is being captured");
  AM_HIP_TRY(hipGraphLaunch((hipGraphExec_t)graph_exec, g_stream));
  return AM_OK;
}

int am_hip_graph_destroy(void* graph_exec) {
  if (!graph_exec) return AM_OK;
  {
    std::lock_guard<std::mutex> lk(g_alloc_mu);
    if (!g_graphs.erase(graph_exec))
      return fail(AM_E_ARG, "am_hip_graph_destroy: %p is not a graph of am_hip_graph_end (or was destroyed already)", graph_exec);
  }
  AM_HIP_TRY(hipStreamSynchronize(g_stream));
  AM_HIP_TRY(hipGraphExecDestroy((hipGraphExec_t)graph_exec));
  std::lock_guard<std::mutex> lk(g_alloc_mu);
  auto it = g_graph_blocks.find(graph_exec);
  if (it != g_graph_blocks.end()) {   // what was freed during its capture is free now
    for (void* q : it->second) (void)free_block_locked(q);
    g_graph_blocks.erase(it);
  }
  return AM_OK;
}

void* am_hip_stream(void) {
  if (ensure_init() != AM_OK) return nullptr;
  return (void*)g_stream;
}

int am_hip_event_create(void** ev) {
  if (!ev) return fail(AM_E_ARG, "am_hip_event_create: null pointer");
  AM_TRY(ensure_init());
  hipEvent_t e;
  AM_HIP_TRY(hipEventCreate(&e));
  *ev = (void*)e;
  return AM_OK;
}

int am_hip_event_record(void* ev) {
  if (!ev) return fail(AM_E_ARG, "am_hip_event_record: null event");
  AM_TRY(ensure_init());
  AM_HIP_TRY(hipEventRecord((hipEvent_t)ev, g_stream));
  return AM_OK;
}

int am_hip_event_elapsed_ms(void* start, void* stop, float* ms) {
  if (!start || !stop || !ms) return fail(AM_E_ARG, "am_hip_event_elapsed_ms: null pointer");
  AM_TRY(ensure_init());
  AM_HIP_TRY(hipEventSynchronize((hipEvent_t)stop));
  AM_HIP_TRY(hipEventElapsedTime(ms, (hipEvent_t)start, (hipEvent_t)stop));
  return AM_OK;
}

int am_hip_event_destroy(void* ev) {
  if (!ev) return AM_OK;
  AM_HIP_TRY(hipEventDestroy((hipEvent_t)ev));
  return AM_OK;
}

}  // extern "C"
