// Library-owned scratch memory of the GEMM family: the split-K workspace (fp32 partial tiles and arrival counters)
// and the buffer for a rewritten operand, one set per (device, stream), allocated on first use; and the static
// device array behind dtas_gemm_f16_static, the entry point that allocates nothing.
#include "gemm_common.h"

// Scratch memory of dtas_gemm_f16_static: arrival counters first, fp32 partial tiles behind them.  Every device the
// library runs on holds its own copy of this array from the moment the code object is loaded until the process
// ends.  In host code the array's name is not a device address: resolve_static_scratch() asks the runtime for the
// address, once per device, and everything else uses that pointer.
static __device__ __align__(256) unsigned char scratch[DTAS_STATIC_SCRATCH_COUNTERS * 4 + DTAS_STATIC_SCRATCH_PARTIAL_BYTES];

namespace dtas {

std::recursive_mutex g_ws_mutex;
thread_local const FixedScratch* t_fixed_scratch = nullptr;

namespace {

// Library-owned scratch memory, one set per (device, stream):
//  * the split-K workspace: nsplit fp32 partial tiles per shared output tile and one arrival counter per tile
//    (zero between launches: the last arriver of a tile re-arms it);
//  * the operand buffer: the fp16 copy of an 8-bit weight matrix (dtas_gemm_q8_f16_fused's two-pass route).
// Allocated on first use by a stream and grown on demand -- the only allocations in the library.  Launches on one
// stream are ordered by it and share its set; launches on different streams use different sets, so they may overlap.
// g_ws_mutex is held from the lookup until the launches that use the set are enqueued: a set is never grown (freed
// and re-allocated: hipFree waits for the device, hence for every launch that may still use it) between a lookup
// and its launch, also with several host threads.  At most kMaxWsStreams streams per device hold a set; beyond
// that the set used longest ago is released first.
constexpr size_t kMaxSplitWsBytes = size_t{1} << 30;
constexpr int kMaxDevices = 64;
constexpr int kMaxWsStreams = 16;
struct StreamWorkspace {
  bool used = false;
  hipStream_t stream = nullptr;
  uint64_t stamp = 0;
  float* partials = nullptr;
  size_t partial_bytes = 0;
  unsigned* arrivals = nullptr;
  size_t tiles = 0;
  void* operand = nullptr;
  size_t operand_bytes = 0;
};
struct DeviceWorkspaces {
  StreamWorkspace slot[kMaxWsStreams];
  uint64_t clock = 0;
};
DeviceWorkspaces g_ws[kMaxDevices];

__global__ void zero_u32_kernel(unsigned* p, size_t count) {
  const size_t i = blockIdx.x * static_cast<size_t>(blockDim.x) + threadIdx.x;
  if (i < count) p[i] = 0u;
}

int release_workspace(StreamWorkspace& w) {
  // kernels of earlier launches may still use the buffers: hipFree waits for the device
  if (w.partials && hipFree(w.partials) != hipSuccess) return fail("workspace: hipFree of the split-K partials failed");
  if (w.arrivals && hipFree(w.arrivals) != hipSuccess) return fail("workspace: hipFree of the split-K counters failed");
  if (w.operand && hipFree(w.operand) != hipSuccess) return fail("workspace: hipFree of the operand buffer failed");
  w = StreamWorkspace{};
  return 0;
}

// The set of `stream` on the current device (g_ws_mutex held by the caller).
int stream_workspace(hipStream_t stream, StreamWorkspace** out) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return fail("workspace: cannot identify the current device");
  DeviceWorkspaces& d = g_ws[dev];
  StreamWorkspace* free_slot = nullptr;
  StreamWorkspace* oldest = nullptr;
  for (StreamWorkspace& w : d.slot) {
    if (w.used && w.stream == stream) {
      w.stamp = ++d.clock;
      *out = &w;
      return 0;
    }
    if (!w.used && !free_slot) free_slot = &w;
    if (w.used && (!oldest || w.stamp < oldest->stamp)) oldest = &w;
  }
  if (!free_slot) {
    if (release_workspace(*oldest) != 0) return -1;
    free_slot = oldest;
  }
  free_slot->used = true;
  free_slot->stream = stream;
  free_slot->stamp = ++d.clock;
  *out = free_slot;
  return 0;
}

int split_workspace(hipStream_t stream, size_t partial_bytes, size_t tiles, float** partials, unsigned** arrivals) {
  StreamWorkspace* w = nullptr;
  if (stream_workspace(stream, &w) != 0) return -1;
  if (partial_bytes > w->partial_bytes) {
    if (w->partials && hipFree(w->partials) != hipSuccess) return fail("gemm: hipFree of the split-K workspace failed");
    w->partials = nullptr;
    w->partial_bytes = 0;
    const size_t want = partial_bytes < (size_t{32} << 20) ? (size_t{32} << 20) : partial_bytes;
    if (hipMalloc(reinterpret_cast<void**>(&w->partials), want) != hipSuccess) {
      (void)hipGetLastError();
      return fail("gemm: cannot allocate %zu bytes of split-K workspace", want);
    }
    w->partial_bytes = want;
  }
  if (tiles > w->tiles) {
    if (w->arrivals && hipFree(w->arrivals) != hipSuccess) return fail("gemm: hipFree of the split-K counters failed");
    w->arrivals = nullptr;
    w->tiles = 0;
    const size_t want = tiles < 4096 ? 4096 : tiles;
    if (hipMalloc(reinterpret_cast<void**>(&w->arrivals), want * sizeof(unsigned)) != hipSuccess) {
      (void)hipGetLastError();
      return fail("gemm: cannot allocate the split-K arrival counters");
    }
    // cleared on the stream that will use them (a clear on the default stream is not ordered with a non-blocking
    // stream), and by a kernel: a memset node recorded into a caller's graph is what a fill kernel avoids
    hipLaunchKernelGGL(zero_u32_kernel, dim3(static_cast<unsigned>(ceil_div(static_cast<int64_t>(want), 256))), dim3(256), 0, stream,
                       w->arrivals, want);
    if (check_launch("gemm") != 0) return -1;
    w->tiles = want;
  }
  *partials = w->partials;
  *arrivals = w->arrivals;
  return 0;
}

void* g_static_scratch[kMaxDevices];  // device address of `scratch` on each device, once resolved
std::mutex g_static_scratch_mutex;


}  // namespace

int operand_workspace(hipStream_t stream, size_t bytes, void** out) {
  StreamWorkspace* w = nullptr;
  if (stream_workspace(stream, &w) != 0) return -1;
  if (bytes > w->operand_bytes) {
    if (bytes > kMaxSplitWsBytes) return fail("operand buffer: a rewritten operand needs %zu bytes (limit %zu)", bytes, kMaxSplitWsBytes);
    if (w->operand && hipFree(w->operand) != hipSuccess) return fail("operand buffer: hipFree failed");
    w->operand = nullptr;
    w->operand_bytes = 0;
    const size_t want = bytes < (size_t{64} << 20) ? (size_t{64} << 20) : bytes;
    if (hipMalloc(&w->operand, want) != hipSuccess) {
      (void)hipGetLastError();
      return fail("operand buffer: cannot allocate %zu bytes", want);
    }
    w->operand_bytes = want;
  }
  *out = w->operand;
  return 0;
}

// Partial tiles and arrival counters of a launch that splits K over `nsplit` workgroups per tile: the static scratch
// if the calling thread is inside dtas_gemm_f16_static, else the stream's workspace, whose lock `lock` then holds
// (the caller keeps it until its kernel is enqueued).
int split_scratch(hipStream_t s, size_t bytes, size_t split_tiles, int nsplit, float** partials, unsigned** arrivals,
                  std::unique_lock<std::recursive_mutex>* lock) {
  if (t_fixed_scratch) {
    const FixedScratch& f = *t_fixed_scratch;
    if (bytes > f.partial_bytes || split_tiles > f.tiles)
      return fail("gemm: K split over %d workgroups needs %zu bytes of partial tiles and %zu counters; the static scratch "
                  "holds %zu bytes and %zu counters (a cfg with split_k = 1 needs none)", nsplit, bytes, split_tiles, f.partial_bytes, f.tiles);
    *partials = f.partials;
    *arrivals = f.arrivals;
    // Every call on this device shares the array and finds what the last one left.  The counters need no clearing:
    // the array is zero when the code object is loaded, and in every kernel that splits K the workgroup that arrives
    // last at a tile sets that tile's counter back to zero, so a finished launch leaves them as it found them.  The
    // partial tiles are overwritten before they are read.
    return 0;
  }
  if (bytes > kMaxSplitWsBytes) return fail("gemm: split_k %d needs %zu bytes of workspace (limit %zu)", nsplit, bytes, kMaxSplitWsBytes);
  *lock = std::unique_lock<std::recursive_mutex>(g_ws_mutex);
  return split_workspace(s, bytes, split_tiles, partials, arrivals);
}

// The device address of the static scratch array on the current device.  hipGetSymbolAddress is asked once per
// device, with that device current (each GPU holds its own copy of the array at its own address).
int resolve_static_scratch(void** out) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return fail("static scratch: cannot identify the current device");
  std::lock_guard<std::mutex> lock(g_static_scratch_mutex);
  if (!g_static_scratch[dev]) {
    void* ptr = nullptr;
    const hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !ptr) {
      (void)hipGetLastError();
      return fail("static scratch: hipGetSymbolAddress failed on device %d: %s", dev, hipGetErrorString(e));
    }
    g_static_scratch[dev] = ptr;
  }
  if (out) *out = g_static_scratch[dev];
  return 0;
}

}  // namespace dtas
