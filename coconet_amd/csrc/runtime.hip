// Runtime glue of libcoconet_hip: device set-up, memory, streams, events, error strings.
#include "ccn_common.hpp"

#include <new>

#include <cstdlib>
#include <cstring>
#include <atomic>
#include <mutex>
#include <unordered_map>

namespace ccn {

thread_local int g_last_hip_error = 0;

int hip_fail(hipError_t e) {
  g_last_hip_error = (int)e;
  (void)hipGetLastError();   // clear the sticky per-thread error so that later calls are not blamed for it
  switch (e) {
    case hipErrorOutOfMemory: return CCN_ENOMEM;
    case hipErrorInvalidValue:
    case hipErrorInvalidDevicePointer: return CCN_EINVAL;
    case hipErrorNoDevice:
    case hipErrorInvalidDevice: return CCN_ENODEV;
    default: return CCN_EHIP;
  }
}

namespace {
constexpr int kMaxDevices = 16;
DeviceInfo g_info[kMaxDevices];
std::once_flag g_once[kMaxDevices];
int g_init_rc[kMaxDevices];

int query_device(int dev) {
  hipDeviceProp_t prop;
  CCN_HIP(hipGetDeviceProperties(&prop, dev));
  DeviceInfo& di = g_info[dev];
  di.cu_count = prop.multiProcessorCount;
  di.hbm_bytes = prop.totalGlobalMem;
  std::strncpy(di.arch, prop.gcnArchName, sizeof(di.arch) - 1);
  if (std::strncmp(di.arch, "gfx950", 6) != 0) return CCN_ENODEV;   // the code object holds gfx950 ISA only
  di.device = dev;
  return CCN_OK;
}
}  // namespace

int current_device_info(const DeviceInfo** out) {
  int dev = -1;
  CCN_HIP(hipGetDevice(&dev));
  if (dev < 0 || dev >= kMaxDevices) return CCN_ENODEV;
  std::call_once(g_once[dev], [dev] { g_init_rc[dev] = query_device(dev); });
  if (g_init_rc[dev] != CCN_OK) return g_init_rc[dev];
  *out = &g_info[dev];
  return CCN_OK;
}

unsigned stream_grid(size_t units, size_t tile) {
  const DeviceInfo* di = nullptr;
  int cus = 256;
  if (current_device_info(&di) == CCN_OK) cus = di->cu_count;
  constexpr int per_cu = 8;   // 8 x 256 threads = one full CU of wavefronts
  size_t need = (units + tile - 1) / tile;
  size_t cap = (size_t)cus * (size_t)per_cu;
  if (need < 1) need = 1;
  return (unsigned)(need < cap ? need : cap);
}

unsigned lds_for_residency(int per_cu) {
  if (per_cu < 2 || per_cu > 16) return 0;
  const unsigned lds = (unsigned)(kLdsPerCu / (size_t)per_cu) & ~1023u;
  return lds > 64 * 1024 ? 64 * 1024 : lds;   // two per CU; larger requests need an opt-in attribute
}

StreamShape stream_shape(int load_bytes, int store_bytes, int grad_bytes, bool starts_alike) {
  StreamShape sh;
  // Single-wavefront workgroups, and fewer of them per CU the more 16-byte loads each thread has in flight.
  // Measured optima on MI355X at N = 2^28 (2^27 beyond 8 ranks), fp32 Adam unless said otherwise, as
  // loads per thread -> wavefronts per CU (% of HBM peak): 2 -> 26 (SGD at 1 rank: 85.5; 256-thread workgroups at full
  // occupancy 82.5), 3 -> 16-20 (SGD at 2 ranks: 84.6; 13: 79), 4 -> 17 (SGD at 3 ranks: 84.6; 13: 81), 5 -> 11-14 (84),
  // 7 -> 12-13 (83), 9 -> 8 (86; SGD at 8 ranks: 84), 11 -> 7 (85.5; 6 or 8 give 82-83), 15 -> 8 (82), 19 -> 6-10 (79).
  // Between 5 and 7 the optimum moves by one or two wavefronts with what else the thread does (% of peak at 11 / 12 /
  // 13 wavefronts): one 16-byte store (SGD) 5 -> 82.9 / 83.8 / 84.4, 6 -> 83.5 / 84.6 / 84.5, 7 -> 85.0 / 83.8 / 82.7;
  // fp32 Adam (three stores) 5 -> 84.9 / 83.4 / 82.5, 6 -> 85.1 / 84.8 / 83.7, 7 -> 82.2 / 82.9 / 82.9; Adam with 16-bit
  // gradients (8-byte loads, so more of them per byte; four stores) 5 -> 80.1 / 83.0 / 82.0, 6 -> 81.0 / 82.0 / 81.4,
  // 7 -> 82.0 / 81.3 / 80.5.
  const int loads = (load_bytes + 15) / 16;
  const int mid = store_bytes <= 16 ? (loads == 7 ? 11 : 13)
                                    : (grad_bytes == 2 ? (loads == 7 ? 11 : 12) : (loads <= 6 ? 11 : 12));
  // From 8 loads on, arrays that all start alike (plain allocations of equal size) want more wavefronts than staggered
  // ones: a thread's loads then queue on one channel and take longer to come back.  fp32 Adam at 8 ranks on plain
  // allocations: 10 per CU 79.4 %, 7 per CU 76.3 % (staggered: 80.2 % and 85.1 %); SGD at 8 ranks: 10 -> 80.3 %, 8 -> 79.0 %.
  const int many = starts_alike ? 10 : (loads <= 10 ? 8 : (loads <= 13 ? 7 : 8));
  const int waves = loads <= 2 ? 26 : (loads <= 4 ? 17 : (loads <= 7 ? mid : many));
  sh.block = 64;
  sh.lds_bytes = ((160u * 1024u / (unsigned)waves) / 1024u) * 1024u;
  return sh;
}

}  // namespace ccn

using namespace ccn;

extern "C" {

int ccn_version(void) { return 1; }

int ccn_init(int device) {
  int count = 0;
  CCN_HIP(hipGetDeviceCount(&count));
  if (device < 0 || device >= count) return CCN_ENODEV;
  CCN_HIP(hipSetDevice(device));
  const DeviceInfo* di = nullptr;
  const int rc = current_device_info(&di);
  if (rc != CCN_OK) return rc;
  return lamb_static_setup();
}

int ccn_device_info(int* cu_count, size_t* hbm_bytes, char* arch, size_t arch_len) {
  const DeviceInfo* di = nullptr;
  int rc = current_device_info(&di);
  if (rc != CCN_OK) return rc;
  if (cu_count) *cu_count = di->cu_count;
  if (hbm_bytes) *hbm_bytes = di->hbm_bytes;
  if (arch && arch_len) {
    std::strncpy(arch, di->arch, arch_len - 1);
    arch[arch_len - 1] = 0;
  }
  return CCN_OK;
}

// Large buffers are handed out at staggered offsets.  The fused kernels walk up to 14 arrays at the same element
// index; when those arrays start a multiple of 16 KiB apart (what same-sized hipMalloc blocks do: they come back
// 2 MiB aligned), their accesses keep landing on the same HBM channels and banks and the P=8 Adam step drops from
// ~82% to ~66% of peak bandwidth.  Successive allocations are therefore shifted by multiples of 4 KiB inside a
// 64 KiB pad (steps of 2 KiB to 1 MiB that are not multiples of 16 KiB all measure within a few percent).
namespace {
constexpr size_t kStaggerMin = 4u << 20;       // only buffers of at least 4 MiB are staggered
constexpr size_t kStaggerStep = 4 * 1024;
constexpr size_t kStaggerSlots = 16;
constexpr size_t kStaggerPad = kStaggerStep * kStaggerSlots;
std::mutex g_alloc_mu;                            // guards the map only; hipMalloc / hipFree run outside it
std::unordered_map<void*, void*> g_alloc_base;   // pointer given to the caller -> hipMalloc base
std::atomic<size_t> g_alloc_count{0};             // staggered allocations so far: picks the slot
std::atomic<size_t> g_alloc_live{0};              // staggered allocations not yet freed: ccn_free skips the map at zero
}  // namespace

int ccn_malloc(void** p, size_t bytes) {
  if (!p) return CCN_EINVAL;
  *p = nullptr;
  if (bytes == 0) return CCN_OK;
  if (bytes < kStaggerMin) {
    CCN_HIP(hipMalloc(p, bytes));
    return CCN_OK;
  }
  void* base = nullptr;
  CCN_HIP(hipMalloc(&base, bytes + kStaggerPad));
  // Allocation c takes slot (c + c/16 + c/256 + c/4096) mod 16: allocations 1, 16, 256 or 4096 apart in the
  // sequence all land in different slots, so the arrays walked in lock step differ whether the caller allocated
  // rank by rank or tensor by tensor.
  const size_t c = g_alloc_count.fetch_add(1, std::memory_order_relaxed);
  const size_t slot = (c + c / 16 + c / 256 + c / 4096) % kStaggerSlots;
  void* const user = static_cast<char*>(base) + slot * kStaggerStep;
  const int rc = guarded([&] {
    std::lock_guard<std::mutex> lock(g_alloc_mu);
    g_alloc_base[user] = base;
    g_alloc_live.fetch_add(1, std::memory_order_release);
    *p = user;
    return CCN_OK;
  });
  if (rc != CCN_OK) (void)hipFree(base);
  return rc;
}

int ccn_free(void* p) {
  if (!p) return CCN_OK;
  void* base = p;
  if (g_alloc_live.load(std::memory_order_acquire) != 0) {   // small buffers, and any buffer while nothing is staggered, go straight on
    std::lock_guard<std::mutex> lock(g_alloc_mu);
    auto it = g_alloc_base.find(p);
    if (it != g_alloc_base.end()) {
      base = it->second;
      g_alloc_base.erase(it);
      g_alloc_live.fetch_sub(1, std::memory_order_release);
    }
  }
  CCN_HIP(hipFree(base));
  return CCN_OK;
}

int ccn_memcpy_h2d(void* dst, const void* src, size_t bytes, void* stream) {
  if (bytes == 0) return CCN_OK;
  if (!dst || !src) return CCN_EINVAL;
  CCN_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, as_stream(stream)));
  return CCN_OK;
}

int ccn_memcpy_d2h(void* dst, const void* src, size_t bytes, void* stream) {
  if (bytes == 0) return CCN_OK;
  if (!dst || !src) return CCN_EINVAL;
  CCN_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, as_stream(stream)));
  CCN_HIP(hipStreamSynchronize(as_stream(stream)));
  return CCN_OK;
}

int ccn_memcpy_d2d(void* dst, const void* src, size_t bytes, void* stream) {
  if (bytes == 0) return CCN_OK;
  if (!dst || !src) return CCN_EINVAL;
  CCN_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, as_stream(stream)));
  return CCN_OK;
}

int ccn_stream_create(void** stream) {
  if (!stream) return CCN_EINVAL;
  hipStream_t s;
  CCN_HIP(hipStreamCreate(&s));   // default priority only
  *stream = (void*)s;
  return CCN_OK;
}

int ccn_stream_destroy(void* stream) {
  if (!stream) return CCN_OK;
  CCN_HIP(hipStreamDestroy(as_stream(stream)));
  return CCN_OK;
}

int ccn_stream_sync(void* stream) {
  CCN_HIP(hipStreamSynchronize(as_stream(stream)));
  return CCN_OK;
}

int ccn_event_create(void** ev) {
  if (!ev) return CCN_EINVAL;
  hipEvent_t e;
  CCN_HIP(hipEventCreate(&e));
  *ev = (void*)e;
  return CCN_OK;
}

int ccn_event_destroy(void* ev) {
  if (!ev) return CCN_OK;
  CCN_HIP(hipEventDestroy((hipEvent_t)ev));
  return CCN_OK;
}

int ccn_event_record(void* ev, void* stream) {
  if (!ev) return CCN_EINVAL;
  CCN_HIP(hipEventRecord((hipEvent_t)ev, as_stream(stream)));
  return CCN_OK;
}

int ccn_stream_wait_event(void* stream, void* ev) {
  if (!ev) return CCN_EINVAL;
  CCN_HIP(hipStreamWaitEvent(as_stream(stream), (hipEvent_t)ev, 0));
  return CCN_OK;
}

int ccn_event_elapsed_ms(void* start, void* stop, float* ms) {
  if (!start || !stop || !ms) return CCN_EINVAL;
  CCN_HIP(hipEventSynchronize((hipEvent_t)stop));
  CCN_HIP(hipEventElapsedTime(ms, (hipEvent_t)start, (hipEvent_t)stop));
  return CCN_OK;
}

struct ccn_graph {
  hipGraph_t graph = nullptr;
  hipGraphExec_t exec = nullptr;
};

int ccn_graph_begin(void* stream) {
  if (!stream) return CCN_EINVAL;   // the null stream cannot be captured
  CCN_HIP(hipStreamBeginCapture(as_stream(stream), hipStreamCaptureModeThreadLocal));
  return CCN_OK;
}

int ccn_graph_end(void* stream, ccn_graph** graph) {
  if (!stream || !graph) return CCN_EINVAL;
  *graph = nullptr;
  hipGraph_t g = nullptr;
  CCN_HIP(hipStreamEndCapture(as_stream(stream), &g));
  if (!g) return CCN_EHIP;
  hipGraphExec_t exec = nullptr;
  const hipError_t e = hipGraphInstantiate(&exec, g, nullptr, nullptr, 0);
  if (e != hipSuccess) {
    (void)hipGraphDestroy(g);
    return hip_fail(e);
  }
  ccn_graph* out = new (std::nothrow) ccn_graph();
  if (!out) {
    (void)hipGraphExecDestroy(exec);
    (void)hipGraphDestroy(g);
    return CCN_ENOMEM;
  }
  out->graph = g;
  out->exec = exec;
  *graph = out;
  return CCN_OK;
}

int ccn_graph_launch(ccn_graph* graph, void* stream) {
  if (!graph || !graph->exec) return CCN_EINVAL;
  CCN_HIP(hipGraphLaunch(graph->exec, as_stream(stream)));
  return CCN_OK;
}

int ccn_graph_destroy(ccn_graph* graph) {
  if (!graph) return CCN_OK;
  int rc = CCN_OK;
  if (graph->exec && hipGraphExecDestroy(graph->exec) != hipSuccess) rc = CCN_EHIP;
  if (graph->graph && hipGraphDestroy(graph->graph) != hipSuccess) rc = CCN_EHIP;
  delete graph;
  return rc;
}

int ccn_last_hip_error(void) { return g_last_hip_error; }

const char* ccn_strerror(int code) {
  switch (code) {
    case CCN_OK: return "success";
    case CCN_EINVAL: return "invalid argument (null pointer, zero size, rank count out of range, bad mode or misaligned buffer)";
    case CCN_ENOMEM: return "out of device memory";
    case CCN_ENODEV: return "no such device, or the device is not gfx950";
    case CCN_EHIP: return "HIP runtime error (see ccn_last_hip_error)";
    case CCN_ERANGE: return "size out of the supported range";
    default: return "unknown error code";
  }
}

}  // extern "C"
