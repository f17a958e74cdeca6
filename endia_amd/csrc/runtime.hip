// Context, buffer pool, copies and timers of libendia_hip.so.
//
// The reference allocates and zero-fills a fresh heap buffer for every op output
// (endia/functional/_utils.mojo:319-327) and frees it when the node dies
// (endia/_array/_array.mojo:177-179). Here the same two calls hit a size-bucketed pool of device
// buffers, so a training step runs without hipMalloc after its first iteration, and buffers
// that a kernel overwrites completely are never memset.
#include "common.h"

#include <map>
#include <string.h>
#include <unordered_map>
#include <vector>

namespace endia {

static Context g_ctx;
Context& ctx() { return g_ctx; }

static thread_local char g_err[512] = "";

int32_t fail(int32_t code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

// ---- pool ---------------------------------------------------------------------------------
// Sizes round up to 512 B below 1 MiB and to 2 MiB above, so the activations of one layer
// shape all land in one bucket.
static int64_t bucket_of(int64_t bytes) {
  if (bytes <= 0) bytes = 1;
  const int64_t small = 512, large = 2ll << 20;
  if (bytes <= (1ll << 20)) return (bytes + small - 1) / small * small;
  return (bytes + large - 1) / large * large;
}

struct Live {
  int64_t bucket;
  int64_t graph;  // 0, or the captured graph during whose capture the buffer was handed out
};

struct Pool {
  std::multimap<int64_t, void*> free_by_size;
  std::unordered_map<void*, Live> live;       // handed out
  std::unordered_map<void*, int64_t> owned;   // every pointer obtained from hipMalloc
  int64_t in_use = 0, cached = 0, n_allocs = 0;
};
static Pool g_pool;

// A captured step keeps every buffer that was handed out while it was being captured: its kernels hold
// those addresses, so the buffers go back to the pool only when the graph is destroyed.
struct Graph {
  hipGraph_t graph = nullptr;
  hipGraphExec_t exec = nullptr;
  std::vector<std::pair<void*, int64_t>> retained;  // released by their holders, kept for replays
};
static std::unordered_map<int64_t, Graph> g_graphs;
static int64_t g_next_graph = 1, g_capture_id = 0;

static void* g_ws = nullptr;
static int64_t g_ws_bytes = 0;
// Workspaces that were outgrown while captured steps existed: kernels recorded in those steps hold the
// old address, so the memory stays allocated until the last captured step has been destroyed.
static std::vector<void*> g_ws_retired;

static void free_retired_workspaces() {
  for (void* p : g_ws_retired) (void)hipFree(p);
  g_ws_retired.clear();
}

int32_t workspace(int64_t bytes, void** out) {
  if (bytes > g_ws_bytes) {
    if (g_ctx.capturing)
      return fail(ENDIA_HIP_ERR_UNSUPPORTED, "workspace: would have to grow during capture; run the step once eagerly first");
    if (g_ws) {
      if (g_graphs.empty())
        (void)hipFree(g_ws);  // blocks until the queued users of the old workspace have finished
      else
        g_ws_retired.push_back(g_ws);
    }
    g_ws = nullptr;
    g_ws_bytes = 0;
    int64_t want = bucket_of(bytes);
    hipError_t e = hipMalloc(&g_ws, (size_t)want);
    if (e != hipSuccess)
      return fail(ENDIA_HIP_ERR_NOMEM, "workspace: hipMalloc(%lld) failed: %s", (long long)want,
                  hipGetErrorString(e));
    g_ws_bytes = want;
  }
  *out = g_ws;
  return ENDIA_HIP_OK;
}

static const int kTimerSlots = 64;
static hipEvent_t g_ev_start[kTimerSlots], g_ev_stop[kTimerSlots];
static bool g_ev_made = false;

}  // namespace endia

using namespace endia;

static void release_graph(int64_t id);

extern "C" {

const char* endia_hip_last_error(void) { return g_err; }

int32_t endia_hip_init(int32_t device) {
  if (g_ctx.ready) {
    if (g_ctx.device == device) return ENDIA_HIP_OK;
    return fail(ENDIA_HIP_ERR_INVALID, "endia_hip_init: already initialised on device %d", g_ctx.device);
  }
  int count = 0;
  hipError_t e = hipGetDeviceCount(&count);
  if (e != hipSuccess || count == 0)
    return fail(ENDIA_HIP_ERR_RUNTIME, "endia_hip_init: no HIP device visible (%s)",
                e == hipSuccess ? "count = 0" : hipGetErrorString(e));
  ENDIA_CHECK_ARG(device >= 0 && device < count, "endia_hip_init: device %d out of range [0,%d)", device, count);
  ENDIA_HIP_CALL(hipSetDevice(device));
  hipDeviceProp_t prop;
  ENDIA_HIP_CALL(hipGetDeviceProperties(&prop, device));
  if (strncmp(prop.gcnArchName, "gfx950", 6) != 0)
    return fail(ENDIA_HIP_ERR_UNSUPPORTED, "endia_hip_init: device is %s; this library holds gfx950 code only",
                prop.gcnArchName);
  ENDIA_HIP_CALL(hipStreamCreateWithFlags(&g_ctx.stream, hipStreamNonBlocking));
  if (!g_ev_made) {
    for (int i = 0; i < kTimerSlots; ++i) {
      ENDIA_HIP_CALL(hipEventCreate(&g_ev_start[i]));
      ENDIA_HIP_CALL(hipEventCreate(&g_ev_stop[i]));
    }
    g_ev_made = true;
  }
  ENDIA_HIP_CALL(hipMalloc(reinterpret_cast<void**>(&g_ctx.tickets), kTicketCount * sizeof(unsigned)));
  ENDIA_HIP_CALL(hipMemset(g_ctx.tickets, 0, kTicketCount * sizeof(unsigned)));
  {
    int32_t rc = static_scratch_init(device);
    if (rc) return rc;
  }
  g_ctx.device = device;
  g_ctx.cu_count = prop.multiProcessorCount;
  g_ctx.clock_mhz = prop.clockRate / 1000;
  g_ctx.ready = true;
  return ENDIA_HIP_OK;
}

int32_t endia_hip_shutdown(void) {
  if (!g_ctx.ready) return ENDIA_HIP_OK;
  if (g_ctx.capturing) {  // abandon the unfinished capture; nothing recorded in it has run
    hipGraph_t dropped = nullptr;
    (void)hipStreamEndCapture(g_ctx.stream, &dropped);
    if (dropped) (void)hipGraphDestroy(dropped);
    (void)hipGetLastError();
    g_ctx.capturing = false;
  }
  (void)hipStreamSynchronize(g_ctx.stream);
  while (!g_graphs.empty()) release_graph(g_graphs.begin()->first);
  free_retired_workspaces();
  for (auto& kv : g_pool.owned) (void)hipFree(kv.first);
  g_pool = Pool();
  if (g_ws) (void)hipFree(g_ws);
  g_ws = nullptr;
  g_ws_bytes = 0;
  if (g_ctx.tickets) (void)hipFree(g_ctx.tickets);
  (void)hipStreamDestroy(g_ctx.stream);
  g_ctx = Context();
  return ENDIA_HIP_OK;
}

int32_t endia_hip_sync(void) {
  ENDIA_REQUIRE_INIT();
  if (g_ctx.capturing) return fail(ENDIA_HIP_ERR_UNSUPPORTED, "%s: not allowed while a step is being captured", __func__);
  ENDIA_HIP_CALL(hipStreamSynchronize(g_ctx.stream));
  return ENDIA_HIP_OK;
}

int32_t endia_hip_device_info(char* buf, int64_t buf_bytes, int32_t* cu_count, int32_t* clock_mhz) {
  ENDIA_REQUIRE_INIT();
  hipDeviceProp_t prop;
  ENDIA_HIP_CALL(hipGetDeviceProperties(&prop, g_ctx.device));
  if (buf && buf_bytes > 0)
    snprintf(buf, (size_t)buf_bytes, "%s %s, %d CUs, %d MHz, %.1f GiB", prop.name, prop.gcnArchName,
             prop.multiProcessorCount, prop.clockRate / 1000, prop.totalGlobalMem / 1073741824.0);
  if (cu_count) *cu_count = prop.multiProcessorCount;
  if (clock_mhz) *clock_mhz = prop.clockRate / 1000;
  return ENDIA_HIP_OK;
}

int32_t endia_hip_malloc(int64_t bytes, void** out) {
  ENDIA_REQUIRE_INIT();
  ENDIA_CHECK_ARG(out != nullptr, "endia_hip_malloc: out is null");
  ENDIA_CHECK_ARG(bytes >= 0, "endia_hip_malloc: negative size %lld", (long long)bytes);
  int64_t b = bucket_of(bytes);
  auto it = g_pool.free_by_size.find(b);
  void* p = nullptr;
  if (it != g_pool.free_by_size.end()) {
    p = it->second;
    g_pool.free_by_size.erase(it);
    g_pool.cached -= b;
  } else {
    hipError_t e = hipMalloc(&p, (size_t)b);
    if (e != hipSuccess) {
      // give cached buffers back to the driver and retry once
      (void)hipStreamSynchronize(g_ctx.stream);
      for (auto& kv : g_pool.free_by_size) {
        (void)hipFree(kv.second);
        g_pool.owned.erase(kv.second);
      }
      g_pool.free_by_size.clear();
      g_pool.cached = 0;
      (void)hipGetLastError();
      e = hipMalloc(&p, (size_t)b);
      if (e != hipSuccess) {
        (void)hipGetLastError();
        *out = nullptr;
        return fail(ENDIA_HIP_ERR_NOMEM, "endia_hip_malloc: hipMalloc(%lld) failed: %s", (long long)b,
                    hipGetErrorString(e));
      }
    }
    g_pool.owned[p] = b;
    g_pool.n_allocs++;
  }
  g_pool.live[p] = Live{b, g_ctx.capturing ? g_capture_id : 0};
  g_pool.in_use += b;
  *out = p;
  return ENDIA_HIP_OK;
}

int32_t endia_hip_free(void* p) {
  ENDIA_REQUIRE_INIT();
  if (!p) return ENDIA_HIP_OK;
  auto it = g_pool.live.find(p);
  ENDIA_CHECK_ARG(it != g_pool.live.end(), "endia_hip_free: %p was not handed out by endia_hip_malloc", p);
  int64_t b = it->second.bucket;
  int64_t owner = it->second.graph;
  g_pool.live.erase(it);
  g_pool.in_use -= b;
  auto g = owner ? g_graphs.find(owner) : g_graphs.end();
  if (g != g_graphs.end()) {
    g->second.retained.emplace_back(p, b);  // still written by replays of that graph
    return ENDIA_HIP_OK;
  }
  g_pool.free_by_size.emplace(b, p);
  g_pool.cached += b;
  return ENDIA_HIP_OK;
}

int32_t endia_hip_pool_stats(int64_t* bytes_in_use, int64_t* bytes_cached, int64_t* n_device_allocs) {
  ENDIA_REQUIRE_INIT();
  if (bytes_in_use) *bytes_in_use = g_pool.in_use;
  if (bytes_cached) *bytes_cached = g_pool.cached;
  if (n_device_allocs) *n_device_allocs = g_pool.n_allocs;
  return ENDIA_HIP_OK;
}

int32_t endia_hip_pool_trim(void) {
  ENDIA_REQUIRE_INIT();
  if (g_ctx.capturing) return fail(ENDIA_HIP_ERR_UNSUPPORTED, "%s: not allowed while a step is being captured", __func__);
  ENDIA_HIP_CALL(hipStreamSynchronize(g_ctx.stream));
  for (auto& kv : g_pool.free_by_size) {
    (void)hipFree(kv.second);
    g_pool.owned.erase(kv.second);
  }
  g_pool.free_by_size.clear();
  g_pool.cached = 0;
  return ENDIA_HIP_OK;
}

int32_t endia_hip_memcpy_h2d(void* dst, const void* src, int64_t bytes) {
  ENDIA_REQUIRE_INIT();
  if (g_ctx.capturing) return fail(ENDIA_HIP_ERR_UNSUPPORTED, "%s: not allowed while a step is being captured", __func__);
  ENDIA_CHECK_ARG(bytes >= 0, "endia_hip_memcpy_h2d: negative size");
  if (bytes == 0) return ENDIA_HIP_OK;
  ENDIA_CHECK_ARG(dst && src, "endia_hip_memcpy_h2d: null pointer");
  // pageable host memory: the copy is staged by the runtime and the host buffer may be reused on return
  ENDIA_HIP_CALL(hipMemcpyAsync(dst, src, (size_t)bytes, hipMemcpyHostToDevice, g_ctx.stream));
  ENDIA_HIP_CALL(hipStreamSynchronize(g_ctx.stream));
  return ENDIA_HIP_OK;
}

int32_t endia_hip_memcpy_d2h(void* dst, const void* src, int64_t bytes) {
  ENDIA_REQUIRE_INIT();
  if (g_ctx.capturing) return fail(ENDIA_HIP_ERR_UNSUPPORTED, "%s: not allowed while a step is being captured", __func__);
  ENDIA_CHECK_ARG(bytes >= 0, "endia_hip_memcpy_d2h: negative size");
  if (bytes == 0) return ENDIA_HIP_OK;
  ENDIA_CHECK_ARG(dst && src, "endia_hip_memcpy_d2h: null pointer");
  ENDIA_HIP_CALL(hipMemcpyAsync(dst, src, (size_t)bytes, hipMemcpyDeviceToHost, g_ctx.stream));
  ENDIA_HIP_CALL(hipStreamSynchronize(g_ctx.stream));
  return ENDIA_HIP_OK;
}

int32_t endia_hip_memcpy_d2d(void* dst, const void* src, int64_t bytes) {
  ENDIA_REQUIRE_INIT();
  ENDIA_CHECK_ARG(bytes >= 0, "endia_hip_memcpy_d2d: negative size");
  if (bytes == 0) return ENDIA_HIP_OK;
  ENDIA_CHECK_ARG(dst && src, "endia_hip_memcpy_d2d: null pointer");
  ENDIA_HIP_CALL(hipMemcpyAsync(dst, src, (size_t)bytes, hipMemcpyDeviceToDevice, g_ctx.stream));
  return ENDIA_HIP_OK;
}

int32_t endia_hip_timer_start(int32_t slot) {
  ENDIA_REQUIRE_INIT();
  if (g_ctx.capturing) return fail(ENDIA_HIP_ERR_UNSUPPORTED, "%s: not allowed while a step is being captured", __func__);
  ENDIA_CHECK_ARG(slot >= 0 && slot < kTimerSlots, "endia_hip_timer_start: slot %d out of range", slot);
  ENDIA_HIP_CALL(hipEventRecord(g_ev_start[slot], g_ctx.stream));
  return ENDIA_HIP_OK;
}

int32_t endia_hip_timer_stop(int32_t slot) {
  ENDIA_REQUIRE_INIT();
  if (g_ctx.capturing) return fail(ENDIA_HIP_ERR_UNSUPPORTED, "%s: not allowed while a step is being captured", __func__);
  ENDIA_CHECK_ARG(slot >= 0 && slot < kTimerSlots, "endia_hip_timer_stop: slot %d out of range", slot);
  ENDIA_HIP_CALL(hipEventRecord(g_ev_stop[slot], g_ctx.stream));
  return ENDIA_HIP_OK;
}

int32_t endia_hip_timer_elapsed_ms(int32_t slot, float* ms) {
  ENDIA_REQUIRE_INIT();
  ENDIA_CHECK_ARG(slot >= 0 && slot < kTimerSlots, "endia_hip_timer_elapsed_ms: slot %d out of range", slot);
  ENDIA_CHECK_ARG(ms != nullptr, "endia_hip_timer_elapsed_ms: ms is null");
  ENDIA_HIP_CALL(hipEventSynchronize(g_ev_stop[slot]));
  ENDIA_HIP_CALL(hipEventElapsedTime(ms, g_ev_start[slot], g_ev_stop[slot]));
  return ENDIA_HIP_OK;
}

// ---- captured steps --------------------------------------------------------------------------
// Everything enqueued between begin and end is recorded into a HIP graph instead of being executed.
// Launch-latency-bound steps (the reference's 1-32-64-128-128-128-64-32-1 sine-fit MLP issues ~60
// kernels of a few microseconds each) are then replayed with one launch.
int32_t endia_hip_graph_begin(void) {
  ENDIA_REQUIRE_INIT();
  ENDIA_CHECK_ARG(!g_ctx.capturing, "endia_hip_graph_begin: a capture is already in progress");
  ENDIA_HIP_CALL(hipStreamSynchronize(g_ctx.stream));
  g_capture_id = g_next_graph++;
  g_graphs[g_capture_id] = Graph();
  hipError_t e = hipStreamBeginCapture(g_ctx.stream, hipStreamCaptureModeRelaxed);
  if (e != hipSuccess) {
    g_graphs.erase(g_capture_id);
    return fail(ENDIA_HIP_ERR_RUNTIME, "endia_hip_graph_begin: hipStreamBeginCapture failed: %s", hipGetErrorString(e));
  }
  g_ctx.capturing = true;
  return ENDIA_HIP_OK;
}

static void release_graph(int64_t id) {
  auto it = g_graphs.find(id);
  if (it == g_graphs.end()) return;
  if (it->second.exec) (void)hipGraphExecDestroy(it->second.exec);
  if (it->second.graph) (void)hipGraphDestroy(it->second.graph);
  for (auto& pb : it->second.retained) {
    g_pool.free_by_size.emplace(pb.second, pb.first);
    g_pool.cached += pb.second;
  }
  g_graphs.erase(it);
  // buffers of this graph that are still held elsewhere become ordinary buffers
  for (auto& kv : g_pool.live)
    if (kv.second.graph == id) kv.second.graph = 0;
  if (g_graphs.empty()) free_retired_workspaces();  // callers have synchronised the stream
}

int32_t endia_hip_graph_end(int64_t* handle) {
  ENDIA_REQUIRE_INIT();
  ENDIA_CHECK_ARG(g_ctx.capturing, "endia_hip_graph_end: no capture in progress");
  g_ctx.capturing = false;
  const int64_t id = g_capture_id;
  Graph& g = g_graphs[id];
  hipError_t e = hipStreamEndCapture(g_ctx.stream, &g.graph);
  if (e == hipSuccess) e = hipGraphInstantiate(&g.exec, g.graph, nullptr, nullptr, 0);
  if (e != hipSuccess || !handle) {
    (void)hipGetLastError();
    release_graph(id);
    if (!handle) return fail(ENDIA_HIP_ERR_INVALID, "endia_hip_graph_end: handle is null");
    return fail(ENDIA_HIP_ERR_RUNTIME, "endia_hip_graph_end: capture failed: %s", hipGetErrorString(e));
  }
  *handle = id;
  return ENDIA_HIP_OK;
}

int32_t endia_hip_graph_launch(int64_t handle) {
  ENDIA_REQUIRE_INIT();
  ENDIA_CHECK_ARG(!g_ctx.capturing, "endia_hip_graph_launch: not allowed while a step is being captured");
  auto it = g_graphs.find(handle);
  ENDIA_CHECK_ARG(it != g_graphs.end() && it->second.exec, "endia_hip_graph_launch: unknown graph %lld", (long long)handle);
  ENDIA_HIP_CALL(hipGraphLaunch(it->second.exec, g_ctx.stream));
  return ENDIA_HIP_OK;
}

int32_t endia_hip_graph_destroy(int64_t handle) {
  ENDIA_REQUIRE_INIT();
  ENDIA_CHECK_ARG(g_graphs.count(handle), "endia_hip_graph_destroy: unknown graph %lld", (long long)handle);
  ENDIA_HIP_CALL(hipStreamSynchronize(g_ctx.stream));
  release_graph(handle);
  return ENDIA_HIP_OK;
}

}  // extern "C"
