// Runtime of libalpha_hip: device, one persistent stream, stream-ordered caching allocator,
// hipGraph capture of whole steps, events.  Replaces the buffer/submit half of the reference's native
// addon (packages/helios/native/helios_vk.c:818-934 slab allocator + slot tables, :1068-1125 timeline
// submit/wait, :3192-3419 batch execute) with the HIP-native equivalents.
#include "common.h"
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <cmath>
#include <map>
#include <unordered_map>
#include <vector>

namespace {

struct Block { void *ptr; size_t bytes; uint64_t graph; };   // graph != 0: owned by that captured graph

struct Graph {
  hipGraph_t graph = nullptr;
  hipGraphExec_t exec = nullptr;
  std::vector<Block> reserved;      // blocks whose addresses are baked into the graph
};

struct Context {
  bool inited = false;
  int device = -1;
  hipStream_t stream = nullptr;
  hipDeviceProp_t prop;
  char err[512] = "";
  // allocator
  std::unordered_map<void *, Block> live;
  std::map<size_t, std::vector<void *>> pool;           // size -> free blocks (global)
  std::map<size_t, std::vector<void *>> capture_pool;   // free blocks reusable only inside the open capture
  uint64_t pool_bytes = 0, live_bytes = 0, device_mallocs = 0, ops = 0;
  // capture
  bool capturing = false;
  uint64_t next_graph = 1, open_graph = 0;
  std::unordered_map<uint64_t, Graph> graphs;
  // scratch
  void *scratch = nullptr;
  size_t scratch_bytes = 0;
  // staging
  void *pinned = nullptr;
  size_t pinned_bytes = 0;
  // ring of small pinned slots: uploads of a few bytes (per-step hyper-parameters) need no stream sync
  char *ring = nullptr;
  unsigned ring_next = 0;
  hipEvent_t ring_ev[2] = {nullptr, nullptr};
};
Context g;

constexpr unsigned RING_SLOTS = 256, RING_SLOT_BYTES = 256;

size_t round_size(size_t b) {
  if (b == 0) b = 1;
  return (b + 511) & ~size_t(511);
}

}  // namespace

namespace ah {
hipStream_t stream() { return g.stream; }
bool ready() { return g.inited; }
int num_cus() { return g.prop.multiProcessorCount; }
int current_device() { return g.device; }
void count_op() { g.ops++; }
int32_t fail(int32_t code, const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g.err, sizeof(g.err), fmt, ap);
  va_end(ap);
  return code;
}
int32_t hip_fail(hipError_t e, const char *what) {
  snprintf(g.err, sizeof(g.err), "HIP error %d (%s) in %s", (int)e, hipGetErrorString(e), what);
  return AH_ERR_HIP;
}
void *scratch(size_t bytes) {
  if (bytes <= g.scratch_bytes) return g.scratch;
  // Growing scratch is only legal while no graph exists or is being captured (a graph replays into the addresses it
  // was captured with); ah_init sizes it for every reduction this library launches, so this branch is a safety net.
  if (g.capturing || !g.graphs.empty()) return nullptr;
  (void)hipStreamSynchronize(g.stream);
  if (g.scratch) (void)hipFree(g.scratch);
  g.scratch = nullptr; g.scratch_bytes = 0;
  if (hipMalloc(&g.scratch, bytes) != hipSuccess) return nullptr;
  g.scratch_bytes = bytes;
  return g.scratch;
}
}  // namespace ah

using namespace ah;

extern "C" {

const char *ah_last_error(void) { return g.err; }

int32_t ah_init(int32_t device) {
  if (g.inited) return AH_OK;
  int n = 0;
  AH_HIP(hipGetDeviceCount(&n));
  if (device < 0 || device >= n) return fail(AH_ERR_ARG, "ah_init: device %d out of range (%d visible)", device, n);
  AH_HIP(hipSetDevice(device));
  AH_HIP(hipGetDeviceProperties(&g.prop, device));
  if (strncmp(g.prop.gcnArchName, "gfx950", 6) != 0)
    return fail(AH_ERR_UNSUPPORTED, "ah_init: this library is built for gfx950 only, device is %s", g.prop.gcnArchName);
  AH_HIP(hipStreamCreateWithFlags(&g.stream, hipStreamNonBlocking));
  g.scratch_bytes = size_t(64) << 20;
  AH_HIP(hipMalloc(&g.scratch, g.scratch_bytes));
  g.pinned_bytes = size_t(64) << 20;
  AH_HIP(hipHostMalloc(&g.pinned, g.pinned_bytes, hipHostMallocDefault));
  AH_HIP(hipHostMalloc((void **)&g.ring, RING_SLOTS * RING_SLOT_BYTES, hipHostMallocDefault));
  AH_HIP(hipEventCreateWithFlags(&g.ring_ev[0], hipEventDisableTiming));
  AH_HIP(hipEventCreateWithFlags(&g.ring_ev[1], hipEventDisableTiming));
  g.device = device;
  { int32_t rc = static_partials_init(device); if (rc != AH_OK) return rc; }
  g.inited = true;
  g.err[0] = 0;
  return AH_OK;
}

int32_t ah_shutdown(void) {
  if (!g.inited) return AH_OK;
  (void)hipStreamSynchronize(g.stream);
  for (auto &kv : g.graphs) {
    if (kv.second.exec) (void)hipGraphExecDestroy(kv.second.exec);
    if (kv.second.graph) (void)hipGraphDestroy(kv.second.graph);
    for (auto &b : kv.second.reserved) (void)hipFree(b.ptr);
  }
  g.graphs.clear();
  for (auto &kv : g.live) (void)hipFree(kv.first);
  g.live.clear();
  for (auto &kv : g.pool) for (void *p : kv.second) (void)hipFree(p);
  g.pool.clear();
  for (auto &kv : g.capture_pool) for (void *p : kv.second) (void)hipFree(p);
  g.capture_pool.clear();
  if (g.scratch) (void)hipFree(g.scratch);
  if (g.pinned) (void)hipHostFree(g.pinned);
  if (g.ring) (void)hipHostFree(g.ring);
  if (g.ring_ev[0]) (void)hipEventDestroy(g.ring_ev[0]);
  if (g.ring_ev[1]) (void)hipEventDestroy(g.ring_ev[1]);
  (void)hipStreamDestroy(g.stream);
  g = Context();
  return AH_OK;
}

int32_t ah_device_info(AhDeviceInfo *out) {
  AH_REQUIRE_READY();
  AH_ARG(out != nullptr, "ah_device_info: null out");
  memset(out, 0, sizeof(*out));
  strncpy(out->name, g.prop.name, sizeof(out->name) - 1);
  strncpy(out->arch, g.prop.gcnArchName, sizeof(out->arch) - 1);
  out->compute_units = g.prop.multiProcessorCount;
  out->wavefront = g.prop.warpSize;
  out->clock_khz = g.prop.clockRate;
  out->lds_bytes_per_block = (int32_t)g.prop.sharedMemPerBlock;
  out->hbm_bytes = g.prop.totalGlobalMem;
  return AH_OK;
}

int32_t ah_sync(void) {
  AH_REQUIRE_READY();
  if (g.capturing) return fail(AH_ERR_STATE, "ah_sync: illegal while a graph is being captured");
  AH_HIP(hipStreamSynchronize(g.stream));
  return AH_OK;
}

int32_t ah_alloc(uint64_t bytes, ah_ptr *out) {
  AH_REQUIRE_READY();
  AH_ARG(out != nullptr, "ah_alloc: null out");
  size_t sz = round_size((size_t)bytes);
  void *p = nullptr;
  if (g.capturing) {
    auto it = g.capture_pool.find(sz);
    if (it != g.capture_pool.end() && !it->second.empty()) { p = it->second.back(); it->second.pop_back(); }
  }
  if (!p) {
    auto it = g.pool.find(sz);
    if (it != g.pool.end() && !it->second.empty()) { p = it->second.back(); it->second.pop_back(); g.pool_bytes -= sz; }
  }
  if (!p) {
    hipError_t e = hipMalloc(&p, sz);
    if (e != hipSuccess) {
      (void)hipGetLastError();
      return fail(AH_ERR_OOM, "ah_alloc: hipMalloc(%zu) failed: %s", sz, hipGetErrorString(e));
    }
    g.device_mallocs++;
  }
  g.live[p] = Block{p, sz, g.capturing ? g.open_graph : 0};
  g.live_bytes += sz;
  *out = (ah_ptr)(uintptr_t)p;
  return AH_OK;
}

int32_t ah_free(ah_ptr ptr) {
  AH_REQUIRE_READY();
  if (ptr == 0) return AH_OK;
  void *p = dp<void>(ptr);
  auto it = g.live.find(p);
  if (it == g.live.end()) return fail(AH_ERR_ARG, "ah_free: %p is not a live ah_alloc block", p);
  Block b = it->second;
  g.live.erase(it);
  g.live_bytes -= b.bytes;
  if (g.capturing) {
    // Reusable by later nodes of this capture only: the graph replays in the same order, so the
    // reuse is as safe on replay as it is now; outside the graph the address must stay reserved.
    g.capture_pool[b.bytes].push_back(p);
  } else if (b.graph != 0 && g.graphs.count(b.graph)) {
    g.graphs[b.graph].reserved.push_back(b);      // an output of a live graph: keep its address reserved
  } else {
    g.pool[b.bytes].push_back(p);
    g.pool_bytes += b.bytes;
  }
  return AH_OK;
}

int32_t ah_upload(ah_ptr dst, const void *host, uint64_t bytes) {
  AH_REQUIRE_READY();
  if (g.capturing) return fail(AH_ERR_STATE, "ah_upload: illegal while a graph is being captured");
  if (bytes == 0) return AH_OK;
  AH_ARG(dst != 0 && host != nullptr, "ah_upload: null pointer");
  if (bytes <= RING_SLOT_BYTES) {
    // Small upload: copy into the next pinned ring slot and enqueue; no wait.  An event per half of the ring
    // guarantees a slot's previous copy has completed before the slot is overwritten.
    unsigned slot = g.ring_next % RING_SLOTS, half = slot / (RING_SLOTS / 2);
    if (slot % (RING_SLOTS / 2) == 0 && g.ring_next >= RING_SLOTS) AH_HIP(hipEventSynchronize(g.ring_ev[half]));
    char *p = g.ring + (size_t)slot * RING_SLOT_BYTES;
    memcpy(p, host, bytes);
    AH_HIP(hipMemcpyAsync(dp<void>(dst), p, bytes, hipMemcpyHostToDevice, g.stream));
    if (slot % (RING_SLOTS / 2) == RING_SLOTS / 2 - 1) AH_HIP(hipEventRecord(g.ring_ev[half], g.stream));
    g.ring_next++;
    return AH_OK;
  }
  // Stage through pinned memory so the caller's buffer is free again when this returns.
  const char *src = (const char *)host;
  uint64_t off = 0;
  while (off < bytes) {
    size_t chunk = (size_t)((bytes - off) < g.pinned_bytes ? (bytes - off) : g.pinned_bytes);
    AH_HIP(hipStreamSynchronize(g.stream));            // previous chunk consumed
    memcpy(g.pinned, src + off, chunk);
    AH_HIP(hipMemcpyAsync(dp<char>(dst) + off, g.pinned, chunk, hipMemcpyHostToDevice, g.stream));
    off += chunk;
  }
  AH_HIP(hipStreamSynchronize(g.stream));              // the staging buffer is reusable on return
  return AH_OK;
}

int32_t ah_download(void *host, ah_ptr src, uint64_t bytes) {
  AH_REQUIRE_READY();
  if (g.capturing) return fail(AH_ERR_STATE, "ah_download: illegal while a graph is being captured");
  if (bytes == 0) return AH_OK;
  AH_ARG(src != 0 && host != nullptr, "ah_download: null pointer");
  char *dst = (char *)host;
  uint64_t off = 0;
  while (off < bytes) {
    size_t chunk = (size_t)((bytes - off) < g.pinned_bytes ? (bytes - off) : g.pinned_bytes);
    AH_HIP(hipMemcpyAsync(g.pinned, dp<char>(src) + off, chunk, hipMemcpyDeviceToHost, g.stream));
    AH_HIP(hipStreamSynchronize(g.stream));
    memcpy(dst + off, g.pinned, chunk);
    off += chunk;
  }
  return AH_OK;
}

int32_t ah_copy(ah_ptr dst, ah_ptr src, uint64_t bytes) {
  AH_REQUIRE_READY();
  if (bytes == 0) return AH_OK;
  AH_ARG(dst != 0 && src != 0, "ah_copy: null pointer");
  AH_HIP(hipMemcpyAsync(dp<void>(dst), dp<void>(src), bytes, hipMemcpyDeviceToDevice, g.stream));
  g.ops++;
  return AH_OK;
}

int32_t ah_stats(AhStats *out) {
  AH_REQUIRE_READY();
  AH_ARG(out != nullptr, "ah_stats: null out");
  out->live_allocs = g.live.size();
  out->live_bytes = g.live_bytes;
  uint64_t nb = 0;
  for (auto &kv : g.pool) nb += kv.second.size();
  out->pool_blocks = nb;
  out->pool_bytes = g.pool_bytes;
  out->device_mallocs = g.device_mallocs;
  out->ops_launched = g.ops;
  out->graphs_live = g.graphs.size();
  return AH_OK;
}

int32_t ah_reset_op_count(void) { g.ops = 0; return AH_OK; }

int32_t ah_trim_pool(void) {
  AH_REQUIRE_READY();
  if (g.capturing) return fail(AH_ERR_STATE, "ah_trim_pool: illegal while a graph is being captured");
  AH_HIP(hipStreamSynchronize(g.stream));
  for (auto &kv : g.pool) for (void *p : kv.second) (void)hipFree(p);
  g.pool.clear();
  g.pool_bytes = 0;
  return AH_OK;
}

int32_t ah_graph_begin(void) {
  AH_REQUIRE_READY();
  if (g.capturing) return fail(AH_ERR_STATE, "ah_graph_begin: a capture is already open");
  // Relaxed mode: allocator calls (hipMalloc) from this thread stay legal while capturing.
  AH_HIP(hipStreamBeginCapture(g.stream, hipStreamCaptureModeRelaxed));
  g.capturing = true;
  g.open_graph = g.next_graph++;
  g.graphs[g.open_graph] = Graph();
  return AH_OK;
}

int32_t ah_graph_end(uint64_t *out_graph) {
  AH_REQUIRE_READY();
  if (!g.capturing) return fail(AH_ERR_STATE, "ah_graph_end: no capture is open");
  Graph &gr = g.graphs[g.open_graph];
  hipError_t e = hipStreamEndCapture(g.stream, &gr.graph);
  g.capturing = false;
  // Blocks freed inside the capture keep their addresses reserved for the graph's lifetime.
  for (auto &kv : g.capture_pool)
    for (void *p : kv.second) gr.reserved.push_back(Block{p, kv.first, g.open_graph});
  g.capture_pool.clear();
  uint64_t id = g.open_graph;
  g.open_graph = 0;
  if (e != hipSuccess) { ah_graph_destroy(id); return hip_fail(e, "hipStreamEndCapture"); }
  e = hipGraphInstantiate(&gr.exec, gr.graph, nullptr, nullptr, 0);
  if (e != hipSuccess) { ah_graph_destroy(id); return hip_fail(e, "hipGraphInstantiate"); }
  if (out_graph) *out_graph = id;
  return AH_OK;
}

int32_t ah_graph_launch(uint64_t graph) {
  AH_REQUIRE_READY();
  auto it = g.graphs.find(graph);
  if (it == g.graphs.end() || !it->second.exec) return fail(AH_ERR_ARG, "ah_graph_launch: unknown graph %llu", (unsigned long long)graph);
  if (g.capturing) return fail(AH_ERR_STATE, "ah_graph_launch: illegal while a graph is being captured");
  AH_HIP(hipGraphLaunch(it->second.exec, g.stream));
  return AH_OK;
}

int32_t ah_graph_destroy(uint64_t graph) {
  AH_REQUIRE_READY();
  auto it = g.graphs.find(graph);
  if (it == g.graphs.end()) return fail(AH_ERR_ARG, "ah_graph_destroy: unknown graph %llu", (unsigned long long)graph);
  (void)hipStreamSynchronize(g.stream);
  if (it->second.exec) (void)hipGraphExecDestroy(it->second.exec);
  if (it->second.graph) (void)hipGraphDestroy(it->second.graph);
  for (auto &b : it->second.reserved) { g.pool[b.bytes].push_back(b.ptr); g.pool_bytes += b.bytes; }
  g.graphs.erase(it);
  return AH_OK;
}

int32_t ah_event_create(uint64_t *out_event) {
  AH_REQUIRE_READY();
  AH_ARG(out_event != nullptr, "ah_event_create: null out");
  hipEvent_t ev;
  AH_HIP(hipEventCreate(&ev));
  *out_event = (uint64_t)(uintptr_t)ev;
  return AH_OK;
}
int32_t ah_event_record(uint64_t event) {
  AH_REQUIRE_READY();
  AH_HIP(hipEventRecord((hipEvent_t)(uintptr_t)event, g.stream));
  return AH_OK;
}
int32_t ah_event_elapsed_ms(uint64_t start, uint64_t stop, float *out_ms) {
  AH_REQUIRE_READY();
  AH_ARG(out_ms != nullptr, "ah_event_elapsed_ms: null out");
  AH_HIP(hipEventSynchronize((hipEvent_t)(uintptr_t)stop));
  AH_HIP(hipEventElapsedTime(out_ms, (hipEvent_t)(uintptr_t)start, (hipEvent_t)(uintptr_t)stop));
  return AH_OK;
}
int32_t ah_event_destroy(uint64_t event) {
  AH_REQUIRE_READY();
  AH_HIP(hipEventDestroy((hipEvent_t)(uintptr_t)event));
  return AH_OK;
}

// ---- SeededRng (host only): packages/core/src/rng.ts:6-68 ----
static inline double rng_next(AhRng *r) {
  uint32_t x = (uint32_t)r->s0;
  const uint32_t y = (uint32_t)r->s1;
  r->s0 = (int32_t)y;
  x ^= x << 23;
  x ^= x >> 17;
  x ^= y;
  x ^= y >> 26;
  r->s1 = (int32_t)x;
  return (double)(uint32_t)(y + x) * (1.0 / 4294967296.0);
}
static inline double rng_gauss(AhRng *r) {
  if (r->has_spare) { r->has_spare = 0; return r->spare; }
  double u, v, s;
  do {
    u = rng_next(r) * 2 - 1;
    v = rng_next(r) * 2 - 1;
    s = u * u + v * v;
  } while (s >= 1 || s == 0);
  double mul = sqrt(-2.0 * log(s) / s);
  r->spare = v * mul;
  r->has_spare = 1;
  return u * mul;
}
int32_t ah_rng_seed(AhRng *r, int32_t seed) {
  if (!r) return fail(AH_ERR_ARG, "ah_rng_seed: null state");
  r->s0 = seed; r->s1 = seed ^ (int32_t)0xdeadbeef; r->has_spare = 0; r->_pad = 0; r->spare = 0;
  for (int i = 0; i < 20; i++) (void)rng_next(r);
  return AH_OK;
}
int32_t ah_rng_next(AhRng *r, double *out) {
  if (!r || !out) return fail(AH_ERR_ARG, "ah_rng_next: null argument");
  *out = rng_next(r);
  return AH_OK;
}
int32_t ah_rng_next_gauss(AhRng *r, double *out) {
  if (!r || !out) return fail(AH_ERR_ARG, "ah_rng_next_gauss: null argument");
  *out = rng_gauss(r);
  return AH_OK;
}
int32_t ah_rng_fill_gauss_f32(AhRng *r, float *out, uint64_t n, double std) {
  if (!r || (!out && n)) return fail(AH_ERR_ARG, "ah_rng_fill_gauss_f32: null argument");
  for (uint64_t i = 0; i < n; i++) out[i] = (float)(rng_gauss(r) * std);
  return AH_OK;
}
int32_t ah_rng_fill_uniform_f64(AhRng *r, double *out, uint64_t n) {
  if (!r || (!out && n)) return fail(AH_ERR_ARG, "ah_rng_fill_uniform_f64: null argument");
  for (uint64_t i = 0; i < n; i++) out[i] = rng_next(r);
  return AH_OK;
}

}  // extern "C"
