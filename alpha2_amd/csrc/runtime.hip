// Runtime of libalpha_hip: device, one persistent stream, stream-ordered caching allocator,
// hipGraph capture of whole steps, events.  Replaces the buffer/submit half of the reference's native
// addon (packages/helios/native/helios_vk.c:818-934 slab allocator + slot tables, :1068-1125 timeline
// submit/wait, :3192-3419 batch execute) with the HIP-native equivalents.
#include "common.h"
#include <algorithm>
#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <cmath>
#include <map>
#include <set>
#include <string>
#include <unordered_map>
#include <vector>

namespace {

struct Block { void *ptr; size_t bytes; uint64_t graph; };   // graph != 0: owned by that captured graph

struct Graph {
  hipGraph_t graph = nullptr;
  hipGraphExec_t exec = nullptr;
  std::vector<Block> reserved;      // blocks whose addresses are baked into the graph
};

// ---- step plans: the kernel launches of one training step, recorded once as hipGraph segments and replayed ----
struct StepOp {
  const void *func = nullptr;
  dim3 grid, block;
  unsigned shmem = 0;
  std::vector<uint32_t> off, size;     // per kernel argument: offset into blob, byte size
  std::vector<char> blob;              // the argument values of the most recent step
  hipGraphNode_t node = nullptr;
  void fill_ptrs(std::vector<void *> &ptrs) {
    ptrs.resize(off.size() + 1);
    for (size_t i = 0; i < off.size(); i++) ptrs[i] = blob.data() + off[i];
    ptrs[off.size()] = nullptr;
  }
};
struct StepSeg {                       // the launches between two points where the host needs the stream
  std::vector<StepOp> ops;
  std::string boundary;                // what ended the segment: "ah_download", "ah_sync", ..., "ah_step_end"
  hipGraph_t graph = nullptr;
  hipGraphExec_t exec = nullptr;
  hipEvent_t done = nullptr;           // recorded after every launch of exec
};
struct PinnedSlot { char *host = nullptr; void *dev = nullptr; size_t bytes = 0; size_t seg = 0; };
struct StepPlan {
  std::vector<StepSeg> segs;
  std::vector<PinnedSlot> slots;       // one per ah_upload of the step, in call order
  bool complete = false, broken = false;
};
enum { STEP_OFF = 0, STEP_RECORD = 1, STEP_VERIFY = 2, STEP_EAGER = 3 };

constexpr unsigned EARLY_SLOTS = 16, EARLY_SLOT_BYTES = 256;
struct Context {
  bool inited = false;
  int device = -1;
  hipStream_t stream = nullptr;
  hipStream_t side = nullptr, cur = nullptr;      // side stream for ah_side_begin .. ah_side_end; cur = where launches go now
  hipEvent_t side_ev[2] = {nullptr, nullptr};     // main -> side ("start after this"), side -> main ("wait for the side work")
  bool side_used = false;
  unsigned chunks_since_host_boundary = 0;        // step plans, RECORD: how many size-limited segments since the host last needed the stream
  hipDeviceProp_t prop;
  char err[512] = "";
  // allocator
  std::unordered_map<void *, Block> live;
  // size -> free blocks, ordered by address: ah_alloc hands out the lowest one, so which block a request gets depends only on
  // WHICH blocks are free at that moment, not on the order in which they were freed (see ah_step_begin)
  std::map<size_t, std::set<void *>> pool;
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
  // read-backs started early (ah_download_begin): small pinned slots.  The copy runs on a stream of its own behind an event of
  // the main stream, and the host waits for the copy's own event on that stream: an event of the main stream cannot be waited
  // for while the main stream is capturing (step plans), one of another stream can.
  char *early = nullptr;
  hipStream_t early_stream = nullptr;
  hipEvent_t early_ev[EARLY_SLOTS] = {}, early_done[EARLY_SLOTS] = {};
  uint64_t early_id[EARLY_SLOTS] = {};
  uint32_t early_bytes[EARLY_SLOTS] = {};
  uint64_t early_next = 1;
  // step plans
  int step_mode = STEP_OFF;
  bool step_capture_open = false, step_fellback = false;
  uint64_t step_key = 0;
  StepPlan *plan = nullptr;
  size_t seg = 0, op = 0, slot = 0;
  std::vector<char> seg_waited;          // per segment: its previous launch is known to have finished (this step)
  std::map<uint64_t, StepPlan> plans;
  uint64_t steps_recorded = 0, steps_replayed = 0, steps_fallback = 0, step_node_updates = 0;
  char step_why[256] = "";
};
Context g;

constexpr unsigned RING_SLOTS = 256, RING_SLOT_BYTES = 256;

size_t round_size(size_t b) {
  if (b == 0) b = 1;
  return (b + 511) & ~size_t(511);
}

}  // namespace

namespace ah {
hipStream_t stream() { return g.cur; }
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
  if (g.cur != g.stream) return nullptr;      // side-stream work would race with main-stream users of the one buffer
  if (bytes <= g.scratch_bytes) return g.scratch;
  // Growing scratch is only legal while no graph or step plan exists or is being captured (their nodes replay into the
  // addresses they were recorded with, and a capturing stream cannot be synchronised); ah_init sizes it for every
  // reduction this library launches, so this branch is a safety net.  Callers fail with AH_ERR_OOM on nullptr.
  if (g.capturing || !g.graphs.empty() || !g.plans.empty() || g.step_capture_open || g.step_mode != STEP_OFF) return nullptr;
  (void)hipStreamSynchronize(g.stream);
  if (g.scratch) (void)hipFree(g.scratch);
  g.scratch = nullptr; g.scratch_bytes = 0;
  if (hipMalloc(&g.scratch, bytes) != hipSuccess) return nullptr;
  g.scratch_bytes = bytes;
  return g.scratch;
}

// ------------------------------------------------------------------------------------------ step plans
namespace {
constexpr size_t STEP_UPLOAD_MAX = size_t(16) << 20;     // larger uploads inside a step are a boundary, not a node
// A segment is closed after this many launches even when the host does not need the stream: on replay the graph of a
// chunk is launched as soon as its last launch has been verified, so the device works on chunk k while the host is still
// issuing (verifying) chunk k+1 -- the overlap eager execution has, at graph-launch cost.
constexpr size_t STEP_CHUNK = 32;

__global__ void k_step_copy(char *__restrict__ dst, const char *__restrict__ src, uint64_t bytes) {
  uint64_t tid = blockIdx.x * (uint64_t)blockDim.x + threadIdx.x, stride = (uint64_t)gridDim.x * blockDim.x;
  if ((((uintptr_t)dst | (uintptr_t)src) & 15u) == 0) {
    uint64_t n16 = bytes >> 4;
    for (uint64_t i = tid; i < n16; i += stride) reinterpret_cast<uint4 *>(dst)[i] = reinterpret_cast<const uint4 *>(src)[i];
    for (uint64_t i = (n16 << 4) + tid; i < bytes; i += stride) dst[i] = src[i];
  } else {
    for (uint64_t i = tid; i < bytes; i += stride) dst[i] = src[i];
  }
}
void step_copy(void *dst, const void *src, uint64_t bytes) {
  uint64_t blocks = (bytes / 16 + 255) / 256;
  if (blocks < 1) blocks = 1;
  if (blocks > 4096) blocks = 4096;
  ah::launch_kernel(k_step_copy, dim3((unsigned)blocks), dim3(256), 0, (char *)dst, (const char *)src, bytes);
}

void plan_destroy(StepPlan &p) {
  for (auto &sg : p.segs) {
    if (sg.done) { (void)hipEventSynchronize(sg.done); (void)hipEventDestroy(sg.done); }
    if (sg.exec) (void)hipGraphExecDestroy(sg.exec);
    if (sg.graph) (void)hipGraphDestroy(sg.graph);
  }
  for (auto &sl : p.slots) if (sl.host) (void)hipHostFree(sl.host);
  p = StepPlan();
}
void step_note(const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g.step_why, sizeof(g.step_why), fmt, ap);
  va_end(ap);
}
// The previous launch of this segment's graph must have finished before its parameters or its pinned slots change.
void seg_wait(size_t si) {
  if (si < g.seg_waited.size() && !g.seg_waited[si]) {
    StepSeg &sg = g.plan->segs[si];
    if (sg.done) (void)hipEventSynchronize(sg.done);
    g.seg_waited[si] = 1;
  }
}
// VERIFY -> EAGER: this step does not follow the plan.  The launches of the current segment that were skipped so far
// are issued now, from the recorded arguments (which are this step's: every difference was copied in); earlier segments
// have already run as graphs.  The plan is dropped at ah_step_end and recorded again by the next step.
void step_fallback(const char *why) {
  if (g.step_mode != STEP_VERIFY) return;
  StepSeg &sg = g.plan->segs[g.seg];
  std::vector<void *> ptrs;
  for (size_t i = 0; i < g.op && i < sg.ops.size(); i++) {
    StepOp &o = sg.ops[i];
    o.fill_ptrs(ptrs);
    (void)hipLaunchKernel(o.func, o.grid, o.block, ptrs.data(), o.shmem, g.stream);
  }
  g.step_mode = STEP_EAGER;
  g.step_fellback = true;
  step_note("%s (segment %zu, launch %zu)", why, g.seg, g.op);
}
bool same_launch(const StepOp &o, const void *func, dim3 grid, dim3 block, unsigned shmem, const uint32_t *sizes, int n) {
  if (o.func != func || o.shmem != shmem || (int)o.size.size() != n) return false;
  if (o.grid.x != grid.x || o.grid.y != grid.y || o.grid.z != grid.z) return false;
  if (o.block.x != block.x || o.block.y != block.y || o.block.z != block.z) return false;
  for (int i = 0; i < n; i++) if (o.size[i] != sizes[i]) return false;
  return true;
}
int32_t step_begin_capture() {
  AH_HIP(hipStreamBeginCapture(g.stream, hipStreamCaptureModeRelaxed));
  g.step_capture_open = true;
  return AH_OK;
}
// RECORD: close the capture of the current segment, instantiate and launch it.
int32_t step_close_segment(const char *what) {
  StepSeg &sg = g.plan->segs.back();
  sg.boundary = what;
  if (g.step_capture_open) {
    g.step_capture_open = false;
    AH_HIP(hipStreamEndCapture(g.stream, &sg.graph));
  }
  if (!sg.ops.empty()) {
    AH_HIP(hipGraphInstantiate(&sg.exec, sg.graph, nullptr, nullptr, 0));
    AH_HIP(hipEventCreateWithFlags(&sg.done, hipEventDisableTiming));
    AH_HIP(hipGraphLaunch(sg.exec, g.stream));
    AH_HIP(hipEventRecord(sg.done, g.stream));
  }
  return AH_OK;
}
}  // namespace

void launch_raw(const void *func, dim3 grid, dim3 block, unsigned shmem, void **args, const uint32_t *sizes, int nargs) {
  if (g.step_mode == STEP_OFF || g.step_mode == STEP_EAGER) {
    (void)hipLaunchKernel(func, grid, block, args, shmem, g.cur);          // an error is picked up by hipGetLastError
    return;
  }
  if (g.step_mode == STEP_RECORD) {
    if (hipLaunchKernel(func, grid, block, args, shmem, g.stream) != hipSuccess) { g.plan->broken = true; return; }
    StepSeg &sg = g.plan->segs.back();
    sg.ops.emplace_back();
    StepOp &o = sg.ops.back();
    o.func = func; o.grid = grid; o.block = block; o.shmem = shmem;
    uint32_t at = 0;
    for (int i = 0; i < nargs; i++) { o.off.push_back(at); o.size.push_back(sizes[i]); at += (sizes[i] + 15u) & ~15u; }
    o.blob.assign(at ? at : 16, 0);
    for (int i = 0; i < nargs; i++) memcpy(o.blob.data() + o.off[i], args[i], sizes[i]);
    hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
    const hipGraphNode_t *deps = nullptr;
    size_t ndeps = 0;
    if (hipStreamGetCaptureInfo_v2(g.stream, &st, nullptr, nullptr, &deps, &ndeps) == hipSuccess &&
        st == hipStreamCaptureStatusActive && ndeps == 1) o.node = deps[0];
    else g.plan->broken = true;            // cannot name the node: this plan will not be replayed
    // After a boundary the host made, the device is idle until the first chunk has been issued: chunks start small there
    // (4, 8, 16, ... launches) and grow to the full size.
    const size_t chunk = g.chunks_since_host_boundary < 3 ? (size_t(4) << g.chunks_since_host_boundary) : STEP_CHUNK;
    if (sg.ops.size() >= chunk && step_boundary("chunk") == AH_OK) {
      g.chunks_since_host_boundary++;
      (void)step_begin_capture();
    }
    return;
  }
  // STEP_VERIFY
  StepSeg &sg = g.plan->segs[g.seg];
  if (g.op < sg.ops.size() && same_launch(sg.ops[g.op], func, grid, block, shmem, sizes, nargs)) {
    StepOp &o = sg.ops[g.op];
    bool differ = false;
    for (int i = 0; i < nargs; i++)
      if (memcmp(o.blob.data() + o.off[i], args[i], sizes[i]) != 0) {
        memcpy(o.blob.data() + o.off[i], args[i], sizes[i]);
        differ = true;
      }
    g.op++;
    if (differ) {
      g.step_node_updates++;
      seg_wait(g.seg);
      std::vector<void *> ptrs;
      o.fill_ptrs(ptrs);
      hipKernelNodeParams kp;
      memset(&kp, 0, sizeof(kp));
      kp.func = const_cast<void *>(o.func); kp.gridDim = o.grid; kp.blockDim = o.block; kp.sharedMemBytes = o.shmem;
      kp.kernelParams = ptrs.data(); kp.extra = nullptr;
      if (hipGraphExecKernelNodeSetParams(sg.exec, o.node, &kp) != hipSuccess) {
        (void)hipGetLastError();
        step_fallback("a kernel node refused new parameters");    // launches [0, g.op) incl. this one, from the blobs
        return;
      }
    }
    if (g.op == sg.ops.size() && sg.boundary == "chunk") (void)step_boundary("chunk");
    return;
  }
  step_fallback("a different kernel launch than the plan's");
  (void)hipLaunchKernel(func, grid, block, args, shmem, g.stream);
}

bool step_active() { return g.step_mode != STEP_OFF; }

int32_t step_boundary(const char *what) {
  if (g.step_mode == STEP_OFF || g.step_mode == STEP_EAGER) return AH_OK;
  if (g.step_mode == STEP_RECORD) {
    if (g.plan->segs.back().ops.empty() && strcmp(what, "ah_step_end") != 0) {
      // nothing recorded since the last boundary: the host may touch the stream without a segment of its own
      g.chunks_since_host_boundary = 0;
      if (g.step_capture_open) {
        g.step_capture_open = false;
        hipGraph_t junk = nullptr;
        AH_HIP(hipStreamEndCapture(g.stream, &junk));
        if (junk) (void)hipGraphDestroy(junk);
      }
      return AH_OK;
    }
    int32_t rc = step_close_segment(what);
    if (rc != AH_OK) { g.plan->broken = true; return rc; }
    g.plan->segs.emplace_back();
    if (strcmp(what, "chunk") != 0 && strcmp(what, "kick") != 0) g.chunks_since_host_boundary = 0;
    return AH_OK;
  }
  StepSeg &sg = g.plan->segs[g.seg];
  if (g.op == 0 && !(sg.ops.empty() && sg.boundary == what) && strcmp(what, "ah_step_end") != 0) return AH_OK;   // likewise on replay
  if (g.op == sg.ops.size() && sg.boundary == what) {
    if (sg.exec) {
      AH_HIP(hipGraphLaunch(sg.exec, g.stream));
      AH_HIP(hipEventRecord(sg.done, g.stream));
      if (g.seg < g.seg_waited.size()) g.seg_waited[g.seg] = 0;
    }
    g.seg++; g.op = 0;
    if (g.seg >= g.plan->segs.size() && strcmp(what, "ah_step_end") != 0) {   // the plan ended here, the step goes on
      g.seg = g.plan->segs.size() - 1;
      g.op = g.plan->segs[g.seg].ops.size();
      g.step_mode = STEP_EAGER; g.step_fellback = true;
      step_note("the step continues past the end of the plan (%s)", what);
    }
    return AH_OK;
  }
  step_fallback(what);
  return AH_OK;
}
// After the blocking part of a boundary: RECORD resumes capturing into the next segment.
static int32_t step_resume() {
  if (g.step_mode == STEP_RECORD && !g.step_capture_open) return step_begin_capture();
  return AH_OK;
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
  AH_HIP(hipStreamCreateWithFlags(&g.side, hipStreamNonBlocking));       // same (default) priority as the main stream
  AH_HIP(hipEventCreateWithFlags(&g.side_ev[0], hipEventDisableTiming));
  AH_HIP(hipEventCreateWithFlags(&g.side_ev[1], hipEventDisableTiming));
  g.cur = g.stream;
  g.scratch_bytes = size_t(64) << 20;
  AH_HIP(hipMalloc(&g.scratch, g.scratch_bytes));
  g.pinned_bytes = size_t(64) << 20;
  AH_HIP(hipHostMalloc(&g.pinned, g.pinned_bytes, hipHostMallocDefault));
  AH_HIP(hipHostMalloc((void **)&g.ring, RING_SLOTS * RING_SLOT_BYTES, hipHostMallocDefault));
  AH_HIP(hipEventCreateWithFlags(&g.ring_ev[0], hipEventDisableTiming));
  AH_HIP(hipEventCreateWithFlags(&g.ring_ev[1], hipEventDisableTiming));
  AH_HIP(hipHostMalloc((void **)&g.early, EARLY_SLOTS * EARLY_SLOT_BYTES, hipHostMallocDefault));
  AH_HIP(hipStreamCreateWithFlags(&g.early_stream, hipStreamNonBlocking));
  for (unsigned i = 0; i < EARLY_SLOTS; i++) {
    AH_HIP(hipEventCreateWithFlags(&g.early_ev[i], hipEventDisableTiming));
    AH_HIP(hipEventCreateWithFlags(&g.early_done[i], hipEventDisableTiming));
    g.early_id[i] = 0;
  }
  g.early_next = 1;
  g.device = device;
  { int32_t rc = static_partials_init(device); if (rc != AH_OK) return rc; }
  g.inited = true;
  g.err[0] = 0;
  return AH_OK;
}

int32_t ah_shutdown(void) {
  if (!g.inited) return AH_OK;
  if (g.step_capture_open) { hipGraph_t junk = nullptr; (void)hipStreamEndCapture(g.stream, &junk); if (junk) (void)hipGraphDestroy(junk); }
  (void)hipStreamSynchronize(g.stream);
  for (auto &kv : g.plans) plan_destroy(kv.second);
  g.plans.clear();
  gemm_plans_forget();
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
  if (g.early) (void)hipHostFree(g.early);
  for (unsigned i = 0; i < EARLY_SLOTS; i++) {
    if (g.early_ev[i]) { (void)hipEventDestroy(g.early_ev[i]); g.early_ev[i] = nullptr; }
    if (g.early_done[i]) { (void)hipEventDestroy(g.early_done[i]); g.early_done[i] = nullptr; }
  }
  if (g.early_stream) { (void)hipStreamDestroy(g.early_stream); g.early_stream = nullptr; }
  g.early = nullptr;
  if (g.side) { (void)hipStreamSynchronize(g.side); (void)hipStreamDestroy(g.side); }
  if (g.side_ev[0]) (void)hipEventDestroy(g.side_ev[0]);
  if (g.side_ev[1]) (void)hipEventDestroy(g.side_ev[1]);
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
  { int32_t rc = step_boundary("ah_sync"); if (rc != AH_OK) return rc; }
  if (g.side_used) AH_HIP(hipStreamSynchronize(g.side));
  AH_HIP(hipStreamSynchronize(g.stream));
  return step_resume();
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
    if (it != g.pool.end() && !it->second.empty()) { p = *it->second.begin(); it->second.erase(it->second.begin()); g.pool_bytes -= sz; }
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
    g.pool[b.bytes].insert(p);
    g.pool_bytes += b.bytes;
  }
  return AH_OK;
}

int32_t ah_upload(ah_ptr dst, const void *host, uint64_t bytes) {
  AH_REQUIRE_READY();
  if (g.capturing) return fail(AH_ERR_STATE, "ah_upload: illegal while a graph is being captured");
  if (bytes == 0) return AH_OK;
  AH_ARG(dst != 0 && host != nullptr, "ah_upload: null pointer");
  if (g.step_mode == STEP_RECORD || g.step_mode == STEP_VERIFY) {
    // Inside a step plan an upload is a pinned slot owned by the plan plus a copy kernel: the graph node reads the slot,
    // and every later step only rewrites the slot's contents.
    if (bytes <= STEP_UPLOAD_MAX) {
      size_t k = g.slot++;
      StepPlan &pl = *g.plan;
      if (g.step_mode == STEP_RECORD) {
        PinnedSlot sl;
        sl.bytes = (size_t)((bytes + 255) & ~uint64_t(255));
        sl.seg = pl.segs.size() - 1;
        if (hipHostMalloc((void **)&sl.host, sl.bytes, hipHostMallocDefault) != hipSuccess ||
            hipHostGetDevicePointer(&sl.dev, sl.host, 0) != hipSuccess) {
          (void)hipGetLastError();
          pl.broken = true;
          return fail(AH_ERR_OOM, "ah_upload: no pinned slot of %zu bytes for the step plan", sl.bytes);
        }
        pl.slots.push_back(sl);
      } else if (k >= pl.slots.size() || pl.slots[k].bytes < bytes || pl.slots[k].seg != g.seg) {
        step_fallback("an upload the plan does not have");
      }
      if (g.step_mode != STEP_EAGER) {
        PinnedSlot &sl = pl.slots[k];
        if (g.step_mode == STEP_VERIFY) seg_wait(g.seg);
        memcpy(sl.host, host, bytes);
        step_copy(dp<void>(dst), sl.dev, bytes);
        AH_LAUNCH_CHECK();
        return AH_OK;
      }
    } else {
      int32_t rc = step_boundary("ah_upload(large)");
      if (rc != AH_OK) return rc;
    }
  }
  struct Resume { ~Resume() { (void)step_resume(); } } resume_capture_on_return;
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
  { int32_t rc = step_boundary("ah_download"); if (rc != AH_OK) return rc; }
  if (g.side_used && !g.capturing) AH_HIP(hipStreamSynchronize(g.side));     // side work may be what wrote `src`
  struct Resume { ~Resume() { (void)step_resume(); } } resume_capture_on_return;
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

int32_t ah_download_begin(ah_ptr src, uint64_t bytes, uint64_t *out_ticket) {
  AH_REQUIRE_READY();
  AH_ARG(out_ticket != nullptr, "ah_download_begin: null out_ticket");
  *out_ticket = 0;
  if (g.capturing) return fail(AH_ERR_STATE, "ah_download_begin: illegal while a graph is being captured");
  AH_ARG(src != 0 && bytes > 0 && bytes <= EARLY_SLOT_BYTES, "ah_download_begin: 1..%u bytes", EARLY_SLOT_BYTES);
  { int32_t rc = step_boundary("ah_download_begin"); if (rc != AH_OK) return rc; }
  struct Resume { ~Resume() { (void)step_resume(); } } resume_capture_on_return;
  const uint64_t id = g.early_next++;
  const unsigned slot = (unsigned)(id % EARLY_SLOTS);
  AH_HIP(hipEventRecord(g.early_ev[slot], g.stream));
  AH_HIP(hipStreamWaitEvent(g.early_stream, g.early_ev[slot], 0));
  AH_HIP(hipMemcpyAsync(g.early + slot * EARLY_SLOT_BYTES, dp<void>(src), bytes, hipMemcpyDeviceToHost, g.early_stream));
  AH_HIP(hipEventRecord(g.early_done[slot], g.early_stream));
  AH_HIP(hipStreamWaitEvent(g.stream, g.early_done[slot], 0));     // later work may overwrite `src`: it queues behind the copy
  g.early_id[slot] = id;
  g.early_bytes[slot] = (uint32_t)bytes;
  *out_ticket = id;
  return AH_OK;
}

int32_t ah_download_end(uint64_t ticket, void *host, uint64_t bytes) {
  AH_REQUIRE_READY();
  AH_ARG(host != nullptr, "ah_download_end: null host");
  const unsigned slot = (unsigned)(ticket % EARLY_SLOTS);
  if (ticket == 0 || g.early_id[slot] != ticket) return fail(AH_ERR_STATE, "ah_download_end: ticket %llu is no longer held (newer read-backs took its slot)", (unsigned long long)ticket);
  AH_ARG(bytes == g.early_bytes[slot], "ah_download_end: %llu bytes asked, %u copied", (unsigned long long)bytes, g.early_bytes[slot]);
  AH_HIP(hipEventSynchronize(g.early_done[slot]));
  memcpy(host, g.early + slot * EARLY_SLOT_BYTES, bytes);
  return AH_OK;
}

int32_t ah_copy(ah_ptr dst, ah_ptr src, uint64_t bytes) {
  AH_REQUIRE_READY();
  if (bytes == 0) return AH_OK;
  AH_ARG(dst != 0 && src != 0, "ah_copy: null pointer");
  if (g.step_mode != STEP_OFF) {                 // a kernel node like every other launch of the step
    step_copy(dp<void>(dst), dp<void>(src), bytes);
    AH_LAUNCH_CHECK();
    return AH_OK;
  }
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
  out->steps_recorded = g.steps_recorded;
  out->steps_replayed = g.steps_replayed;
  out->steps_fallback = g.steps_fallback;
  out->step_node_updates = g.step_node_updates;
  return AH_OK;
}

int32_t ah_reset_op_count(void) { g.ops = 0; return AH_OK; }

int32_t ah_trim_pool(void) {
  AH_REQUIRE_READY();
  if (g.capturing) return fail(AH_ERR_STATE, "ah_trim_pool: illegal while a graph is being captured");
  { int32_t rc = step_boundary("ah_trim_pool"); if (rc != AH_OK) return rc; }
  struct Resume { ~Resume() { (void)step_resume(); } } resume_capture_on_return;
  AH_HIP(hipStreamSynchronize(g.stream));
  for (auto &kv : g.pool) for (void *p : kv.second) (void)hipFree(p);
  g.pool.clear();
  g.pool_bytes = 0;
  return AH_OK;
}

int32_t ah_graph_begin(void) {
  AH_REQUIRE_READY();
  if (g.capturing) return fail(AH_ERR_STATE, "ah_graph_begin: a capture is already open");
  if (g.step_mode != STEP_OFF) return fail(AH_ERR_STATE, "ah_graph_begin: illegal inside ah_step_begin .. ah_step_end");
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
  if (g.cur != g.stream || g.side_used) {                 // a capture cannot end with forked work outstanding
    g.cur = g.stream;
    if (g.side_used) { (void)hipEventRecord(g.side_ev[1], g.side); (void)hipStreamWaitEvent(g.stream, g.side_ev[1], 0); g.side_used = false; }
  }
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
  if (g.step_mode != STEP_OFF) return fail(AH_ERR_STATE, "ah_graph_launch: illegal inside ah_step_begin .. ah_step_end");
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
  for (auto &b : it->second.reserved) { g.pool[b.bytes].insert(b.ptr); g.pool_bytes += b.bytes; }
  g.graphs.erase(it);
  return AH_OK;
}

int32_t ah_side_begin(void) {
  AH_REQUIRE_READY();
  if (g.cur != g.stream) return fail(AH_ERR_STATE, "ah_side_begin: the side stream is already open");
  if (g.step_mode != STEP_OFF) return AH_OK;              // inside a step plan everything stays on the one recorded stream
  AH_HIP(hipEventRecord(g.side_ev[0], g.stream));
  AH_HIP(hipStreamWaitEvent(g.side, g.side_ev[0], 0));
  g.cur = g.side;
  g.side_used = true;
  return AH_OK;
}
int32_t ah_side_end(void) {
  AH_REQUIRE_READY();
  g.cur = g.stream;
  return AH_OK;
}
int32_t ah_side_join(void) {
  AH_REQUIRE_READY();
  if (g.cur != g.stream) return fail(AH_ERR_STATE, "ah_side_join: ah_side_end first");
  if (!g.side_used) return AH_OK;
  AH_HIP(hipEventRecord(g.side_ev[1], g.side));
  AH_HIP(hipStreamWaitEvent(g.stream, g.side_ev[1], 0));
  g.side_used = false;
  return AH_OK;
}

int32_t ah_step_begin(uint64_t key) {
  AH_REQUIRE_READY();
  if (g.capturing) return fail(AH_ERR_STATE, "ah_step_begin: illegal while a graph is being captured");
  if (g.step_mode != STEP_OFF) return fail(AH_ERR_STATE, "ah_step_begin: a step is already open");
  // What makes replays cheap is that a step gets the addresses the last one got: free lists hand out their lowest address,
  // so steps that allocate and free in the same sequence get the same blocks whatever order the frees of the step before
  // came in, and whether they came before or after this call (most-recently-freed-first lists, even when sorted here,
  // settled into a cycle of two address sets on a 24-layer model with four micro-steps: 1500 rewritten nodes per step).
  StepPlan &pl = g.plans[key];
  g.plan = &pl; g.step_key = key; g.seg = 0; g.op = 0; g.slot = 0; g.step_fellback = false; g.step_why[0] = 0;
  if (pl.complete) {
    g.seg_waited.assign(pl.segs.size(), 0);
    g.step_mode = STEP_VERIFY;
    return AH_OK;
  }
  plan_destroy(pl);
  pl.segs.emplace_back();
  g.step_mode = STEP_RECORD;
  g.chunks_since_host_boundary = 0;
  int32_t rc = step_begin_capture();
  if (rc != AH_OK) { g.step_mode = STEP_OFF; g.plans.erase(key); g.plan = nullptr; }
  return rc;
}

int32_t ah_step_end(int32_t *out_how) {
  AH_REQUIRE_READY();
  if (g.step_mode == STEP_OFF) return fail(AH_ERR_STATE, "ah_step_end: no step is open");
  int32_t how = AH_STEP_EAGER, rc = AH_OK;
  if (g.step_mode == STEP_VERIFY && g.seg == 0 && g.op == 0 && g.slot == 0) {
    // nothing was issued since ah_step_begin (a bracket opened after the last step of a run): the plan stays as it is
  } else if (g.step_mode == STEP_RECORD && g.plan->segs.size() == 1 && g.plan->segs[0].ops.empty()) {
    if (g.step_capture_open) { hipGraph_t junk = nullptr; (void)hipStreamEndCapture(g.stream, &junk); if (junk) (void)hipGraphDestroy(junk); }
    plan_destroy(*g.plan);
    g.plans.erase(g.step_key);
  } else if (g.step_mode == STEP_RECORD) {
    rc = step_close_segment("ah_step_end");
    if (rc == AH_OK && !g.plan->broken) { g.plan->complete = true; how = AH_STEP_RECORDED; g.steps_recorded++; }
    else { (void)hipStreamSynchronize(g.stream); plan_destroy(*g.plan); g.plans.erase(g.step_key); }
  } else {
    if (g.step_mode == STEP_VERIFY) rc = step_boundary("ah_step_end");     // launches the last segment, or falls back
    if (g.step_fellback || rc != AH_OK) {
      how = AH_STEP_FELL_BACK; g.steps_fallback++;
      (void)hipStreamSynchronize(g.stream);
      plan_destroy(*g.plan);
      g.plans.erase(g.step_key);
    } else { how = AH_STEP_REPLAYED; g.steps_replayed++; }
  }
  g.step_mode = STEP_OFF; g.plan = nullptr; g.step_capture_open = false;
  if (out_how) *out_how = how;
  return rc;
}

int32_t ah_step_kick(void) {
  AH_REQUIRE_READY();
  if (g.step_mode != STEP_RECORD && g.step_mode != STEP_VERIFY) return AH_OK;
  int32_t rc = step_boundary("kick");
  if (rc != AH_OK) return rc;
  return step_resume();
}

int32_t ah_step_reset(uint64_t key) {
  AH_REQUIRE_READY();
  if (g.step_mode != STEP_OFF) return fail(AH_ERR_STATE, "ah_step_reset: illegal while a step is open");
  auto it = g.plans.find(key);
  if (it != g.plans.end()) { (void)hipStreamSynchronize(g.stream); plan_destroy(it->second); g.plans.erase(it); }
  return AH_OK;
}

const char *ah_step_note(void) { return g.step_why; }

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
  { int32_t rc = step_boundary("ah_event_record"); if (rc != AH_OK) return rc; }
  AH_HIP(hipEventRecord((hipEvent_t)(uintptr_t)event, g.stream));
  return step_resume();
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
