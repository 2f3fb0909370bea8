// Runtime of libwebdnn_hip.so: device selection, the single stream, the
// handle table, a size-bucketed device-memory pool, pinned staging for
// host<->device copies, and event timing.
//
// Stands in for the WASM worker's buffer-id protocol of the reference
// (src/descriptor_runner/backend/wasm/wasmContextImpl.ts:113-163,
//  src/shader/wasm/pre.js:4-91, src/shader/wasm/src/core/allocation.cpp:4-15).
#include <stdarg.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <map>
#include <string>
#include <utility>
#include <vector>

#include "common.h"

namespace {

constexpr size_t kStagingBytes = 32u << 20;  // per pinned buffer, two of them
// Uploads go through the staging buffers in pieces of kUploadPiece, each with an event of its
// own, so that the host's copy of piece i+1 into pinned memory overlaps the DMA of piece i.
constexpr size_t kUploadPiece = 4u << 20;
constexpr int kUploadSlots = (int)(2 * kStagingBytes / kUploadPiece);
constexpr size_t kSmallGranule = 512;        // allocation rounding below 1 MiB
constexpr size_t kLargeGranule = 1u << 20;   // and above

thread_local char g_error[512] = "";

struct Slot {
  void *ptr = nullptr;   // nullptr => slot is free
  size_t bytes = 0;      // bytes the caller asked for
  size_t cap = 0;        // bytes of the underlying block
  int arena = 0;         // > 0: the block belongs to the memory of captured graph arena-1
};

// A captured run (wdh_graph_begin .. wdh_graph_end).  The addresses of every
// buffer the run touched are baked into the graph, so the blocks allocated
// while capturing stay with the graph -- recycled among its own tensors, never
// handed to anybody else -- until the graph is destroyed.
struct GraphRec {
  hipGraph_t graph = nullptr;
  hipGraphExec_t exec = nullptr;
  std::multimap<size_t, void *> free_blocks;  // blocks of this graph not held by a handle
  bool live = false;
};

struct Runtime {
  bool ready = false;
  int device = -1;
  hipStream_t stream = nullptr;            // the current lane's stream: every call works on this one
  hipStream_t lanes[WDH_LANES] = {};       // lanes[0] is created by wdh_init, the others on first use
  int lane = 0;
  // lanes >= 1: work may have been enqueued since the lane was last waited for.  The pool hands blocks
  // from lane to lane, so whoever frees a block first waits for these lanes (settle_side_lanes).
  bool lane_dirty[WDH_LANES] = {};
  // A side branch of the run being recorded (wdh_branch_begin / _end / _join): work recorded between begin
  // and end goes to branch_stream and depends only on what was recorded before begin; the join makes what
  // follows depend on it.  0 = none, 1 = recording the branch, 2 = branch recorded, not joined yet.
  int branch = 0;
  hipStream_t branch_stream = nullptr, trunk_stream = nullptr;
  hipEvent_t branch_fork = nullptr, branch_done = nullptr;
  // blocks freed while a branch is open: nobody may take them before the join, because the two sides of
  // the fork are not ordered against each other
  struct FreedBlock { size_t cap; void *ptr; int arena; };
  std::vector<FreedBlock> branch_freed;
  hipDeviceProp_t prop;
  // handle table; handle = index + 1
  std::vector<Slot> slots;
  std::vector<int64_t> free_slots;
  // pool: capacity -> cached blocks
  std::multimap<size_t, void *> cache;
  uint64_t in_use = 0, cached = 0, reserved = 0, peak = 0;
  uint64_t limit = 0;  // "memory_limit_mib": the pool asks the driver for no more than this (0 = no limit)
  // pinned staging, ping-pong
  void *stage[2] = {nullptr, nullptr};
  hipEvent_t stage_done[2] = {nullptr, nullptr};   // downloads: one event per buffer
  hipEvent_t up_done[kUploadSlots] = {};            // uploads: one event per piece
  bool up_busy[kUploadSlots] = {};
  int up_next = 0;
  // timing events, created lazily
  hipEvent_t events[WDH_MAX_EVENTS] = {};
  // one-element dummy so that zero-byte buffers have a valid address
  void *dummy = nullptr;
  // captured graphs; `capturing` = index + 1 of the one being recorded, 0 = none
  std::vector<GraphRec> graphs;
  int capturing = 0;
  bool capture_failed = false;
};

Runtime g;

size_t round_up(size_t bytes) {
  if (bytes == 0) return kSmallGranule;
  size_t gran = bytes < (1u << 20) ? kSmallGranule : kLargeGranule;
  return (bytes + gran - 1) / gran * gran;
}

}  // namespace
namespace wdh {
void set_memory_limit(uint64_t bytes) { g.limit = bytes; }
}  // namespace wdh
namespace {

// Waits for the work of every lane (pool blocks and graph arenas may be referenced from any of them).
void drain_lanes() {
  for (hipStream_t s : g.lanes)
    if (s) (void)hipStreamSynchronize(s);
}

// Before a block goes back to the pool (where the next taker may sit on another lane): waits for the side
// lanes that have work in flight.  Lane 0 needs no wait: what is allocated on a side lane waits for it.
void settle_side_lanes() {
  if (g.capturing) return;  // (wdh_graph_begin has settled them, and the host has enqueued nothing since)
  for (int i = 1; i < WDH_LANES; i++)
    if (g.lanes[i] && g.lane_dirty[i]) {
      (void)hipStreamSynchronize(g.lanes[i]);
      g.lane_dirty[i] = false;
    }
}

void release_cache(size_t keep) {
  // Blocks may still be referenced by enqueued work: drain the streams first.
  if (g.cached <= keep) return;
  drain_lanes();
  for (auto it = g.cache.begin(); it != g.cache.end() && g.cached > keep;) {
    (void)hipFree(it->second);
    g.cached -= it->first;
    g.reserved -= it->first;
    it = g.cache.erase(it);
  }
}

// Returns the blocks of graph `id` that no handle holds to the general pool and
// hands the rest over to their handles.
void dissolve_graph(int id) {
  settle_side_lanes();  // (a replay of this graph may be in flight on one of them)
  GraphRec &r = g.graphs[id];
  if (r.exec) (void)hipGraphExecDestroy(r.exec);
  if (r.graph) (void)hipGraphDestroy(r.graph);
  for (auto &kv : r.free_blocks) {
    g.cache.emplace(kv.first, kv.second);
    g.cached += kv.first;
    g.in_use -= kv.first;
  }
  for (auto &s : g.slots)
    if (s.ptr && s.arena == id + 1) s.arena = 0;
  r = GraphRec();
}

}  // namespace

namespace wdh {

int fail(int code, const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
  return code;
}

void clear_error() { g_error[0] = '\0'; }
bool initialised() { return g.ready; }
bool capturing() { return g.capturing != 0; }
void poison_capture() { g.capture_failed = true; }
hipStream_t stream() { return g.stream; }
int lane() { return g.lane; }
bool branch_open() { return g.branch != 0; }
int compute_units() { return g.prop.multiProcessorCount; }
int device() { return g.device; }

void *resolve(wdh_buf h, size_t *bytes) {
  if (h <= 0 || (size_t)h > g.slots.size() || g.slots[h - 1].ptr == nullptr) {
    fail(WDH_EINVAL, "unknown buffer handle %lld", (long long)h);
    return nullptr;
  }
  const Slot &s = g.slots[h - 1];
  if (bytes) *bytes = s.bytes;
  return s.ptr;
}

bool operand(wdh_buf h, size_t need, const char *what, void **out) {
  size_t have = 0;
  void *p = resolve(h, &have);
  if (!p) {
    char prev[400];
    snprintf(prev, sizeof(prev), "%s", g_error);
    fail(WDH_EINVAL, "%s: %s", what, prev);
    return false;
  }
  if (have < need) {
    fail(WDH_EINVAL, "%s: buffer holds %zu bytes, operation needs %zu", what,
         have, need);
    return false;
  }
  *out = p;
  return true;
}

}  // namespace wdh

using wdh::fail;

extern "C" {

const char *wdh_last_error(void) { return g_error; }

// WDH_OPTIONS="name=value,name=value": wdh_set_option calls made on behalf of a caller that
// cannot make them itself (a model run through an unmodified host).  The whole string is
// checked before anything is applied or any device resource exists, so a bad item leaves the
// library uninitialised instead of half configured.
static int parse_env_options(std::vector<std::pair<std::string, int>> *out) {
  const char *env = getenv("WDH_OPTIONS");
  if (!env) return WDH_OK;
  if (strlen(env) > 511) return fail(WDH_EINVAL, "WDH_OPTIONS: longer than 511 characters");
  char buf[512];
  snprintf(buf, sizeof(buf), "%s", env);
  for (char *item = strtok(buf, ","); item; item = strtok(nullptr, ",")) {
    char *eq = strchr(item, '=');
    if (!eq || eq == item) return fail(WDH_EINVAL, "WDH_OPTIONS: \"%s\" is not name=value", item);
    *eq = '\0';
    char *end = nullptr;
    const long v = strtol(eq + 1, &end, 10);
    if (end == eq + 1 || *end != '\0' || v < -0x7fffffffL || v > 0x7fffffffL)
      return fail(WDH_EINVAL, "WDH_OPTIONS: value of \"%s\" is not an integer", item);
    out->emplace_back(item, (int)v);
  }
  return WDH_OK;
}

static void release_everything();

static int init_device(int device) {
  int count = 0;
  hipError_t e = hipGetDeviceCount(&count);
  if (e != hipSuccess || count <= 0) {
    (void)hipGetLastError();
    return fail(WDH_ENODEV, "wdh_init: no HIP device (%s)",
                e == hipSuccess ? "device count is 0" : hipGetErrorString(e));
  }
  if (device < 0 || device >= count)
    return fail(WDH_ENODEV, "wdh_init: device %d out of range (have %d)",
                device, count);
  WDH_HIP_CHECK(hipSetDevice(device));
  WDH_HIP_CHECK(hipGetDeviceProperties(&g.prop, device));
  if (strncmp(g.prop.gcnArchName, "gfx950", 6) != 0)
    return fail(WDH_ENODEV,
                "wdh_init: device %d is %s; this library holds gfx950 code only",
                device, g.prop.gcnArchName);
  WDH_HIP_CHECK(hipStreamCreateWithFlags(&g.lanes[0], hipStreamNonBlocking));
  g.stream = g.lanes[0];
  g.lane = 0;
  for (int i = 0; i < 2; i++) {
    if (hipHostMalloc(&g.stage[i], kStagingBytes, hipHostMallocDefault) !=
        hipSuccess)
      return fail(WDH_ENOMEM, "wdh_init: pinned staging allocation failed");
    WDH_HIP_CHECK(
        hipEventCreateWithFlags(&g.stage_done[i], hipEventDisableTiming));
  }
  for (int i = 0; i < kUploadSlots; i++) {
    WDH_HIP_CHECK(hipEventCreateWithFlags(&g.up_done[i], hipEventDisableTiming));
    g.up_busy[i] = false;
  }
  g.up_next = 0;
  WDH_HIP_CHECK(hipMalloc(&g.dummy, 256));
  int rc = wdh::init_static_scratch(device);
  if (rc == WDH_OK) rc = wdh::init_attention();
  if (rc == WDH_OK) rc = wdh::init_contraction(device);
  return rc;
}

int wdh_init(int device) {
  if (g.ready) {
    if (device == g.device) return WDH_OK;
    return fail(WDH_EINVAL, "wdh_init: already initialised on device %d",
                g.device);
  }
  // Options first: wdh_set_option checks names and ranges and touches plain variables only, so a
  // bad WDH_OPTIONS fails here, before any device resource exists.
  std::vector<std::pair<std::string, int>> options;
  if (int rc = parse_env_options(&options)) return rc;
  for (auto &kv : options)
    if (int rc = wdh_set_option(kv.first.c_str(), kv.second)) return rc;
  if (int rc = init_device(device)) {
    release_everything();  // whatever was created before the failing step (the error text stays)
    return rc;
  }
  g.device = device;
  g.ready = true;
  wdh::clear_error();
  return WDH_OK;
}

void wdh_shutdown(void) {
  if (!g.ready) return;
  release_everything();
}

// Releases whatever exists (also after a wdh_init that failed half way): every step copes with
// its resource missing.
static void release_everything() {
  if (g.capturing) {
    hipGraph_t dropped = nullptr;
    if (g.branch == 1) g.stream = g.trunk_stream;  // (the capture began on the trunk)
    (void)hipStreamEndCapture(g.stream, &dropped);
    if (dropped) (void)hipGraphDestroy(dropped);
    g.capturing = 0;
  }
  drain_lanes();
  for (size_t i = 0; i < g.graphs.size(); i++)
    if (g.graphs[i].live) dissolve_graph((int)i);
  g.graphs.clear();
  wdh::release_conv_tables();
  wdh::release_contraction();
  for (auto &s : g.slots)
    if (s.ptr && s.ptr != g.dummy) (void)hipFree(s.ptr);
  g.slots.clear();
  g.free_slots.clear();
  for (auto &kv : g.cache) (void)hipFree(kv.second);
  g.cache.clear();
  g.in_use = g.cached = g.reserved = g.peak = 0;
  for (int i = 0; i < 2; i++) {
    if (g.stage[i]) (void)hipHostFree(g.stage[i]);
    if (g.stage_done[i]) (void)hipEventDestroy(g.stage_done[i]);
    g.stage[i] = nullptr;
    g.stage_done[i] = nullptr;
  }
  for (int i = 0; i < kUploadSlots; i++) {
    if (g.up_done[i]) (void)hipEventDestroy(g.up_done[i]);
    g.up_done[i] = nullptr;
    g.up_busy[i] = false;
  }
  for (auto &ev : g.events) {
    if (ev) (void)hipEventDestroy(ev);
    ev = nullptr;
  }
  if (g.dummy) (void)hipFree(g.dummy);
  g.dummy = nullptr;
  for (hipStream_t &s : g.lanes) {
    if (s) (void)hipStreamDestroy(s);
    s = nullptr;
  }
  if (g.branch_stream) (void)hipStreamDestroy(g.branch_stream);
  if (g.branch_fork) (void)hipEventDestroy(g.branch_fork);
  if (g.branch_done) (void)hipEventDestroy(g.branch_done);
  g.branch_stream = nullptr;
  g.branch_fork = g.branch_done = nullptr;
  g.branch = 0;
  for (auto &b : g.branch_freed) (void)hipFree(b.ptr);  // (held by neither a handle nor the pool)
  g.branch_freed.clear();
  g.stream = nullptr;
  g.lane = 0;
  g.ready = false;
  g.device = -1;
}

int wdh_device_info(char *name, int name_cap, int *compute_units,
                    int *clock_mhz, uint64_t *hbm_bytes) {
  WDH_REQUIRE_INIT();
  if (name && name_cap > 0) snprintf(name, name_cap, "%s", g.prop.gcnArchName);
  if (compute_units) *compute_units = g.prop.multiProcessorCount;
  if (clock_mhz) *clock_mhz = g.prop.clockRate / 1000;
  if (hbm_bytes) *hbm_bytes = g.prop.totalGlobalMem;
  return WDH_OK;
}

wdh_buf wdh_alloc(size_t bytes) {
  if (!g.ready) {
    fail(WDH_ESTATE, "wdh_alloc: wdh_init() has not succeeded");
    return 0;
  }
  Slot s;
  s.bytes = bytes;
  if (bytes == 0) {
    s.ptr = g.dummy;
    s.cap = 0;
  } else {
    // a block taken on a side lane may have been freed by work still in flight on lane 0
    // (not while recording: wdh_graph_begin has waited, and the host has been on this lane since)
    if (g.lane != 0 && !g.capturing) (void)hipStreamSynchronize(g.lanes[0]);
    const size_t cap = round_up(bytes);
    const auto fits = [cap](size_t have) { return have <= cap + cap / 4; };
    s.arena = g.capturing;
    if (g.capturing) {
      // first choice: a block this graph already owns and no tensor holds any
      // more (such blocks stay counted as in use until the graph is destroyed)
      auto &mine = g.graphs[g.capturing - 1].free_blocks;
      auto mt = mine.lower_bound(cap);
      if (mt != mine.end() && fits(mt->first)) {
        s.ptr = mt->second;
        s.cap = mt->first;
        mine.erase(mt);
      }
    }
    if (!s.ptr) {
      auto it = g.cache.lower_bound(cap);
      if (it != g.cache.end() && fits(it->first)) {
        s.ptr = it->second;
        s.cap = it->first;
        g.cached -= s.cap;
        g.cache.erase(it);
      } else {
        void *p = nullptr;
        if (g.limit && g.reserved + cap > g.limit && !g.capturing) release_cache(0);
        if (g.limit && g.reserved + cap > g.limit) {
          fail(WDH_ENOMEM, "wdh_alloc: %zu bytes on top of %llu reserved exceed memory_limit_mib (%llu MiB)", cap,
               (unsigned long long)g.reserved, (unsigned long long)(g.limit >> 20));
          return 0;
        }
        hipError_t e = hipMalloc(&p, cap);
        if (e != hipSuccess && !g.capturing) {
          // give cached blocks back to the driver and retry once (this drains
          // the stream, which a capture would not survive)
          (void)hipGetLastError();
          release_cache(0);
          e = hipMalloc(&p, cap);
        }
        if (e != hipSuccess) {
          (void)hipGetLastError();
          fail(WDH_ENOMEM, "wdh_alloc: hipMalloc(%zu) failed: %s", cap,
               hipGetErrorString(e));
          return 0;
        }
        s.ptr = p;
        s.cap = cap;
        g.reserved += cap;
        if (g.reserved > g.peak) g.peak = g.reserved;
      }
      g.in_use += s.cap;
    }
  }
  int64_t idx;
  if (!g.free_slots.empty()) {
    idx = g.free_slots.back();
    g.free_slots.pop_back();
    g.slots[idx] = s;
  } else {
    idx = (int64_t)g.slots.size();
    g.slots.push_back(s);
  }
  return idx + 1;
}

// A block nobody holds any more: to the graph it belongs to, or to the pool.
static void give_back(size_t cap, void *ptr, int arena) {
  if (arena && g.graphs[arena - 1].live) {
    // memory of a captured graph: stays with it
    g.graphs[arena - 1].free_blocks.emplace(cap, ptr);
  } else {
    g.cache.emplace(cap, ptr);
    g.cached += cap;
    g.in_use -= cap;
  }
}

int wdh_free(wdh_buf h) {
  WDH_REQUIRE_INIT();
  if (h <= 0 || (size_t)h > g.slots.size() || g.slots[h - 1].ptr == nullptr)
    return fail(WDH_EINVAL, "wdh_free: unknown buffer handle %lld",
                (long long)h);
  wdh::conv_forget_weights(h);
  Slot &s = g.slots[h - 1];
  if (s.cap) {
    settle_side_lanes();
    if (g.branch && g.capturing)
      g.branch_freed.push_back({s.cap, s.ptr, s.arena});
    else
      give_back(s.cap, s.ptr, s.arena);
  }
  s = Slot();
  g.free_slots.push_back(h - 1);
  return WDH_OK;
}

// ---- captured runs ----------------------------------------------------------
#define WDH_NOT_WHILE_CAPTURING(what)                                             \
  do {                                                                            \
    if (g.capturing) {                                                            \
      g.capture_failed = true;                                                    \
      return fail(WDH_ESTATE, what ": not possible while a graph is being captured"); \
    }                                                                             \
  } while (0)

// Blocks until no upload piece is still on its way out of the staging buffers.
static int wait_for_uploads() {
  for (int i = 0; i < kUploadSlots; i++)
    if (g.up_busy[i]) {
      WDH_HIP_CHECK(hipEventSynchronize(g.up_done[i]));
      g.up_busy[i] = false;
    }
  return WDH_OK;
}

int wdh_graph_begin(void) {
  WDH_REQUIRE_INIT();
  if (g.capturing) return fail(WDH_ESTATE, "wdh_graph_begin: a capture is already open");
  if (int rc = wait_for_uploads()) return rc;
  // the blocks the capture takes from the pool, or gives back to it, may still be in use on another lane
  settle_side_lanes();
  if (g.lane != 0) WDH_HIP_CHECK(hipStreamSynchronize(g.lanes[0]));
  int id = -1;
  for (size_t i = 0; i < g.graphs.size(); i++)
    if (!g.graphs[i].live) id = (int)i;
  if (id < 0) {
    id = (int)g.graphs.size();
    g.graphs.emplace_back();
  }
  // relaxed: hipMalloc stays legal while capturing (a pool miss)
  WDH_HIP_CHECK(hipStreamBeginCapture(g.stream, hipStreamCaptureModeRelaxed));
  g.graphs[id] = GraphRec();
  g.graphs[id].live = true;
  g.capturing = id + 1;
  g.capture_failed = false;
  return WDH_OK;
}

// The blocks freed while the branch was open become available (to the graph being recorded, or to the pool).
static void branch_release_blocks() {
  for (auto &b : g.branch_freed) give_back(b.cap, b.ptr, b.arena);
  g.branch_freed.clear();
}

int wdh_branch_begin(void) {
  WDH_REQUIRE_INIT();
  if (!g.capturing) return WDH_OK;  // executing, not recording: one stream, the order of the calls
  if (g.branch) {
    g.capture_failed = true;
    return fail(WDH_ESTATE, "wdh_branch_begin: a branch is open already (one at a time)");
  }
  if (!g.branch_stream) {
    WDH_HIP_CHECK(hipStreamCreateWithFlags(&g.branch_stream, hipStreamNonBlocking));
    WDH_HIP_CHECK(hipEventCreateWithFlags(&g.branch_fork, hipEventDisableTiming));
    WDH_HIP_CHECK(hipEventCreateWithFlags(&g.branch_done, hipEventDisableTiming));
  }
  // the branch stream joins the capture behind everything recorded so far
  WDH_HIP_CHECK(hipEventRecord(g.branch_fork, g.stream));
  WDH_HIP_CHECK(hipStreamWaitEvent(g.branch_stream, g.branch_fork, 0));
  g.trunk_stream = g.stream;
  g.stream = g.branch_stream;
  g.branch = 1;
  return WDH_OK;
}

int wdh_branch_end(void) {
  WDH_REQUIRE_INIT();
  if (!g.capturing) return WDH_OK;
  if (g.branch != 1) {
    g.capture_failed = true;
    return fail(WDH_ESTATE, "wdh_branch_end: no branch is being recorded");
  }
  WDH_HIP_CHECK(hipEventRecord(g.branch_done, g.branch_stream));
  g.stream = g.trunk_stream;
  g.branch = 2;
  return WDH_OK;
}

int wdh_branch_join(void) {
  WDH_REQUIRE_INIT();
  if (!g.capturing) return WDH_OK;
  if (g.branch != 2) {
    g.capture_failed = true;
    return fail(WDH_ESTATE, "wdh_branch_join: no recorded branch to join (wdh_branch_begin, _end first)");
  }
  WDH_HIP_CHECK(hipStreamWaitEvent(g.stream, g.branch_done, 0));
  g.branch = 0;
  branch_release_blocks();
  return WDH_OK;
}

int wdh_graph_end(int *graph_id) {
  WDH_REQUIRE_INIT();
  if (!g.capturing) return fail(WDH_ESTATE, "wdh_graph_end: no capture is open");
  // a branch left open (a run that failed half way): close it, so that the capture can end
  if (g.branch == 1) {
    (void)hipEventRecord(g.branch_done, g.branch_stream);
    g.stream = g.trunk_stream;
    g.branch = 2;
  }
  if (g.branch == 2) {
    (void)hipStreamWaitEvent(g.stream, g.branch_done, 0);
    g.branch = 0;
  }
  branch_release_blocks();
  const int id = g.capturing - 1;
  g.capturing = 0;
  hipGraph_t graph = nullptr;
  hipError_t e = hipStreamEndCapture(g.stream, &graph);
  g.graphs[id].graph = graph;
  if (e == hipSuccess && graph && !g.capture_failed)
    e = hipGraphInstantiate(&g.graphs[id].exec, graph, nullptr, nullptr, 0);
  if (e != hipSuccess || !graph || g.capture_failed || !graph_id) {
    const bool poisoned = g.capture_failed;
    (void)hipGetLastError();
    dissolve_graph(id);
    if (!graph_id) return fail(WDH_EINVAL, "wdh_graph_end: graph_id is NULL");
    if (poisoned)
      return fail(WDH_ESTATE, "wdh_graph_end: the capture was abandoned: a call made while capturing cannot be recorded");
    return fail(WDH_EHIP, "wdh_graph_end: %s", e == hipSuccess ? "empty capture" : hipGetErrorString(e));
  }
  *graph_id = id;
  return WDH_OK;
}

int wdh_graph_launch(int graph_id) {
  WDH_REQUIRE_INIT();
  WDH_NOT_WHILE_CAPTURING("wdh_graph_launch");
  if (g.lane) g.lane_dirty[g.lane] = true;  // work is about to be enqueued on a side lane
  if (graph_id < 0 || (size_t)graph_id >= g.graphs.size() || !g.graphs[graph_id].live ||
      !g.graphs[graph_id].exec)
    return fail(WDH_EINVAL, "wdh_graph_launch: unknown graph %d", graph_id);
  WDH_HIP_CHECK(hipGraphLaunch(g.graphs[graph_id].exec, g.stream));
  return WDH_OK;
}

int wdh_graph_destroy(int graph_id) {
  WDH_REQUIRE_INIT();
  WDH_NOT_WHILE_CAPTURING("wdh_graph_destroy");
  if (graph_id < 0 || (size_t)graph_id >= g.graphs.size() || !g.graphs[graph_id].live)
    return fail(WDH_EINVAL, "wdh_graph_destroy: unknown graph %d", graph_id);
  dissolve_graph(graph_id);
  return WDH_OK;
}

int wdh_write(wdh_buf h, size_t dst_offset, const void *src, size_t bytes) {
  WDH_REQUIRE_INIT();
  WDH_NOT_WHILE_CAPTURING("wdh_write");
  if (g.lane) g.lane_dirty[g.lane] = true;  // work is about to be enqueued on a side lane
  size_t have = 0;
  char *dst = (char *)wdh::resolve(h, &have);
  if (!dst) return WDH_EINVAL;
  if (dst_offset > have || bytes > have - dst_offset)
    return fail(WDH_EINVAL, "wdh_write: %zu bytes at offset %zu exceed buffer of %zu",
                bytes, dst_offset, have);
  if (bytes && !src) return fail(WDH_EINVAL, "wdh_write: src is NULL");
  wdh::conv_forget_weights(h);
  const char *s = (const char *)src;
  size_t done = 0;
  while (done < bytes) {
    const size_t chunk = bytes - done < kUploadPiece ? bytes - done : kUploadPiece;
    const int slot = g.up_next;
    g.up_next = (g.up_next + 1) % kUploadSlots;
    if (g.up_busy[slot]) {
      WDH_HIP_CHECK(hipEventSynchronize(g.up_done[slot]));
      g.up_busy[slot] = false;
    }
    const size_t per_buffer = kStagingBytes / kUploadPiece;
    char *piece = (char *)g.stage[slot / per_buffer] + (slot % per_buffer) * kUploadPiece;
    memcpy(piece, s + done, chunk);
    WDH_HIP_CHECK(hipMemcpyAsync(dst + dst_offset + done, piece, chunk, hipMemcpyHostToDevice, g.stream));
    WDH_HIP_CHECK(hipEventRecord(g.up_done[slot], g.stream));
    g.up_busy[slot] = true;
    done += chunk;
  }
  return WDH_OK;
}

int wdh_read(wdh_buf h, size_t src_offset, void *dst, size_t bytes) {
  WDH_REQUIRE_INIT();
  WDH_NOT_WHILE_CAPTURING("wdh_read");
  if (g.lane) g.lane_dirty[g.lane] = true;  // work is about to be enqueued on a side lane
  size_t have = 0;
  const char *src = (const char *)wdh::resolve(h, &have);
  if (!src) return WDH_EINVAL;
  if (src_offset > have || bytes > have - src_offset)
    return fail(WDH_EINVAL, "wdh_read: %zu bytes at offset %zu exceed buffer of %zu",
                bytes, src_offset, have);
  if (bytes && !dst) return fail(WDH_EINVAL, "wdh_read: dst is NULL");
  // staging buffers may still carry an in-flight upload
  if (int rc = wait_for_uploads()) return rc;
  char *d = (char *)dst;
  size_t issued = 0, copied = 0;
  size_t chunk_of[2] = {0, 0};
  int which = 0;
  // ping-pong: the D2H of chunk i+1 overlaps the host memcpy of chunk i
  if (bytes) {
    chunk_of[0] = bytes < kStagingBytes ? bytes : kStagingBytes;
    WDH_HIP_CHECK(hipMemcpyAsync(g.stage[0], src + src_offset, chunk_of[0],
                                 hipMemcpyDeviceToHost, g.stream));
    WDH_HIP_CHECK(hipEventRecord(g.stage_done[0], g.stream));
    issued = chunk_of[0];
  } else {
    WDH_HIP_CHECK(hipStreamSynchronize(g.stream));
  }
  while (copied < bytes) {
    int next = which ^ 1;
    if (issued < bytes) {
      chunk_of[next] =
          bytes - issued < kStagingBytes ? bytes - issued : kStagingBytes;
      WDH_HIP_CHECK(hipMemcpyAsync(g.stage[next], src + src_offset + issued,
                                   chunk_of[next], hipMemcpyDeviceToHost,
                                   g.stream));
      WDH_HIP_CHECK(hipEventRecord(g.stage_done[next], g.stream));
      issued += chunk_of[next];
    }
    WDH_HIP_CHECK(hipEventSynchronize(g.stage_done[which]));
    memcpy(d + copied, g.stage[which], chunk_of[which]);
    copied += chunk_of[which];
    which = next;
  }
  g.lane_dirty[g.lane] = false;     // (the stream has drained up to the data just read)
  return wdh::contraction_check();
}

int wdh_copy(wdh_buf dst, size_t dst_offset, wdh_buf src, size_t src_offset,
             size_t bytes) {
  WDH_REQUIRE_INIT();
  size_t dhave = 0, shave = 0;
  char *d = (char *)wdh::resolve(dst, &dhave);
  if (!d) return WDH_EINVAL;
  const char *s = (const char *)wdh::resolve(src, &shave);
  if (!s) return WDH_EINVAL;
  if (dst_offset > dhave || bytes > dhave - dst_offset || src_offset > shave ||
      bytes > shave - src_offset)
    return fail(WDH_EINVAL, "wdh_copy: range exceeds a buffer");
  wdh::conv_forget_weights(dst);
  if (g.lane) {
    g.lane_dirty[g.lane] = true;
    // the source may be an upload still on its way on another lane (a tensor moved to the device just
    // before it is submitted): uploads are the one kind of cross-lane producer the library can see
    if (!g.capturing)
      if (int rc = wait_for_uploads()) return rc;
  }
  if (bytes)
    WDH_HIP_CHECK(hipMemcpyAsync(d + dst_offset, s + src_offset, bytes,
                                 hipMemcpyDeviceToDevice, g.stream));
  return WDH_OK;
}

int wdh_set_lane(int lane) {
  WDH_REQUIRE_INIT();
  WDH_NOT_WHILE_CAPTURING("wdh_set_lane");
  if (lane < 0 || lane >= WDH_LANES) return fail(WDH_EINVAL, "wdh_set_lane: lane %d (have 0..%d)", lane, WDH_LANES - 1);
  if (!g.lanes[lane]) {
    if (int rc = wdh::contraction_lane_init(lane)) return rc;
    WDH_HIP_CHECK(hipStreamCreateWithFlags(&g.lanes[lane], hipStreamNonBlocking));
  }
  g.lane = lane;
  g.stream = g.lanes[lane];
  if (lane) g.lane_dirty[lane] = true;
  return WDH_OK;
}

int wdh_sync(void) {
  WDH_REQUIRE_INIT();
  WDH_NOT_WHILE_CAPTURING("wdh_sync");
  WDH_HIP_CHECK(hipStreamSynchronize(g.stream));
  g.lane_dirty[g.lane] = false;
  return wdh::contraction_check();
}

int wdh_mem_stats(uint64_t *in_use, uint64_t *cached, uint64_t *peak) {
  WDH_REQUIRE_INIT();
  if (in_use) *in_use = g.in_use;
  if (cached) *cached = g.cached;
  if (peak) *peak = g.peak;
  return WDH_OK;
}

int wdh_trim(size_t keep_bytes) {
  WDH_REQUIRE_INIT();
  WDH_NOT_WHILE_CAPTURING("wdh_trim");
  release_cache(keep_bytes);
  return WDH_OK;
}

int wdh_event_record(int id) {
  WDH_REQUIRE_INIT();
  WDH_NOT_WHILE_CAPTURING("wdh_event_record");
  if (g.lane) g.lane_dirty[g.lane] = true;  // work is about to be enqueued on a side lane
  if (id < 0 || id >= WDH_MAX_EVENTS)
    return fail(WDH_EINVAL, "wdh_event_record: id %d out of range", id);
  if (!g.events[id]) WDH_HIP_CHECK(hipEventCreate(&g.events[id]));
  WDH_HIP_CHECK(hipEventRecord(g.events[id], g.stream));
  return WDH_OK;
}

int wdh_event_elapsed_ms(int start_id, int stop_id, float *ms) {
  WDH_REQUIRE_INIT();
  WDH_NOT_WHILE_CAPTURING("wdh_event_elapsed_ms");
  if (start_id < 0 || start_id >= WDH_MAX_EVENTS || stop_id < 0 ||
      stop_id >= WDH_MAX_EVENTS || !g.events[start_id] || !g.events[stop_id])
    return fail(WDH_EINVAL, "wdh_event_elapsed_ms: event not recorded");
  if (!ms) return fail(WDH_EINVAL, "wdh_event_elapsed_ms: ms is NULL");
  WDH_HIP_CHECK(hipEventSynchronize(g.events[stop_id]));
  WDH_HIP_CHECK(hipEventElapsedTime(ms, g.events[start_id], g.events[stop_id]));
  return WDH_OK;
}

}  // extern "C"
