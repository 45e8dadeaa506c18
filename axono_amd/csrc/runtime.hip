// Device runtime of libaxhip: caching allocator, current stream, hipGraph capture with an
// address-stable capture pool, events and copies.  Host code only (plus two tiny kernels that live
// in rowops.hip for fills and device-to-device copies).
//
// Memory model.  One MI355X holds 288 GB of HBM3E, so the allocator's default budget is half of
// the device (the KV cache and the weights are long-lived allocations; the cache only has to keep
// the step's temporaries from ever reaching hipMalloc again).  Sizes are rounded up to 256 bytes
// and kept in exact-size free lists; eviction is oldest-first.
#include <cstdio>
#include <cstring>
#include <deque>
#include <mutex>
#include <unordered_map>
#include <vector>

#include "common.hpp"

extern "C" int axhip_internal_copy(const void *src, void *dst, int64_t n, hipStream_t st);
extern "C" int axhip_internal_fill_zero(void *dst, int64_t n, hipStream_t st);

namespace axhip {
namespace {

constexpr size_t kGranule = 256;

struct Block {
  size_t size;      // rounded size
  int device;
  bool pool_owned;  // owned by the capture pool or by a graph: axhip_free leaves it alone
};

struct GraphExec {
  hipGraph_t graph = nullptr;
  hipGraphExec_t exec = nullptr;
  hipStream_t stream = nullptr;
  hipEvent_t ev_in = nullptr, ev_out = nullptr;
  std::vector<void *> blocks;  // capture-pool blocks the captured kernels write to
};

std::mutex g_mu;
std::unordered_map<void *, Block> g_live;
std::unordered_map<uint64_t, std::vector<void *>> g_free;  // key: device << 48 | size/granule
std::deque<std::pair<uint64_t, void *>> g_evict;            // oldest first; may hold stale entries
std::unordered_map<void *, uint64_t> g_cached;              // cached ptr -> key (validates g_evict)
size_t g_cached_bytes = 0, g_allocated_bytes = 0, g_budget = 0;
bool g_budget_set = false;

std::unordered_map<uint64_t, std::deque<void *>> g_pool;  // capture pool, FIFO per size
std::vector<void *> g_pool_unclaimed;                     // registered, not yet claimed by a capture

thread_local bool t_recording = false;
thread_local bool t_capturing = false;
thread_local hipStream_t t_capture_stream = nullptr;
thread_local std::vector<void *> t_capture_blocks;

inline size_t round_up(size_t b) { return (b + kGranule - 1) / kGranule * kGranule; }
inline uint64_t key_of(int dev, size_t rounded) {
  return (static_cast<uint64_t>(dev) << 48) | (rounded / kGranule);
}
inline size_t size_of_key(uint64_t key) { return (key & ((1ull << 48) - 1)) * kGranule; }

size_t budget_locked() {
  if (!g_budget_set) {
    size_t free_b = 0, total_b = 0;
    if (hipMemGetInfo(&free_b, &total_b) == hipSuccess && total_b > 0) {
      g_budget = total_b / 2;
      g_budget_set = true;
    } else {
      return size_t(2) << 30;
    }
  }
  return g_budget;
}

// Frees cached blocks, oldest first, until the cache fits `limit`.  Called with g_mu held.
void evict_locked(size_t limit) {
  while (g_cached_bytes > limit && !g_evict.empty()) {
    auto [key, ptr] = g_evict.front();
    g_evict.pop_front();
    auto it = g_cached.find(ptr);
    if (it == g_cached.end() || it->second != key) continue;  // stale: block was reused since
    g_cached.erase(it);
    auto &lst = g_free[key];
    for (size_t i = 0; i < lst.size(); ++i) {
      if (lst[i] == ptr) {
        lst[i] = lst.back();
        lst.pop_back();
        break;
      }
    }
    g_cached_bytes -= size_of_key(key);
    (void)hipFree(ptr);
  }
}

// The eviction queue is only consumed while the cache is over its budget, and a block that is reused
// leaves its entry behind: once stale entries outnumber the cached blocks the queue is rebuilt from its
// valid entries (the newest entry of every block that is cached now), oldest first as before.
void compact_evict_locked() {
  if (g_evict.size() <= 2 * g_cached.size() + 64) return;
  std::deque<std::pair<uint64_t, void *>> kept;
  std::unordered_map<void *, bool> seen;
  for (auto it = g_evict.rbegin(); it != g_evict.rend(); ++it) {
    auto c = g_cached.find(it->second);
    if (c == g_cached.end() || c->second != it->first || seen.count(it->second)) continue;
    seen[it->second] = true;
    kept.push_front(*it);
  }
  g_evict.swap(kept);
}

void cache_block_locked(void *ptr, const Block &b) {
  const uint64_t key = key_of(b.device, b.size);
  g_free[key].push_back(ptr);
  g_cached[ptr] = key;
  g_evict.emplace_back(key, ptr);
  compact_evict_locked();
  g_cached_bytes += b.size;
  evict_locked(budget_locked());
}

// Takes a cached block of exactly this size or asks the driver.  Called with g_mu held.
void *acquire_locked(int dev, size_t rounded) {
  const uint64_t key = key_of(dev, rounded);
  auto it = g_free.find(key);
  if (it != g_free.end() && !it->second.empty()) {
    void *p = it->second.back();
    it->second.pop_back();
    g_cached.erase(p);
    g_cached_bytes -= rounded;
    return p;
  }
  void *p = nullptr;
  if (hipMalloc(&p, rounded) != hipSuccess) {
    (void)hipGetLastError();
    evict_locked(0);  // give everything cached back to the driver and try once more
    if (hipMalloc(&p, rounded) != hipSuccess) {
      (void)hipGetLastError();
      return nullptr;
    }
  }
  return p;
}

hipStream_t current_stream() { return t_capturing ? t_capture_stream : nullptr; }
thread_local int t_ticket_lane = 0;
thread_local int t_plan_reuse = 0;

}  // namespace
}  // namespace axhip

using namespace axhip;

extern "C" {

AXHIP_API const char *axhip_version(void) { return "0.2.0-hip"; }

AXHIP_API int axhip_device_count(int *count) {
  if (!count) return AXHIP_INVALID_PTR;
  int n = 0;
  if (hipGetDeviceCount(&n) != hipSuccess) {
    (void)hipGetLastError();
    n = 0;
  }
  *count = n;
  return AXHIP_OK;
}

AXHIP_API int axhip_set_device(int device_id) {
  return hipSetDevice(device_id) == hipSuccess ? AXHIP_OK : AXHIP_DEVICE_ERROR;
}

AXHIP_API int axhip_device_info(int device_id, char *name, size_t name_len, int *is_gfx950,
                                size_t *total_bytes, int *compute_units) {
  hipDeviceProp_t prop;
  if (hipGetDeviceProperties(&prop, device_id) != hipSuccess) return AXHIP_DEVICE_ERROR;
  if (name && name_len > 0) {
    std::snprintf(name, name_len, "%s (%s)", prop.name, prop.gcnArchName);
  }
  if (is_gfx950) *is_gfx950 = std::strncmp(prop.gcnArchName, "gfx950", 6) == 0;
  if (total_bytes) *total_bytes = prop.totalGlobalMem;
  if (compute_units) *compute_units = prop.multiProcessorCount;
  return AXHIP_OK;
}

// ---- allocator ---------------------------------------------------------------------------------
AXHIP_API int axhip_alloc(size_t bytes, int zero, void **out) {
  if (!out) return AXHIP_INVALID_PTR;
  *out = nullptr;
  if (bytes == 0) return AXHIP_OK;
  const size_t rounded = round_up(bytes);
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return AXHIP_DEVICE_ERROR;
  void *p = nullptr;
  {
    std::lock_guard<std::mutex> lk(g_mu);
    const uint64_t key = key_of(dev, rounded);
    if (t_capturing) {
      // same-size request during capture: hand out the block the warm-up run registered, so the
      // captured kernels see the warm-up's addresses
      auto it = g_pool.find(key);
      if (it != g_pool.end() && !it->second.empty()) {
        p = it->second.front();
        it->second.pop_front();
        for (size_t i = 0; i < g_pool_unclaimed.size(); ++i) {
          if (g_pool_unclaimed[i] == p) {
            g_pool_unclaimed[i] = g_pool_unclaimed.back();
            g_pool_unclaimed.pop_back();
            break;
          }
        }
        t_capture_blocks.push_back(p);
      }
    }
    if (!p) {
      p = acquire_locked(dev, rounded);
      if (!p) return AXHIP_OUT_OF_MEMORY;
      Block b{rounded, dev, false};
      if (t_capturing) {  // not covered by the warm-up: the graph owns it from now on
        b.pool_owned = true;
        t_capture_blocks.push_back(p);
      } else if (t_recording) {
        b.pool_owned = true;
        g_pool[key].push_back(p);
        g_pool_unclaimed.push_back(p);
      }
      g_live[p] = b;
      g_allocated_bytes += rounded;
    }
  }
  if (zero) {
    const int rc = axhip_internal_fill_zero(p, static_cast<int64_t>(rounded), current_stream());
    if (rc != AXHIP_OK) return rc;
  }
  *out = p;
  return AXHIP_OK;
}

AXHIP_API int axhip_free(void *ptr) {
  if (!ptr) return AXHIP_OK;
  std::lock_guard<std::mutex> lk(g_mu);
  auto it = g_live.find(ptr);
  if (it == g_live.end()) return AXHIP_INVALID_PTR;
  if (it->second.pool_owned) return AXHIP_OK;  // released by the pool reset or the graph's destroy
  const Block b = it->second;
  g_live.erase(it);
  g_allocated_bytes -= b.size;
  cache_block_locked(ptr, b);
  return AXHIP_OK;
}

AXHIP_API int axhip_block_is_capture_owned(const void *ptr, int *owned) {
  if (!owned) return AXHIP_INVALID_PTR;
  std::lock_guard<std::mutex> lk(g_mu);
  auto it = g_live.find(const_cast<void *>(ptr));
  if (it == g_live.end()) return AXHIP_INVALID_PTR;
  *owned = it->second.pool_owned ? 1 : 0;
  return AXHIP_OK;
}

AXHIP_API size_t axhip_cached_bytes(void) {
  std::lock_guard<std::mutex> lk(g_mu);
  return g_cached_bytes;
}

AXHIP_API size_t axhip_allocated_bytes(void) {
  std::lock_guard<std::mutex> lk(g_mu);
  return g_allocated_bytes;
}

AXHIP_API int axhip_set_cache_budget(size_t bytes) {
  std::lock_guard<std::mutex> lk(g_mu);
  g_budget = bytes;
  g_budget_set = true;
  evict_locked(g_budget);
  return AXHIP_OK;
}

AXHIP_API size_t axhip_cache_budget(void) {
  std::lock_guard<std::mutex> lk(g_mu);
  return budget_locked();
}

AXHIP_API int axhip_reset_tickets(void) {
  if (t_capturing) return AXHIP_INVALID_ARGUMENT;
  int n = 0;
  if (hipGetDeviceCount(&n) != hipSuccess || n <= 0) {
    (void)hipGetLastError();
    return AXHIP_OK;  // no device: no counters
  }
  const int a = reset_attention_tickets(), b = reset_argmax_tickets();
  return a != AXHIP_OK ? a : b;
}

// Gives every cached block back to the driver.  The ticket counters are not touched: they return to zero
// at the end of every completed launch, and zeroing them here would race with a launch another thread has
// in flight (axhip_reset_tickets is the explicit call for the recovery case).
AXHIP_API int axhip_empty_cache(void) {
  std::lock_guard<std::mutex> lk(g_mu);
  evict_locked(0);
  return AXHIP_OK;
}

// ---- copies ------------------------------------------------------------------------------------
AXHIP_API int axhip_memcpy_h2d(void *dst, const void *src, size_t bytes) {
  if (bytes == 0) return AXHIP_OK;
  if (!dst || !src) return AXHIP_INVALID_PTR;
  if (t_capturing) return AXHIP_INVALID_ARGUMENT;
  return hipMemcpy(dst, src, bytes, hipMemcpyHostToDevice) == hipSuccess ? AXHIP_OK
                                                                         : AXHIP_DEVICE_ERROR;
}

AXHIP_API int axhip_memcpy_d2h(void *dst, const void *src, size_t bytes) {
  if (bytes == 0) return AXHIP_OK;
  if (!dst || !src) return AXHIP_INVALID_PTR;
  if (t_capturing) return AXHIP_INVALID_ARGUMENT;
  return hipMemcpy(dst, src, bytes, hipMemcpyDeviceToHost) == hipSuccess ? AXHIP_OK
                                                                         : AXHIP_DEVICE_ERROR;
}

AXHIP_API int axhip_memcpy_d2d(void *dst, const void *src, size_t bytes) {
  if (bytes == 0) return AXHIP_OK;
  if (!dst || !src) return AXHIP_INVALID_PTR;
  return axhip_internal_copy(src, dst, static_cast<int64_t>(bytes), current_stream());
}

AXHIP_API int axhip_fill_zero(void *dst, size_t bytes) {
  if (bytes == 0) return AXHIP_OK;
  if (!dst) return AXHIP_INVALID_PTR;
  return axhip_internal_fill_zero(dst, static_cast<int64_t>(bytes), current_stream());
}

// ---- stream / capture state ----------------------------------------------------------------------
AXHIP_API axhip_stream axhip_current_stream(void) { return current_stream(); }

AXHIP_API int axhip_set_ticket_lane(int lane) {
  if (lane < 0 || lane >= AXHIP_TICKET_LANES) return AXHIP_INVALID_ARGUMENT;
  t_ticket_lane = lane;
  return AXHIP_OK;
}
AXHIP_API int axhip_ticket_lane(void) { return t_ticket_lane; }
AXHIP_API int axhip_set_plan_reuse(int mode) {
  if (mode < 0 || mode > 2) return AXHIP_INVALID_ARGUMENT;
  t_plan_reuse = mode;
  return AXHIP_OK;
}
AXHIP_API int axhip_plan_reuse(void) { return t_plan_reuse; }
AXHIP_API int axhip_is_capturing(void) { return t_capturing ? 1 : 0; }

AXHIP_API int axhip_synchronize(void) {
  if (t_capturing) return AXHIP_INVALID_ARGUMENT;
  return hipDeviceSynchronize() == hipSuccess ? AXHIP_OK : AXHIP_DEVICE_ERROR;
}

AXHIP_API int axhip_capture_pool_set_recording(int on) {
  t_recording = on != 0;
  return AXHIP_OK;
}

AXHIP_API int axhip_capture_pool_reset(void) {
  // blocks registered by a warm-up that no capture claimed go back to the allocator's cache
  std::lock_guard<std::mutex> lk(g_mu);
  for (void *p : g_pool_unclaimed) {
    auto it = g_live.find(p);
    if (it == g_live.end()) continue;
    const Block b{it->second.size, it->second.device, false};
    g_live.erase(it);
    g_allocated_bytes -= b.size;
    cache_block_locked(p, b);
  }
  g_pool_unclaimed.clear();
  g_pool.clear();
  return AXHIP_OK;
}

AXHIP_API int axhip_graph_begin_capture(axhip_stream *stream_out) {
  if (!stream_out) return AXHIP_INVALID_PTR;
  if (t_capturing) return AXHIP_INVALID_ARGUMENT;
  (void)hipGetLastError();  // a stale error must not poison the capture
  hipStream_t st = nullptr;
  if (hipStreamCreateWithFlags(&st, hipStreamNonBlocking) != hipSuccess) return AXHIP_DEVICE_ERROR;
  // work issued earlier on the default stream (weights, inputs) must be visible to the graph's
  // stream; waiting here keeps the capture itself free of cross-stream edges
  if (hipDeviceSynchronize() != hipSuccess) {
    (void)hipStreamDestroy(st);
    return AXHIP_DEVICE_ERROR;
  }
  if (hipStreamBeginCapture(st, hipStreamCaptureModeRelaxed) != hipSuccess) {
    (void)hipGetLastError();
    (void)hipStreamDestroy(st);
    return AXHIP_DEVICE_ERROR;
  }
  t_capturing = true;
  t_capture_stream = st;
  t_capture_blocks.clear();
  *stream_out = st;
  return AXHIP_OK;
}

namespace {
void release_graph_blocks(std::vector<void *> &blocks) {
  std::lock_guard<std::mutex> lk(g_mu);
  for (void *p : blocks) {
    auto it = g_live.find(p);
    if (it == g_live.end()) continue;
    const Block b{it->second.size, it->second.device, false};
    g_live.erase(it);
    g_allocated_bytes -= b.size;
    cache_block_locked(p, b);
  }
  blocks.clear();
}
}  // namespace

AXHIP_API int axhip_graph_abort_capture(axhip_stream stream) {
  hipStream_t st = as_stream(stream);
  if (!t_capturing || st != t_capture_stream) return AXHIP_INVALID_ARGUMENT;
  hipGraph_t g = nullptr;
  (void)hipStreamEndCapture(st, &g);
  if (g) (void)hipGraphDestroy(g);
  (void)hipGetLastError();
  t_capturing = false;
  t_capture_stream = nullptr;
  release_graph_blocks(t_capture_blocks);
  (void)hipStreamDestroy(st);
  return AXHIP_OK;
}

AXHIP_API int axhip_graph_end_capture(axhip_stream stream, axhip_graph *graph_out,
                                      size_t *num_nodes_out) {
  hipStream_t st = as_stream(stream);
  if (!graph_out) return AXHIP_INVALID_PTR;
  if (!t_capturing || st != t_capture_stream) return AXHIP_INVALID_ARGUMENT;
  hipGraph_t g = nullptr;
  const hipError_t e = hipStreamEndCapture(st, &g);
  t_capturing = false;
  t_capture_stream = nullptr;
  auto fail = [&](int code) {
    if (g) (void)hipGraphDestroy(g);
    (void)hipGetLastError();
    release_graph_blocks(t_capture_blocks);
    (void)hipStreamDestroy(st);
    return code;
  };
  if (e != hipSuccess || !g) return fail(AXHIP_DEVICE_ERROR);
  size_t n = 0;
  if (hipGraphGetNodes(g, nullptr, &n) != hipSuccess) return fail(AXHIP_DEVICE_ERROR);
  if (n == 0) return fail(AXHIP_INVALID_ARGUMENT);  // nothing was captured
  GraphExec *ge = new GraphExec();
  if (hipGraphInstantiate(&ge->exec, g, nullptr, nullptr, 0) != hipSuccess) {
    delete ge;
    return fail(AXHIP_DEVICE_ERROR);
  }
  ge->graph = g;
  ge->stream = st;
  ge->blocks.swap(t_capture_blocks);
  if (hipEventCreateWithFlags(&ge->ev_in, hipEventDisableTiming) != hipSuccess ||
      hipEventCreateWithFlags(&ge->ev_out, hipEventDisableTiming) != hipSuccess) {
    (void)hipGraphExecDestroy(ge->exec);
    t_capture_blocks.swap(ge->blocks);
    delete ge;
    return fail(AXHIP_DEVICE_ERROR);
  }
  *graph_out = ge;
  if (num_nodes_out) *num_nodes_out = n;
  return AXHIP_OK;
}

AXHIP_API int axhip_graph_launch(axhip_graph graph) {
  GraphExec *ge = static_cast<GraphExec *>(graph);
  if (!ge || !ge->exec) return AXHIP_INVALID_ARGUMENT;
  if (t_capturing) return AXHIP_INVALID_ARGUMENT;
  (void)hipGetLastError();
  // order the replay after earlier default-stream work (input refreshes) and later default-stream
  // work after the replay; the graph's own stream is non-blocking
  if (hipEventRecord(ge->ev_in, nullptr) != hipSuccess) return AXHIP_DEVICE_ERROR;
  if (hipStreamWaitEvent(ge->stream, ge->ev_in, 0) != hipSuccess) return AXHIP_DEVICE_ERROR;
  if (hipGraphLaunch(ge->exec, ge->stream) != hipSuccess) return AXHIP_DEVICE_ERROR;
  if (hipEventRecord(ge->ev_out, ge->stream) != hipSuccess) return AXHIP_DEVICE_ERROR;
  if (hipStreamWaitEvent(nullptr, ge->ev_out, 0) != hipSuccess) return AXHIP_DEVICE_ERROR;
  return AXHIP_OK;
}

AXHIP_API int axhip_graph_launch_async(axhip_graph graph) {
  GraphExec *ge = static_cast<GraphExec *>(graph);
  if (!ge || !ge->exec) return AXHIP_INVALID_ARGUMENT;
  if (t_capturing) return AXHIP_INVALID_ARGUMENT;
  (void)hipGetLastError();
  // on the graph's own stream only: no edge to or from the default stream, so replays of different
  // graphs run side by side; replays of one graph keep their order
  return hipGraphLaunch(ge->exec, ge->stream) == hipSuccess ? AXHIP_OK : AXHIP_DEVICE_ERROR;
}

AXHIP_API int axhip_graph_replay(axhip_graph graph) {
  GraphExec *ge = static_cast<GraphExec *>(graph);
  if (!ge || !ge->exec) return AXHIP_INVALID_ARGUMENT;
  if (t_capturing) return AXHIP_INVALID_ARGUMENT;
  (void)hipGetLastError();
  // earlier default-stream work (input refreshes) is waited for on the host, then the graph runs on its
  // own stream and is waited for: the same order as axhip_graph_launch + axhip_graph_sync without the two
  // event edges between the streams (measured 0.2 ms per replay of a 200-node graph)
  if (hipStreamSynchronize(nullptr) != hipSuccess) return AXHIP_DEVICE_ERROR;
  if (hipGraphLaunch(ge->exec, ge->stream) != hipSuccess) return AXHIP_DEVICE_ERROR;
  return hipStreamSynchronize(ge->stream) == hipSuccess ? AXHIP_OK : AXHIP_DEVICE_ERROR;
}

AXHIP_API int axhip_graph_sync(axhip_graph graph) {
  GraphExec *ge = static_cast<GraphExec *>(graph);
  if (!ge || !ge->stream) return AXHIP_INVALID_ARGUMENT;
  return hipStreamSynchronize(ge->stream) == hipSuccess ? AXHIP_OK : AXHIP_DEVICE_ERROR;
}

AXHIP_API int axhip_graph_destroy(axhip_graph graph) {
  GraphExec *ge = static_cast<GraphExec *>(graph);
  if (!ge) return AXHIP_OK;
  if (ge->stream) (void)hipStreamSynchronize(ge->stream);
  if (ge->exec) (void)hipGraphExecDestroy(ge->exec);
  if (ge->graph) (void)hipGraphDestroy(ge->graph);
  if (ge->ev_in) (void)hipEventDestroy(ge->ev_in);
  if (ge->ev_out) (void)hipEventDestroy(ge->ev_out);
  if (ge->stream) (void)hipStreamDestroy(ge->stream);
  release_graph_blocks(ge->blocks);
  delete ge;
  return AXHIP_OK;
}

// ---- events ------------------------------------------------------------------------------------
AXHIP_API int axhip_event_create(axhip_event *out) {
  if (!out) return AXHIP_INVALID_PTR;
  hipEvent_t ev = nullptr;
  if (hipEventCreate(&ev) != hipSuccess) return AXHIP_DEVICE_ERROR;
  *out = ev;
  return AXHIP_OK;
}

AXHIP_API int axhip_event_record(axhip_event ev, axhip_stream stream) {
  if (!ev) return AXHIP_INVALID_PTR;
  return hipEventRecord(static_cast<hipEvent_t>(ev), as_stream(stream)) == hipSuccess
             ? AXHIP_OK
             : AXHIP_DEVICE_ERROR;
}

AXHIP_API int axhip_event_elapsed_ms(axhip_event start, axhip_event stop, float *ms_out) {
  if (!start || !stop || !ms_out) return AXHIP_INVALID_PTR;
  if (hipEventSynchronize(static_cast<hipEvent_t>(stop)) != hipSuccess) return AXHIP_DEVICE_ERROR;
  return hipEventElapsedTime(ms_out, static_cast<hipEvent_t>(start),
                             static_cast<hipEvent_t>(stop)) == hipSuccess
             ? AXHIP_OK
             : AXHIP_DEVICE_ERROR;
}

AXHIP_API int axhip_event_destroy(axhip_event ev) {
  if (!ev) return AXHIP_OK;
  return hipEventDestroy(static_cast<hipEvent_t>(ev)) == hipSuccess ? AXHIP_OK : AXHIP_DEVICE_ERROR;
}

}  // extern "C"
