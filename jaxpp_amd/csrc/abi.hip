// Error reporting and the device plumbing a host without a GPU runtime of its
// own needs (allocation, copies, streams, events).
#include <stdarg.h>
#include <stdio.h>

#include <algorithm>

#include "common.h"

#include <mutex>
#include <string>
#include <utility>
#include <vector>

namespace {
thread_local char g_err[1024] = "";

// The launch probe.  One probe at a time, shared by every host thread: all of its state sits
// behind `mu`, which a probed launch holds from the event in front of the kernel to the event
// behind it, so launches from several threads cannot interleave their brackets.  Events come
// from a pool of at most kProbeRing pairs: when every pair is in use the oldest one is waited
// for, read and reused, so the number of live events is bounded however long the probe stays
// open.  The first HIP error is kept and reported by jpp_probe_end; after it the probe stops
// recording (launches go on unbracketed).
constexpr size_t kProbeRing = 4096;

struct Probe {
  std::mutex mu;                 // guards every field below
  std::mutex launch_mu;          // held across one bracketed launch
  bool active = false;
  std::string cls;
  std::vector<std::pair<hipEvent_t, hipEvent_t>> ring;  // created on demand, reused
  std::vector<int> ring_class;   // class of the launch a pair brackets
  size_t head = 0, live = 0;     // oldest pair in flight, number in flight
  bool open = false;             // ring[(head + live) % size].first has been recorded
  int open_class = 0;
  // per class (one entry unless the probe was opened for every class, "*")
  struct Stat { std::string name; int64_t launches = 0; double ms = 0, flops = 0, bytes = 0; };
  std::vector<Stat> stats;
  int class_id(const char* name) {
    for (size_t i = 0; i < stats.size(); ++i)
      if (stats[i].name == name) return (int)i;
    stats.emplace_back();
    stats.back().name = name;
    return (int)stats.size() - 1;
  }
  hipError_t err = hipSuccess;
  char err_what[96] = "";

  void fail(hipError_t e, const char* what) {
    if (err == hipSuccess) {
      err = e;
      snprintf(err_what, sizeof(err_what), "%s", what);
    }
  }
  // waits for the oldest pair in flight and folds its duration into the total
  void retire_oldest() {
    auto& ev = ring[head];
    float t = 0;
    hipError_t e = hipEventSynchronize(ev.second);
    if (e == hipSuccess) e = hipEventElapsedTime(&t, ev.first, ev.second);
    if (e != hipSuccess) fail(e, "reading a launch's events");
    else stats[ring_class[head]].ms += t;
    head = (head + 1) % ring.size();
    --live;
  }
} g_probe;
}  // namespace

bool jpp_probe_wants(const char* kernel_class) {
  std::lock_guard<std::mutex> lock(g_probe.mu);
  return g_probe.active && g_probe.err == hipSuccess &&
         (g_probe.cls == "*" || g_probe.cls == kernel_class);
}

// A bracket opened inside another one on the same thread (a launcher that hands over to
// another launcher of the same class) is ignored: the outer bracket covers it, and locking
// launch_mu twice from one thread would never return.
thread_local int t_probe_depth = 0;

void jpp_probe_open(hipStream_t stream, const char* kernel_class) {
  if (t_probe_depth++ > 0) return;
  g_probe.launch_mu.lock();      // released by jpp_probe_close
  std::lock_guard<std::mutex> lock(g_probe.mu);
  Probe& p = g_probe;
  if (!p.active || p.err != hipSuccess) return;
  if (p.live == p.ring.size()) {
    if (p.ring.size() < kProbeRing) {
      // grow: only while the ring has not wrapped (head == 0), so order is kept
      hipEvent_t a = nullptr, b = nullptr;
      hipError_t e = hipEventCreate(&a);
      if (e == hipSuccess) e = hipEventCreate(&b);
      if (e != hipSuccess) {
        if (a) hipEventDestroy(a);
        p.fail(e, "hipEventCreate");
        return;
      }
      if (p.head != 0) {         // rotate so that the oldest pair is first again
        std::rotate(p.ring.begin(), p.ring.begin() + p.head, p.ring.end());
        std::rotate(p.ring_class.begin(), p.ring_class.begin() + p.head, p.ring_class.end());
        p.head = 0;
      }
      p.ring.emplace_back(a, b);
      p.ring_class.push_back(0);
    } else {
      p.retire_oldest();
    }
  }
  auto& ev = p.ring[(p.head + p.live) % p.ring.size()];
  const hipError_t e = hipEventRecord(ev.first, stream);
  if (e != hipSuccess) {
    p.fail(e, "hipEventRecord in front of a launch");
    return;
  }
  p.open = true;
  p.open_class = p.class_id(kernel_class);
}

void jpp_probe_close(hipStream_t stream, double flops, double bytes) {
  if (--t_probe_depth > 0) return;
  {
    std::lock_guard<std::mutex> lock(g_probe.mu);
    Probe& p = g_probe;
    if (p.open) {
      p.open = false;
      auto& ev = p.ring[(p.head + p.live) % p.ring.size()];
      const hipError_t e = hipEventRecord(ev.second, stream);
      if (e != hipSuccess) {
        p.fail(e, "hipEventRecord behind a launch");
      } else {
        p.ring_class[(p.head + p.live) % p.ring.size()] = p.open_class;
        ++p.live;
        Probe::Stat& st = p.stats[p.open_class];
        ++st.launches;
        st.flops += flops;
        st.bytes += bytes;
      }
    }
  }
  g_probe.launch_mu.unlock();
}

int jpp_set_error(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

extern "C" {

const char* jpp_last_error(void) { return g_err; }
int jpp_version(void) { return 100; }

int jpp_device_count(int* count) {
  JPP_REQUIRE(count, "device_count: null");
  hipError_t e = hipGetDeviceCount(count);
  if (e != hipSuccess) {
    *count = 0;
    return jpp_set_error(JPP_ERR_HIP, "hipGetDeviceCount: %s", hipGetErrorString(e));
  }
  return JPP_OK;
}
int jpp_set_device(int device) {
  JPP_CHECK_HIP(hipSetDevice(device));
  return JPP_OK;
}
int jpp_malloc(void** ptr, size_t bytes) {
  JPP_REQUIRE(ptr, "malloc: null");
  *ptr = nullptr;
  if (bytes == 0) return JPP_OK;
  JPP_CHECK_HIP(hipMalloc(ptr, bytes));
  return JPP_OK;
}
int jpp_free(void* ptr) {
  if (ptr) JPP_CHECK_HIP(hipFree(ptr));
  return JPP_OK;
}
int jpp_memcpy_h2d(void* dst, const void* src, size_t bytes) {
  if (bytes) JPP_CHECK_HIP(hipMemcpy(dst, src, bytes, hipMemcpyHostToDevice));
  return JPP_OK;
}
int jpp_memcpy_d2h(void* dst, const void* src, size_t bytes) {
  if (bytes) JPP_CHECK_HIP(hipMemcpy(dst, src, bytes, hipMemcpyDeviceToHost));
  return JPP_OK;
}
int jpp_memcpy_d2d_async(void* dst, const void* src, size_t bytes, void* stream) {
  if (bytes)
    JPP_CHECK_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, (hipStream_t)stream));
  return JPP_OK;
}
int jpp_stream_create(void** stream) {
  JPP_REQUIRE(stream, "stream_create: null");
  hipStream_t s;
  JPP_CHECK_HIP(hipStreamCreateWithFlags(&s, hipStreamNonBlocking));
  *stream = s;
  return JPP_OK;
}
int jpp_stream_destroy(void* stream) {
  if (stream) JPP_CHECK_HIP(hipStreamDestroy((hipStream_t)stream));
  return JPP_OK;
}
int jpp_stream_sync(void* stream) {
  JPP_CHECK_HIP(hipStreamSynchronize((hipStream_t)stream));
  return JPP_OK;
}
int jpp_device_sync(void) {
  JPP_CHECK_HIP(hipDeviceSynchronize());
  return JPP_OK;
}
int jpp_event_create(void** event) {
  JPP_REQUIRE(event, "event_create: null");
  hipEvent_t e;
  JPP_CHECK_HIP(hipEventCreate(&e));
  *event = e;
  return JPP_OK;
}
int jpp_event_destroy(void* event) {
  if (event) JPP_CHECK_HIP(hipEventDestroy((hipEvent_t)event));
  return JPP_OK;
}
int jpp_event_record(void* event, void* stream) {
  JPP_CHECK_HIP(hipEventRecord((hipEvent_t)event, (hipStream_t)stream));
  return JPP_OK;
}
int jpp_stream_wait_event(void* stream, void* event) {
  JPP_REQUIRE(event, "stream_wait_event: null event");
  JPP_CHECK_HIP(hipStreamWaitEvent((hipStream_t)stream, (hipEvent_t)event, 0));
  return JPP_OK;
}
// ---- HIP graphs: a recorded sequence of calls replayed without host launch work ----
int jpp_graph_begin(void* stream) {
  JPP_REQUIRE(stream, "graph_begin: capture needs a stream of its own, not the null stream");
  JPP_CHECK_HIP(hipStreamBeginCapture((hipStream_t)stream, hipStreamCaptureModeRelaxed));
  return JPP_OK;
}
int jpp_graph_end(void* stream, void** graph_exec) {
  JPP_REQUIRE(stream && graph_exec, "graph_end: null argument");
  hipGraph_t graph = nullptr;
  JPP_CHECK_HIP(hipStreamEndCapture((hipStream_t)stream, &graph));
  hipGraphExec_t exec = nullptr;
  const hipError_t err = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0);
  hipGraphDestroy(graph);
  if (err != hipSuccess)
    return jpp_set_error(JPP_ERR_HIP, "graph_end: instantiate: %s", hipGetErrorString(err));
  *graph_exec = exec;
  return JPP_OK;
}
int jpp_graph_launch(void* graph_exec, void* stream) {
  JPP_REQUIRE(graph_exec, "graph_launch: null graph");
  JPP_CHECK_HIP(hipGraphLaunch((hipGraphExec_t)graph_exec, (hipStream_t)stream));
  return JPP_OK;
}
int jpp_graph_destroy(void* graph_exec) {
  if (graph_exec) JPP_CHECK_HIP(hipGraphExecDestroy((hipGraphExec_t)graph_exec));
  return JPP_OK;
}
int jpp_event_sync(void* event) {
  JPP_CHECK_HIP(hipEventSynchronize((hipEvent_t)event));
  return JPP_OK;
}
int jpp_event_elapsed_ms(void* start, void* stop, float* ms) {
  JPP_REQUIRE(ms, "event_elapsed: null");
  JPP_CHECK_HIP(hipEventElapsedTime(ms, (hipEvent_t)start, (hipEvent_t)stop));
  return JPP_OK;
}
int jpp_probe_begin(const char* kernel_class) {
  JPP_REQUIRE(kernel_class && *kernel_class, "probe_begin: empty class name");
  std::lock_guard<std::mutex> lock(g_probe.mu);
  JPP_REQUIRE(!g_probe.active, "probe_begin: a probe is already active");
  g_probe.active = true;
  g_probe.cls = kernel_class;
  g_probe.head = g_probe.live = 0;
  g_probe.open = false;
  g_probe.stats.clear();
  g_probe.err = hipSuccess;
  g_probe.err_what[0] = 0;
  return JPP_OK;
}
int jpp_probe_end(int64_t* launches, double* total_ms, double* total_flops, double* total_bytes) {
  std::lock_guard<std::mutex> launch_lock(g_probe.launch_mu);  // no bracket half open
  std::lock_guard<std::mutex> lock(g_probe.mu);
  Probe& p = g_probe;
  JPP_REQUIRE(p.active, "probe_end: no active probe");
  p.active = false;
  while (p.live) p.retire_oldest();
  int64_t n = 0;
  double ms = 0, flops = 0, bytes = 0;
  for (auto& st : p.stats) { n += st.launches; ms += st.ms; flops += st.flops; bytes += st.bytes; }
  if (launches) *launches = n;
  if (total_ms) *total_ms = ms;
  if (total_flops) *total_flops = flops;
  if (total_bytes) *total_bytes = bytes;
  if (p.err != hipSuccess)
    return jpp_set_error(JPP_ERR_HIP, "probe: %s failed: %s (timings are incomplete)", p.err_what,
                         hipGetErrorString(p.err));
  return JPP_OK;
}
int jpp_probe_class(int index, const char** name, int64_t* launches, double* total_ms,
                    double* total_flops, double* total_bytes) {
  std::lock_guard<std::mutex> lock(g_probe.mu);
  Probe& p = g_probe;
  JPP_REQUIRE(!p.active, "probe_class: the probe is still open");
  if (index < 0 || index >= (int)p.stats.size())
    return jpp_set_error(JPP_ERR_INVALID, "probe_class: index %d of %d classes", index,
                         (int)p.stats.size());
  const Probe::Stat& st = p.stats[index];
  if (name) *name = st.name.c_str();
  if (launches) *launches = st.launches;
  if (total_ms) *total_ms = st.ms;
  if (total_flops) *total_flops = st.flops;
  if (total_bytes) *total_bytes = st.bytes;
  return JPP_OK;
}
size_t jpp_workspace_bytes(int op, int64_t d0, int64_t d1, int64_t d2) {
  if (d0 < 0 || d1 < 0 || d2 < 0) return 0;
  switch (op) {
    case JPP_WS_NORM_BWD: return (size_t)2 * JPP_NORM_PARTIALS * d0 * 4;
    case JPP_WS_COLSUM: return (size_t)JPP_NORM_PARTIALS * d0 * 4;
    case JPP_WS_ATTN_DELTA: return (size_t)2 * d0 * d1 * d2 * 4;
    case JPP_WS_MSE: return (size_t)JPP_NORM_PARTIALS * 4;
    case JPP_WS_MOE_WORK: return (size_t)2 * ((d0 + 255) / 256) * d1 * 4;
    case JPP_WS_MOE_ROUTER_WGRAD: return (size_t)64 * d0 * d1 * 4;
    case JPP_WS_SPLIT_WGRAD: return (size_t)d0 * d1 * d2 * 4;
    default: return 0;
  }
}
int jpp_mem_info(size_t* free_bytes, size_t* total_bytes) {
  JPP_REQUIRE(free_bytes && total_bytes, "mem_info: null");
  JPP_CHECK_HIP(hipMemGetInfo(free_bytes, total_bytes));
  return JPP_OK;
}

}  // extern "C"
