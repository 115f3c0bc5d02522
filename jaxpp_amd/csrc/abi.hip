// Error reporting and the device plumbing a host without a GPU runtime of its
// own needs (allocation, copies, streams, events).
#include <stdarg.h>
#include <stdio.h>

#include "common.h"

#include <string>
#include <utility>
#include <vector>

namespace {
thread_local char g_err[1024] = "";

struct Probe {
  bool active = false;
  std::string cls;
  std::vector<std::pair<hipEvent_t, hipEvent_t>> events;
  hipEvent_t open_ev = nullptr;
  double flops = 0, bytes = 0;
} g_probe;
}  // namespace

bool jpp_probe_wants(const char* kernel_class) {
  return g_probe.active && g_probe.cls == kernel_class;
}
void jpp_probe_open(hipStream_t stream) {
  hipEventCreate(&g_probe.open_ev);
  hipEventRecord(g_probe.open_ev, stream);
}
void jpp_probe_close(hipStream_t stream, double flops, double bytes) {
  hipEvent_t stop;
  hipEventCreate(&stop);
  hipEventRecord(stop, stream);
  g_probe.events.emplace_back(g_probe.open_ev, stop);
  g_probe.open_ev = nullptr;
  g_probe.flops += flops;
  g_probe.bytes += bytes;
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
  JPP_REQUIRE(!g_probe.active, "probe_begin: a probe is already active");
  g_probe.active = true;
  g_probe.cls = kernel_class;
  g_probe.flops = g_probe.bytes = 0;
  return JPP_OK;
}
int jpp_probe_end(int64_t* launches, double* total_ms, double* total_flops, double* total_bytes) {
  JPP_REQUIRE(g_probe.active, "probe_end: no active probe");
  g_probe.active = false;
  double ms = 0;
  hipError_t err = hipSuccess;
  for (auto& ev : g_probe.events) {
    float t = 0;
    hipError_t e = hipEventSynchronize(ev.second);
    if (e == hipSuccess) e = hipEventElapsedTime(&t, ev.first, ev.second);
    if (e != hipSuccess) err = e;
    ms += t;
    hipEventDestroy(ev.first);
    hipEventDestroy(ev.second);
  }
  if (launches) *launches = (int64_t)g_probe.events.size();
  if (total_ms) *total_ms = ms;
  if (total_flops) *total_flops = g_probe.flops;
  if (total_bytes) *total_bytes = g_probe.bytes;
  g_probe.events.clear();
  if (err != hipSuccess)
    return jpp_set_error(JPP_ERR_HIP, "probe_end: %s", hipGetErrorString(err));
  return JPP_OK;
}
int jpp_mem_info(size_t* free_bytes, size_t* total_bytes) {
  JPP_REQUIRE(free_bytes && total_bytes, "mem_info: null");
  JPP_CHECK_HIP(hipMemGetInfo(free_bytes, total_bytes));
  return JPP_OK;
}

}  // extern "C"
