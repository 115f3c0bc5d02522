// Error reporting and the device plumbing a host without a GPU runtime of its
// own needs (allocation, copies, streams, events).
#include <stdarg.h>
#include <stdio.h>

#include "common.h"

namespace {
thread_local char g_err[1024] = "";
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
int jpp_event_sync(void* event) {
  JPP_CHECK_HIP(hipEventSynchronize((hipEvent_t)event));
  return JPP_OK;
}
int jpp_event_elapsed_ms(void* start, void* stop, float* ms) {
  JPP_REQUIRE(ms, "event_elapsed: null");
  JPP_CHECK_HIP(hipEventElapsedTime(ms, (hipEvent_t)start, (hipEvent_t)stop));
  return JPP_OK;
}
int jpp_mem_info(size_t* free_bytes, size_t* total_bytes) {
  JPP_REQUIRE(free_bytes && total_bytes, "mem_info: null");
  JPP_CHECK_HIP(hipMemGetInfo(free_bytes, total_bytes));
  return JPP_OK;
}

}  // extern "C"
