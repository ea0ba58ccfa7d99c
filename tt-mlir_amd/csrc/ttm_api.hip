// Device, memory, stream and event plumbing of the C ABI, plus error state and options.
#include <stdarg.h>
#include <string.h>

#include <map>
#include <mutex>
#include <string>

#include "ttm_common.h"

static thread_local char g_err[512] = "";

int ttm_set_error(int code, const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

TTM_EXPORT const char *ttm_last_error(void) { return g_err; }

// ---- options
static std::mutex g_opt_mu;
static std::map<std::string, int> &opts() {
  static std::map<std::string, int> m = {
      {"tilize_variant", 0}, {"untilize_variant", 0}, {"pack_variant", 0}, {"unpack_variant", 0},
      {"linear_variant", 0}, {"linear_small_m_max", 64}, {"linear_ntw", 0}, {"linear_split_k", 0},
  };
  return m;
}
int ttm_option(const char *name) {
  std::lock_guard<std::mutex> g(g_opt_mu);
  auto it = opts().find(name);
  return it == opts().end() ? 0 : it->second;
}
TTM_EXPORT int ttm_set_option(const char *name, int value) {
  TTM_REQUIRE(name != nullptr, "ttm_set_option: null name");
  std::lock_guard<std::mutex> g(g_opt_mu);
  auto it = opts().find(name);
  if (it == opts().end()) return ttm_set_error(TTM_ERR_INVALID, "ttm_set_option: unknown option '%s'", name);
  it->second = value;
  return TTM_OK;
}
TTM_EXPORT int ttm_get_option(const char *name, int *value) {
  TTM_REQUIRE(name != nullptr && value != nullptr, "ttm_get_option: null argument");
  std::lock_guard<std::mutex> g(g_opt_mu);
  auto it = opts().find(name);
  if (it == opts().end()) return ttm_set_error(TTM_ERR_INVALID, "ttm_get_option: unknown option '%s'", name);
  *value = it->second;
  return TTM_OK;
}

// ---- device / memory
TTM_EXPORT int ttm_device_count(int *count) {
  TTM_REQUIRE(count != nullptr, "ttm_device_count: null argument");
  hipError_t e = hipGetDeviceCount(count);
  if (e != hipSuccess) {
    *count = 0;
    (void)hipGetLastError();
    return ttm_set_error(TTM_ERR_HIP, "hipGetDeviceCount: %s", hipGetErrorString(e));
  }
  return TTM_OK;
}
TTM_EXPORT int ttm_set_device(int device) {
  TTM_HIP(hipSetDevice(device));
  return TTM_OK;
}
TTM_EXPORT int ttm_device_name(char *buf, size_t len) {
  TTM_REQUIRE(buf != nullptr && len > 0, "ttm_device_name: bad buffer");
  int dev = 0;
  TTM_HIP(hipGetDevice(&dev));
  hipDeviceProp_t p;
  TTM_HIP(hipGetDeviceProperties(&p, dev));
  snprintf(buf, len, "%s (%s, %d CUs)", p.name, p.gcnArchName, p.multiProcessorCount);
  return TTM_OK;
}
TTM_EXPORT int ttm_mem_info(size_t *free_bytes, size_t *total_bytes) {
  TTM_REQUIRE(free_bytes && total_bytes, "ttm_mem_info: null argument");
  TTM_HIP(hipMemGetInfo(free_bytes, total_bytes));
  return TTM_OK;
}
TTM_EXPORT int ttm_malloc(void **dptr, size_t bytes) {
  TTM_REQUIRE(dptr != nullptr, "ttm_malloc: null out pointer");
  *dptr = nullptr;
  if (bytes == 0) return TTM_OK;
  TTM_HIP(hipMalloc(dptr, bytes));
  return TTM_OK;
}
TTM_EXPORT int ttm_free(void *dptr) {
  if (dptr) TTM_HIP(hipFree(dptr));
  return TTM_OK;
}
TTM_EXPORT int ttm_host_alloc(void **hptr, size_t bytes) {
  TTM_REQUIRE(hptr != nullptr, "ttm_host_alloc: null out pointer");
  *hptr = nullptr;
  if (bytes == 0) return TTM_OK;
  TTM_HIP(hipHostMalloc(hptr, bytes, hipHostMallocDefault));
  return TTM_OK;
}
TTM_EXPORT int ttm_host_free(void *hptr) {
  if (hptr) TTM_HIP(hipHostFree(hptr));
  return TTM_OK;
}
TTM_EXPORT int ttm_memcpy_h2d(void *dst, const void *src, size_t bytes, void *stream) {
  if (bytes == 0) return TTM_OK;
  TTM_REQUIRE(dst && src, "ttm_memcpy_h2d: null pointer");
  TTM_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, (hipStream_t)stream));
  return TTM_OK;
}
TTM_EXPORT int ttm_memcpy_d2h(void *dst, const void *src, size_t bytes, void *stream) {
  if (bytes == 0) return TTM_OK;
  TTM_REQUIRE(dst && src, "ttm_memcpy_d2h: null pointer");
  TTM_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, (hipStream_t)stream));
  return TTM_OK;
}
TTM_EXPORT int ttm_memcpy_d2d(void *dst, const void *src, size_t bytes, void *stream) {
  if (bytes == 0) return TTM_OK;
  TTM_REQUIRE(dst && src, "ttm_memcpy_d2d: null pointer");
  TTM_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, (hipStream_t)stream));
  return TTM_OK;
}

__global__ void ttm_fill_u32_kernel(uint32_t *dst, uint32_t v, size_t n) {
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  size_t stride = (size_t)gridDim.x * blockDim.x;
  for (; i < n; i += stride) dst[i] = v;
}
TTM_EXPORT int ttm_fill_u32(void *dst, uint32_t value, size_t count, void *stream) {
  if (count == 0) return TTM_OK;
  TTM_REQUIRE(dst != nullptr, "ttm_fill_u32: null pointer");
  TTM_REQUIRE(((uintptr_t)dst & 3) == 0, "ttm_fill_u32: dst not 4-byte aligned");
  size_t blocks = (count + 255) / 256;
  if (blocks > 65536) blocks = 65536;
  hipLaunchKernelGGL(ttm_fill_u32_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream,
                     (uint32_t *)dst, value, count);
  TTM_LAUNCH_CHECK();
  return TTM_OK;
}

// ---- streams / events (default priority only)
TTM_EXPORT int ttm_stream_create(void **stream) {
  TTM_REQUIRE(stream != nullptr, "ttm_stream_create: null out pointer");
  hipStream_t s;
  TTM_HIP(hipStreamCreateWithFlags(&s, hipStreamNonBlocking));
  *stream = (void *)s;
  return TTM_OK;
}
TTM_EXPORT int ttm_stream_destroy(void *stream) {
  if (stream) TTM_HIP(hipStreamDestroy((hipStream_t)stream));
  return TTM_OK;
}
TTM_EXPORT int ttm_stream_sync(void *stream) {
  TTM_HIP(hipStreamSynchronize((hipStream_t)stream));
  return TTM_OK;
}
TTM_EXPORT int ttm_device_sync(void) {
  TTM_HIP(hipDeviceSynchronize());
  return TTM_OK;
}
TTM_EXPORT int ttm_event_create(void **event) {
  TTM_REQUIRE(event != nullptr, "ttm_event_create: null out pointer");
  hipEvent_t e;
  TTM_HIP(hipEventCreate(&e));
  *event = (void *)e;
  return TTM_OK;
}
TTM_EXPORT int ttm_event_destroy(void *event) {
  if (event) TTM_HIP(hipEventDestroy((hipEvent_t)event));
  return TTM_OK;
}
TTM_EXPORT int ttm_event_record(void *event, void *stream) {
  TTM_REQUIRE(event != nullptr, "ttm_event_record: null event");
  TTM_HIP(hipEventRecord((hipEvent_t)event, (hipStream_t)stream));
  return TTM_OK;
}
TTM_EXPORT int ttm_event_sync(void *event) {
  TTM_REQUIRE(event != nullptr, "ttm_event_sync: null event");
  TTM_HIP(hipEventSynchronize((hipEvent_t)event));
  return TTM_OK;
}
TTM_EXPORT int ttm_event_elapsed_ms(float *ms, void *start, void *stop) {
  TTM_REQUIRE(ms && start && stop, "ttm_event_elapsed_ms: null argument");
  TTM_HIP(hipEventElapsedTime(ms, (hipEvent_t)start, (hipEvent_t)stop));
  return TTM_OK;
}
