// Device, memory, stream and event plumbing of the C ABI, plus error state and options.
#include <stdarg.h>
#include <string.h>

#include <map>
#include <mutex>
#include <string>
#include <utility>
#include <vector>

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
      {"rowwise_variant", 0}, {"sdpa_variant", 0}, {"linear_variant", 0}, {"linear_small_m_max", 64}, {"linear_ntw", 0}, {"linear_split_k", 0}, {"linear_two_part", 0}, {"linear_decode_split", 0}, {"linear_decode_wide", 0}, {"linear_glu_main", 0}, {"linear_decode_variant", 0}, {"linear_two_pass", 0}, {"linear_img_variant", 0},
      {"check_extents", getenv("TTMLIR_AMD_CHECK_EXTENTS") && getenv("TTMLIR_AMD_CHECK_EXTENTS")[0] == '1' ? 1 : 0},
  };
  return m;
}
int ttm_option(const char *name) {
  std::lock_guard<std::mutex> g(g_opt_mu);
  auto it = opts().find(name);
  return it == opts().end() ? 0 : it->second;
}
// ---- operand extents
bool ttm_check_extents_on() { return ttm_option("check_extents") != 0; }
int TtmExtentChecker::operator()(const char *what, const void *p, int64_t bytes, bool optional) const {
  (void)optional;
  if (!p || bytes <= 0) return TTM_OK;   // a missing operand is the entry point's own argument check to report
  hipDeviceptr_t base = nullptr;
  size_t size = 0;
  if (hipMemGetAddressRange(&base, &size, (hipDeviceptr_t)p) != hipSuccess) {
    (void)hipGetLastError();   // the failed lookup must not be reported by the next HIP call
    return ttm_set_error(TTM_ERR_INVALID, "out of bounds: %s: %s (%p) is not device memory", fn, what, p);
  }
  const int64_t room = (int64_t)((const uint8_t *)base + size - (const uint8_t *)p);
  if (bytes > room)
    return ttm_set_error(TTM_ERR_INVALID,
                         "out of bounds: %s: %s has %lld bytes behind it in its allocation, the kernels touch %lld (a TILE tensor [batch, R, C] is "
                         "backed by batch * ceil(R / 32) * ceil(C / 32) whole tiles)",
                         fn, what, (long long)room, (long long)bytes);
  return TTM_OK;
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
namespace {
struct StreamWorkspace {
  void *ptr = nullptr;
  size_t bytes = 0;
  bool recorded = false;          // handed out while the stream was capturing
  std::vector<void *> retired;    // outgrown allocations that a graph may still name
};
std::mutex g_ws_mu;
std::map<std::pair<int, hipStream_t>, StreamWorkspace> g_ws;
}  // namespace

int ttm_stream_workspace(hipStream_t stream, size_t bytes, void **ptr) {
  int dev = 0;
  TTM_HIP(hipGetDevice(&dev));
  hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
  TTM_HIP(hipStreamIsCapturing(stream, &st));
  const bool capturing = st != hipStreamCaptureStatusNone;
  std::lock_guard<std::mutex> g(g_ws_mu);
  StreamWorkspace &w = g_ws[{dev, stream}];
  if (w.bytes < bytes) {
    if (capturing)
      return ttm_set_error(TTM_ERR_INVALID,
                           "a kernel needs %zu bytes of stream workspace while the stream is capturing: run the same work "
                           "once outside the capture first", bytes);
    if (w.ptr) {
      if (w.recorded) {
        w.retired.push_back(w.ptr);
      } else {
        TTM_HIP(hipStreamSynchronize(stream));
        TTM_HIP(hipFree(w.ptr));
      }
      w.ptr = nullptr; w.bytes = 0; w.recorded = false;
    }
    const size_t unit = (size_t)2 << 20;
    size_t want = (bytes + unit - 1) / unit * unit;
    TTM_HIP(hipMalloc(&w.ptr, want));
    w.bytes = want;
  }
  w.recorded |= capturing;
  *ptr = w.ptr;
  return TTM_OK;
}

TTM_EXPORT int ttm_stream_destroy(void *stream) {
  if (!stream) return TTM_OK;
  TTM_HIP(hipStreamSynchronize((hipStream_t)stream));
  {
    int dev = 0;
    TTM_HIP(hipGetDevice(&dev));
    std::lock_guard<std::mutex> g(g_ws_mu);
    auto it = g_ws.find({dev, (hipStream_t)stream});
    if (it != g_ws.end()) {
      if (it->second.ptr) (void)hipFree(it->second.ptr);
      for (void *q : it->second.retired) (void)hipFree(q);
      g_ws.erase(it);
    }
  }
  TTM_HIP(hipStreamDestroy((hipStream_t)stream));
  return TTM_OK;
}

// ---- HIP graphs: record the launches issued on a stream once, replay them with one launch
TTM_EXPORT int ttm_graph_begin_capture(void *stream) {
  TTM_REQUIRE(stream != nullptr, "ttm_graph_begin_capture: capture needs a stream of its own, not the null stream");
  // relaxed mode: allocation calls made by the capturing thread stay legal (they are not recorded)
  TTM_HIP(hipStreamBeginCapture((hipStream_t)stream, hipStreamCaptureModeRelaxed));
  return TTM_OK;
}
TTM_EXPORT int ttm_graph_end_capture(void *stream, void **graph_exec, size_t *num_nodes) {
  TTM_REQUIRE(stream && graph_exec, "ttm_graph_end_capture: null argument");
  *graph_exec = nullptr;
  hipGraph_t graph = nullptr;
  TTM_HIP(hipStreamEndCapture((hipStream_t)stream, &graph));
  TTM_REQUIRE(graph != nullptr, "ttm_graph_end_capture: the capture was invalidated");
  size_t n = 0;
  hipError_t e = hipGraphGetNodes(graph, nullptr, &n);
  if (e == hipSuccess && num_nodes) *num_nodes = n;
  hipGraphExec_t exec = nullptr;
  e = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0);
  (void)hipGraphDestroy(graph);
  if (e != hipSuccess) return ttm_set_error(TTM_ERR_HIP, "hipGraphInstantiate failed: %s", hipGetErrorString(e));
  *graph_exec = (void *)exec;
  return TTM_OK;
}
TTM_EXPORT int ttm_graph_launch(void *graph_exec, void *stream) {
  TTM_REQUIRE(graph_exec != nullptr, "ttm_graph_launch: null graph");
  TTM_HIP(hipGraphLaunch((hipGraphExec_t)graph_exec, (hipStream_t)stream));
  return TTM_OK;
}
TTM_EXPORT int ttm_graph_destroy(void *graph_exec) {
  if (graph_exec) TTM_HIP(hipGraphExecDestroy((hipGraphExec_t)graph_exec));
  return TTM_OK;
}
TTM_EXPORT int ttm_stream_is_capturing(void *stream, int *capturing) {
  TTM_REQUIRE(capturing != nullptr, "ttm_stream_is_capturing: null out pointer");
  hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
  TTM_HIP(hipStreamIsCapturing((hipStream_t)stream, &st));
  *capturing = st != hipStreamCaptureStatusNone;
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
