// A device in host memory that checks everything and computes on the host: a stand-in for libttmlir_amd_hip.so on a
// machine without a GPU, built by the tests (g++ -shared, linked against the CPU oracle) and put in front of the real library
// with LD_LIBRARY_PATH.  "Device memory" is zeroed host memory with a registry of the live allocations; copies are memcpy;
// streams are dummies.  Every kernel entry point first holds each pointer argument against the registry: the pointer must
// lie in a live allocation and have behind it the bytes the real kernels touch (include/ttmlir_amd_hip.h: a tile tensor is
// backed by its whole padded extent).  A violation is an error return with a message, which the runtime turns into an
// exception - on the GPU the same call would be a memory fault.
// Every entry point then computes its result on the host with the oracle's arithmetic (f32, one rounding to the output
// type), so programs give the values the oracle gives.  A "launch" is a closure: between ttm_graph_begin_capture and
// ttm_graph_end_capture closures are recorded instead of run, as a capturing HIP stream records kernels, and
// ttm_graph_launch runs the recorded closures against whatever the recorded addresses hold by then.  With this the host
// runtime (executor, tensor pool, caches, fused launches, traces) runs whole programs on the CPU with checkable values.
#include <atomic>
#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cmath>
#include <cstring>
#include <functional>
#include <map>
#include <mutex>
#include <string>
#include <vector>

#include "ttmlir_amd_hip.h"
#include "ttm_extents.h"   // tt-mlir_amd/csrc: the bytes every entry point touches, shared with the kernel library

#define EXPORT extern "C" __attribute__((visibility("default")))

namespace {
thread_local std::string g_err;
std::mutex g_mu;
std::map<uintptr_t, size_t> g_allocs;            // base -> bytes
std::map<std::string, int> g_options;
std::atomic<long> g_kernel_calls{0}, g_capture_mark{-1};

int fail(const char *fmt, ...) {
  char buf[512];
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(buf, sizeof buf, fmt, ap);
  va_end(ap);
  g_err = std::string("null device: ") + buf;
  return TTM_ERR_INVALID;
}

using ttm_extents::pad32;
using ttm_extents::elem_bytes;
using ttm_extents::tile_bytes;
using ttm_extents::split3;

// `bytes` from p on lie in one live allocation
int span(const char *fn, const char *what, const void *p, int64_t bytes, bool optional = false) {
  if (!p) return optional ? TTM_OK : fail("%s: %s is null", fn, what);
  if (bytes <= 0) return TTM_OK;
  const uintptr_t a = (uintptr_t)p;
  std::lock_guard<std::mutex> g(g_mu);
  auto it = g_allocs.upper_bound(a);
  // every message of this function says "out of bounds": on the GPU the call would be a memory fault, not an error return
  if (it == g_allocs.begin()) return fail("out of bounds: %s: %s (%p) is not device memory", fn, what, p);
  --it;
  if (a >= it->first + it->second) return fail("out of bounds: %s: %s (%p) is not in a live device allocation", fn, what, p);
  const int64_t room = (int64_t)(it->first + it->second - a);
  if (bytes > room)
    return fail("out of bounds: %s: %s has %lld bytes behind it in its allocation, the kernels touch %lld", fn, what, (long long)room,
                (long long)bytes);
  return TTM_OK;
}
struct Chk {   // the checker the shared extent rules call
  const char *fn;
  int operator()(const char *what, const void *p, int64_t bytes, bool optional) const { return span(fn, what, p, bytes, optional); }
};
#define EXT(rule, ...) do { if (int rc_ = ttm_extents::rule(Chk{__func__}, __VA_ARGS__)) return rc_; } while (0)
#define SPAN(what, p, bytes) do { if (int rc_ = span(__func__, what, p, bytes)) return rc_; } while (0)

// a launch: run now, or recorded while a capture is in progress (the runtime serialises the work of a device)
using Launch = std::function<void()>;
struct Graph { std::vector<Launch> nodes; };
std::vector<Launch> *g_recording = nullptr;
// TTMLIR_AMD_NULL_DEVICE_COMPUTE=0: arithmetic launches are counted and recorded but do nothing (programs at benchmark
// sizes, where only the extents matter); copies and fills always run
const bool g_compute = !(getenv("TTMLIR_AMD_NULL_DEVICE_COMPUTE") && std::string(getenv("TTMLIR_AMD_NULL_DEVICE_COMPUTE")) == "0");
int launch(Launch f, bool cheap = false) {
  ++g_kernel_calls;
  if (!g_compute && !cheap) f = [] {};
  if (g_recording) g_recording->push_back(std::move(f)); else f();
  return TTM_OK;
}
int kernel() { return launch([] {}); }   // an entry point that computes nothing

// strided view (ttm_copy_view): the shared rule, with its "view reaches below offset 0" case as an error of its own
int view_span(const char *fn, const char *what, const void *p, int64_t rows, int64_t cols, int layout, int elem, int rank, const int64_t *extent,
              const int64_t *stride, int64_t base, int64_t extra_max) {
  bool negative = false;
  const int rc = ttm_extents::view(Chk{fn}, what, p, rows, cols, layout, elem, rank, extent, stride, base, extra_max, &negative);
  return negative ? fail("out of bounds: %s: the %s view reaches a negative logical offset", fn, what) : rc;
}

// ---- host arithmetic.  The oracle (oracle/ttm_oracle.c) supplies the formulas; tensors pass through dense row-major f32.
extern "C" {
void orc_tilize(const void *in, void *out, int64_t batch, int64_t rows, int64_t cols, int elem);
void orc_untilize(const void *in, void *out, int64_t batch, int64_t rows, int64_t cols, int elem);
void orc_bfp_pack_rm(const float *rm, uint8_t *out, int64_t batch, int64_t rows, int64_t cols, int fmt);
void orc_bfp_unpack_rm(const uint8_t *in, float *rm, int64_t batch, int64_t rows, int64_t cols, int fmt);
void orc_f32_to_bf16(const float *in, uint16_t *out, int64_t n);
void orc_f16_to_bf16(const uint16_t *in, uint16_t *out, int64_t n);
void orc_bf16_to_f16(const uint16_t *in, uint16_t *out, int64_t n);
void orc_unary_f32(int op, const float *in, float *out, int64_t n, float param);
void orc_binary_f32(int op, const float *a, const int64_t *ashape, const float *b, const int64_t *bshape, float *out,
                    const int64_t *oshape, int rank);
void orc_linear_f32(const float *A, const float *B, const float *bias, float *C, int64_t M, int64_t N, int64_t K, int transA,
                    int transB, int act);
void orc_rmsnorm_f32(const float *x, const float *w, const float *b, float *out, int64_t rows, int64_t cols, float eps);
void orc_softmax_f32(const float *x, float *out, int64_t outer, int64_t dim, int64_t inner);
void orc_reduce_f32(int op, const float *x, float *out, int64_t outer, int64_t dim, int64_t inner);
void orc_rotary_embedding_f32(const float *x, const float *cosc, const float *sinc, float *out, int64_t batch, int64_t rows, int64_t D,
                              int64_t token_index);
void orc_sdpa_decode_f32(const float *q, const float *k, const float *v, const int32_t *cur_pos, const float *mask, int mask_heads, float *out,
                         int64_t B, int64_t H, int64_t Hkv, int64_t S, int64_t D, int is_causal, float scale, int64_t window, const float *sink);
void orc_sdpa_f32(const float *q, const float *k, const float *v, const float *mask, int mask_heads, float *out, int64_t B,
                  int64_t Hq, int64_t Hkv, int64_t Sq, int64_t Sk, int64_t D, int is_causal, float scale, int64_t window,
                  const float *sink);
}

using Dense = std::vector<float>;
int64_t tiled_off(int64_t r, int64_t c, int64_t ct) {
  return ((r >> 5) * ct + (c >> 5)) * 1024 + (((r >> 4) & 1) * 2 + ((c >> 4) & 1)) * 256 + (r & 15) * 16 + (c & 15);
}
// physical element offset of logical (b, r, c) in a [batch, rows, cols] tensor
int64_t elem_off(int layout, int64_t rows, int64_t cols, int64_t b, int64_t r, int64_t c) {
  if (layout != TTM_TILE) return (b * rows + r) * cols + c;
  return b * pad32(rows) * pad32(cols) + tiled_off(r, c, pad32(cols) / 32);
}
float bf16_f32(uint16_t h) { uint32_t u = (uint32_t)h << 16; float f; memcpy(&f, &u, 4); return f; }
uint16_t f32_bf16(float f) { uint16_t h; orc_f32_to_bf16(&f, &h, 1); return h; }
float round_bf16(float f) { return bf16_f32(f32_bf16(f)); }
double load_scalar(const void *p, int dtype, int64_t i) {
  switch (dtype) {
  case TTM_F32: return ((const float *)p)[i];
  case TTM_BF16: return bf16_f32(((const uint16_t *)p)[i]);
  case TTM_F16: { uint16_t b; orc_f16_to_bf16((const uint16_t *)p + i, &b, 1); return bf16_f32(b); }   // callers that need f16 exactly do not exist
  case TTM_U32: return ((const uint32_t *)p)[i];
  case TTM_I32: return ((const int32_t *)p)[i];
  case TTM_U16: return ((const uint16_t *)p)[i];
  case TTM_U8: return ((const uint8_t *)p)[i];
  default: return 0.0;
  }
}
template <typename T> T saturate(double v, double lo, double hi) { return v != v ? (T)0 : (T)(v < lo ? lo : (v > hi ? hi : std::trunc(v))); }
void store_scalar(void *p, int dtype, int64_t i, double v) {
  switch (dtype) {
  case TTM_F32: ((float *)p)[i] = (float)v; break;
  case TTM_BF16: ((uint16_t *)p)[i] = f32_bf16((float)v); break;
  case TTM_F16: { uint16_t b = f32_bf16((float)v); orc_bf16_to_f16(&b, (uint16_t *)p + i, 1); break; }
  case TTM_U32: ((uint32_t *)p)[i] = saturate<uint32_t>(v, 0, 4294967295.0); break;
  case TTM_I32: ((int32_t *)p)[i] = saturate<int32_t>(v, -2147483648.0, 2147483647.0); break;
  case TTM_U16: ((uint16_t *)p)[i] = saturate<uint16_t>(v, 0, 65535.0); break;
  case TTM_U8: ((uint8_t *)p)[i] = saturate<uint8_t>(v, 0, 255.0); break;
  default: break;
  }
}
bool block_float(int dt) { return dt == TTM_BFP8B || dt == TTM_BFP4B; }
Dense load_dense(const void *p, int dtype, int layout, int64_t batch, int64_t rows, int64_t cols) {
  Dense d((size_t)(batch * rows * cols));
  if (block_float(dtype)) {
    orc_bfp_unpack_rm((const uint8_t *)p, d.data(), batch, rows, cols, dtype == TTM_BFP8B ? 8 : 4);
    return d;
  }
  for (int64_t b = 0; b < batch; ++b)
    for (int64_t r = 0; r < rows; ++r)
      for (int64_t c = 0; c < cols; ++c) d[(size_t)((b * rows + r) * cols + c)] = (float)load_scalar(p, dtype, elem_off(layout, rows, cols, b, r, c));
  return d;
}
// writes the tensor and, in TILE layout, zeros in its padding
void store_dense(const Dense &d, void *p, int dtype, int layout, int64_t batch, int64_t rows, int64_t cols) {
  if (block_float(dtype)) {
    orc_bfp_pack_rm(d.data(), (uint8_t *)p, batch, rows, cols, dtype == TTM_BFP8B ? 8 : 4);
    return;
  }
  if (layout == TTM_TILE) memset(p, 0, (size_t)tile_bytes(dtype, batch, rows, cols));
  for (int64_t b = 0; b < batch; ++b)
    for (int64_t r = 0; r < rows; ++r)
      for (int64_t c = 0; c < cols; ++c) store_scalar(p, dtype, elem_off(layout, rows, cols, b, r, c), d[(size_t)((b * rows + r) * cols + c)]);
}
Dense load_vec(const void *p, int dtype, int layout, int64_t cols) { return load_dense(p, dtype, layout, 1, 1, cols); }
void round_all_bf16(Dense &d) { for (float &f : d) f = round_bf16(f); }

// act(a w + bias) rounded to bf16, then the optional tail op with its own rounding: dense [batch, M, N]
Dense linear_host(const void *a, const void *w, int w_dtype, int transpose_w, const void *bias, int bias_dtype, int bias_layout, int64_t batch,
                  int64_t w_batch, int64_t M, int64_t N, int64_t K, int act, int tail_op, const void *tail) {
  Dense A = load_dense(a, TTM_BF16, TTM_TILE, batch, M, K);
  Dense W = transpose_w ? load_dense(w, w_dtype, TTM_TILE, w_batch, N, K) : load_dense(w, w_dtype, TTM_TILE, w_batch, K, N);
  Dense B;
  if (bias) B = load_vec(bias, bias_dtype, bias_layout, N);
  Dense C((size_t)(batch * M * N));
  for (int64_t b = 0; b < batch; ++b)
    orc_linear_f32(A.data() + b * M * K, W.data() + (w_batch == 1 ? 0 : b) * K * N, bias ? B.data() : nullptr, C.data() + b * M * N, M, N, K, 0,
                   transpose_w ? 1 : 0, act);
  round_all_bf16(C);
  if (tail_op != TTM_TAIL_NONE) {
    Dense T = load_dense(tail, TTM_BF16, TTM_TILE, batch, M, N);
    for (size_t i = 0; i < C.size(); ++i) C[i] = round_bf16(tail_op == TTM_TAIL_ADD ? C[i] + T[i] : C[i] * T[i]);
  }
  return C;
}
Dense rms_norm_host(const Dense &x, const void *weight, int weight_layout, const void *bias, int bias_layout, int dtype, int64_t rows, int64_t cols,
                    float eps) {
  Dense w, b, out(x.size());
  if (weight) w = load_vec(weight, dtype, weight_layout, cols);
  if (bias) b = load_vec(bias, dtype, bias_layout, cols);
  orc_rmsnorm_f32(x.data(), weight ? w.data() : nullptr, bias ? b.data() : nullptr, out.data(), rows, cols, eps);
  return out;
}
std::vector<int64_t> vec64(const int64_t *p, int n) { return p ? std::vector<int64_t>(p, p + n) : std::vector<int64_t>(); }
// a strided view copy on logical indices (include/ttmlir_amd_hip.h, ttm_copy_view)
void copy_view_host(const void *src, int64_t src_rows, int64_t src_cols, int src_layout, void *dst, int64_t dst_rows, int64_t dst_cols, int dst_layout,
                    int elem, const std::vector<int64_t> &extent, const std::vector<int64_t> &sstride, int64_t sbase,
                    const std::vector<int64_t> &dstride, int64_t dbase) {
  const int rank = (int)extent.size();
  int64_t n = 1;
  for (int64_t e : extent) n *= e;
  auto phys = [](int64_t idx, int64_t rows, int64_t cols, int layout) {
    const int64_t per = rows * cols;
    return elem_off(layout, rows, cols, idx / per, (idx % per) / cols, idx % cols);
  };
  for (int64_t i = 0; i < n; ++i) {
    int64_t rem = i, si = sbase, di = dbase;
    for (int d = rank - 1; d >= 0; --d) {
      const int64_t c = rem % extent[d]; rem /= extent[d];
      si += c * sstride[d]; di += c * dstride[d];
    }
    memcpy((uint8_t *)dst + phys(di, dst_rows, dst_cols, dst_layout) * elem, (const uint8_t *)src + phys(si, src_rows, src_cols, src_layout) * elem, elem);
  }
}
}  // namespace

EXPORT const char *ttm_last_error(void) { return g_err.c_str(); }

// ---- device, memory, streams, events
EXPORT int ttm_device_count(int *count) { if (!count) return fail("null count"); *count = 1; return TTM_OK; }
EXPORT int ttm_set_device(int device) { return device == 0 ? TTM_OK : fail("device %d does not exist", device); }
EXPORT int ttm_device_name(char *buf, size_t len) { if (buf && len) snprintf(buf, len, "null device (host memory, extent checks)"); return TTM_OK; }
EXPORT int ttm_mem_info(size_t *free_bytes, size_t *total_bytes) {
  if (free_bytes) *free_bytes = (size_t)1 << 34;
  if (total_bytes) *total_bytes = (size_t)1 << 34;
  return TTM_OK;
}
EXPORT int ttm_malloc(void **dptr, size_t bytes) {
  if (!dptr) return fail("ttm_malloc: null out pointer");
  if (bytes > ((size_t)2 << 30)) return fail("ttm_malloc: %zu bytes are more than this device has", bytes);   // damaged programs ask for anything
  void *p = nullptr;
  if (posix_memalign(&p, 256, bytes ? bytes : 1)) return fail("ttm_malloc: out of host memory (%zu bytes)", bytes);
  memset(p, 0, bytes);
  std::lock_guard<std::mutex> g(g_mu);
  g_allocs[(uintptr_t)p] = bytes;
  *dptr = p;
  return TTM_OK;
}
EXPORT int ttm_free(void *dptr) {
  if (!dptr) return TTM_OK;
  {
    std::lock_guard<std::mutex> g(g_mu);
    auto it = g_allocs.find((uintptr_t)dptr);
    if (it == g_allocs.end()) return fail("ttm_free: %p is not the start of a live device allocation", dptr);
    g_allocs.erase(it);
  }
  free(dptr);
  return TTM_OK;
}
EXPORT int ttm_host_alloc(void **hptr, size_t bytes) { if (!hptr) return fail("null"); *hptr = malloc(bytes ? bytes : 1); return *hptr ? TTM_OK : fail("out of memory"); }
EXPORT int ttm_host_free(void *hptr) { free(hptr); return TTM_OK; }
EXPORT int ttm_memcpy_h2d(void *dst, const void *src, size_t bytes, void *) {
  if (!bytes) return TTM_OK;
  if (!src) return fail("ttm_memcpy_h2d: null source");
  SPAN("destination", dst, (int64_t)bytes);
  memcpy(dst, src, bytes);
  return TTM_OK;
}
EXPORT int ttm_memcpy_d2h(void *dst, const void *src, size_t bytes, void *) {
  if (!bytes) return TTM_OK;
  if (!dst) return fail("ttm_memcpy_d2h: null destination");
  SPAN("source", src, (int64_t)bytes);
  memcpy(dst, src, bytes);
  return TTM_OK;
}
EXPORT int ttm_memcpy_d2d(void *dst, const void *src, size_t bytes, void *) {
  if (!bytes) return TTM_OK;
  SPAN("destination", dst, (int64_t)bytes);
  SPAN("source", src, (int64_t)bytes);
  return launch([=] { memmove(dst, src, bytes); }, true);
}
EXPORT int ttm_fill_u32(void *dst, uint32_t value, size_t count, void *) {
  if (!count) return TTM_OK;
  SPAN("destination", dst, (int64_t)count * 4);
  return launch([=] { for (size_t i = 0; i < count; ++i) ((uint32_t *)dst)[i] = value; }, true);
}
EXPORT int ttm_stream_create(void **stream) { if (!stream) return fail("null"); *stream = malloc(8); return TTM_OK; }
EXPORT int ttm_stream_destroy(void *stream) { free(stream); return TTM_OK; }
EXPORT int ttm_stream_sync(void *) { return TTM_OK; }
EXPORT int ttm_device_sync(void) { return TTM_OK; }
EXPORT int ttm_event_create(void **event) { if (!event) return fail("null"); *event = malloc(8); return TTM_OK; }
EXPORT int ttm_event_destroy(void *event) { free(event); return TTM_OK; }
EXPORT int ttm_event_record(void *, void *) { return TTM_OK; }
EXPORT int ttm_event_sync(void *) { return TTM_OK; }
EXPORT int ttm_event_elapsed_ms(float *ms, void *, void *) { if (ms) *ms = 0.0f; return TTM_OK; }

// ---- graphs: the launches between begin and end are recorded, not run; a replay runs them in order
EXPORT int ttm_graph_begin_capture(void *) {
  if (g_capture_mark >= 0) return fail("ttm_graph_begin_capture: a capture is already in progress");
  g_capture_mark = g_kernel_calls.load();
  g_recording = new std::vector<Launch>;
  return TTM_OK;
}
EXPORT int ttm_graph_end_capture(void *, void **graph_exec, size_t *num_nodes) {
  if (g_capture_mark < 0) return fail("ttm_graph_end_capture: no capture in progress");
  if (num_nodes) *num_nodes = (size_t)(g_kernel_calls.load() - g_capture_mark.load());
  g_capture_mark = -1;
  Graph *g = new Graph;
  g->nodes.swap(*g_recording);
  delete g_recording;
  g_recording = nullptr;
  if (graph_exec) *graph_exec = g; else delete g;
  return TTM_OK;
}
EXPORT int ttm_graph_launch(void *graph_exec, void *) {
  if (!graph_exec) return fail("ttm_graph_launch: null graph");
  if (g_recording) return fail("ttm_graph_launch: a capture is in progress");
  for (const Launch &f : ((Graph *)graph_exec)->nodes) f();
  return TTM_OK;
}
EXPORT int ttm_graph_destroy(void *graph_exec) { delete (Graph *)graph_exec; return TTM_OK; }
EXPORT int ttm_stream_is_capturing(void *, int *capturing) { if (capturing) *capturing = g_capture_mark >= 0; return TTM_OK; }

EXPORT int ttm_set_option(const char *name, int value) { if (!name) return fail("null"); g_options[name] = value; return TTM_OK; }
EXPORT int ttm_get_option(const char *name, int *value) { if (!name || !value) return fail("null"); *value = g_options[name]; return TTM_OK; }

// ---- layout, block float, typecast
EXPORT int ttm_copy_kernel(const void *src, void *dst, size_t bytes, void *) {
  EXT(copy_kernel, src, dst, bytes);
  return launch([=] { memmove(dst, src, bytes); }, true);
}
EXPORT int ttm_tilize(const void *src, void *dst, int64_t batch, int64_t rows, int64_t cols, int elem, void *) {
  if (batch * rows * cols == 0) return TTM_OK;
  EXT(tilize, src, dst, batch, rows, cols, elem);
  return launch([=] { orc_tilize(src, dst, batch, rows, cols, elem); });
}
EXPORT int ttm_untilize(const void *src, void *dst, int64_t batch, int64_t rows, int64_t cols, int elem, void *) {
  if (batch * rows * cols == 0) return TTM_OK;
  EXT(untilize, src, dst, batch, rows, cols, elem);
  return launch([=] { orc_untilize(src, dst, batch, rows, cols, elem); });
}
EXPORT int64_t ttm_bfp_tile_bytes(int fmt) { return fmt == TTM_BFP8B ? 1088 : (fmt == TTM_BFP4B ? 576 : -1); }
EXPORT int ttm_bfp_pack(const void *src, int src_dtype, int src_layout, void *dst, int fmt, int64_t batch, int64_t rows, int64_t cols, void *) {
  if (batch * rows * cols == 0) return TTM_OK;
  EXT(bfp_pack, src, src_dtype, src_layout, dst, fmt, batch, rows, cols);
  return launch([=] { store_dense(load_dense(src, src_dtype, src_layout, batch, rows, cols), dst, fmt, TTM_TILE, batch, rows, cols); });
}
EXPORT int ttm_bfp_unpack(const void *src, int fmt, void *dst, int dst_dtype, int dst_layout, int64_t batch, int64_t rows, int64_t cols, void *) {
  if (batch * rows * cols == 0) return TTM_OK;
  EXT(bfp_unpack, src, fmt, dst, dst_dtype, dst_layout, batch, rows, cols);
  return launch([=] { store_dense(load_dense(src, fmt, TTM_TILE, batch, rows, cols), dst, dst_dtype, dst_layout, batch, rows, cols); });
}
EXPORT int ttm_typecast(const void *in, int src_dtype, void *out, int dst_dtype, int64_t n, void *) {
  if (n == 0) return TTM_OK;
  EXT(typecast, in, src_dtype, out, dst_dtype, n);
  return launch([=] { for (int64_t i = 0; i < n; ++i) store_scalar(out, dst_dtype, i, load_scalar(in, src_dtype, i)); });
}

// ---- matmul / linear
static int linear_check(const char *fn, const void *a, int a_dtype, const void *w, int w_dtype, int transpose_w, const void *bias, int bias_dtype,
                        int bias_layout, void *out, int out_dtype, int64_t batch, int64_t w_batch, int64_t M, int64_t N, int64_t K, int act, int tail_op,
                        const void *tail) {
  if (batch * M * N == 0) return TTM_OK;
  if (int rc = ttm_extents::linear(Chk{fn}, a, a_dtype, w, w_dtype, bias, bias_dtype, bias_layout, out, out_dtype, batch, w_batch, M, N, K, tail_op, tail))
    return rc;
  if (a_dtype != TTM_BF16 || out_dtype != TTM_BF16) return kernel();
  return launch([=] {
    store_dense(linear_host(a, w, w_dtype, transpose_w, bias, bias_dtype, bias_layout, batch, w_batch, M, N, K, act, tail_op, tail), out, TTM_BF16,
                TTM_TILE, batch, M, N);
  });
}
EXPORT int ttm_linear(const void *a, int a_dtype, const void *w, int w_dtype, int transpose_w, const void *bias, int bias_dtype, int bias_layout,
                      void *out, int out_dtype, int64_t batch, int64_t w_batch, int64_t M, int64_t N, int64_t K, int act, void *) {
  return linear_check(__func__, a, a_dtype, w, w_dtype, transpose_w, bias, bias_dtype, bias_layout, out, out_dtype, batch, w_batch, M, N, K, act,
                      TTM_TAIL_NONE, nullptr);
}
EXPORT int ttm_linear_tail(const void *a, int a_dtype, const void *w, int w_dtype, int transpose_w, const void *bias, int bias_dtype, int bias_layout,
                           void *out, int out_dtype, int64_t batch, int64_t w_batch, int64_t M, int64_t N, int64_t K, int act, int tail_op,
                           const void *tail, void *) {
  return linear_check(__func__, a, a_dtype, w, w_dtype, transpose_w, bias, bias_dtype, bias_layout, out, out_dtype, batch, w_batch, M, N, K, act,
                      tail_op, tail);
}
EXPORT int ttm_linear_group(const void *a, int n, const void *const *w, int w_dtype, void *const *out, const int64_t *N, const int *act, int64_t M,
                            int64_t K, void *) {
  if (n < 1 || n > 4 || !w || !out || !N) return fail("ttm_linear_group: one to four members with weights, outputs and widths");
  EXT(linear_group, a, n, w, w_dtype, out, N, M, K);
  std::vector<const void *> ws(w, w + n);
  std::vector<void *> outs(out, out + n);
  std::vector<int64_t> ns(N, N + n);
  std::vector<int> acts(n, TTM_ACT_NONE);
  if (act) acts.assign(act, act + n);
  return launch([=] {
    for (int i = 0; i < n; ++i)
      store_dense(linear_host(a, ws[i], w_dtype, 0, nullptr, TTM_BF16, TTM_TILE, 1, 1, M, ns[i], K, acts[i], TTM_TAIL_NONE, nullptr), outs[i], TTM_BF16,
                  TTM_TILE, 1, M, ns[i]);
  });
}
EXPORT int ttm_linear_pair(const void *a, const void *w0, const void *w1, int w_dtype, void *out0, void *out1, int64_t M, int64_t N, int64_t K, void *) {
  EXT(linear_pair, a, w0, w1, w_dtype, out0, out1, M, N, K);
  return launch([=] {
    store_dense(linear_host(a, w0, w_dtype, 0, nullptr, TTM_BF16, TTM_TILE, 1, 1, M, N, K, TTM_ACT_NONE, TTM_TAIL_NONE, nullptr), out0, TTM_BF16, TTM_TILE, 1, M, N);
    store_dense(linear_host(a, w1, w_dtype, 0, nullptr, TTM_BF16, TTM_TILE, 1, 1, M, N, K, TTM_ACT_NONE, TTM_TAIL_NONE, nullptr), out1, TTM_BF16, TTM_TILE, 1, M, N);
  });
}
// the predicates of the real library at its default options
EXPORT int ttm_linear_glu_supported(int w_dtype, int64_t M, int64_t N, int64_t K) {
  const int64_t groups = ((N + 31) / 32 + 1) / 2, kt = (K + 31) / 32;
  if (w_dtype == TTM_BFP8B && M > 64 && M <= 1024 && K > 0 && N >= 1 && g_options["linear_two_pass"] != 2 && g_options["linear_glu_main"] != 1) {
    // the gated form of the fused main kernel, where the real library's model keeps the pair of projections in one pass (256 CUs)
    const int64_t ksteps = (kt + 1) / 2, nt = (N + 31) / 32, blocks = ((M + 255) / 256) * ((2 * nt + 7) / 8), rounds = (blocks + 255) / 256;
    const double fused = rounds * (ksteps + 12) * 1.65, first = 3.0 + static_cast<double>(kt) * 2 * nt * (1088.0 + 2048.0) / 5.5e6;
    const double multiply = 3.0 + 3.0 * static_cast<double>((M + 31) / 32) * nt * 2048.0 / 5.5e6;
    if (g_options["linear_two_pass"] == 1 || !(0.28 * fused - first > multiply)) return 1;
  }
  return block_float(w_dtype) && M >= 1 && M <= 32 && K > 0 && N >= 1 && std::min<int64_t>(256 / groups, kt / 32) <= 1;
}
EXPORT int ttm_linear_glu(const void *a, const void *w_gate, const void *w_up, int w_dtype, void *out, int64_t M, int64_t N, int64_t K, int act_gate,
                          int act_up, void *) {
  if (!ttm_linear_glu_supported(w_dtype, M, N, K)) return fail("ttm_linear_glu: unsupported shape");
  EXT(linear_glu, a, w_gate, w_up, w_dtype, out, M, N, K);
  return launch([=] {
    // the op sequence it stands for: the gate projection stored as bf16 tiles, then the up projection with the multiply as its tail
    std::vector<uint8_t> gate(static_cast<size_t>(((M + 31) / 32) * ((N + 31) / 32)) * 2048);
    store_dense(linear_host(a, w_gate, w_dtype, 0, nullptr, TTM_BF16, TTM_TILE, 1, 1, M, N, K, act_gate, TTM_TAIL_NONE, nullptr), gate.data(), TTM_BF16,
                TTM_TILE, 1, M, N);
    store_dense(linear_host(a, w_up, w_dtype, 0, nullptr, TTM_BF16, TTM_TILE, 1, 1, M, N, K, act_up, TTM_TAIL_MUL, gate.data()), out, TTM_BF16, TTM_TILE, 1,
                M, N);
  });
}
EXPORT int ttm_linear_add_rms_norm_supported(int w_dtype, int64_t M, int64_t N, int64_t K) {
  return block_float(w_dtype) && M >= 1 && M <= 32 && K > 0 && N >= 1 && (N + 31) / 32 * 4 <= 8 * 256;
}
EXPORT int ttm_linear_add_rms_norm(const void *a, const void *w, int w_dtype, const void *residual, void *sum_out, const void *norm_weight,
                                   int weight_layout, const void *norm_bias, int bias_layout, float eps, void *norm_out, int64_t M, int64_t N, int64_t K,
                                   void *) {
  if (!ttm_linear_add_rms_norm_supported(w_dtype, M, N, K)) return fail("ttm_linear_add_rms_norm: unsupported shape");
  EXT(linear_add_rms_norm, a, w, w_dtype, residual, sum_out, norm_weight, weight_layout, norm_bias, bias_layout, norm_out, M, N, K);
  if (sum_out == residual || norm_out == sum_out || norm_out == residual) return fail("ttm_linear_add_rms_norm: the outputs alias");
  return launch([=] {
    Dense x1 = linear_host(a, w, w_dtype, 0, nullptr, TTM_BF16, TTM_TILE, 1, 1, M, N, K, TTM_ACT_NONE, TTM_TAIL_ADD, residual);
    store_dense(x1, sum_out, TTM_BF16, TTM_TILE, 1, M, N);
    store_dense(rms_norm_host(x1, norm_weight, weight_layout, norm_bias, bias_layout, TTM_BF16, M, N, eps), norm_out, TTM_BF16, TTM_TILE, 1, M, N);
  });
}
EXPORT int ttm_linear_qkv_decode_supported(int w_dtype, int64_t users, int64_t K, int64_t heads, int64_t kv_heads, int64_t head_dim) {
  return block_float(w_dtype) && users >= 1 && users <= 32 && K > 0 && heads >= 1 && kv_heads >= 1 && head_dim >= 32 && head_dim % 32 == 0;
}
EXPORT int ttm_linear_qkv_decode(const void *a, const void *wq, const void *wk, const void *wv, int w_dtype, int64_t users, int64_t K, int64_t heads,
                                 int64_t kv_heads, int64_t head_dim, const void *cos_cache, const void *sin_cache, int64_t cache_rows,
                                 int64_t token_index, void *q_out, void *k_cache, void *v_cache, int64_t cache_users, int64_t max_seq,
                                 const int32_t *update_index, int64_t batch_offset, void *) {
  if (!ttm_linear_qkv_decode_supported(w_dtype, users, K, heads, kv_heads, head_dim)) return fail("ttm_linear_qkv_decode: unsupported shape");
  if (token_index < 0 || token_index >= cache_rows) return fail("ttm_linear_qkv_decode: token_index outside the cached positions");
  if (batch_offset < 0 || batch_offset + users > cache_users) return fail("ttm_linear_qkv_decode: batch_offset + users exceeds the cache");
  EXT(linear_qkv_decode, a, wq, wk, wv, w_dtype, users, K, heads, kv_heads, head_dim, cos_cache, sin_cache, cache_rows, q_out, k_cache, v_cache,
      cache_users, max_seq, update_index);
  return launch([=] {
    // the op sequence it replaces: three projections rounded to bf16, rotary embedding of q and k at row token_index, q as
    // [1, users, heads, head_dim] with zeroed padding rows, k and v rows into the caches at *update_index
    const int64_t D = head_dim, nq = heads * D, nk = kv_heads * D;
    Dense Q = linear_host(a, wq, w_dtype, 0, nullptr, TTM_BF16, TTM_TILE, 1, 1, users, nq, K, TTM_ACT_NONE, TTM_TAIL_NONE, nullptr);
    Dense Kp = linear_host(a, wk, w_dtype, 0, nullptr, TTM_BF16, TTM_TILE, 1, 1, users, nk, K, TTM_ACT_NONE, TTM_TAIL_NONE, nullptr);
    Dense Vp = linear_host(a, wv, w_dtype, 0, nullptr, TTM_BF16, TTM_TILE, 1, 1, users, nk, K, TTM_ACT_NONE, TTM_TAIL_NONE, nullptr);
    Dense C = load_dense(cos_cache, TTM_BF16, TTM_TILE, 1, cache_rows, D), S_ = load_dense(sin_cache, TTM_BF16, TTM_TILE, 1, cache_rows, D);
    Dense Qr(Q.size()), Kr(Kp.size());
    orc_rotary_embedding_f32(Q.data(), C.data(), S_.data(), Qr.data(), 1, users * heads, D, token_index);
    orc_rotary_embedding_f32(Kp.data(), C.data(), S_.data(), Kr.data(), 1, users * kv_heads, D, token_index);
    store_dense(Qr, q_out, TTM_BF16, TTM_TILE, users, heads, D);
    const int64_t at = *update_index;
    if (at < 0 || at >= max_seq) return;
    for (int64_t u = 0; u < users; ++u)
      for (int64_t h = 0; h < kv_heads; ++h)
        for (int64_t d = 0; d < D; ++d) {
          const int64_t off = elem_off(TTM_TILE, max_seq, D, (batch_offset + u) * kv_heads + h, at, d);
          store_scalar(k_cache, TTM_BF16, off, Kr[(size_t)((u * kv_heads + h) * D + d)]);
          store_scalar(v_cache, TTM_BF16, off, Vp[(size_t)((u * kv_heads + h) * D + d)]);
        }
  });
}

// ---- element-wise
EXPORT int ttm_eltwise_unary(int op, const void *in, void *out, int dtype, int layout, int64_t batch, int64_t rows, int64_t cols, float param, void *) {
  if (batch * rows * cols == 0) return TTM_OK;
  EXT(unary, in, out, dtype, layout, batch, rows, cols);
  return launch([=] {
    Dense x = load_dense(in, dtype, layout, batch, rows, cols), y(x.size());
    orc_unary_f32(op, x.data(), y.data(), (int64_t)x.size(), param);
    store_dense(y, out, dtype, layout, batch, rows, cols);
  });
}
EXPORT int ttm_clamp(const void *in, void *out, int dtype, int layout, int64_t batch, int64_t rows, int64_t cols, float lo, float hi, void *) {
  if (batch * rows * cols == 0) return TTM_OK;
  EXT(unary, in, out, dtype, layout, batch, rows, cols);
  return launch([=] {
    Dense x = load_dense(in, dtype, layout, batch, rows, cols);
    for (float &f : x) f = f != f ? f : std::fmin(std::fmax(f, lo), hi);
    store_dense(x, out, dtype, layout, batch, rows, cols);
  });
}
// the real library refuses operands that do not broadcast to the output
static int broadcasts(const char *fn, const int64_t *shape, const int64_t *out_shape, int rank) {
  for (int d = 0; d < rank; ++d)
    if (shape && out_shape && shape[d] != out_shape[d] && shape[d] != 1) return fail("%s: shapes do not broadcast at dim %d", fn, d);
  return TTM_OK;
}
EXPORT int ttm_eltwise_binary(int op, const void *a, const int64_t *a_shape, const void *b, const int64_t *b_shape, void *out, const int64_t *out_shape,
                              int rank, int dtype, int layout, void *) {
  if (rank < 0 || rank > 8) return fail("ttm_eltwise_binary: rank");
  if (int rc = broadcasts(__func__, a_shape, out_shape, rank)) return rc;
  if (int rc = broadcasts(__func__, b_shape, out_shape, rank)) return rc;
  EXT(binary, a, a_shape, b, b_shape, out, out_shape, rank, dtype, layout);
  const bool oracle_op = op == 0 || op == 1 || (op >= 3 && op <= 10), extremum = op == 100 || op == 101;   // maximum, minimum
  if (!oracle_op && !extremum) return kernel();
  const std::vector<int64_t> as = vec64(a_shape, rank), bs = vec64(b_shape, rank), os = vec64(out_shape, rank);
  return launch([=] {
    int64_t ab, ar, ac, bb, br, bc, ob, orr, oc;
    split3(as.data(), rank, ab, ar, ac); split3(bs.data(), rank, bb, br, bc); split3(os.data(), rank, ob, orr, oc);
    Dense x = load_dense(a, dtype, layout, ab, ar, ac), y = load_dense(b, dtype, layout, bb, br, bc), z((size_t)(ob * orr * oc));
    if (oracle_op) {
      orc_binary_f32(op, x.data(), as.data(), y.data(), bs.data(), z.data(), os.data(), rank);
    } else {   // select through two comparisons of the oracle, then put NaN where either operand has one
      Dense ge(z.size()), xe(z.size()), ye(z.size()), zero(1, 0.0f);
      std::vector<int64_t> ones(rank, 1);
      orc_binary_f32(op == 100 ? 6 : 8, x.data(), as.data(), y.data(), bs.data(), ge.data(), os.data(), rank);
      orc_binary_f32(0, x.data(), as.data(), zero.data(), ones.data(), xe.data(), os.data(), rank);   // operands broadcast to the output
      orc_binary_f32(0, y.data(), bs.data(), zero.data(), ones.data(), ye.data(), os.data(), rank);
      for (size_t i = 0; i < z.size(); ++i) z[i] = (xe[i] != xe[i] || ye[i] != ye[i]) ? NAN : (ge[i] != 0.0f ? xe[i] : ye[i]);
    }
    store_dense(z, out, dtype, layout, ob, orr, oc);
  });
}
EXPORT int ttm_where(const void *cond, const int64_t *cond_shape, const void *a, const int64_t *a_shape, const void *b, const int64_t *b_shape, void *out,
                     const int64_t *out_shape, int rank, int dtype, int layout, void *) {
  if (rank < 0 || rank > 4) return fail("ttm_where: rank");
  for (const int64_t *sh : {cond_shape, a_shape, b_shape})
    if (int rc = broadcasts(__func__, sh, out_shape, rank)) return rc;
  EXT(where, cond, cond_shape, a, a_shape, b, b_shape, out, out_shape, rank, dtype, layout);
  const std::vector<int64_t> cs = vec64(cond_shape, rank), as = vec64(a_shape, rank), bs = vec64(b_shape, rank), os = vec64(out_shape, rank);
  return launch([=] {
    int64_t cb, cr, cc, ab, ar, ac, bb, br, bc, ob, orr, oc;
    split3(cs.data(), rank, cb, cr, cc); split3(as.data(), rank, ab, ar, ac); split3(bs.data(), rank, bb, br, bc); split3(os.data(), rank, ob, orr, oc);
    Dense c = load_dense(cond, dtype, layout, cb, cr, cc), x = load_dense(a, dtype, layout, ab, ar, ac), y = load_dense(b, dtype, layout, bb, br, bc);
    Dense ce((size_t)(ob * orr * oc)), xe(ce.size()), ye(ce.size()), zero(1, 0.0f), one(1, 1.0f);
    std::vector<int64_t> ones(rank, 1);
    orc_binary_f32(5, c.data(), cs.data(), zero.data(), ones.data(), ce.data(), os.data(), rank);   // cond != 0 (true for NaN)
    orc_binary_f32(1, x.data(), as.data(), one.data(), ones.data(), xe.data(), os.data(), rank);    // operands broadcast to the output
    orc_binary_f32(1, y.data(), bs.data(), one.data(), ones.data(), ye.data(), os.data(), rank);
    for (size_t i = 0; i < ce.size(); ++i) xe[i] = ce[i] != 0.0f ? xe[i] : ye[i];
    store_dense(xe, out, dtype, layout, ob, orr, oc);
  });
}
EXPORT int ttm_embedding(const void *indices, int index_dtype, const void *weight, void *out, int elem, int64_t rows, int64_t vocab, int64_t dim, void *) {
  if (rows * dim == 0) return TTM_OK;
  EXT(embedding, indices, weight, out, elem, rows, vocab, dim);
  return launch([=] {
    for (int64_t r = 0; r < rows; ++r) {
      int64_t i = index_dtype == TTM_U32 ? (int64_t)((const uint32_t *)indices)[r] : (int64_t)((const int32_t *)indices)[r];
      i = i < 0 ? 0 : (i >= vocab ? vocab - 1 : i);
      memcpy((uint8_t *)out + r * dim * elem, (const uint8_t *)weight + i * dim * elem, (size_t)(dim * elem));
    }
  });
}
EXPORT int ttm_argmax(const void *in, int dtype, int32_t *out, int64_t rows, int64_t cols, void *) {
  if (rows * cols == 0) return TTM_OK;
  EXT(argmax, in, dtype, out, rows, cols);
  return launch([=] {
    for (int64_t r = 0; r < rows; ++r) {
      int64_t best = 0;
      float bv = (float)load_scalar(in, dtype, r * cols);
      for (int64_t c = 1; c < cols && bv == bv; ++c) {   // the first NaN wins, else the first largest
        const float v = (float)load_scalar(in, dtype, r * cols + c);
        if (v != v || v > bv) { bv = v; best = c; }
      }
      out[r] = (int32_t)best;
    }
  });
}
EXPORT int ttm_arange(void *out, int dtype, int64_t n, double start, double step, void *) {
  if (n == 0) return TTM_OK;
  EXT(arange, out, dtype, n);
  return launch([=] { for (int64_t i = 0; i < n; ++i) store_scalar(out, dtype, i, (float)start + (float)i * (float)step); });
}

// ---- row-wise
EXPORT int ttm_rms_norm(const void *x, const void *weight, int weight_layout, const void *bias, int bias_layout, void *out, int dtype, int64_t batch,
                        int64_t rows, int64_t cols, float eps, void *) {
  if (batch * rows * cols == 0) return TTM_OK;
  EXT(rms_norm, x, weight, weight_layout, bias, bias_layout, out, dtype, batch, rows, cols);
  return launch([=] {
    store_dense(rms_norm_host(load_dense(x, dtype, TTM_TILE, batch, rows, cols), weight, weight_layout, bias, bias_layout, dtype, batch * rows, cols, eps),
                out, dtype, TTM_TILE, batch, rows, cols);
  });
}
EXPORT int ttm_softmax_lastdim(const void *x, void *out, int dtype, int64_t batch, int64_t rows, int64_t cols, void *) {
  if (batch * rows * cols == 0) return TTM_OK;
  EXT(softmax, x, out, dtype, batch, rows, cols);
  return launch([=] {
    Dense in = load_dense(x, dtype, TTM_TILE, batch, rows, cols), y(in.size());
    orc_softmax_f32(in.data(), y.data(), batch * rows, cols, 1);
    store_dense(y, out, dtype, TTM_TILE, batch, rows, cols);
  });
}
EXPORT int ttm_reduce_lastdim(int op, const void *x, void *out, int dtype, int64_t batch, int64_t rows, int64_t cols, void *) {
  if (batch * rows * cols == 0) return TTM_OK;
  EXT(reduce, x, out, dtype, batch, rows, cols);
  return launch([=] {
    Dense in = load_dense(x, dtype, TTM_TILE, batch, rows, cols), y((size_t)(batch * rows));
    orc_reduce_f32(op, in.data(), y.data(), batch * rows, cols, 1);
    store_dense(y, out, dtype, TTM_TILE, batch, rows, 1);
  });
}

// ---- strided views
EXPORT int ttm_copy_view(const void *src, int64_t src_rows, int64_t src_cols, int src_layout, void *dst, int64_t dst_rows, int64_t dst_cols,
                         int dst_layout, int elem, int rank, const int64_t *extent, const int64_t *src_stride, int64_t src_base,
                         const int64_t *dst_stride, int64_t dst_base, void *) {
  if (rank < 0 || rank > 8 || (rank > 0 && (!extent || !src_stride || !dst_stride))) return fail("ttm_copy_view: rank / descriptors");
  if (int rc = view_span(__func__, "source", src, src_rows, src_cols, src_layout, elem, rank, extent, src_stride, src_base, 0)) return rc;
  if (int rc = view_span(__func__, "destination", dst, dst_rows, dst_cols, dst_layout, elem, rank, extent, dst_stride, dst_base, 0)) return rc;
  const std::vector<int64_t> ex = vec64(extent, rank), ss = vec64(src_stride, rank), ds = vec64(dst_stride, rank);
  return launch([=] { copy_view_host(src, src_rows, src_cols, src_layout, dst, dst_rows, dst_cols, dst_layout, elem, ex, ss, src_base, ds, dst_base); });
}
EXPORT int ttm_copy_view_at(const void *src, int64_t src_rows, int64_t src_cols, int src_layout, void *dst, int64_t dst_rows, int64_t dst_cols,
                            int dst_layout, int elem, int rank, const int64_t *extent, const int64_t *src_stride, int64_t src_base,
                            const int64_t *dst_stride, int64_t dst_base, const int32_t *index, int64_t index_stride, int64_t index_limit, void *) {
  if (rank < 0 || rank > 8 || (rank > 0 && (!extent || !src_stride || !dst_stride))) return fail("ttm_copy_view_at: rank / descriptors");
  SPAN("index", index, 4);
  if (int rc = view_span(__func__, "source", src, src_rows, src_cols, src_layout, elem, rank, extent, src_stride, src_base, 0)) return rc;
  const int64_t far = index_limit > 0 ? (index_limit - 1) * index_stride : 0;
  if (int rc = view_span(__func__, "destination", dst, dst_rows, dst_cols, dst_layout, elem, rank, extent, dst_stride, dst_base, far)) return rc;
  const std::vector<int64_t> ex = vec64(extent, rank), ss = vec64(src_stride, rank), ds = vec64(dst_stride, rank);
  return launch([=] {
    const int64_t at = *index;   // read when the launch runs: a replayed graph sees the current position
    if (at < 0 || at >= index_limit) return;
    copy_view_host(src, src_rows, src_cols, src_layout, dst, dst_rows, dst_cols, dst_layout, elem, ex, ss, src_base, ds, dst_base + at * index_stride);
  });
}

// ---- attention
// [B, S, H * D] <-> [B, H, S, D]
static Dense heads_outer(const Dense &x, int64_t B, int64_t H, int64_t S, int64_t D, bool inverse) {
  Dense y(x.size());
  for (int64_t b = 0; b < B; ++b)
    for (int64_t h = 0; h < H; ++h)
      for (int64_t s_ = 0; s_ < S; ++s_)
        for (int64_t d = 0; d < D; ++d) {
          const size_t inner = (size_t)(((b * S + s_) * H + h) * D + d), outer = (size_t)(((b * H + h) * S + s_) * D + d);
          if (inverse) y[inner] = x[outer]; else y[outer] = x[inner];
        }
  return y;
}
static int sdpa_check(const char *fn, const void *q, const void *k, const void *v, const void *mask, int mask_heads, int64_t mask_batch, void *out, int dtype,
                      int64_t B, int64_t Hq, int64_t Hkv, int64_t Sq, int64_t Sk, int64_t D, const void *sink, int is_causal = 0, float scale = 0.0f,
                      int heads_inner = 0, int64_t window = -1) {
  if (B * Hq * Sq * D == 0) return TTM_OK;
  if (Hkv < 1 || Hq % Hkv != 0) return fail("%s: query heads must be a multiple of kv heads", fn);
  if (int rc = ttm_extents::sdpa(Chk{fn}, q, k, v, mask, mask_heads, mask_batch, out, dtype, B, Hq, Hkv, Sq, Sk, D, sink)) return rc;
  return launch([=] {
    auto operand = [&](const void *p, int64_t H, int64_t S, bool inner) {
      return inner ? heads_outer(load_dense(p, dtype, TTM_TILE, B, S, H * D), B, H, S, D, false) : load_dense(p, dtype, TTM_TILE, B * H, S, D);
    };
    Dense Q = operand(q, Hq, Sq, heads_inner & 1), K = operand(k, Hkv, Sk, heads_inner & 2), V = operand(v, Hkv, Sk, heads_inner & 4), M, S_, O(Q.size());
    if (mask) {
      M = load_dense(mask, dtype, TTM_TILE, mask_batch * mask_heads, Sq, Sk);
      if (mask_batch == 1 && B > 1) { Dense one = M; for (int64_t b = 1; b < B; ++b) M.insert(M.end(), one.begin(), one.end()); }
    }
    if (sink) S_ = load_dense(sink, TTM_BF16, TTM_TILE, Hq, 1, 1);
    orc_sdpa_f32(Q.data(), K.data(), V.data(), mask ? M.data() : nullptr, mask_heads, O.data(), B, Hq, Hkv, Sq, Sk, D, is_causal, scale, window < 0 ? -1 : window,
                 sink ? S_.data() : nullptr);
    if (heads_inner & 8) store_dense(heads_outer(O, B, Hq, Sq, D, true), out, dtype, TTM_TILE, B, Sq, Hq * D);
    else store_dense(O, out, dtype, TTM_TILE, B * Hq, Sq, D);
  });
}
EXPORT int ttm_sdpa(const void *q, const void *k, const void *v, const void *mask, int mask_heads, void *out, int dtype, int64_t B, int64_t Hq, int64_t Hkv,
                    int64_t Sq, int64_t Sk, int64_t D, int is_causal, float scale, void *) {
  return sdpa_check(__func__, q, k, v, mask, mask_heads, B, out, dtype, B, Hq, Hkv, Sq, Sk, D, nullptr, is_causal, scale);
}
EXPORT int ttm_sdpa_heads_inner(const void *q, const void *k, const void *v, const void *mask, int mask_heads, void *out, int dtype, int64_t B, int64_t Hq,
                                int64_t Hkv, int64_t Sq, int64_t Sk, int64_t D, int is_causal, float scale, int heads_inner, void *) {
  return sdpa_check(__func__, q, k, v, mask, mask_heads, B, out, dtype, B, Hq, Hkv, Sq, Sk, D, nullptr, is_causal, scale, heads_inner);
}
EXPORT int ttm_sdpa_windowed(const void *q, const void *k, const void *v, const void *mask, int mask_heads, int64_t mask_batch, void *out, int dtype,
                             int64_t B, int64_t Hq, int64_t Hkv, int64_t Sq, int64_t Sk, int64_t D, int is_causal, float scale, int heads_inner,
                             int64_t sliding_window, const void *attention_sink, void *) {
  return sdpa_check(__func__, q, k, v, mask, mask_heads, mask_batch, out, dtype, B, Hq, Hkv, Sq, Sk, D, attention_sink, is_causal, scale, heads_inner,
                    sliding_window);
}
static int decode_check(const char *fn, const void *q, const void *k, const void *v, const int32_t *cur_pos, const void *mask, int mask_heads,
                        int64_t mask_batch, const int32_t *page_table, int64_t pages_per_user, int64_t page_block, int64_t page_blocks, void *out, int dtype,
                        int64_t batch, int64_t heads, int64_t kv_heads, int64_t seq, int64_t head_dim, int concat_heads, const void *sink,
                        int is_causal = 0, float scale = 0.0f, int64_t window = -1) {
  if (batch * heads * head_dim == 0) return TTM_OK;
  if (int rc = ttm_extents::sdpa_decode(Chk{fn}, q, k, v, cur_pos, mask, mask_heads, mask_batch, page_table, pages_per_user, page_block, page_blocks, out,
                                        dtype, batch, heads, kv_heads, seq, head_dim, concat_heads, sink))
    return rc;
  if (kv_heads < 1 || heads % kv_heads != 0) return fail("%s: query heads must be a multiple of kv heads", fn);
  return launch([=] {
    const int64_t B = batch, H = heads, Hk = kv_heads, S = seq, D = head_dim;
    Dense Q = load_dense(q, dtype, TTM_TILE, B, H, D), K((size_t)(B * Hk * S * D)), V(K.size()), O(Q.size());
    // the keys a user sees, as an additive mask: the caller's mask, the keys past cur_pos (the kernels apply both) and the
    // positions whose page-table entry names no page
    const int mh = mask ? mask_heads : 1;
    Dense M((size_t)(B * mh * S), 0.0f);
    if (mask) {
      Dense m = load_dense(mask, dtype, TTM_TILE, mask_batch, mask_heads, S);
      for (int64_t b = 0; b < B; ++b)
        for (int64_t i = 0; i < mh * S; ++i) M[(size_t)(b * mh * S + i)] = m[(size_t)((mask_batch == 1 ? 0 : b) * mh * S + i)];
    }
    if (page_table) {
      Dense PK = load_dense(k, dtype, TTM_TILE, page_blocks * Hk, page_block, D), PV = load_dense(v, dtype, TTM_TILE, page_blocks * Hk, page_block, D);
      for (int64_t b = 0; b < B; ++b)
        for (int64_t j = 0; j < S; ++j) {
          const int64_t page = page_table[b * pages_per_user + j / page_block];
          const bool ok = page >= 0 && page < page_blocks;
          for (int64_t h = 0; h < Hk; ++h)
            for (int64_t d = 0; d < D; ++d) {
              const size_t to = (size_t)(((b * Hk + h) * S + j) * D + d), from = (size_t)((((ok ? page : 0) * Hk + h) * page_block + j % page_block) * D + d);
              K[to] = ok ? PK[from] : 0.0f;
              V[to] = ok ? PV[from] : 0.0f;
            }
          if (!ok)
            for (int64_t hh = 0; hh < mh; ++hh) M[(size_t)((b * mh + hh) * S + j)] = -INFINITY;
        }
    } else {
      K = load_dense(k, dtype, TTM_TILE, B * Hk, S, D);
      V = load_dense(v, dtype, TTM_TILE, B * Hk, S, D);
    }
    if (is_causal && cur_pos)
      for (int64_t b = 0; b < B; ++b)
        for (int64_t hh = 0; hh < mh; ++hh)
          for (int64_t j = cur_pos[b] + 1; j < S; ++j)
            if (j >= 0) M[(size_t)((b * mh + hh) * S + j)] = -INFINITY;
    for (Dense *t : {&K, &V})
      for (float &f : *t) f = f != f ? 0.0f : f;   // rows past the position may hold anything: their weight is exactly zero
    Dense sk;
    if (sink) {
      Dense t = load_dense(sink, TTM_BF16, TTM_TILE, 1, H, 32);
      for (int64_t h = 0; h < H; ++h) sk.push_back(t[(size_t)(h * 32)]);
    }
    orc_sdpa_decode_f32(Q.data(), K.data(), V.data(), cur_pos, M.data(), mh, O.data(), B, H, Hk, S, D, is_causal, scale, window < 0 ? -1 : window,
                        sink ? sk.data() : nullptr);
    if (concat_heads) store_dense(O, out, dtype, TTM_TILE, 1, B, H * D);
    else store_dense(O, out, dtype, TTM_TILE, B, H, D);
  });
}
EXPORT int ttm_sdpa_decode(const void *q, const void *k, const void *v, const int32_t *cur_pos, const void *mask, int mask_heads, const int32_t *page_table,
                           int64_t pages_per_user, int64_t page_block, int64_t page_blocks, void *out, int dtype, int64_t batch, int64_t heads,
                           int64_t kv_heads, int64_t seq, int64_t head_dim, int is_causal, float scale, void *) {
  return decode_check(__func__, q, k, v, cur_pos, mask, mask_heads, batch, page_table, pages_per_user, page_block, page_blocks, out, dtype, batch, heads,
                      kv_heads, seq, head_dim, 0, nullptr, is_causal, scale);
}
EXPORT int ttm_sdpa_decode_concat_heads(const void *q, const void *k, const void *v, const int32_t *cur_pos, const void *mask, int mask_heads,
                                        const int32_t *page_table, int64_t pages_per_user, int64_t page_block, int64_t page_blocks, void *out, int dtype,
                                        int64_t batch, int64_t heads, int64_t kv_heads, int64_t seq, int64_t head_dim, int is_causal, float scale, void *) {
  return decode_check(__func__, q, k, v, cur_pos, mask, mask_heads, batch, page_table, pages_per_user, page_block, page_blocks, out, dtype, batch, heads,
                      kv_heads, seq, head_dim, 1, nullptr, is_causal, scale);
}
EXPORT int ttm_sdpa_decode_windowed(const void *q, const void *k, const void *v, const int32_t *cur_pos, const void *mask, int mask_heads, int64_t mask_batch,
                                    const int32_t *page_table, int64_t pages_per_user, int64_t page_block, int64_t page_blocks, void *out, int dtype,
                                    int64_t batch, int64_t heads, int64_t kv_heads, int64_t seq, int64_t head_dim, int is_causal, float scale,
                                    int concat_heads, int64_t sliding_window, const void *attention_sink, void *) {
  return decode_check(__func__, q, k, v, cur_pos, mask, mask_heads, mask_batch, page_table, pages_per_user, page_block, page_blocks, out, dtype, batch,
                      heads, kv_heads, seq, head_dim, concat_heads, attention_sink, is_causal, scale, sliding_window);
}
EXPORT int ttm_sdpa_decode_static(const void *q, const void *k, const void *v, const int32_t *cur_pos, const void *mask, int mask_heads, int64_t mask_batch,
                                  const int32_t *page_table, int64_t pages_per_user, int64_t page_block, int64_t page_blocks, void *out, int dtype,
                                  int64_t batch, int64_t heads, int64_t kv_heads, int64_t seq, int64_t head_dim, int is_causal, float scale,
                                  int concat_heads, int64_t sliding_window, const void *attention_sink, void *) {
  return decode_check(__func__, q, k, v, cur_pos, mask, mask_heads, mask_batch, page_table, pages_per_user, page_block, page_blocks, out, dtype, batch,
                      heads, kv_heads, seq, head_dim, concat_heads, attention_sink, is_causal, scale, sliding_window);
}

// ---- decode path
EXPORT int ttm_rotary_embedding(const void *x, const void *cos_cache, const void *sin_cache, void *out, int dtype, int64_t batch, int64_t rows, int64_t cols,
                                int64_t cache_rows, int64_t token_index, void *) {
  if (batch * rows * cols == 0) return TTM_OK;
  if (token_index >= cache_rows || (token_index < 0 && rows > cache_rows)) return fail("ttm_rotary_embedding: position outside the cos / sin caches");
  EXT(rotary_embedding, x, cos_cache, sin_cache, out, dtype, batch, rows, cols, cache_rows);
  return launch([=] {
    Dense X = load_dense(x, dtype, TTM_TILE, batch, rows, cols), C = load_dense(cos_cache, dtype, TTM_TILE, 1, cache_rows, cols),
          S_ = load_dense(sin_cache, dtype, TTM_TILE, 1, cache_rows, cols), O(X.size());
    orc_rotary_embedding_f32(X.data(), C.data(), S_.data(), O.data(), batch, rows, cols, token_index);
    store_dense(O, out, dtype, TTM_TILE, batch, rows, cols);
  });
}
EXPORT int ttm_rotary_embedding_split_heads(const void *x, const void *cos_cache, const void *sin_cache, void *out, int dtype, int64_t batch, int64_t heads,
                                            int64_t head_dim, int64_t cache_rows, int64_t token_index, void *) {
  if (batch * heads * head_dim == 0) return TTM_OK;
  if (token_index < 0 || token_index >= cache_rows) return fail("ttm_rotary_embedding_split_heads: position outside the cos / sin caches");
  EXT(rotary_embedding_split_heads, x, cos_cache, sin_cache, out, dtype, batch, heads, head_dim, cache_rows);
  return launch([=] {   // [batch, heads * head_dim] row-major is [batch * heads, head_dim] row-major
    Dense X = load_dense(x, dtype, TTM_TILE, 1, batch, heads * head_dim), C = load_dense(cos_cache, dtype, TTM_TILE, 1, cache_rows, head_dim),
          S_ = load_dense(sin_cache, dtype, TTM_TILE, 1, cache_rows, head_dim), O(X.size());
    orc_rotary_embedding_f32(X.data(), C.data(), S_.data(), O.data(), 1, batch * heads, head_dim, token_index);
    store_dense(O, out, dtype, TTM_TILE, batch, heads, head_dim);
  });
}
EXPORT int ttm_rotary_embedding_llama(const void *x, const void *cos_cache, const void *sin_cache, const void *trans_mat, void *out, int dtype, int64_t batch,
                                      int64_t rows, int64_t cols, int64_t cs_batch, int64_t cs_rows, void *) {
  if (batch * rows * cols == 0) return TTM_OK;
  EXT(rotary_embedding_llama, x, cos_cache, sin_cache, trans_mat, out, dtype, batch, rows, cols, cs_batch, cs_rows);
  return launch([=] {   // out = x cos + (x T) sin, T applied to every 32-column tile; f32, one rounding
    Dense X = load_dense(x, dtype, TTM_TILE, batch, rows, cols), C = load_dense(cos_cache, dtype, TTM_TILE, cs_batch, cs_rows, cols),
          S_ = load_dense(sin_cache, dtype, TTM_TILE, cs_batch, cs_rows, cols), T = load_dense(trans_mat, TTM_BF16, TTM_TILE, 1, 32, 32), O(X.size());
    for (int64_t b = 0; b < batch; ++b)
      for (int64_t r = 0; r < rows; ++r)
        for (int64_t c = 0; c < cols; ++c) {
          float rot = 0.0f;
          for (int64_t j = 0; j < 32; ++j) rot += X[(size_t)((b * rows + r) * cols + c / 32 * 32 + j)] * T[(size_t)(j * 32 + c % 32)];
          const size_t cs = (size_t)(((b % cs_batch) * cs_rows + (cs_rows == 1 ? 0 : r)) * cols + c);
          O[(size_t)((b * rows + r) * cols + c)] = X[(size_t)((b * rows + r) * cols + c)] * C[cs] + rot * S_[cs];
        }
    store_dense(O, out, dtype, TTM_TILE, batch, rows, cols);
  });
}
EXPORT int ttm_update_cache(void *cache, const void *input, const int32_t *update_index, int dtype, int64_t users, int64_t heads, int64_t max_seq,
                            int64_t head_dim, int64_t input_users, int64_t batch_offset, void *) {
  if (batch_offset < 0 || batch_offset + input_users > users) return fail("ttm_update_cache: batch_offset + input users exceeds the cache");
  EXT(update_cache, cache, input, update_index, dtype, users, heads, max_seq, head_dim, input_users);
  return launch([=] {
    const int64_t at = *update_index;   // read when the launch runs
    if (at < 0 || at >= max_seq) return;
    for (int64_t b = 0; b < input_users; ++b)
      for (int64_t h = 0; h < heads; ++h)
        for (int64_t d = 0; d < head_dim; ++d)
          store_scalar(cache, dtype, elem_off(TTM_TILE, max_seq, head_dim, (batch_offset + b) * heads + h, at, d),
                       load_scalar(input, dtype, elem_off(TTM_TILE, input_users, head_dim, h, b, d)));
  });
}
EXPORT int ttm_fill_cache(void *cache, const void *input, int dtype, int64_t users, int64_t heads, int64_t max_seq, int64_t head_dim, int64_t seq,
                          int64_t batch_offset, void *) {
  if (batch_offset < 0 || batch_offset >= users || seq > max_seq) return fail("ttm_fill_cache: the input does not fit the cache entry");
  EXT(fill_cache, cache, input, dtype, users, heads, max_seq, head_dim, seq);
  return launch([=] {
    for (int64_t h = 0; h < heads; ++h)
      for (int64_t r = 0; r < pad32(seq) && r < max_seq; ++r)   // the rows up to the next multiple of 32 receive the input's zero padding
        for (int64_t d = 0; d < head_dim; ++d)
          store_scalar(cache, dtype, elem_off(TTM_TILE, max_seq, head_dim, batch_offset * heads + h, r, d),
                       r < seq ? load_scalar(input, dtype, elem_off(TTM_TILE, seq, head_dim, h, r, d)) : 0.0);
  });
}
EXPORT int ttm_paged_update_cache(void *cache, const void *input, const int32_t *update_index, const int32_t *page_table, int dtype, int64_t blocks,
                                  int64_t heads, int64_t block_size, int64_t head_dim, int64_t users, int64_t pages_per_user, int share_cache, void *) {
  EXT(paged_update_cache, cache, input, update_index, page_table, dtype, blocks, heads, block_size, head_dim, users, pages_per_user);
  return launch([=] {
    for (int64_t u = 0; u < users; ++u) {
      const int64_t pos = update_index[u];
      int64_t block, row;
      if (page_table) {
        if (pos < 0 || pos / block_size >= pages_per_user) continue;
        block = page_table[u * pages_per_user + pos / block_size]; row = pos % block_size;
      } else {
        block = share_cache ? 0 : u; row = pos;
      }
      if (pos < 0 || block < 0 || block >= blocks || row >= block_size) continue;
      for (int64_t h = 0; h < heads; ++h)
        for (int64_t d = 0; d < head_dim; ++d)
          store_scalar(cache, dtype, elem_off(TTM_TILE, block_size, head_dim, block * heads + h, row, d),
                       load_scalar(input, dtype, elem_off(TTM_TILE, heads, head_dim, u, h, d)));
    }
  });
}
EXPORT int ttm_paged_fill_cache(void *cache, const void *input, const int32_t *page_table, const int32_t *batch_idx, int dtype, int64_t blocks, int64_t heads,
                                int64_t block_size, int64_t head_dim, int64_t in_batch, int64_t seq, int64_t table_rows, int64_t pages_per_user, void *) {
  EXT(paged_fill_cache, cache, input, page_table, batch_idx, dtype, blocks, heads, block_size, head_dim, in_batch, seq, table_rows, pages_per_user);
  return launch([=] {
    for (int64_t b = 0; b < in_batch; ++b) {
      const int64_t row = batch_idx ? batch_idx[b] : b;
      if (row < 0 || row >= table_rows) continue;
      for (int64_t s_ = 0; s_ < seq; ++s_) {
        if (s_ / block_size >= pages_per_user) continue;
        const int64_t block = page_table[row * pages_per_user + s_ / block_size];
        if (block < 0 || block >= blocks) continue;
        for (int64_t h = 0; h < heads; ++h)
          for (int64_t d = 0; d < head_dim; ++d)
            store_scalar(cache, dtype, elem_off(TTM_TILE, block_size, head_dim, block * heads + h, s_ % block_size, d),
                         load_scalar(input, dtype, elem_off(TTM_TILE, seq, head_dim, b * heads + h, s_, d)));
      }
    }
  });
}
EXPORT int ttm_paged_gather(const void *cache, const int32_t *page_table, void *out, int dtype, int64_t blocks, int64_t heads, int64_t block_size,
                            int64_t head_dim, int64_t users, int64_t pages_per_user, void *) {
  EXT(paged_gather, cache, page_table, out, dtype, blocks, heads, block_size, head_dim, users, pages_per_user);
  return launch([=] {
    const int64_t S = pages_per_user * block_size;
    for (int64_t u = 0; u < users; ++u)
      for (int64_t j = 0; j < S; ++j) {
        const int64_t block = page_table[u * pages_per_user + j / block_size];
        const bool ok = block >= 0 && block < blocks;
        for (int64_t h = 0; h < heads; ++h)
          for (int64_t d = 0; d < head_dim; ++d)
            store_scalar(out, dtype, elem_off(TTM_TILE, S, head_dim, u * heads + h, j, d),
                         ok ? load_scalar(cache, dtype, elem_off(TTM_TILE, block_size, head_dim, block * heads + h, j % block_size, d)) : 0.0);
      }
  });
}
EXPORT int ttm_chunk_causal_mask(void *mask, const int32_t *chunk_start, int64_t rows, int64_t cols, void *) {
  EXT(chunk_causal_mask, mask, chunk_start, rows, cols);
  return launch([=] {
    const int64_t start = *chunk_start;
    memset(mask, 0, (size_t)tile_bytes(TTM_BF16, 1, rows, cols));
    for (int64_t r = 0; r < rows; ++r)
      for (int64_t c = 0; c < cols; ++c) store_scalar(mask, TTM_BF16, elem_off(TTM_TILE, rows, cols, 0, r, c), c <= start + r ? 0.0 : -INFINITY);
  });
}
