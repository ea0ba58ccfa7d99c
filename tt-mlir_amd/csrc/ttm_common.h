// Shared helpers of the gfx950 kernel library: error reporting, launch checks, tile addressing.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

#include "ttmlir_amd_hip.h"
#include "ttm_extents.h"

// native clang vectors (usable with the nontemporal load/store builtins)
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

#define TTM_EXPORT extern "C" __attribute__((visibility("default")))

int ttm_set_error(int code, const char *fmt, ...) __attribute__((format(printf, 2, 3)));

#define TTM_HIP(expr)                                                                          \
  do {                                                                                         \
    hipError_t _e = (expr);                                                                    \
    if (_e != hipSuccess)                                                                      \
      return ttm_set_error(TTM_ERR_HIP, "%s failed: %s (%s:%d)", #expr, hipGetErrorString(_e), \
                           __FILE__, __LINE__);                                                \
  } while (0)

#define TTM_REQUIRE(cond, ...)                                        \
  do {                                                                \
    if (!(cond)) return ttm_set_error(TTM_ERR_INVALID, __VA_ARGS__);  \
  } while (0)

#define TTM_LAUNCH_CHECK() TTM_HIP(hipGetLastError())

int ttm_option(const char *name);  // 0 when unset

// Opt-in host-side check of operand extents (option "check_extents", or TTMLIR_AMD_CHECK_EXTENTS=1 in the environment):
// before anything is launched, the bytes the kernels touch behind every pointer argument (ttm_extents.h) must lie inside
// one device allocation (hipMemGetAddressRange); otherwise the entry point returns TTM_ERR_INVALID with the operand, the
// bytes it has and the bytes the kernels touch in the message, where the launch would have been a GPU memory fault.
bool ttm_check_extents_on();
struct TtmExtentChecker {
  const char *fn;
  int operator()(const char *what, const void *p, int64_t bytes, bool optional) const;
};
#define TTM_EXTENTS(rule, ...)                                                                               \
  do {                                                                                                       \
    if (ttm_check_extents_on())                                                                              \
      if (int rc_ = ttm_extents::rule(TtmExtentChecker{__func__}, __VA_ARGS__)) return rc_;                  \
  } while (0)
#define TTM_EXTENTS_SPAN(what, p, bytes)                                                                     \
  do {                                                                                                       \
    if (ttm_check_extents_on())                                                                              \
      if (int rc_ = TtmExtentChecker{__func__}(what, p, bytes, false)) return rc_;                           \
  } while (0)
// source and destination of a strided view (ttm_copy_view); `extra` is the largest offset added to the destination base
#define TTM_EXTENTS_VIEW(src, srows, scols, slay, dst, drows, dcols, dlay, elem, rank, extent, sstride, sbase, dstride, dbase, extra)     \
  do {                                                                                                                                     \
    if (ttm_check_extents_on()) {                                                                                                          \
      bool neg_ = false;                                                                                                                   \
      int rc_ = ttm_extents::view(TtmExtentChecker{__func__}, "source", src, srows, scols, slay, elem, rank, extent, sstride, sbase, 0, &neg_); \
      if (!rc_ && !neg_)                                                                                                                   \
        rc_ = ttm_extents::view(TtmExtentChecker{__func__}, "destination", dst, drows, dcols, dlay, elem, rank, extent, dstride, dbase, extra, &neg_); \
      if (neg_) return ttm_set_error(TTM_ERR_INVALID, "out of bounds: %s: the view reaches a negative logical offset", __func__);          \
      if (rc_) return rc_;                                                                                                                 \
    }                                                                                                                                      \
  } while (0)

// Streaming kernels run fastest with a bounded number of bytes in flight per CU (64 - 96 KiB measured on MI355X): more
// resident wavefronts than that only lengthen the queues in front of the memory channels.  TTM_MAX_WAVES(n) caps a
// kernel's wavefronts per SIMD (= 256-lane workgroups per CU) at n; n may depend on template parameters, 8 is no cap.
#define TTM_MAX_WAVES(n) __attribute__((amdgpu_waves_per_eu((n) < 8 ? (n) : 1, (n))))

// Scratch memory of a stream for kernels that need device memory beyond their operands (split-K partial sums).
// One grow-only allocation per (device, stream): launches on a stream are ordered, so consecutive users do not overlap.
// Growing allocates with hipMalloc and is refused while the stream is capturing; an allocation that a captured graph may
// have recorded is never freed before the stream is destroyed.
int ttm_stream_workspace(hipStream_t stream, size_t bytes, void **ptr);

// RMSNorm that starts from the fp32 partial sums of a split-K projection of one row tile plus a residual (ttm_rowwise.hip)
bool ttm_rowwise_partials_supported(int64_t rows, int64_t cols);
int ttm_rowwise_rmsnorm_from_partials(const float *partial, int slices, int64_t per, const void *residual, void *sum_out,
                                      const void *weight, int weight_layout, const void *bias, int bias_layout, void *out,
                                      int64_t rows, int64_t cols, float eps, hipStream_t s);

__host__ __device__ static inline int64_t ttm_round_up32(int64_t v) { return (v + 31) / 32 * 32; }
static inline int64_t ttm_cdiv(int64_t a, int64_t b) { return (a + b - 1) / b; }

static inline int ttm_dtype_bytes(int dtype) {
  switch (dtype) {
  case TTM_F32: case TTM_U32: case TTM_I32: return 4;
  case TTM_F16: case TTM_BF16: case TTM_U16: return 2;
  case TTM_U8: return 1;
  default: return 0;
  }
}

// One element of a rotary embedding, x cos + rot(x) sin with rot(x) = sign * partner: two products and a sum, each rounded
// to fp32 (the arithmetic of the CPU path's separate multiply and add ops; no fused multiply-add)
__device__ __forceinline__ float ttm_rotary_value(float x, float partner, float c, float s, float sign) {
#pragma clang fp contract(off)
  const float a = x * c, b = (sign * partner) * s;
  return a + b;
}

// Element offset of (r, c) inside a tiled [Rt*32, Ct*32] matrix: tiles row-major, faces
// (0,0) (0,1) (1,0) (1,1), 16 contiguous elements per face row.
__host__ __device__ static inline int64_t ttm_tiled_offset(int64_t r, int64_t c, int64_t ct) {
  int64_t tile = (r >> 5) * ct + (c >> 5);
  int face = (int)(((r >> 4) & 1) * 2 + ((c >> 4) & 1));
  return tile * 1024 + face * 256 + (r & 15) * 16 + (c & 15);
}

// Maximum and minimum that return NaN when either operand is NaN (one v_maximum3_f32 / v_minimum3_f32 on gfx950), as
// tosa.reduce_max / arith.maximumf of the CPU lowering and torch.max do; fmaxf / fminf return the other operand.
__device__ __forceinline__ float ttm_max(float a, float b) { return __builtin_elementwise_maximum(a, b); }
__device__ __forceinline__ float ttm_min(float a, float b) { return __builtin_elementwise_minimum(a, b); }

__device__ static inline float ttm_bf16_to_f32(uint16_t h) { return __uint_as_float((uint32_t)h << 16); }
// f32 -> bf16, round to nearest even (v_cvt_pk_bf16_f32 on gfx950; NaN stays a quiet NaN)
typedef __bf16 ttm_bf16x2 __attribute__((ext_vector_type(2)));
typedef float ttm_f32x2 __attribute__((ext_vector_type(2)));
__device__ static inline uint32_t ttm_pack_bf16x2(float lo, float hi) {
  ttm_f32x2 v = {lo, hi};
  ttm_bf16x2 h = __builtin_convertvector(v, ttm_bf16x2);
  return *(uint32_t *)&h;
}
__device__ static inline uint16_t ttm_f32_to_bf16(float f) { return (uint16_t)(ttm_pack_bf16x2(f, 0.0f) & 0xFFFFu); }
