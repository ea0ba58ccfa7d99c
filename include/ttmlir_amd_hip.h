/*
 * ttmlir_amd_hip.h -- C ABI of the MI355X (gfx950) kernel library, libttmlir_amd_hip.so.
 *
 * This is the only layer that touches HIP.  The C++ op runners (one per TTNN flatbuffer op
 * table) and any foreign-language binding call these entry points with plain device pointers,
 * sizes and a stream handle.  Each entry point replaces one `::ttnn::*` call made by the
 * tt-mlir TTNN runtime; the citation names that call site (paths relative to the tt-mlir tree).
 *
 * Conventions
 *  - every function returns 0 on success, a TTM_ERR_* code otherwise; ttm_last_error() gives
 *    the thread-local message.  Nothing throws, nothing aborts.
 *  - `stream` is a hipStream_t passed as void* (NULL = the default stream).  Launches are
 *    asynchronous; no entry point synchronises unless its name says so.
 *  - dtype codes are the values of tt::target::DataType (include/ttmlir/Target/Common/types.fbs:19-43),
 *    layout codes those of tt::target::TensorLayout (:65-69).
 *  - TILE layout is physical: a [batch, R, C] tensor is stored as batch * ceil(R/32) * ceil(C/32)
 *    tiles, row-major over tiles, each tile 4 faces of 16x16 (face order (0,0) (0,1) (1,0) (1,1)),
 *    zero padded (lib/Dialect/TTCore/IR/TTCoreOpsTypes.cpp:1857-1903).  Block-float tiles are
 *    1088 B (bfp8_b) / 576 B (bfp4_b): 64 shared-exponent bytes then the mantissas (:1875-1887).
 */
#ifndef TTMLIR_AMD_HIP_H
#define TTMLIR_AMD_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum { TTM_OK = 0, TTM_ERR_INVALID = 1, TTM_ERR_HIP = 2, TTM_ERR_UNSUPPORTED = 3 };

enum {
  TTM_F32 = 0, TTM_F16 = 1, TTM_BF16 = 2, TTM_BFP8B = 4, TTM_BFP4B = 6,
  TTM_U32 = 9, TTM_U16 = 10, TTM_U8 = 11, TTM_I32 = 12
};
enum { TTM_ROW_MAJOR = 0, TTM_TILE = 1 };

/* activation fused after bias (activation strings "gelu"/"silu"/"sigmoid"/"relu",
 * lib/Dialect/TTNN/Transforms/TTNNFusing.cpp:155-159) */
enum { TTM_ACT_NONE = 0, TTM_ACT_GELU = 1, TTM_ACT_SILU = 2, TTM_ACT_SIGMOID = 3, TTM_ACT_RELU = 4 };

const char *ttm_last_error(void);

/* ---- device, memory, streams, events: the plumbing under openMeshDevice / to_device /
 * from_device / wait (runtime/lib/ttnn/runtime.cpp:582-624, 824-853;
 * runtime/lib/ttnn/types/layout_converter.cpp:54-64) */
int ttm_device_count(int *count);
int ttm_set_device(int device);
int ttm_device_name(char *buf, size_t len);
int ttm_mem_info(size_t *free_bytes, size_t *total_bytes);
int ttm_malloc(void **dptr, size_t bytes);
int ttm_free(void *dptr);
int ttm_host_alloc(void **hptr, size_t bytes); /* pinned */
int ttm_host_free(void *hptr);
int ttm_memcpy_h2d(void *dst, const void *src, size_t bytes, void *stream);
int ttm_memcpy_d2h(void *dst, const void *src, size_t bytes, void *stream);
int ttm_memcpy_d2d(void *dst, const void *src, size_t bytes, void *stream);
int ttm_fill_u32(void *dst, uint32_t value, size_t count, void *stream); /* fill kernel, graph safe */
int ttm_stream_create(void **stream);
int ttm_stream_destroy(void *stream);
int ttm_stream_sync(void *stream);
int ttm_device_sync(void);
int ttm_event_create(void **event);
int ttm_event_destroy(void *event);
int ttm_event_record(void *event, void *stream);
int ttm_event_sync(void *event);
int ttm_event_elapsed_ms(float *ms, void *start, void *stop);

/* Plain 16-byte-per-lane device copy kernel: the measured HBM ceiling the layout kernels are
 * compared with, and the calibration kernel for FETCH_SIZE / WRITE_SIZE counters. */
int ttm_copy_kernel(const void *src, void *dst, size_t bytes, void *stream);

/* ---- tilize / untilize: ::ttnn::to_layout(TILE | ROW_MAJOR)
 * (runtime/lib/ttnn/operations/layout/to_layout.cpp:12-38, types/layout_converter.cpp:35-45,
 * runtime/lib/ttnn/runtime.cpp:164-235).  Pure permutation, bit exact.  src is row-major
 * [batch, rows, cols] (tilize) or tiled (untilize); elem_bytes in {1, 2, 4}. */
int ttm_tilize(const void *src, void *dst, int64_t batch, int64_t rows, int64_t cols, int elem_bytes,
               void *stream);
int ttm_untilize(const void *src, void *dst, int64_t batch, int64_t rows, int64_t cols, int elem_bytes,
                 void *stream);

/* ---- block-float pack / unpack: ::ttnn::typecast to / from BFLOAT8_B, BFLOAT4_B
 * (runtime/lib/ttnn/operations/layout/typecast.cpp:14-31, types/layout_converter.cpp:47-52,
 * host readback runtime/lib/ttnn/runtime.cpp:450-466).  fmt is TTM_BFP8B or TTM_BFP4B.
 * The plain-dtype side is TTM_F32 or TTM_BF16 in TTM_ROW_MAJOR (tilize fused) or TTM_TILE. */
int64_t ttm_bfp_tile_bytes(int fmt);
int ttm_bfp_pack(const void *src, int src_dtype, int src_layout, void *dst, int fmt, int64_t batch,
                 int64_t rows, int64_t cols, void *stream);
int ttm_bfp_unpack(const void *src, int fmt, void *dst, int dst_dtype, int dst_layout, int64_t batch,
                   int64_t rows, int64_t cols, void *stream);

/* ---- matmul / linear: ::ttnn::matmul, ::ttnn::linear
 * (runtime/lib/ttnn/operations/matmul/matmul.cpp:47-83, 86-125; semantics
 * include/ttmlir/Dialect/TTIR/IR/TTIROps.td:5169-5290).
 * out[b] = act(a[b] . w[b or 0] + bias), fp32 accumulation.  Every operand is in TILE layout:
 * a [batch, M, K] BFloat16; w [w_batch, K, N] BFloat16, BFP_BFloat8 or BFP_BFloat4 packed tiles
 * (transpose_w: w holds [w_batch, N, K], BFloat16 only); bias BFloat16 [N] either TILE (a [1,N]
 * tensor padded to 32 rows) or ROW_MAJOR, may be NULL; out [batch, M, N] BFloat16.
 * w_batch is 1 (weights shared by every batch entry) or equal to batch.  act is TTM_ACT_*,
 * applied after the bias (tools/golden/mapping.py:7792-7796). */
int ttm_linear(const void *a, int a_dtype, const void *w, int w_dtype, int transpose_w, const void *bias,
               int bias_dtype, int bias_layout, void *out, int out_dtype, int64_t batch, int64_t w_batch,
               int64_t M, int64_t N, int64_t K, int act, void *stream);

/* Kernel-variant selection for measurement (name -> small integer); unknown names fail. */
int ttm_set_option(const char *name, int value);
int ttm_get_option(const char *name, int *value);

#ifdef __cplusplus
}
#endif
#endif
