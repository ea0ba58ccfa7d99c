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
 *  - the entry points take logical extents and no buffer sizes: a TILE operand or result of logical
 *    shape [batch, R, C] must be backed by the whole padded tensor, batch * ceil(R/32) * ceil(C/32)
 *    tiles, and the kernels read and write all of it (a [1, C] tensor is one full tile row of 32
 *    rows).  A buffer sized for the logical extents alone is read and written past its end.
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

/* ---- HIP graphs, the device side of trace capture / replay (ttnn begin_trace_capture / end_trace_capture /
 * execute_trace as called from runtime/lib/ttnn/operations/trace/{begin_trace_capture,end_trace_capture,
 * execute_trace}.cpp).  Between begin and end every launch made through this library on `stream` is recorded, not run;
 * end returns an executable graph (and the number of recorded nodes) that ttm_graph_launch replays with one launch.
 * Recorded launches name their operand addresses: the caller keeps those allocations alive and in place until
 * ttm_graph_destroy.  Host transfers and synchronisation are not legal on a capturing stream. */
int ttm_graph_begin_capture(void *stream);
int ttm_graph_end_capture(void *stream, void **graph_exec, size_t *num_nodes);
int ttm_graph_launch(void *graph_exec, void *stream);
int ttm_graph_destroy(void *graph_exec);
int ttm_stream_is_capturing(void *stream, int *capturing);

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
/* ttm_linear followed by one element-wise op with a second BFloat16 TILE tensor of the output's shape, in the same pass:
 * out = round(round(act(a w + bias)) (+ | *) tail).  This is what the executor calls for a MatmulOp / LinearOp whose only
 * consumer is the next `add` (residual connection) or `multiply` (SiLU(gate) * up, runtime/lib/ttnn/operations/eltwise/
 * binary/binary.cpp:38-126); both roundings are kept so that the result equals the two ops run one after the other. */
#define TTM_TAIL_NONE 0
#define TTM_TAIL_ADD 1
#define TTM_TAIL_MUL 2
int ttm_linear_tail(const void *a, int a_dtype, const void *w, int w_dtype, int transpose_w, const void *bias, int bias_dtype,
                    int bias_layout, void *out, int out_dtype, int64_t batch, int64_t w_batch, int64_t M, int64_t N,
                    int64_t K, int act, int tail_op, const void *tail, void *stream);
/* out0 = a w0 and out1 = a w1 in one launch, for two weight tensors of one shape and format applied to the same activations
 * (the K and V projections of an attention layer); the two weight tensors and the two outputs may live anywhere.  No bias,
 * activation or tail.  One launch fills the device where two small ones would each leave part of it idle. */
/* Up to four block-float weight matrices [K, N_i] (one dtype, any widths) applied to the same activations in one launch,
 * each with its own output [M, N_i] and its own activation (act[i], TTM_ACT_*; NULL = none): the Q, K and V projections
 * of an attention layer, or the gate and up projections of an MLP at token counts where one of them alone would not
 * fill the device.  No bias or tail.  Results are those of separate ttm_linear calls up to the accumulation order the
 * launch plan implies. */
int ttm_linear_group(const void *a, int n, const void *const *w, int w_dtype, void *const *out, const int64_t *N,
                     const int *act, int64_t M, int64_t K, void *stream);
int ttm_linear_pair(const void *a, const void *w0, const void *w1, int w_dtype, void *out0, void *out1, int64_t M, int64_t N,
                    int64_t K, void *stream);
/* out = round(round(act_gate(a w_gate)) * round(act_up(a w_up))) in one launch: the gate and up projections of an MLP and the
 * multiply that joins them (SiLU(gate) * up).  a [M, K] and out [M, N] are bf16 tiles, the two weight matrices block-float
 * [K, N] of one format.  Two forms: for M <= 32 rows (a decode step) a workgroup of the decode kernel streams the same 64
 * columns of both matrices; for 65 <= M <= 1024 rows and BFP_BFloat8 weights a block of the fused main kernel takes four
 * column tiles of each matrix instead of eight of one.  Either way the activations pass through a CU once for both and the
 * two results meet in registers; the three bf16 roundings of the op sequence are kept and the result is bit-identical to
 * ttm_linear (act_gate) + ttm_linear_tail (act_up, TTM_TAIL_MUL) on the same kernel, which is what it replaces
 * (runtime/lib/ttnn/operations/matmul/matmul.cpp:47-83, eltwise/binary/binary.cpp:38-126).
 * ttm_linear_glu_supported returns 1 when the shapes and the selected kernel variants allow it, else 0: block-float weights,
 * M <= 32 and enough columns that one projection alone would not split K over workgroups; or BFP_BFloat8 weights,
 * 65 <= M <= 1024 and a shape at which the library's cost model puts this launch ahead of the grouped projections followed
 * by a multiply (narrow weight matrices, which are cheap to rewrite as bf16 images first, stay with that sequence). */
int ttm_linear_glu_supported(int w_dtype, int64_t M, int64_t N, int64_t K);
int ttm_linear_glu(const void *a, const void *w_gate, const void *w_up, int w_dtype, void *out, int64_t M, int64_t N, int64_t K,
                   int act_gate, int act_up, void *stream);
/* x1 = residual + a w and norm_out = rms_norm(x1) * norm_weight + norm_bias for M <= 32 rows in two launches (the output
 * projection of a decode step's attention block with its residual connection and the RMSNorm in front of the MLP):
 * the projection leaves fp32 partial sums and the RMSNorm kernel starts from them.  a [M, K], residual, sum_out (receives x1)
 * and norm_out [M, N] are bf16 tiles, w block-float [K, N]; norm_weight / norm_bias [N] bf16 in the given layout, or NULL.
 * Bit-identical to ttm_linear_tail(.., TTM_TAIL_ADD, residual) followed by ttm_rms_norm (runtime/lib/ttnn/operations/
 * matmul/matmul.cpp:47-83, eltwise/binary/binary.cpp:38-126, normalization/rms_norm.cpp:10-49).
 * ttm_linear_add_rms_norm_supported returns 1 when the shapes and the selected kernel variants allow it, else 0. */
int ttm_linear_add_rms_norm_supported(int w_dtype, int64_t M, int64_t N, int64_t K);
int ttm_linear_add_rms_norm(const void *a, const void *w, int w_dtype, const void *residual, void *sum_out, const void *norm_weight,
                            int weight_layout, const void *norm_bias, int bias_layout, float eps, void *norm_out, int64_t M, int64_t N,
                            int64_t K, void *stream);
/* The front of a decode step's attention block in two launches: the Q, K and V projections of `users` <= 32 tokens (one
 * per user, activations a [users, K] bf16 tiles, block-float weights [K, heads * head_dim] and twice
 * [K, kv_heads * head_dim]), then in one kernel the head split, the rotary embedding of q and k with row `token_index` of
 * the cos / sin caches ([1, 1, cache_rows, head_dim] bf16 tiles), q written as [1, users, heads, head_dim] bf16 tiles and k
 * and v written into their caches [cache_users, kv_heads, max_seq, head_dim] at row *update_index (device memory; out of
 * range writes nothing) of users batch_offset .. batch_offset + users - 1.  It replaces, with bit-identical results, the
 * op sequence matmul x 3 -> reshape -> RotaryEmbeddingOp x 2 -> permute -> UpdateCacheOp x 2 of a decode layer
 * (test/ttmlir/models/single_blocks_and_layers/llama_3_8b_decode_layer.mlir:51-82; runtime/lib/ttnn/operations/matmul/
 * matmul.cpp:47-83, transformer/rotary_embedding.cpp:14-31, kv_cache/update_cache.cpp:14-55).
 * ttm_linear_qkv_decode_supported returns 1 when the shapes and the selected kernel variant allow it, else 0. */
int ttm_linear_qkv_decode_supported(int w_dtype, int64_t users, int64_t K, int64_t heads, int64_t kv_heads, int64_t head_dim);
int ttm_linear_qkv_decode(const void *a, const void *wq, const void *wk, const void *wv, int w_dtype, int64_t users, int64_t K,
                          int64_t heads, int64_t kv_heads, int64_t head_dim, const void *cos_cache, const void *sin_cache,
                          int64_t cache_rows, int64_t token_index, void *q_out, void *k_cache, void *v_cache, int64_t cache_users,
                          int64_t max_seq, const int32_t *update_index, int64_t batch_offset, void *stream);

/* ---- elementwise: ::ttnn::<unary>, ::ttnn::<binary>
 * (runtime/lib/ttnn/operations/eltwise/unary/unary.cpp:159-205, eltwise/binary/binary.cpp:38-126;
 * CPU lowering lib/Conversion/TTIRToLinalg/EltwiseUnary.cpp:251-326).  `op` is the value of
 * EltwiseUnaryOpType / EltwiseBinaryOpType (include/ttmlir/Target/TTNN/operations/eltwise.fbs).
 * fp32 math, result stored in `dtype` (TTM_BF16 or TTM_F32).  Unary takes a [batch, rows, cols]
 * tensor in `layout`.  Binary broadcasts numpy-style: the three shapes have `rank` entries (<= 8);
 * `layout` is the layout of all three tensors.  The zero padding of TILE tensors is preserved. */
int ttm_eltwise_unary(int op, const void *in, void *out, int dtype, int layout, int64_t batch, int64_t rows,
                      int64_t cols, float param, void *stream);
int ttm_eltwise_binary(int op, const void *a, const int64_t *a_shape, const void *b, const int64_t *b_shape,
                       void *out, const int64_t *out_shape, int rank, int dtype, int layout, void *stream);
/* ttm_eltwise_unary also takes 100 + EltwiseUnaryCompositeOpType for Cbrt (100) and Log1p (103)
 * (runtime/lib/ttnn/operations/eltwise/unary/unary_composite.cpp:104-135); ClampScalar is ttm_clamp: min(max(x, lo), hi),
 * NaN kept (golden tools/golden/mapping.py:5267-5276, torch.clamp). */
int ttm_clamp(const void *in, void *out, int dtype, int layout, int64_t batch, int64_t rows, int64_t cols, float lo, float hi,
              void *stream);
/* ttm_eltwise_binary also takes 100 + EltwiseBinaryCompositeOpType for Maximum, Minimum, Remainder, Pow and Atan2
 * (runtime/lib/ttnn/operations/eltwise/binary/binary_composite.cpp; goldens tools/golden/mapping.py:4493-4570, 5516-5530:
 * torch.maximum / minimum (NaN propagates), torch.remainder (sign of the divisor), torch.pow, torch.atan2).
 *
 * ttm_where: ::ttnn::where(first, second, third) (runtime/lib/ttnn/operations/eltwise/ternary/where.cpp:14-33; golden
 * tools/golden/mapping.py:5579-5586, torch.where): out = cond != 0 ? a : b, the three operands broadcasting numpy-style
 * to the output (rank <= 4), all four tensors in `dtype` (BFloat16 or Float32) and `layout`.  Values move as bits. */
int ttm_where(const void *cond, const int64_t *cond_shape, const void *a, const int64_t *a_shape, const void *b,
              const int64_t *b_shape, void *out, const int64_t *out_shape, int rank, int dtype, int layout, void *stream);

/* ---- index-driven ops of a decoder layer's head and tail, ROW_MAJOR on both sides.
 * ttm_embedding: ::ttnn::embedding (runtime/lib/ttnn/operations/embedding/embedding.cpp:14-43; golden
 *   tools/golden/mapping.py:2900-2912): out[r, :] = weight[clamp(indices[r], 0, vocab - 1), :]; indices Int32 / UInt32,
 *   weight [vocab, dim] and out [rows, dim] of `elem_bytes`-byte elements.
 * ttm_argmax: ::ttnn::argmax over the last dim (operations/reduction/argmax.cpp:14-28; golden mapping.py:5222-5265,
 *   torch.argmax): out[r] = index of the first largest element of row r of in [rows, cols] (NaN counts as largest).
 * ttm_arange: ::ttnn::arange (operations/creation/arange.cpp:14-42; golden mapping.py:4269-4290): out[i] = start + i * step
 *   formed in fp32 and cast to `dtype` (Float32, BFloat16, Int32, UInt32), n = ceil((end - start) / step) elements. */
int ttm_embedding(const void *indices, int index_dtype, const void *weight, void *out, int elem_bytes, int64_t rows,
                  int64_t vocab, int64_t dim, void *stream);
int ttm_argmax(const void *in, int dtype, int32_t *out, int64_t rows, int64_t cols, void *stream);
int ttm_arange(void *out, int dtype, int64_t n, double start, double step, void *stream);

/* ---- typecast between plain dtypes: ::ttnn::typecast
 * (runtime/lib/ttnn/operations/layout/typecast.cpp:14-31).  Layout is preserved, so n counts the
 * (padded) elements.  Float -> integer truncates toward zero and saturates; integer narrowing
 * saturates (runtime/include/tt/runtime/utils.h:26-150). */
int ttm_typecast(const void *in, int src_dtype, void *out, int dst_dtype, int64_t n, void *stream);

/* ---- row-wise ops on TILE tensors [batch, rows, cols], reduced over the last dim, fp32 math.
 * rms_norm: ::ttnn::rms_norm (runtime/lib/ttnn/operations/normalization/rms_norm.cpp:10-49;
 *   op order lib/Dialect/TTIR/Transforms/DecomposeComposites.cpp:47-111); weight / bias are [cols]
 *   vectors of the same dtype, TILE (a [1,cols] tensor) or ROW_MAJOR, may be NULL.  A ROW_MAJOR vector is read in
 *   16-byte chunks up to the next multiple of 32 elements (what lies past cols is never used): its allocation must
 *   reach that far, as every allocation of at least 128-byte granularity does.
 * softmax: ::ttnn::softmax over the last dim, always max-subtracted
 *   (normalization/softmax.cpp:12-36; lib/Conversion/TTIRToLinalg/TTIRToLinalg.cpp:944-1017).
 * reduce: ::ttnn::sum/mean/max/min over the last dim (reduction/reduction.cpp:13-63); op is
 *   ReductionOpType; the result is the TILE tensor [batch, rows, 1]. */
int ttm_rms_norm(const void *x, const void *weight, int weight_layout, const void *bias, int bias_layout,
                 void *out, int dtype, int64_t batch, int64_t rows, int64_t cols, float eps, void *stream);
int ttm_softmax_lastdim(const void *x, void *out, int dtype, int64_t batch, int64_t rows, int64_t cols,
                        void *stream);
int ttm_reduce_lastdim(int op, const void *x, void *out, int dtype, int64_t batch, int64_t rows, int64_t cols,
                       void *stream);

/* ---- generic data movement: reshape / permute / transpose / slice / concat / repeat_interleave
 * (runtime/lib/ttnn/operations/data_movement/ *.cpp).  A view of `rank` extents maps view index v to
 * the logical linear index src_base + sum v[d]*src_stride[d] of the source and likewise of the
 * destination; logical indices are row-major over [batch, rows, cols] and converted to the
 * layout of each tensor.  Padding of a TILE destination is not written. */
int ttm_copy_view(const void *src, int64_t src_rows, int64_t src_cols, int src_layout, void *dst,
                  int64_t dst_rows, int64_t dst_cols, int dst_layout, int elem_bytes, int rank,
                  const int64_t *extent, const int64_t *src_stride, int64_t src_base,
                  const int64_t *dst_stride, int64_t dst_base, void *stream);
/* ttm_copy_view whose destination base is advanced by a position held in DEVICE memory (read by the kernel, so the
 * launch can be recorded into a graph): dst_base + *index * index_stride; an *index outside [0, index_limit) writes
 * nothing.  With dst = a KV cache [users, heads, max_seq, head_dim], index_stride = head_dim and index_limit = max_seq
 * this is ::ttnn::update_cache (runtime/lib/ttnn/operations/kv_cache/update_cache.cpp:14-60) reading its input through a
 * view, i.e. with the permute / reshape that produces the [1, heads, users, head_dim] operand folded in. */
int ttm_copy_view_at(const void *src, int64_t src_rows, int64_t src_cols, int src_layout, void *dst,
                     int64_t dst_rows, int64_t dst_cols, int dst_layout, int elem_bytes, int rank,
                     const int64_t *extent, const int64_t *src_stride, int64_t src_base,
                     const int64_t *dst_stride, int64_t dst_base, const int32_t *index, int64_t index_stride,
                     int64_t index_limit, void *stream);

/* ---- attention: ::ttnn::transformer::scaled_dot_product_attention
 * (runtime/lib/ttnn/operations/transformer/scaled_dot_product_attention.cpp:14-55; golden
 * tools/golden/mapping.py:8398-8500).  q [B,Hq,Sq,D], k/v [B,Hkv,Sk,D], out [B,Hq,Sq,D], all
 * BFloat16 TILE; query head h reads kv head h / (Hq/Hkv); mask is additive BFloat16 TILE
 * [B,mask_heads,Sq,Sk] (mask_heads 1 or Hq) or NULL; is_causal masks key > query; scale <= 0
 * means 1/sqrt(D); softmax in fp32. */
int ttm_sdpa(const void *q, const void *k, const void *v, const void *mask, int mask_heads, void *out, int dtype,
             int64_t B, int64_t Hq, int64_t Hkv, int64_t Sq, int64_t Sk, int64_t D, int is_causal, float scale,
             void *stream);
/* ttm_sdpa on operands that keep their heads side by side, as the projections leave them and the output projection
 * wants them: heads_inner bit 0: q is [B, Sq, Hq * D]; bit 1: k is [B, Sk, Hkv * D]; bit 2: v likewise; bit 3: out is
 * [B, Sq, Hq * D].  Both layouts hold the same 32 x 32 tiles in another order, so the head split (reshape + permute in
 * front, or ::ttnn::transformer::split_query_key_value_and_split_heads) and the head merge (permute + reshape behind, or
 * ::ttnn::transformer::concatenate_heads, runtime/lib/ttnn/operations/transformer/concatenate_heads.cpp) cost nothing. */
int ttm_sdpa_heads_inner(const void *q, const void *k, const void *v, const void *mask, int mask_heads, void *out,
                         int dtype, int64_t B, int64_t Hq, int64_t Hkv, int64_t Sq, int64_t Sk, int64_t D, int is_causal,
                         float scale, int heads_inner, void *stream);
/* ttm_sdpa_heads_inner with the two remaining attributes of the op (include/ttmlir/Target/TTNN/operations/transformer.fbs:
 * 70-82; runtime/lib/ttnn/operations/transformer/scaled_dot_product_attention.cpp:33-45; golden tools/golden/mapping.py:
 * 8450-8494).  sliding_window >= 0: query i sees key j only when 0 <= i - j < sliding_window under is_causal, and when
 * |i - j| <= sliding_window / 2 otherwise; < 0: no window.  A mask, when given as well, is added on top; it is
 * [mask_batch, mask_heads, Sq, Sk] with mask_batch 1 (shared by the batch) or B (TTNNOps.td:4273-4275).  Key tiles
 * wholly outside the window are neither read nor multiplied.  attention_sink: [1, Hq, 1, 1] BFloat16 in TILE layout (one
 * tile per head) or null; per head one more logit, sink * scale, that takes part in the softmax and has no value row (the
 * kernel applies the scale to the sink as to the scores, which is what the compiler's lowering compensates for,
 * lib/Conversion/TTIRToTTNN/TTIRToTTNN.cpp:3507-3533).  A query that sees no key gives a row of zeros. */
int ttm_sdpa_windowed(const void *q, const void *k, const void *v, const void *mask, int mask_heads, int64_t mask_batch,
                      void *out, int dtype, int64_t B, int64_t Hq, int64_t Hkv, int64_t Sq, int64_t Sk, int64_t D, int is_causal, float scale,
                      int heads_inner, int64_t sliding_window, const void *attention_sink, void *stream);

/* ---- decode path: rotary embedding, KV-cache writes, attention of one new token over the cache.  TILE layout
 * throughout; positions (update index, current position, page table) are Int32 / UInt32 values in DEVICE memory, read
 * by the kernels, so the launches can be recorded into a graph and replayed with new positions.
 *
 * ttm_rotary_embedding: ::ttnn::experimental::rotary_embedding (runtime/lib/ttnn/operations/transformer/
 *   rotary_embedding.cpp:14-31; formula include/ttmlir/Dialect/TTNN/IR/TTNNOps.td:4002-4016 and
 *   test/python/golden/ttir_ops/fusing/test_rope_fusing.py:24-33): out = x * cos + rotate_half(x) * sin with
 *   rotate_half(x) = concat(-x[D/2:], x[:D/2]).  x / out [batch, rows, cols], cos / sin [cache_rows, cols], BFloat16 or
 *   Float32; row s uses cache row s, or cache row token_index for every row when token_index >= 0 (decode mode).
 * ttm_update_cache: ::ttnn::update_cache (operations/kv_cache/update_cache.cpp:14-60; golden tools/golden/mapping.py:
 *   3614-3671): cache[batch_offset + b, h, *update_index, :] = input[0, h, b, :] for b < input_users; cache
 *   [users, heads, max_seq, head_dim], input [1, heads, input_users, head_dim]; an index outside [0, max_seq) writes nothing.
 * ttm_fill_cache: ::ttnn::fill_cache (operations/kv_cache/fill_cache.cpp:12-18; golden mapping.py:3582-3611):
 *   cache[batch_offset, :, 0:seq, :] = input[0, :, :, :], input [1, heads, seq, head_dim]; the rows up to the next
 *   multiple of 32 receive the input's tile padding (zeros), as in the golden.
 * ttm_sdpa_decode: ::ttnn::transformer::scaled_dot_product_attention_decode and its paged form
 *   (operations/transformer/scaled_dot_product_attention_decode.cpp, paged_scaled_dot_product_attention_decode.cpp;
 *   golden mapping.py:2417-2481): q / out [1, batch, heads, head_dim]; k / v [batch, kv_heads, seq, head_dim], or with a
 *   page table [batch, pages_per_user] pages [blocks, kv_heads, page_block, head_dim] where seq = pages_per_user *
 *   page_block and page_blocks = blocks (page-table entries outside [0, page_blocks), e.g. -1 in an unused slot, mask the
 *   keys of that page instead of being followed); BFloat16.  scores = (q k^T + mask) * scale, mask additive BFloat16 [batch, 1, mask_heads, seq] or NULL;
 *   with is_causal and cur_pos [batch] keys after cur_pos[b] are excluded; scale <= 0 means 1/sqrt(head_dim); softmax in
 *   fp32.  Uses the stream's workspace for per-slice partial results.  Up to 8 query heads per kv head are served by one
 *   launch; more (multi-query attention) by several launches over the same cache.
 * ttm_paged_update_cache: ::ttnn::experimental::paged_update_cache (operations/kv_cache/paged_update_cache.cpp:14-57;
 *   shapes lib/Dialect/TTNN/IR/TTNNOps.cpp:4719-4820; golden tools/golden/mapping.py:8926-8963): cache
 *   [blocks, heads, block_size, head_dim], input [1, users, heads, head_dim], update_index [users], page_table
 *   [users, pages_per_user] or NULL.  cache[page_table[u, p / block_size], h, p % block_size, :] = input[0, u, h, :] with
 *   p = update_index[u]; without a page table the cache is [users, heads, max_seq, head_dim] and user u writes entry u
 *   (entry 0 when share_cache).  Positions, pages and blocks out of range write nothing (the golden clamps them).
 * ttm_paged_fill_cache: ::ttnn::experimental::paged_fill_cache (operations/kv_cache/paged_fill_cache.cpp; golden
 *   mapping.py:8966-9008): input [in_batch, heads, seq, head_dim], page_table [table_rows, pages_per_user], batch_idx
 *   [in_batch] or NULL (then row b).  cache[page_table[row(b), s / block_size], h, s % block_size, :] = input[b, h, s, :]. */
int ttm_rotary_embedding(const void *x, const void *cos_cache, const void *sin_cache, void *out, int dtype, int64_t batch,
                         int64_t rows, int64_t cols, int64_t cache_rows, int64_t token_index, void *stream);
/* The head split in front of the rotary embedding folded in: x is the [batch, heads * head_dim] TILE matrix a projection
 * leaves, out is [batch, heads, head_dim] (= [1, batch, heads, head_dim]) TILE with zero padding rows; decode mode only
 * (token_index >= 0), since rows are heads here. */
int ttm_rotary_embedding_split_heads(const void *x, const void *cos_cache, const void *sin_cache, void *out, int dtype,
                                     int64_t batch, int64_t heads, int64_t head_dim, int64_t cache_rows, int64_t token_index,
                                     void *stream);
int ttm_update_cache(void *cache, const void *input, const int32_t *update_index, int dtype, int64_t users, int64_t heads,
                     int64_t max_seq, int64_t head_dim, int64_t input_users, int64_t batch_offset, void *stream);
int ttm_paged_update_cache(void *cache, const void *input, const int32_t *update_index, const int32_t *page_table, int dtype,
                           int64_t blocks, int64_t heads, int64_t block_size, int64_t head_dim, int64_t users,
                           int64_t pages_per_user, int share_cache, void *stream);
int ttm_paged_fill_cache(void *cache, const void *input, const int32_t *page_table, const int32_t *batch_idx, int dtype,
                         int64_t blocks, int64_t heads, int64_t block_size, int64_t head_dim, int64_t in_batch, int64_t seq,
                         int64_t table_rows, int64_t pages_per_user, void *stream);
int ttm_fill_cache(void *cache, const void *input, int dtype, int64_t users, int64_t heads, int64_t max_seq,
                   int64_t head_dim, int64_t seq, int64_t batch_offset, void *stream);
int ttm_sdpa_decode(const void *q, const void *k, const void *v, const int32_t *cur_pos, const void *mask, int mask_heads,
                    const int32_t *page_table, int64_t pages_per_user, int64_t page_block, int64_t page_blocks, void *out, int dtype,
                    int64_t batch, int64_t heads, int64_t kv_heads, int64_t seq, int64_t head_dim, int is_causal,
                    float scale, void *stream);
/* ttm_sdpa_decode whose output already has its heads concatenated: out is the [batch, heads * head_dim] TILE matrix that
 * ::ttnn::experimental::nlp_concat_heads_decode (runtime/lib/ttnn/operations/transformer/nlp_concat_heads_decode.cpp) or
 * a reshape would make of [1, batch, heads, head_dim]; padding rows below the last user are written as zeros. */
int ttm_sdpa_decode_concat_heads(const void *q, const void *k, const void *v, const int32_t *cur_pos, const void *mask,
                                 int mask_heads, const int32_t *page_table, int64_t pages_per_user, int64_t page_block,
                                 int64_t page_blocks, void *out, int dtype, int64_t batch, int64_t heads, int64_t kv_heads, int64_t seq,
                                 int64_t head_dim, int is_causal, float scale, void *stream);
/* ttm_sdpa_decode / ttm_sdpa_decode_concat_heads (concat_heads = 0 / 1) with the op's sliding_window_size and
 * attention_sink (runtime/lib/ttnn/operations/transformer/scaled_dot_product_attention_decode.cpp:36-50,
 * paged_scaled_dot_product_attention_decode.cpp:36-50; include/ttmlir/Dialect/TTNN/IR/TTNNOps.td:4109-4137).
 * sliding_window >= 0: only the last sliding_window keys up to the decode position p are visible, keys
 * [max(0, p - sliding_window + 1), p] (golden tools/golden/mapping.py:8814-8824), p = cur_pos[b], or seq - 1 without
 * cur_pos; the cache in front of the window is not read.  attention_sink: [heads, 32] BFloat16 in TILE layout, column 0,
 * or null; one more logit per head, sink * scale, in the softmax, without a value row.  mask: [mask_batch, 1, mask_heads,
 * seq] with mask_batch 1 (shared by the users) or batch (TTNNOps.td:4123-4125). */
int ttm_sdpa_decode_windowed(const void *q, const void *k, const void *v, const int32_t *cur_pos, const void *mask,
                             int mask_heads, int64_t mask_batch, const int32_t *page_table, int64_t pages_per_user,
                             int64_t page_block, int64_t page_blocks, void *out, int dtype, int64_t batch, int64_t heads, int64_t kv_heads,
                             int64_t seq, int64_t head_dim, int is_causal, float scale, int concat_heads, int64_t sliding_window,
                             const void *attention_sink, void *stream);

/* ---- chunked prefill over a paged cache: ::ttnn::transformer::chunked_scaled_dot_product_attention
 * (runtime/lib/ttnn/operations/transformer/chunked_scaled_dot_product_attention.cpp; golden tools/golden/mapping.py:8847-8913)
 * is three launches: ttm_paged_gather brings the pages of every user into a contiguous [users, heads, pages_per_user *
 * block_size, head_dim] TILE tensor (cache [blocks, heads, block_size, head_dim], page_table [users, pages_per_user] in
 * device memory; entries outside [0, blocks) read as zeros), ttm_chunk_causal_mask writes the additive BFloat16 TILE mask
 * [rows, cols] of a chunk whose first query stands at position *chunk_start (device memory): 0 where col <= *chunk_start +
 * row, -inf elsewhere, and ttm_sdpa_windowed attends with that mask.  Nothing is read on the host, so the op can be
 * recorded into a graph and replayed with another chunk_start.
 *
 * ttm_rotary_embedding_llama: ::ttnn::experimental::rotary_embedding_llama (runtime/lib/ttnn/operations/transformer/
 * rotary_embedding_llama.cpp:11-34; operand shapes lib/Dialect/TTNN/IR/TTNNOps.cpp:6293-6380): out = x * cos + (x T) * sin
 * with the 32 x 32 BFloat16 TILE matrix T applied to every 32-column tile of a row; x / out [batch, rows, cols], cos / sin
 * [cs_batch, cs_rows, cols] broadcast over batch (entry b % cs_batch) and, when cs_rows is 1, over rows. */
int ttm_paged_gather(const void *cache, const int32_t *page_table, void *out, int dtype, int64_t blocks, int64_t heads,
                     int64_t block_size, int64_t head_dim, int64_t users, int64_t pages_per_user, void *stream);
int ttm_chunk_causal_mask(void *mask, const int32_t *chunk_start, int64_t rows, int64_t cols, void *stream);
int ttm_rotary_embedding_llama(const void *x, const void *cos_cache, const void *sin_cache, const void *trans_mat, void *out,
                               int dtype, int64_t batch, int64_t rows, int64_t cols, int64_t cs_batch, int64_t cs_rows, void *stream);

/* ttm_sdpa_decode_windowed that allocates nothing.  It has no counterpart in the reference; it is for callers that cannot
 * call hipMalloc: code under HIP graph capture, tight serving loops, harnesses that forbid allocation.  Same arguments, same
 * kernels and bit-identical results; the per-slice partial results (max, sum, unnormalised output) go to a static device
 * array of 8 MiB that the library holds on every GPU it runs on until the process ends, instead of the stream's grow-only
 * workspace.  A call whose partial results need more (batch * kv_heads * slices * min(heads / kv_heads, 8) * (head_dim + 2)
 * floats; the config-5 decode shape of 32 users x 8 kv heads x 2048 positions takes 1 MiB) fails with TTM_ERR_INVALID and
 * launches nothing.  No hipMalloc, hipFree or allocating library call is made; the first call on a device looks the
 * array's address up (hipGetSymbolAddress), so make that call outside a capture.  All calls on one GPU share the array:
 * calls that overlap in time on one GPU (different streams) race; calls on one stream are ordered and safe. */
int ttm_sdpa_decode_static(const void *q, const void *k, const void *v, const int32_t *cur_pos, const void *mask,
                           int mask_heads, int64_t mask_batch, const int32_t *page_table, int64_t pages_per_user,
                           int64_t page_block, int64_t page_blocks, void *out, int dtype, int64_t batch, int64_t heads, int64_t kv_heads,
                           int64_t seq, int64_t head_dim, int is_causal, float scale, int concat_heads, int64_t sliding_window,
                           const void *attention_sink, void *stream);

/* Kernel-variant selection for measurement (name -> small integer); unknown names fail. */
int ttm_set_option(const char *name, int value);
int ttm_get_option(const char *name, int *value);

#ifdef __cplusplus
}
#endif
#endif
