// The bytes every entry point of include/ttmlir_amd_hip.h touches behind each pointer argument, in one place.  The entry
// points take logical extents and no buffer sizes: a TILE operand of logical shape [batch, R, C] is read and written as
// batch * ceil(R / 32) * ceil(C / 32) whole tiles, whatever R and C are.  A caller that sized a buffer for the logical
// extents alone gets a GPU memory fault, not an error return.  These rules let a host-side check refuse such a call before
// anything is launched: the kernel library applies them when the option "check_extents" is set (each range must lie inside
// one device allocation), and a host stand-in for the library can apply them against its own registry of allocations.
//
// One function per entry point, named after it.  `span(what, ptr, bytes, optional)` is the checker: it returns 0 when
// `bytes` bytes from `ptr` on are accessible (or ptr is null and optional), else an error code that the rule returns at once.
// Plain host C++, no HIP.
#pragma once
#include <stdint.h>

#include "ttmlir_amd_hip.h"

namespace ttm_extents {

inline int64_t pad32(int64_t n) { return (n + 31) / 32 * 32; }
inline int64_t elem_bytes(int dtype) {
  switch (dtype) {
  case TTM_F32: case TTM_U32: case TTM_I32: return 4;
  case TTM_F16: case TTM_BF16: case TTM_U16: return 2;
  case TTM_U8: return 1;
  default: return 0;
  }
}
// bytes of a [batch, rows, cols] TILE tensor of a plain or block-float type
inline int64_t tile_bytes(int dtype, int64_t batch, int64_t rows, int64_t cols) {
  const int64_t tiles = batch * (pad32(rows) / 32) * (pad32(cols) / 32);
  if (dtype == TTM_BFP8B) return tiles * 1088;
  if (dtype == TTM_BFP4B) return tiles * 576;
  return tiles * 1024 * elem_bytes(dtype);
}
inline int64_t tensor_bytes(int dtype, int layout, int64_t batch, int64_t rows, int64_t cols) {
  return layout == TTM_TILE ? tile_bytes(dtype, batch, rows, cols) : batch * rows * cols * elem_bytes(dtype);
}
// a [cols] weight / bias vector: one tile row in TILE layout; a ROW_MAJOR vector is read in 16-byte chunks up to the next
// multiple of 32 elements
inline int64_t vec_bytes(int dtype, int layout, int64_t cols) {
  return layout == TTM_TILE ? tile_bytes(dtype, 1, 1, cols) : cols * elem_bytes(dtype);
}
// a [.., rows, cols] shape of `rank` entries as (batch, rows, cols); rank 1 is one row
inline void split3(const int64_t *shape, int rank, int64_t &b, int64_t &r, int64_t &c) {
  b = 1; r = 1; c = 1;
  if (rank >= 1) c = shape[rank - 1];
  if (rank >= 2) r = shape[rank - 2];
  for (int i = 0; i + 2 < rank; ++i) b *= shape[i];
}
template <class Span>
int shaped(Span &&span, const char *what, const void *p, const int64_t *shape, int rank, int dtype, int layout) {
  if (!shape) return span(what, nullptr, 1, false);   // reported as a null operand
  int64_t b, r, c;
  split3(shape, rank, b, r, c);
  return span(what, p, tensor_bytes(dtype, layout, b, r, c), false);
}
// strided view over a tensor whose last two dims are [rows, cols]: the tensor must hold every matrix up to the one the
// largest logical offset lies in.  Returns -1 through `negative` when the view reaches below offset 0.
template <class Span>
int view(Span &&span, const char *what, const void *p, int64_t rows, int64_t cols, int layout, int elem, int rank, const int64_t *extent,
         const int64_t *stride, int64_t base, int64_t extra_max, bool *negative) {
  int64_t lo = base, hi = base + extra_max;
  *negative = false;
  for (int i = 0; i < rank; ++i) {
    if (extent[i] <= 0) return 0;   // empty view
    const int64_t d = (extent[i] - 1) * stride[i];
    if (d >= 0) hi += d; else lo += d;
  }
  if (lo < 0) { *negative = true; return 0; }
  const int64_t per = rows * cols, mats = per > 0 ? hi / per + 1 : 0;
  const int64_t bytes = layout == TTM_TILE ? mats * pad32(rows) * pad32(cols) * elem : (hi + 1) * elem;
  return span(what, p, bytes, false);
}

#define TTM_EXT(call) do { if (int rc_ = (call)) return rc_; } while (0)

template <class Span> int copy_kernel(Span &&span, const void *src, void *dst, size_t bytes) {
  TTM_EXT(span("source", src, (int64_t)bytes, false)); TTM_EXT(span("destination", dst, (int64_t)bytes, false));
  return 0;
}
template <class Span> int tilize(Span &&span, const void *src, void *dst, int64_t batch, int64_t rows, int64_t cols, int elem) {
  if (batch * rows * cols == 0) return 0;
  TTM_EXT(span("row-major input", src, batch * rows * cols * elem, false));
  TTM_EXT(span("tile output", dst, batch * pad32(rows) * pad32(cols) * elem, false));
  return 0;
}
template <class Span> int untilize(Span &&span, const void *src, void *dst, int64_t batch, int64_t rows, int64_t cols, int elem) {
  if (batch * rows * cols == 0) return 0;
  TTM_EXT(span("tile input", src, batch * pad32(rows) * pad32(cols) * elem, false));
  TTM_EXT(span("row-major output", dst, batch * rows * cols * elem, false));
  return 0;
}
template <class Span>
int bfp_pack(Span &&span, const void *src, int src_dtype, int src_layout, void *dst, int fmt, int64_t batch, int64_t rows, int64_t cols) {
  if (batch * rows * cols == 0) return 0;
  TTM_EXT(span("input", src, tensor_bytes(src_dtype, src_layout, batch, rows, cols), false));
  TTM_EXT(span("block-float output", dst, tile_bytes(fmt, batch, rows, cols), false));
  return 0;
}
template <class Span>
int bfp_unpack(Span &&span, const void *src, int fmt, void *dst, int dst_dtype, int dst_layout, int64_t batch, int64_t rows, int64_t cols) {
  if (batch * rows * cols == 0) return 0;
  TTM_EXT(span("block-float input", src, tile_bytes(fmt, batch, rows, cols), false));
  TTM_EXT(span("output", dst, tensor_bytes(dst_dtype, dst_layout, batch, rows, cols), false));
  return 0;
}
template <class Span> int typecast(Span &&span, const void *in, int src_dtype, void *out, int dst_dtype, int64_t n) {
  if (n == 0) return 0;
  TTM_EXT(span("input", in, n * elem_bytes(src_dtype), false)); TTM_EXT(span("output", out, n * elem_bytes(dst_dtype), false));
  return 0;
}
template <class Span>
int linear(Span &&span, const void *a, int a_dtype, const void *w, int w_dtype, const void *bias, int bias_dtype, int bias_layout, void *out,
           int out_dtype, int64_t batch, int64_t w_batch, int64_t M, int64_t N, int64_t K, int tail_op, const void *tail) {
  if (batch * M * N == 0) return 0;
  TTM_EXT(span("activations [batch, M, K]", a, tile_bytes(a_dtype, batch, M, K), false));
  TTM_EXT(span("weights [w_batch, K, N]", w, tile_bytes(w_dtype, w_batch, K, N), false));
  TTM_EXT(span("bias", bias, vec_bytes(bias_dtype, bias_layout, N), true));
  TTM_EXT(span("output [batch, M, N]", out, tile_bytes(out_dtype, batch, M, N), false));
  if (tail_op != TTM_TAIL_NONE) TTM_EXT(span("tail operand [batch, M, N]", tail, tile_bytes(TTM_BF16, batch, M, N), false));
  return 0;
}
template <class Span>
int linear_group(Span &&span, const void *a, int n, const void *const *w, int w_dtype, void *const *out, const int64_t *N, int64_t M, int64_t K) {
  TTM_EXT(span("activations [M, K]", a, tile_bytes(TTM_BF16, 1, M, K), false));
  for (int i = 0; i < n; ++i) {
    TTM_EXT(span("weights [K, N_i]", w[i], tile_bytes(w_dtype, 1, K, N[i]), false));
    TTM_EXT(span("output [M, N_i]", out[i], tile_bytes(TTM_BF16, 1, M, N[i]), false));
  }
  return 0;
}
template <class Span>
int linear_pair(Span &&span, const void *a, const void *w0, const void *w1, int w_dtype, void *out0, void *out1, int64_t M, int64_t N, int64_t K) {
  TTM_EXT(span("activations [M, K]", a, tile_bytes(TTM_BF16, 1, M, K), false));
  TTM_EXT(span("weights 0", w0, tile_bytes(w_dtype, 1, K, N), false)); TTM_EXT(span("weights 1", w1, tile_bytes(w_dtype, 1, K, N), false));
  TTM_EXT(span("output 0", out0, tile_bytes(TTM_BF16, 1, M, N), false)); TTM_EXT(span("output 1", out1, tile_bytes(TTM_BF16, 1, M, N), false));
  return 0;
}
template <class Span>
int linear_glu(Span &&span, const void *a, const void *w_gate, const void *w_up, int w_dtype, void *out, int64_t M, int64_t N, int64_t K) {
  TTM_EXT(span("activations [M, K]", a, tile_bytes(TTM_BF16, 1, M, K), false));
  TTM_EXT(span("gate weights [K, N]", w_gate, tile_bytes(w_dtype, 1, K, N), false));
  TTM_EXT(span("up weights [K, N]", w_up, tile_bytes(w_dtype, 1, K, N), false));
  TTM_EXT(span("output [M, N]", out, tile_bytes(TTM_BF16, 1, M, N), false));
  return 0;
}
template <class Span>
int linear_add_rms_norm(Span &&span, const void *a, const void *w, int w_dtype, const void *residual, void *sum_out, const void *norm_weight,
                        int weight_layout, const void *norm_bias, int bias_layout, void *norm_out, int64_t M, int64_t N, int64_t K) {
  TTM_EXT(span("activations [M, K]", a, tile_bytes(TTM_BF16, 1, M, K), false));
  TTM_EXT(span("weights [K, N]", w, tile_bytes(w_dtype, 1, K, N), false));
  TTM_EXT(span("residual [M, N]", residual, tile_bytes(TTM_BF16, 1, M, N), false));
  TTM_EXT(span("sum output [M, N]", sum_out, tile_bytes(TTM_BF16, 1, M, N), false));
  TTM_EXT(span("norm output [M, N]", norm_out, tile_bytes(TTM_BF16, 1, M, N), false));
  TTM_EXT(span("norm weight", norm_weight, vec_bytes(TTM_BF16, weight_layout, N), true));
  TTM_EXT(span("norm bias", norm_bias, vec_bytes(TTM_BF16, bias_layout, N), true));
  return 0;
}
template <class Span>
int linear_qkv_decode(Span &&span, const void *a, const void *wq, const void *wk, const void *wv, int w_dtype, int64_t users, int64_t K, int64_t heads,
                      int64_t kv_heads, int64_t head_dim, const void *cos_cache, const void *sin_cache, int64_t cache_rows, void *q_out,
                      void *k_cache, void *v_cache, int64_t cache_users, int64_t max_seq, const int32_t *update_index) {
  TTM_EXT(span("activations [users, K]", a, tile_bytes(TTM_BF16, 1, users, K), false));
  TTM_EXT(span("q weights", wq, tile_bytes(w_dtype, 1, K, heads * head_dim), false));
  TTM_EXT(span("k weights", wk, tile_bytes(w_dtype, 1, K, kv_heads * head_dim), false));
  TTM_EXT(span("v weights", wv, tile_bytes(w_dtype, 1, K, kv_heads * head_dim), false));
  TTM_EXT(span("cos cache", cos_cache, tile_bytes(TTM_BF16, 1, cache_rows, head_dim), false));
  TTM_EXT(span("sin cache", sin_cache, tile_bytes(TTM_BF16, 1, cache_rows, head_dim), false));
  TTM_EXT(span("q output [1, users, heads, head_dim]", q_out, tile_bytes(TTM_BF16, users, heads, head_dim), false));
  TTM_EXT(span("k cache", k_cache, tile_bytes(TTM_BF16, cache_users * kv_heads, max_seq, head_dim), false));
  TTM_EXT(span("v cache", v_cache, tile_bytes(TTM_BF16, cache_users * kv_heads, max_seq, head_dim), false));
  TTM_EXT(span("update index", update_index, 4, false));
  return 0;
}
template <class Span>
int unary(Span &&span, const void *in, void *out, int dtype, int layout, int64_t batch, int64_t rows, int64_t cols) {
  if (batch * rows * cols == 0) return 0;
  TTM_EXT(span("input", in, tensor_bytes(dtype, layout, batch, rows, cols), false));
  TTM_EXT(span("output", out, tensor_bytes(dtype, layout, batch, rows, cols), false));
  return 0;
}
template <class Span>
int binary(Span &&span, const void *a, const int64_t *a_shape, const void *b, const int64_t *b_shape, void *out, const int64_t *out_shape, int rank,
           int dtype, int layout) {
  TTM_EXT(shaped(span, "left operand", a, a_shape, rank, dtype, layout));
  TTM_EXT(shaped(span, "right operand", b, b_shape, rank, dtype, layout));
  TTM_EXT(shaped(span, "output", out, out_shape, rank, dtype, layout));
  return 0;
}
template <class Span>
int where(Span &&span, const void *cond, const int64_t *cond_shape, const void *a, const int64_t *a_shape, const void *b, const int64_t *b_shape,
          void *out, const int64_t *out_shape, int rank, int dtype, int layout) {
  TTM_EXT(shaped(span, "condition", cond, cond_shape, rank, dtype, layout));
  TTM_EXT(shaped(span, "first operand", a, a_shape, rank, dtype, layout));
  TTM_EXT(shaped(span, "second operand", b, b_shape, rank, dtype, layout));
  TTM_EXT(shaped(span, "output", out, out_shape, rank, dtype, layout));
  return 0;
}
template <class Span>
int embedding(Span &&span, const void *indices, const void *weight, void *out, int elem, int64_t rows, int64_t vocab, int64_t dim) {
  if (rows * dim == 0) return 0;
  TTM_EXT(span("indices", indices, rows * 4, false)); TTM_EXT(span("weight [vocab, dim]", weight, vocab * dim * elem, false));
  TTM_EXT(span("output [rows, dim]", out, rows * dim * elem, false));
  return 0;
}
template <class Span> int argmax(Span &&span, const void *in, int dtype, int32_t *out, int64_t rows, int64_t cols) {
  if (rows * cols == 0) return 0;
  TTM_EXT(span("input [rows, cols]", in, rows * cols * elem_bytes(dtype), false)); TTM_EXT(span("output [rows]", out, rows * 4, false));
  return 0;
}
template <class Span> int arange(Span &&span, void *out, int dtype, int64_t n) {
  if (n == 0) return 0;
  return span("output", out, n * elem_bytes(dtype), false);
}
template <class Span>
int rms_norm(Span &&span, const void *x, const void *weight, int weight_layout, const void *bias, int bias_layout, void *out, int dtype, int64_t batch,
             int64_t rows, int64_t cols) {
  if (batch * rows * cols == 0) return 0;
  TTM_EXT(span("input", x, tile_bytes(dtype, batch, rows, cols), false)); TTM_EXT(span("output", out, tile_bytes(dtype, batch, rows, cols), false));
  TTM_EXT(span("weight", weight, vec_bytes(dtype, weight_layout, cols), true)); TTM_EXT(span("bias", bias, vec_bytes(dtype, bias_layout, cols), true));
  return 0;
}
template <class Span> int softmax(Span &&span, const void *x, void *out, int dtype, int64_t batch, int64_t rows, int64_t cols) {
  if (batch * rows * cols == 0) return 0;
  TTM_EXT(span("input", x, tile_bytes(dtype, batch, rows, cols), false)); TTM_EXT(span("output", out, tile_bytes(dtype, batch, rows, cols), false));
  return 0;
}
template <class Span> int reduce(Span &&span, const void *x, void *out, int dtype, int64_t batch, int64_t rows, int64_t cols) {
  if (batch * rows * cols == 0) return 0;
  TTM_EXT(span("input", x, tile_bytes(dtype, batch, rows, cols), false));
  TTM_EXT(span("output [.., rows, 1]", out, tile_bytes(dtype, batch, rows, 1), false));
  return 0;
}
template <class Span>
int sdpa(Span &&span, const void *q, const void *k, const void *v, const void *mask, int mask_heads, int64_t mask_batch, void *out, int dtype, int64_t B,
         int64_t Hq, int64_t Hkv, int64_t Sq, int64_t Sk, int64_t D, const void *sink) {
  if (B * Hq * Sq * D == 0) return 0;
  // heads side by side or heads as matrices: the same tiles in another order, the same bytes (D is a multiple of 32)
  TTM_EXT(span("q", q, tile_bytes(dtype, B * Hq, Sq, D), false));
  TTM_EXT(span("k", k, tile_bytes(dtype, B * Hkv, Sk, D), false));
  TTM_EXT(span("v", v, tile_bytes(dtype, B * Hkv, Sk, D), false));
  TTM_EXT(span("mask", mask, tile_bytes(dtype, mask_batch * mask_heads, Sq, Sk), true));
  TTM_EXT(span("attention sink", sink, tile_bytes(TTM_BF16, Hq, 1, 1), true));
  TTM_EXT(span("output", out, tile_bytes(dtype, B * Hq, Sq, D), false));
  return 0;
}
template <class Span>
int sdpa_decode(Span &&span, const void *q, const void *k, const void *v, const int32_t *cur_pos, const void *mask, int mask_heads, int64_t mask_batch,
                const int32_t *page_table, int64_t pages_per_user, int64_t page_block, int64_t page_blocks, void *out, int dtype, int64_t batch,
                int64_t heads, int64_t kv_heads, int64_t seq, int64_t head_dim, int concat_heads, const void *sink) {
  if (batch * heads * head_dim == 0) return 0;
  TTM_EXT(span("q [1, batch, heads, head_dim]", q, tile_bytes(dtype, batch, heads, head_dim), false));
  const int64_t kv = page_table ? tile_bytes(dtype, page_blocks * kv_heads, page_block, head_dim) : tile_bytes(dtype, batch * kv_heads, seq, head_dim);
  TTM_EXT(span("k", k, kv, false));
  TTM_EXT(span("v", v, kv, false));
  TTM_EXT(span("cur_pos", cur_pos, batch * 4, true));
  TTM_EXT(span("mask [mask_batch, 1, mask_heads, seq]", mask, tile_bytes(dtype, mask_batch, mask_heads, seq), true));
  TTM_EXT(span("page table", page_table, batch * pages_per_user * 4, true));
  TTM_EXT(span("attention sink [heads, 32]", sink, tile_bytes(TTM_BF16, 1, heads, 32), true));
  TTM_EXT(span("output", out, concat_heads ? tile_bytes(dtype, 1, batch, heads * head_dim) : tile_bytes(dtype, batch, heads, head_dim), false));
  return 0;
}
template <class Span>
int rotary_embedding(Span &&span, const void *x, const void *cos_cache, const void *sin_cache, void *out, int dtype, int64_t batch, int64_t rows,
                     int64_t cols, int64_t cache_rows) {
  if (batch * rows * cols == 0) return 0;
  TTM_EXT(span("input", x, tile_bytes(dtype, batch, rows, cols), false)); TTM_EXT(span("output", out, tile_bytes(dtype, batch, rows, cols), false));
  TTM_EXT(span("cos cache", cos_cache, tile_bytes(dtype, 1, cache_rows, cols), false));
  TTM_EXT(span("sin cache", sin_cache, tile_bytes(dtype, 1, cache_rows, cols), false));
  return 0;
}
template <class Span>
int rotary_embedding_split_heads(Span &&span, const void *x, const void *cos_cache, const void *sin_cache, void *out, int dtype, int64_t batch,
                                 int64_t heads, int64_t head_dim, int64_t cache_rows) {
  if (batch * heads * head_dim == 0) return 0;
  TTM_EXT(span("input [batch, heads * head_dim]", x, tile_bytes(dtype, 1, batch, heads * head_dim), false));
  TTM_EXT(span("output [batch, heads, head_dim]", out, tile_bytes(dtype, batch, heads, head_dim), false));
  TTM_EXT(span("cos cache", cos_cache, tile_bytes(dtype, 1, cache_rows, head_dim), false));
  TTM_EXT(span("sin cache", sin_cache, tile_bytes(dtype, 1, cache_rows, head_dim), false));
  return 0;
}
template <class Span>
int rotary_embedding_llama(Span &&span, const void *x, const void *cos_cache, const void *sin_cache, const void *trans_mat, void *out, int dtype,
                           int64_t batch, int64_t rows, int64_t cols, int64_t cs_batch, int64_t cs_rows) {
  if (batch * rows * cols == 0) return 0;
  TTM_EXT(span("input", x, tile_bytes(dtype, batch, rows, cols), false)); TTM_EXT(span("output", out, tile_bytes(dtype, batch, rows, cols), false));
  TTM_EXT(span("cos", cos_cache, tile_bytes(dtype, cs_batch, cs_rows, cols), false));
  TTM_EXT(span("sin", sin_cache, tile_bytes(dtype, cs_batch, cs_rows, cols), false));
  TTM_EXT(span("transformation matrix", trans_mat, tile_bytes(TTM_BF16, 1, 32, 32), false));
  return 0;
}
template <class Span>
int update_cache(Span &&span, void *cache, const void *input, const int32_t *update_index, int dtype, int64_t users, int64_t heads, int64_t max_seq,
                 int64_t head_dim, int64_t input_users) {
  TTM_EXT(span("cache", cache, tile_bytes(dtype, users * heads, max_seq, head_dim), false));
  TTM_EXT(span("input [1, heads, users, head_dim]", input, tile_bytes(dtype, heads, input_users, head_dim), false));
  TTM_EXT(span("update index", update_index, 4, false));
  return 0;
}
template <class Span>
int fill_cache(Span &&span, void *cache, const void *input, int dtype, int64_t users, int64_t heads, int64_t max_seq, int64_t head_dim, int64_t seq) {
  TTM_EXT(span("cache", cache, tile_bytes(dtype, users * heads, max_seq, head_dim), false));
  TTM_EXT(span("input [1, heads, seq, head_dim]", input, tile_bytes(dtype, heads, seq, head_dim), false));
  return 0;
}
template <class Span>
int paged_update_cache(Span &&span, void *cache, const void *input, const int32_t *update_index, const int32_t *page_table, int dtype, int64_t blocks,
                       int64_t heads, int64_t block_size, int64_t head_dim, int64_t users, int64_t pages_per_user) {
  TTM_EXT(span("cache", cache, tile_bytes(dtype, blocks * heads, block_size, head_dim), false));
  TTM_EXT(span("input [1, users, heads, head_dim]", input, tile_bytes(dtype, users, heads, head_dim), false));
  TTM_EXT(span("update index [users]", update_index, users * 4, false));
  TTM_EXT(span("page table", page_table, users * pages_per_user * 4, true));
  return 0;
}
template <class Span>
int paged_fill_cache(Span &&span, void *cache, const void *input, const int32_t *page_table, const int32_t *batch_idx, int dtype, int64_t blocks,
                     int64_t heads, int64_t block_size, int64_t head_dim, int64_t in_batch, int64_t seq, int64_t table_rows, int64_t pages_per_user) {
  TTM_EXT(span("cache", cache, tile_bytes(dtype, blocks * heads, block_size, head_dim), false));
  TTM_EXT(span("input [in_batch, heads, seq, head_dim]", input, tile_bytes(dtype, in_batch * heads, seq, head_dim), false));
  TTM_EXT(span("page table", page_table, table_rows * pages_per_user * 4, false));
  TTM_EXT(span("batch index", batch_idx, in_batch * 4, true));
  return 0;
}
template <class Span>
int paged_gather(Span &&span, const void *cache, const int32_t *page_table, void *out, int dtype, int64_t blocks, int64_t heads, int64_t block_size,
                 int64_t head_dim, int64_t users, int64_t pages_per_user) {
  TTM_EXT(span("cache", cache, tile_bytes(dtype, blocks * heads, block_size, head_dim), false));
  TTM_EXT(span("page table", page_table, users * pages_per_user * 4, false));
  TTM_EXT(span("output", out, tile_bytes(dtype, users * heads, pages_per_user * block_size, head_dim), false));
  return 0;
}
template <class Span> int chunk_causal_mask(Span &&span, void *mask, const int32_t *chunk_start, int64_t rows, int64_t cols) {
  TTM_EXT(span("mask [rows, cols]", mask, tile_bytes(TTM_BF16, 1, rows, cols), false));
  TTM_EXT(span("chunk start", chunk_start, 4, false));
  return 0;
}

#undef TTM_EXT
}  // namespace ttm_extents
