// Decode-path transformer kernels: rotary embedding, KV-cache update / fill, single-token attention over a KV cache.
// All tensors are TILE layout (32 x 32 tiles of four 16 x 16 faces); every kernel here is bound by HBM bandwidth.
#include <mutex>

#include "ttm_common.h"

namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4v __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));

// 8 consecutive elements <-> 8 floats
__device__ __forceinline__ void load8(const uint16_t *p, float *v) {
  const u32x4 r = *(const u32x4 *)p;
  const uint32_t w[4] = {r.x, r.y, r.z, r.w};
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    v[2 * j] = __uint_as_float(w[j] << 16);
    v[2 * j + 1] = __uint_as_float(w[j] & 0xFFFF0000u);
  }
}
__device__ __forceinline__ void load8(const float *p, float *v) {
  const f32x4 a = *(const f32x4 *)p, b = *(const f32x4 *)(p + 4);
  v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w; v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
}
__device__ __forceinline__ void store8(uint16_t *p, const float *v) {
  u32x4 r;
  r.x = ttm_pack_bf16x2(v[0], v[1]);
  r.y = ttm_pack_bf16x2(v[2], v[3]);
  r.z = ttm_pack_bf16x2(v[4], v[5]);
  r.w = ttm_pack_bf16x2(v[6], v[7]);
  *(u32x4 *)p = r;
}
__device__ __forceinline__ void store8(float *p, const float *v) {
  *(f32x4 *)p = f32x4{v[0], v[1], v[2], v[3]};
  *(f32x4 *)(p + 4) = f32x4{v[4], v[5], v[6], v[7]};
}

// ------------------------------------------------------------------------------------------------ rotary embedding
// out[b, s, d] = x[b, s, d] * cos[r, d] + rot(x)[b, s, d] * sin[r, d],  rot(x)[d] = d < D/2 ? -x[d + D/2] : x[d - D/2],
// r = token_index when given, else s.  One thread per 8 consecutive columns of a face row: the partner columns
// d +- D/2 are 8 consecutive elements of another face row because D/2 is a multiple of 16.
// src_cols > 0: x is not laid out like `out` but is the [batch, rows * cols] matrix a projection leaves (row b holds
// the `rows` heads of user b side by side); the head split [batch, rows * cols] -> [batch, rows, cols] happens on the
// way in and the padding rows of `out` are written as zeros.
template <typename T>
__global__ __launch_bounds__(256) void ttm_rotary_k(const T *__restrict__ x, const T *__restrict__ cosc,
                                                    const T *__restrict__ sinc, T *__restrict__ out, int64_t rows_pad,
                                                    int64_t cols, int64_t per_batch, int64_t total8, int64_t token_index,
                                                    int64_t rows, int64_t src_cols) {
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= total8) return;
  const int64_t ct = cols >> 5, half = cols >> 1;
  const int64_t e = i * 8, b = e / per_batch, o = e % per_batch;
  // o -> (row, col) of the tiled [rows_pad, cols] matrix
  const int64_t tile = o >> 10;
  const int in = (int)(o & 1023), face = in >> 8, fr = (in >> 4) & 15, fc = in & 15;
  const int64_t r = (tile / ct) * 32 + (face >> 1) * 16 + fr, c = (tile % ct) * 32 + (face & 1) * 16 + fc;
  const int64_t cr = token_index >= 0 ? token_index : r;
  const int64_t pc = c < half ? c + half : c - half;
  const float sign = c < half ? -1.0f : 1.0f;
  const T *xp = x + b * per_batch;
  const int64_t co = ttm_tiled_offset(cr, c, ct);
  float xv[8], pv[8], cv[8], sv[8], ov[8];
  if (src_cols > 0) {
    if (r >= rows) {
#pragma unroll
      for (int j = 0; j < 8; ++j) ov[j] = 0.0f;
      store8(out + b * per_batch + o, ov);
      return;
    }
    load8(x + ttm_tiled_offset(b, r * cols + c, src_cols >> 5), xv);
    load8(x + ttm_tiled_offset(b, r * cols + pc, src_cols >> 5), pv);
  } else {
    load8(xp + o, xv);
    load8(xp + ttm_tiled_offset(r, pc, ct), pv);
  }
  load8(cosc + co, cv);
  load8(sinc + co, sv);
#pragma unroll
  for (int j = 0; j < 8; ++j) ov[j] = ttm_rotary_value(xv[j], pv[j], cv[j], sv[j], sign);
  store8(out + b * per_batch + o, ov);
}

// ------------------------------------------------------------------------------------------------ cache update / fill
// cache[batch_offset + b, h, *index, :] = input[0, h, b, :]; one thread per 8 elements (never straddles a face row)
template <typename T>
__global__ __launch_bounds__(256) void ttm_update_cache_k(T *__restrict__ cache, const T *__restrict__ input,
                                                          const int32_t *__restrict__ index, int64_t heads, int64_t seq_pad,
                                                          int64_t max_seq, int64_t dim, int64_t in_users, int64_t in_users_pad,
                                                          int64_t batch_offset, int64_t total8) {
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= total8) return;
  const int64_t pos = index[0];
  if (pos < 0 || pos >= max_seq) return;          // out of range positions write nothing
  const int64_t d8 = dim >> 3;
  const int64_t c = (i % d8) * 8, b = (i / d8) % in_users, h = i / (d8 * in_users);
  const int64_t ct = dim >> 5;
  const T *src = input + h * in_users_pad * dim + ttm_tiled_offset(b, c, ct);
  T *dst = cache + ((batch_offset + b) * heads + h) * seq_pad * dim + ttm_tiled_offset(pos, c, ct);
  *(u32x4 *)dst = *(const u32x4 *)src;
  if (sizeof(T) == 4) *(u32x4 *)(dst + 4) = *(const u32x4 *)(src + 4);
}

// cache[batch_offset, h, 0:seq_tiles*32, :] = input[0, h, :, :] tile by tile (the padding rows of the last tile come along)
__global__ __launch_bounds__(256) void ttm_fill_cache_k(u32x4 *__restrict__ cache, const u32x4 *__restrict__ input,
                                                        int64_t head_stride_cache16, int64_t head_stride_in16, int64_t base16,
                                                        int64_t total16) {
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= total16) return;
  const int64_t h = i / head_stride_in16, o = i % head_stride_in16;
  cache[base16 + h * head_stride_cache16 + o] = input[i];
}

// Paged cache writes.  The cache is [blocks, heads, block_size, dim]; a user's positions live in the blocks its row of
// the page table names.  Without a page table the cache is [users, heads, max_seq, dim] (block_size = max_seq) and user
// u owns entry u (entry 0 for all users when the cache is shared).  Positions, page numbers and block numbers outside
// their ranges write nothing.
//
// update: cache[block(u, pos_u), h, pos_u % block_size, :] = input[0, u, h, :] with pos_u = index[u]; one thread per 8 elements
template <typename T>
__global__ __launch_bounds__(256) void ttm_paged_update_cache_k(T *__restrict__ cache, const T *__restrict__ input,
                                                                const int32_t *__restrict__ index, const int32_t *__restrict__ table,
                                                                int64_t blocks, int64_t heads, int64_t block_size, int64_t dim,
                                                                int64_t users, int64_t pages, int shared, int64_t total8) {
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= total8) return;
  const int64_t d8 = dim >> 3, ct = dim >> 5;
  const int64_t c = (i % d8) * 8, h = (i / d8) % heads, u = i / (d8 * heads);
  const int64_t pos = index[u];
  if (pos < 0) return;
  int64_t blk, off;
  if (table) {
    const int64_t page = pos / block_size;
    if (page >= pages) return;
    blk = table[u * pages + page];
    off = pos % block_size;
  } else {
    if (pos >= block_size) return;
    blk = shared ? 0 : u;
    off = pos;
  }
  if (blk < 0 || blk >= blocks) return;
  const int64_t heads_pad = ttm_round_up32(heads), bs_pad = ttm_round_up32(block_size);
  const T *src = input + u * heads_pad * dim + ttm_tiled_offset(h, c, ct);
  T *dst = cache + (blk * heads + h) * bs_pad * dim + ttm_tiled_offset(off, c, ct);
  *(u32x4 *)dst = *(const u32x4 *)src;
  if (sizeof(T) == 4) *(u32x4 *)(dst + 4) = *(const u32x4 *)(src + 4);
}

// fill: cache[table[row(b), s / block_size], h, s % block_size, :] = input[b, h, s, :] for s < seq, where row(b) is
// batch_idx[b] when given and b otherwise; one thread per 8 elements
template <typename T>
__global__ __launch_bounds__(256) void ttm_paged_fill_cache_k(T *__restrict__ cache, const T *__restrict__ input,
                                                              const int32_t *__restrict__ table, const int32_t *__restrict__ batch_idx,
                                                              int64_t blocks, int64_t heads, int64_t block_size, int64_t dim,
                                                              int64_t seq, int64_t table_rows, int64_t pages, int64_t total8) {
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= total8) return;
  const int64_t d8 = dim >> 3, ct = dim >> 5;
  const int64_t c = (i % d8) * 8, s = (i / d8) % seq, h = (i / (d8 * seq)) % heads, b = i / (d8 * seq * heads);
  const int64_t row = batch_idx ? batch_idx[b] : b;
  const int64_t page = s / block_size;
  if (row < 0 || row >= table_rows || page >= pages) return;
  const int64_t blk = table[row * pages + page];
  if (blk < 0 || blk >= blocks) return;
  const int64_t seq_pad = ttm_round_up32(seq), bs_pad = ttm_round_up32(block_size);
  const T *src = input + (b * heads + h) * seq_pad * dim + ttm_tiled_offset(s, c, ct);
  T *dst = cache + (blk * heads + h) * bs_pad * dim + ttm_tiled_offset(s % block_size, c, ct);
  *(u32x4 *)dst = *(const u32x4 *)src;
  if (sizeof(T) == 4) *(u32x4 *)(dst + 4) = *(const u32x4 *)(src + 4);
}

// gather: out[b, h, s, :] = cache[table[b, s / block_size], h, s % block_size, :] for s < pages * block_size, the inverse
// of the paged fill; positions whose page is outside the cache read as zeros; one thread per 8 elements
template <typename T>
__global__ __launch_bounds__(256) void ttm_paged_gather_k(const T *__restrict__ cache, const int32_t *__restrict__ table, T *__restrict__ out,
                                                          int64_t blocks, int64_t heads, int64_t block_size, int64_t dim, int64_t pages,
                                                          int64_t total8) {
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= total8) return;
  const int64_t d8 = dim >> 3, ct = dim >> 5, seq = pages * block_size;
  const int64_t c = (i % d8) * 8, s = (i / d8) % seq, h = (i / (d8 * seq)) % heads, b = i / (d8 * seq * heads);
  const int64_t blk = table[b * pages + s / block_size];
  T *dst = out + (b * heads + h) * seq * dim + ttm_tiled_offset(s, c, ct);
  u32x4 lo = {0, 0, 0, 0}, hi = {0, 0, 0, 0};
  if (blk >= 0 && blk < blocks) {
    const T *src = cache + (blk * heads + h) * block_size * dim + ttm_tiled_offset(s % block_size, c, ct);
    lo = *(const u32x4 *)src;
    if (sizeof(T) == 4) hi = *(const u32x4 *)(src + 4);
  }
  *(u32x4 *)dst = lo;
  if (sizeof(T) == 4) *(u32x4 *)(dst + 4) = hi;
}

// additive mask of a prefill chunk: query row i stands at absolute position *start + i and sees the keys up to it;
// mask[i, j] = 0 where j <= *start + i, -inf elsewhere.  bf16 tiles [rows_pad, cols_pad]; the offset is read from device
// memory, so the launch can be recorded into a graph and replayed for the next chunk
__global__ __launch_bounds__(256) void ttm_chunk_mask_k(uint16_t *__restrict__ mask, const int32_t *__restrict__ start, int64_t rows_pad,
                                                        int64_t cols_pad, int64_t total8) {
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= total8) return;
  const int64_t c8 = cols_pad >> 3, r = i / c8, c = (i % c8) * 8;
  const int64_t limit = (int64_t)start[0] + r;
  uint32_t w[4];
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    const uint32_t lo = c + 2 * k <= limit ? 0u : 0xFF80u, hi = c + 2 * k + 1 <= limit ? 0u : 0xFF80u;
    w[k] = lo | (hi << 16);
  }
  *(u32x4 *)(mask + ttm_tiled_offset(r, c, cols_pad >> 5)) = u32x4{w[0], w[1], w[2], w[3]};
}

// rotary embedding with a transformation matrix: out = x * cos + (x T) * sin, where T is a 32 x 32 matrix applied to
// every 32-column tile of a row (for the matrix Llama uses this rotates the interleaved pairs (x[2i], x[2i+1])).
// x / out [batch, rows, cols] tiles; cos / sin [cs_batch, cs_rows, cols] tiles, row r of batch entry b reads cos row
// (r if cs_rows > 1 else 0) of entry (b % cs_batch if cs_batch > 1 else 0).  One thread per element; T sits in LDS.
__global__ __launch_bounds__(256) void ttm_rotary_llama_k(const uint16_t *__restrict__ x, const uint16_t *__restrict__ cosc,
                                                          const uint16_t *__restrict__ sinc, const uint16_t *__restrict__ tmat,
                                                          uint16_t *__restrict__ out, int64_t rows, int64_t rows_pad, int64_t cols,
                                                          int64_t cs_batch, int64_t cs_rows, int64_t cs_rows_pad, int64_t total) {
  __shared__ float T[32][33];
  for (int e = threadIdx.x; e < 1024; e += 256) T[e >> 5][e & 31] = ttm_bf16_to_f32(tmat[ttm_tiled_offset(e >> 5, e & 31, 1)]);
  __syncthreads();
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= total) return;
  const int64_t c = i % cols, r = (i / cols) % rows_pad, b = i / (cols * rows_pad), ct = cols >> 5;
  const int64_t off = b * rows_pad * cols + ttm_tiled_offset(r, c, ct);
  if (r >= rows) { out[off] = 0; return; }   // tile padding stays zero
  const int64_t cb = cs_batch > 1 ? b % cs_batch : 0, cr = cs_rows > 1 ? r : 0;
  const int64_t coff = cb * cs_rows_pad * cols + ttm_tiled_offset(cr, c, ct);
  const uint16_t *xr = x + b * rows_pad * cols;
  float rot = 0.0f;
  const int64_t c0 = c & ~(int64_t)31;
#pragma unroll 8
  for (int j = 0; j < 32; ++j) rot += ttm_bf16_to_f32(xr[ttm_tiled_offset(r, c0 + j, ct)]) * T[j][c & 31];
  // fp32 throughout, one rounding at the end (the convention of the CPU path: compute in f32, cast back)
  out[off] = ttm_f32_to_bf16(ttm_bf16_to_f32(x[off]) * ttm_bf16_to_f32(cosc[coff]) + rot * ttm_bf16_to_f32(sinc[coff]));
}

// ------------------------------------------------------------------------------------------------ attention, one query token
// q [1, B, H, D], k / v [B, Hkv, S, D] (or pages [blocks, Hkv, block, D] behind a page table), out [1, B, H, D], bf16 tiles.
// grid (splits, B * Hkv), 256 threads.  A block owns the G = H / Hkv query heads of one kv head and one slice of the keys:
//   1. scores = Q K^T with v_mfma_f32_16x16x32_bf16 (queries are the 16 rows, padded with zeros), written to LDS
//      as (score + mask) * scale, -inf outside the valid keys;
//   2. softmax numerators per query head, rounded to bf16 and stored as pairs of keys 16 apart, and their sum;
//   3. P V on the vector ALU with v_dot2_f32_bf16: a wave reads the two halves of a V tile (2 x 1 KiB contiguous), every
//      lane keeps 8 columns x G heads of partial sums, lanes are combined once per column tile;
//   4. (max, sum, unnormalised output) go to the split's slot of the workspace; ttm_sdpa_decode_combine_k merges the slots
//      (merging in the last workgroup to arrive was measured: the device-scope fences it needs double the kernel time).
struct DecodeArgs {
  const uint16_t *q, *k, *v, *mask;
  const int32_t *cur_pos, *page_table;
  float *part;        // [B * Hkv][splits][G][D + 2]
  uint16_t *out;
  int B, H, Hkv, G, S, D, splits, keys_per_split, block, pages_per_user, mask_heads, is_causal;
  int blocks;         // number of blocks in a paged cache: page-table entries outside [0, blocks) are masked
  int concat_heads;   // out is [B, H * D] (row b holds user b's heads side by side) instead of [B, H, D]
  int Gt, g0;         // query heads per kv head in the tensors, and the first of them this launch serves (it serves G of them)
  int mask_b;         // 1: one mask per user, 0: one mask shared by all
  int window;         // >= 0: only the last `window` keys up to the decode position are visible
  const uint16_t *sink;   // [H, 32] in tiles, column 0: one more logit per head (times scale) with a zero value row; or null
  float scale;
};

constexpr int kMaxG = 8;
// K and V are read once per launch: streaming (nontemporal) loads keep them from displacing each other in the caches on
// the way (measured at 32 users x 8 kv heads x 2048 positions: 59 -> 54 us).  STREAM = false when several launches share
// one cache (more than kMaxG query heads per kv head), where the later launches profit from what the first one left.
template <bool STREAM, typename T>
__device__ __forceinline__ T kv_load(const T *p) {
  if constexpr (STREAM) return __builtin_nontemporal_load(p);
  else return *p;
}
#ifndef SPLIT_TARGET
#define SPLIT_TARGET 512
#endif

__device__ __forceinline__ const uint16_t *kv_tile_row(const uint16_t *base, const DecodeArgs &p, int b, int hk, int key_tile, bool &ok) {
  // start of the row of tiles holding keys [32 key_tile, 32 key_tile + 32) of (b, hk).  A page-table entry outside the
  // cache's blocks (an unused slot, -1) gives ok = false and the address of block 0: the caller treats those keys as masked
  const int64_t row_elems = (int64_t)32 * p.D;
  ok = true;
  if (p.page_table) {
    const int tiles_per_block = p.block >> 5;
    int page = p.page_table[(int64_t)b * p.pages_per_user + key_tile / tiles_per_block];
    ok = page >= 0 && page < p.blocks;
    page = ok ? page : 0;
    return base + (((int64_t)page * p.Hkv + hk) * tiles_per_block + key_tile % tiles_per_block) * row_elems;
  }
  return base + (((int64_t)b * p.Hkv + hk) * (p.S >> 5) + key_tile) * row_elems;
}

template <bool STREAM>
__global__ __launch_bounds__(256) void ttm_sdpa_decode_k(DecodeArgs p) {
  extern __shared__ float lds[];
  const int split = blockIdx.x, bh = blockIdx.y, b = bh / p.Hkv, hk = bh % p.Hkv;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int G = p.G, D = p.D, DT = D >> 5;
  int valid = p.S, pos = p.S - 1;
  if (p.cur_pos) {
    pos = p.cur_pos[b];
    if (p.is_causal) {
      const int cp = pos + 1;
      valid = cp < valid ? (cp < 0 ? 0 : cp) : valid;
    }
  }
  // first visible key; the tiles in front of it are not read at all
  const int lo = p.window >= 0 && pos + 1 > p.window ? pos + 1 - p.window : 0;
  const int k0 = max(split * p.keys_per_split, lo & ~31);
  int k1 = (split + 1) * p.keys_per_split;
  k1 = k1 < valid ? k1 : valid;
  const int nkeys = k1 > k0 ? k1 - k0 : 0;
  const int ngroups = (nkeys + 15) >> 4;
  float *sc = lds;                                        // [G][keys_per_split] scores
  float *osum = lds + (size_t)G * p.keys_per_split;       // [G][D]
  float *stat = osum + (size_t)G * D;                     // [G][2]: max, sum
  uint32_t *pp = (uint32_t *)(stat + 2 * G);              // [G][keys_per_split / 2] bf16 pairs of softmax numerators
  float *slot = p.part + ((size_t)bh * p.splits + split) * G * (D + 2);

  for (int i = tid; i < G * D; i += 256) osum[i] = 0.0f;
  if (nkeys == 0) {
    for (int i = tid; i < G * (D + 2); i += 256) {
      const int c = i % (D + 2);
      slot[i] = c == D ? -INFINITY : 0.0f;
    }
  } else {

  // ---- 1. scores
  {
    // query fragments: lane supplies query row lane % 16, columns 32 c + 8 (lane / 16) .. + 7
    const int g = lane & 15, dq = (lane >> 4) * 8;
    bf16x8 qf[8];
    const int h = hk * p.Gt + p.g0 + g;
    const uint16_t *qb = p.q + (int64_t)b * ttm_round_up32(p.H) * D;
#pragma unroll
    for (int c = 0; c < 8; ++c) {
      u32x4 z = {0, 0, 0, 0};
      if (c < DT && g < G) z = *(const u32x4 *)(qb + ttm_tiled_offset(h, 32 * c + dq, DT));
      qf[c] = *(bf16x8 *)&z;
    }
    const int hrow = hk * p.Gt + p.g0;  // mask rows of this block's heads
    constexpr int KU = 1;
    for (int g0 = wave; g0 < ngroups; g0 += 4 * KU) {
      // KU groups of 16 keys per wavefront and pass, all their loads issued before the first product (one group: 8 KiB per
      // wavefront in flight; two measured 1.5 % slower, three and four slower still)
      u32x4 kf[KU][8];
      int grp[KU];
      bool kok[KU];
#pragma unroll
      for (int u = 0; u < KU; ++u) {
        grp[u] = g0 + 4 * u < ngroups ? g0 + 4 * u : g0;   // the tail repeats a valid group and skips its result
        const int key = k0 + grp[u] * 16 + (lane & 15);     // this lane's key column of the B operand
        const uint16_t *kt = kv_tile_row(p.k, p, b, hk, key >> 5, kok[u]);
        // inside a tile: face (key half, column half), row key % 16, columns dq % 16 .. + 7
        const int in_tile = (((key >> 4) & 1) * 2 + (dq >> 4)) * 256 + (key & 15) * 16 + (dq & 15);
#pragma unroll
        for (int c = 0; c < 8; ++c)
          if (c < DT) kf[u][c] = kv_load<STREAM>((const u32x4 *)(kt + (int64_t)c * 1024 + in_tile));
      }
#pragma unroll
      for (int u = 0; u < KU; ++u) {
        if (u == 1 && g0 + 4 >= ngroups) break;
        f32x4v acc = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int c = 0; c < 8; ++c)
          if (c < DT) acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(qf[c], *(bf16x8 *)&kf[u][c], acc, 0, 0, 0);
        // acc[i] = score of query 4 (lane / 16) + i against key lane % 16 of the group
        const int kk = grp[u] * 16 + (lane & 15);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int gq = (lane >> 4) * 4 + i;
          if (gq < G) {
            float sv = acc[i];
            if (p.mask) {
              const int mh = p.mask_heads == 1 ? 0 : hrow + gq;
              const int64_t mrows = ttm_round_up32(p.mask_heads);
              sv += ttm_bf16_to_f32(p.mask[(int64_t)b * p.mask_b * mrows * p.S + ttm_tiled_offset(mh, k0 + kk, p.S >> 5)]);
            }
            sc[gq * p.keys_per_split + kk] = (k0 + kk < k1 && k0 + kk >= lo && kok[u]) ? sv * p.scale : -INFINITY;
          }
        }
      }
    }
  }
  __syncthreads();

  // ---- 2. softmax numerators: wave w serves heads w, w + 4, ...  The numerators are rounded to bf16 and stored in pairs
  // (key r, key r + 16 of a 32-key tile) so that the next phase multiplies two keys per instruction; their sum is taken
  // over the rounded values, which keeps numerator and denominator consistent.
  const int padded = ngroups * 16, ntiles = (ngroups + 1) >> 1;
  for (int g = wave; g < G; g += 4) {
    const float *row = sc + g * p.keys_per_split;
    uint32_t *prow = pp + g * (p.keys_per_split >> 1);
    float m = -INFINITY;
    for (int i = lane; i < padded; i += 64) m = fmaxf(m, row[i]);
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) m = fmaxf(m, __shfl_xor(m, o));
    float l = 0.0f;
    for (int i = lane; i < ntiles * 16; i += 64) {
      const int klo = (i >> 4) * 32 + (i & 15), khi = klo + 16;
      const float elo = (m == -INFINITY || klo >= padded) ? 0.0f : __expf(row[klo] - m);
      const float ehi = (m == -INFINITY || khi >= padded) ? 0.0f : __expf(row[khi] - m);
      const uint32_t pair = ttm_pack_bf16x2(elo, ehi);
      prow[i] = pair;
      l += __uint_as_float(pair << 16) + __uint_as_float(pair & 0xFFFF0000u);
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) l += __shfl_xor(l, o);
    if (lane == 0) { stat[2 * g] = m; stat[2 * g + 1] = l; }
  }
  __syncthreads();

  // ---- 3. P V with v_dot2_f32_bf16: work items are (column tile, stride class of key tiles).  Per key tile a lane reads
  // 8 columns of key r (faces 0 / 1) and of key r + 16 (faces 2 / 3), r = (lane % 32) / 2, columns
  // 16 (lane / 32) + 8 (lane % 2) .. + 7; the two rows are interleaved to (v[r][d], v[r + 16][d]) pairs and multiplied with
  // the stored (p[r], p[r + 16]) pair.
  {
    const int share = DT == 1 ? 4 : (DT == 2 ? 2 : 1);   // with one or two column tiles several waves split the keys of one
    const int items = DT * share;
    const int krow = (lane & 31) >> 1;
    constexpr int UT = 4;                                  // key tiles in flight per pass (8 KiB per wave)
    for (int item = wave; item < items; item += 4) {
      const int dt = item % DT, tfirst = item / DT;
      float o[kMaxG][8];
#pragma unroll
      for (int g = 0; g < kMaxG; ++g)
#pragma unroll
        for (int j = 0; j < 8; ++j) o[g][j] = 0.0f;
      for (int t0 = tfirst; t0 < ntiles; t0 += UT * share) {
        u32x4 ra[UT], rb[UT];
        bool vok[UT];
#pragma unroll
        for (int u = 0; u < UT; ++u) {
          const int t = t0 + u * share < ntiles ? t0 + u * share : t0;
          const uint16_t *vt = kv_tile_row(p.v, p, b, hk, (k0 >> 5) + t, vok[u]) + (int64_t)dt * 1024;
          ra[u] = kv_load<STREAM>((const u32x4 *)(vt + lane * 8));
          rb[u] = kv_load<STREAM>((const u32x4 *)(vt + 512 + lane * 8));
        }
#pragma unroll
        for (int u = 0; u < UT; ++u) {
          const int t = t0 + u * share;
          if (t >= ntiles) break;
          uint32_t a[4] = {ra[u].x, ra[u].y, ra[u].z, ra[u].w}, c[4] = {rb[u].x, rb[u].y, rb[u].z, rb[u].w};
          if (t * 32 + 32 > nkeys || k0 + t * 32 < lo || !vok[u]) {   // boundary tile: rows outside the visible keys may hold anything, NaN included
            const bool la = vok[u] && t * 32 + krow < nkeys && k0 + t * 32 + krow >= lo;
            const bool lb = vok[u] && t * 32 + 16 + krow < nkeys && k0 + t * 32 + 16 + krow >= lo;
#pragma unroll
            for (int j = 0; j < 4; ++j) { a[j] = la ? a[j] : 0u; c[j] = lb ? c[j] : 0u; }
          }
          uint32_t vp[8];   // vp[2 j] = (a.col 2j, c.col 2j), vp[2 j + 1] = (a.col 2j+1, c.col 2j+1)
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            vp[2 * j] = __builtin_amdgcn_perm(c[j], a[j], 0x05040100u);
            vp[2 * j + 1] = __builtin_amdgcn_perm(c[j], a[j], 0x07060302u);
          }
#pragma unroll
          for (int g = 0; g < kMaxG; ++g) {
            if (g < G) {
              const uint32_t pg = pp[g * (p.keys_per_split >> 1) + t * 16 + krow];
#pragma unroll
              for (int j = 0; j < 8; ++j)
                o[g][j] = __builtin_amdgcn_fdot2_f32_bf16(*(bf16x2 *)&vp[j], *(const bf16x2 *)&pg, o[g][j], false);
            }
          }
        }
      }
      // combine the 16 lanes that hold the same columns (they differ in bits 1..4 of the lane id)
#pragma unroll
      for (int g = 0; g < kMaxG; ++g) {
        if (g < G) {
#pragma unroll
          for (int j = 0; j < 8; ++j) {
            float v = o[g][j];
            v += __shfl_xor(v, 2);
            v += __shfl_xor(v, 4);
            v += __shfl_xor(v, 8);
            v += __shfl_xor(v, 16);
            o[g][j] = v;
          }
        }
      }
      if (((lane >> 1) & 15) == 0) {
        const int col = dt * 32 + (lane >> 5) * 16 + (lane & 1) * 8;
#pragma unroll
        for (int g = 0; g < kMaxG; ++g)
          if (g < G)
#pragma unroll
            for (int j = 0; j < 8; ++j) {
              if (share == 1) osum[g * D + col + j] = o[g][j];
              else atomicAdd(&osum[g * D + col + j], o[g][j]);
            }
      }
    }
  }
  __syncthreads();

  // ---- 4. the split's slot
  for (int i = tid; i < G * (D + 2); i += 256) {
    const int g = i / (D + 2), c = i % (D + 2);
    slot[i] = c < D ? osum[g * D + c] : stat[2 * g + (c - D)];
  }
  }  // nkeys != 0
}

// merges the slots of one query head: out = sum_s o_s exp(m_s - M) / sum_s l_s exp(m_s - M).  grid (B * Hkv, G), 256 lanes:
// the weights exp(m_s - M) of the slices are formed once in LDS; 256 / D lanes share a column and take every (256 / D)-th
// slice, so that a long cache cut into many slices for a few users (one user, 32768 positions: 64 slices) is merged by all
// lanes of 32 workgroups instead of by eight workgroups looping over the slices.
constexpr int kMaxCombineSlices = 1024;
__global__ __launch_bounds__(256) void ttm_sdpa_decode_combine_k(DecodeArgs p) {
  __shared__ float wgt[kMaxCombineSlices];
  __shared__ float red[256];
  __shared__ float stats[2];
  const int bh = blockIdx.x, tid = threadIdx.x;
  const int b = bh / p.Hkv, hk = bh % p.Hkv;
  const int G = p.G, D = p.D, S = p.splits;
  for (int g = blockIdx.y; g < G; g += gridDim.y) {   // grid.y = G: one head per workgroup (workgroup-uniform)
  const float *base = p.part + (size_t)bh * S * G * (D + 2) + (size_t)g * (D + 2);   // slice s: + s * G * (D + 2)
  const size_t sstride = (size_t)G * (D + 2);
  const int h = hk * p.Gt + p.g0 + g;
  const float sinkv = p.sink ? ttm_bf16_to_f32(p.sink[ttm_tiled_offset(h, 0, 1)]) * p.scale : -INFINITY;
  // M = max over the slices (and the sink)
  float m = sinkv;
  for (int s = tid; s < S; s += 256) m = fmaxf(m, base[s * sstride + D]);
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) m = fmaxf(m, __shfl_xor(m, o));
  if ((tid & 63) == 0) red[tid >> 6] = m;
  __syncthreads();
  const float M = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
  __syncthreads();
  // weights and the denominator
  float den = 0.0f;
  for (int s = tid; s < S; s += 256) {
    const float ms = base[s * sstride + D];
    const float w = ms == -INFINITY ? 0.0f : __expf(ms - M);
    wgt[s] = w;
    den += base[s * sstride + D + 1] * w;
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) den += __shfl_xor(den, o);
  if ((tid & 63) == 0) red[tid >> 6] = den;
  __syncthreads();
  if (tid == 0) stats[0] = (red[0] + red[1]) + (red[2] + red[3]) + (p.sink ? __expf(sinkv - M) : 0.0f);
  __syncthreads();
  den = stats[0];
  // numerators: lane (c, sub) sums the slices sub, sub + nsub, ... of column c
  const int nsub = 256 / D > 0 ? 256 / D : 1;
  for (int c0 = 0; c0 < D; c0 += 256) {   // one round unless D > 256
    const int c = c0 + (tid % (D < 256 ? D : 256)), sub = D < 256 ? tid / D : 0;
    float num = 0.0f;
    if (c < D && sub < nsub)
      for (int s = sub; s < S; s += nsub) num += base[s * sstride + c] * wgt[s];
    red[tid] = num;
    __syncthreads();
    if (c < D && sub == 0) {
      for (int u = 1; u < nsub; ++u) num += red[tid + u * D];
      const uint16_t val = ttm_f32_to_bf16(den > 0.0f ? num / den : 0.0f);
      if (p.concat_heads) p.out[ttm_tiled_offset(b, h * D + c, (p.H * D) >> 5)] = val;
      else p.out[(int64_t)b * ttm_round_up32(p.H) * D + ttm_tiled_offset(h, c, D >> 5)] = val;
    }
    __syncthreads();
  }
  }  // heads of this workgroup
  if (blockIdx.y != 0) return;   // the padding belongs to the first head's workgroup
  if (p.concat_heads) {   // padding rows below the last user, this kv head's columns
    if (b == p.B - 1) {
      const int pad = (int)ttm_round_up32(p.B) - p.B;
      for (int i = tid; i < pad * G * D; i += 256)
        p.out[ttm_tiled_offset(p.B + i / (G * D), (hk * p.Gt + p.g0) * D + i % (G * D), (p.H * D) >> 5)] = 0;
    }
    return;
  }
  if (hk == p.Hkv - 1 && p.g0 + G == p.Gt) {   // padding rows of the last head tile
    const int pad = (int)ttm_round_up32(p.H) - p.H;
    for (int i = tid; i < pad * D; i += 256)
      p.out[(int64_t)b * ttm_round_up32(p.H) * D + ttm_tiled_offset(p.H + i / D, i % D, D >> 5)] = 0;
  }
}

}  // namespace

static int rotary_entry(const void *x, const void *cos_cache, const void *sin_cache, void *out, int dtype, int64_t batch, int64_t rows,
                        int64_t cols, int64_t cache_rows, int64_t token_index, bool split, void *stream) {
  TTM_REQUIRE(x && cos_cache && sin_cache && out, "ttm_rotary_embedding: null pointer");
  TTM_REQUIRE(!split || token_index >= 0, "ttm_rotary_embedding_split_heads: rows are heads here, so the position must come from token_index");
  TTM_REQUIRE(dtype == TTM_BF16 || dtype == TTM_F32, "ttm_rotary_embedding: dtype must be BFloat16 or Float32");
  TTM_REQUIRE(batch >= 0 && rows > 0 && cols > 0 && cols % 32 == 0, "ttm_rotary_embedding: head dim must be a positive multiple of 32");
  if (token_index >= 0)
    TTM_REQUIRE(token_index < cache_rows, "ttm_rotary_embedding: token_index %lld outside the %lld cached positions",
                (long long)token_index, (long long)cache_rows);
  else
    TTM_REQUIRE(cache_rows >= rows, "ttm_rotary_embedding: cos / sin caches hold %lld positions, input has %lld",
                (long long)cache_rows, (long long)rows);
  if (batch == 0) return TTM_OK;
  const int64_t rows_pad = ttm_round_up32(rows), per_batch = rows_pad * cols, total8 = batch * per_batch / 8;
  const int64_t src_cols = split ? rows * cols : 0;
  const dim3 grid((unsigned)ttm_cdiv(total8, 256));
  if (dtype == TTM_BF16)
    hipLaunchKernelGGL(ttm_rotary_k<uint16_t>, grid, dim3(256), 0, (hipStream_t)stream, (const uint16_t *)x,
                       (const uint16_t *)cos_cache, (const uint16_t *)sin_cache, (uint16_t *)out, rows_pad, cols, per_batch,
                       total8, token_index, rows, src_cols);
  else
    hipLaunchKernelGGL(ttm_rotary_k<float>, grid, dim3(256), 0, (hipStream_t)stream, (const float *)x, (const float *)cos_cache,
                       (const float *)sin_cache, (float *)out, rows_pad, cols, per_batch, total8, token_index, rows, src_cols);
  TTM_LAUNCH_CHECK();
  return TTM_OK;
}

TTM_EXPORT int ttm_rotary_embedding(const void *x, const void *cos_cache, const void *sin_cache, void *out, int dtype,
                                    int64_t batch, int64_t rows, int64_t cols, int64_t cache_rows, int64_t token_index,
                                    void *stream) {
  TTM_EXTENTS(rotary_embedding, x, cos_cache, sin_cache, out, dtype, batch, rows, cols, cache_rows);
  return rotary_entry(x, cos_cache, sin_cache, out, dtype, batch, rows, cols, cache_rows, token_index, false, stream);
}

TTM_EXPORT int ttm_rotary_embedding_split_heads(const void *x, const void *cos_cache, const void *sin_cache, void *out, int dtype,
                                                int64_t batch, int64_t heads, int64_t head_dim, int64_t cache_rows,
                                                int64_t token_index, void *stream) {
  TTM_EXTENTS(rotary_embedding_split_heads, x, cos_cache, sin_cache, out, dtype, batch, heads, head_dim, cache_rows);
  return rotary_entry(x, cos_cache, sin_cache, out, dtype, batch, heads, head_dim, cache_rows, token_index, true, stream);
}

TTM_EXPORT int ttm_update_cache(void *cache, const void *input, const int32_t *update_index, int dtype, int64_t users,
                                int64_t heads, int64_t max_seq, int64_t head_dim, int64_t input_users, int64_t batch_offset,
                                void *stream) {
  TTM_EXTENTS(update_cache, cache, input, update_index, dtype, users, heads, max_seq, head_dim, input_users);
  TTM_REQUIRE(cache && input && update_index, "ttm_update_cache: null pointer");
  TTM_REQUIRE(dtype == TTM_BF16 || dtype == TTM_F32, "ttm_update_cache: dtype must be BFloat16 or Float32");
  TTM_REQUIRE(head_dim > 0 && head_dim % 32 == 0, "ttm_update_cache: head dim must be a positive multiple of 32");
  TTM_REQUIRE(batch_offset >= 0 && input_users >= 0 && batch_offset + input_users <= users,
              "ttm_update_cache: users [%lld, %lld) outside the cache's %lld", (long long)batch_offset,
              (long long)(batch_offset + input_users), (long long)users);
  const int64_t total8 = heads * input_users * (head_dim / 8);
  if (total8 == 0) return TTM_OK;
  const dim3 grid((unsigned)ttm_cdiv(total8, 256));
  const int64_t seq_pad = ttm_round_up32(max_seq), in_pad = ttm_round_up32(input_users);
  if (dtype == TTM_BF16)
    hipLaunchKernelGGL(ttm_update_cache_k<uint16_t>, grid, dim3(256), 0, (hipStream_t)stream, (uint16_t *)cache,
                       (const uint16_t *)input, update_index, heads, seq_pad, max_seq, head_dim, input_users, in_pad, batch_offset,
                       total8);
  else
    hipLaunchKernelGGL(ttm_update_cache_k<float>, grid, dim3(256), 0, (hipStream_t)stream, (float *)cache, (const float *)input,
                       update_index, heads, seq_pad, max_seq, head_dim, input_users, in_pad, batch_offset, total8);
  TTM_LAUNCH_CHECK();
  return TTM_OK;
}

TTM_EXPORT int ttm_fill_cache(void *cache, const void *input, int dtype, int64_t users, int64_t heads, int64_t max_seq,
                              int64_t head_dim, int64_t seq, int64_t batch_offset, void *stream) {
  TTM_EXTENTS(fill_cache, cache, input, dtype, users, heads, max_seq, head_dim, seq);
  TTM_REQUIRE(cache && input, "ttm_fill_cache: null pointer");
  const int eb = ttm_dtype_bytes(dtype);
  TTM_REQUIRE(eb == 2 || eb == 4, "ttm_fill_cache: element size must be 2 or 4 bytes");
  TTM_REQUIRE(head_dim > 0 && head_dim % 32 == 0, "ttm_fill_cache: head dim must be a positive multiple of 32");
  TTM_REQUIRE(batch_offset >= 0 && batch_offset < users, "ttm_fill_cache: batch offset %lld outside the cache's %lld users",
              (long long)batch_offset, (long long)users);
  TTM_REQUIRE(seq >= 0 && seq <= max_seq, "ttm_fill_cache: %lld positions do not fit a cache of %lld", (long long)seq, (long long)max_seq);
  const int64_t in16 = ttm_round_up32(seq) * head_dim * eb / 16, cache16 = ttm_round_up32(max_seq) * head_dim * eb / 16;
  const int64_t total16 = heads * in16;
  if (total16 == 0) return TTM_OK;
  hipLaunchKernelGGL(ttm_fill_cache_k, dim3((unsigned)ttm_cdiv(total16, 256)), dim3(256), 0, (hipStream_t)stream, (u32x4 *)cache,
                     (const u32x4 *)input, cache16, in16, batch_offset * heads * cache16, total16);
  TTM_LAUNCH_CHECK();
  return TTM_OK;
}

TTM_EXPORT int ttm_paged_update_cache(void *cache, const void *input, const int32_t *update_index, const int32_t *page_table,
                                      int dtype, int64_t blocks, int64_t heads, int64_t block_size, int64_t head_dim, int64_t users,
                                      int64_t pages_per_user, int share_cache, void *stream) {
  TTM_EXTENTS(paged_update_cache, cache, input, update_index, page_table, dtype, blocks, heads, block_size, head_dim, users, pages_per_user);
  TTM_REQUIRE(cache && input && update_index, "ttm_paged_update_cache: null pointer");
  TTM_REQUIRE(dtype == TTM_BF16 || dtype == TTM_F32, "ttm_paged_update_cache: dtype must be BFloat16 or Float32");
  TTM_REQUIRE(head_dim > 0 && head_dim % 32 == 0, "ttm_paged_update_cache: head dim must be a positive multiple of 32");
  TTM_REQUIRE(blocks > 0 && heads > 0 && block_size > 0 && users >= 0, "ttm_paged_update_cache: bad extents");
  TTM_REQUIRE(!page_table || pages_per_user > 0, "ttm_paged_update_cache: a page table needs pages_per_user > 0");
  TTM_REQUIRE(page_table || share_cache || users <= blocks, "ttm_paged_update_cache: %lld users do not fit a cache of %lld entries",
              (long long)users, (long long)blocks);
  const int64_t total8 = users * heads * (head_dim / 8);
  if (total8 == 0) return TTM_OK;
  const dim3 grid((unsigned)ttm_cdiv(total8, 256));
  if (dtype == TTM_BF16)
    hipLaunchKernelGGL(ttm_paged_update_cache_k<uint16_t>, grid, dim3(256), 0, (hipStream_t)stream, (uint16_t *)cache,
                       (const uint16_t *)input, update_index, page_table, blocks, heads, block_size, head_dim, users, pages_per_user,
                       share_cache, total8);
  else
    hipLaunchKernelGGL(ttm_paged_update_cache_k<float>, grid, dim3(256), 0, (hipStream_t)stream, (float *)cache, (const float *)input,
                       update_index, page_table, blocks, heads, block_size, head_dim, users, pages_per_user, share_cache, total8);
  TTM_LAUNCH_CHECK();
  return TTM_OK;
}

TTM_EXPORT int ttm_paged_fill_cache(void *cache, const void *input, const int32_t *page_table, const int32_t *batch_idx, int dtype,
                                    int64_t blocks, int64_t heads, int64_t block_size, int64_t head_dim, int64_t in_batch, int64_t seq,
                                    int64_t table_rows, int64_t pages_per_user, void *stream) {
  TTM_EXTENTS(paged_fill_cache, cache, input, page_table, batch_idx, dtype, blocks, heads, block_size, head_dim, in_batch, seq, table_rows, pages_per_user);
  TTM_REQUIRE(cache && input && page_table, "ttm_paged_fill_cache: null pointer");
  TTM_REQUIRE(dtype == TTM_BF16 || dtype == TTM_F32, "ttm_paged_fill_cache: dtype must be BFloat16 or Float32");
  TTM_REQUIRE(head_dim > 0 && head_dim % 32 == 0, "ttm_paged_fill_cache: head dim must be a positive multiple of 32");
  TTM_REQUIRE(blocks > 0 && heads > 0 && block_size > 0 && in_batch >= 0 && seq >= 0 && table_rows > 0 && pages_per_user > 0,
              "ttm_paged_fill_cache: bad extents");
  const int64_t total8 = in_batch * heads * seq * (head_dim / 8);
  if (total8 == 0) return TTM_OK;
  const dim3 grid((unsigned)ttm_cdiv(total8, 256));
  if (dtype == TTM_BF16)
    hipLaunchKernelGGL(ttm_paged_fill_cache_k<uint16_t>, grid, dim3(256), 0, (hipStream_t)stream, (uint16_t *)cache,
                       (const uint16_t *)input, page_table, batch_idx, blocks, heads, block_size, head_dim, seq, table_rows,
                       pages_per_user, total8);
  else
    hipLaunchKernelGGL(ttm_paged_fill_cache_k<float>, grid, dim3(256), 0, (hipStream_t)stream, (float *)cache, (const float *)input,
                       page_table, batch_idx, blocks, heads, block_size, head_dim, seq, table_rows, pages_per_user, total8);
  TTM_LAUNCH_CHECK();
  return TTM_OK;
}

// ---- scratch of ttm_sdpa_decode_static: the per-slice (max, sum, output) slots live in a device array of the library's
// own instead of the stream's workspace, so that entry point never allocates.  Every GPU holds its own copy of the array at
// its own address until the process ends; in host code the array's name is only a handle for hipGetSymbolAddress, the
// kernels get the address that call returned for the current device.
constexpr size_t kDecodeScratchBytes = (size_t)8 << 20;
static __device__ __align__(256) float scratch[kDecodeScratchBytes / sizeof(float)];

constexpr int kMaxDevices = 64;
static std::mutex g_scratch_mu;
static float *g_scratch_ptr[kMaxDevices];   // per device, set on the first call with that device current

static int decode_scratch_ptr(void **ptr) {
  int dev = 0;
  TTM_HIP(hipGetDevice(&dev));
  TTM_REQUIRE(dev >= 0 && dev < kMaxDevices, "ttm_sdpa_decode_static: device ordinal %d beyond %d", dev, kMaxDevices);
  std::lock_guard<std::mutex> g(g_scratch_mu);
  if (!g_scratch_ptr[dev]) {
    float *d = nullptr;
    TTM_HIP(hipGetSymbolAddress((void **)&d, HIP_SYMBOL(scratch)));
    TTM_REQUIRE(d != nullptr, "ttm_sdpa_decode_static: hipGetSymbolAddress returned a null address");
    g_scratch_ptr[dev] = d;
  }
  *ptr = g_scratch_ptr[dev];
  return TTM_OK;
}

static int sdpa_decode_entry(const void *q, const void *k, const void *v, const int32_t *cur_pos, const void *mask, int mask_heads,
                             const int32_t *page_table, int64_t pages_per_user, int64_t page_block, int64_t page_blocks, void *out, int dtype, int64_t batch,
                             int64_t heads, int64_t kv_heads, int64_t seq, int64_t head_dim, int is_causal, float scale, int concat_heads,
                             int64_t window, const void *sink, int64_t mask_batch, bool static_scratch, void *stream) {
  TTM_REQUIRE(q && k && v && out, "ttm_sdpa_decode: null pointer");
  TTM_REQUIRE(dtype == TTM_BF16, "ttm_sdpa_decode: tensors must be BFloat16");
  TTM_REQUIRE(batch > 0 && heads > 0 && kv_heads > 0 && heads % kv_heads == 0, "ttm_sdpa_decode: heads must be a multiple of kv heads");
  // a launch serves up to kMaxG query heads per kv head; more (multi-query attention) take several launches over the same cache
  const int64_t Gt = heads / kv_heads, G = Gt < kMaxG ? Gt : kMaxG;
  TTM_REQUIRE(head_dim % 32 == 0 && head_dim >= 32 && head_dim <= 256, "ttm_sdpa_decode: head dim must be a multiple of 32 up to 256");
  TTM_REQUIRE(seq > 0 && seq % 32 == 0, "ttm_sdpa_decode: cache length must be a positive multiple of 32");
  TTM_REQUIRE(!mask || mask_heads == 1 || mask_heads == heads, "ttm_sdpa_decode: mask must have 1 or %lld head rows", (long long)heads);
  if (page_table) {
    TTM_REQUIRE(page_block > 0 && page_block % 32 == 0 && pages_per_user * page_block == seq,
                "ttm_sdpa_decode: page table of %lld blocks x %lld positions does not cover %lld positions",
                (long long)pages_per_user, (long long)page_block, (long long)seq);
    TTM_REQUIRE(page_blocks > 0 && page_blocks <= INT32_MAX, "ttm_sdpa_decode: a page table needs the number of blocks in the cache (got %lld)",
                (long long)page_blocks);
  }
  hipStream_t s = (hipStream_t)stream;
  // enough blocks to fill the device, slices small enough for the score rows to fit in LDS
  int64_t splits = ttm_cdiv(SPLIT_TARGET, batch * kv_heads);
  const int64_t max_keys = (48 * 1024 / 6) / G / 32 * 32;   // 4 bytes of score + 2 of numerator per key and head
  if (splits > seq / 256) splits = seq / 256 > 0 ? seq / 256 : 1;
  if (ttm_cdiv(seq, splits) > max_keys) splits = ttm_cdiv(seq, max_keys);
  const int64_t keys = ttm_round_up32(ttm_cdiv(seq, splits));
  splits = ttm_cdiv(seq, keys);
  TTM_REQUIRE(splits <= kMaxCombineSlices, "ttm_sdpa_decode: a cache of %lld positions takes %lld key slices, the merge handles %d", (long long)seq,
              (long long)splits, kMaxCombineSlices);
  DecodeArgs p;
  p.q = (const uint16_t *)q; p.k = (const uint16_t *)k; p.v = (const uint16_t *)v; p.mask = (const uint16_t *)mask;
  p.cur_pos = cur_pos; p.page_table = page_table; p.out = (uint16_t *)out;
  p.B = (int)batch; p.H = (int)heads; p.Hkv = (int)kv_heads; p.G = (int)G; p.S = (int)seq; p.D = (int)head_dim;
  p.splits = (int)splits; p.keys_per_split = (int)keys; p.block = (int)page_block; p.pages_per_user = (int)pages_per_user;
  p.blocks = (int)page_blocks;
  p.mask_heads = mask_heads; p.is_causal = is_causal; p.concat_heads = concat_heads;
  p.scale = scale > 0.0f ? scale : 1.0f / sqrtf((float)head_dim);
  p.Gt = (int)Gt;
  p.window = window < 0 ? -1 : (int)(window < seq ? window : seq);
  p.sink = (const uint16_t *)sink;
  TTM_REQUIRE(!mask || mask_batch == 1 || mask_batch == batch, "ttm_sdpa_decode: mask batch must be 1 or %lld", (long long)batch);
  p.mask_b = mask_batch == 1 ? 0 : 1;
  void *ws = nullptr;
  const size_t part_bytes = (size_t)(batch * kv_heads * splits * G * (head_dim + 2)) * sizeof(float);
  if (static_scratch) {
    TTM_REQUIRE(part_bytes <= kDecodeScratchBytes,
                "ttm_sdpa_decode_static: the per-slice partial results of this call take %zu bytes, the static scratch holds %zu "
                "(batch * kv_heads * slices * heads-per-kv-head * (head_dim + 2) floats): use ttm_sdpa_decode_windowed",
                part_bytes, (size_t)kDecodeScratchBytes);
    if (int rc = decode_scratch_ptr(&ws)) return rc;
  } else {
    if (int rc = ttm_stream_workspace(s, part_bytes, &ws)) return rc;
  }
  p.part = (float *)ws;
  for (int64_t g0 = 0; g0 < Gt; g0 += kMaxG) {   // the launches of one call follow each other on the stream and share the workspace
    p.g0 = (int)g0;
    p.G = (int)(Gt - g0 < kMaxG ? Gt - g0 : kMaxG);
    const size_t lds = (size_t)(p.G * keys + p.G * head_dim + 2 * p.G + p.G * keys / 2) * sizeof(float);
    if (Gt <= kMaxG) hipLaunchKernelGGL(ttm_sdpa_decode_k<true>, dim3((unsigned)splits, (unsigned)(batch * kv_heads)), dim3(256), lds, s, p);
    else hipLaunchKernelGGL(ttm_sdpa_decode_k<false>, dim3((unsigned)splits, (unsigned)(batch * kv_heads)), dim3(256), lds, s, p);
    TTM_LAUNCH_CHECK();
    hipLaunchKernelGGL(ttm_sdpa_decode_combine_k, dim3((unsigned)(batch * kv_heads), (unsigned)p.G), dim3(256), 0, s, p);
    TTM_LAUNCH_CHECK();
  }
  return TTM_OK;
}

TTM_EXPORT int ttm_sdpa_decode(const void *q, const void *k, const void *v, const int32_t *cur_pos, const void *mask,
                               int mask_heads, const int32_t *page_table, int64_t pages_per_user, int64_t page_block, int64_t page_blocks,
                               void *out, int dtype, int64_t batch, int64_t heads, int64_t kv_heads, int64_t seq, int64_t head_dim,
                               int is_causal, float scale, void *stream) {
  TTM_EXTENTS(sdpa_decode, q, k, v, cur_pos, mask, mask_heads, batch, page_table, pages_per_user, page_block, page_blocks, out, dtype, batch, heads, kv_heads, seq, head_dim, 0, nullptr);
  return sdpa_decode_entry(q, k, v, cur_pos, mask, mask_heads, page_table, pages_per_user, page_block, page_blocks, out, dtype, batch, heads, kv_heads,
                           seq, head_dim, is_causal, scale, 0, -1, nullptr, batch, false, stream);
}

TTM_EXPORT int ttm_sdpa_decode_concat_heads(const void *q, const void *k, const void *v, const int32_t *cur_pos, const void *mask,
                                            int mask_heads, const int32_t *page_table, int64_t pages_per_user, int64_t page_block,
                                            int64_t page_blocks, void *out, int dtype, int64_t batch, int64_t heads, int64_t kv_heads,
                                            int64_t seq, int64_t head_dim, int is_causal, float scale, void *stream) {
  TTM_EXTENTS(sdpa_decode, q, k, v, cur_pos, mask, mask_heads, batch, page_table, pages_per_user, page_block, page_blocks, out, dtype, batch, heads, kv_heads, seq, head_dim, 1, nullptr);
  return sdpa_decode_entry(q, k, v, cur_pos, mask, mask_heads, page_table, pages_per_user, page_block, page_blocks, out, dtype, batch, heads, kv_heads,
                           seq, head_dim, is_causal, scale, 1, -1, nullptr, batch, false, stream);
}

TTM_EXPORT int ttm_sdpa_decode_windowed(const void *q, const void *k, const void *v, const int32_t *cur_pos, const void *mask,
                                        int mask_heads, int64_t mask_batch, const int32_t *page_table, int64_t pages_per_user,
                                        int64_t page_block, int64_t page_blocks, void *out, int dtype, int64_t batch, int64_t heads, int64_t kv_heads,
                                        int64_t seq, int64_t head_dim, int is_causal, float scale, int concat_heads, int64_t sliding_window,
                                        const void *attention_sink, void *stream) {
  TTM_EXTENTS(sdpa_decode, q, k, v, cur_pos, mask, mask_heads, mask_batch, page_table, pages_per_user, page_block, page_blocks, out, dtype, batch, heads, kv_heads, seq, head_dim, concat_heads, attention_sink);
  return sdpa_decode_entry(q, k, v, cur_pos, mask, mask_heads, page_table, pages_per_user, page_block, page_blocks, out, dtype, batch, heads, kv_heads,
                           seq, head_dim, is_causal, scale, concat_heads != 0, sliding_window, attention_sink, mask_batch, false, stream);
}

// ttm_sdpa_decode_windowed for callers that cannot allocate: the slots come from the library's static device array.
TTM_EXPORT int ttm_sdpa_decode_static(const void *q, const void *k, const void *v, const int32_t *cur_pos, const void *mask,
                                      int mask_heads, int64_t mask_batch, const int32_t *page_table, int64_t pages_per_user,
                                      int64_t page_block, int64_t page_blocks, void *out, int dtype, int64_t batch, int64_t heads, int64_t kv_heads,
                                      int64_t seq, int64_t head_dim, int is_causal, float scale, int concat_heads, int64_t sliding_window,
                                      const void *attention_sink, void *stream) {
  TTM_EXTENTS(sdpa_decode, q, k, v, cur_pos, mask, mask_heads, mask_batch, page_table, pages_per_user, page_block, page_blocks, out, dtype, batch, heads, kv_heads, seq, head_dim, concat_heads, attention_sink);
  return sdpa_decode_entry(q, k, v, cur_pos, mask, mask_heads, page_table, pages_per_user, page_block, page_blocks, out, dtype, batch, heads, kv_heads,
                           seq, head_dim, is_causal, scale, concat_heads != 0, sliding_window, attention_sink, mask_batch, true, stream);
}

TTM_EXPORT int ttm_paged_gather(const void *cache, const int32_t *page_table, void *out, int dtype, int64_t blocks, int64_t heads,
                                int64_t block_size, int64_t head_dim, int64_t users, int64_t pages_per_user, void *stream) {
  TTM_EXTENTS(paged_gather, cache, page_table, out, dtype, blocks, heads, block_size, head_dim, users, pages_per_user);
  TTM_REQUIRE(cache && page_table && out, "ttm_paged_gather: null pointer");
  TTM_REQUIRE(dtype == TTM_BF16 || dtype == TTM_F32, "ttm_paged_gather: dtype must be BFloat16 or Float32");
  TTM_REQUIRE(head_dim > 0 && head_dim % 32 == 0, "ttm_paged_gather: head dim must be a positive multiple of 32");
  TTM_REQUIRE(block_size > 0 && block_size % 32 == 0, "ttm_paged_gather: block size must be a positive multiple of 32");
  TTM_REQUIRE(blocks > 0 && heads > 0 && users >= 0 && pages_per_user > 0, "ttm_paged_gather: bad extents");
  const int64_t total8 = users * heads * pages_per_user * block_size * (head_dim / 8);
  if (total8 == 0) return TTM_OK;
  const dim3 grid((unsigned)ttm_cdiv(total8, 256));
  if (dtype == TTM_BF16)
    hipLaunchKernelGGL(ttm_paged_gather_k<uint16_t>, grid, dim3(256), 0, (hipStream_t)stream, (const uint16_t *)cache, page_table,
                       (uint16_t *)out, blocks, heads, block_size, head_dim, pages_per_user, total8);
  else
    hipLaunchKernelGGL(ttm_paged_gather_k<float>, grid, dim3(256), 0, (hipStream_t)stream, (const float *)cache, page_table, (float *)out,
                       blocks, heads, block_size, head_dim, pages_per_user, total8);
  TTM_LAUNCH_CHECK();
  return TTM_OK;
}

TTM_EXPORT int ttm_chunk_causal_mask(void *mask, const int32_t *chunk_start, int64_t rows, int64_t cols, void *stream) {
  TTM_EXTENTS(chunk_causal_mask, mask, chunk_start, rows, cols);
  TTM_REQUIRE(mask && chunk_start, "ttm_chunk_causal_mask: null pointer");
  TTM_REQUIRE(rows > 0 && cols > 0, "ttm_chunk_causal_mask: bad extents");
  const int64_t rp = ttm_round_up32(rows), cp = ttm_round_up32(cols), total8 = rp * cp / 8;
  hipLaunchKernelGGL(ttm_chunk_mask_k, dim3((unsigned)ttm_cdiv(total8, 256)), dim3(256), 0, (hipStream_t)stream, (uint16_t *)mask,
                     chunk_start, rp, cp, total8);
  TTM_LAUNCH_CHECK();
  return TTM_OK;
}

TTM_EXPORT int ttm_rotary_embedding_llama(const void *x, const void *cos_cache, const void *sin_cache, const void *trans_mat, void *out,
                                          int dtype, int64_t batch, int64_t rows, int64_t cols, int64_t cs_batch, int64_t cs_rows,
                                          void *stream) {
  TTM_EXTENTS(rotary_embedding_llama, x, cos_cache, sin_cache, trans_mat, out, dtype, batch, rows, cols, cs_batch, cs_rows);
  TTM_REQUIRE(x && cos_cache && sin_cache && trans_mat && out, "ttm_rotary_embedding_llama: null pointer");
  TTM_REQUIRE(dtype == TTM_BF16, "ttm_rotary_embedding_llama: tensors must be BFloat16");
  TTM_REQUIRE(batch >= 0 && rows > 0 && cols > 0 && cols % 32 == 0 && cols <= 256,
              "ttm_rotary_embedding_llama: head dim must be a multiple of 32 up to 256");
  TTM_REQUIRE(cs_batch >= 1 && (cs_rows == 1 || cs_rows == rows), "ttm_rotary_embedding_llama: cos / sin must have 1 or %lld rows",
              (long long)rows);
  const int64_t rp = ttm_round_up32(rows), total = batch * rp * cols;
  if (total == 0) return TTM_OK;
  hipLaunchKernelGGL(ttm_rotary_llama_k, dim3((unsigned)ttm_cdiv(total, 256)), dim3(256), 0, (hipStream_t)stream, (const uint16_t *)x,
                     (const uint16_t *)cos_cache, (const uint16_t *)sin_cache, (const uint16_t *)trans_mat, (uint16_t *)out, rows, rp, cols,
                     cs_batch, cs_rows, ttm_round_up32(cs_rows), total);
  TTM_LAUNCH_CHECK();
  return TTM_OK;
}
