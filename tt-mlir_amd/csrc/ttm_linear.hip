// Dense contraction: C[M,N] = act(A[M,K] . W[K,N] + bias[N]), bf16 activations, bf16 or
// block-float (bfp8_b / bfp4_b) weights, fp32 accumulation on the bf16 MFMA pipe, bf16 output.
// All operands are in Tenstorrent tile order (32x32 tiles, 16x16 faces); block-float weights are
// consumed as packed tiles straight from HBM and dequantised on the way into LDS.
//
// Mapping to the matrix core.  v_mfma_f32_32x32x16_bf16 wants, for both inputs, 8 consecutive k
// per lane.  The weight tile is the MFMA "A" input (rows = n) and the activation tile the "B"
// input (columns = m), so a lane's four accumulator registers of one group are four consecutive
// n of one m: an 8-byte store into the output face row, and bias is a per-register constant.
//
// LDS image (both operands): [row][8 chunks of 8 k] with the chunk slot XOR-swizzled by the row (lds_swz);
// a fragment read is one ds_read_b128 per lane and is bank-conflict free.
//
// Weight dequantisation (bfp8_b).  A lane owns an 8 (k) x 4 (n) block (8 x 8 in the fallback and small-M
// kernels): eight row words plus the eight row exponents.  Sign-magnitude bytes are turned into
// offset-binary bytes with packed integer ops (t = 128 +- mag), so an element is cvt_f32_ubyte + one fma:
//     w = t * 2^(E-133) - 128 * 2^(E-133)          (exact)
// and pairs along k are packed to bf16 by taking the high halves (exact: 7 significant bits).
// Rows whose shared exponent is below 7 (|w| < 2^-120) are flushed to zero.
//
// Kernels, by use: ttm_linear_dma_k (block-float weights, M > 64), ttm_linear_reg_k (bf16 weights, M > 64),
// ttm_linear_big_k (64-bit-addressed fallback), ttm_linear_decode_k / ttm_linear_small_k (M <= 64),
// ttm_linear_reduce_k (second half of a split-K launch).
#include <type_traits>

#include "ttm_common.h"
#include "ttm_math.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

enum { WF_BFP8 = 0, WF_BFP4 = 1, WF_BF16_KN = 2, WF_BF16_NK = 3 };

struct LinearArgs {
  const uint8_t *A;     // bf16, tile order, [Mt*32, Kt*32]
  const uint8_t *W;     // weights, format WF_*
  const uint16_t *bias; // bf16 or null
  uint8_t *C;           // bf16, tile order, [Mt*32, Nt*32]
  int Mt, Nt, Kt;       // extents in tiles
  int act, bias_tiled;
  int64_t a_batch, w_batch, c_batch;  // byte strides between batch entries (w_batch 0 = shared weights)
  int m_blocks, n_blocks;
  int ntw;                            // block-float main kernel: column tiles per wavefront (block width / 2)
  int nt_split, n_blocks1, ntw2;      // two-part grid: blocks [0, n_blocks1) cover column tiles [0, nt_split) at width ntw,
                                      // the rest cover [nt_split, Nt) at width ntw2; nt_split = 0: one part
  int k_slice;                        // k-tiles per grid.y slice (split-K); Kt when the reduction is not split
  float *partial;                     // split-K: fp32 partial sums [slices][Mt * Nt * 1024] in output tile order
  int img_zero_step;                  // two-pass launch: W points at the dequantised images, this step index holds zeros
  // group launch (group_n >= 2): several weight matrices [K, N_i] applied to the same activations, each with its own
  // output; W / C / Nt above describe the virtual concatenation (Nt = sum of the members' column tiles) and are not
  // dereferenced.  Each member may have its own activation; no bias, tail or batch in a group.
  int group_n;
  const uint8_t *gW[4];
  uint8_t *gC[4];
  int gNt[4];
  int gAct[4];                        // per-member activation
  int glu;                            // gated pair (decode kernel only): C = gC[0] = act0(A gW[0]) x act1(A gW[1]), both [K, gNt[0] * 32]
  int tail;                           // 0 none, 1 add, 2 multiply: element-wise tail with a tensor laid out like the output
  int64_t tail_delta;                 // byte distance from an output element to its tail operand
  const struct QkvFinishArgs *qkv;    // host side only: the decode launch leaves partial sums and ttm_qkv_finish_k ends it
  const struct NormFinishArgs *norm;  // host side only: ... and the RMSNorm kernel ends it (residual add, then the norm)
};

// x1 = residual + projection (stored to sum_out), then out = rms_norm(x1): the operands of the second launch
struct NormFinishArgs {
  const void *residual, *weight, *bias;
  int weight_layout, bias_layout;
  void *sum_out, *out;
  int64_t rows, cols;
  float eps;
};

// What follows the Q, K and V projections of a decode step (one token per user): head split, rotary embedding of q and k
// at the cos / sin row `cos_row`, q to its own tensor, k and v into the cache row of position *index.
struct QkvFinishArgs {
  const float *partial;               // [slices][per] fp32 in tile order over the concatenation q | k | v (one row tile)
  int slices;
  int64_t per;
  int users, heads, heads_pad, kv_heads, dim;
  const uint16_t *cosc, *sinc;        // [.., dim] bf16 tiles
  int64_t cos_row;
  uint16_t *q_out;                    // [1, users, heads, dim] bf16 tiles
  uint16_t *k_cache, *v_cache;        // [cache users, kv_heads, max_seq, dim] bf16 tiles
  int64_t max_seq, seq_pad, batch_offset;
  const int32_t *index;               // device memory: the position all users write
};

// The member of a group launch that owns column unit `u`, where a unit is `unit_tiles` column tiles and every member's
// units are numbered one after another (a member's last unit may be partial).  Constant indices only: the arrays stay in
// scalar registers.
struct GroupMember {
  const uint8_t *W;
  uint8_t *C;
  int Nt, local, tile_base, act;   // column tiles, unit index inside the member, first column tile in the concatenation
};
__device__ __forceinline__ GroupMember group_member(const LinearArgs &p, int u, int unit_tiles) {
  GroupMember m = {p.gW[0], p.gC[0], p.gNt[0], u, 0, p.gAct[0]};
  int start = 0, tiles = 0;
  bool found = false;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    if (j < p.group_n) {
      const int n = (p.gNt[j] + unit_tiles - 1) / unit_tiles;
      if (!found && (u < start + n || j == p.group_n - 1)) {
        found = true;
        m.W = p.gW[j]; m.C = p.gC[j]; m.Nt = p.gNt[j]; m.local = u - start; m.tile_base = tiles; m.act = p.gAct[j];
      }
      start += n; tiles += p.gNt[j];
    }
  }
  return m;
}

template <int ACT>
__device__ __forceinline__ float apply_act(float x) {
  if (ACT == TTM_ACT_GELU) return ttm_gelu_fast(x);
  if (ACT == TTM_ACT_SILU) return ttm_silu(x);
  if (ACT == TTM_ACT_SIGMOID) return ttm_sigmoid(x);
  if (ACT == TTM_ACT_RELU) return ttm_max(x, 0.0f);   // keeps NaN, as arith.maximumf does
  return x;
}

typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef float f32x2_t __attribute__((ext_vector_type(2)));
// two floats -> packed bf16 pair, round to nearest even (v_cvt_pk_bf16_f32)
__device__ __forceinline__ uint32_t pack_bf16(float a, float b) {
  f32x2_t v = {a, b};
  bf16x2_t h = __builtin_convertvector(v, bf16x2_t);
  return *(uint32_t *)&h;
}

// Four consecutive outputs -> bf16, optionally followed by the element-wise tail.  The result is rounded to bf16 before the
// tail and again after it, exactly as a separate binary op on the stored result would do.
__device__ __forceinline__ u32x2 finish_quad(const LinearArgs &p, const uint8_t *cptr, const float (&v)[4]) {
  u32x2 o = {pack_bf16(v[0], v[1]), pack_bf16(v[2], v[3])};
  if (p.tail != 0) {   // uniform
    const u32x2 r = *(const u32x2 *)(cptr + p.tail_delta);
    const float y[4] = {__uint_as_float(o.x << 16), __uint_as_float(o.x & 0xFFFF0000u), __uint_as_float(o.y << 16),
                        __uint_as_float(o.y & 0xFFFF0000u)};
    const float t[4] = {__uint_as_float(r.x << 16), __uint_as_float(r.x & 0xFFFF0000u), __uint_as_float(r.y << 16),
                        __uint_as_float(r.y & 0xFFFF0000u)};
    float z[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) z[i] = p.tail == 1 ? y[i] + t[i] : y[i] * t[i];
    o = u32x2{pack_bf16(z[0], z[1]), pack_bf16(z[2], z[3])};
  }
  return o;
}

// LDS image of an operand block: [row][8 chunks of 8 k], chunk slot XOR-swizzled by the row so that every
// group of 8 consecutive lanes hits 8 distinct 16-byte slots in all three access patterns: fragment
// reads (8 consecutive rows), activation copies (4 rows x 2 chunks) and dequantised weight writes
// (rows 8 apart x 2 chunks).
__device__ __forceinline__ int lds_swz(int row) { return (((row << 1) & 6) | ((row >> 2) & 1)) ^ (((row >> 3) & 3) << 1); }
__device__ __forceinline__ int lds_chunk(int row, int kc) { return row * 8 + (kc ^ lds_swz(row)); }
// The images of the two-pass route (written by the image pass, read by the second pass as 16 rows x four chunks per
// ds_read_b128 for v_mfma_f32_16x16x32_bf16) swizzle the slot by the low three row bits instead: under that read the
// swizzle above puts pairs of lanes on one bank group (51 against 32 cycles per instruction with eight wavefronts reading),
// this one none.
__device__ __forceinline__ int lds_swz16(int row) { return row & 7; }
__device__ __forceinline__ int lds_chunk16(int row, int kc) { return row * 8 + (kc ^ lds_swz16(row)); }

// high halves of two floats -> packed bf16 pair (lo = a, hi = b); exact for dequantised weights
__device__ __forceinline__ uint32_t pack_hi(float a, float b) {
  return __builtin_amdgcn_perm(__float_as_uint(b), __float_as_uint(a), 0x07060302u);
}

// ---- bfp8: 8 rows (k) x 8 bytes (n) + 8 exponents -> 8 chunks (one per n) of 8 k
__device__ __forceinline__ void dequant_bfp8_block(const u32x2 (&rows)[8], u32x2 exps, u32x4 (&out)[8]) {
  float f[8][8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    uint32_t E = ((i < 4 ? exps.x : exps.y) >> (8 * (i & 3))) & 0xFFu;
    E = max(E, 7u);
    float scale = __uint_as_float((E - 6u) << 23);       // 2^(E-133)
    float nscale = -128.0f * scale;
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      uint32_t d = h ? rows[i].y : rows[i].x;
      uint32_t sg = d & 0x80808080u;
      uint32_t sb = sg >> 7;
      uint32_t t = (d ^ 0x80808080u ^ (sg - sb)) + sb;    // per byte: 128 + mag or 128 - mag
#pragma unroll
      for (int b = 0; b < 4; ++b)
        f[i][h * 4 + b] = fmaf((float)((t >> (8 * b)) & 0xFFu), scale, nscale);
    }
  }
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    out[j].x = pack_hi(f[0][j], f[1][j]);
    out[j].y = pack_hi(f[2][j], f[3][j]);
    out[j].z = pack_hi(f[4][j], f[5][j]);
    out[j].w = pack_hi(f[6][j], f[7][j]);
  }
}

// ---- bfp4: 8 rows (k) x 8 nibbles (n)
__device__ __forceinline__ void dequant_bfp4_block(const uint32_t (&rows)[8], u32x2 exps, u32x4 (&out)[8]) {
  float f[8][8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    uint32_t E = ((i < 4 ? exps.x : exps.y) >> (8 * (i & 3))) & 0xFFu;
    E = max(E, 3u);
    float scale = __uint_as_float((E - 2u) << 23);       // 2^(E-129)
    float nscale = -8.0f * scale;
    uint32_t d = rows[i];
    uint32_t sg = d & 0x88888888u;
    uint32_t sb = sg >> 3;
    uint32_t t = (d ^ 0x88888888u ^ (sg - sb)) + sb;      // per nibble: 8 + mag or 8 - mag
#pragma unroll
    for (int b = 0; b < 8; ++b) f[i][b] = fmaf((float)((t >> (4 * b)) & 0xFu), scale, nscale);
  }
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    out[j].x = pack_hi(f[0][j], f[1][j]);
    out[j].y = pack_hi(f[2][j], f[3][j]);
    out[j].z = pack_hi(f[4][j], f[5][j]);
    out[j].w = pack_hi(f[6][j], f[7][j]);
  }
}

// ---- bf16 [K,N]: 8 rows (k) x 8 bf16 (n) -> transpose
__device__ __forceinline__ void transpose_bf16_block(const u32x4 (&rows)[8], u32x4 (&out)[8]) {
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    const uint32_t sel = (j & 1) ? 0x07060302u : 0x05040100u;
#pragma unroll
    for (int p = 0; p < 4; ++p)
      out[j][p] = __builtin_amdgcn_perm(rows[2 * p + 1][j >> 1], rows[2 * p][j >> 1], sel);
  }
}

// =============================================================================================
// Large-M kernel: 256 (m) x 256 (n) block tile, BK = 64, 4 wavefronts of 128 x 128.
// =============================================================================================
template <int WF>
struct WRegs {  // raw weight data of one k-step held by a lane between the global load and the LDS write
  u32x2 rows8[WF == WF_BFP8 ? 8 : 1];
  uint32_t rows4[WF == WF_BFP4 ? 8 : 1];
  u32x4 rows16[WF == WF_BF16_KN ? 8 : 1];
  u32x4 direct[WF == WF_BF16_NK ? 8 : 1];
  u32x2 exps;
};

template <int WF>
__device__ __forceinline__ void load_w(const LinearArgs &p, const uint8_t *W, int nt0, int kt0, int tid, WRegs<WF> &r) {
  if constexpr (WF == WF_BF16_NK) {
    // weights stored [N,K] in tile order: same chunk copy as the activations
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      int nt = nt0 + i, kt = kt0 + (tid >> 7);
      bool ok = nt < p.Nt && kt < p.Kt;
      const u32x4 *src = (const u32x4 *)(W + ((int64_t)nt * p.Kt + kt0) * 2048) + tid;
      r.direct[i] = ok ? *src : u32x4{0, 0, 0, 0};
    }
    return;
  }
  const int tile_l = tid >> 4, w = tid & 15;
  const int kt = kt0 + (tile_l >> 3), nt = nt0 + (tile_l & 7);
  const int face = w >> 2, khalf = (w >> 1) & 1, oct = w & 1;
  const bool ok = kt < p.Kt && nt < p.Nt;
  const int64_t tile = (int64_t)kt * p.Nt + nt;
  if constexpr (WF == WF_BFP8) {
    const uint8_t *t = W + tile * 1088;
    r.exps = ok ? *(const u32x2 *)(t + face * 16 + khalf * 8) : u32x2{0, 0};
    const uint8_t *m = t + 64 + face * 256 + khalf * 128 + oct * 8;
#pragma unroll
    for (int i = 0; i < 8; ++i) r.rows8[i] = ok ? *(const u32x2 *)(m + i * 16) : u32x2{0, 0};
  } else if constexpr (WF == WF_BFP4) {
    const uint8_t *t = W + tile * 576;
    r.exps = ok ? *(const u32x2 *)(t + face * 16 + khalf * 8) : u32x2{0, 0};
    const uint8_t *m = t + 64 + face * 128 + khalf * 64 + oct * 4;
#pragma unroll
    for (int i = 0; i < 8; ++i) r.rows4[i] = ok ? *(const uint32_t *)(m + i * 8) : 0u;
  } else {
    const uint8_t *m = W + tile * 2048 + face * 512 + khalf * 256 + oct * 16;
#pragma unroll
    for (int i = 0; i < 8; ++i) r.rows16[i] = ok ? *(const u32x4 *)(m + i * 32) : u32x4{0, 0, 0, 0};
  }
}

// chunk position of the tile-order copy pattern used for activations (and [N,K] weights):
// lane tid covers chunk `tid` of a 4 KiB pair of k-tiles; iteration i selects row tile i.
__device__ __forceinline__ int copy_lds_chunk(int tid, int i) {
  int kt_l = tid >> 7, cc = tid & 127;
  int face = cc >> 5, row = (cc & 31) >> 1, half = cc & 1;
  int r = i * 32 + (face >> 1) * 16 + row;
  int kc = kt_l * 4 + (face & 1) * 2 + half;
  return lds_chunk(r, kc);
}

template <int WF>
__device__ __forceinline__ void store_w(u32x4 *ldsW, int tid, const WRegs<WF> &r) {
  if constexpr (WF == WF_BF16_NK) {
#pragma unroll
    for (int i = 0; i < 8; ++i) ldsW[copy_lds_chunk(tid, i)] = r.direct[i];
  } else {
    const int tile_l = tid >> 4, w = tid & 15;
    const int face = w >> 2, khalf = (w >> 1) & 1, oct = w & 1;
    const int kc = (tile_l >> 3) * 4 + (face >> 1) * 2 + khalf;
    const int n0 = (tile_l & 7) * 32 + (face & 1) * 16 + oct * 8;
    u32x4 out[8];
    if constexpr (WF == WF_BFP8) dequant_bfp8_block(r.rows8, r.exps, out);
    else if constexpr (WF == WF_BFP4) dequant_bfp4_block(r.rows4, r.exps, out);
    else transpose_bf16_block(r.rows16, out);
#pragma unroll
    for (int j = 0; j < 8; ++j) ldsW[lds_chunk(n0 + j, kc)] = out[j];
  }
}

// bias, activation, bf16, 8-byte stores into the output face rows.  acc[a][b]: n tile a, m tile b of the
// wavefront; a lane holds m = lane % 32 and n = 8 g + 4 (lane / 32) + r in register g * 4 + r.
// bias, activation, bf16, and 8-byte stores into the output face rows for a wavefront's NA x MB accumulator tiles;
// column tiles at or beyond nt_end are left alone
template <int ACT, int NA, int MB>
__device__ __forceinline__ void linear_epilogue(const LinearArgs &p, uint8_t *C, f32x16 (&acc)[NA][MB], int mtw, int ntw, int nt_end, int lane) {
  const int m_in = lane & 31;
#pragma unroll
  for (int a = 0; a < NA; ++a) {
    const int nt = ntw + a;
    if (nt >= nt_end) continue;
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const int n_in = g * 8 + (lane >> 5) * 4;
      float bv[4] = {0.f, 0.f, 0.f, 0.f};
      if (p.bias) {
        const int n = nt * 32 + n_in;
        const uint16_t *bp = p.bias_tiled ? p.bias + (int64_t)nt * 1024 + (n_in >> 4) * 256 + (n_in & 15) : p.bias + n;
        u32x2 raw = *(const u32x2 *)bp;
        bv[0] = __uint_as_float(raw.x << 16); bv[1] = __uint_as_float(raw.x & 0xFFFF0000u);
        bv[2] = __uint_as_float(raw.y << 16); bv[3] = __uint_as_float(raw.y & 0xFFFF0000u);
      }
#pragma unroll
      for (int b = 0; b < MB; ++b) {
        const int mt = mtw + b;
        if (mt >= p.Mt) continue;
        float v[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) v[r] = apply_act<ACT>(acc[a][b][g * 4 + r] + bv[r]);
        int64_t off = ((int64_t)mt * p.Nt + nt) * 1024 + ((m_in >> 4) * 2 + (n_in >> 4)) * 256 + (m_in & 15) * 16 + (n_in & 15);
        *(u32x2 *)(C + off * 2) = finish_quad(p, C + off * 2, v);
      }
    }
  }
}
// split-K: fp32 partial sums of a wavefront's accumulator tiles, same element order as the bf16 output
template <int NA, int MB>
__device__ __forceinline__ void linear_store_partial(const LinearArgs &p, float *P, f32x16 (&acc)[NA][MB], int mtw, int ntw, int nt_end, int lane) {
  const int m_in = lane & 31;
#pragma unroll
  for (int a = 0; a < NA; ++a) {
    const int nt = ntw + a;
    if (nt >= nt_end) continue;
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const int n_in = g * 8 + (lane >> 5) * 4;
#pragma unroll
      for (int b = 0; b < MB; ++b) {
        const int mt = mtw + b;
        if (mt >= p.Mt) continue;
        const int64_t off = ((int64_t)mt * p.Nt + nt) * 1024 + ((m_in >> 4) * 2 + (n_in >> 4)) * 256 + (m_in & 15) * 16 + (n_in & 15);
        *(f32x4 *)(P + off) = f32x4{acc[a][b][g * 4], acc[a][b][g * 4 + 1], acc[a][b][g * 4 + 2], acc[a][b][g * 4 + 3]};
      }
    }
  }
}

// gated launch: the wavefront's accumulator tiles alternate between the two matrices (tile 2 j: columns of the first, tile
// 2 j + 1: the same columns of the second); out = round(round(act0(first)) x round(act1(second))) into column tile
// ntw / 2 + j of the output, whose rows are NtR tiles long.  No bias.
__device__ __forceinline__ float linear_act_rt(int act, float x) {
  switch (act) {
  case TTM_ACT_GELU: return apply_act<TTM_ACT_GELU>(x);
  case TTM_ACT_SILU: return apply_act<TTM_ACT_SILU>(x);
  case TTM_ACT_SIGMOID: return apply_act<TTM_ACT_SIGMOID>(x);
  case TTM_ACT_RELU: return apply_act<TTM_ACT_RELU>(x);
  default: return x;
  }
}
template <int NA, int MB>
__device__ __forceinline__ void linear_epilogue_glu(const LinearArgs &p, uint8_t *C, f32x16 (&acc)[NA][MB], int mtw, int ntw, int nt_end, int NtR, int lane) {
  static_assert(NA % 2 == 0, "pairs of column tiles");
  const int m_in = lane & 31;
  const int act0 = p.gAct[0], act1 = p.gAct[1];
#pragma unroll
  for (int j = 0; j < NA / 2; ++j) {
    if (ntw + 2 * j >= nt_end) continue;
    const int nt = (ntw >> 1) + j;
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const int n_in = g * 8 + (lane >> 5) * 4;
#pragma unroll
      for (int b = 0; b < MB; ++b) {
        const int mt = mtw + b;
        if (mt >= p.Mt) continue;
        float x[4], y[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          x[r] = linear_act_rt(act0, acc[2 * j][b][g * 4 + r]);
          y[r] = linear_act_rt(act1, acc[2 * j + 1][b][g * 4 + r]);
        }
        const u32x2 gq = {pack_bf16(x[0], x[1]), pack_bf16(x[2], x[3])}, uq = {pack_bf16(y[0], y[1]), pack_bf16(y[2], y[3])};
        const float z[4] = {__uint_as_float(gq.x << 16) * __uint_as_float(uq.x << 16), __uint_as_float(gq.x & 0xFFFF0000u) * __uint_as_float(uq.x & 0xFFFF0000u),
                            __uint_as_float(gq.y << 16) * __uint_as_float(uq.y << 16), __uint_as_float(gq.y & 0xFFFF0000u) * __uint_as_float(uq.y & 0xFFFF0000u)};
        const int64_t off = ((int64_t)mt * NtR + nt) * 1024 + ((m_in >> 4) * 2 + (n_in >> 4)) * 256 + (m_in & 15) * 16 + (n_in & 15);
        *(u32x2 *)(C + off * 2) = u32x2{pack_bf16(z[0], z[1]), pack_bf16(z[2], z[3])};
      }
    }
  }
}

// split-K: sums the slices, then bias, activation and bf16 as in the fused epilogue; one lane per four elements
__global__ __launch_bounds__(256) void ttm_linear_reduce_k(LinearArgs p, int slices) {
  const int64_t per = (int64_t)p.Mt * p.Nt * 1024;
  const int64_t q = (int64_t)blockIdx.x * 256 + threadIdx.x;   // group of four consecutive elements
  if (q * 4 >= per) return;
  const float *P = p.partial + (int64_t)blockIdx.z * slices * per + q * 4;
  f32x4 sum = *(const f32x4 *)P;
  for (int s = 1; s < slices; ++s) sum += *(const f32x4 *)(P + s * per);
  const int64_t off = q * 4;
  const int nt = (int)((off >> 10) % p.Nt), in = (int)(off & 1023);
  const int n_in = ((in >> 8) & 1) * 16 + (in & 15);
  float bv[4] = {0.f, 0.f, 0.f, 0.f};
  if (p.bias) {
    const uint16_t *bp = p.bias_tiled ? p.bias + (int64_t)nt * 1024 + (n_in >> 4) * 256 + (n_in & 15) : p.bias + nt * 32 + n_in;
    u32x2 raw = *(const u32x2 *)bp;
    bv[0] = __uint_as_float(raw.x << 16); bv[1] = __uint_as_float(raw.x & 0xFFFF0000u);
    bv[2] = __uint_as_float(raw.y << 16); bv[3] = __uint_as_float(raw.y & 0xFFFF0000u);
  }
  GroupMember m = {};
  int act = p.act;
  if (p.group_n > 1) {   // one row tile (decode): tile nt of the concatenation belongs to one member
    m = group_member(p, nt, 1);
    act = m.act;
  }
  float v[4];
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    float x = sum[r] + bv[r];
    switch (act) {
    case TTM_ACT_GELU: x = apply_act<TTM_ACT_GELU>(x); break;
    case TTM_ACT_SILU: x = apply_act<TTM_ACT_SILU>(x); break;
    case TTM_ACT_SIGMOID: x = apply_act<TTM_ACT_SIGMOID>(x); break;
    case TTM_ACT_RELU: x = apply_act<TTM_ACT_RELU>(x); break;
    default: break;
    }
    v[r] = x;
  }
  if (p.group_n > 1) {
    uint8_t *Cm = m.C + ((int64_t)m.local * 1024 + in) * 2;
    *(u32x2 *)Cm = finish_quad(p, Cm, v);
    return;
  }
  uint8_t *C = p.C + (int64_t)blockIdx.z * p.c_batch;
  *(u32x2 *)(C + off * 2) = finish_quad(p, C + off * 2, v);
}

template <int NA, int MB>
__device__ __forceinline__ void linear_epilogue_act(const LinearArgs &p, uint8_t *C, f32x16 (&acc)[NA][MB], int mtw, int ntw, int nt_end, int lane) {
  switch (p.act) {   // uniform
  case TTM_ACT_GELU: linear_epilogue<TTM_ACT_GELU>(p, C, acc, mtw, ntw, nt_end, lane); break;
  case TTM_ACT_SILU: linear_epilogue<TTM_ACT_SILU>(p, C, acc, mtw, ntw, nt_end, lane); break;
  case TTM_ACT_SIGMOID: linear_epilogue<TTM_ACT_SIGMOID>(p, C, acc, mtw, ntw, nt_end, lane); break;
  case TTM_ACT_RELU: linear_epilogue<TTM_ACT_RELU>(p, C, acc, mtw, ntw, nt_end, lane); break;
  default: linear_epilogue<TTM_ACT_NONE>(p, C, acc, mtw, ntw, nt_end, lane); break;
  }
}

// The same three steps for accumulators of v_mfma_f32_16x16x32_bf16: acc[u][v] is the 16 (n) x 16 (m) tile u of the
// wavefront's columns and v of its rows; a lane holds m = lane % 16 and n = 4 (lane / 16) + r in register r.
template <int ACT, int NU, int NV>
__device__ __forceinline__ void linear_epilogue16(const LinearArgs &p, uint8_t *C, f32x4 (&acc)[NU][NV], int mtw, int ntw, int nt_end, int lane) {
  const int m16 = lane & 15, n4 = (lane >> 4) * 4;
#pragma unroll
  for (int u = 0; u < NU; ++u) {
    const int nt = ntw + (u >> 1);
    if (nt >= nt_end) continue;
    const int n_in = (u & 1) * 16 + n4;
    float bv[4] = {0.f, 0.f, 0.f, 0.f};
    if (p.bias) {
      const uint16_t *bp = p.bias_tiled ? p.bias + (int64_t)nt * 1024 + (n_in >> 4) * 256 + (n_in & 15) : p.bias + nt * 32 + n_in;
      u32x2 raw = *(const u32x2 *)bp;
      bv[0] = __uint_as_float(raw.x << 16); bv[1] = __uint_as_float(raw.x & 0xFFFF0000u);
      bv[2] = __uint_as_float(raw.y << 16); bv[3] = __uint_as_float(raw.y & 0xFFFF0000u);
    }
#pragma unroll
    for (int v = 0; v < NV; ++v) {
      const int mt = mtw + (v >> 1);
      if (mt >= p.Mt) continue;
      const int m_in = (v & 1) * 16 + m16;
      float x[4];
#pragma unroll
      for (int r = 0; r < 4; ++r) x[r] = apply_act<ACT>(acc[u][v][r] + bv[r]);
      const int64_t off = ((int64_t)mt * p.Nt + nt) * 1024 + ((m_in >> 4) * 2 + (n_in >> 4)) * 256 + (m_in & 15) * 16 + (n_in & 15);
      *(u32x2 *)(C + off * 2) = finish_quad(p, C + off * 2, x);
    }
  }
}
template <int NU, int NV>
__device__ __forceinline__ void linear_store_partial16(const LinearArgs &p, float *P, f32x4 (&acc)[NU][NV], int mtw, int ntw, int nt_end, int lane) {
  const int m16 = lane & 15, n4 = (lane >> 4) * 4;
#pragma unroll
  for (int u = 0; u < NU; ++u) {
    const int nt = ntw + (u >> 1);
    if (nt >= nt_end) continue;
    const int n_in = (u & 1) * 16 + n4;
#pragma unroll
    for (int v = 0; v < NV; ++v) {
      const int mt = mtw + (v >> 1);
      if (mt >= p.Mt) continue;
      const int m_in = (v & 1) * 16 + m16;
      const int64_t off = ((int64_t)mt * p.Nt + nt) * 1024 + ((m_in >> 4) * 2 + (n_in >> 4)) * 256 + (m_in & 15) * 16 + (n_in & 15);
      *(f32x4 *)(P + off) = acc[u][v];
    }
  }
}
template <int NU, int NV>
__device__ __forceinline__ void linear_epilogue_act16(const LinearArgs &p, uint8_t *C, f32x4 (&acc)[NU][NV], int mtw, int ntw, int nt_end, int lane) {
  switch (p.act) {   // uniform
  case TTM_ACT_GELU: linear_epilogue16<TTM_ACT_GELU>(p, C, acc, mtw, ntw, nt_end, lane); break;
  case TTM_ACT_SILU: linear_epilogue16<TTM_ACT_SILU>(p, C, acc, mtw, ntw, nt_end, lane); break;
  case TTM_ACT_SIGMOID: linear_epilogue16<TTM_ACT_SIGMOID>(p, C, acc, mtw, ntw, nt_end, lane); break;
  case TTM_ACT_RELU: linear_epilogue16<TTM_ACT_RELU>(p, C, acc, mtw, ntw, nt_end, lane); break;
  default: linear_epilogue16<TTM_ACT_NONE>(p, C, acc, mtw, ntw, nt_end, lane); break;
  }
}

template <int WF>
__global__ __launch_bounds__(256) void ttm_linear_big_k(LinearArgs p) {
  extern __shared__ u32x4 smem[];  // 2 stages x (A 2048 chunks + W 2048 chunks) = 128 KiB
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wn = wave & 1, wm = wave >> 1;

  // XCD-aware tile order: consecutive workgroup ids land on different XCDs, so give every XCD a
  // contiguous run of logical tiles (same weight panel, successive m blocks).
  const int nblk = p.m_blocks * p.n_blocks;
  int bid = blockIdx.x;
  if (nblk % 8 == 0) bid = (bid & 7) * (nblk >> 3) + (bid >> 3);
  const int nb = bid / p.m_blocks, mb = bid % p.m_blocks;
  const int mt0 = mb * 8, nt0 = nb * 8;
  const uint8_t *A = p.A + (int64_t)blockIdx.z * p.a_batch;
  const uint8_t *W = p.W + (int64_t)blockIdx.z * p.w_batch;
  uint8_t *C = p.C + (int64_t)blockIdx.z * p.c_batch;

  f32x16 acc[4][4];
#pragma unroll
  for (int a = 0; a < 4; ++a)
#pragma unroll
    for (int b = 0; b < 4; ++b)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[a][b][r] = 0.0f;

  u32x4 areg[8];
  WRegs<WF> wreg;
  const int ksteps = (p.Kt + 1) / 2;

  auto load_a = [&](int kt0) {
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      int mt = mt0 + i, kt = kt0 + (tid >> 7);
      bool ok = mt < p.Mt && kt < p.Kt;
      const u32x4 *src = (const u32x4 *)(A + ((int64_t)mt * p.Kt + kt0) * 2048) + tid;
      areg[i] = ok ? *src : u32x4{0, 0, 0, 0};
    }
  };
  auto store_a = [&](u32x4 *ldsA) {
#pragma unroll
    for (int i = 0; i < 8; ++i) ldsA[copy_lds_chunk(tid, i)] = areg[i];
  };

  load_a(0);
  load_w<WF>(p, W, nt0, 0, tid, wreg);
  store_a(smem);
  store_w<WF>(smem + 2048, tid, wreg);
  __syncthreads();

  for (int ks = 0; ks < ksteps; ++ks) {
    u32x4 *ldsA = smem + (ks & 1) * 4096, *ldsW = ldsA + 2048;
    u32x4 *nxtA = smem + ((ks + 1) & 1) * 4096, *nxtW = nxtA + 2048;
    const bool more = ks + 1 < ksteps;
    if (more) {
      load_a((ks + 1) * 2);
      load_w<WF>(p, W, nt0, (ks + 1) * 2, tid, wreg);
    }
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      bf16x8 wf[4], af[4];
      const int kc = 2 * s + (lane >> 5);
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        int rn = wn * 128 + t * 32 + (lane & 31);
        int rm = wm * 128 + t * 32 + (lane & 31);
        u32x4 a = ldsW[lds_chunk(rn, kc)], b = ldsA[lds_chunk(rm, kc)];
        wf[t] = *(bf16x8 *)&a;
        af[t] = *(bf16x8 *)&b;
      }
#pragma unroll
      for (int a = 0; a < 4; ++a)
#pragma unroll
        for (int b = 0; b < 4; ++b)
          acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wf[a], af[b], acc[a][b], 0, 0, 0);
    }
    if (more) {
      store_a(nxtA);
      store_w<WF>(nxtW, tid, wreg);
    }
    __syncthreads();
  }

  linear_epilogue_act(p, C, acc, mt0 + wm * 4, nt0 + wn * 4, p.Nt, lane);
}

template <int WF>
struct W8Regs {  // raw weights of one k-step: an 8 (k) x 4 (n) block per lane (8 x 8 for bf16 [K,N])
  uint32_t rows8[WF == WF_BFP8 ? 8 : 1];
  uint16_t rows4[WF == WF_BFP4 ? 8 : 1];
  u32x2 rows16[WF == WF_BF16_KN ? 8 : 1];
  u32x4 direct[WF == WF_BF16_NK ? 4 : 1];
  u32x2 exps;
};

// activation-style copy with 512 lanes: lane covers chunk (tid & 255) of the 4 KiB k-tile pair of row tile (tid >> 8) + 2 i
__device__ __forceinline__ int copy8_lds_chunk(int tid, int i) { return copy_lds_chunk(tid & 255, (tid >> 8) + 2 * i); }

// =============================================================================================
// Main kernel, operands staged through registers (used for bf16 weights).  512 lanes = 8 wavefronts, each
// owning a 128 (n) x 64 (m) piece of a 256 x 256 output block (128 accumulator registers per lane); k
// advances 64 per step.  Per step a wavefront stores the activations it fetched one step earlier into LDS,
// converts its 8 x 4 weight block into LDS, re-issues the global loads, and runs 24 ds_read_b128 + 32 MFMA
// on the stage converted one step earlier, all in one instruction stream.
// The issue port of a SIMD is shared by MFMA and VALU, which makes the number of VALU instructions per
// step the second budget next to MFMA time.  Hence: every LDS address is a per-lane constant plus an
// immediate (the step loop is unrolled by two so the stage is an immediate too), and every global address
// is a wavefront-uniform base, advanced on the scalar unit, plus a per-lane 32-bit constant.
// LDS: activations 2 x 32 KiB at 0, converted weights 2 x 32 KiB at 64 KiB.
// =============================================================================================
template <int WF>
__global__ __launch_bounds__(512) void ttm_linear_reg_k(LinearArgs p) {
  extern __shared__ u32x4 smem[];
  uint8_t *lds = (uint8_t *)smem;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wn = wave & 1, wm = wave >> 1;
  const int nblk = p.m_blocks * p.n_blocks;
  int bid = blockIdx.x;
  if (nblk % 8 == 0) bid = (bid & 7) * (nblk >> 3) + (bid >> 3);
  const int nb = bid / p.m_blocks, mb = bid % p.m_blocks;
  const int mt0 = mb * 8, nt0 = nb * 8;
  const uint8_t *A = p.A + (int64_t)blockIdx.z * p.a_batch;
  const uint8_t *W = p.W + (int64_t)blockIdx.z * p.w_batch;
  uint8_t *C = p.C + (int64_t)blockIdx.z * p.c_batch;
  constexpr uint32_t LDS_W = 65536, STAGE = 32768;

  f32x16 acc[4][2];
#pragma unroll
  for (int a = 0; a < 4; ++a)
#pragma unroll
    for (int b = 0; b < 2; ++b)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[a][b][r] = 0.0f;

  // ---- per-lane constants
  uint32_t rdW[4], rdA[4];   // fragment reads: + 4096 t + STAGE stage
#pragma unroll
  for (int s = 0; s < 4; ++s) {
    rdW[s] = LDS_W + 16u * lds_chunk(wn * 128 + (lane & 31), 2 * s + (lane >> 5));
    rdA[s] = 16u * lds_chunk(wm * 64 + (lane & 31), 2 * s + (lane >> 5));
  }
  const uint32_t wrA = 16u * copy8_lds_chunk(tid, 0);  // activation copy: + 8192 i + STAGE stage
  // weight unit of this lane: tile (ukt, unt) of the 2 x 8 tiles, face, 8-row half, 4-column quad
  const int ukt = wave >> 2, unt = (tid >> 5) & 7, wq = tid & 31;
  const int face = wq >> 3, khalf = (wq >> 2) & 1, quad = wq & 3;
  uint32_t wrW[4];
  {
    const int kc = ukt * 4 + (face >> 1) * 2 + khalf;
    const int n0 = unt * 32 + (face & 1) * 16 + quad * 4;
#pragma unroll
    for (int j = 0; j < 4; ++j) wrW[j] = LDS_W + 16u * lds_chunk(n0 + j, kc);
  }
  // global offsets relative to the k-tile row (activations: k-tile column) of the step
  const int sub_kt = (wave >> 1) & 1;      // k-tile of the pair that this wavefront copies
  uint32_t offA[4], offWd[4], offWm = 0, offWe = 0;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int mt = min(mt0 + (wave >> 2) + 2 * i, p.Mt - 1);
    offA[i] = (uint32_t)(mt * p.Kt) * 2048u + (uint32_t)(tid & 127) * 16u;
    const int nt = min(nt0 + (wave >> 2) + 2 * i, p.Nt - 1);
    offWd[i] = (uint32_t)(nt * p.Kt) * 2048u + (uint32_t)(tid & 127) * 16u;
  }
  {
    const uint32_t nt = (uint32_t)min(nt0 + unt, p.Nt - 1);
    if constexpr (WF == WF_BFP8) {
      offWe = nt * 1088u + face * 16 + khalf * 8;
      offWm = nt * 1088u + 64 + face * 256 + khalf * 128 + quad * 4;
    } else if constexpr (WF == WF_BFP4) {
      offWe = nt * 576u + face * 16 + khalf * 8;
      offWm = nt * 576u + 64 + face * 128 + khalf * 64 + quad * 2;
    } else if constexpr (WF == WF_BF16_KN) {
      offWm = nt * 2048u + face * 512 + khalf * 256 + quad * 8;
    }
  }
  constexpr uint32_t W_TILE = WF == WF_BFP8 ? 1088u : (WF == WF_BFP4 ? 576u : 2048u);

  const int ksteps = (p.Kt + 1) / 2;
  u32x4 areg[4];
  W8Regs<WF> wreg;

  auto load_regs = [&](int kt0) {
    {
      const int kt = min(kt0 + sub_kt, p.Kt - 1);
      const uint8_t *Ak = A + (int64_t)kt * 2048;
#pragma unroll
      for (int i = 0; i < 4; ++i) areg[i] = *(const u32x4 *)(Ak + offA[i]);
    }
    if constexpr (WF == WF_BF16_NK) {
      const int kt = min(kt0 + sub_kt, p.Kt - 1);
      const uint8_t *Wk = W + (int64_t)kt * 2048;
#pragma unroll
      for (int i = 0; i < 4; ++i) wreg.direct[i] = *(const u32x4 *)(Wk + offWd[i]);
      if (kt0 + sub_kt >= p.Kt) {   // k tail: uniform
#pragma unroll
        for (int i = 0; i < 4; ++i) wreg.direct[i] = u32x4{0, 0, 0, 0};
      }
    } else {
      const int kt = min(kt0 + ukt, p.Kt - 1);
      const uint8_t *Wk = W + (int64_t)kt * p.Nt * W_TILE;
      if constexpr (WF == WF_BFP8) {
        wreg.exps = *(const u32x2 *)(Wk + offWe);
#pragma unroll
        for (int i = 0; i < 8; ++i) wreg.rows8[i] = *(const uint32_t *)(Wk + offWm + i * 16);
      } else if constexpr (WF == WF_BFP4) {
        wreg.exps = *(const u32x2 *)(Wk + offWe);
#pragma unroll
        for (int i = 0; i < 8; ++i) wreg.rows4[i] = *(const uint16_t *)(Wk + offWm + i * 8);
      } else {
#pragma unroll
        for (int i = 0; i < 8; ++i) wreg.rows16[i] = *(const u32x2 *)(Wk + offWm + i * 32);
      }
      // k tail (uniform): block-float tiles get zero exponents, which dequantise to exact zeros
      if constexpr (WF == WF_BFP8 || WF == WF_BFP4) {
        const uint32_t keep = kt0 + ukt >= p.Kt ? 0u : 0xFFFFFFFFu;
        wreg.exps.x &= keep;
        wreg.exps.y &= keep;
      } else if (kt0 + ukt >= p.Kt) {
#pragma unroll
        for (int i = 0; i < 8; ++i) wreg.rows16[i] = u32x2{0, 0};
      }
    }
  };

  // ---- rotated pipeline: MFMA of one stage overlaps the conversion of the next, all in one instruction stream.
  // A step is four chunks of 16 k.  Chunk q multiplies, requests the fragments of the following chunk,
  // stores activation register c and converts weight rows 2c, 2c+1 with c = (q + 1) % 4, and re-issues the
  // global loads of the registers it has just consumed (5 VALU instructions are scheduled behind every MFMA:
  // that is what the matrix core leaves free on the issue port).  The block barrier sits between chunks 2
  // and 3: chunk 3 multiplies from fragments that were requested before the barrier and already requests
  // chunk 0 of the next stage, so the matrix core does not drain at the barrier; its conversion quarter
  // (c = 0) already belongs to the step after next and goes into the stage that the barrier has just freed.
  constexpr bool BFP = WF == WF_BFP8 || WF == WF_BFP4;
  u32x4 fw[2][4], fa[2][2], out[4];
  u32x2 exps_next = {0, 0};
  auto bases = [&](int kt0, const uint8_t *&Ak, const uint8_t *&Wk, uint32_t &keep) {
    const int ktA = min(kt0 + sub_kt, p.Kt - 1);
    Ak = A + (int64_t)ktA * 2048;
    const int ktW = WF == WF_BF16_NK ? ktA : min(kt0 + ukt, p.Kt - 1);
    Wk = W + (int64_t)ktW * (WF == WF_BF16_NK ? 2048 : (int64_t)p.Nt * W_TILE);
    keep = kt0 + (WF == WF_BF16_NK ? sub_kt : ukt) >= p.Kt ? 0u : 0xFFFFFFFFu;   // k tail: zero weights
  };
  auto fetch = [&](int s2, uint32_t so, u32x4 (&w)[4], u32x4 (&a)[2]) {
#pragma unroll
    for (int t = 0; t < 4; ++t) w[t] = *(const u32x4 *)(lds + rdW[s2] + t * 4096 + so);
#pragma unroll
    for (int t = 0; t < 2; ++t) a[t] = *(const u32x4 *)(lds + rdA[s2] + t * 4096 + so);
  };
  // conversion quarter c into the stage at byte offset so; afterwards reloads the consumed registers from (Ak, Wk)
  auto quarter = [&](int c, uint32_t so, const uint8_t *Ak, const uint8_t *Wk, uint32_t keep) {
    *(u32x4 *)(lds + wrA + c * 8192 + so) = areg[c];
    areg[c] = *(const u32x4 *)(Ak + offA[c]);
    if constexpr (WF == WF_BF16_NK) {
      *(u32x4 *)(lds + wrA + LDS_W + c * 8192 + so) = wreg.direct[c];
      u32x4 v = *(const u32x4 *)(Wk + offWd[c]);
      wreg.direct[c] = u32x4{v.x & keep, v.y & keep, v.z & keep, v.w & keep};
    } else if constexpr (WF == WF_BF16_KN) {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const uint32_t sel = (j & 1) ? 0x07060302u : 0x05040100u;
        out[j][c] = __builtin_amdgcn_perm(wreg.rows16[2 * c + 1][j >> 1], wreg.rows16[2 * c][j >> 1], sel);
      }
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        u32x2 v = *(const u32x2 *)(Wk + offWm + (2 * c + h) * 32);
        wreg.rows16[2 * c + h] = u32x2{v.x & keep, v.y & keep};
      }
    } else {
      float f[2][4];
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        const int i = 2 * c + h;
        uint32_t E = ((i < 4 ? wreg.exps.x : wreg.exps.y) >> (8 * (i & 3))) & 0xFFu;
        if constexpr (WF == WF_BFP8) {
          E = max(E, 6u);   // rows below 2^-120, and the zeroed exponents of the k tail, dequantise to zero
          const float scale = __uint_as_float((E - 6u) << 23), nscale = -128.0f * scale;
          const uint32_t d = wreg.rows8[i];
          const uint32_t sg = d & 0x80808080u, sb = sg >> 7;
          const uint32_t t = (d ^ 0x80808080u ^ (sg - sb)) + sb;
#pragma unroll
          for (int b = 0; b < 4; ++b) f[h][b] = fmaf((float)((t >> (8 * b)) & 0xFFu), scale, nscale);
          wreg.rows8[i] = *(const uint32_t *)(Wk + offWm + i * 16);
        } else {
          E = max(E, 2u);
          const float scale = __uint_as_float((E - 2u) << 23), nscale = -8.0f * scale;
          const uint32_t d = wreg.rows4[i];
          const uint32_t sg = d & 0x8888u, sb = sg >> 3;
          const uint32_t t = (d ^ 0x8888u ^ (sg - sb)) + sb;
#pragma unroll
          for (int b = 0; b < 4; ++b) f[h][b] = fmaf((float)((t >> (4 * b)) & 0xFu), scale, nscale);
          wreg.rows4[i] = *(const uint16_t *)(Wk + offWm + i * 8);
        }
      }
#pragma unroll
      for (int j = 0; j < 4; ++j) out[j][c] = pack_hi(f[0][j], f[1][j]);
    }
    if (c == 3 && WF != WF_BF16_NK) {
#pragma unroll
      for (int j = 0; j < 4; ++j) *(u32x4 *)(lds + wrW[j] + so) = out[j];
    }
  };
  auto mfma8 = [&](int buf) {
#pragma unroll
    for (int a = 0; a < 4; ++a)
#pragma unroll
      for (int b = 0; b < 2; ++b)
        acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(*(bf16x8 *)&fw[buf][a], *(bf16x8 *)&fa[buf][b], acc[a][b], 0, 0, 0);
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x002, 5, 0);
    }
  };

  const uint8_t *Ak, *Wk;
  uint32_t keep;
  // prologue: step 0 into stage 0, first quarter of step 1 into stage 1, registers refilled behind each use
  load_regs(0);
  bases(2, Ak, Wk, keep);
#pragma unroll
  for (int c = 0; c < 4; ++c) quarter(c, 0, Ak, Wk, keep);
  if constexpr (BFP) {
    u32x2 e = *(const u32x2 *)(Wk + offWe);
    wreg.exps = u32x2{e.x & keep, e.y & keep};
  }
  __syncthreads();
  fetch(0, 0, fw[0], fa[0]);
  bases(4, Ak, Wk, keep);
  quarter(0, STAGE, Ak, Wk, keep);

  auto step = [&](auto stage_c, int ks) {
    constexpr uint32_t CUR = decltype(stage_c)::value * STAGE, NXT = STAGE - CUR;
    bases((ks + 2) * 2, Ak, Wk, keep);
#pragma unroll
    for (int q = 0; q < 3; ++q) {
      fetch(q + 1, CUR, fw[(q + 1) & 1], fa[(q + 1) & 1]);
      quarter(q + 1, NXT, Ak, Wk, keep);
      if (q == 0 && BFP) {
        u32x2 e = *(const u32x2 *)(Wk + offWe);
        exps_next = u32x2{e.x & keep, e.y & keep};
      }
      mfma8(q & 1);
      __builtin_amdgcn_sched_barrier(0);
    }
    if constexpr (BFP) wreg.exps = exps_next;
    __syncthreads();
    bases((ks + 3) * 2, Ak, Wk, keep);
    fetch(0, NXT, fw[0], fa[0]);
    quarter(0, CUR, Ak, Wk, keep);
    mfma8(1);
    __builtin_amdgcn_sched_barrier(0);
  };
  // an odd number of steps is rounded up: the extra step multiplies zeroed weights
  for (int ks = 0; ks < ksteps; ks += 2) {
    step(std::integral_constant<int, 0>{}, ks);
    step(std::integral_constant<int, 1>{}, ks + 1);
  }
  linear_epilogue_act(p, C, acc, mt0 + wm * 2, nt0 + wn * 4, p.Nt, lane);
}


// =============================================================================================
// Block-float main kernel with LDS-direct global loads.  Same tiling and the same rotated pipeline as
// the fused kernel above, but no operand passes through vector registers on its way in: a wavefront
// instruction that returns 1 KiB into the register file costs issue and register-port time that the
// matrix core would otherwise use, and the activation copy needed a ds_write on top.  Here
//   activations : global_load_lds_dwordx4 straight into the swizzled fragment image (each wavefront loads
//                 the 32 rows of one row tile; the lane -> global chunk map applies the swizzle);
//   mantissas   : global_load_lds_dwordx4 of whole tiles into a raw staging area; the conversion picks its
//                 8 (k) x 4 (n) block out of it with ds_read_b32 (row r = 8 a + i of a tile sits at chunk
//                 8 a + (i ^ a ^ tile parity): conflict free);
//   exponents   : one 8-byte global load per lane and step, as before.
// All LDS-direct loads of a step are issued right behind the block barrier and must have landed at the
// next one (s_waitcnt vmcnt(0) in front of it), one full step later.
// LDS: activations 2 x 32 KiB at 0, dequantised weights 2 x 32 KiB at 64 KiB, raw mantissas 2 x 16 KiB
// (bfp4: 2 x 8 KiB) at 128 KiB.
// =============================================================================================
__device__ __forceinline__ void lds_dma16(const void *base, uint32_t lane_off, uint32_t lds_addr) {
  // lds_addr is wavefront-uniform; lane l of the wavefront writes 16 bytes at lds_addr + 16 l
  asm volatile("s_mov_b32 m0, %2\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(lane_off), "s"(base), "s"(lds_addr) : "memory");
}

// One output block of 2 NTW x 8 tiles (NTW = 4, 3 or 2 column tiles per wavefront); bid / nblk number the blocks of
// the column range [nt_first, nt_end) that this body covers.
// IMG = true is the second pass of a two-pass launch: p.W holds the weights already dequantised to bf16, one 4 KiB
// LDS fragment image per (k-step, column tile) (ttm_linear_image_k), so a step's weights are a straight LDS-direct copy
// and the conversion, the raw staging area and the exponent loads drop out of the loop.
// BN_ = 7 (second pass only) is a block of seven column tiles: the wavefronts of one half take four of them (this body
// with NTW = 4), those of the other half three (NTW = 3), and the two halves are dealt out so that every SIMD runs one
// wavefront of each kind.  Both bodies execute the same sequence of barriers.
template <int WF, int NTW, bool IMG = false, int BN_ = 2 * NTW, bool GLU = false>
__device__ __forceinline__ void linear_dma_block(const LinearArgs &p, int bid, int nblk, int nt_first, int nt_end) {
  static_assert(WF == WF_BFP8 || WF == WF_BFP4, "block-float weights only");
  // GLU: the block's column tiles alternate between two bfp8_b matrices [K, NtR * 32] (p.gW[0], p.gW[1]; tile 2 j holds
  // columns of the first, 2 j + 1 the same columns of the second; p.Nt = 2 NtR counts both) and the epilogue multiplies the
  // pairs: act0(A W0) x act1(A W1), e.g. SiLU(gate) x up, without either factor leaving the registers
  static_assert(!GLU || (WF == WF_BFP8 && !IMG && BN_ == 2 * NTW && NTW % 2 == 0), "the gated form exists for the fused bfp8_b kernel");
  static_assert(BN_ == 2 * NTW || (IMG && BN_ == 7 && (NTW == 4 || NTW == 3)), "uneven blocks exist for the second pass only");
  constexpr int MB = 2;          // row tiles (32 m) per wavefront
  constexpr int BN = BN_;        // column tiles per block
  extern __shared__ u32x4 smem[];
  uint8_t *lds = (uint8_t *)smem;
  const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t *)lds;   // LDS byte address of the image
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  int wn, wm, wcol;   // column half, row quarter, first column tile of this wavefront inside the block
  if constexpr (BN_ == 2 * NTW) {
    wn = wave & 1; wm = wave >> 1; wcol = wn * NTW;
  } else {   // wavefronts w and w + 4 share a SIMD: one of them is the wide one
    const int sd = wave & 3, hf = wave >> 2;
    wn = (sd & 1) ^ hf; wm = (sd >> 1) + 2 * hf; wcol = wn ? BN_ - NTW : 0;
  }
  if (nblk % 8 == 0) bid = (bid & 7) * (nblk >> 3) + (bid >> 3);   // consecutive blocks of one XCD share weight columns
  const int nb = bid / p.m_blocks, mb = bid % p.m_blocks;
  const int mt0 = mb * 8, nt0 = nt_first + nb * BN;
  const uint8_t *A = p.A + (int64_t)blockIdx.z * p.a_batch;
  const uint8_t *W = GLU ? p.gW[0] : p.W + (int64_t)blockIdx.z * p.w_batch;
  const uint8_t *W1 = GLU ? p.gW[1] : W;                  // GLU: the matrix of the odd tile slots
  uint8_t *C = GLU ? p.gC[0] : p.C + (int64_t)blockIdx.z * p.c_batch;
  const int NtW = GLU ? p.gNt[0] : p.Nt;                  // column tiles of a weight matrix (GLU: p.Nt counts both matrices)
  constexpr uint32_t LDS_W = 65536, LDS_RAW = 131072, STAGE = 32768;
  constexpr uint32_t RAW_TILE = WF == WF_BFP8 ? 1024u : 512u, RAW_STAGE = 16 * RAW_TILE;
  constexpr uint32_t W_TILE = WF == WF_BFP8 ? 1088u : 576u;

  f32x16 acc[NTW][MB];
#pragma unroll
  for (int a = 0; a < NTW; ++a)
#pragma unroll
    for (int b = 0; b < MB; ++b)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[a][b][r] = 0.0f;

  // ---- per-lane constants
  uint32_t rdW[4], rdA[4];   // fragment reads: + 4096 t + STAGE stage
#pragma unroll
  for (int s = 0; s < 4; ++s) {
    rdW[s] = LDS_W + 16u * (IMG ? lds_chunk16(wcol * 32 + (lane & 31), 2 * s + (lane >> 5)) : lds_chunk(wcol * 32 + (lane & 31), 2 * s + (lane >> 5)));
    rdA[s] = 16u * lds_chunk(wm * (32 * MB) + (lane & 31), 2 * s + (lane >> 5));
  }
  // weight block of this lane: tile slot tid >> 5 of the 2 x 8 tiles of a step (slot = 8 * k-tile + column tile);
  // inside the tile: face, 8-row half, 4-column quad.  A wavefront owns two neighbouring column tiles of one
  // k-tile; with fewer than 8 column tiles per block the wavefronts of the unused slots skip the conversion.
  const int ukt = wave >> 2, unt = (tid >> 5) & 7, wq = tid & 31;
  const bool converts = 2 * (wave & 3) < BN;   // wavefront-uniform
  const int face = wq >> 3, khalf = (wq >> 2) & 1, quad = wq & 3;
  uint32_t wrW[4];
  {
    const int kc = ukt * 4 + (face >> 1) * 2 + khalf;
    const int n0 = unt * 32 + (face & 1) * 16 + quad * 4;
#pragma unroll
    for (int j = 0; j < 4; ++j) wrW[j] = LDS_W + 16u * lds_chunk(n0 + j, kc);
  }
  // raw staging reads: row i of the block at rawRd ^ (16 i) (bfp8) or rawRd + 8 i (bfp4)
  uint32_t rawRd;
  {
    const int tile_l = tid >> 5, a = face * 2 + khalf;
    if constexpr (WF == WF_BFP8) rawRd = LDS_RAW + tile_l * 1024 + a * 128 + ((a ^ (tile_l & 1)) << 4) + quad * 4;
    else rawRd = LDS_RAW + tile_l * 512 + a * 64 + quad * 2;
  }
  const uint32_t offWe = (uint32_t)min(GLU ? (nt0 + unt) >> 1 : nt0 + unt, NtW - 1) * W_TILE + face * 16 + khalf * 8;
  const uint8_t *We = GLU && (unt & 1) ? W1 : W;          // per lane: the matrix its tile slot belongs to
  // LDS-direct loads of the activations: wavefront w fills rows 32 w .. 32 w + 31 (row tile mt0 + w) with four
  // instructions of 8 rows each; lane l writes slot l & 7 of row 8 i + (l >> 3), i.e. k-chunk slot ^ swizzle(row)
  uint32_t dmaA[4];
  bool dmaA_sub[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r32 = 8 * i + (lane >> 3);
    const int kc = (lane & 7) ^ lds_swz(r32);   // the swizzle only looks at the low five row bits
    dmaA[i] = (uint32_t)(((r32 >> 4) * 2 + ((kc & 3) >> 1)) * 512 + (r32 & 15) * 32 + (kc & 1) * 16);
    dmaA_sub[i] = (kc >> 2) != 0;
  }
  const int64_t a_row = (int64_t)min(mt0 + wave, p.Mt - 1) * p.Kt * 2048;
  // mantissas: the wavefront stages its two tile slots 2 w, 2 w + 1
  uint32_t dmaW;   // bfp8: lane offset inside the tile; bfp4: inside the k-tile row (one instruction, two tiles)
  int64_t w_col[2] = {0, 0};
  if constexpr (WF == WF_BFP8) {
    const int a = lane >> 3;
    dmaW = 64u + (uint32_t)(8 * a + ((lane & 7) ^ a)) * 16u;   // tile parity is folded in at the call site (XOR 16)
#pragma unroll
    for (int x = 0; x < 2; ++x) w_col[x] = (int64_t)min(GLU ? (nt0 + 2 * (wave & 3)) >> 1 : nt0 + 2 * (wave & 3) + x, NtW - 1) * W_TILE;
  } else {
    dmaW = (uint32_t)(min(nt0 + 2 * (wave & 3) + (lane >> 5), NtW - 1) * (int)W_TILE) + 64u + (uint32_t)(lane & 31) * 16u;
  }

  // split-K: this block reduces k-tiles [kbase, kt_end); k-tiles past kt_end get zero weights
  const int kbase = blockIdx.y * p.k_slice, kt_end = min(p.Kt, kbase + p.k_slice);
  const int ksteps = (kt_end - kbase + 1) / 2;
  u32x2 exps = {0, 0}, exps_next = {0, 0};
  uint32_t keep = 0, keep_next = 0;
  u32x4 fw[2][NTW], fa[2][MB], out[4];

  // instructions [i0, i1) of the four that stage this wavefront's 32 activation rows of step kt0
  auto issue_a = [&](int kt0, uint32_t stage_off, int i0 = 0, int i1 = 4) {
    kt0 += kbase;
    const int kt = min(kt0, p.Kt - 1);
    const uint32_t sub = kt0 + 1 < p.Kt ? 2048u : 0u;   // k tail: the second tile of the pair repeats the first (its weights are zero)
    const uint8_t *base = A + a_row + (int64_t)kt * 2048;
#pragma unroll
    for (int i = 0; i < 4; ++i)
      if (i >= i0 && i < i1) lds_dma16(base, dmaA[i] + (dmaA_sub[i] ? sub : 0u), lds0 + stage_off + (uint32_t)(wave * 256 + i * 64) * 16u);
  };
  // second pass: instructions [i0, i1) of the four that copy this wavefront's column tile image of step `step` (counted
  // from the slice's first k-step) into the weight stage; steps past the slice's end read the all-zero image
  auto issue_img = [&](int step, uint32_t stage_off, int i0 = 0, int i1 = 4) {
    if (wave >= BN) return;   // wavefront-uniform: one image per column tile of the block
    const int ksg = (kbase >> 1) + step;
    const int ksc = kbase + 2 * step < kt_end ? ksg : p.img_zero_step;
    const uint8_t *base = W + ((int64_t)ksc * p.Nt + min(nt0 + wave, p.Nt - 1)) * 4096;
#pragma unroll
    for (int i = 0; i < 4; ++i)
      if (i >= i0 && i < i1) lds_dma16(base, (uint32_t)(lane * 16 + i * 1024), lds0 + LDS_W + stage_off + (uint32_t)(wave * 4096 + i * 1024));
  };
  auto issue_raw = [&](int kt0, uint32_t stage_off) {
    if constexpr (IMG) return;
    if (!converts) return;
    const int kt = min(kbase + kt0 + ukt, p.Kt - 1);
    const uint8_t *row = W + (int64_t)kt * NtW * W_TILE;
    if constexpr (WF == WF_BFP8) {
#pragma unroll
      for (int x = 0; x < 2; ++x)
        lds_dma16((GLU && x ? W1 + (int64_t)kt * NtW * W_TILE : row) + w_col[x], dmaW ^ (x << 4), lds0 + LDS_RAW + stage_off + (uint32_t)(2 * wave + x) * 1024u);
    } else {
      lds_dma16(row, dmaW, lds0 + LDS_RAW + stage_off + (uint32_t)(2 * wave) * 512u);
    }
  };
  // exponents of step kt0: the raw load and, separately, the k-tail mask (zero exponents dequantise to zero weights).
  // The mask is applied when the value is taken into use; masking right behind the load would wait for it, and with
  // it for every LDS-direct load issued before.
  auto load_exps = [&](int kt0, uint32_t &keep) {
    if constexpr (IMG) { keep = 0; return u32x2{0, 0}; }
    kt0 += kbase;
    const int kt = min(kt0 + ukt, p.Kt - 1);
    keep = kt0 + ukt >= kt_end ? 0u : 0xFFFFFFFFu;
    return *(const u32x2 *)(We + (int64_t)kt * NtW * W_TILE + offWe);
  };
  auto fetch = [&](int s2, uint32_t so, u32x4 (&w)[NTW], u32x4 (&a)[MB]) {
#pragma unroll
    for (int t = 0; t < NTW; ++t) w[t] = *(const u32x4 *)(lds + rdW[s2] + t * 4096 + so);
#pragma unroll
    for (int t = 0; t < MB; ++t) a[t] = *(const u32x4 *)(lds + rdA[s2] + t * 4096 + so);
  };
  // conversion quarter c: rows 2c, 2c+1 of the lane's block from the raw stage at raw_off; c == 3 stores the block
  auto quarter = [&](int c, uint32_t raw_off, uint32_t w_off) {
    if constexpr (IMG) return;
    if (!converts) return;
    float f[2][4];
#pragma unroll
    for (int r = 0; r < 2; ++r) {
      const int i = 2 * c + r;
      uint32_t E = ((i < 4 ? exps.x : exps.y) >> (8 * (i & 3))) & 0xFFu;
      if constexpr (WF == WF_BFP8) {
        E = max(E, 6u);   // rows below 2^-120, and the zeroed exponents of the k tail, dequantise to zero
        const float scale = __uint_as_float((E - 6u) << 23), nscale = -128.0f * scale;
        const uint32_t d = *(const uint32_t *)(lds + (rawRd ^ (i << 4)) + raw_off);
        const uint32_t sg = d & 0x80808080u, sb = sg >> 7;
        const uint32_t t = (d ^ 0x80808080u ^ (sg - sb)) + sb;   // per byte: 128 + mag or 128 - mag
#pragma unroll
        for (int b = 0; b < 4; ++b) f[r][b] = fmaf((float)((t >> (8 * b)) & 0xFFu), scale, nscale);
      } else {
        E = max(E, 2u);
        const float scale = __uint_as_float((E - 2u) << 23), nscale = -8.0f * scale;
        const uint32_t d = *(const uint16_t *)(lds + rawRd + i * 8 + raw_off);
        const uint32_t sg = d & 0x8888u, sb = sg >> 3;
        const uint32_t t = (d ^ 0x8888u ^ (sg - sb)) + sb;       // per nibble: 8 + mag or 8 - mag
#pragma unroll
        for (int b = 0; b < 4; ++b) f[r][b] = fmaf((float)((t >> (4 * b)) & 0xFu), scale, nscale);
      }
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) out[j][c] = pack_hi(f[0][j], f[1][j]);
    // the block is stored in two halves (k 0..3 after quarter 1, k 4..7 after quarter 3) to halve the store burst
    if (c == 1) {
#pragma unroll
      for (int j = 0; j < 4; ++j) *(u32x2 *)(lds + wrW[j] + w_off) = u32x2{out[j][0], out[j][1]};
    }
    if (c == 3) {
#pragma unroll
      for (int j = 0; j < 4; ++j) *(u32x2 *)(lds + wrW[j] + 8 + w_off) = u32x2{out[j][2], out[j][3]};
    }
  };
  auto mfma_chunk = [&](int buf) {
#pragma unroll
    for (int a = 0; a < NTW; ++a)
#pragma unroll
      for (int b = 0; b < MB; ++b)
        acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(*(bf16x8 *)&fw[buf][a], *(bf16x8 *)&fa[buf][b], acc[a][b], 0, 0, 0);
#pragma unroll
    for (int i = 0; i < NTW * MB; ++i) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x002, 32 / (NTW * MB), 0);
    }
  };
  auto landed_barrier = [&]() {
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
  };

  // ---- prologue: step 0 staged and converted, step 1 staged and its first quarter converted
  issue_a(0, 0);
  if constexpr (IMG) issue_img(0, 0);
  issue_raw(0, 0);
  issue_raw(2, RAW_STAGE);
  exps = load_exps(0, keep);
  landed_barrier();
  exps = u32x2{exps.x & keep, exps.y & keep};
#pragma unroll
  for (int c = 0; c < 4; ++c) quarter(c, 0, 0);
  exps = load_exps(2, keep);
  landed_barrier();            // weights of step 0 visible, raw stage 0 free
  exps = u32x2{exps.x & keep, exps.y & keep};
  issue_a(2, STAGE);
  if constexpr (IMG) issue_img(1, STAGE);
  issue_raw(4, 0);
  exps_next = load_exps(4, keep_next);
  fetch(0, 0, fw[0], fa[0]);
  quarter(0, RAW_STAGE, STAGE);

  // ---- rotated pipeline.  A step is four chunks of 16 k.  Chunk q multiplies, requests the fragments of the
  // following chunk and converts weight rows 2c, 2c+1 with c = (q + 1) % 4; the scheduler is asked to put the
  // conversion's VALU instructions behind the MFMAs, four apiece (the matrix core leaves five to six slots free
  // on the issue port).  The block barrier sits between chunks 2 and 3: chunk 3 multiplies from fragments that
  // were requested before the barrier and already requests chunk 0 of the next stage, so the matrix core does
  // not drain at the barrier; its conversion quarter (c = 0) belongs to the step after next.
  auto step = [&](auto stage_c, int ks) {
    constexpr uint32_t CUR = decltype(stage_c)::value * STAGE, NXT = STAGE - CUR;
    constexpr uint32_t RCUR = decltype(stage_c)::value * RAW_STAGE, RNXT = RAW_STAGE - RCUR;
#pragma unroll
    for (int q = 0; q < 3; ++q) {
      // the global-memory pipe takes about 16 cycles per LDS-direct instruction: the activation loads of a step are
      // spread over three chunks (1 + 2 + 1) so that no wavefront queues behind the whole block's burst
      if (q == 0 && ks > 0) issue_a((ks + 1) * 2, NXT, 1, 3);
      if (q == 1 && ks > 0) issue_a((ks + 1) * 2, NXT, 3, 4);
      if constexpr (IMG) {
        if (q == 0 && ks > 0) issue_img(ks + 1, NXT, 1, 3);
        if (q == 1 && ks > 0) issue_img(ks + 1, NXT, 3, 4);
      }
      fetch(q + 1, CUR, fw[(q + 1) & 1], fa[(q + 1) & 1]);
      quarter(q + 1, RNXT, NXT);
      mfma_chunk(q & 1);
      __builtin_amdgcn_sched_barrier(0);
    }
    landed_barrier();
    exps = u32x2{exps_next.x & keep_next, exps_next.y & keep_next};
    // stage CUR of the activations and stage RNXT of the mantissas are free now
    exps_next = load_exps((ks + 3) * 2, keep_next);
    issue_raw((ks + 3) * 2, RNXT);
    issue_a((ks + 2) * 2, CUR, 0, 1);
    if constexpr (IMG) issue_img(ks + 2, CUR, 0, 1);
    fetch(0, NXT, fw[0], fa[0]);
    quarter(0, RCUR, CUR);
    mfma_chunk(1);
    __builtin_amdgcn_sched_barrier(0);
  };
  // an odd number of steps is rounded up: the extra step multiplies zeroed weights
  for (int ks = 0; ks < ksteps; ks += 2) {
    step(std::integral_constant<int, 0>{}, ks);
    step(std::integral_constant<int, 1>{}, ks + 1);
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // nothing may still be in flight towards LDS when the block ends

  if constexpr (GLU) linear_epilogue_glu(p, C, acc, mt0 + wm * MB, nt0 + wcol, nt_end, NtW, lane);
  else if (p.partial) linear_store_partial(p, p.partial + ((int64_t)blockIdx.z * gridDim.y + blockIdx.y) * ((int64_t)p.Mt * p.Nt * 1024), acc,
                                           mt0 + wm * MB, nt0 + wcol, nt_end, lane);
  else linear_epilogue_act(p, C, acc, mt0 + wm * MB, nt0 + wcol, nt_end, lane);
}


// The second pass (weights already bf16 fragment images) with v_mfma_f32_16x16x32_bf16 in place of 32x32x16: the same LDS
// images, the same staging and barriers, the same 64 (m) x 32 NTW (n) outputs per wavefront, now as 2 NTW x 4 accumulator
// tiles of 16 x 16.  The smaller shape moves half the accumulator bytes per multiply-add through the register file; under
// the power cap that is clock: an MFMA-only loop on random bf16 operands sustains 2.02 PFLOP/s with this shape and 1.78
// with 32x32x16 on the same part (2.45 either way on all-zero operands, where nothing is power-limited), and the vendor
// library's bf16 GEMM uses it as well.
// A step (64 k) is two chunks of 32 k.  In a chunk, n tile u multiplies its weight fragment with the four activation
// fragments of the chunk; weight fragments are requested two tiles ahead.  The block barrier sits after n tile 3 of the
// second chunk: tiles 4 .. 7 of that chunk multiply from fragments requested before the barrier, and the first fragments
// of the next step are requested right behind it, so the matrix core does not drain at the barrier.
template <int WF, int NTW, int BN_ = 2 * NTW>
__device__ __forceinline__ void linear_img16_block(const LinearArgs &p, int bid, int nblk, int nt_first, int nt_end) {
  static_assert(BN_ == 2 * NTW || (BN_ == 7 && (NTW == 4 || NTW == 3)), "block of 2 NTW column tiles, or the uneven seven");
  constexpr int MB = 2, BN = BN_, NU = 2 * NTW, NV = 2 * MB;
  constexpr int PF = 2;   // weight fragments are requested PF tiles ahead (one ahead measured half a percent slower)
  extern __shared__ u32x4 smem[];
  uint8_t *lds = (uint8_t *)smem;
  const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t *)lds;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  int wn, wm, wcol;
  if constexpr (BN_ == 2 * NTW) {
    wn = wave & 1; wm = wave >> 1; wcol = wn * NTW;
  } else {
    const int sd = wave & 3, hf = wave >> 2;
    wn = (sd & 1) ^ hf; wm = (sd >> 1) + 2 * hf; wcol = wn ? BN_ - NTW : 0;
  }
  if (nblk % 8 == 0) bid = (bid & 7) * (nblk >> 3) + (bid >> 3);   // consecutive blocks of one XCD share weight columns
  const int nb = bid / p.m_blocks, mb = bid % p.m_blocks;
  const int mt0 = mb * 8, nt0 = nt_first + nb * BN;
  const uint8_t *A = p.A + (int64_t)blockIdx.z * p.a_batch;
  const uint8_t *W = p.W + (int64_t)blockIdx.z * p.w_batch;
  uint8_t *C = p.C + (int64_t)blockIdx.z * p.c_batch;
  constexpr uint32_t LDS_W = 65536, STAGE = 32768;

  f32x4 acc[NU][NV];
#pragma unroll
  for (int u = 0; u < NU; ++u)
#pragma unroll
    for (int v = 0; v < NV; ++v) acc[u][v] = f32x4{0.f, 0.f, 0.f, 0.f};

  // fragment reads: 16 rows x four 8-k chunks per instruction.  Row bit 4 (the odd 16-row tiles) enters the swizzle, so
  // even and odd tiles have their own per-lane constant; + 4096 (tile / 2) + STAGE stage.
  uint32_t rdW[2][2], rdA[2][2];   // [chunk][tile parity]
#pragma unroll
  for (int c = 0; c < 2; ++c)
#pragma unroll
    for (int par = 0; par < 2; ++par) {
      rdW[c][par] = LDS_W + 16u * lds_chunk16(wcol * 32 + par * 16 + (lane & 15), 4 * c + (lane >> 4));
      rdA[c][par] = 16u * lds_chunk16(wm * (32 * MB) + par * 16 + (lane & 15), 4 * c + (lane >> 4));
    }
  uint32_t dmaA[4];
  bool dmaA_sub[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r32 = 8 * i + (lane >> 3);
    const int kc = (lane & 7) ^ lds_swz16(r32);
    dmaA[i] = (uint32_t)(((r32 >> 4) * 2 + ((kc & 3) >> 1)) * 512 + (r32 & 15) * 32 + (kc & 1) * 16);
    dmaA_sub[i] = (kc >> 2) != 0;
  }
  const int64_t a_row = (int64_t)min(mt0 + wave, p.Mt - 1) * p.Kt * 2048;
  const int kbase = blockIdx.y * p.k_slice, kt_end = min(p.Kt, kbase + p.k_slice);
  const int ksteps = (kt_end - kbase + 1) / 2;

  auto issue_a = [&](int kt0, uint32_t stage_off, int i0 = 0, int i1 = 4) {
    kt0 += kbase;
    const int kt = min(kt0, p.Kt - 1);
    const uint32_t sub = kt0 + 1 < p.Kt ? 2048u : 0u;
    const uint8_t *base = A + a_row + (int64_t)kt * 2048;
#pragma unroll
    for (int i = 0; i < 4; ++i)
      if (i >= i0 && i < i1) lds_dma16(base, dmaA[i] + (dmaA_sub[i] ? sub : 0u), lds0 + stage_off + (uint32_t)(wave * 256 + i * 64) * 16u);
  };
  auto issue_img = [&](int step, uint32_t stage_off, int i0 = 0, int i1 = 4) {
    if (wave >= BN) return;
    const int ksg = (kbase >> 1) + step;
    const int ksc = kbase + 2 * step < kt_end ? ksg : p.img_zero_step;
    const uint8_t *base = W + ((int64_t)ksc * p.Nt + min(nt0 + wave, p.Nt - 1)) * 4096;
#pragma unroll
    for (int i = 0; i < 4; ++i)
      if (i >= i0 && i < i1) lds_dma16(base, (uint32_t)(lane * 16 + i * 1024), lds0 + LDS_W + stage_off + (uint32_t)(wave * 4096 + i * 1024));
  };
  // A fragment address is a per-lane base plus a constant (tile pair and stage) that belongs in the instruction's offset
  // field.  The bases pass through an empty asm in every step: seen as loop-invariant, base + constant would be hoisted
  // into registers of their own - one per tile pair - and those spill.
  auto refresh_bases = [&]() {   // the values stay
#pragma unroll
    for (int c = 0; c < 2; ++c)
#pragma unroll
      for (int par = 0; par < 2; ++par) asm volatile("" : "+v"(rdW[c][par]), "+v"(rdA[c][par]));
  };
  auto fetch_w = [&](int c, int u, uint32_t so) { return *(const u32x4 *)(lds + rdW[c][u & 1] + ((u >> 1) * 4096 + so)); };
  auto fetch_a1 = [&](int c, int v, uint32_t so) { return *(const u32x4 *)(lds + rdA[c][v & 1] + ((v >> 1) * 4096 + so)); };
  auto fetch_a = [&](int c, uint32_t so, u32x4 (&a)[NV]) {
#pragma unroll
    for (int v = 0; v < NV; ++v) a[v] = fetch_a1(c, v, so);
  };
  auto mfma_tile = [&](int u, const u32x4 &w, const u32x4 (&a)[NV]) {
#pragma unroll
    for (int v = 0; v < NV; ++v) acc[u][v] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(*(const bf16x8 *)&w, *(const bf16x8 *)&a[v], acc[u][v], 0, 0, 0);
  };
  auto landed_barrier = [&]() {
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
  };

  // ---- prologue: step 0 staged, step 1 on its way
  issue_a(0, 0);
  issue_img(0, 0);
  landed_barrier();
  issue_a(2, STAGE);
  issue_img(1, STAGE);
  u32x4 fa[2][NV], fw[NU];   // activation fragments of the two chunks; weight fragments of the chunk in flight
  refresh_bases();
  fetch_a(0, 0, fa[0]);
#pragma unroll
  for (int u = 0; u < PF; ++u) fw[u] = fetch_w(0, u, 0);

  auto step = [&](auto stage_c, int ks) {
    constexpr uint32_t CUR = decltype(stage_c)::value * STAGE, NXT = STAGE - CUR;
    constexpr int H = NU / 2;
    refresh_bases();
    // chunk 0: weight fragments are requested PF tiles ahead (fw[0 .. PF - 1] are there on entry); the activation
    // fragments of chunk 1 in its second half
#pragma unroll
    for (int u = 0; u < NU; ++u) {
      if (u == 0 && ks > 0) { issue_a((ks + 1) * 2, NXT, 1, 3); issue_img(ks + 1, NXT, 1, 3); }
      if (u == H && ks > 0) { issue_a((ks + 1) * 2, NXT, 3, 4); issue_img(ks + 1, NXT, 3, 4); }
      if (u >= NU - 4) fa[1][u - (NU - 4)] = fetch_a1(1, u - (NU - 4), CUR);
      fw[(u + PF) % NU] = u + PF < NU ? fetch_w(0, u + PF, CUR) : fetch_w(1, u + PF - NU, CUR);
      mfma_tile(u, fw[u], fa[0]);
      __builtin_amdgcn_sched_barrier(0);
    }
    // chunk 1, first half; the fragments of the second half are all requested before the barrier
#pragma unroll
    for (int u = 0; u < H; ++u) {
      fw[u + PF] = fetch_w(1, u + PF, CUR);
      if (u + PF + H < NU) fw[u + PF + H] = fetch_w(1, u + PF + H, CUR);
      mfma_tile(u, fw[u], fa[1]);
      __builtin_amdgcn_sched_barrier(0);
    }
    landed_barrier();
    // stage CUR is free: the first instruction of the step after next
    issue_a((ks + 2) * 2, CUR, 0, 1);
    issue_img(ks + 2, CUR, 0, 1);
    // the fragments the next step starts from (four of the activations, PF of the weights) are requested between the
    // remaining tiles, as registers come free: fa[0] and fw[0 .. PF - 1] were last used before the barrier
#pragma unroll
    for (int u = H; u < NU; ++u) {
#pragma unroll
      for (int f = 0; f < 4 + PF; ++f) {
        if (f * H / (4 + PF) != u - H) continue;
        if (f < 4) fa[0][f] = fetch_a1(0, f, NXT);
        else fw[f - 4] = fetch_w(0, f - 4, NXT);
      }
      mfma_tile(u, fw[u], fa[1]);
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  for (int ks = 0; ks < ksteps; ks += 2) {
    step(std::integral_constant<int, 0>{}, ks);
    step(std::integral_constant<int, 1>{}, ks + 1);
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");

  if (p.partial) linear_store_partial16(p, p.partial + ((int64_t)blockIdx.z * gridDim.y + blockIdx.y) * ((int64_t)p.Mt * p.Nt * 1024), acc,
                                        mt0 + wm * MB, nt0 + wcol, nt_end, lane);
  else linear_epilogue_act16(p, C, acc, mt0 + wm * MB, nt0 + wcol, nt_end, lane);
}

// group launch: the block's member becomes an ordinary single launch over that member's columns (p is rebound); the
// XCD-aware renumbering is applied to the whole grid here, so the body is told not to repeat it (nblk = 1)
__device__ __forceinline__ void linear_group_rebind(LinearArgs &p, int &bid, int &nblk, int &end) {
  if (nblk % 8 == 0) bid = (bid & 7) * (nblk >> 3) + (bid >> 3);
  const int nb = bid / p.m_blocks, mb = bid % p.m_blocks;
  const GroupMember m = group_member(p, nb, p.ntw == 7 ? 7 : 2 * p.ntw);
  p.W = m.W; p.C = m.C; p.Nt = m.Nt; p.act = m.act; p.group_n = 0;
  bid = m.local * p.m_blocks + mb;
  nblk = 1;
  end = m.Nt;
}

template <int WF>
__global__ __launch_bounds__(512) void ttm_linear_dma_k(LinearArgs p) {
  int bid = blockIdx.x, nblk = gridDim.x, first = 0, end = p.Nt, ntw = p.ntw;
  if (p.group_n > 1) linear_group_rebind(p, bid, nblk, end);   // workgroup-uniform
  if (p.nt_split > 0) {   // workgroup-uniform
    if (bid < p.n_blocks1) { nblk = p.n_blocks1; end = p.nt_split; }
    else { bid -= p.n_blocks1; nblk -= p.n_blocks1; first = p.nt_split; ntw = p.ntw2; }
  }
  if (ntw == 4) linear_dma_block<WF, 4>(p, bid, nblk, first, end);
  else if (ntw == 3) linear_dma_block<WF, 3>(p, bid, nblk, first, end);
  else linear_dma_block<WF, 2>(p, bid, nblk, first, end);
}

// the gated form of the fused kernel (bfp8_b): blocks of eight tile slots = four column tiles of either matrix
__global__ __launch_bounds__(512) void ttm_linear_dma_glu_k(LinearArgs p) {
  linear_dma_block<WF_BFP8, 4, false, 8, true>(p, blockIdx.x, gridDim.x, 0, p.Nt);
}

template <int WF, bool M16 = true>   // M16: v_mfma_f32_16x16x32_bf16 (linear_img16_block); else 32x32x16
__global__ __launch_bounds__(512) void ttm_linear_img_k(LinearArgs p) {
  int bid = blockIdx.x, nblk = gridDim.x, first = 0, end = p.Nt, ntw = p.ntw;
  if (p.group_n > 1) linear_group_rebind(p, bid, nblk, end);   // workgroup-uniform
  if (p.nt_split > 0) {   // workgroup-uniform
    if (bid < p.n_blocks1) { nblk = p.n_blocks1; end = p.nt_split; }
    else { bid -= p.n_blocks1; nblk -= p.n_blocks1; first = p.nt_split; ntw = p.ntw2; }
  }
  if constexpr (M16) {
    if (ntw == 7) {   // seven tiles wide: wide and narrow wavefronts (wavefront-uniform branch)
      const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
      if ((((wave & 3) & 1) ^ (wave >> 2)) == 0) linear_img16_block<WF, 4, 7>(p, bid, nblk, first, end);
      else linear_img16_block<WF, 3, 7>(p, bid, nblk, first, end);
    } else if (ntw == 4) linear_img16_block<WF, 4>(p, bid, nblk, first, end);
    else if (ntw == 3) linear_img16_block<WF, 3>(p, bid, nblk, first, end);
    else linear_img16_block<WF, 2>(p, bid, nblk, first, end);
  } else {
    if (ntw == 7) {
      const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
      if ((((wave & 3) & 1) ^ (wave >> 2)) == 0) linear_dma_block<WF, 4, true, 7>(p, bid, nblk, first, end);
      else linear_dma_block<WF, 3, true, 7>(p, bid, nblk, first, end);
    } else if (ntw == 4) linear_dma_block<WF, 4, true>(p, bid, nblk, first, end);
    else if (ntw == 3) linear_dma_block<WF, 3, true>(p, bid, nblk, first, end);
    else linear_dma_block<WF, 2, true>(p, bid, nblk, first, end);
  }
}

// First pass of a two-pass launch: block-float tiles -> bf16 LDS fragment images.  img[(ks * Nt + nt) * 4096 ..] is the
// 32 (n) x 64 (k) block of k-step ks and column tile nt exactly as the main loop wants it in LDS (row n, eight 16-byte
// chunks of 8 k, chunk slot swizzled by the row).  k-tiles at or past Kt - the second half of the last step when Kt is
// odd, and the extra step ks = ceil(Kt / 2) that slices read past their end - are zeros.  Same arithmetic as the fused
// kernel's conversion, so both routes give identical results.
// grid (ceil(Nt / 4), ceil(Kt / 2) + 1, weight sets), 256 lanes: half-wavefront h converts k-tile 2 ks + (h >> 2) of
// column tile 4 x + (h & 3); a lane owns an 8 (k) x 4 (n) block as in the decode kernel.
template <bool BFP4>
__device__ __forceinline__ void linear_image_body(const uint8_t *W, uint8_t *img, int Nt, int Kt, int xg) {
  constexpr uint32_t TB = BFP4 ? 576u : 1088u, FACE = BFP4 ? 128u : 256u, ROW = BFP4 ? 8u : 16u;
  const int tid = threadIdx.x, h = tid >> 5, wq = tid & 31;
  const int ks = blockIdx.y, nt = 4 * xg + (h & 3), kt = 2 * ks + (h >> 2);   // xg: group of four column tiles
  if (nt >= Nt) return;
  const int face = wq >> 3, khalf = (wq >> 2) & 1, quad = wq & 3;
  u32x4 out[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) out[j] = u32x4{0, 0, 0, 0};
  if (kt < Kt) {
    const uint8_t *t = W + ((int64_t)kt * Nt + nt) * TB;
    const u32x2 ex = *(const u32x2 *)(t + face * 16 + khalf * 8);
    const uint8_t *m = t + 64 + face * FACE + khalf * (FACE / 2) + quad * (ROW / 4);
    uint32_t rows[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) rows[i] = BFP4 ? (uint32_t) * (const uint16_t *)(m + i * ROW) : *(const uint32_t *)(m + i * ROW);
    float f[8][4];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      uint32_t E = ((i < 4 ? ex.x : ex.y) >> (8 * (i & 3))) & 0xFFu;
      constexpr uint32_t EB = BFP4 ? 2u : 6u, SIGN = BFP4 ? 0x08080808u : 0x80808080u, SH = BFP4 ? 3u : 7u;
      E = max(E, EB);
      const float scale = __uint_as_float((E - EB) << 23), nscale = (BFP4 ? -8.0f : -128.0f) * scale;
      uint32_t d = rows[i];
      if (BFP4) {
        d = (d | (d << 8)) & 0x00FF00FFu;
        d = (d | (d << 4)) & 0x0F0F0F0Fu;
      }
      const uint32_t sg = d & SIGN, sb = sg >> SH;
      const uint32_t tt = (d ^ SIGN ^ (sg - sb)) + sb;
#pragma unroll
      for (int b = 0; b < 4; ++b) f[i][b] = fmaf((float)((tt >> (8 * b)) & 0xFFu), scale, nscale);
    }
#pragma unroll
    for (int j = 0; j < 4; ++j)
      out[j] = u32x4{pack_hi(f[0][j], f[1][j]), pack_hi(f[2][j], f[3][j]), pack_hi(f[4][j], f[5][j]), pack_hi(f[6][j], f[7][j])};
  }
  u32x4 *dst = (u32x4 *)(img + ((int64_t)ks * Nt + nt) * 4096);
  const int kc = (h >> 2) * 4 + (face >> 1) * 2 + khalf, n0 = (face & 1) * 16 + quad * 4;
#pragma unroll
  for (int j = 0; j < 4; ++j) dst[lds_chunk16(n0 + j, kc)] = out[j];
}
// three workgroups per CU: the pass is a pure stream (read 1 byte, write 2); [4096, 14336] about 2.5 us faster than without
// a cap (the group form below measured no faster with one)
template <bool BFP4>
__global__ __launch_bounds__(256) TTM_MAX_WAVES(3) void ttm_linear_image_k(const uint8_t *W, int64_t w_batch, uint8_t *img, int64_t img_batch, int Nt, int Kt) {
  linear_image_body<BFP4>(W + (int64_t)blockIdx.z * w_batch, img + (int64_t)blockIdx.z * img_batch, Nt, Kt, blockIdx.x);
}
// The same images from bf16 weights, [K, N] tiles (NK = false) or [N, K] tiles (NK = true): a permutation, no arithmetic.
// With the weights in this form the second pass serves them exactly like block-float ones (seven-wide blocks, split K).
template <bool NK>
__global__ __launch_bounds__(256) TTM_MAX_WAVES(3) void ttm_linear_image_bf16_k(const uint8_t *W, int64_t w_batch, uint8_t *img, int64_t img_batch, int Nt, int Kt) {
  W += (int64_t)blockIdx.z * w_batch;
  img += (int64_t)blockIdx.z * img_batch;
  const int tid = threadIdx.x, h = tid >> 5, wq = tid & 31;
  const int ks = blockIdx.y, nt = 4 * (int)blockIdx.x + (h & 3), kt = 2 * ks + (h >> 2);
  if (nt >= Nt) return;
  const int face = wq >> 3, khalf = (wq >> 2) & 1, quad = wq & 3;   // face: (k half of the tile) * 2 + (n half)
  u32x4 out[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) out[j] = u32x4{0, 0, 0, 0};
  if (kt < Kt) {
    if (NK) {   // [N, K] tiles: the eight k of a column are 16 contiguous bytes
      const uint8_t *t = W + ((int64_t)nt * Kt + kt) * 2048 + ((face & 1) * 2 + (face >> 1)) * 512 + khalf * 16;
#pragma unroll
      for (int j = 0; j < 4; ++j) out[j] = *(const u32x4 *)(t + (quad * 4 + j) * 32);
    } else {    // [K, N] tiles: eight rows of four columns, regrouped by column
      const uint8_t *t = W + ((int64_t)kt * Nt + nt) * 2048 + face * 512 + khalf * 256 + quad * 8;
      u32x2 r[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) r[i] = *(const u32x2 *)(t + i * 32);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        out[0][i] = __builtin_amdgcn_perm(r[2 * i + 1].x, r[2 * i].x, 0x05040100u);
        out[1][i] = __builtin_amdgcn_perm(r[2 * i + 1].x, r[2 * i].x, 0x07060302u);
        out[2][i] = __builtin_amdgcn_perm(r[2 * i + 1].y, r[2 * i].y, 0x05040100u);
        out[3][i] = __builtin_amdgcn_perm(r[2 * i + 1].y, r[2 * i].y, 0x07060302u);
      }
    }
  }
  u32x4 *dst = (u32x4 *)(img + ((int64_t)ks * Nt + nt) * 4096);
  const int kc = (h >> 2) * 4 + (face >> 1) * 2 + khalf, n0 = (face & 1) * 16 + quad * 4;
#pragma unroll
  for (int j = 0; j < 4; ++j) dst[lds_chunk16(n0 + j, kc)] = out[j];
}
// the members of a group launch: grid.x numbers the members' groups of four column tiles one after another
struct ImageGroup {
  const uint8_t *W[4];
  uint8_t *img[4];
  int Nt[4];
  int n;
};
template <bool BFP4>
__global__ __launch_bounds__(256) void ttm_linear_image_group_k(ImageGroup g, int Kt) {
  const uint8_t *W = g.W[0];
  uint8_t *img = g.img[0];
  int Nt = g.Nt[0], xg = blockIdx.x, start = 0;
  bool found = false;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    if (j < g.n) {
      const int cnt = (g.Nt[j] + 3) / 4;
      if (!found && ((int)blockIdx.x < start + cnt || j == g.n - 1)) {
        found = true;
        W = g.W[j]; img = g.img[j]; Nt = g.Nt[j]; xg = blockIdx.x - start;
      }
      start += cnt;
    }
  }
  linear_image_body<BFP4>(W, img, Nt, Kt, xg);
}

// =============================================================================================
// Small-M kernel (M <= 32, decode): weight streaming.  One workgroup per 32-wide column tile,
// four wavefronts split K; each wavefront dequantises 4 weight tiles (128 k) per iteration into
// its private LDS region and multiplies them with activation fragments read from global (L2
// resident).  Partial sums are reduced through LDS.
// =============================================================================================
template <int WF>
__global__ __launch_bounds__(256) void ttm_linear_small_k(LinearArgs p) {
  __shared__ u32x4 smem[4 * 512];  // per wave: 32 rows x 16 chunks (128 k)
  __shared__ float red[3][16][64];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int nt = blockIdx.x;
  const uint8_t *A = p.A + (int64_t)blockIdx.z * p.a_batch;
  const uint8_t *W = p.W + (int64_t)blockIdx.z * p.w_batch;
  uint8_t *C = p.C + (int64_t)blockIdx.z * p.c_batch;
  u32x4 *lds = smem + wave * 512;
  f32x16 acc;
#pragma unroll
  for (int r = 0; r < 16; ++r) acc[r] = 0.0f;

  // k-tiles are dealt to the four waves in groups of 4
  const int groups = (p.Kt + 3) / 4;
  const int tile_l = lane >> 4, w = lane & 15;
  const int face = w >> 2, khalf = (w >> 1) & 1, oct = w & 1;
  for (int g = wave; g < groups; g += 4) {
    const int kt = g * 4 + tile_l;
    const bool ok = kt < p.Kt;
    const int64_t tile = (int64_t)kt * p.Nt + nt;
    u32x4 out[8];
    if constexpr (WF == WF_BF16_NK) {
      // weights stored [N,K] in tile order are already k-contiguous: fragments straight from global
#pragma unroll
      for (int s = 0; s < 8; ++s) {
        const int kt_s = g * 4 + (s >> 1), r_in = lane & 31;
        const uint8_t *ws = W + ((int64_t)nt * p.Kt + kt_s) * 2048 + ((r_in >> 4) * 2 + (s & 1)) * 512 +
                            (r_in & 15) * 32 + (lane >> 5) * 16;
        const uint8_t *as = A + (int64_t)kt_s * 2048 + ((r_in >> 4) * 2 + (s & 1)) * 512 + (r_in & 15) * 32 +
                            (lane >> 5) * 16;
        u32x4 wv = kt_s < p.Kt ? *(const u32x4 *)ws : u32x4{0, 0, 0, 0};
        u32x4 av = kt_s < p.Kt ? *(const u32x4 *)as : u32x4{0, 0, 0, 0};
        acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(*(bf16x8 *)&wv, *(bf16x8 *)&av, acc, 0, 0, 0);
      }
      continue;
    }
    if constexpr (WF == WF_BFP8) {
      const uint8_t *t = W + tile * 1088;
      u32x2 exps = ok ? *(const u32x2 *)(t + face * 16 + khalf * 8) : u32x2{0, 0};
      const uint8_t *m = t + 64 + face * 256 + khalf * 128 + oct * 8;
      u32x2 rows[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) rows[i] = ok ? *(const u32x2 *)(m + i * 16) : u32x2{0, 0};
      dequant_bfp8_block(rows, exps, out);
    } else if constexpr (WF == WF_BFP4) {
      const uint8_t *t = W + tile * 576;
      u32x2 exps = ok ? *(const u32x2 *)(t + face * 16 + khalf * 8) : u32x2{0, 0};
      const uint8_t *m = t + 64 + face * 128 + khalf * 64 + oct * 4;
      uint32_t rows[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) rows[i] = ok ? *(const uint32_t *)(m + i * 8) : 0u;
      dequant_bfp4_block(rows, exps, out);
    } else {
      const uint8_t *m = W + tile * 2048 + face * 512 + khalf * 256 + oct * 16;
      u32x4 rows[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) rows[i] = ok ? *(const u32x4 *)(m + i * 32) : u32x4{0, 0, 0, 0};
      transpose_bf16_block(rows, out);
    }
    // activation fragments for the 8 k16 steps of this group, straight from global
    bf16x8 af[8];
#pragma unroll
    for (int s = 0; s < 8; ++s) {
      const int kt_s = g * 4 + (s >> 1);
      const int m_in = lane & 31;
      const uint8_t *src = A + (int64_t)kt_s * 2048 + ((m_in >> 4) * 2 + (s & 1)) * 512 + (m_in & 15) * 32 + (lane >> 5) * 16;
      u32x4 v = kt_s < p.Kt ? *(const u32x4 *)src : u32x4{0, 0, 0, 0};
      af[s] = *(bf16x8 *)&v;
    }
    {
      const int kc = tile_l * 4 + (face >> 1) * 2 + khalf;  // 16 chunks of 8 k
      const int n0 = (face & 1) * 16 + oct * 8;
#pragma unroll
      for (int j = 0; j < 8; ++j) lds[(n0 + j) * 16 + (kc ^ ((n0 + j) & 15))] = out[j];
    }
    // LDS traffic of one wavefront is processed in order; the fences only pin the compiler's order
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int s = 0; s < 8; ++s) {
      const int n = lane & 31, kc = 2 * s + (lane >> 5);
      u32x4 v = lds[n * 16 + (kc ^ (n & 15))];
      acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(*(bf16x8 *)&v, af[s], acc, 0, 0, 0);
    }
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    __builtin_amdgcn_wave_barrier();
  }
  // reduce the four partial accumulators
  if (wave > 0) {
#pragma unroll
    for (int r = 0; r < 16; ++r) red[wave - 1][r][lane] = acc[r];
  }
  __syncthreads();
  if (wave != 0) return;
#pragma unroll
  for (int r = 0; r < 16; ++r) acc[r] += red[0][r][lane] + red[1][r][lane] + red[2][r][lane];
  const int m_in = lane & 31;
#pragma unroll
  for (int g = 0; g < 4; ++g) {
    const int n_in = g * 8 + (lane >> 5) * 4;
    float bv[4] = {0.f, 0.f, 0.f, 0.f};
    if (p.bias) {
      const uint16_t *bp = p.bias_tiled ? p.bias + (int64_t)nt * 1024 + (n_in >> 4) * 256 + (n_in & 15)
                                        : p.bias + nt * 32 + n_in;
      u32x2 raw = *(const u32x2 *)bp;
      bv[0] = __uint_as_float(raw.x << 16); bv[1] = __uint_as_float(raw.x & 0xFFFF0000u);
      bv[2] = __uint_as_float(raw.y << 16); bv[3] = __uint_as_float(raw.y & 0xFFFF0000u);
    }
    float v[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      float x = acc[g * 4 + r] + bv[r];
      switch (p.act) {
      case TTM_ACT_GELU: x = apply_act<TTM_ACT_GELU>(x); break;
      case TTM_ACT_SILU: x = apply_act<TTM_ACT_SILU>(x); break;
      case TTM_ACT_SIGMOID: x = apply_act<TTM_ACT_SIGMOID>(x); break;
      case TTM_ACT_RELU: x = apply_act<TTM_ACT_RELU>(x); break;
      default: break;
      }
      v[r] = x;
    }
    int64_t off = (int64_t)nt * 1024 + ((m_in >> 4) * 2 + (n_in >> 4)) * 256 + (m_in & 15) * 16 + (n_in & 15);
    *(u32x2 *)(C + off * 2) = finish_quad(p, C + off * 2, v);
  }
}

// =============================================================================================
// Decode kernel for bfp8_b weights (M <= 32 per launch): pure weight streaming, no LDS on the way in.
// A workgroup owns 64 output columns (two weight tiles); its 8 wavefronts take every 8th k-tile and are
// summed through LDS at the end.  Per k-tile a lane needs an 8 (k) x 4 (n) block as eight 4-byte words (bfp8_b: the four
// lanes of a quad fetch the 128-byte line that holds their four blocks as two whole 16-byte rows each and transpose
// it between them with DPP moves; bfp4_b: eight 2-byte loads), dequantises it in registers and feeds byte j of the words to MFMA j: with
// v_mfma_f32_16x16x32_bf16 lane l supplies row l % 16 and k = 8 (l / 16) .. + 7 of the 16 x 32 weight
// operand, and MFMA j's row r stands for column n = 4 r + j, so one accumulator register of the four
// MFMAs is four consecutive n again.  Loads run two k-tiles ahead (register ring): with eight wavefronts that is
// 74 KiB in flight per CU; four ahead measured 5 % slower ([4096, 14336] at M = 32: 17.4 -> 16.5 us), one or five slower still.
// =============================================================================================
typedef float f32x4v __attribute__((ext_vector_type(4)));

// BFP4 = true reads bfp4_b tiles (576 bytes, two elements per byte, low nibble first): a lane's 4 (n) of a k row are one
// 16-bit word, whose nibbles are spread into the bytes of a word before the same sign-magnitude -> offset-binary step.
//
// TWO_TERM = true builds the bf16 operands with bit operations alone instead of int -> float conversions.  A weight is
// +-mag x 2^(E - 133) (bfp8_b; mag x 2^(E - 129) for bfp4_b).  The bf16 number with the sign, exponent field E + 1 and
// mantissa field mag (mag << 4 for bfp4_b) is V = +-(1 + mag / 128) x 2^(E - 126) = weight + S with S = +-2^(E - 126),
// the same bits with a zero mantissa.  Both are made for two k rows at a time with a byte permute and three mask / shift /
// or steps, V and S go through the matrix cores into two accumulators, and the result is their difference: twice the
// MFMAs (which were idle) for less than half the vector instructions.  The two sums are each a few times larger than
// their difference, so the fp32 rounding error grows by that factor - still four decimal orders below a bf16 result.
template <bool BFP4, bool TWO_TERM, int NP, bool GLU>
__global__ __launch_bounds__(512) void ttm_linear_decode_k(LinearArgs p) {
  extern __shared__ u32x4 smem[];   // partial sums: NP x 8 wavefronts x 8 x 64 float4 = NP x 64 KiB
  constexpr int D = 2;
  constexpr bool WL = !BFP4;   // whole-row loads and a transpose within lane quads (bfp8_b)
  constexpr uint32_t TB = BFP4 ? 576u : 1088u, FACE = BFP4 ? 128u : 256u, ROW = BFP4 ? 8u : 16u;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  int cg = blockIdx.x, Nt = p.Nt, tile_base = 0, act = p.act;   // column pair, column tiles of the matrix, its first tile in a group's concatenation
  const uint8_t *A = p.A + (int64_t)blockIdx.z * p.a_batch;
  const uint8_t *W = p.W + (int64_t)blockIdx.z * p.w_batch;
  uint8_t *C = p.C + (int64_t)blockIdx.z * p.c_batch;
  static_assert(!GLU || NP == 2, "the gated form multiplies the two tile pairs of a workgroup");
  if constexpr (GLU) {
    W = p.gW[0]; C = p.gC[0]; Nt = p.gNt[0];
  } else if (p.group_n > 1) {   // workgroup-uniform
    const GroupMember m = group_member(p, cg, 2 * NP);
    W = m.W; C = m.C; Nt = m.Nt; cg = m.local; tile_base = m.tile_base; act = m.act;
  }
  const uint8_t *W2 = GLU ? p.gW[1] : W;   // GLU: tile pair 1 is the same column pair of the second matrix
  const int q16 = lane & 15, kg = lane >> 4;   // weight operand row and 8-k group of this lane
  const int fc = (q16 >> 2) & 1, quad = q16 & 3, fr = kg >> 1, half = kg & 1;
  uint32_t offW[NP], offE[NP];   // tile pair pr of the workgroup: column tiles 2 NP cg + 2 pr, + 1
#pragma unroll
  for (int pr = 0; pr < NP; ++pr) {
    const uint32_t nt_l = (uint32_t)min(GLU ? 2 * cg + (q16 >> 3) : 2 * NP * cg + 2 * pr + (q16 >> 3), Nt - 1);
    offW[pr] = nt_l * TB + 64u + (fr * 2 + fc) * FACE + half * (FACE / 2) + quad * (WL ? ROW : ROW / 4);   // + ROW i (WL: row quad, + 4 ROW)
    offE[pr] = nt_l * TB + (fr * 2 + fc) * 16 + half * 8;
  }
  const uint32_t offA = fr * 512 + q16 * 32 + half * 16;                                     // + 1024 h

  f32x4v acc[NP][2][4], accs[NP][2][4];   // accs: the sum over the S terms (TWO_TERM)
#pragma unroll
  for (int pr = 0; pr < NP; ++pr)
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
      for (int j = 0; j < 4; ++j) acc[pr][h][j] = accs[pr][h][j] = f32x4v{0.f, 0.f, 0.f, 0.f};

  uint32_t rows[D][NP][8], keeps[D];
  u32x2 ex[D][NP];
  u32x4 af[D][2];
  // split-K: workgroup y of the grid takes k-tiles [y k_slice, (y + 1) k_slice) and leaves fp32 partial sums
  const int kbase = p.partial ? (int)blockIdx.y * p.k_slice : 0;
  const int kend = p.partial ? min(kbase + p.k_slice, p.Kt) : p.Kt;
  const int nchunks = (kend - kbase + 7) / 8;
  auto load_slot = [&](int s, int c) {
    const int kt = kbase + wave + 8 * c;
    const int ktc = min(kt, kend - 1);
    const uint32_t keep = kt < kend ? 0xFFFFFFFFu : 0u;   // past the end: zero exponents, zero weights
    const uint8_t *Wk0 = W + (int64_t)ktc * Nt * TB, *Wk1 = W2 + (int64_t)ktc * Nt * TB;
    const uint8_t *Ak = A + (int64_t)ktc * 2048;
#pragma unroll
    for (int pr = 0; pr < NP; ++pr) {
      const uint8_t *Wk = pr == 0 ? Wk0 : Wk1;
      if constexpr (WL) {
        // the four lanes of a quad need one 128-byte line between them (8 k rows x 16 n bytes, a dword column each): every
        // lane fetches two whole rows of it (rows quad and quad + 4) and the quad transposes in registers when the slot is
        // consumed - 2 loads and 32 cache-line look-ups per wavefront and tile pair instead of 8 and 128
        const u32x4 x = *(const u32x4 *)(Wk + offW[pr]), y = *(const u32x4 *)(Wk + offW[pr] + 64);
        rows[s][pr][0] = x.x; rows[s][pr][1] = x.y; rows[s][pr][2] = x.z; rows[s][pr][3] = x.w;
        rows[s][pr][4] = y.x; rows[s][pr][5] = y.y; rows[s][pr][6] = y.z; rows[s][pr][7] = y.w;
      } else {
#pragma unroll
        for (int i = 0; i < 8; ++i)   // the eight loads share their cache lines: cached loads
          rows[s][pr][i] = BFP4 ? (uint32_t) * (const uint16_t *)(Wk + offW[pr] + i * ROW) : *(const uint32_t *)(Wk + offW[pr] + i * ROW);
      }
      ex[s][pr] = *(const u32x2 *)(Wk + offE[pr]);
    }
    keeps[s] = keep;   // applied when the slot is consumed: masking here would wait for the load
#pragma unroll
    for (int h = 0; h < 2; ++h) af[s][h] = *(const u32x4 *)(Ak + offA + h * 1024);
  };
  // 4 x 4 transpose of dwords within every quad of lanes: lane q ends up with dword q of the rows that lanes 0..3 hold
  auto quad_transpose = [&](uint32_t *v) __attribute__((always_inline)) {
    const bool odd = (lane & 1) != 0, hi = (lane & 2) != 0;
#pragma unroll
    for (int a = 0; a < 4; a += 2) {   // lanes 2 j and 2 j + 1 exchange (v[a + 1] of the even, v[a] of the odd)
      const uint32_t ta = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v[a], 0xB1, 0xF, 0xF, true);
      const uint32_t tb = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v[a + 1], 0xB1, 0xF, 0xF, true);
      v[a + 1] = odd ? v[a + 1] : ta;
      v[a] = odd ? tb : v[a];
    }
#pragma unroll
    for (int a = 0; a < 2; ++a) {      // lanes j and j + 2 exchange (v[a + 2] of the lower, v[a] of the upper)
      const uint32_t ta = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v[a], 0x4E, 0xF, 0xF, true);
      const uint32_t tb = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v[a + 2], 0x4E, 0xF, 0xF, true);
      v[a + 2] = hi ? v[a + 2] : ta;
      v[a] = hi ? tb : v[a];
    }
  };
  auto process_pair = [&](int s, int pr) __attribute__((always_inline)) {
    if constexpr (WL) {
      if (!TWO_TERM || keeps[s] != 0u) { quad_transpose(&rows[s][pr][0]); quad_transpose(&rows[s][pr][4]); }
    }
    if constexpr (TWO_TERM) {
      if (keeps[s] == 0u) return;   // wavefront-uniform: a k-tile past the end contributes nothing
      // (E + 1) << 7 for the rows 2 ip and 2 ip + 1, in the two halves of a word; E is capped so that the field stays 8 bits
      uint32_t epk[4];
#pragma unroll
      for (int ip = 0; ip < 4; ++ip) {
        const uint32_t src = ip < 2 ? ex[s][pr].x : ex[s][pr].y;
        uint32_t e2 = __builtin_amdgcn_perm(0u, src, (ip & 1) ? 0x0c030c02u : 0x0c010c00u);
        typedef unsigned short u16x2 __attribute__((ext_vector_type(2)));
        const u16x2 capped = __builtin_elementwise_min(*(const u16x2 *)&e2, u16x2{0xFD, 0xFD});
        e2 = *(const uint32_t *)&capped;
        epk[ip] = (e2 + 0x00010001u) << 7;
      }
      uint32_t pk[4] = {0u, 0u, 0u, 0u};
      if constexpr (BFP4) {
#pragma unroll
        for (int ip = 0; ip < 4; ++ip) pk[ip] = rows[s][pr][2 * ip] | (rows[s][pr][2 * ip + 1] << 16);   // four nibbles per row
      }
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        u32x4 wv, ws;
#pragma unroll
        for (int ip = 0; ip < 4; ++ip) {
          uint32_t sb, v;
          if constexpr (BFP4) {
            const uint32_t q = pk[ip] >> (4 * j);            // nibble j of either row in bits 0..3 and 16..19
            sb = ((q & 0x00080008u) << 12) | epk[ip];
            v = ((q & 0x00070007u) << 4) | sb;
          } else {
            const uint32_t q = __builtin_amdgcn_perm(rows[s][pr][2 * ip + 1], rows[s][pr][2 * ip], 0x0c040c00u + 0x00010001u * j);
            sb = ((q & 0x00800080u) << 8) | epk[ip];
            v = (q & 0x007F007Fu) | sb;
          }
          wv[ip] = v;
          ws[ip] = sb;
        }
#pragma unroll
        for (int h = 0; h < 2; ++h) {
          acc[pr][h][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(*(bf16x8 *)&wv, *(bf16x8 *)&af[s][h], acc[pr][h][j], 0, 0, 0);
          accs[pr][h][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(*(bf16x8 *)&ws, *(bf16x8 *)&af[s][h], accs[pr][h][j], 0, 0, 0);
        }
      }
      return;
    }
    float f[8][4];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      uint32_t E = (((i < 4 ? ex[s][pr].x : ex[s][pr].y) & keeps[s]) >> (8 * (i & 3))) & 0xFFu;
      // value = magnitude x 2^(E - 127 - 6) (bfp8_b) or 2^(E - 127 - 2) (bfp4_b); smaller exponents flush to zero
      constexpr uint32_t EB = BFP4 ? 2u : 6u, SIGN = BFP4 ? 0x08080808u : 0x80808080u, SH = BFP4 ? 3u : 7u;
      E = max(E, EB);
      const float scale = __uint_as_float((E - EB) << 23), nscale = (BFP4 ? -8.0f : -128.0f) * scale;
      uint32_t d = rows[s][pr][i];
      if (BFP4) {   // nibbles n3 n2 n1 n0 of the low half -> one per byte
        d = (d | (d << 8)) & 0x00FF00FFu;
        d = (d | (d << 4)) & 0x0F0F0F0Fu;
      }
      const uint32_t sg = d & SIGN, sb = sg >> SH;
      const uint32_t t = (d ^ SIGN ^ (sg - sb)) + sb;
#pragma unroll
      for (int b = 0; b < 4; ++b) f[i][b] = fmaf((float)((t >> (8 * b)) & 0xFFu), scale, nscale);
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      u32x4 w = {pack_hi(f[0][j], f[1][j]), pack_hi(f[2][j], f[3][j]), pack_hi(f[4][j], f[5][j]), pack_hi(f[6][j], f[7][j])};
#pragma unroll
      for (int h = 0; h < 2; ++h)
        acc[pr][h][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(*(bf16x8 *)&w, *(bf16x8 *)&af[s][h], acc[pr][h][j], 0, 0, 0);
    }
  };
  auto process = [&](int s) __attribute__((always_inline)) {
#pragma unroll
    for (int pr = 0; pr < NP; ++pr) process_pair(s, pr);
  };
#pragma unroll
  for (int s = 0; s < D; ++s) {
    load_slot(s, s);
    __builtin_amdgcn_sched_barrier(0);
  }
  // straight-line loop body (exact load counters): the chunk count is rounded up to the ring depth, and the
  // extra chunks contribute zeros
  for (int c0 = 0; c0 < nchunks; c0 += D) {
#pragma unroll
    for (int s = 0; s < D; ++s) {
      process(s);
      __builtin_amdgcn_sched_barrier(0);   // keep the loads in slot order, D - 1 slots ahead of their use
      load_slot(s, c0 + s + D);
      __builtin_amdgcn_sched_barrier(0);
    }
  }

  if constexpr (TWO_TERM) {
#pragma unroll
    for (int pr = 0; pr < NP; ++pr)
#pragma unroll
      for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[pr][h][j] -= accs[pr][h][j];
  }
  // partial sums -> LDS as float4 (four consecutive n of one m): slot (((pr * 8 + wave) * 8 + h * 4 + i) * 64 + lane)
  f32x4v *part = (f32x4v *)smem;
#pragma unroll
  for (int pr = 0; pr < NP; ++pr)
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
      for (int i = 0; i < 4; ++i)
        part[((pr * 8 + wave) * 8 + h * 4 + i) * 64 + lane] = f32x4v{acc[pr][h][0][i], acc[pr][h][1][i], acc[pr][h][2][i], acc[pr][h][3][i]};
  __syncthreads();
  const int h = tid >> 8, i = (tid >> 6) & 3;
  if constexpr (GLU) {
    // thread t holds the same four outputs of both matrices: out = bf16(bf16(act0(gate)) x bf16(act1(up))), the roundings
    // of the two projections stored by themselves and of the multiply that would read them
    f32x4v s0 = part[tid], s1 = part[4096 + tid];
#pragma unroll
    for (int w = 1; w < 8; ++w) { s0 += part[w * 512 + tid]; s1 += part[4096 + w * 512 + tid]; }
    const int nt = 2 * cg + (kg >> 1);
    if (nt >= Nt) return;
    const int n_in = 16 * (kg & 1) + 4 * i;
    const int64_t off = (int64_t)nt * 1024 + (h * 2 + (n_in >> 4)) * 256 + q16 * 16 + (n_in & 15);
    float v0[4], v1[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      float x = s0[r], y = s1[r];
      switch (p.gAct[0]) {
      case TTM_ACT_GELU: x = apply_act<TTM_ACT_GELU>(x); break;
      case TTM_ACT_SILU: x = apply_act<TTM_ACT_SILU>(x); break;
      case TTM_ACT_SIGMOID: x = apply_act<TTM_ACT_SIGMOID>(x); break;
      case TTM_ACT_RELU: x = apply_act<TTM_ACT_RELU>(x); break;
      default: break;
      }
      switch (p.gAct[1]) {
      case TTM_ACT_GELU: y = apply_act<TTM_ACT_GELU>(y); break;
      case TTM_ACT_SILU: y = apply_act<TTM_ACT_SILU>(y); break;
      case TTM_ACT_SIGMOID: y = apply_act<TTM_ACT_SIGMOID>(y); break;
      case TTM_ACT_RELU: y = apply_act<TTM_ACT_RELU>(y); break;
      default: break;
      }
      v0[r] = x; v1[r] = y;
    }
    const u32x2 g = {pack_bf16(v0[0], v0[1]), pack_bf16(v0[2], v0[3])}, u = {pack_bf16(v1[0], v1[1]), pack_bf16(v1[2], v1[3])};
    const float z[4] = {__uint_as_float(g.x << 16) * __uint_as_float(u.x << 16), __uint_as_float(g.x & 0xFFFF0000u) * __uint_as_float(u.x & 0xFFFF0000u),
                        __uint_as_float(g.y << 16) * __uint_as_float(u.y << 16), __uint_as_float(g.y & 0xFFFF0000u) * __uint_as_float(u.y & 0xFFFF0000u)};
    *(u32x2 *)(C + off * 2) = u32x2{pack_bf16(z[0], z[1]), pack_bf16(z[2], z[3])};
    return;
  }
#pragma unroll
  for (int pr = 0; pr < NP; ++pr) {
  // thread t finishes slot t of the pair's 512: (h, i, lane) = (t >> 8, (t >> 6) & 3, t & 63)
  f32x4v sum = part[pr * 4096 + tid];
#pragma unroll
  for (int w = 1; w < 8; ++w) sum += part[pr * 4096 + w * 512 + tid];
  const int nt = 2 * NP * cg + 2 * pr + (kg >> 1);
  if (nt >= Nt) continue;
  const int n_in = 16 * (kg & 1) + 4 * i;
  const int64_t off = (int64_t)nt * 1024 + (h * 2 + (n_in >> 4)) * 256 + q16 * 16 + (n_in & 15);
  if (p.partial) {   // bias, activation and rounding happen in ttm_linear_reduce_k
    const int64_t per = (int64_t)p.Nt * 1024;   // a group's partial sums are laid out as the concatenation
    *(f32x4v *)(p.partial + ((int64_t)blockIdx.z * gridDim.y + blockIdx.y) * per + (int64_t)tile_base * 1024 + off) = sum;
    continue;
  }
  float bv[4] = {0.f, 0.f, 0.f, 0.f};
  if (p.bias) {
    const uint16_t *bp = p.bias_tiled ? p.bias + (int64_t)nt * 1024 + (n_in >> 4) * 256 + (n_in & 15) : p.bias + nt * 32 + n_in;
    u32x2 raw = *(const u32x2 *)bp;
    bv[0] = __uint_as_float(raw.x << 16); bv[1] = __uint_as_float(raw.x & 0xFFFF0000u);
    bv[2] = __uint_as_float(raw.y << 16); bv[3] = __uint_as_float(raw.y & 0xFFFF0000u);
  }
  float v[4];
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    float x = sum[r] + bv[r];
    switch (act) {
    case TTM_ACT_GELU: x = apply_act<TTM_ACT_GELU>(x); break;
    case TTM_ACT_SILU: x = apply_act<TTM_ACT_SILU>(x); break;
    case TTM_ACT_SIGMOID: x = apply_act<TTM_ACT_SIGMOID>(x); break;
    case TTM_ACT_RELU: x = apply_act<TTM_ACT_RELU>(x); break;
    default: break;
    }
    v[r] = x;
  }
  *(u32x2 *)(C + off * 2) = finish_quad(p, C + off * 2, v);
  }
}

// Ends the decode step's Q / K / V launch.  One lane per four consecutive columns of one user: sums the k-slices, rounds to
// bf16 (the projection's own output rounding), applies the rotary embedding to q and k (the partner columns d +- dim / 2 are
// another four consecutive partial sums), and writes q in [1, users, heads, dim] order and k / v into the caches at the
// position read from device memory (out of range: nothing is written).  Lanes past the partial sums zero the padding rows
// of q.  The result equals ttm_linear_group + ttm_rotary_embedding_split_heads + the cache updates bit for bit.
__global__ __launch_bounds__(256) void ttm_qkv_finish_k(QkvFinishArgs p) {
  const int64_t q = (int64_t)blockIdx.x * 256 + threadIdx.x, nq = p.per / 4;
  const int D = p.dim, ct = D >> 5, d4 = D >> 2;
  if (q >= nq) {
    const int padh = p.heads_pad - p.heads;
    const int64_t z = q - nq;
    if (z >= (int64_t)p.users * padh * d4) return;
    const int d = (int)(z % d4) * 4, h = p.heads + (int)((z / d4) % padh), b = (int)(z / ((int64_t)d4 * padh));
    *(u32x2 *)(p.q_out + (int64_t)b * p.heads_pad * D + ttm_tiled_offset(h, d, ct)) = u32x2{0u, 0u};
    return;
  }
  const int64_t off = q * 4;
  const int nt = (int)(off >> 10), in = (int)(off & 1023);
  const int m = ((in >> 9) & 1) * 16 + ((in >> 4) & 15);
  if (m >= p.users) return;
  const int n = nt * 32 + ((in >> 8) & 1) * 16 + (in & 15);
  const int nQ = p.heads * D, nK = p.kv_heads * D;
  auto sum4 = [&](int64_t o) {
    f32x4 s = *(const f32x4 *)(p.partial + o);
    for (int sl = 1; sl < p.slices; ++sl) s += *(const f32x4 *)(p.partial + sl * p.per + o);
    return s;
  };
  auto r16 = [](float x) { return ttm_bf16_to_f32(ttm_f32_to_bf16(x)); };
  const int64_t pos = p.index[0];
  if (n >= nQ + nK) {   // v
    if (pos < 0 || pos >= p.max_seq) return;
    const int c = n - nQ - nK, hk = c / D, d = c % D;
    const f32x4 s = sum4(off);
    *(u32x2 *)(p.v_cache + ((p.batch_offset + m) * p.kv_heads + hk) * p.seq_pad * D + ttm_tiled_offset(pos, d, ct)) =
        u32x2{ttm_pack_bf16x2(s.x, s.y), ttm_pack_bf16x2(s.z, s.w)};
    return;
  }
  const bool isq = n < nQ;
  if (!isq && (pos < 0 || pos >= p.max_seq)) return;
  const int c = isq ? n : n - nQ, h = c / D, d = c % D, half = D >> 1;
  const int pn = n - d + (d < half ? d + half : d - half);   // partner column in the concatenation
  const float sign = d < half ? -1.0f : 1.0f;
  const int64_t poff = (int64_t)(pn >> 5) * 1024 + ((m >> 4) * 2 + ((pn >> 4) & 1)) * 256 + (m & 15) * 16 + (pn & 15);
  const f32x4 x = sum4(off), xp = sum4(poff);
  const int64_t co = ttm_tiled_offset(p.cos_row, d, ct);
  const u32x2 cr = *(const u32x2 *)(p.cosc + co), sr = *(const u32x2 *)(p.sinc + co);
  const float cv[4] = {__uint_as_float(cr.x << 16), __uint_as_float(cr.x & 0xFFFF0000u), __uint_as_float(cr.y << 16), __uint_as_float(cr.y & 0xFFFF0000u)};
  const float sv[4] = {__uint_as_float(sr.x << 16), __uint_as_float(sr.x & 0xFFFF0000u), __uint_as_float(sr.y << 16), __uint_as_float(sr.y & 0xFFFF0000u)};
  float o[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) o[j] = ttm_rotary_value(r16(x[j]), r16(xp[j]), cv[j], sv[j], sign);
  const u32x2 packed = {ttm_pack_bf16x2(o[0], o[1]), ttm_pack_bf16x2(o[2], o[3])};
  if (isq) *(u32x2 *)(p.q_out + (int64_t)m * p.heads_pad * D + ttm_tiled_offset(h, d, ct)) = packed;
  else *(u32x2 *)(p.k_cache + ((p.batch_offset + m) * p.kv_heads + h) * p.seq_pad * D + ttm_tiled_offset(pos, d, ct)) = packed;
}

static int device_cu_count() {
  static int cus = 0;
  if (cus == 0) {
    int dev = 0, n = 0;
    if (hipGetDevice(&dev) == hipSuccess && hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && n > 0) cus = n;
    else cus = 256;
  }
  return cus;
}

// Grid of the block-float main kernel: block width (8, 6 or 4 column tiles) and number of k-slices, chosen by a
// small cost model fitted to measurements on the config shapes.  A block costs (k-steps + 12) x 1.65 us at full width
// (the 12 stand for prologue and epilogue), 0.92 / 0.78 of that at 6 / 4 tiles (a narrower block keeps the whole
// activation traffic of a wide one); blocks run in rounds of one per CU; a split reduction adds its fp32 partial
// traffic, (slices + 0.5) x M x N x 4 bytes, at 4 TB/s.  force_* != 0 pin a choice (tests, measurements).
// column units of `unit_tiles` tiles in a launch: a group numbers its members' units one after another
static int column_units(const LinearArgs &p, int unit_tiles) {
  if (p.group_n <= 1) return (p.Nt + unit_tiles - 1) / unit_tiles;
  int n = 0;
  for (int j = 0; j < p.group_n; ++j) n += (p.gNt[j] + unit_tiles - 1) / unit_tiles;
  return n;
}

static int plan_dma_grid(LinearArgs &p, int cus, int force_ntw, int force_slices, int two_part = 0) {
  const int mbk = p.m_blocks, ksteps = (p.Kt + 1) / 2;
  static const double width_cost[5] = {0, 0, 0.78, 0.92, 1.0};
  double best = 1e30;
  int best_ntw = 4, best_slices = 1;
  for (int ntw = 4; ntw >= 2; --ntw) {
    if (force_ntw && ntw != force_ntw) continue;
    const int blocks = mbk * column_units(p, 2 * ntw);
    for (int slices = 1; slices <= 8; slices *= 2) {
      if (force_slices ? slices != 1 : (slices > 1 && ksteps / slices < 8)) continue;
      const int rounds = (blocks * slices + cus - 1) / cus;
      double t = rounds * width_cost[ntw] * ((ksteps + slices - 1) / slices + 12) * 1.65;
      if (slices > 1) t += (slices + 0.5) * (double)p.Mt * p.Nt * 4096.0 / 4.0e6;
      if (t < best * 0.97) { best = t; best_ntw = ntw; best_slices = slices; }   // ties go to the wider, unsplit choice
    }
  }
  if (force_slices) best_slices = force_slices;
  p.ntw = best_ntw;
  p.n_blocks = mbk * column_units(p, 2 * best_ntw);   // blocks per k-slice
  p.nt_split = 0;
  // Optional (linear_two_part = 1): unsplit, full-width grids whose last round is partly filled keep the full rounds at
  // 8 tiles and cover the remaining columns with narrower blocks when the model says those cost fewer CU-rounds.
  // [2048, 4096] x [4096, 14336]: 256 blocks of 8 tiles + 256 blocks of 6 tiles instead of 448 of 8 - modelled 1.92
  // rounds instead of 2, measured 262 us instead of 250, so it is off unless asked for.
  if (best_slices == 1 && best_ntw == 4 && !force_ntw && two_part != 0 && p.group_n <= 1) {
    const int full_rounds = p.n_blocks / cus;
    const int cols1 = full_rounds * cus / mbk;            // column blocks (8 tiles) the full rounds cover
    const int rem = p.Nt - 8 * cols1;                      // column tiles left
    if (full_rounds >= 1 && rem > 0 && p.n_blocks % cus != 0) {
      const double step = (ksteps + 12) * 1.65;
      double t_one = ((p.n_blocks + cus - 1) / cus) * step, t_best = t_one;
      int pick = 0;
      for (int ntw2 = 3; ntw2 >= 2; --ntw2) {
        const int blocks2 = mbk * ((rem + 2 * ntw2 - 1) / (2 * ntw2));
        const double t = full_rounds * step + ((blocks2 + cus - 1) / cus) * width_cost[ntw2] * step;
        if (t < t_best * 0.99) { t_best = t; pick = ntw2; }
      }
      if (pick) {
        p.nt_split = 8 * cols1;
        p.n_blocks1 = mbk * cols1;
        p.ntw2 = pick;
        p.n_blocks = p.n_blocks1 + mbk * ((rem + 2 * pick - 1) / (2 * pick));
      }
    }
  }
  return best_slices;
}

template <typename K>
static int set_lds_limit(K kernel, int bytes) {
  hipError_t e = hipFuncSetAttribute((const void *)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
  if (e != hipSuccess) return ttm_set_error(TTM_ERR_HIP, "hipFuncSetAttribute(LDS %d): %s", bytes, hipGetErrorString(e));
  return 0;
}

template <int WF>
static int launch_linear(const LinearArgs &a, int64_t batch, hipStream_t s) {
  constexpr bool BFP = WF == WF_BFP8 || WF == WF_BFP4;
  // up to linear_small_m_max rows (64) the small kernels run once per row tile; bf16 weights leave them after one row tile
  // (from two on the image route is faster: [14336, 4096] at M = 64 116 us against 75 us)
  if (a.Mt == 1 || (BFP && a.Mt * 32 <= ttm_option("linear_small_m_max"))) {
    // the small kernel handles one row tile per launch
    LinearArgs p = a;
    const bool decode = BFP && ttm_option("linear_variant") != 1 && (int64_t)a.Nt * 1088 < (int64_t)1 << 32;
    if (a.group_n > 1 && !decode) return ttm_set_error(TTM_ERR_INVALID, "ttm_linear_group: the selected kernel variant has no group form");
    // the decode kernel has one workgroup per 64 columns: narrow outputs split K until there is one workgroup per CU,
    // as long as a slice keeps 32 k-tiles (four per wavefront, the depth of its load ring); the slices leave fp32
    // partial sums that ttm_linear_reduce_k finishes.  Measured at M = 32: [4096, 4096] 14.3 -> 10.6 us,
    // [14336, 4096] 38 -> 19 us with 4 slices; 8 slices or splitting a [4096, 14336] weight are slower than not splitting.
    int slices = 1, np = 1;
    int64_t units = a.Nt;   // workgroups along the columns
    if (a.glu && !decode) return ttm_set_error(TTM_ERR_INVALID, "ttm_linear_glu: the selected kernel variant has no gated form");
    if (decode) {
      const int cus = device_cu_count();
      if (a.glu) {   // a workgroup's two tile pairs are the same 64 columns of the two matrices
        np = 2;
        units = (a.gNt[0] + 1) / 2;
      } else {
        // A workgroup owns 64 columns, or 128 (linear_decode_wide: 0 = by the rule, 1 = never, 2 = always): the wide form reads
        // the activations once per 128 columns and fills a CU with one workgroup where the narrow form needs two, which pays
        // when it also rounds better to whole rounds of the device.  Measured at M = 32, K = 4096 (narrow / wide, us):
        // N = 28672 30.7 / 27.3, 32000 31.3 / 28.3, 43008 44.3 / 50.0, 57344 57.3 / 53.3, 128256 121.3 / 114.7; one round of
        // wide workgroups costs 1.8 narrow ones.  Launches that split K stay narrow (N = 14336 in two slices: 17.3 against 16.1 us).
        const int wide = ttm_option("linear_decode_wide");
        const int64_t gn = (int64_t)column_units(a, 2) * batch, gw = (int64_t)column_units(a, 4) * batch;
        np = wide == 2 || (wide == 0 && gn >= cus && ((gw + cus - 1) / cus) * 9 < ((gn + cus - 1) / cus) * 5) ? 2 : 1;
        units = column_units(a, 2 * np);
      }
      const int64_t groups = units * batch;
      slices = a.glu ? 1 : ttm_option("linear_decode_split");
      if (slices <= 0) {
        slices = (int)(cus / groups);
        if (slices > a.Kt / 32) slices = a.Kt / 32;
      }
      if (slices > a.Kt) slices = a.Kt;
      if (slices < 1) slices = 1;
      if (slices > 1) {
        p.k_slice = (a.Kt + slices - 1) / slices;
        slices = (a.Kt + p.k_slice - 1) / p.k_slice;
      }
    }
    const int64_t per = (int64_t)a.Nt * 1024;
    if (a.qkv && (!decode || a.Mt != 1 || batch != 1)) return ttm_set_error(TTM_ERR_INVALID, "ttm_linear_qkv_decode: the selected kernel variant cannot end in the fused step");
    if (a.norm && (!decode || a.Mt != 1 || batch != 1)) return ttm_set_error(TTM_ERR_INVALID, "ttm_linear_add_rms_norm: the selected kernel variant cannot end in the fused step");
    if (slices > 1 || a.qkv || a.norm) {
      void *ws = nullptr;
      if (int rc = ttm_stream_workspace(s, (size_t)(per * slices * batch) * sizeof(float), &ws)) return rc;
      p.partial = (float *)ws;
      p.Mt = 1;   // the reduction sees one row tile per launch
    }
    for (int mt = 0; mt < a.Mt; ++mt) {
      p.A = a.A + (int64_t)mt * a.Kt * 2048;
      p.C = a.C + (int64_t)mt * a.Nt * 2048;
      for (int j = 0; j < a.group_n; ++j) p.gC[j] = a.gC[j] + (int64_t)mt * a.gNt[j] * 2048;
      const dim3 grid((unsigned)units, slices, (unsigned)batch);
      const bool two_term = ttm_option("linear_decode_variant") != 1;   // 1 = operands by int -> float conversion
      if (decode) {
        constexpr bool B4 = WF == WF_BFP4;
        if (np == 2) {
          static bool attr = false;
          if (!attr) {
            if (int rc = set_lds_limit(ttm_linear_decode_k<B4, true, 2, false>, 131072)) return rc;
            if (int rc = set_lds_limit(ttm_linear_decode_k<B4, false, 2, false>, 131072)) return rc;
            if (int rc = set_lds_limit(ttm_linear_decode_k<B4, true, 2, true>, 131072)) return rc;
            if (int rc = set_lds_limit(ttm_linear_decode_k<B4, false, 2, true>, 131072)) return rc;
            attr = true;
          }
          if (a.glu) {
            if (two_term) hipLaunchKernelGGL((ttm_linear_decode_k<B4, true, 2, true>), grid, dim3(512), 131072, s, p);
            else hipLaunchKernelGGL((ttm_linear_decode_k<B4, false, 2, true>), grid, dim3(512), 131072, s, p);
          } else if (two_term) hipLaunchKernelGGL((ttm_linear_decode_k<B4, true, 2, false>), grid, dim3(512), 131072, s, p);
          else hipLaunchKernelGGL((ttm_linear_decode_k<B4, false, 2, false>), grid, dim3(512), 131072, s, p);
        } else if (two_term) hipLaunchKernelGGL((ttm_linear_decode_k<B4, true, 1, false>), grid, dim3(512), 65536, s, p);
        else hipLaunchKernelGGL((ttm_linear_decode_k<B4, false, 1, false>), grid, dim3(512), 65536, s, p);
      }
      else hipLaunchKernelGGL((ttm_linear_small_k<WF>), dim3(a.Nt, 1, (unsigned)batch), dim3(256), 0, s, p);
      if (a.qkv) {
        QkvFinishArgs f = *a.qkv;
        f.partial = p.partial; f.slices = slices; f.per = per;
        const int64_t lanes = per / 4 + (int64_t)f.users * (f.heads_pad - f.heads) * (f.dim / 4);
        hipLaunchKernelGGL(ttm_qkv_finish_k, dim3((unsigned)((lanes + 255) / 256)), dim3(256), 0, s, f);
      } else if (a.norm) {
        const NormFinishArgs &f = *a.norm;
        if (int rc = ttm_rowwise_rmsnorm_from_partials(p.partial, slices, per, f.residual, f.sum_out, f.weight, f.weight_layout, f.bias,
                                                       f.bias_layout, f.out, f.rows, f.cols, f.eps, s))
          return rc;
      } else if (slices > 1)
        hipLaunchKernelGGL(ttm_linear_reduce_k, dim3((unsigned)((per / 4 + 255) / 256), 1, (unsigned)batch), dim3(256), 0, s, p, slices);
    }
    return 0;
  }
  // linear_variant: 0 = automatic, 1 = 64-bit-addressed fallback, 5 = register-staged kernel, 6 = LDS-direct kernel
  int variant = ttm_option("linear_variant");
  // the main kernels keep per-lane 32-bit offsets into one batch entry of the activations ([N,K] weights too)
  const bool fits32 = (int64_t)a.Mt * a.Kt * 2048 < (int64_t)1 << 32 && (int64_t)a.Nt * a.Kt * 2048 < (int64_t)1 << 32;
  if (variant == 0) variant = !fits32 ? 1 : 6;
  // bf16 weights reach the LDS-direct kernel through images of one weight set, which it addresses with 32 bits
  if (!BFP && variant == 6 && (int64_t)((a.Kt + 1) / 2 + 1) * a.Nt * 4096 >= ((int64_t)1 << 31)) variant = 5;
  if ((variant == 5 || variant == 6) && !fits32) return ttm_set_error(TTM_ERR_INVALID, "ttm_linear: operand too large for the selected kernel variant");
  if (a.group_n > 1 && variant != 6) return ttm_set_error(TTM_ERR_INVALID, "ttm_linear_group: the selected kernel variant has no group form");
  const int lds_bytes = 2 * 4096 * 16;
  {
    if (variant == 6) {
      // bf16 weights always take two passes: the first rewrites them as the same images (a permutation), which gives them
      // the block-float path's second pass with its seven-wide blocks and split K; the register-staged kernel that served
      // them before (linear_variant = 5) has neither and loops over K at a third of the speed
      constexpr int WI = BFP ? WF : WF_BFP8;   // the second pass only sees images
      const int lds6 = 131072 + (WF == WF_BFP8 ? 32768 : 16384);
      if constexpr (BFP) {
        static bool attr = false;
        if (!attr) {
          if (int rc = set_lds_limit(ttm_linear_dma_k<WF>, lds6)) return rc;
          attr = true;
        }
      }
      LinearArgs p = a;
      const int cus = device_cu_count();
      const int force_ntw = ttm_option("linear_ntw") == 7 ? 0 : ttm_option("linear_ntw");   // 7 exists in the second pass only
      // a group is not split along K: its partial sums would need a reduction that knows the members
      int slices = plan_dma_grid(p, cus, force_ntw, a.group_n > 1 ? 1 : ttm_option("linear_split_k"), ttm_option("linear_two_part") == 1);
      slices = slices < 1 ? 1 : (slices > a.Kt ? a.Kt : slices);
      if (slices > 1) {
        p.k_slice = (a.Kt + slices - 1) / slices;
        p.k_slice += p.k_slice & 1;                         // whole k-steps per slice
        slices = (a.Kt + p.k_slice - 1) / p.k_slice;
      }
      // Two passes when the conversion is repeated often enough: every block of 256 rows dequantises the weights it
      // multiplies, so with M / 256 row blocks the same conversion runs M / 256 times.  The first pass writes the weights
      // once as bf16 fragment images into the stream's workspace, the second runs the main loop without conversion
      // (measured at [2048, 4096] x [4096, 14336]: 230 us fused; 26 us for the image pass + 188 us for the second pass).
      // Modelled: the fused loop costs what plan_dma_grid says, the first pass 3 us + (tile bytes + 2048) per tile at
      // 5.5 TB/s, and the second pass saves a share of the fused loop that depends on what the conversion cost there:
      // 0.28 for bfp8_b and 0.22 for bfp4_b, whose conversion is cheaper; for launches that split K 0.18 and 0.08
      // (measured: [2048, 4096] x [4096, 4096] bfp8_b 87 us fused, 80 us in two passes; [2048, 14336] x [14336, 4096]
      // bfp4_b 225 us fused, 231 us in two passes; [1024, 4096] x [4096, 14336] bfp8_b 112 against 114 us).
      // linear_two_pass: 0 = by the model, 1 = never, 2 = always.
      const int ksteps = (a.Kt + 1) / 2;
      const int64_t sets = a.w_batch == 0 ? 1 : batch;
      const int64_t img_set = (int64_t)(ksteps + 1) * a.Nt * 4096;   // a group: the members' image sets back to back
      bool two_pass = ttm_option("linear_two_pass") == 2 || !BFP;
      if (BFP && ttm_option("linear_two_pass") == 0) {
        static const double width_cost[5] = {0, 0, 0.78, 0.92, 1.0};
        const int64_t rounds = ((int64_t)p.n_blocks * slices * batch + cus - 1) / cus;
        const double fused = rounds * width_cost[p.ntw] * ((ksteps + slices - 1) / slices + 12) * 1.65;
        const double first = 3.0 + (double)sets * a.Kt * a.Nt * ((WF == WF_BFP8 ? 1088.0 : 576.0) + 2048.0) / 5.5e6;
        const double gain = WF == WF_BFP8 ? (slices == 1 ? 0.28 : 0.18) : (slices == 1 ? 0.22 : 0.08);
        two_pass = gain * fused > first && img_set < ((int64_t)1 << 31);
      }
      const int64_t per = (int64_t)a.Mt * a.Nt * 1024;
      const size_t img_bytes = two_pass ? (size_t)((img_set * sets + 255) / 256 * 256) : 0;
      const size_t part_bytes = slices > 1 ? (size_t)(per * slices * batch) * sizeof(float) : 0;
      uint8_t *ws = nullptr;
      if (img_bytes + part_bytes > 0)
        if (int rc = ttm_stream_workspace(s, img_bytes + part_bytes, (void **)&ws)) return rc;
      if (slices > 1) p.partial = (float *)(ws + img_bytes);
      if (two_pass && slices == 1 && p.nt_split == 0) {
        // without the conversion a block may be seven tiles wide (the wavefronts of a SIMD take 4 + 3): worth it when
        // that fills the last round, e.g. 8 x 448 tiles = 448 blocks of 8 (1.75 rounds on 256 CUs, paid as 2) against 512
        // blocks of 7 (2 rounds at 7/8 of the work each).  linear_ntw = 7 forces it.
        const int64_t blocks7 = (int64_t)p.m_blocks * column_units(a, 7);
        const int64_t rounds8 = ((int64_t)p.n_blocks * batch + cus - 1) / cus, rounds7 = (blocks7 * batch + cus - 1) / cus;
        static const double width_cost8[5] = {0, 0, 0.78, 0.92, 1.0};
        const bool pick7 = ttm_option("linear_ntw") == 7 || (ttm_option("linear_ntw") == 0 && rounds7 * 0.92 < rounds8 * width_cost8[p.ntw] * 0.98);
        if (pick7) { p.ntw = 7; p.n_blocks = (int)blocks7; }
      }
      if (two_pass) {
        static bool attr2 = false;
        if (!attr2) {
          if (int rc = set_lds_limit(ttm_linear_img_k<WI>, 131072)) return rc;
          attr2 = true;
        }
        if constexpr (!BFP) {
          hipLaunchKernelGGL((ttm_linear_image_bf16_k<WF == WF_BF16_NK>), dim3((a.Nt + 3) / 4, ksteps + 1, (unsigned)sets), dim3(256), 0, s, a.W,
                             a.w_batch, ws, img_set, a.Nt, a.Kt);
        } else if (a.group_n > 1) {
          ImageGroup g = {};
          g.n = a.group_n;
          uint8_t *at = ws;
          for (int j = 0; j < a.group_n; ++j) {
            g.W[j] = a.gW[j]; g.img[j] = at; g.Nt[j] = a.gNt[j];
            p.gW[j] = at;                                   // the second pass reads the images
            at += (int64_t)(ksteps + 1) * a.gNt[j] * 4096;
          }
          hipLaunchKernelGGL((ttm_linear_image_group_k<WF == WF_BFP4>), dim3(column_units(a, 4), ksteps + 1, 1), dim3(256), 0, s, g, a.Kt);
        } else {
          hipLaunchKernelGGL((ttm_linear_image_k<WF == WF_BFP4>), dim3((a.Nt + 3) / 4, ksteps + 1, (unsigned)sets), dim3(256), 0, s, a.W,
                             a.w_batch, ws, img_set, a.Nt, a.Kt);
        }
        p.W = ws;
        p.w_batch = a.w_batch == 0 ? 0 : img_set;
        p.img_zero_step = ksteps;
        if (ttm_option("linear_img_variant") == 1) {   // the 32x32x16 form of the second pass, for comparison
          if (int rc = set_lds_limit(ttm_linear_img_k<WI, false>, 131072)) return rc;
          hipLaunchKernelGGL((ttm_linear_img_k<WI, false>), dim3(p.n_blocks, slices, (unsigned)batch), dim3(512), 131072, s, p);
        } else {
          hipLaunchKernelGGL((ttm_linear_img_k<WI>), dim3(p.n_blocks, slices, (unsigned)batch), dim3(512), 131072, s, p);
        }
      } else if constexpr (BFP) {
        hipLaunchKernelGGL((ttm_linear_dma_k<WF>), dim3(p.n_blocks, slices, (unsigned)batch), dim3(512), lds6, s, p);
      }
      if (slices > 1)
        hipLaunchKernelGGL(ttm_linear_reduce_k, dim3((unsigned)((per / 4 + 255) / 256), 1, (unsigned)batch), dim3(256), 0, s, p, slices);
      return 0;
    }
  }
  if (variant == 5) {
    static bool attr = false;
    if (!attr) {
      if (int rc = set_lds_limit(ttm_linear_reg_k<WF>, lds_bytes)) return rc;
      attr = true;
    }
    hipLaunchKernelGGL((ttm_linear_reg_k<WF>), dim3(a.m_blocks * a.n_blocks, 1, (unsigned)batch), dim3(512), lds_bytes, s, a);
    return 0;
  }
  static bool attr = false;
  if (!attr) {
    if (int rc = set_lds_limit(ttm_linear_big_k<WF>, lds_bytes)) return rc;
    attr = true;
  }
  hipLaunchKernelGGL((ttm_linear_big_k<WF>), dim3(a.m_blocks * a.n_blocks, 1, (unsigned)batch), dim3(256), lds_bytes, s, a);
  return 0;
}

TTM_EXPORT int ttm_linear(const void *a, int a_dtype, const void *w, int w_dtype, int transpose_w, const void *bias,
                          int bias_dtype, int bias_layout, void *out, int out_dtype, int64_t batch,
                          int64_t w_batch, int64_t M, int64_t N, int64_t K, int act, void *stream) {
  TTM_EXTENTS(linear, a, a_dtype, w, w_dtype, bias, bias_dtype, bias_layout, out, out_dtype, batch, w_batch, M, N, K, TTM_TAIL_NONE, nullptr);
  return ttm_linear_tail(a, a_dtype, w, w_dtype, transpose_w, bias, bias_dtype, bias_layout, out, out_dtype, batch, w_batch, M, N, K, act,
                         TTM_TAIL_NONE, nullptr, stream);
}

// strides: optional byte strides between batch entries of the activations, weights and output, for operands that are not
// stored back to back (a pair of weight matrices applied to the same activations)
static int linear_entry(const void *a, int a_dtype, const void *w, int w_dtype, int transpose_w, const void *bias, int bias_dtype,
                        int bias_layout, void *out, int out_dtype, int64_t batch, int64_t w_batch, int64_t M, int64_t N, int64_t K,
                        int act, int tail_op, const void *tail, const int64_t *strides, void *stream,
                        const NormFinishArgs *norm = nullptr) {
  TTM_REQUIRE(tail_op >= TTM_TAIL_NONE && tail_op <= TTM_TAIL_MUL, "ttm_linear: unknown tail op %d", tail_op);
  TTM_REQUIRE((tail_op == TTM_TAIL_NONE) == (tail == nullptr), "ttm_linear: a tail op needs its operand, and only then");
  TTM_REQUIRE(((uintptr_t)tail & 15) == 0, "ttm_linear: the tail operand must be 16-byte aligned");
  TTM_REQUIRE(tail != out, "ttm_linear: the tail operand must not be the output");
  TTM_REQUIRE(a_dtype == TTM_BF16 && out_dtype == TTM_BF16, "ttm_linear: activations and output must be BFloat16");
  TTM_REQUIRE(w_dtype == TTM_BF16 || w_dtype == TTM_BFP8B || w_dtype == TTM_BFP4B,
              "ttm_linear: weights must be BFloat16, BFP_BFloat8 or BFP_BFloat4 (got %d)", w_dtype);
  TTM_REQUIRE(!(transpose_w && w_dtype != TTM_BF16), "ttm_linear: transposed block-float weights are not supported");
  TTM_REQUIRE(bias == nullptr || bias_dtype == TTM_BF16, "ttm_linear: bias must be BFloat16");
  TTM_REQUIRE(bias_layout == TTM_ROW_MAJOR || bias_layout == TTM_TILE, "ttm_linear: bad bias layout");
  TTM_REQUIRE(act >= TTM_ACT_NONE && act <= TTM_ACT_RELU, "ttm_linear: unknown activation %d", act);
  TTM_REQUIRE(batch >= 0 && M >= 0 && N >= 0 && K >= 0, "ttm_linear: negative dimension");
  TTM_REQUIRE(w_batch == 1 || w_batch == batch, "ttm_linear: weight batch must be 1 or equal the activation batch");
  if (batch == 0 || M == 0 || N == 0) return TTM_OK;
  TTM_REQUIRE(K > 0, "ttm_linear: K must be positive");
  TTM_REQUIRE(a && w && out, "ttm_linear: null pointer");
  TTM_REQUIRE(((uintptr_t)a & 15) == 0 && ((uintptr_t)w & 15) == 0 && ((uintptr_t)out & 15) == 0 &&
                  ((uintptr_t)bias & 7) == 0,
              "ttm_linear: operands must be 16-byte aligned (bias 8)");
  LinearArgs p;
  p.A = (const uint8_t *)a; p.W = (const uint8_t *)w; p.bias = (const uint16_t *)bias; p.C = (uint8_t *)out;
  p.Mt = (int)ttm_cdiv(M, 32); p.Nt = (int)ttm_cdiv(N, 32); p.Kt = (int)ttm_cdiv(K, 32);
  p.act = act; p.bias_tiled = bias_layout == TTM_TILE;
  const int64_t w_tile = w_dtype == TTM_BFP8B ? 1088 : (w_dtype == TTM_BFP4B ? 576 : 2048);
  p.a_batch = (int64_t)p.Mt * p.Kt * 2048;
  p.w_batch = w_batch == 1 ? 0 : (int64_t)p.Kt * p.Nt * w_tile;
  p.c_batch = (int64_t)p.Mt * p.Nt * 2048;
  p.m_blocks = (p.Mt + 7) / 8; p.n_blocks = (p.Nt + 7) / 8;
  p.ntw = 4;
  p.k_slice = p.Kt; p.partial = nullptr;
  p.nt_split = p.n_blocks1 = p.ntw2 = 0;
  p.img_zero_step = 0;
  p.group_n = 0; p.glu = 0;
  for (int j = 0; j < 4; ++j) { p.gW[j] = nullptr; p.gC[j] = nullptr; p.gNt[j] = 0; p.gAct[j] = TTM_ACT_NONE; }
  p.tail = tail_op;
  p.tail_delta = tail ? (const uint8_t *)tail - (const uint8_t *)out : 0;
  p.qkv = nullptr;
  p.norm = norm;
  if (strides) { p.a_batch = strides[0]; p.w_batch = strides[1]; p.c_batch = strides[2]; }
  TTM_REQUIRE(batch <= 65535, "ttm_linear: batch too large");
  hipStream_t s = (hipStream_t)stream;
  int rc;
  if (w_dtype == TTM_BFP8B) rc = launch_linear<WF_BFP8>(p, batch, s);
  else if (w_dtype == TTM_BFP4B) rc = launch_linear<WF_BFP4>(p, batch, s);
  else if (transpose_w) rc = launch_linear<WF_BF16_NK>(p, batch, s);
  else rc = launch_linear<WF_BF16_KN>(p, batch, s);
  if (rc) return rc;
  TTM_LAUNCH_CHECK();
  return TTM_OK;
}

TTM_EXPORT int ttm_linear_tail(const void *a, int a_dtype, const void *w, int w_dtype, int transpose_w, const void *bias,
                               int bias_dtype, int bias_layout, void *out, int out_dtype, int64_t batch, int64_t w_batch,
                               int64_t M, int64_t N, int64_t K, int act, int tail_op, const void *tail, void *stream) {
  TTM_EXTENTS(linear, a, a_dtype, w, w_dtype, bias, bias_dtype, bias_layout, out, out_dtype, batch, w_batch, M, N, K, tail_op, tail);
  return linear_entry(a, a_dtype, w, w_dtype, transpose_w, bias, bias_dtype, bias_layout, out, out_dtype, batch, w_batch, M, N, K, act,
                      tail_op, tail, nullptr, stream);
}

TTM_EXPORT int ttm_linear_add_rms_norm_supported(int w_dtype, int64_t M, int64_t N, int64_t K) {
  return (w_dtype == TTM_BFP8B || w_dtype == TTM_BFP4B) && M >= 1 && M <= 32 && K > 0 && N >= 1 && ttm_rowwise_partials_supported(M, N) &&
         ttm_option("linear_variant") != 1 && ttm_option("linear_small_m_max") >= 32 && ttm_cdiv(N, 32) * 1088 < (int64_t)1 << 32;
}

TTM_EXPORT int ttm_linear_add_rms_norm(const void *a, const void *w, int w_dtype, const void *residual, void *sum_out, const void *norm_weight,
                                       int weight_layout, const void *norm_bias, int bias_layout, float eps, void *norm_out, int64_t M,
                                       int64_t N, int64_t K, void *stream) {
  TTM_EXTENTS(linear_add_rms_norm, a, w, w_dtype, residual, sum_out, norm_weight, weight_layout, norm_bias, bias_layout, norm_out, M, N, K);
  TTM_REQUIRE(ttm_linear_add_rms_norm_supported(w_dtype, M, N, K),
              "ttm_linear_add_rms_norm: needs block-float weights, 1..32 rows and at most 16384 columns");
  TTM_REQUIRE(residual && sum_out && norm_out, "ttm_linear_add_rms_norm: null pointer");
  TTM_REQUIRE(sum_out != residual && norm_out != sum_out && norm_out != residual, "ttm_linear_add_rms_norm: the outputs must not alias the residual or each other");
  TTM_REQUIRE((((uintptr_t)residual | (uintptr_t)norm_out) & 15) == 0, "ttm_linear_add_rms_norm: operands must be 16-byte aligned");
  NormFinishArgs f = {residual, norm_weight, norm_bias, weight_layout, bias_layout, sum_out, norm_out, M, N, eps};
  return linear_entry(a, TTM_BF16, w, w_dtype, 0, nullptr, TTM_BF16, TTM_TILE, sum_out, TTM_BF16, 1, 1, M, N, K, TTM_ACT_NONE, TTM_TAIL_NONE,
                      nullptr, nullptr, stream, &f);
}

TTM_EXPORT int ttm_linear_pair(const void *a, const void *w0, const void *w1, int w_dtype, void *out0, void *out1, int64_t M,
                               int64_t N, int64_t K, void *stream) {
  TTM_EXTENTS(linear_pair, a, w0, w1, w_dtype, out0, out1, M, N, K);
  TTM_REQUIRE(w0 && w1 && out0 && out1 && w0 != w1 && out0 != out1, "ttm_linear_pair: two distinct weight and output tensors are needed");
  TTM_REQUIRE((((uintptr_t)w1 | (uintptr_t)out1) & 15) == 0, "ttm_linear_pair: operands must be 16-byte aligned");
  const int64_t strides[3] = {0, (const uint8_t *)w1 - (const uint8_t *)w0, (uint8_t *)out1 - (uint8_t *)out0};
  return linear_entry(a, TTM_BF16, w0, w_dtype, 0, nullptr, TTM_BF16, TTM_TILE, out0, TTM_BF16, 2, 2, M, N, K, TTM_ACT_NONE,
                      TTM_TAIL_NONE, nullptr, strides, stream);
}

// The rule of launch_linear for a single projection of this shape: does the decode kernel run it unsplit?
static bool decode_runs_unsplit(int64_t N, int64_t K) {
  const int64_t groups = (ttm_cdiv(N, 32) + 1) / 2, kt = ttm_cdiv(K, 32);
  int64_t slices = ttm_option("linear_decode_split");
  if (slices <= 0) slices = std::min<int64_t>(device_cu_count() / groups, kt / 32);
  return slices <= 1;
}

// Token counts at which the gated form of the fused main kernel is used: those where the two projections would otherwise
// share one launch and leave their product to an element-wise kernel (a projection alone would split K to fill the device).
static bool glu_main_ok(int w_dtype, int64_t M, int64_t N, int64_t K) {
  const int64_t Mt = ttm_cdiv(M, 32), Nt = ttm_cdiv(N, 32), Kt = ttm_cdiv(K, 32);
  const int variant = ttm_option("linear_variant");
  if (!(w_dtype == TTM_BFP8B && M > 64 && M <= 1024 && M > ttm_option("linear_small_m_max") && (variant == 0 || variant == 6) &&
        ttm_option("linear_two_pass") != 2 && ttm_option("linear_glu_main") != 1 && Mt * Kt * 2048 < (int64_t)1 << 32 &&
        Nt * Kt * 2048 < (int64_t)1 << 32 && Nt * 1088 < (int64_t)1 << 31))
    return false;
  if (ttm_option("linear_two_pass") == 1) return true;
  // The other sequence is the group launch of the two projections and an element-wise multiply.  Where launch_linear's model
  // sends the group through the image pass (the gated kernel converts its weights in every block of 256 rows), that sequence
  // wins if the image pass gains more than the multiply costs (3 us + three tensors of M x N bf16 at 5.5 TB/s).  Measured,
  // sequence / gated in us, K x N = 4096 x 14336: M = 128 105 / 101, 512 138 / 125, 768 248 / 226, 1024 311 / 240;
  // 4096 x 4096: 512 84 / 99, 1024 102 / 110; 1024 x 2816: 1024 35 / 37; 2048 x 8192: 1024 91 / 77; 8192 x 28672: 512 508 / 491.
  const int cus = device_cu_count();
  const int64_t ksteps = (Kt + 1) / 2, blocks = ttm_cdiv(Mt, 8) * ttm_cdiv(2 * Nt, 8), rounds = (blocks + cus - 1) / cus;
  const double fused = rounds * (ksteps + 12) * 1.65, first = 3.0 + (double)Kt * 2 * Nt * (1088.0 + 2048.0) / 5.5e6;
  const double multiply = 3.0 + 3.0 * (double)Mt * Nt * 2048.0 / 5.5e6;
  return !(0.28 * fused - first > multiply);
}

TTM_EXPORT int ttm_linear_glu_supported(int w_dtype, int64_t M, int64_t N, int64_t K) {
  if (M >= 1 && K > 0 && N >= 1 && glu_main_ok(w_dtype, M, N, K)) return 1;
  return (w_dtype == TTM_BFP8B || w_dtype == TTM_BFP4B) && M >= 1 && M <= 32 && K > 0 && N >= 1 && ttm_option("linear_variant") != 1 &&
         ttm_option("linear_decode_wide") != 1 && ttm_option("linear_small_m_max") >= 32 && ttm_cdiv(N, 32) * 1088 < (int64_t)1 << 32 &&
         decode_runs_unsplit(N, K);
}

TTM_EXPORT int ttm_linear_glu(const void *a, const void *w_gate, const void *w_up, int w_dtype, void *out, int64_t M, int64_t N, int64_t K,
                              int act_gate, int act_up, void *stream) {
  TTM_EXTENTS(linear_glu, a, w_gate, w_up, w_dtype, out, M, N, K);
  TTM_REQUIRE(ttm_linear_glu_supported(w_dtype, M, N, K),
              "ttm_linear_glu: needs block-float weights and 1..32 rows with enough columns for the decode kernel to run unsplit, or bfp8_b weights and 65..1024 rows");
  TTM_REQUIRE(a && w_gate && w_up && out, "ttm_linear_glu: null pointer");
  TTM_REQUIRE((((uintptr_t)a | (uintptr_t)w_gate | (uintptr_t)w_up | (uintptr_t)out) & 15) == 0, "ttm_linear_glu: operands must be 16-byte aligned");
  TTM_REQUIRE(act_gate >= TTM_ACT_NONE && act_gate <= TTM_ACT_RELU && act_up >= TTM_ACT_NONE && act_up <= TTM_ACT_RELU,
              "ttm_linear_glu: unknown activation %d / %d", act_gate, act_up);
  LinearArgs p;
  p.A = (const uint8_t *)a; p.W = (const uint8_t *)w_gate; p.bias = nullptr; p.C = (uint8_t *)out;
  p.Mt = 1; p.Kt = (int)ttm_cdiv(K, 32); p.Nt = (int)ttm_cdiv(N, 32);
  p.group_n = 0; p.glu = 1;
  for (int j = 0; j < 4; ++j) { p.gW[j] = nullptr; p.gC[j] = nullptr; p.gNt[j] = 0; p.gAct[j] = TTM_ACT_NONE; }
  p.gW[0] = (const uint8_t *)w_gate; p.gW[1] = (const uint8_t *)w_up; p.gC[0] = (uint8_t *)out;
  p.gNt[0] = p.gNt[1] = p.Nt; p.gAct[0] = act_gate; p.gAct[1] = act_up;
  p.act = TTM_ACT_NONE; p.bias_tiled = 1;
  p.a_batch = p.w_batch = p.c_batch = 0;
  p.m_blocks = 1; p.n_blocks = (p.Nt + 7) / 8;
  p.ntw = 4;
  p.k_slice = p.Kt; p.partial = nullptr;
  p.nt_split = p.n_blocks1 = p.ntw2 = 0;
  p.img_zero_step = 0;
  p.tail = TTM_TAIL_NONE; p.tail_delta = 0;
  p.qkv = nullptr; p.norm = nullptr;
  hipStream_t s = (hipStream_t)stream;
  if (M > 32) {   // the fused main kernel over the tile slots of both matrices: blocks of 256 rows x four column tiles of each
    p.Mt = (int)ttm_cdiv(M, 32);
    p.Nt = 2 * p.gNt[0];
    p.m_blocks = (p.Mt + 7) / 8;
    p.n_blocks = p.m_blocks * ((p.Nt + 7) / 8);
    static bool attr = false;
    if (!attr) {
      if (int rc = set_lds_limit(ttm_linear_dma_glu_k, 131072 + 32768)) return rc;
      attr = true;
    }
    hipLaunchKernelGGL(ttm_linear_dma_glu_k, dim3((unsigned)p.n_blocks), dim3(512), 131072 + 32768, s, p);
    TTM_LAUNCH_CHECK();
    return TTM_OK;
  }
  const int rc = w_dtype == TTM_BFP8B ? launch_linear<WF_BFP8>(p, 1, s) : launch_linear<WF_BFP4>(p, 1, s);
  if (rc) return rc;
  TTM_LAUNCH_CHECK();
  return TTM_OK;
}

static int linear_group_entry(const void *a, int n, const void *const *w, int w_dtype, void *const *out, const int64_t *N,
                              const int *act, int64_t M, int64_t K, const QkvFinishArgs *qkv, void *stream) {
  TTM_REQUIRE(n >= 1 && n <= 4, "ttm_linear_group: 1 to 4 members (got %d)", n);
  TTM_REQUIRE(a && w && out && N, "ttm_linear_group: null pointer");
  TTM_REQUIRE(w_dtype == TTM_BFP8B || w_dtype == TTM_BFP4B, "ttm_linear_group: weights must be BFP_BFloat8 or BFP_BFloat4 (got %d)", w_dtype);
  TTM_REQUIRE(M >= 0 && K > 0, "ttm_linear_group: bad dimension");
  for (int j = 0; j < n; ++j) {
    TTM_REQUIRE(w[j] && out[j] && N[j] > 0, "ttm_linear_group: member %d has a null pointer or no columns", j);
    TTM_REQUIRE((((uintptr_t)w[j] | (uintptr_t)out[j]) & 15) == 0, "ttm_linear_group: operands must be 16-byte aligned");
    for (int i = 0; i < j; ++i) TTM_REQUIRE(out[i] != out[j], "ttm_linear_group: members %d and %d share an output", i, j);
    TTM_REQUIRE(!act || (act[j] >= TTM_ACT_NONE && act[j] <= TTM_ACT_RELU), "ttm_linear_group: unknown activation %d", act ? act[j] : 0);
  }
  if (n == 1 && !qkv)
    return ttm_linear(a, TTM_BF16, w[0], w_dtype, 0, nullptr, TTM_BF16, TTM_TILE, out[0], TTM_BF16, 1, 1, M, N[0], K, act ? act[0] : TTM_ACT_NONE, stream);
  if (M == 0) return TTM_OK;
  TTM_REQUIRE(((uintptr_t)a & 15) == 0, "ttm_linear_group: operands must be 16-byte aligned");
  LinearArgs p;
  p.A = (const uint8_t *)a; p.W = (const uint8_t *)w[0]; p.bias = nullptr; p.C = (uint8_t *)out[0];
  p.Mt = (int)ttm_cdiv(M, 32); p.Kt = (int)ttm_cdiv(K, 32); p.Nt = 0;
  p.group_n = n; p.glu = 0;
  for (int j = 0; j < 4; ++j) {
    p.gW[j] = j < n ? (const uint8_t *)w[j] : nullptr;
    p.gC[j] = j < n ? (uint8_t *)out[j] : nullptr;
    p.gNt[j] = j < n ? (int)ttm_cdiv(N[j], 32) : 0;
    p.gAct[j] = j < n && act ? act[j] : TTM_ACT_NONE;
    p.Nt += p.gNt[j];
  }
  p.act = TTM_ACT_NONE; p.bias_tiled = 1;
  p.a_batch = p.w_batch = p.c_batch = 0;
  p.m_blocks = (p.Mt + 7) / 8; p.n_blocks = (p.Nt + 7) / 8;
  p.ntw = 4;
  p.k_slice = p.Kt; p.partial = nullptr;
  p.nt_split = p.n_blocks1 = p.ntw2 = 0;
  p.img_zero_step = 0;
  p.tail = TTM_TAIL_NONE; p.tail_delta = 0;
  p.qkv = qkv;
  p.norm = nullptr;
  hipStream_t s = (hipStream_t)stream;
  const int rc = w_dtype == TTM_BFP8B ? launch_linear<WF_BFP8>(p, 1, s) : launch_linear<WF_BFP4>(p, 1, s);
  if (rc) return rc;
  TTM_LAUNCH_CHECK();
  return TTM_OK;
}

TTM_EXPORT int ttm_linear_group(const void *a, int n, const void *const *w, int w_dtype, void *const *out, const int64_t *N,
                                const int *act, int64_t M, int64_t K, void *stream) {
  if (n >= 1 && n <= 4 && w && out && N) TTM_EXTENTS(linear_group, a, n, w, w_dtype, out, N, M, K);
  return linear_group_entry(a, n, w, w_dtype, out, N, act, M, K, nullptr, stream);
}

TTM_EXPORT int ttm_linear_qkv_decode_supported(int w_dtype, int64_t users, int64_t K, int64_t heads, int64_t kv_heads, int64_t head_dim) {
  const int64_t Nt = (heads + 2 * kv_heads) * head_dim / 32;
  return (w_dtype == TTM_BFP8B || w_dtype == TTM_BFP4B) && users >= 1 && users <= 32 && K > 0 && heads >= 1 && kv_heads >= 1 &&
         head_dim >= 32 && head_dim % 32 == 0 && ttm_option("linear_variant") != 1 && ttm_option("linear_small_m_max") >= 32 &&
         Nt * 1088 < (int64_t)1 << 32;
}

TTM_EXPORT int ttm_linear_qkv_decode(const void *a, const void *wq, const void *wk, const void *wv, int w_dtype, int64_t users, int64_t K,
                                     int64_t heads, int64_t kv_heads, int64_t head_dim, const void *cos_cache, const void *sin_cache,
                                     int64_t cache_rows, int64_t token_index, void *q_out, void *k_cache, void *v_cache,
                                     int64_t cache_users, int64_t max_seq, const int32_t *update_index, int64_t batch_offset,
                                     void *stream) {
  TTM_EXTENTS(linear_qkv_decode, a, wq, wk, wv, w_dtype, users, K, heads, kv_heads, head_dim, cos_cache, sin_cache, cache_rows, q_out, k_cache, v_cache, cache_users, max_seq, update_index);
  TTM_REQUIRE(ttm_linear_qkv_decode_supported(w_dtype, users, K, heads, kv_heads, head_dim),
              "ttm_linear_qkv_decode: needs block-float weights, 1..32 users and a head_dim that is a multiple of 32");
  TTM_REQUIRE(a && wq && wk && wv && cos_cache && sin_cache && q_out && k_cache && v_cache && update_index, "ttm_linear_qkv_decode: null pointer");
  TTM_REQUIRE(cache_rows >= 1 && token_index >= 0 && token_index < cache_rows,
              "ttm_linear_qkv_decode: token_index %lld is outside the %lld cached positions", (long long)token_index, (long long)cache_rows);
  TTM_REQUIRE(max_seq >= 1 && batch_offset >= 0 && batch_offset + users <= cache_users,
              "ttm_linear_qkv_decode: batch_offset + users exceeds the cache");
  TTM_REQUIRE((((uintptr_t)cos_cache | (uintptr_t)sin_cache | (uintptr_t)q_out | (uintptr_t)k_cache | (uintptr_t)v_cache) & 15) == 0,
              "ttm_linear_qkv_decode: operands must be 16-byte aligned");
  QkvFinishArgs f = {};
  f.users = (int)users; f.heads = (int)heads; f.heads_pad = (int)ttm_round_up32(heads); f.kv_heads = (int)kv_heads; f.dim = (int)head_dim;
  f.cosc = (const uint16_t *)cos_cache; f.sinc = (const uint16_t *)sin_cache; f.cos_row = token_index;
  f.q_out = (uint16_t *)q_out; f.k_cache = (uint16_t *)k_cache; f.v_cache = (uint16_t *)v_cache;
  f.max_seq = max_seq; f.seq_pad = ttm_round_up32(max_seq); f.batch_offset = batch_offset; f.index = update_index;
  const void *w[3] = {wq, wk, wv};
  void *out[3] = {q_out, k_cache, v_cache};   // distinct, never written through these
  const int64_t N[3] = {heads * head_dim, kv_heads * head_dim, kv_heads * head_dim};
  return linear_group_entry(a, 3, w, w_dtype, out, N, nullptr, users, K, &f, stream);
}
