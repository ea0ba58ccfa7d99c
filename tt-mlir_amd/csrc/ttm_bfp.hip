// bfp8_b / bfp4_b block-float pack and unpack.
//
// Format (per 32x32 tile, faces in order (0,0) (0,1) (1,0) (1,1), 16 rows x 16 columns each):
//   bytes [0,64)   one shared exponent per 16-element face row: the largest biased fp32 exponent
//   bfp8_b         1024 mantissa bytes, sign<<7 | 7-bit magnitude
//   bfp4_b         512 mantissa bytes, two elements per byte, even column in the low nibble,
//                  nibble = sign<<3 | 3-bit magnitude
// Encode: hidden bit added, shifted right by (shared - own exponent), rounded to nearest even to
// the kept width, saturated; a magnitude of 0 drops the sign.  Decode: mag * 2^(E-127-(W-1)).
//
// Work split: one lane owns 4 consecutive elements of a face row, so a face row is a quad of
// lanes and a 64-lane wavefront owns one face.  The shared exponent is a max-reduction over the
// quad with two DPP quad_perm moves.  Mantissa writes of a wavefront are 256 (bfp8) / 128 (bfp4)
// contiguous bytes; reads from a row-major source are 64-byte (fp32) face-row segments.
#include "ttm_common.h"

template <int W>
__device__ __forceinline__ uint32_t bfp_encode(uint32_t bits, uint32_t E) {
  uint32_t e = (bits >> 23) & 0xFF;
  uint32_t sign = bits >> 31;
  uint32_t m = 0x800000u | (bits & 0x7FFFFFu);
  uint32_t shift = E - e;
  m = shift > 31 ? 0u : (m >> shift);
  constexpr int DROP = 24 - W;
  uint32_t keep = m >> DROP;
  uint32_t rem = m & ((1u << DROP) - 1);
  constexpr uint32_t HALF = 1u << (DROP - 1);
  keep += (rem > HALF || (rem == HALF && (keep & 1))) ? 1u : 0u;
  constexpr uint32_t MAXV = (1u << W) - 1;
  keep = keep > MAXV ? MAXV : keep;
  keep = ((bits & 0x7FFFFFFFu) == 0) ? 0u : keep;
  sign = keep == 0 ? 0u : sign;
  return (sign << W) | keep;
}

template <int W>
__device__ __forceinline__ float bfp_decode(uint32_t code, int E) {
  uint32_t mag = code & ((1u << W) - 1);
  uint32_t sign = (code >> W) & 1u;
  if (mag == 0) return 0.0f;
  int p = 31 - __clz(mag);
  int e = E - (W - 1) + p;  // biased exponent of the result
  uint32_t frac = (mag << (23 - p)) & 0x7FFFFFu;
  uint32_t bits;
  if (e >= 255) bits = 0x7F800000u;
  else if (e > 0) bits = ((uint32_t)e << 23) | frac;
  else bits = (0x800000u | frac) >> (1 - e);  // subnormal result, exact: at most 7 bits dropped, all zero
  return __uint_as_float(bits | (sign << 31));
}

__device__ __forceinline__ uint32_t quad_max(uint32_t v) {
  // quad_perm [1,0,3,2] then [2,3,0,1]
  uint32_t o = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0xB1, 0xF, 0xF, true);
  v = v > o ? v : o;
  o = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x4E, 0xF, 0xF, true);
  return v > o ? v : o;
}

struct QuadPos {
  int64_t tile;  // global tile index (over batch, tile rows, tile cols)
  int face, dy, q;
};
__device__ __forceinline__ QuadPos quad_pos(int64_t g) {
  QuadPos p;
  p.tile = g >> 8;
  int w = (int)(g & 255);
  p.face = w >> 6;
  p.dy = (w >> 2) & 15;
  p.q = w & 3;
  return p;
}

// SRC_BF16: plain side is bf16 (else fp32).  ROWMAJOR: plain side is row-major [batch, rows, cols]
// (else tile order).  PADDED: rows/cols not multiples of 32 (scalar, bounds-checked accesses).
template <int W, bool SRC_BF16, bool ROWMAJOR, bool PADDED>
__global__ __launch_bounds__(256) void ttm_bfp_pack_k(const void *__restrict__ src_, uint8_t *__restrict__ dst,
                                                      int64_t nquads, int64_t rows, int64_t cols, int64_t yt,
                                                      int64_t xt) {
  constexpr int TILE_BYTES = 64 + (W == 7 ? 1024 : 512);
  int64_t g = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (g >= nquads) return;  // nquads is a multiple of 256: whole blocks only
  QuadPos p = quad_pos(g);
  uint32_t bits[4];
  if (ROWMAJOR) {
    int64_t tx = p.tile % xt, tyb = p.tile / xt;
    int64_t b = tyb / yt, ty = tyb % yt;
    int64_t r = ty * 32 + (p.face >> 1) * 16 + p.dy;
    int64_t c = tx * 32 + (p.face & 1) * 16 + p.q * 4;
    int64_t off = (b * rows + r) * cols + c;
    if (PADDED) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        bool in = r < rows && (c + i) < cols;
        if (SRC_BF16) bits[i] = in ? ((uint32_t)((const uint16_t *)src_)[off + i] << 16) : 0u;
        else bits[i] = in ? ((const uint32_t *)src_)[off + i] : 0u;
      }
    } else if (SRC_BF16) {
      u32x2 v = __builtin_nontemporal_load((const u32x2 *)((const uint16_t *)src_ + off));
      bits[0] = v.x << 16; bits[1] = v.x & 0xFFFF0000u; bits[2] = v.y << 16; bits[3] = v.y & 0xFFFF0000u;
    } else {
      u32x4 v = __builtin_nontemporal_load((const u32x4 *)((const uint32_t *)src_ + off));
      bits[0] = v.x; bits[1] = v.y; bits[2] = v.z; bits[3] = v.w;
    }
  } else if (SRC_BF16) {
    u32x2 v = __builtin_nontemporal_load((const u32x2 *)src_ + g);
    bits[0] = v.x << 16; bits[1] = v.x & 0xFFFF0000u; bits[2] = v.y << 16; bits[3] = v.y & 0xFFFF0000u;
  } else {
    u32x4 v = __builtin_nontemporal_load((const u32x4 *)src_ + g);
    bits[0] = v.x; bits[1] = v.y; bits[2] = v.z; bits[3] = v.w;
  }
  uint32_t e0 = (bits[0] >> 23) & 0xFF, e1 = (bits[1] >> 23) & 0xFF;
  uint32_t e2 = (bits[2] >> 23) & 0xFF, e3 = (bits[3] >> 23) & 0xFF;
  uint32_t E = max(max(e0, e1), max(e2, e3));
  E = quad_max(E);
  uint32_t c0 = bfp_encode<W>(bits[0], E), c1 = bfp_encode<W>(bits[1], E);
  uint32_t c2 = bfp_encode<W>(bits[2], E), c3 = bfp_encode<W>(bits[3], E);
  uint8_t *tile = dst + p.tile * TILE_BYTES;
  if (p.q == 0) tile[p.face * 16 + p.dy] = (uint8_t)E;
  if (W == 7) {
    uint32_t word = c0 | (c1 << 8) | (c2 << 16) | (c3 << 24);
    __builtin_nontemporal_store(word, (uint32_t *)(tile + 64) + (g & 255));
  } else {
    uint16_t half = (uint16_t)(c0 | (c1 << 4) | (c2 << 8) | (c3 << 12));
    __builtin_nontemporal_store(half, (uint16_t *)(tile + 64) + (g & 255));
  }
}

template <int W, bool DST_BF16, bool ROWMAJOR, bool PADDED>
__global__ __launch_bounds__(256) void ttm_bfp_unpack_k(const uint8_t *__restrict__ src, void *__restrict__ dst_,
                                                        int64_t nquads, int64_t rows, int64_t cols, int64_t yt,
                                                        int64_t xt) {
  constexpr int TILE_BYTES = 64 + (W == 7 ? 1024 : 512);
  int64_t g = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (g >= nquads) return;
  QuadPos p = quad_pos(g);
  const uint8_t *tile = src + p.tile * TILE_BYTES;
  int E = tile[p.face * 16 + p.dy];
  float f[4];
  if (W == 7) {
    uint32_t word = __builtin_nontemporal_load((const uint32_t *)(tile + 64) + (g & 255));
#pragma unroll
    for (int i = 0; i < 4; ++i) f[i] = bfp_decode<7>((word >> (8 * i)) & 0xFF, E);
  } else {
    uint32_t half = __builtin_nontemporal_load((const uint16_t *)(tile + 64) + (g & 255));
#pragma unroll
    for (int i = 0; i < 4; ++i) f[i] = bfp_decode<3>((half >> (4 * i)) & 0xF, E);
  }
  int64_t off;
  int64_t r = 0, c = 0;
  if (ROWMAJOR) {
    int64_t tx = p.tile % xt, tyb = p.tile / xt;
    int64_t b = tyb / yt, ty = tyb % yt;
    r = ty * 32 + (p.face >> 1) * 16 + p.dy;
    c = tx * 32 + (p.face & 1) * 16 + p.q * 4;
    off = (b * rows + r) * cols + c;
  } else {
    off = g * 4;
  }
  if (ROWMAJOR && PADDED) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      if (r < rows && (c + i) < cols) {
        if (DST_BF16) ((uint16_t *)dst_)[off + i] = (uint16_t)(__float_as_uint(f[i]) >> 16);
        else ((float *)dst_)[off + i] = f[i];
      }
    }
  } else if (DST_BF16) {
    // exact: a decoded value has at most 7 significant bits
    u32x2 v;
    v.x = (__float_as_uint(f[0]) >> 16) | (__float_as_uint(f[1]) & 0xFFFF0000u);
    v.y = (__float_as_uint(f[2]) >> 16) | (__float_as_uint(f[3]) & 0xFFFF0000u);
    __builtin_nontemporal_store(v, (u32x2 *)((uint16_t *)dst_ + off));
  } else {
    f32x4 v = {f[0], f[1], f[2], f[3]};
    __builtin_nontemporal_store(v, (f32x4 *)((float *)dst_ + off));
  }
}

TTM_EXPORT int64_t ttm_bfp_tile_bytes(int fmt) { return fmt == TTM_BFP8B ? 1088 : (fmt == TTM_BFP4B ? 576 : -1); }

template <bool PACK>
static int run_bfp(const void *src, void *dst, int fmt, int dtype, int layout, int64_t batch, int64_t rows,
                   int64_t cols, void *stream, const char *who) {
  TTM_REQUIRE(fmt == TTM_BFP8B || fmt == TTM_BFP4B, "%s: fmt must be BFP_BFloat8 (4) or BFP_BFloat4 (6), got %d",
              who, fmt);
  TTM_REQUIRE(dtype == TTM_F32 || dtype == TTM_BF16, "%s: plain dtype must be Float32 or BFloat16, got %d", who,
              dtype);
  TTM_REQUIRE(layout == TTM_ROW_MAJOR || layout == TTM_TILE, "%s: bad layout %d", who, layout);
  TTM_REQUIRE(batch >= 0 && rows >= 0 && cols >= 0, "%s: negative dimension", who);
  if (batch == 0 || rows == 0 || cols == 0) return TTM_OK;
  TTM_REQUIRE(src && dst, "%s: null pointer", who);
  const void *plain = PACK ? src : dst;
  const void *packed = PACK ? dst : src;
  TTM_REQUIRE(((uintptr_t)plain & 15) == 0 && ((uintptr_t)packed & 15) == 0, "%s: pointers must be 16-byte aligned",
              who);
  const int64_t pr = ttm_round_up32(rows), pc = ttm_round_up32(cols);
  const int64_t yt = pr / 32, xt = pc / 32;
  const int64_t ntiles = batch * yt * xt;
  const int64_t nquads = ntiles * 256;
  const bool rm = layout == TTM_ROW_MAJOR;
  // vector access on the row-major side needs 4-element alignment of every row start
  const bool padded = rm && (rows != pr || cols != pc);
  const bool bf16 = dtype == TTM_BF16;
  TTM_REQUIRE(ntiles < (1ll << 31), "%s: tensor too large", who);
  dim3 grid((unsigned)ntiles), block(256);
  hipStream_t s = (hipStream_t)stream;
#define LAUNCH(Wv, B16, RM, PAD)                                                                              \
  do {                                                                                                        \
    if (PACK)                                                                                                 \
      hipLaunchKernelGGL((ttm_bfp_pack_k<Wv, B16, RM, PAD>), grid, block, 0, s, src, (uint8_t *)dst, nquads,   \
                         rows, cols, yt, xt);                                                                 \
    else                                                                                                      \
      hipLaunchKernelGGL((ttm_bfp_unpack_k<Wv, B16, RM, PAD>), grid, block, 0, s, (const uint8_t *)src, dst,   \
                         nquads, rows, cols, yt, xt);                                                         \
  } while (0)
#define PICK_PAD(Wv, B16, RM)            \
  do {                                   \
    if (padded) LAUNCH(Wv, B16, RM, true); \
    else LAUNCH(Wv, B16, RM, false);     \
  } while (0)
#define PICK_RM(Wv, B16)                 \
  do {                                   \
    if (rm) PICK_PAD(Wv, B16, true);     \
    else LAUNCH(Wv, B16, false, false);  \
  } while (0)
#define PICK_B16(Wv)                     \
  do {                                   \
    if (bf16) PICK_RM(Wv, true);         \
    else PICK_RM(Wv, false);             \
  } while (0)
  if (fmt == TTM_BFP8B) PICK_B16(7);
  else PICK_B16(3);
#undef PICK_B16
#undef PICK_RM
#undef PICK_PAD
#undef LAUNCH
  TTM_LAUNCH_CHECK();
  return TTM_OK;
}

TTM_EXPORT int ttm_bfp_pack(const void *src, int src_dtype, int src_layout, void *dst, int fmt, int64_t batch,
                            int64_t rows, int64_t cols, void *stream) {
  return run_bfp<true>(src, dst, fmt, src_dtype, src_layout, batch, rows, cols, stream, "ttm_bfp_pack");
}

TTM_EXPORT int ttm_bfp_unpack(const void *src, int fmt, void *dst, int dst_dtype, int dst_layout, int64_t batch,
                              int64_t rows, int64_t cols, void *stream) {
  return run_bfp<false>(src, dst, fmt, dst_dtype, dst_layout, batch, rows, cols, stream, "ttm_bfp_unpack");
}
