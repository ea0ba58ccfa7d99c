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
// Work split: a lane owns one 16-byte chunk of the plain side (4 fp32 or 8 bf16 elements of one
// face row), so a face row is a quad (fp32) or a pair (bf16) of adjacent lanes and the shared
// exponent is a max-reduction with DPP quad_perm moves.  A 256-lane workgroup owns 1024 chunks:
// on a row-major plain side that is a strip of 32 rows x 512 bytes which is read / written in
// fully contiguous 512-byte row segments and permuted through a padded LDS image, exactly like
// the tilize kernel; the packed side of a strip is one contiguous run of tiles.
// Shapes whose rows are not a multiple of 512 bytes, or that need zero padding, take a generic
// kernel with one face row quad per lane group and bounds-checked scalar accesses.
#include "ttm_common.h"

// ------------------------------------------------------------------------------------ element math
// W = magnitude bits (7 or 3).  Returns the magnitude only; signs are merged per chunk.
template <int W>
__device__ __forceinline__ uint32_t bfp_mag(uint32_t bits, uint32_t E) {
  constexpr int DROP = 24 - W;
  uint32_t a = bits & 0x7FFFFFFFu;
  uint32_t e = a >> 23;
  uint32_t shift = min(E - e, 31u);
  uint32_t m = (a & 0x7FFFFFu) | (min(a, 1u) << 23);  // hidden bit unless the value is +-0
  m >>= shift;
  m += ((1u << (DROP - 1)) - 1) + ((m >> DROP) & 1u);  // round to nearest, ties to even
  return min(m >> DROP, (1u << W) - 1);
}

template <int W>
__device__ __forceinline__ uint32_t bfp_encode(uint32_t bits, uint32_t E) {
  uint32_t k = bfp_mag<W>(bits, E);
  return k ? (k | ((bits >> 31) << W)) : 0u;
}

template <int W>
__device__ __forceinline__ float bfp_decode(uint32_t mag, uint32_t signbit_at31, int E) {
  // mag * 2^(E - 127 - (W-1)), exact (subnormal results included); the sign is dropped at 0
  float v = ldexpf((float)mag, E - 127 - (W - 1));
  return mag ? __uint_as_float(__float_as_uint(v) | (signbit_at31 & 0x80000000u)) : 0.0f;
}

template <int LANES>
__device__ __forceinline__ uint32_t group_max(uint32_t v) {
  uint32_t o = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0xB1, 0xF, 0xF, true);  // quad_perm [1,0,3,2]
  v = max(v, o);
  if (LANES == 4) {
    o = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x4E, 0xF, 0xF, true);  // quad_perm [2,3,0,1]
    v = max(v, o);
  }
  return v;
}

// Encode one chunk of EPT elements (bit patterns of fp32 values) of a face row.
// out[] receives EPT*(W+1)/32 packed words (bfp8: EPT/4 words, bfp4: EPT/8 words, or a half word).
template <int W, int EPT>
__device__ __forceinline__ uint32_t encode_chunk(const uint32_t (&bits)[EPT], uint32_t (&out)[2]) {
  uint32_t E = 0;
#pragma unroll
  for (int i = 0; i < EPT; ++i) E = max(E, (bits[i] >> 23) & 0xFFu);
  E = group_max<16 / EPT>(E);
  out[0] = out[1] = 0;
  if (W == 7) {
#pragma unroll
    for (int w = 0; w < EPT / 4; ++w) {
      uint32_t k0 = bfp_mag<7>(bits[4 * w + 0], E), k1 = bfp_mag<7>(bits[4 * w + 1], E);
      uint32_t k2 = bfp_mag<7>(bits[4 * w + 2], E), k3 = bfp_mag<7>(bits[4 * w + 3], E);
      uint32_t mags = k0 | (k1 << 8) | (k2 << 16) | (k3 << 24);
      uint32_t nz = (mags + 0x7F7F7F7Fu) & 0x80808080u;  // 0x80 in every byte whose magnitude is non-zero
      uint32_t top = __builtin_amdgcn_perm(bits[4 * w + 1], bits[4 * w + 0], 0x0C0C0703u) |
                     __builtin_amdgcn_perm(bits[4 * w + 3], bits[4 * w + 2], 0x07030C0Cu);  // the four sign bytes
      out[w] = mags | (top & nz);
    }
  } else {
    uint32_t word = 0;
#pragma unroll
    for (int i = 0; i < EPT; ++i) word |= bfp_encode<3>(bits[i], E) << (4 * i);
    out[0] = word;
  }
  return E;
}

template <bool BF16, int EPT>
__device__ __forceinline__ void chunk_to_bits(const u32x4 &v, uint32_t (&bits)[EPT]) {
  if (BF16) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      bits[2 * i] = v[i] << 16;
      bits[2 * i + 1] = v[i] & 0xFFFF0000u;
    }
  } else {
#pragma unroll
    for (int i = 0; i < 4; ++i) bits[i] = v[i];
  }
}

// Decode EPT elements from packed words into one 16-byte chunk of the plain side.
template <int W, bool BF16, int EPT>
__device__ __forceinline__ u32x4 decode_chunk(const uint32_t (&in)[2], int E) {
  float f[EPT];
  if (W == 7) {
#pragma unroll
    for (int i = 0; i < EPT; ++i) {
      uint32_t word = in[i / 4];
      int b = i & 3;
      f[i] = bfp_decode<7>((word >> (8 * b)) & 0x7Fu, word << (24 - 8 * b), E);
    }
  } else {
#pragma unroll
    for (int i = 0; i < EPT; ++i) f[i] = bfp_decode<3>((in[0] >> (4 * i)) & 0x7u, in[0] << (28 - 4 * i), E);
  }
  u32x4 v;
  if (BF16) {  // exact: a decoded value has at most 7 significant bits
#pragma unroll
    for (int i = 0; i < 4; ++i) v[i] = (__float_as_uint(f[2 * i]) >> 16) | (__float_as_uint(f[2 * i + 1]) & 0xFFFF0000u);
  } else {
#pragma unroll
    for (int i = 0; i < 4; ++i) v[i] = __float_as_uint(f[i]);
  }
  return v;
}

// ------------------------------------------------------------------------------------ strip kernels
// ELEM = bytes per plain element (4: fp32, 2: bf16).  A tile is CPT = 64*ELEM chunks; a face row is
// ELEM chunks.  The workgroup handles 1024 chunks = 16/ELEM tiles.
// Packing bfp8_b from row-major fp32 gains from four workgroups per CU (8192 x 8192: 53.2 -> 50.9 us); every other
// combination is fastest without a cap.
template <int W, int ELEM, bool ROWMAJOR, bool PACK>
__global__ __launch_bounds__(256) TTM_MAX_WAVES((PACK && ROWMAJOR && W == 7 && ELEM == 4) ? 4 : 8) void ttm_bfp_strip_k(const void *__restrict__ src_, void *__restrict__ dst_,
                                                       int64_t xt, int64_t strips_per_row) {
  constexpr int EPT = 16 / ELEM;
  constexpr int CPT = 64 * ELEM;
  constexpr int TILE_BYTES = 64 + (W == 7 ? 1024 : 512);
  constexpr int CHUNK_OUT = EPT * (W + 1) / 8;  // packed bytes per chunk: 4, 8 (bfp8) or 2, 4 (bfp4)
  constexpr int PITCH = 33;
  __shared__ u32x4 lds[ROWMAJOR ? 32 * PITCH : 1];
  // PACK to bfp4_b: the workgroup's 16 / ELEM packed tiles are contiguous in the output; they are assembled here (exponent
  // bytes and 2- or 4-byte mantissa pieces per lane) and leave as 16-byte stores (8192 x 8192 fp32: 51 -> 46 us; bfp8_b with
  // its 4- and 8-byte pieces is faster storing them directly: 53 against 55 us)
  constexpr int PK_BYTES = (16 / ELEM) * TILE_BYTES;
  constexpr bool VIA_LDS = PACK && W == 3;
  __shared__ __attribute__((aligned(16))) uint8_t pk[VIA_LDS ? PK_BYTES : 16];
  const int tid = threadIdx.x;
  const int64_t strip = blockIdx.x;
  const int64_t tyb = ROWMAJOR ? strip / strips_per_row : 0;
  const int64_t sx = ROWMAJOR ? strip % strips_per_row : 0;
  const int64_t row_chunks = xt * 2 * ELEM;
  // first tile of this workgroup on the packed / tile-ordered side
  const int64_t tile0 = ROWMAJOR ? (tyb * xt + sx * (16 / ELEM)) : strip * (16 / ELEM);
  const u32x4 *plain_in = (const u32x4 *)src_;
  u32x4 *plain_out = (u32x4 *)dst_;
  const uint8_t *packed_in = (const uint8_t *)src_;
  uint8_t *packed_out = (uint8_t *)dst_;
  const int64_t rm_base = tyb * 32 * row_chunks + sx * 32;

  u32x4 v[4];
  if (PACK) {
    if (ROWMAJOR) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        int r = i * 8 + (tid >> 5), j = tid & 31;
        v[i] = __builtin_nontemporal_load(&plain_in[rm_base + r * row_chunks + j]);
      }
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        int r = i * 8 + (tid >> 5), j = tid & 31;
        lds[r * PITCH + j] = v[i];
      }
      __syncthreads();
    } else {
#pragma unroll
      for (int i = 0; i < 4; ++i) v[i] = __builtin_nontemporal_load(&plain_in[tile0 * CPT + i * 256 + tid]);
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      int oc = i * 256 + tid;
      int tl = oc / CPT, w = oc % CPT;
      int face = w / (16 * ELEM), dy = (w / ELEM) % 16, q = w % ELEM;
      if (ROWMAJOR) {
        int r = (face >> 1) * 16 + dy, j = tl * 2 * ELEM + (face & 1) * ELEM + q;
        v[i] = lds[r * PITCH + j];
      }
      uint32_t bits[EPT], out[2];
      chunk_to_bits<ELEM == 2, EPT>(v[i], bits);
      uint32_t E = encode_chunk<W, EPT>(bits, out);
      if constexpr (VIA_LDS) {
        uint8_t *tile = pk + tl * TILE_BYTES;
        if (q == 0) tile[face * 16 + dy] = (uint8_t)E;
        uint8_t *m = tile + 64 + w * CHUNK_OUT;
        if (CHUNK_OUT == 4) *(uint32_t *)m = out[0];
        else *(uint16_t *)m = (uint16_t)out[0];
      } else {
        uint8_t *tile = packed_out + (tile0 + tl) * TILE_BYTES;
        if (q == 0) tile[face * 16 + dy] = (uint8_t)E;
        uint8_t *m = tile + 64 + w * CHUNK_OUT;
        if (CHUNK_OUT == 8) {
          u32x2 o = {out[0], out[1]};
          __builtin_nontemporal_store(o, (u32x2 *)m);
        } else {
          __builtin_nontemporal_store(out[0], (uint32_t *)m);
        }
      }
    }
    if constexpr (VIA_LDS) {
      __syncthreads();
      u32x4 *dst16 = (u32x4 *)(packed_out + tile0 * TILE_BYTES);   // tile sizes are multiples of 16 bytes
      for (int c = tid; c < PK_BYTES / 16; c += 256) __builtin_nontemporal_store(((const u32x4 *)pk)[c], &dst16[c]);
    }
  } else {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      int oc = i * 256 + tid;
      int tl = oc / CPT, w = oc % CPT;
      int face = w / (16 * ELEM), dy = (w / ELEM) % 16;
      const uint8_t *tile = packed_in + (tile0 + tl) * TILE_BYTES;
      int E = tile[face * 16 + dy];
      const uint8_t *m = tile + 64 + w * CHUNK_OUT;
      uint32_t in[2] = {0, 0};
      if (CHUNK_OUT == 8) {
        u32x2 t = __builtin_nontemporal_load((const u32x2 *)m);
        in[0] = t.x; in[1] = t.y;
      } else if (CHUNK_OUT == 4) {
        in[0] = __builtin_nontemporal_load((const uint32_t *)m);
      } else {
        in[0] = __builtin_nontemporal_load((const uint16_t *)m);
      }
      v[i] = decode_chunk<W, ELEM == 2, EPT>(in, E);
    }
    if (ROWMAJOR) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        int oc = i * 256 + tid;
        int tl = oc / CPT, w = oc % CPT;
        int face = w / (16 * ELEM), dy = (w / ELEM) % 16, q = w % ELEM;
        int r = (face >> 1) * 16 + dy, j = tl * 2 * ELEM + (face & 1) * ELEM + q;
        lds[r * PITCH + j] = v[i];
      }
      __syncthreads();
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        int r = i * 8 + (tid >> 5), j = tid & 31;
        __builtin_nontemporal_store(lds[r * PITCH + j], &plain_out[rm_base + r * row_chunks + j]);
      }
    } else {
#pragma unroll
      for (int i = 0; i < 4; ++i) __builtin_nontemporal_store(v[i], &plain_out[tile0 * CPT + i * 256 + tid]);
    }
  }
}

// ------------------------------------------------------------------------------------ generic kernels
// One lane per 4 elements of a face row; grid = (tile columns, tile rows, batch).
template <int W, bool BF16, bool PACK>
__global__ __launch_bounds__(256) void ttm_bfp_generic_k(const void *__restrict__ src_, void *__restrict__ dst_,
                                                         int64_t rows, int64_t cols, int rowmajor) {
  constexpr int TILE_BYTES = 64 + (W == 7 ? 1024 : 512);
  const int64_t xt = gridDim.x, yt = gridDim.y;
  const int64_t tx = blockIdx.x, ty = blockIdx.y, b = blockIdx.z;
  const int64_t tile_idx = (b * yt + ty) * xt + tx;
  const int w = threadIdx.x;
  const int face = w >> 6, dy = (w >> 2) & 15, q = w & 3;
  const int64_t r = ty * 32 + (face >> 1) * 16 + dy;
  const int64_t c = tx * 32 + (face & 1) * 16 + q * 4;
  const int64_t off = rowmajor ? (b * rows + r) * cols + c : tile_idx * 1024 + w * 4;
  uint8_t *tile = (uint8_t *)(PACK ? dst_ : const_cast<void *>(src_)) + tile_idx * TILE_BYTES;
  if (PACK) {
    uint32_t bits[4], out[2];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      bool in = !rowmajor || (r < rows && (c + i) < cols);
      if (BF16) bits[i] = in ? ((uint32_t)((const uint16_t *)src_)[off + i] << 16) : 0u;
      else bits[i] = in ? ((const uint32_t *)src_)[off + i] : 0u;
    }
    uint32_t E = encode_chunk<W, 4>(bits, out);
    if (q == 0) tile[face * 16 + dy] = (uint8_t)E;
    if (W == 7) ((uint32_t *)(tile + 64))[w] = out[0];
    else ((uint16_t *)(tile + 64))[w] = (uint16_t)out[0];
  } else {
    int E = tile[face * 16 + dy];
    uint32_t in[2] = {0, 0};
    if (W == 7) in[0] = ((const uint32_t *)(tile + 64))[w];
    else in[0] = ((const uint16_t *)(tile + 64))[w];
    u32x4 v = decode_chunk<W, false, 4>(in, E);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      bool inb = !rowmajor || (r < rows && (c + i) < cols);
      if (inb) {
        if (BF16) ((uint16_t *)dst_)[off + i] = (uint16_t)(v[i] >> 16);
        else ((uint32_t *)dst_)[off + i] = v[i];
      }
    }
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
  const int64_t pr = ttm_round_up32(rows), pc = ttm_round_up32(cols);
  const int64_t yt = pr / 32, xt = pc / 32;
  const int64_t ntiles = batch * yt * xt;
  const bool rm = layout == TTM_ROW_MAJOR;
  const bool bf16 = dtype == TTM_BF16;
  const int elem = bf16 ? 2 : 4;
  const bool aligned = ((uintptr_t)src & 15) == 0 && ((uintptr_t)dst & 15) == 0;
  const bool padded = rm && (rows != pr || cols != pc);
  hipStream_t s = (hipStream_t)stream;
  const int tiles_per_wg = 16 / elem;
  bool strip = aligned && !padded && ttm_option(PACK ? "pack_variant" : "unpack_variant") == 0;
  int64_t strips_per_row = 0, blocks = 0;
  if (strip) {
    if (rm) {
      strip = (cols * elem) % 512 == 0;
      strips_per_row = cols * elem / 512;
      blocks = batch * yt * strips_per_row;
    } else {
      strip = ntiles % tiles_per_wg == 0;
      blocks = ntiles / tiles_per_wg;
    }
  }
  if (strip) {
    TTM_REQUIRE(blocks < (1ll << 31), "%s: tensor too large", who);
    dim3 grid((unsigned)blocks), block(256);
#define STRIP(Wv, EL, RM) \
  hipLaunchKernelGGL((ttm_bfp_strip_k<Wv, EL, RM, PACK>), grid, block, 0, s, src, dst, xt, strips_per_row)
#define STRIP_RM(Wv, EL)        \
  do {                          \
    if (rm) STRIP(Wv, EL, true); \
    else STRIP(Wv, EL, false);  \
  } while (0)
    if (fmt == TTM_BFP8B) { if (bf16) STRIP_RM(7, 2); else STRIP_RM(7, 4); }
    else { if (bf16) STRIP_RM(3, 2); else STRIP_RM(3, 4); }
#undef STRIP_RM
#undef STRIP
  } else {
    TTM_REQUIRE(yt <= 65535 && batch <= 65535, "%s: more than 65535 tile rows or batches on the generic path", who);
    TTM_REQUIRE(((uintptr_t)(PACK ? dst : src) & 3) == 0, "%s: packed buffer must be 4-byte aligned", who);
    dim3 grid((unsigned)xt, (unsigned)yt, (unsigned)batch), block(256);
#define GEN(Wv, B16) \
  hipLaunchKernelGGL((ttm_bfp_generic_k<Wv, B16, PACK>), grid, block, 0, s, src, dst, rows, cols, (int)rm)
    if (fmt == TTM_BFP8B) { if (bf16) GEN(7, true); else GEN(7, false); }
    else { if (bf16) GEN(3, true); else GEN(3, false); }
#undef GEN
  }
  TTM_LAUNCH_CHECK();
  return TTM_OK;
}

TTM_EXPORT int ttm_bfp_pack(const void *src, int src_dtype, int src_layout, void *dst, int fmt, int64_t batch,
                            int64_t rows, int64_t cols, void *stream) {
  TTM_EXTENTS(bfp_pack, src, src_dtype, src_layout, dst, fmt, batch, rows, cols);
  return run_bfp<true>(src, dst, fmt, src_dtype, src_layout, batch, rows, cols, stream, "ttm_bfp_pack");
}

TTM_EXPORT int ttm_bfp_unpack(const void *src, int fmt, void *dst, int dst_dtype, int dst_layout, int64_t batch,
                              int64_t rows, int64_t cols, void *stream) {
  TTM_EXTENTS(bfp_unpack, src, fmt, dst, dst_dtype, dst_layout, batch, rows, cols);
  return run_bfp<false>(src, dst, fmt, dst_dtype, dst_layout, batch, rows, cols, stream, "ttm_bfp_unpack");
}
