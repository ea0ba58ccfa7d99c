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
// LDS image (both operands): [row][8 chunks of 8 k] with chunk index XOR (row & 7); a fragment
// read is one ds_read_b128 per lane and is bank-conflict free.
//
// Weight dequantisation (bfp8_b).  A lane owns an 8(k) x 8(n) block: eight 8-byte row loads plus the
// eight row exponents.  Sign-magnitude bytes are turned into offset-binary bytes with packed
// integer ops (t = 128 +- mag), so an element is cvt_f32_ubyte + one fma:
//     w = t * 2^(E-133) - 128 * 2^(E-133)          (exact)
// and pairs along k are packed to bf16 by taking the high halves (exact: 7 significant bits).
// Rows whose shared exponent is below 7 (|w| < 2^-120) are flushed towards zero.
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
};

__device__ __forceinline__ float apply_act(int act, float x) {
  switch (act) {
  case TTM_ACT_GELU: return ttm_gelu_fast(x);
  case TTM_ACT_SILU: return ttm_silu(x);
  case TTM_ACT_SIGMOID: return ttm_sigmoid(x);
  case TTM_ACT_RELU: return x > 0.0f ? x : 0.0f;
  default: return x;
  }
}

__device__ __forceinline__ int lds_chunk(int row, int kc) { return row * 8 + (kc ^ (row & 7)); }

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

  // epilogue: bias, activation, bf16, 8-byte stores into the output face rows
  const int m_in = lane & 31;
#pragma unroll
  for (int a = 0; a < 4; ++a) {
    const int nt = nt0 + wn * 4 + a;
    if (nt >= p.Nt) continue;
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
      for (int b = 0; b < 4; ++b) {
        const int mt = mt0 + wm * 4 + b;
        if (mt >= p.Mt) continue;
        uint32_t h[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) h[r] = ttm_f32_to_bf16(apply_act(p.act, acc[a][b][g * 4 + r] + bv[r]));
        u32x2 o = {h[0] | (h[1] << 16), h[2] | (h[3] << 16)};
        int64_t off = ((int64_t)mt * p.Nt + nt) * 1024 + ((m_in >> 4) * 2 + (n_in >> 4)) * 256 + (m_in & 15) * 16 +
                      (n_in & 15);
        *(u32x2 *)(C + off * 2) = o;
      }
    }
  }
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
      for (int i = 0; i < 8; ++i) rows[i] = ok ? __builtin_nontemporal_load((const u32x2 *)(m + i * 16)) : u32x2{0, 0};
      dequant_bfp8_block(rows, exps, out);
    } else if constexpr (WF == WF_BFP4) {
      const uint8_t *t = W + tile * 576;
      u32x2 exps = ok ? *(const u32x2 *)(t + face * 16 + khalf * 8) : u32x2{0, 0};
      const uint8_t *m = t + 64 + face * 128 + khalf * 64 + oct * 4;
      uint32_t rows[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) rows[i] = ok ? __builtin_nontemporal_load((const uint32_t *)(m + i * 8)) : 0u;
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
    uint32_t h[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) h[r] = ttm_f32_to_bf16(apply_act(p.act, acc[g * 4 + r] + bv[r]));
    u32x2 o = {h[0] | (h[1] << 16), h[2] | (h[3] << 16)};
    int64_t off = (int64_t)nt * 1024 + ((m_in >> 4) * 2 + (n_in >> 4)) * 256 + (m_in & 15) * 16 + (n_in & 15);
    *(u32x2 *)(C + off * 2) = o;
  }
}

template <int WF>
static int launch_linear(const LinearArgs &a, int64_t batch, hipStream_t s) {
  if (a.Mt == 1 || a.Mt * 32 <= ttm_option("linear_small_m_max")) {
    // the small kernel handles one row tile per launch row: loop row tiles through grid.y
    LinearArgs p = a;
    for (int mt = 0; mt < a.Mt; ++mt) {
      p.A = a.A + (int64_t)mt * a.Kt * 2048;
      p.C = a.C + (int64_t)mt * a.Nt * 2048;
      hipLaunchKernelGGL((ttm_linear_small_k<WF>), dim3(a.Nt, 1, (unsigned)batch), dim3(256), 0, s, p);
    }
    return 0;
  }
  static bool attr_set = false;
  const int lds_bytes = 2 * 4096 * 16;
  if (!attr_set) {
    hipError_t e = hipFuncSetAttribute((const void *)ttm_linear_big_k<WF>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                       lds_bytes);
    if (e != hipSuccess) return ttm_set_error(TTM_ERR_HIP, "hipFuncSetAttribute(LDS %d): %s", lds_bytes, hipGetErrorString(e));
    attr_set = true;
  }
  hipLaunchKernelGGL((ttm_linear_big_k<WF>), dim3(a.m_blocks * a.n_blocks, 1, (unsigned)batch), dim3(256), lds_bytes, s, a);
  return 0;
}

TTM_EXPORT int ttm_linear(const void *a, int a_dtype, const void *w, int w_dtype, int transpose_w, const void *bias,
                          int bias_dtype, int bias_layout, void *out, int out_dtype, int64_t batch,
                          int64_t w_batch, int64_t M, int64_t N, int64_t K, int act, void *stream) {
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
