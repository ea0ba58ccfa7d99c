// Fused scaled-dot-product attention (prefill): softmax(Q K^T * scale + mask) V with grouped-query
// heads, causal masking, fp32 online softmax, bf16 MFMA.  Q [B,Hq,Sq,D], K/V [B,Hkv,Sk,D], mask
// (optional, additive) [B,1|Hq,Sq,Sk], out [B,Hq,Sq,D]; all bf16 in tile order.
//
// Everything is computed transposed so that no accumulator ever has to be shuffled between lanes:
//   S^T[key][q] = K . Q^T     (MFMA A = K rows, 8 consecutive d per lane straight from the tiled K;
//                              MFMA B = Q, kept in registers for the whole key loop)
//   O^T[d][q]   = V^T . P^T   (MFMA B = P^T taken directly from the S^T accumulator registers: a lane
//                              holds q = lane % 32 and keys 8g + 4h + {0..3}; the k-slot order this
//                              implies is matched on the V^T side)
// A lane therefore owns one query column of every accumulator: the running max / sum and the
// rescale factor are per-lane scalars, shared only with lane ^ 32.
// Workgroup = 4 wavefronts x 32 queries; K and V^T blocks of 32 keys are staged in LDS.
#include "ttm_common.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef __bf16 sdpa_bf16x2 __attribute__((ext_vector_type(2)));

struct SdpaArgs {
  const uint8_t *q, *k, *v, *mask;
  uint8_t *out;
  int B, Hq, Hkv, Sq, Sk;
  int sqt, skt;      // tiles along the sequence dims
  int mask_heads;    // 1 or Hq
  int mask_b;        // 1: one mask per batch entry, 0: one mask shared by all
  // query i sees key j when i - lo_off <= j <= i + hi_off.  Causal: hi_off = 0; a sliding window of w keys: lo_off = w - 1
  // under a causal pass, lo_off = hi_off = w / 2 otherwise; kNoLimit where a side is open.
  int hi_off, lo_off;
  const uint8_t *sink;   // [1, Hq, 1, 1] in tiles (one tile per head, value at its first element), or null
  float scale;
  // Where a row of tiles of one head lives, per operand, in bytes: matrix (b, h) starts at b * batch + h * head, its tile
  // row t at + t * pitch (the D / 32 tiles of a tile row are contiguous).  [B, H, S, D]: pitch = D / 32 tiles, head =
  // S / 32 * pitch, batch = H * head.  [B, S, H * D] (heads side by side, as a projection leaves them): pitch = H * D / 32
  // tiles, head = D / 32 tiles, batch = S / 32 * pitch.  Same 32 x 32 tiles either way.
  int64_t q_pitch, q_head, q_batch, k_pitch, k_head, k_batch, v_pitch, v_head, v_batch, o_pitch, o_head, o_batch;
  // Few query blocks against many keys (a chunk of a long prefill, cross attention): the keys of a query block are divided
  // among ksplits workgroups, which leave their running maximum, sum and unnormalised output per query tile here, in the
  // order (split, b, h, query tile); ttm_sdpa_combine_k merges them.  ksplits = 1: the workgroup writes the output itself.
  int ksplits;
  float *part_o;    // [slots][D / 32][1024] fp32, elements of a tile in tile order
  float *part_ml;   // [slots][32][2]: running maximum (log2 domain) and sum of each query of the tile
};

constexpr int kNoLimit = 1 << 29;

// first and one-past-last 32-key tile that the queries [q_first, q_last] can see
__device__ __forceinline__ int first_key_tile(const SdpaArgs &p, int q_first) {
  const int lo = q_first - p.lo_off;
  return lo > 0 ? lo >> 5 : 0;
}
__device__ __forceinline__ int end_key_tile(const SdpaArgs &p, int q_last) {
  return min(p.skt, ((q_last + p.hi_off) >> 5) + 1);
}
// the attention sink is one more logit per head with a zero value row: it enters the running maximum and the running
// sum before the first key does, and the online softmax carries it from there
__device__ __forceinline__ void sink_start(const SdpaArgs &p, int h, float scale2, float &m_run, float &l_run) {
  if (p.sink) {
    m_run = __uint_as_float((uint32_t)(*(const uint16_t *)(p.sink + (int64_t)h * 2048)) << 16) * scale2;
    l_run = 1.0f;
  }
}

__device__ __forceinline__ uint32_t pack_bf16_rne(float a, float b) {
  return ttm_pack_bf16x2(a, b);
}

// Workgroups go to the eight XCDs in turn, in the order of their flat index, and every XCD has an L2 of its own.  The
// workgroups that read one K / V matrix (the query blocks of the query heads of one kv head) are therefore given flat
// indices that are equal modulo 8: an XCD's L2 then holds the K and V of a few kv heads, each read by all its users,
// instead of every XCD streaming all of them.  x, h, b come in as blockIdx and go out as the block, head and batch entry
// this workgroup serves (a permutation of the grid; the identity when the matrices do not divide among eight XCDs).
__device__ __forceinline__ void sdpa_xcd_order(const SdpaArgs &p, int &x, int &h, int &b) {
  if ((p.B * p.Hkv) % 8 != 0) return;
  const int flat = x + (int)gridDim.x * (h + p.Hq * b), gq = p.Hq / p.Hkv, users = (int)gridDim.x * gq;
  const int xcd = flat % 8, idx = flat / 8;
  const int group = (idx / users) * 8 + xcd, member = idx % users;   // group: (batch entry, kv head)
  b = group / p.Hkv;
  h = (group % p.Hkv) * gq + member % gq;
  x = member / gq;
}

template <int DT>  // head_dim / 32
__global__ __launch_bounds__(256) void ttm_sdpa_k(SdpaArgs p) {
  constexpr int D = DT * 32;
  constexpr int VPITCH = 40;                           // V^T row pitch in bf16 (32 keys + pad)
  __shared__ __attribute__((aligned(16))) uint8_t ldsK[32 * D * 2];
  __shared__ __attribute__((aligned(16))) uint16_t ldsV[D * VPITCH];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int qb = blockIdx.x, h = blockIdx.y, b = blockIdx.z;
  const int hk = h / (p.Hq / p.Hkv);
  const int qt = qb * 4 + wave;                         // this wave's query tile
  const bool wave_ok = qt < p.sqt;
  const int l31 = lane & 31, hh = lane >> 5;
  const int64_t q_mat = b * p.q_batch + h * p.q_head, o_mat = b * p.o_batch + h * p.o_head;
  const int64_t k_mat = b * p.k_batch + hk * p.k_head, v_mat = b * p.v_batch + hk * p.v_head;

  // Q fragments: B operand, lane (q = l31, hh): d = 16 s + 8 hh .. +7
  bf16x8 qf[2 * DT];
#pragma unroll
  for (int s = 0; s < 2 * DT; ++s) {
    u32x4 v = {0, 0, 0, 0};
    if (wave_ok)
      v = *(const u32x4 *)(p.q + q_mat + qt * p.q_pitch + (s >> 1) * 2048 + ((l31 >> 4) * 2 + (s & 1)) * 512 +
                           (l31 & 15) * 32 + hh * 16);
    qf[s] = *(bf16x8 *)&v;
  }
  f32x16 o[DT];
#pragma unroll
  for (int d = 0; d < DT; ++d)
#pragma unroll
    for (int r = 0; r < 16; ++r) o[d][r] = 0.0f;
  float m_run = -INFINITY, l_run = 0.0f;
  const int q_glob = qt * 32 + l31;
  constexpr float LOG2E = 1.4426950408889634f;
  const float scale2 = p.scale * LOG2E;
  sink_start(p, h, scale2, m_run, l_run);

  // key tiles any wave of this workgroup needs
  const int kt_begin = first_key_tile(p, qb * 128), kt_end = end_key_tile(p, min(qb * 4 + 4, p.sqt) * 32 - 1);
  // K and V blocks travel global -> registers -> LDS; the loads of block kt + 1 are issued before block kt is
  // computed, so their latency hides behind the MFMA and softmax work
  constexpr int NC = (DT * 128 + 255) / 256;   // 16-byte chunks of a K (or V) block per lane
  u32x4 kreg[NC], vreg[NC];
  auto load_block = [&](int kt) {
    const u32x4 *ks = (const u32x4 *)(p.k + k_mat + kt * p.k_pitch);
    const u32x4 *vs = (const u32x4 *)(p.v + v_mat + kt * p.v_pitch);
#pragma unroll
    for (int i = 0; i < NC; ++i) {
      if (tid + 256 * i < DT * 128) {
        kreg[i] = ks[tid + 256 * i];
        vreg[i] = vs[tid + 256 * i];
      }
    }
  };
  if (kt_end > kt_begin) load_block(kt_begin);
  for (int kt = kt_begin; kt < kt_end; ++kt) {
    __syncthreads();  // previous block fully consumed
#pragma unroll
    for (int i = 0; i < NC; ++i) {
      const int c = tid + 256 * i;
      if (c >= DT * 128) break;
      // K block: DT tiles, contiguous (32 * D * 2 bytes); copied as is
      ((u32x4 *)ldsK)[c] = kreg[i];
      // V block -> V^T[d][key]
      const u32x4 v = vreg[i];
      const int tile = c >> 7, cc = c & 127;
      const int face = cc >> 5, row = (cc & 31) >> 1, half = cc & 1;
      const int key = (face >> 1) * 16 + row;
      const int d0 = tile * 32 + (face & 1) * 16 + half * 8;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        ldsV[(d0 + 2 * e) * VPITCH + key] = (uint16_t)(v[e] & 0xFFFF);
        ldsV[(d0 + 2 * e + 1) * VPITCH + key] = (uint16_t)(v[e] >> 16);
      }
    }
    __syncthreads();
    if (kt + 1 < kt_end) load_block(kt + 1);
    const bool skip = !wave_ok || kt * 32 > qt * 32 + 31 + p.hi_off || kt * 32 + 31 < qt * 32 - p.lo_off;
    if (skip) continue;

    // S^T = K . Q^T for 32 keys x 32 queries
    f32x16 s;
#pragma unroll
    for (int r = 0; r < 16; ++r) s[r] = 0.0f;
#pragma unroll
    for (int st = 0; st < 2 * DT; ++st) {
      u32x4 kv = *(const u32x4 *)(ldsK + (st >> 1) * 2048 + ((l31 >> 4) * 2 + (st & 1)) * 512 + (l31 & 15) * 32 + hh * 16);
      s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(*(bf16x8 *)&kv, qf[st], s, 0, 0, 0);
    }
    // scale, mask; lane holds q = q_glob, keys kt*32 + 8g + 4hh + r.  Scores are kept in the log2 domain
    // (scale and mask multiplied by log2 e) so that the exponential is a bare v_exp_f32.
    // masking by position is only needed where a block crosses a limit of the visible range and on a ragged last block
    const bool edge = kt * 32 + 31 > qt * 32 + p.hi_off || kt * 32 < qt * 32 + 31 - p.lo_off || kt * 32 + 32 > p.Sk;   // wavefront-uniform
    float mx = -INFINITY;
    if (p.mask || edge) {
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int key0 = kt * 32 + g * 8 + hh * 4;
        float mk[4] = {0.f, 0.f, 0.f, 0.f};
        if (p.mask) {
          const int64_t mm = ((int64_t)b * p.mask_b * p.mask_heads + (p.mask_heads == 1 ? 0 : h)) * p.sqt * p.skt * 2048;
          const int kin = g * 8 + hh * 4;
          const uint8_t *mp = p.mask + mm + ((int64_t)qt * p.skt + kt) * 2048 +
                              (((l31 >> 4) * 2 + (kin >> 4)) * 256 + (l31 & 15) * 16 + (kin & 15)) * 2;
          u32x2 raw = *(const u32x2 *)mp;
          mk[0] = __uint_as_float(raw.x << 16); mk[1] = __uint_as_float(raw.x & 0xFFFF0000u);
          mk[2] = __uint_as_float(raw.y << 16); mk[3] = __uint_as_float(raw.y & 0xFFFF0000u);
        }
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          float v = fmaf(s[g * 4 + r], scale2, mk[r] * LOG2E);
          const int key = key0 + r;
          if (key >= p.Sk || key > q_glob + p.hi_off || key < q_glob - p.lo_off) v = -INFINITY;
          s[g * 4 + r] = v;
          mx = fmaxf(mx, v);
        }
      }
    } else {
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        s[r] *= scale2;
        mx = fmaxf(mx, s[r]);
      }
    }
    mx = fmaxf(mx, __shfl_xor(mx, 32));
    const float m_new = fmaxf(m_run, mx);
    // fully masked so far: keep everything at zero without producing NaN
    const float m_use = m_new == -INFINITY ? 0.0f : m_new;
    const float alpha = __builtin_amdgcn_exp2f(m_run - m_use);
    float rs = 0.0f;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      float e = __builtin_amdgcn_exp2f(s[r] - m_use);
      s[r] = e;
      rs += e;
    }
    rs += __shfl_xor(rs, 32);
    l_run = l_run * alpha + rs;
    m_run = m_new;
    // the running maximum seldom moves after the first blocks: rescale only when some lane needs it
    if (__builtin_amdgcn_ballot_w64(alpha != 1.0f) != 0) {
#pragma unroll
      for (int d = 0; d < DT; ++d)
#pragma unroll
        for (int r = 0; r < 16; ++r) o[d][r] *= alpha;
    }
    // O^T += V^T . P^T, two k16 steps
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      u32x4 pb;
      pb.x = pack_bf16_rne(s[8 * t + 0], s[8 * t + 1]);
      pb.y = pack_bf16_rne(s[8 * t + 2], s[8 * t + 3]);
      pb.z = pack_bf16_rne(s[8 * t + 4], s[8 * t + 5]);
      pb.w = pack_bf16_rne(s[8 * t + 6], s[8 * t + 7]);
#pragma unroll
      for (int d = 0; d < DT; ++d) {
        const uint16_t *vr = ldsV + (d * 32 + l31) * VPITCH + 16 * t + 4 * hh;
        u32x2 lo = *(const u32x2 *)vr, hi = *(const u32x2 *)(vr + 8);
        u32x4 va = {lo.x, lo.y, hi.x, hi.y};
        o[d] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(*(bf16x8 *)&va, *(bf16x8 *)&pb, o[d], 0, 0, 0);
      }
    }
  }
  if (!wave_ok) return;
  const float inv = l_run > 0.0f ? 1.0f / l_run : 0.0f;
  const bool q_ok = q_glob < p.Sq;
#pragma unroll
  for (int d = 0; d < DT; ++d)
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const int din = g * 8 + hh * 4;
      u32x2 ov;
      ov.x = q_ok ? pack_bf16_rne(o[d][g * 4 + 0] * inv, o[d][g * 4 + 1] * inv) : 0u;
      ov.y = q_ok ? pack_bf16_rne(o[d][g * 4 + 2] * inv, o[d][g * 4 + 3] * inv) : 0u;
      uint8_t *op = p.out + o_mat + qt * p.o_pitch + d * 2048 +
                    (((l31 >> 4) * 2 + (din >> 4)) * 256 + (l31 & 15) * 16 + (din & 15)) * 2;
      *(u32x2 *)op = ov;
    }
}

// Same computation with 64 keys per pass (head_dim <= 128): half as many barriers and loop turns, two independent
// accumulator chains for S; K and V go to LDS as they lie in their tiles and the V^T fragments of the second product are
// made by transposing LDS reads.
constexpr int kSdpaVPitch = 68;   // sizes the V staging area: head_dim rows of 68 bf16 (64 keys x head_dim bf16 are used)

// one block of 128 queries (4 wavefronts x 32) of head h against all the keys it needs
template <int DT>  // head_dim / 32
__device__ __forceinline__ void sdpa64_query_block(const SdpaArgs &p, int qb, int h, int b, uint8_t *ldsK, uint16_t *ldsV) {
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int hk = h / (p.Hq / p.Hkv);
  const int qt = qb * 4 + wave;                         // this wave's query tile
  const bool wave_ok = qt < p.sqt;
  const int l31 = lane & 31, hh = lane >> 5;
  const int64_t q_mat = b * p.q_batch + h * p.q_head, o_mat = b * p.o_batch + h * p.o_head;
  const int64_t k_mat = b * p.k_batch + hk * p.k_head, v_mat = b * p.v_batch + hk * p.v_head;

  bf16x8 qf[2 * DT];
#pragma unroll
  for (int s = 0; s < 2 * DT; ++s) {
    u32x4 v = {0, 0, 0, 0};
    if (wave_ok)
      v = *(const u32x4 *)(p.q + q_mat + qt * p.q_pitch + (s >> 1) * 2048 + ((l31 >> 4) * 2 + (s & 1)) * 512 +
                           (l31 & 15) * 32 + hh * 16);
    qf[s] = *(bf16x8 *)&v;
  }
  f32x16 o[DT];
#pragma unroll
  for (int d = 0; d < DT; ++d)
#pragma unroll
    for (int r = 0; r < 16; ++r) o[d][r] = 0.0f;
  float m_run = -INFINITY, l_run = 0.0f;
  const int q_glob = qt * 32 + l31, q_last = qt * 32 + 31;

  // 32-key tiles any wave of this workgroup needs, and the 64-key passes that cover them
  const int kt_begin = first_key_tile(p, qb * 128), kt_end = end_key_tile(p, min(qb * 4 + 4, p.sqt) * 32 - 1);
  const int kb_begin = kt_begin >> 1, kb_end = (kt_end + 1) >> 1;
  // a lane moves DT 16-byte chunks of K and of V per pass: chunk c = tid + 256 i lies in tile row c / (DT * 128)
  u32x4 kreg[DT], vreg[DT];
  auto load_block = [&](int kb) {
#pragma unroll
    for (int i = 0; i < DT; ++i) {
      const int c = tid + 256 * i, tr = c / (DT * 128), cc = c % (DT * 128);
      const int kt = min(2 * kb + tr, p.skt - 1);       // an odd tile count repeats the last tile; its keys are masked
      kreg[i] = ((const u32x4 *)(p.k + k_mat + kt * p.k_pitch))[cc];
      vreg[i] = ((const u32x4 *)(p.v + v_mat + kt * p.v_pitch))[cc];
    }
  };
  if (kb_end > kb_begin) load_block(kb_begin);
  // per-lane part of the V^T fragment addresses: the face of this lane's column half, its key row and 4 columns
  const int dhalf = (lane >> 4) & 1, s16 = lane & 15;
  const uint8_t *vbase = (const uint8_t *)ldsV + dhalf * 512;
  const int vlo = ((4 * hh + (s16 >> 2)) * 32 + 8 * (s16 & 3) + 128 * dhalf) & 511, vhi = (vlo + 256) & 511;
  auto tr_read = [](const uint8_t *a) {
    typedef short s16x4 __attribute__((ext_vector_type(4)));
    const s16x4 v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3))) *)a);
    return *(const u32x2 *)&v;
  };
  constexpr float LOG2E = 1.4426950408889634f;
  const float scale2 = p.scale * LOG2E;
  sink_start(p, h, scale2, m_run, l_run);
  for (int kb = kb_begin; kb < kb_end; ++kb) {
    __syncthreads();  // previous block fully consumed
#pragma unroll
    for (int i = 0; i < DT; ++i) {
      const int c = tid + 256 * i, tr = c / (DT * 128), cc = c % (DT * 128);
      ((u32x4 *)ldsK)[c] = kreg[i];
      // V as it lies in its tiles (rows are keys), the faces of the upper 16 columns rotated by four rows so that the
      // transposing reads below touch every bank once
      const int c7 = cc & 127, face = c7 >> 5;
      *(u32x4 *)((uint8_t *)ldsV + (c - c7) * 16 + face * 512 + (((c7 & 31) * 16 + 128 * (face & 1)) & 511)) = vreg[i];
    }
    __syncthreads();
    if (kb + 1 < kb_end) load_block(kb + 1);
    const int key_base = kb * 64;
    if (!wave_ok || key_base > q_last + p.hi_off || key_base + 63 < qt * 32 - p.lo_off) continue;
    // the second half of the pass is skipped when the upper limit or the key count makes it empty for this wave
    const bool second = key_base + 32 <= q_last + p.hi_off && key_base + 32 < p.Sk;   // wavefront-uniform

    f32x16 s0, s1;
#pragma unroll
    for (int r = 0; r < 16; ++r) { s0[r] = 0.0f; s1[r] = 0.0f; }
#pragma unroll
    for (int st = 0; st < 2 * DT; ++st) {
      const uint8_t *kp = ldsK + (st >> 1) * 2048 + ((l31 >> 4) * 2 + (st & 1)) * 512 + (l31 & 15) * 32 + hh * 16;
      u32x4 ka = *(const u32x4 *)kp;
      s0 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(*(bf16x8 *)&ka, qf[st], s0, 0, 0, 0);
      if (second) {
        u32x4 kb2 = *(const u32x4 *)(kp + DT * 2048);
        s1 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(*(bf16x8 *)&kb2, qf[st], s1, 0, 0, 0);
      }
    }
    // scale, mask; a lane holds q = q_glob and keys key_base + 32 half + 8 g + 4 hh + r.  Scores stay in the log2
    // domain so that the exponential is a bare v_exp_f32.
    const bool edge = key_base + 63 > qt * 32 + p.hi_off || key_base < q_last - p.lo_off || key_base + 64 > p.Sk;   // wavefront-uniform
    float mx = -INFINITY;
    auto finish_scores = [&](f32x16 &s, int half) {
      if (p.mask || edge) {
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          const int kin = g * 8 + hh * 4;
          const int key0 = key_base + 32 * half + kin;
          float mk[4] = {0.f, 0.f, 0.f, 0.f};
          if (p.mask) {
            const int kt = min(2 * kb + half, p.skt - 1);
            const int64_t mm = ((int64_t)b * p.mask_b * p.mask_heads + (p.mask_heads == 1 ? 0 : h)) * p.sqt * p.skt * 2048;
            const uint8_t *mp = p.mask + mm + ((int64_t)qt * p.skt + kt) * 2048 +
                                (((l31 >> 4) * 2 + (kin >> 4)) * 256 + (l31 & 15) * 16 + (kin & 15)) * 2;
            u32x2 raw = *(const u32x2 *)mp;
            mk[0] = __uint_as_float(raw.x << 16); mk[1] = __uint_as_float(raw.x & 0xFFFF0000u);
            mk[2] = __uint_as_float(raw.y << 16); mk[3] = __uint_as_float(raw.y & 0xFFFF0000u);
          }
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            float v = fmaf(s[g * 4 + r], scale2, mk[r] * LOG2E);
            const int key = key0 + r;
            if (key >= p.Sk || key > q_glob + p.hi_off || key < q_glob - p.lo_off) v = -INFINITY;
            s[g * 4 + r] = v;
            mx = fmaxf(mx, v);
          }
        }
      } else {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          s[r] *= scale2;
          mx = fmaxf(mx, s[r]);
        }
      }
    };
    finish_scores(s0, 0);
    if (second) finish_scores(s1, 1);
    mx = fmaxf(mx, __shfl_xor(mx, 32));
    const float m_new = fmaxf(m_run, mx);
    const float m_use = m_new == -INFINITY ? 0.0f : m_new;   // fully masked so far: stay at zero without producing NaN
    const float alpha = __builtin_amdgcn_exp2f(m_run - m_use);
    float rs = 0.0f;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const float e = __builtin_amdgcn_exp2f(s0[r] - m_use);
      s0[r] = e;
      rs += e;
    }
    if (second) {
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const float e = __builtin_amdgcn_exp2f(s1[r] - m_use);
        s1[r] = e;
        rs += e;
      }
    }
    rs += __shfl_xor(rs, 32);
    l_run = l_run * alpha + rs;
    m_run = m_new;
    if (__builtin_amdgcn_ballot_w64(alpha != 1.0f) != 0) {   // the running maximum seldom moves after the first passes
#pragma unroll
      for (int d = 0; d < DT; ++d)
#pragma unroll
        for (int r = 0; r < 16; ++r) o[d][r] *= alpha;
    }
    // O^T += V^T . P^T, k16 steps over the 32 or 64 keys
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      if (t >= 2 && !second) break;
      const f32x16 &s = t < 2 ? s0 : s1;
      const int t8 = 8 * (t & 1);
      u32x4 pb;
      pb.x = pack_bf16_rne(s[t8 + 0], s[t8 + 1]);
      pb.y = pack_bf16_rne(s[t8 + 2], s[t8 + 3]);
      pb.z = pack_bf16_rne(s[t8 + 4], s[t8 + 5]);
      pb.w = pack_bf16_rne(s[t8 + 6], s[t8 + 7]);
#pragma unroll
      for (int d = 0; d < DT; ++d) {
        // V^T fragment: column d * 32 + l31, keys 16 t + 4 hh .. + 3 and eight further on, by two transposing LDS reads
        // (ds_read_b64_tr_b16: of the 16 lanes of a group, lane 4 u + c receives element c of the rows that lanes
        // u, u + 4, u + 8, u + 12 address; lane u + 4 j addresses key j of the four, columns 4 u .. + 3)
        const uint8_t *vb = vbase + (t >> 1) * DT * 2048 + d * 2048 + (t & 1) * 1024;
        const u32x2 lo = tr_read(vb + vlo), hi = tr_read(vb + vhi);
        u32x4 va = {lo.x, lo.y, hi.x, hi.y};
        o[d] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(*(bf16x8 *)&va, *(bf16x8 *)&pb, o[d], 0, 0, 0);
      }
    }
  }
  if (!wave_ok) return;
  const float inv = l_run > 0.0f ? 1.0f / l_run : 0.0f;
  const bool q_ok = q_glob < p.Sq;
#pragma unroll
  for (int d = 0; d < DT; ++d)
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const int din = g * 8 + hh * 4;
      u32x2 ov;
      ov.x = q_ok ? pack_bf16_rne(o[d][g * 4 + 0] * inv, o[d][g * 4 + 1] * inv) : 0u;
      ov.y = q_ok ? pack_bf16_rne(o[d][g * 4 + 2] * inv, o[d][g * 4 + 3] * inv) : 0u;
      uint8_t *op = p.out + o_mat + qt * p.o_pitch + d * 2048 +
                    (((l31 >> 4) * 2 + (din >> 4)) * 256 + (l31 & 15) * 16 + (din & 15)) * 2;
      *(u32x2 *)op = ov;
    }
}


// Causal attention gives query block qb work proportional to qb + 1.  With one workgroup per query block all workgroups of a
// launch are resident at once and the launch lasts as long as the heaviest of them; a workgroup therefore takes the pair
// (last - i, i), heavy block first, so that every workgroup has the same amount of work.
template <int DT>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2))) void ttm_sdpa64_k(SdpaArgs p, int paired) {
  constexpr int D = DT * 32;
  __shared__ __attribute__((aligned(16))) uint8_t ldsK[64 * D * 2];
  __shared__ __attribute__((aligned(16))) uint16_t ldsV[D * kSdpaVPitch];
  const int nqb = (p.sqt + 3) / 4;
  int x = blockIdx.x, h = blockIdx.y, b = blockIdx.z;
  sdpa_xcd_order(p, x, h, b);
  if (!paired) {
    sdpa64_query_block<DT>(p, nqb - 1 - x, h, b, ldsK, ldsV);
    return;
  }
  const int heavy = nqb - 1 - x, light = x;
  sdpa64_query_block<DT>(p, heavy, h, b, ldsK, ldsV);
  if (light < heavy) sdpa64_query_block<DT>(p, light, h, b, ldsK, ldsV);
}

// The same pass with eight wavefronts: wavefront w serves query tile w % 4 and the key half w / 4 of every 64-key pass,
// with its own running maximum, sum and output; the two halves of a query tile are merged through LDS at the end.  A launch
// that has only one workgroup per CU (a single sequence of a few thousand tokens) then still keeps two wavefronts on every
// SIMD, so that one's softmax overlaps the other's matrix products; staging K and V is shared by twice as many lanes.
template <int DT>  // head_dim / 32
__device__ __forceinline__ void sdpa64_split_block(const SdpaArgs &p, int qb, int h, int b, uint8_t *ldsK, uint16_t *ldsV, int ks = 0) {
  constexpr int NT = 512, CHUNKS = DT * 256, NCH = (CHUNKS + NT - 1) / NT;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int qw = wave & 3, kh = wave >> 2;
  const int hk = h / (p.Hq / p.Hkv);
  const int qt = qb * 4 + qw;                           // this wave's query tile
  const bool wave_ok = qt < p.sqt;
  const int l31 = lane & 31, hh = lane >> 5;
  const int64_t q_mat = b * p.q_batch + h * p.q_head, o_mat = b * p.o_batch + h * p.o_head;
  const int64_t k_mat = b * p.k_batch + hk * p.k_head, v_mat = b * p.v_batch + hk * p.v_head;

  bf16x8 qf[2 * DT];
#pragma unroll
  for (int s = 0; s < 2 * DT; ++s) {
    u32x4 v = {0, 0, 0, 0};
    if (wave_ok)
      v = *(const u32x4 *)(p.q + q_mat + qt * p.q_pitch + (s >> 1) * 2048 + ((l31 >> 4) * 2 + (s & 1)) * 512 +
                           (l31 & 15) * 32 + hh * 16);
    qf[s] = *(bf16x8 *)&v;
  }
  f32x16 o[DT];
#pragma unroll
  for (int d = 0; d < DT; ++d)
#pragma unroll
    for (int r = 0; r < 16; ++r) o[d][r] = 0.0f;
  float m_run = -INFINITY, l_run = 0.0f;
  const int q_glob = qt * 32 + l31, q_last = qt * 32 + 31;

  const int kt_begin = first_key_tile(p, qb * 128), kt_end = end_key_tile(p, min(qb * 4 + 4, p.sqt) * 32 - 1);
  int kb_begin = kt_begin >> 1, kb_end = (kt_end + 1) >> 1;
  if (p.ksplits > 1) {   // this workgroup's share of the query block's keys (workgroup-uniform)
    const int chunk = (kb_end - kb_begin + p.ksplits - 1) / p.ksplits;
    kb_begin += ks * chunk;
    kb_end = min(kb_end, kb_begin + chunk);
  }
  u32x4 kreg[NCH], vreg[NCH];
  auto load_block = [&](int kb) {
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
      const int c = tid + NT * i;
      if (c < CHUNKS) {
        const int tr = c / (DT * 128), cc = c % (DT * 128);
        const int kt = min(2 * kb + tr, p.skt - 1);     // an odd tile count repeats the last tile; its keys are masked
        kreg[i] = ((const u32x4 *)(p.k + k_mat + kt * p.k_pitch))[cc];
        vreg[i] = ((const u32x4 *)(p.v + v_mat + kt * p.v_pitch))[cc];
      }
    }
  };
  if (kb_end > kb_begin) load_block(kb_begin);
  // per-lane part of the V^T fragment addresses: tile row kh, the face of this lane's column half, its key row and 4 columns
  const int dhalf = (lane >> 4) & 1, s16 = lane & 15;
  const uint8_t *vbase = (const uint8_t *)ldsV + kh * DT * 2048 + dhalf * 512;
  const int vlo = ((4 * hh + (s16 >> 2)) * 32 + 8 * (s16 & 3) + 128 * dhalf) & 511, vhi = (vlo + 256) & 511;
  auto tr_read = [](const uint8_t *a) {
    typedef short s16x4 __attribute__((ext_vector_type(4)));
    const s16x4 v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3))) *)a);
    return *(const u32x2 *)&v;
  };
  constexpr float LOG2E = 1.4426950408889634f;
  const float scale2 = p.scale * LOG2E;
  if (kh == 0 && ks == 0) sink_start(p, h, scale2, m_run, l_run);   // the sink belongs to one of the two halves (and one key share) only
  for (int kb = kb_begin; kb < kb_end; ++kb) {
    __syncthreads();  // previous block fully consumed
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
      const int c = tid + NT * i;
      if (c < CHUNKS) {   // uniform over a wavefront: CHUNKS is a multiple of 64
        const int tr = c / (DT * 128), cc = c % (DT * 128);
        ((u32x4 *)ldsK)[c] = kreg[i];
        // V as it lies in its tiles (rows are keys), the faces of the upper 16 columns rotated by four rows so that the
        // transposing reads below touch every bank once
        const int c7 = cc & 127, face = c7 >> 5;
        *(u32x4 *)((uint8_t *)ldsV + (c - c7) * 16 + face * 512 + (((c7 & 31) * 16 + 128 * (face & 1)) & 511)) = vreg[i];
      }
    }
    __syncthreads();
    if (kb + 1 < kb_end) load_block(kb + 1);
    const int key_base = kb * 64 + 32 * kh;             // this wavefront's 32 keys of the pass
    if (!wave_ok || key_base > q_last + p.hi_off || key_base + 31 < qt * 32 - p.lo_off || key_base >= p.Sk) continue;

    f32x16 s;
#pragma unroll
    for (int r = 0; r < 16; ++r) s[r] = 0.0f;
#pragma unroll
    for (int st = 0; st < 2 * DT; ++st) {
      const uint8_t *kp = ldsK + kh * DT * 2048 + (st >> 1) * 2048 + ((l31 >> 4) * 2 + (st & 1)) * 512 + (l31 & 15) * 32 + hh * 16;
      u32x4 ka = *(const u32x4 *)kp;
      s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(*(bf16x8 *)&ka, qf[st], s, 0, 0, 0);
    }
    const bool edge = key_base + 31 > qt * 32 + p.hi_off || key_base < q_last - p.lo_off || key_base + 32 > p.Sk;   // wavefront-uniform
    float mx = -INFINITY, mul = 1.0f;
    if (p.mask || edge) {
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int kin = g * 8 + hh * 4;
        const int key0 = key_base + kin;
        float mk[4] = {0.f, 0.f, 0.f, 0.f};
        if (p.mask) {
          const int kt = min(2 * kb + kh, p.skt - 1);
          const int64_t mm = ((int64_t)b * p.mask_b * p.mask_heads + (p.mask_heads == 1 ? 0 : h)) * p.sqt * p.skt * 2048;
          const uint8_t *mp = p.mask + mm + ((int64_t)qt * p.skt + kt) * 2048 +
                              (((l31 >> 4) * 2 + (kin >> 4)) * 256 + (l31 & 15) * 16 + (kin & 15)) * 2;
          u32x2 raw = *(const u32x2 *)mp;
          mk[0] = __uint_as_float(raw.x << 16); mk[1] = __uint_as_float(raw.x & 0xFFFF0000u);
          mk[2] = __uint_as_float(raw.y << 16); mk[3] = __uint_as_float(raw.y & 0xFFFF0000u);
        }
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          float v = fmaf(s[g * 4 + r], scale2, mk[r] * LOG2E);
          const int key = key0 + r;
          if (key >= p.Sk || key > q_glob + p.hi_off || key < q_glob - p.lo_off) v = -INFINITY;
          s[g * 4 + r] = v;
          mx = fmaxf(mx, v);
        }
      }
    } else {   // plain block: the scale (positive) is folded into the exponent's multiply-add, the maximum is taken first
#pragma unroll
      for (int r = 0; r < 16; ++r) mx = fmaxf(mx, s[r]);
      mx *= scale2;
      mul = scale2;
    }
    mx = fmaxf(mx, __shfl_xor(mx, 32));
    const float m_new = fmaxf(m_run, mx);
    const float m_use = m_new == -INFINITY ? 0.0f : m_new;   // fully masked so far: stay at zero without producing NaN
    const float alpha = __builtin_amdgcn_exp2f(m_run - m_use);
    float rs = 0.0f;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const float e = __builtin_amdgcn_exp2f(fmaf(s[r], mul, -m_use));
      s[r] = e;
      rs += e;
    }
    rs += __shfl_xor(rs, 32);
    l_run = l_run * alpha + rs;
    m_run = m_new;
    if (__builtin_amdgcn_ballot_w64(alpha != 1.0f) != 0) {
#pragma unroll
      for (int d = 0; d < DT; ++d)
#pragma unroll
        for (int r = 0; r < 16; ++r) o[d][r] *= alpha;
    }
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      u32x4 pb;
      pb.x = pack_bf16_rne(s[8 * t + 0], s[8 * t + 1]);
      pb.y = pack_bf16_rne(s[8 * t + 2], s[8 * t + 3]);
      pb.z = pack_bf16_rne(s[8 * t + 4], s[8 * t + 5]);
      pb.w = pack_bf16_rne(s[8 * t + 6], s[8 * t + 7]);
#pragma unroll
      for (int d = 0; d < DT; ++d) {
        // V^T fragment: column d * 32 + l31, keys 16 t + 4 hh .. + 3 and eight further on, by two transposing LDS reads
        // (ds_read_b64_tr_b16: of the 16 lanes of a group, lane 4 u + c receives element c of the rows that lanes
        // u, u + 4, u + 8, u + 12 address; lane u + 4 j addresses key j of the four, columns 4 u .. + 3)
        const uint8_t *vb = vbase + d * 2048 + t * 1024;
        const u32x2 lo = tr_read(vb + vlo), hi = tr_read(vb + vhi);
        u32x4 va = {lo.x, lo.y, hi.x, hi.y};
        o[d] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(*(bf16x8 *)&va, *(bf16x8 *)&pb, o[d], 0, 0, 0);
      }
    }
  }
  // merge the two key halves of every query tile: the upper half hands over (max, sum) through the V region and its
  // output, 4 DT values per lane at a time, through the K region (DT * 4 KiB = 256 lanes x DT float4)
  __syncthreads();
  float *ml = (float *)ldsV;
  f32x4 *ox = (f32x4 *)ldsK;
  const int slot = qw * 64 + lane;
  if (kh == 1) { ml[2 * slot] = m_run; ml[2 * slot + 1] = l_run; }
  __syncthreads();
  float a0 = 1.0f, a1 = 0.0f;
  if (kh == 0) {
    const float m1 = ml[2 * slot], l1 = ml[2 * slot + 1];
    const float m = fmaxf(m_run, m1), m_use = m == -INFINITY ? 0.0f : m;
    a0 = __builtin_amdgcn_exp2f(m_run - m_use);
    a1 = __builtin_amdgcn_exp2f(m1 - m_use);
    l_run = l_run * a0 + l1 * a1;
    m_run = m;   // what the merged sum and output are relative to (a key share hands it on)
  }
#pragma unroll
  for (int r4 = 0; r4 < 4; ++r4) {
    if (kh == 1) {
#pragma unroll
      for (int d = 0; d < DT; ++d) ox[slot * DT + d] = f32x4{o[d][4 * r4], o[d][4 * r4 + 1], o[d][4 * r4 + 2], o[d][4 * r4 + 3]};
    }
    __syncthreads();
    if (kh == 0) {
#pragma unroll
      for (int d = 0; d < DT; ++d) {
        const f32x4 x = ox[slot * DT + d];
#pragma unroll
        for (int e = 0; e < 4; ++e) o[d][4 * r4 + e] = o[d][4 * r4 + e] * a0 + x[e] * a1;
      }
    }
    __syncthreads();
  }
  if (kh != 0 || !wave_ok) return;   // no barrier follows inside this block; the next block starts with one
  if (p.ksplits > 1) {   // one share of the keys: leave (max, sum, unnormalised output) for ttm_sdpa_combine_k
    const int64_t slot_q = (((int64_t)ks * p.B + b) * p.Hq + h) * p.sqt + qt;
    if (hh == 0) { p.part_ml[slot_q * 64 + 2 * l31] = m_run; p.part_ml[slot_q * 64 + 2 * l31 + 1] = l_run; }
#pragma unroll
    for (int d = 0; d < DT; ++d)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int din = g * 8 + hh * 4;
        *(f32x4 *)(p.part_o + (slot_q * DT + d) * 1024 + ((l31 >> 4) * 2 + (din >> 4)) * 256 + (l31 & 15) * 16 + (din & 15)) =
            f32x4{o[d][g * 4], o[d][g * 4 + 1], o[d][g * 4 + 2], o[d][g * 4 + 3]};
      }
    return;
  }
  const float inv = l_run > 0.0f ? 1.0f / l_run : 0.0f;
  const bool q_ok = q_glob < p.Sq;
#pragma unroll
  for (int d = 0; d < DT; ++d)
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const int din = g * 8 + hh * 4;
      u32x2 ov;
      ov.x = q_ok ? pack_bf16_rne(o[d][g * 4 + 0] * inv, o[d][g * 4 + 1] * inv) : 0u;
      ov.y = q_ok ? pack_bf16_rne(o[d][g * 4 + 2] * inv, o[d][g * 4 + 3] * inv) : 0u;
      uint8_t *op = p.out + o_mat + qt * p.o_pitch + d * 2048 +
                    (((l31 >> 4) * 2 + (din >> 4)) * 256 + (l31 & 15) * 16 + (din & 15)) * 2;
      *(u32x2 *)op = ov;
    }
}

template <int DT>
__global__ __launch_bounds__(512) void ttm_sdpa64_split_k(SdpaArgs p, int paired) {
  constexpr int D = DT * 32;
  __shared__ __attribute__((aligned(16))) uint8_t ldsK[64 * D * 2];
  __shared__ __attribute__((aligned(16))) uint16_t ldsV[D * kSdpaVPitch];
  const int nqb = (p.sqt + 3) / 4;
  int x = blockIdx.x, h = blockIdx.y, b = blockIdx.z;
  sdpa_xcd_order(p, x, h, b);
  if (!paired) {   // with key shares grid.x numbers (query block, share)
    const int xb = x / p.ksplits, ks = x - xb * p.ksplits;
    sdpa64_split_block<DT>(p, nqb - 1 - xb, h, b, ldsK, ldsV, ks);
    return;
  }
  const int heavy = nqb - 1 - x, light = x;
  sdpa64_split_block<DT>(p, heavy, h, b, ldsK, ldsV);
  if (light < heavy) sdpa64_split_block<DT>(p, light, h, b, ldsK, ldsV);   // workgroup-uniform
}

// The eight-wavefront pass as a software pipeline.  ttm_sdpa64_split_k runs a pass as a chain (stage K and V through
// registers, barrier, fragment reads, scores, softmax, second product, barrier): all wavefronts ask LDS for their
// fragments at the same time, then the matrix core at the same time, then the vector ALU at the same time.  Here
//   * K and V go global -> LDS with LDS-direct loads (no staging registers, no ds_write) into a ring of five 64-key
//     stages, requested three passes ahead and issued one at a time between the MFMAs; one barrier per pass, and a pass has
//     landed one barrier before it is multiplied;
//   * a wavefront computes the scores of pass i while it takes the exponentials of pass i - 1: every MFMA of the score
//     product is followed by one score's share of the softmax, and the second product of pass i - 1 follows with the rest;
//   * the fragments a step starts with (K of the first 64 columns, V^T of the first 16 keys) are requested at the end of
//     the step before, across the barrier, so that the reads of the eight wavefronts do not pile up behind it;
//   * a wavefront's passes are an interval (causal and window limits are bands): first pass scores only, last pass softmax
//     only, the loop between them is free of conditions;
//   * the running maximum is only moved when some query's maximum grew by more than 8 (in the log2 domain): sums and
//     outputs stay relative to the older maximum (probabilities up to 2^8, exact in bf16's range), and the rescale of the
//     output accumulators, 16 DT multiplies per lane, becomes rare;
//   * the two halves of a query's maximum and sum are exchanged with v_permlane32_swap instead of through LDS.
// Same fragment layouts, same arithmetic per score as the kernels above.
__device__ __forceinline__ void sdpa_dma16(const void *base, uint32_t lane_off, uint32_t lds_addr) {
  // lds_addr is wavefront-uniform; lane l of the wavefront writes 16 bytes at lds_addr + 16 l
  asm volatile("s_mov_b32 m0, %2\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(lane_off), "s"(base), "s"(lds_addr) : "memory");
}
template <int IMM>
__device__ __forceinline__ void sdpa_dma16_at(const void *base, uint32_t lane_off, uint32_t lds_addr) {   // to lds_addr + IMM
  asm volatile("s_add_u32 m0, %2, %3\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(lane_off), "s"(base), "s"(lds_addr), "n"(IMM) : "memory", "scc");
}
__device__ __forceinline__ float sdpa_max_halves(float x) {
  const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float sdpa_sum_halves(float x) {
  const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}
template <bool B> struct SdpaFlag { static constexpr bool value = B; };
template <int I> struct SdpaIdx { static constexpr int value = I; };

// KH = 2: eight wavefronts, 64 keys per pass, the two key halves of a query tile in two wavefronts (merged at the end).
// KH = 1: four wavefronts, 32 keys per pass, no halves: half the ring, so that two workgroups share a CU and the two
// wavefronts of a SIMD belong to different workgroups - no common barrier, no merge.
template <int DT, int KH>  // head_dim / 32: 2 or 4
__device__ __forceinline__ void sdpa_pipe_block(const SdpaArgs &p, int qb, int h, int b, uint8_t *lds) {
  static_assert((DT == 2 || DT == 4) && (KH == 1 || KH == 2), "64 or 128 columns");
  constexpr int TROW = DT * 2048;      // one 32-key tile row of K or V
  constexpr int STAGE = 2 * KH * TROW; // a pass of 32 KH keys: KH tile rows of K, then of V
  constexpr int LANES = 256 * KH;
  constexpr int NST = 5;               // stages of the ring
  constexpr int NL = DT;               // LDS-direct loads per wavefront and pass: DT / 2 of K, DT / 2 of V
  const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t *)lds;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int qw = wave & 3, kh = wave >> 2;
  const int hk = h / (p.Hq / p.Hkv);
  const int qt = qb * 4 + qw;                           // this wave's query tile
  const bool wave_ok = qt < p.sqt;
  const int l31 = lane & 31, hh = lane >> 5;
  const int64_t q_mat = b * p.q_batch + h * p.q_head, o_mat = b * p.o_batch + h * p.o_head;
  const int64_t k_mat = b * p.k_batch + hk * p.k_head, v_mat = b * p.v_batch + hk * p.v_head;

  bf16x8 qf[2 * DT];
#pragma unroll
  for (int s = 0; s < 2 * DT; ++s) {
    u32x4 v = {0, 0, 0, 0};
    if (wave_ok)
      v = *(const u32x4 *)(p.q + q_mat + qt * p.q_pitch + (s >> 1) * 2048 + ((l31 >> 4) * 2 + (s & 1)) * 512 +
                           (l31 & 15) * 32 + hh * 16);
    qf[s] = *(bf16x8 *)&v;
  }
  f32x16 o[DT];
#pragma unroll
  for (int d = 0; d < DT; ++d)
#pragma unroll
    for (int r = 0; r < 16; ++r) o[d][r] = 0.0f;
  float m_run = -INFINITY, l_run = 0.0f;
  const int q_glob = qt * 32 + l31, q_last = qt * 32 + 31;
  const int kt_begin = first_key_tile(p, qb * 128), kt_end = end_key_tile(p, min(qb * 4 + 4, p.sqt) * 32 - 1);
  const int kb_begin = kt_begin / KH, kb_end = (kt_end + KH - 1) / KH;
  // This wavefront's 32 keys of pass kb start at 32 KH kb + 32 kh; the passes in which one of them is visible to one of its
  // queries (not behind the causal or window limit, not in front of the window, not past the last key) are an interval.
  int w_begin, w_end;
  {
    const int x = qt * 32 - p.lo_off - 31 - 32 * kh;
    const int y = min(q_last + p.hi_off, p.Sk - 1) - 32 * kh;
    w_begin = max(x > 0 ? (x + 32 * KH - 1) / (32 * KH) : 0, kb_begin);
    w_end = min(y >= 0 ? y / (32 * KH) + 1 : 0, kb_end);
    if (!wave_ok || w_begin >= w_end) w_begin = w_end = kb_end;
  }

  // Staging.  The instructions of a wavefront cover 64 consecutive 16-byte chunks of LDS each; chunk c of a pass's K lies
  // in tile row c / (128 DT).  K is copied as it lies in its tiles (but for the exchange below); V too, but the faces of the upper 16 columns are
  // rotated by eight chunks (four rows) so that the transposing reads touch every bank once: the lane that fills a chunk
  // of such a face fetches the chunk eight further back.
  const int c0 = wave * 64;                               // with 128 DT chunks per tile row, load i of a wavefront (chunk
  const int ccl = c0 % (DT * 128) + lane;                 // c0 + LANES (i / 2) + lane of the pass's K or V) lies in tile row
                                                          // (c0 + LANES (i / 2)) / (128 DT); ccl is its chunk there for i < 2
  // K is copied as it lies in its tiles but for one exchange: in the faces' rows 8..15 the two 16-byte halves of a row swap
  // places, so that the 16 lanes whose fragment reads go out together (rows 0..15, one half) touch 16 different bank groups
  // instead of 8 twice.  The lane that fills a chunk fetches its partner's.
  const uint32_t koff = (ccl ^ ((ccl >> 4) & 1)) * 16;
  const uint32_t voff = ((ccl & ~31) + (((ccl & 31) - 8 * ((ccl >> 5) & 1)) & 31)) * 16;
  const uint8_t *kg = p.k + k_mat, *vg = p.v + v_mat;
  auto next_stage = [](int st) { return st + STAGE == NST * STAGE ? 0 : st + STAGE; };   // byte offsets of the ring's stages
  // The ring's loads walk the passes in order, three ahead of the pass being multiplied, so what a load needs is carried
  // from pass to pass in scalar registers instead of being worked out from the pass number (64-bit multiplies, a chain
  // of stage selects: 60 scalar instructions per pass, of which a wavefront issues one per four cycles): the addresses
  // of the pass's first K and V tile rows, its stage, and the distance to its second tile row - zero when an odd tile
  // count ends inside the pass: the last tile is fetched twice and its keys are masked.  Past the last pass the loads
  // stay on it while the stage moves on: every pass of the loop requests NL loads, so that the counted wait below
  // always has the same meaning; what they fetch then lands in the stage that is free at that point and is never read.
  const uint32_t ld_m0 = lds0 + c0 * 16;
  int ld_kb = kb_begin, ld_st = 0;
  const uint8_t *ld_k = kg + (int64_t)(KH * kb_begin) * p.k_pitch, *ld_v = vg + (int64_t)(KH * kb_begin) * p.v_pitch;
  // KH = 2: this wavefront's loads of the second half (DT = 4) or all its loads (DT = 2) are tile row 1.  KH = 1: the
  // second half (DT = 4) is the second half of the one tile row, 4096 bytes on.
  const bool ld_row1 = DT == 4 || wave >= 4;
  uint32_t koff1 = koff + (KH == 1 ? 4096u : 0u), voff1 = voff + (KH == 1 ? 4096u : 0u);   // lane offsets of that half
  auto ld_second = [&]() {
    if constexpr (KH == 2) {
      const bool second = ld_row1 && 2 * ld_kb + 1 < p.skt;
      koff1 = koff + (second ? (uint32_t)p.k_pitch : 0u);
      voff1 = voff + (second ? (uint32_t)p.v_pitch : 0u);
    }
  };
  ld_second();
  auto dma = [&](auto i_tag) {   // load i of this wavefront for the pass the ring is at: K for even i, V for odd
    constexpr int i = decltype(i_tag)::value;
    constexpr bool r1 = KH == 2 && DT == 2 ? true : (i >> 1) != 0;
    if constexpr (i & 1) sdpa_dma16_at<(i >> 1) * LANES * 16 + KH * TROW>(ld_v, r1 ? voff1 : voff, ld_m0 + ld_st);
    else sdpa_dma16_at<(i >> 1) * LANES * 16>(ld_k, r1 ? koff1 : koff, ld_m0 + ld_st);
  };
  auto ld_advance = [&]() {   // on to the next pass
    const bool more = ld_kb + 1 < kb_end;
    ld_kb += more ? 1 : 0;
    ld_k += more ? KH * p.k_pitch : 0;
    ld_v += more ? KH * p.v_pitch : 0;
    ld_st = next_stage(ld_st);
    ld_second();
  };
  auto dma_all = [&]() {
    dma(SdpaIdx<0>{}); dma(SdpaIdx<1>{});
    if constexpr (NL > 2) { dma(SdpaIdx<2>{}); dma(SdpaIdx<3>{}); }
    ld_advance();
  };
  // All but this wavefront's last NL loads have landed, hence pass kb + 1 (requested two passes ago), and after the barrier
  // every wavefront's share of it; and every wavefront is through with pass kb - 2, whose stage pass kb + 3 overwrites.
  auto sync = [&]() {
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(NL) : "memory");
    __syncthreads();
  };
  // per-lane parts of the fragment addresses inside a stage
  const int dhalf = (lane >> 4) & 1, s16 = lane & 15;
  const int kfrag = kh * TROW + (l31 >> 4) * 1024 + (l31 & 15) * 32 + (hh ^ ((l31 >> 3) & 1)) * 16;
  const int vfrag = KH * TROW + kh * TROW + dhalf * 512;
  const int vlo = ((4 * hh + (s16 >> 2)) * 32 + 8 * (s16 & 3) + 128 * dhalf) & 511, vhi = (vlo + 256) & 511;
  const uint8_t *kfp = lds + kfrag, *vlp = lds + vfrag + vlo, *vhp = lds + vfrag + vhi;
  u32x4 ka[DT];   // K fragments of DT of a pass's 2 DT steps at a time
  u32x4 va[DT];   // V^T fragments of 16 of a pass's 32 keys at a time
  auto read_k = [&](const uint8_t *kp, int st) {   // step st of the pass whose stage kp points into
    ka[st % DT] = *(const u32x4 *)(kp + (st >> 1) * 2048 + (st & 1) * 512);
  };
  auto read_v = [&](const uint8_t *vl, const uint8_t *vh, int t, int d) {
    // V^T fragment: column d * 32 + l31, keys 16 t + 4 hh .. + 3 and eight further on, by two transposing LDS reads
    // (ds_read_b64_tr_b16: of the 16 lanes of a group, lane 4 u + c receives element c of the rows that lanes
    // u, u + 4, u + 8, u + 12 address; lane u + 4 j addresses key j of the four, columns 4 u .. + 3)
    typedef short s16x4 __attribute__((ext_vector_type(4)));
    const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3))) *)(vl + d * 2048 + t * 1024));
    const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3))) *)(vh + d * 2048 + t * 1024));
    const u32x2 l2 = *(const u32x2 *)&lo, h2 = *(const u32x2 *)&hi;
    va[d] = u32x4{l2.x, l2.y, h2.x, h2.y};
  };
  constexpr float LOG2E = 1.4426950408889634f;
  const float scale2 = p.scale * LOG2E;
  if (kh == 0) sink_start(p, h, scale2, m_run, l_run);   // the sink belongs to one of the two halves only
  float m_use = m_run == -INFINITY ? 0.0f : m_run;       // what the exponentials are relative to: zero while nothing is seen

  // The ring as this wavefront walks it: byte offset of the stage of the pass being multiplied and the fragment addresses
  // in it, in the stage before (V of the pass whose softmax is under way) and, computed in the step, in the stage after.
  int st_cur = 0;
  const uint8_t *k_cur = kfp, *vl_prev = vlp, *vh_prev = vhp, *vl_cur = vlp, *vh_cur = vhp;
  const uint32_t ones = 0x3F803F80u;   // two bf16 ones: v_dot2_f32_bf16 with them adds a pair of probabilities as the matrix core sees them

  // One pipeline step at pass kb: the score product of pass kb into sn (QK) beside the softmax and the second product of
  // pass kb - 1, whose scores are in sc (SM).  On entry ka holds the K fragments of the first DT steps of pass kb (QK) and
  // va the V^T fragments of the first 16 keys of pass kb - 1 (SM); on exit they hold those of the next step.  RING: the
  // step requests pass kb + 3 (not the step behind the last barrier).
  auto step = [&](auto qk_tag, auto sm_tag, auto ring_tag, int kb, f32x16 &sc, f32x16 &sn) {
    constexpr bool QK = decltype(qk_tag)::value, SM = decltype(sm_tag)::value, RING = decltype(ring_tag)::value;
    const int st_next = next_stage(st_cur);
    const uint8_t *k_next = kfp + st_next;
    float mul = scale2, rs = 0.0f;
    if constexpr (SM) {
      const int key_base = (kb - 1) * 32 * KH + 32 * kh;
      const bool edge = key_base + 31 > qt * 32 + p.hi_off || key_base < q_last - p.lo_off || key_base + 32 > p.Sk;   // wavefront-uniform
      float mx = -INFINITY;
      if (p.mask || edge) {
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          const int kin = g * 8 + hh * 4;
          const int key0 = key_base + kin;
          float mk[4] = {0.f, 0.f, 0.f, 0.f};
          if (p.mask) {
            const int kt = min(KH * (kb - 1) + kh, p.skt - 1);
            const int64_t mm = ((int64_t)b * p.mask_b * p.mask_heads + (p.mask_heads == 1 ? 0 : h)) * p.sqt * p.skt * 2048;
            const uint8_t *mp = p.mask + mm + ((int64_t)qt * p.skt + kt) * 2048 +
                                (((l31 >> 4) * 2 + (kin >> 4)) * 256 + (l31 & 15) * 16 + (kin & 15)) * 2;
            u32x2 raw = *(const u32x2 *)mp;
            mk[0] = __uint_as_float(raw.x << 16); mk[1] = __uint_as_float(raw.x & 0xFFFF0000u);
            mk[2] = __uint_as_float(raw.y << 16); mk[3] = __uint_as_float(raw.y & 0xFFFF0000u);
          }
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            float v = fmaf(sc[g * 4 + r], scale2, mk[r] * LOG2E);
            const int key = key0 + r;
            if (key >= p.Sk || key > q_glob + p.hi_off || key < q_glob - p.lo_off) v = -INFINITY;
            sc[g * 4 + r] = v;
            mx = fmaxf(mx, v);
          }
        }
        mul = 1.0f;
      } else {   // plain block: the scale (positive) is folded into the exponent's multiply-add, the maximum is taken first
#pragma unroll
        for (int r = 0; r < 16; ++r) mx = fmaxf(mx, sc[r]);
        mx *= scale2;
      }
      mx = sdpa_max_halves(mx);
      if (__builtin_amdgcn_ballot_w64(mx > m_run + 8.0f) != 0) {   // some query's maximum grew by more than 2^8: all move
        const float m_new = fmaxf(m_run, mx);
        const float m_to = m_new == -INFINITY ? 0.0f : m_new;   // fully masked so far: stay at zero without producing NaN
        const float alpha = __builtin_amdgcn_exp2f(m_run - m_to);
        l_run *= alpha;
#pragma unroll
        for (int d = 0; d < DT; ++d)
#pragma unroll
          for (int r = 0; r < 16; ++r) o[d][r] *= alpha;
        m_run = m_new;
        m_use = m_to;
      }
    }
    const float neg_m = -m_use;
    auto elem = [&](int r) { sc[r] = __builtin_amdgcn_exp2f(fmaf(sc[r], mul, neg_m)); };
    auto pack8 = [&](int r0) {   // eight probabilities as bf16, and their sum as rounded
      u32x4 pb;
      pb.x = pack_bf16_rne(sc[r0 + 0], sc[r0 + 1]);
      pb.y = pack_bf16_rne(sc[r0 + 2], sc[r0 + 3]);
      pb.z = pack_bf16_rne(sc[r0 + 4], sc[r0 + 5]);
      pb.w = pack_bf16_rne(sc[r0 + 6], sc[r0 + 7]);
      const uint32_t w[4] = {pb.x, pb.y, pb.z, pb.w};
#pragma unroll
      for (int j = 0; j < 4; ++j) rs = __builtin_amdgcn_fdot2_f32_bf16(*(const sdpa_bf16x2 *)&w[j], *(const sdpa_bf16x2 *)&ones, rs, false);
      return pb;
    };
    __builtin_amdgcn_sched_barrier(0);
    // first half of the exponentials, one MFMA of the score product in front of each share; behind the MFMA its K
    // register is refilled: second half of this pass, then first half of the next
    const f32x16 zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int st = 0; st < 2 * DT; ++st) {
      if constexpr (QK) {
        sn = __builtin_amdgcn_mfma_f32_32x32x16_bf16(*(bf16x8 *)&ka[st % DT], qf[st], st == 0 ? zero : sn, 0, 0, 0);
        if (st < DT) read_k(k_cur, st + DT);
        else read_k(k_next, st - DT);
      }
      if constexpr (RING) {   // the ring's loads are spread over the step: the addresser takes one wavefront's at a time
        if (st == 0) dma(SdpaIdx<0>{});
        if constexpr (NL > 2) { if (st == DT) dma(SdpaIdx<2>{}); }
      }
      if constexpr (SM) {
#pragma unroll
        for (int e = 0; e < 8 / (2 * DT); ++e) elem(st * (8 / (2 * DT)) + e);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    if constexpr (SM) {
      u32x4 pb = pack8(0);
      __builtin_amdgcn_sched_barrier(0);
      // second half of the exponentials beside the second product of the first 16 keys; the V^T fragments of the other
      // 16 keys follow into the same registers
#pragma unroll
      for (int d = 0; d < DT; ++d) {
        o[d] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(*(bf16x8 *)&va[d], *(bf16x8 *)&pb, o[d], 0, 0, 0);
        read_v(vl_prev, vh_prev, 1, d);
        if constexpr (RING) {
          if (d == 0) dma(SdpaIdx<1>{});
        }
#pragma unroll
        for (int e = 0; e < 8 / DT; ++e) elem(8 + d * (8 / DT) + e);
        __builtin_amdgcn_sched_barrier(0);
      }
      pb = pack8(8);
#pragma unroll
      for (int d = 0; d < DT; ++d) {
        o[d] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(*(bf16x8 *)&va[d], *(bf16x8 *)&pb, o[d], 0, 0, 0);
        if constexpr (QK) read_v(vl_cur, vh_cur, 0, d);   // for the next step
        if constexpr (RING) {
          if constexpr (NL > 2) { if (d == 0) dma(SdpaIdx<3>{}); }
        }
      }
      l_run += sdpa_sum_halves(rs);
    } else {
#pragma unroll
      for (int d = 0; d < DT; ++d) read_v(vl_cur, vh_cur, 0, d);
      if constexpr (RING) {
        dma(SdpaIdx<1>{});
        if constexpr (NL > 2) dma(SdpaIdx<3>{});
      }
    }
    if constexpr (RING) ld_advance();
    // one pass on: the stage multiplied next is the one after, the stage of this pass is the one the softmax looks back to
    st_cur = st_next;
    k_cur = k_next;
    vl_prev = vl_cur; vh_prev = vh_cur;
    vl_cur = vlp + st_next; vh_cur = vhp + st_next;
  };
  auto skip = [&](int kb) {   // a pass outside this wavefront's interval: its share of the staging only
    sync();
    dma_all();
    st_cur = next_stage(st_cur);
  };

  f32x16 sa, sb;
#pragma unroll
  for (int r = 0; r < 16; ++r) sa[r] = sb[r] = 0.0f;
  {
    for (int i = 0; i < 3; ++i) dma_all();   // the first pass lies in stage 0
  }
  // Q is used here, in front of the loops, so that the wait for its loads stands here (and covers the requests above, whose
  // first passes the first barrier needs anyway): a counted wait for it further down would also wait for the
  // LDS-direct loads issued there, which the compiler does not count, and drain the ring at every step.
#pragma unroll
  for (int s = 0; s < 2 * DT; ++s) asm volatile("" : "+v"(qf[s]));
  int kb = kb_begin;
  for (; kb < w_begin; ++kb) skip(kb);
  if (w_begin < w_end) {
    sync();
    k_cur = kfp + st_cur; vl_cur = vlp + st_cur; vh_cur = vhp + st_cur;
#pragma unroll
    for (int st = 0; st < DT; ++st) read_k(k_cur, st);
    step(SdpaFlag<true>{}, SdpaFlag<false>{}, SdpaFlag<true>{}, kb, sb, sa);   // scores of the first pass into sa
    for (kb = w_begin + 1; kb + 1 < w_end; kb += 2) {
      sync();
      step(SdpaFlag<true>{}, SdpaFlag<true>{}, SdpaFlag<true>{}, kb, sa, sb);
      sync();
      step(SdpaFlag<true>{}, SdpaFlag<true>{}, SdpaFlag<true>{}, kb + 1, sb, sa);
    }
    if (kb < w_end) {
      sync();
      step(SdpaFlag<true>{}, SdpaFlag<true>{}, SdpaFlag<true>{}, kb, sa, sb);
      sa = sb;
      ++kb;
    }
    // kb = w_end: the last pass's softmax and second product; behind the last barrier nothing is requested any more
    // (other wavefronts may still be reading the stage that would be overwritten)
    if (kb < kb_end) {
      sync();
      step(SdpaFlag<false>{}, SdpaFlag<true>{}, SdpaFlag<true>{}, kb, sa, sb);
    } else {
      step(SdpaFlag<false>{}, SdpaFlag<true>{}, SdpaFlag<false>{}, kb, sa, sb);
    }
    for (++kb; kb < kb_end; ++kb) skip(kb);
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  if constexpr (KH == 2) {
  // merge the two key halves of every query tile: the upper half hands over (max, sum) and its output (16 DT values per
  // lane: 256 lanes x 16 DT floats = DT * 16 KiB) through the ring, which nobody reads or fills any more
  __syncthreads();
  float *ml = (float *)(lds + 4 * STAGE);
  f32x4 *ox = (f32x4 *)lds;
  const int slot = qw * 64 + lane;
  if (kh == 1) {
    ml[2 * slot] = m_run; ml[2 * slot + 1] = l_run;
#pragma unroll
    for (int r4 = 0; r4 < 4; ++r4)
#pragma unroll
      for (int d = 0; d < DT; ++d)
        ox[(r4 * DT + d) * 256 + slot] = f32x4{o[d][4 * r4], o[d][4 * r4 + 1], o[d][4 * r4 + 2], o[d][4 * r4 + 3]};
  }
  __syncthreads();
  if (kh == 0) {
    const float m1 = ml[2 * slot], l1 = ml[2 * slot + 1];
    const float m = fmaxf(m_run, m1), m_to = m == -INFINITY ? 0.0f : m;
    const float a0 = __builtin_amdgcn_exp2f(m_run - m_to), a1 = __builtin_amdgcn_exp2f(m1 - m_to);
    l_run = l_run * a0 + l1 * a1;
#pragma unroll
    for (int r4 = 0; r4 < 4; ++r4)
#pragma unroll
      for (int d = 0; d < DT; ++d) {
        const f32x4 x = ox[(r4 * DT + d) * 256 + slot];
#pragma unroll
        for (int e = 0; e < 4; ++e) o[d][4 * r4 + e] = o[d][4 * r4 + e] * a0 + x[e] * a1;
      }
  }
  __syncthreads();   // the next block of the pair fills the ring again
  }
  if (kh != 0 || !wave_ok) return;   // no barrier follows inside this block; the next block starts with one
  const float inv = l_run > 0.0f ? 1.0f / l_run : 0.0f;
  const bool q_ok = q_glob < p.Sq;
#pragma unroll
  for (int d = 0; d < DT; ++d)
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const int din = g * 8 + hh * 4;
      u32x2 ov;
      ov.x = q_ok ? pack_bf16_rne(o[d][g * 4 + 0] * inv, o[d][g * 4 + 1] * inv) : 0u;
      ov.y = q_ok ? pack_bf16_rne(o[d][g * 4 + 2] * inv, o[d][g * 4 + 3] * inv) : 0u;
      uint8_t *op = p.out + o_mat + qt * p.o_pitch + d * 2048 +
                    (((l31 >> 4) * 2 + (din >> 4)) * 256 + (l31 & 15) * 16 + (din & 15)) * 2;
      *(u32x2 *)op = ov;
    }
}

template <int DT, int KH>
__global__ __launch_bounds__(256 * KH) __attribute__((amdgpu_waves_per_eu(2, 2))) void ttm_sdpa_pipe_k(SdpaArgs p, int paired) {
  extern __shared__ u32x4 sdpa_ring[];
  uint8_t *lds = (uint8_t *)sdpa_ring;
  const int nqb = (p.sqt + 3) / 4;
  int x = blockIdx.x, h = blockIdx.y, b = blockIdx.z;
  sdpa_xcd_order(p, x, h, b);
  if constexpr (KH == 1) {
    // One query block per workgroup, two workgroups per CU.  Under a causal mask a block's work grows with its number:
    // the first half of a matrix's workgroups (the first to be placed, one per CU) take the upper blocks from the last
    // down, the second half (placed beside them) the lower blocks from the first up, so that the two that share a CU
    // carry about the same work together wherever the dispatcher keeps to that order; nothing depends on it.
    const int upper = (nqb + 1) / 2;
    sdpa_pipe_block<DT, 1>(p, x < upper ? nqb - 1 - x : x - upper, h, b, lds);
    return;
  }
  const int heavy = nqb - 1 - x, light = x;
  const int parts = paired && light < heavy ? 2 : 1;   // workgroup-uniform
  for (int part = 0; part < parts; ++part) sdpa_pipe_block<DT, KH>(p, part == 0 ? heavy : light, h, b, lds);
}

// Merges the key shares of ttm_sdpa64_split_k: one workgroup per (b, h, query tile).  With M = max_s m_s, every output is
// sum_s o_s 2^(m_s - M) / sum_s l_s 2^(m_s - M); a share that saw no key has m = -inf and weighs nothing; a row without any
// visible key gives zeros, as the single-workgroup path does.
template <int DT>
__global__ __launch_bounds__(256) void ttm_sdpa_combine_k(SdpaArgs p) {
  const int qt = blockIdx.x, h = blockIdx.y, b = blockIdx.z, tid = threadIdx.x;
  const int64_t slots = (int64_t)p.B * p.Hq * p.sqt, slot0 = ((int64_t)b * p.Hq + h) * p.sqt + qt;
  uint8_t *op = p.out + b * p.o_batch + h * p.o_head + qt * p.o_pitch;
  for (int g = tid; g < DT * 256; g += 256) {   // groups of four consecutive columns of one query
    const int d = g >> 8, e = (g & 255) * 4, row = ((e >> 8) >> 1) * 16 + ((e >> 4) & 15);
    float M = -INFINITY;
    for (int ks = 0; ks < p.ksplits; ++ks) M = fmaxf(M, p.part_ml[(slot0 + ks * slots) * 64 + 2 * row]);
    f32x4 num = {0.f, 0.f, 0.f, 0.f};
    float den = 0.0f;
    for (int ks = 0; ks < p.ksplits; ++ks) {
      const int64_t sl = slot0 + ks * slots;
      const float m = p.part_ml[sl * 64 + 2 * row], w = m == -INFINITY ? 0.0f : __builtin_amdgcn_exp2f(m - M);
      den += p.part_ml[sl * 64 + 2 * row + 1] * w;
      num += *(const f32x4 *)(p.part_o + (sl * DT + d) * 1024 + e) * w;
    }
    const float inv = den > 0.0f ? 1.0f / den : 0.0f;
    const bool q_ok = qt * 32 + row < p.Sq;
    u32x2 ov;
    ov.x = q_ok ? pack_bf16_rne(num[0] * inv, num[1] * inv) : 0u;
    ov.y = q_ok ? pack_bf16_rne(num[2] * inv, num[3] * inv) : 0u;
    *(u32x2 *)(op + d * 2048 + e * 2) = ov;
  }
}

static int sdpa_entry(const void *q, const void *k, const void *v, const void *mask, int mask_heads, void *out, int dtype, int64_t B,
                      int64_t Hq, int64_t Hkv, int64_t Sq, int64_t Sk, int64_t D, int is_causal, float scale, int heads_inner, int64_t window,
                      const void *sink, int64_t mask_batch, void *stream) {
  TTM_REQUIRE(dtype == TTM_BF16, "ttm_sdpa: tensors must be BFloat16 (got %d)", dtype);
  TTM_REQUIRE(B >= 0 && Hq >= 0 && Hkv > 0 && Sq >= 0 && Sk >= 0 && D > 0, "ttm_sdpa: bad dimension");
  TTM_REQUIRE(Hq % Hkv == 0, "ttm_sdpa: query heads (%ld) must be a multiple of kv heads (%ld)", (long)Hq, (long)Hkv);
  TTM_REQUIRE(D % 32 == 0 && (D == 32 || D == 64 || D == 128 || D == 256), "ttm_sdpa: head_dim must be 32, 64, 128 or 256 (got %ld)", (long)D);
  TTM_REQUIRE(mask == nullptr || mask_heads == 1 || mask_heads == Hq, "ttm_sdpa: mask heads must be 1 or Hq");
  if (B == 0 || Hq == 0 || Sq == 0) return TTM_OK;
  TTM_REQUIRE(Sk > 0, "ttm_sdpa: empty key sequence");
  TTM_REQUIRE(q && k && v && out, "ttm_sdpa: null pointer");
  TTM_REQUIRE(Hq <= 65535 && B <= 65535, "ttm_sdpa: too many heads or batches");
  SdpaArgs p;
  p.q = (const uint8_t *)q; p.k = (const uint8_t *)k; p.v = (const uint8_t *)v; p.mask = (const uint8_t *)mask;
  p.out = (uint8_t *)out;
  p.B = (int)B; p.Hq = (int)Hq; p.Hkv = (int)Hkv; p.Sq = (int)Sq; p.Sk = (int)Sk;
  p.sqt = (int)ttm_cdiv(Sq, 32); p.skt = (int)ttm_cdiv(Sk, 32);
  TTM_REQUIRE(mask == nullptr || mask_batch == 1 || mask_batch == B, "ttm_sdpa: mask batch must be 1 or B");
  p.mask_heads = mask_heads; p.mask_b = mask_batch == 1 ? 0 : 1;
  if (window >= kNoLimit) window = kNoLimit - 1;   // longer than any sequence: no different from that length
  p.hi_off = is_causal ? 0 : kNoLimit; p.lo_off = kNoLimit;
  if (window >= 0) {   // a causal window holds the last `window` keys, a symmetric one window / 2 keys on either side
    p.lo_off = is_causal ? (int)window - 1 : (int)(window / 2);
    if (!is_causal) p.hi_off = (int)(window / 2);
  }
  p.sink = (const uint8_t *)sink;
  p.scale = scale > 0.0f ? scale : 1.0f / sqrtf((float)D);
  TTM_REQUIRE(heads_inner >= 0 && heads_inner < 16, "ttm_sdpa: unknown layout flags %d", heads_inner);
  auto place = [&](bool inner, int64_t heads, int st, int64_t &pitch, int64_t &head, int64_t &batch) {
    const int64_t dt = D / 32 * 2048;   // bytes of the tiles of one head in one tile row
    if (inner) { pitch = heads * dt; head = dt; batch = st * pitch; }
    else { pitch = dt; head = st * dt; batch = heads * head; }
  };
  place(heads_inner & 1, Hq, p.sqt, p.q_pitch, p.q_head, p.q_batch);
  place(heads_inner & 2, Hkv, p.skt, p.k_pitch, p.k_head, p.k_batch);
  place(heads_inner & 4, Hkv, p.skt, p.v_pitch, p.v_head, p.v_batch);
  place(heads_inner & 8, Hq, p.sqt, p.o_pitch, p.o_head, p.o_batch);
  dim3 grid((unsigned)ttm_cdiv(p.sqt, 4), (unsigned)Hq, (unsigned)B), block(256);
  hipStream_t s = (hipStream_t)stream;
  const int variant = ttm_option("sdpa_variant");   // 1 = 32 keys per pass, 2 = 64 keys without pairing query blocks
  const bool wide = variant != 1;
  const int nqb = (int)ttm_cdiv(p.sqt, 4);
  const int paired = is_causal && nqb >= 2 && variant != 2;
  const dim3 grid64(paired ? (unsigned)((nqb + 1) / 2) : (unsigned)nqb, (unsigned)Hq, (unsigned)B);
  // eight wavefronts per workgroup (two key halves per query tile) when the launch would otherwise leave every SIMD with a
  // single wavefront: no more workgroups than CUs (only one eight-wavefront workgroup fits a CU, so a larger launch would
  // take a second round where the four-wavefront kernel runs two workgroups side by side).  sdpa_variant 3 forces it, 4
  // forbids it, 6 keeps the chained form of it.
  int cus = 0, devid = 0;
  if (hipGetDevice(&devid) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, devid) != hipSuccess || cus <= 0) cus = 256;
  const int64_t wgs = (int64_t)grid64.x * grid64.y * grid64.z;
  // (with 64 or 128 columns the eight-wavefront form is the pipelined kernel, which is the faster one at every launch size:
  // [2, 32 / 8, 4096, 128] causal 293 against 350 us, [1, 32 / 8, 8192, 128] 539 against 665 us)
  const bool split = wide && D <= 128 && (variant == 3 || ((variant == 0 || variant == 6) && wgs <= (int64_t)cus) ||
                                          ((variant == 0 || variant == 7 || variant == 8) && (D == 64 || D == 128)));
  p.ksplits = 1; p.part_o = nullptr; p.part_ml = nullptr;
  if (split) {
    const dim3 block8(512);
    // few workgroups against many keys (not the paired causal launch, whose query blocks carry equal work already): the
    // keys of a query block are shared out until the device is full, at least four 64-key passes per share
    int64_t ks = 1;
    if (!paired && wgs * 2 <= (int64_t)cus && ttm_option("sdpa_variant") != 5) {
      ks = (int64_t)cus / wgs;
      if (ks > p.skt / 8) ks = p.skt / 8;
      if (ks > 16) ks = 16;
      if (ks < 1) ks = 1;
    }
    dim3 g = grid64;
    if (ks > 1) {
      const int64_t slots = (int64_t)B * Hq * p.sqt * ks;
      void *ws = nullptr;
      if (int rc = ttm_stream_workspace(s, (size_t)slots * (D * 32 + 64) * sizeof(float), &ws)) return rc;
      p.ksplits = (int)ks;
      p.part_o = (float *)ws;
      p.part_ml = p.part_o + slots * D * 32;
      g.x = (unsigned)(grid64.x * ks);
    }
    // one workgroup per query block (or pair) and 64 or 128 columns: the pipelined form.  sdpa_variant 6 keeps the chained one.
    // (its ring loads add the distance between two tile rows to a 32-bit lane offset)
    if (ks == 1 && (D == 128 || D == 64) && variant != 6 && p.k_pitch < ((int64_t)1 << 30) && p.v_pitch < ((int64_t)1 << 30)) {
      // The four-wavefront form runs two workgroups per CU side by side, one query block each and 32 keys per pass: the two
      // wavefronts of a SIMD then share no barrier, nothing is merged at the end, and one workgroup's first and last passes
      // overlap the other's middle.  It pays for many short query-block columns (several sequences of up to ~3000 tokens,
      // 128 columns: [2..8, 32 / 8, 2048, 128] causal 5..13 % faster, [1, 32 / 8, 3000, 128] 12 %); a single sequence of 2048
      // tokens has only two blocks per CU, of very different length, and is 8 % slower that way, 4096 tokens 4 % slower,
      // 8192 the same.  sdpa_variant 7 forces it, 8 keeps the eight-wavefront form.
      const int64_t blocks = (int64_t)nqb * Hq * B;
      const bool four = variant == 7 || (variant == 0 && D == 128 && blocks >= 3 * (int64_t)cus && nqb <= 24);
      const int ring = (int)D / 32 * (four ? 20480 : 40960);   // five stages of 32 or 64 keys of K and V
      const void *fn = four ? (D == 128 ? (const void *)ttm_sdpa_pipe_k<4, 1> : (const void *)ttm_sdpa_pipe_k<2, 1>)
                            : (D == 128 ? (const void *)ttm_sdpa_pipe_k<4, 2> : (const void *)ttm_sdpa_pipe_k<2, 2>);
      hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, ring);
      if (e != hipSuccess) return ttm_set_error(TTM_ERR_HIP, "hipFuncSetAttribute(LDS %d): %s", ring, hipGetErrorString(e));
      if (four) {
        const dim3 g4((unsigned)nqb, (unsigned)Hq, (unsigned)B);
        if (D == 128) hipLaunchKernelGGL((ttm_sdpa_pipe_k<4, 1>), g4, dim3(256), ring, s, p, 0);
        else hipLaunchKernelGGL((ttm_sdpa_pipe_k<2, 1>), g4, dim3(256), ring, s, p, 0);
      } else if (D == 128) hipLaunchKernelGGL((ttm_sdpa_pipe_k<4, 2>), g, block8, ring, s, p, paired);
      else hipLaunchKernelGGL((ttm_sdpa_pipe_k<2, 2>), g, block8, ring, s, p, paired);
      TTM_LAUNCH_CHECK();
      return TTM_OK;
    }
    switch (D) {
    case 32: hipLaunchKernelGGL(ttm_sdpa64_split_k<1>, g, block8, 0, s, p, paired); break;
    case 64: hipLaunchKernelGGL(ttm_sdpa64_split_k<2>, g, block8, 0, s, p, paired); break;
    default: hipLaunchKernelGGL(ttm_sdpa64_split_k<4>, g, block8, 0, s, p, paired); break;
    }
    TTM_LAUNCH_CHECK();
    if (ks > 1) {
      const dim3 cg((unsigned)p.sqt, (unsigned)Hq, (unsigned)B);
      switch (D) {
      case 32: hipLaunchKernelGGL(ttm_sdpa_combine_k<1>, cg, dim3(256), 0, s, p); break;
      case 64: hipLaunchKernelGGL(ttm_sdpa_combine_k<2>, cg, dim3(256), 0, s, p); break;
      default: hipLaunchKernelGGL(ttm_sdpa_combine_k<4>, cg, dim3(256), 0, s, p); break;
      }
      TTM_LAUNCH_CHECK();
    }
    return TTM_OK;
  }
  switch (D) {
  case 32: if (wide) hipLaunchKernelGGL(ttm_sdpa64_k<1>, grid64, block, 0, s, p, paired); else hipLaunchKernelGGL(ttm_sdpa_k<1>, grid, block, 0, s, p); break;
  case 64: if (wide) hipLaunchKernelGGL(ttm_sdpa64_k<2>, grid64, block, 0, s, p, paired); else hipLaunchKernelGGL(ttm_sdpa_k<2>, grid, block, 0, s, p); break;
  case 128: if (wide) hipLaunchKernelGGL(ttm_sdpa64_k<4>, grid64, block, 0, s, p, paired); else hipLaunchKernelGGL(ttm_sdpa_k<4>, grid, block, 0, s, p); break;
  default: hipLaunchKernelGGL(ttm_sdpa_k<8>, grid, block, 0, s, p); break;   // 256 columns: the 64-key staging would not fit in LDS
  }
  TTM_LAUNCH_CHECK();
  return TTM_OK;
}

TTM_EXPORT int ttm_sdpa(const void *q, const void *k, const void *v, const void *mask, int mask_heads, void *out,
                        int dtype, int64_t B, int64_t Hq, int64_t Hkv, int64_t Sq, int64_t Sk, int64_t D,
                        int is_causal, float scale, void *stream) {
  TTM_EXTENTS(sdpa, q, k, v, mask, mask_heads, B, out, dtype, B, Hq, Hkv, Sq, Sk, D, nullptr);
  return sdpa_entry(q, k, v, mask, mask_heads, out, dtype, B, Hq, Hkv, Sq, Sk, D, is_causal, scale, 0, -1, nullptr, B, stream);
}

TTM_EXPORT int ttm_sdpa_heads_inner(const void *q, const void *k, const void *v, const void *mask, int mask_heads, void *out,
                                    int dtype, int64_t B, int64_t Hq, int64_t Hkv, int64_t Sq, int64_t Sk, int64_t D,
                                    int is_causal, float scale, int heads_inner, void *stream) {
  TTM_EXTENTS(sdpa, q, k, v, mask, mask_heads, B, out, dtype, B, Hq, Hkv, Sq, Sk, D, nullptr);
  return sdpa_entry(q, k, v, mask, mask_heads, out, dtype, B, Hq, Hkv, Sq, Sk, D, is_causal, scale, heads_inner, -1, nullptr, B, stream);
}

TTM_EXPORT int ttm_sdpa_windowed(const void *q, const void *k, const void *v, const void *mask, int mask_heads, int64_t mask_batch, void *out,
                                 int dtype, int64_t B, int64_t Hq, int64_t Hkv, int64_t Sq, int64_t Sk, int64_t D,
                                 int is_causal, float scale, int heads_inner, int64_t sliding_window, const void *attention_sink,
                                 void *stream) {
  TTM_EXTENTS(sdpa, q, k, v, mask, mask_heads, mask_batch, out, dtype, B, Hq, Hkv, Sq, Sk, D, attention_sink);
  return sdpa_entry(q, k, v, mask, mask_heads, out, dtype, B, Hq, Hkv, Sq, Sk, D, is_causal, scale, heads_inner,
                    sliding_window < 0 ? -1 : sliding_window, attention_sink, mask_batch, stream);
}
