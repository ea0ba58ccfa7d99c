// Row-wise bandwidth kernels on tile-ordered tensors: RMSNorm, softmax and reductions over the
// last dimension.  A workgroup owns RPB = 32 or 8 rows of one tile row (32 logical rows x all columns,
// one contiguous run of tiles in memory); 8 rows per workgroup are used when whole tile rows would
// leave most CUs without work.  Thread (r = tid % RPB, j = tid / RPB) walks the chunks of row r with
// stride 256 / RPB; the lanes of a step read whole face rows, so global accesses are contiguous runs
// of at least 256 bytes.  Partial results of the lanes of a row meet in LDS.  Math is fp32; columns beyond
// the logical width are masked with the operation's identity, rows beyond the logical height are
// written as zeros.
#include "ttm_common.h"
#include "ttm_math.h"

enum { RW_RMSNORM = 0, RW_SOFTMAX = 1, RW_SUM = 2, RW_MEAN = 3, RW_MAX = 4, RW_MIN = 5 };

struct RowArgs {
  const void *x;
  void *out;
  const void *w, *b;   // rmsnorm weight / bias (same dtype as x) or null
  int w_tiled, b_tiled;
  int64_t rows, cols;  // logical extent of the last two dims
  int rt, ct;          // tiles per batch entry
  float eps;
  int out_ct;          // reductions: column tiles of the output (1), keepdim layout [.., rows, 1]
  // ttm_rowwise_row_k<.., PRE = true>: x is not read but made on the way in from the fp32 partial sums of a split-K
  // projection of one row tile, x = bf16(bf16(sum over slices) + residual), and also stored to sum_out
  const float *partial;
  int slices;
  int64_t per;         // floats per slice
  const void *residual;
  void *sum_out;
};

template <int ELEM>
struct ChunkPos {  // chunk q of row r inside a tile row
  int64_t off;     // element offset from the start of the tile row
  int c0;          // logical column of the chunk's first element
};
template <int ELEM>
__device__ __forceinline__ ChunkPos<ELEM> chunk_pos(int r, int q) {
  constexpr int EPC = 16 / ELEM;
  int tile = q / (2 * ELEM), fx = (q % (2 * ELEM)) / ELEM, part = q % ELEM;
  ChunkPos<ELEM> p;
  p.off = (int64_t)tile * 1024 + ((r >> 4) * 2 + fx) * 256 + (r & 15) * 16 + part * EPC;
  p.c0 = tile * 32 + fx * 16 + part * EPC;
  return p;
}

template <int ELEM>
__device__ __forceinline__ void unpack_vals(u32x4 v, float (&f)[16 / ELEM]) {
  if (ELEM == 2) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      f[2 * i] = __uint_as_float(v[i] << 16);
      f[2 * i + 1] = __uint_as_float(v[i] & 0xFFFF0000u);
    }
  } else {
#pragma unroll
    for (int i = 0; i < 4; ++i) f[i] = __uint_as_float(v[i]);
  }
}
template <int ELEM>
__device__ __forceinline__ void load_vals(const void *base, int64_t off, float (&f)[16 / ELEM]) {
  u32x4 v = *(const u32x4 *)((const uint8_t *)base + off * ELEM);
  if (ELEM == 2) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      f[2 * i] = __uint_as_float(v[i] << 16);
      f[2 * i + 1] = __uint_as_float(v[i] & 0xFFFF0000u);
    }
  } else {
#pragma unroll
    for (int i = 0; i < 4; ++i) f[i] = __uint_as_float(v[i]);
  }
}
template <int ELEM>
__device__ __forceinline__ void store_vals(void *base, int64_t off, const float (&f)[16 / ELEM]) {
  u32x4 v;
  if (ELEM == 2) {
#pragma unroll
    for (int i = 0; i < 4; ++i) v[i] = ttm_pack_bf16x2(f[2 * i], f[2 * i + 1]);
  } else {
#pragma unroll
    for (int i = 0; i < 4; ++i) v[i] = __float_as_uint(f[i]);
  }
  *(u32x4 *)((uint8_t *)base + off * ELEM) = v;
}

// weight / bias vector element c: tiled [1, C] tensor (row 0 of a 32-row tile) or plain [C]
template <int ELEM>
__device__ __forceinline__ void load_vec(const void *v, int tiled, int c0, float (&f)[16 / ELEM]) {
  int64_t off = tiled ? (int64_t)(c0 >> 5) * 1024 + ((c0 >> 4) & 1) * 256 + (c0 & 15) : c0;
  load_vals<ELEM>(v, off, f);
}

template <int MODE, int ELEM, int RPB>
__global__ __launch_bounds__(256) void ttm_rowwise_k(RowArgs p) {
  constexpr int EPC = 16 / ELEM;
  constexpr int J = 256 / RPB;                           // lanes per row
  __shared__ float part[J][RPB];
  __shared__ float part2[J][RPB];
  const int tid = threadIdx.x, j = tid / RPB;
  const int r = (int)(blockIdx.x % (32 / RPB)) * RPB + tid % RPB;   // row inside the tile row
  const int rl = tid % RPB;
  const int64_t trow = blockIdx.x / (32 / RPB);          // tile row over all batch entries
  const int64_t row = (trow % p.rt) * 32 + r;            // logical row inside the batch entry
  const bool row_ok = row < p.rows;
  const int nq = p.ct * 2 * ELEM;                        // chunks per row
  const uint8_t *x = (const uint8_t *)p.x + trow * p.ct * 1024 * ELEM;
  const int cols = (int)p.cols;

  constexpr bool IS_MAX = MODE == RW_SOFTMAX || MODE == RW_MAX;
  float acc = IS_MAX ? -INFINITY : (MODE == RW_MIN ? INFINITY : 0.0f);
  #pragma unroll 4
  for (int q = j; q < nq; q += J) {
    ChunkPos<ELEM> cp = chunk_pos<ELEM>(r, q);
    float f[EPC];
    load_vals<ELEM>(x, cp.off, f);
#pragma unroll
    for (int i = 0; i < EPC; ++i) {
      bool ok = cp.c0 + i < cols;
      if (MODE == RW_RMSNORM) acc += ok ? f[i] * f[i] : 0.0f;
      else if (IS_MAX) acc = ok ? ttm_max(acc, f[i]) : acc;
      else if (MODE == RW_MIN) acc = ok ? ttm_min(acc, f[i]) : acc;
      else acc += ok ? f[i] : 0.0f;
    }
  }
  part[j][rl] = acc;
  __syncthreads();
  float stat = part[0][rl];
#pragma unroll
  for (int k = 1; k < J; ++k) {
    float o = part[k][rl];
    stat = IS_MAX ? ttm_max(stat, o) : (MODE == RW_MIN ? ttm_min(stat, o) : stat + o);
  }

  if (MODE == RW_SUM || MODE == RW_MEAN || MODE == RW_MAX || MODE == RW_MIN) {
    // output [.., rows, 1] in tile order: one column tile per tile row; zero padded
    if (MODE == RW_MEAN) stat = stat / (float)cols;
    uint8_t *o = (uint8_t *)p.out + trow * 1024 * ELEM;
    // the lanes clear the block's rows of the tile (both faces), then column 0 is written
    for (int e = tid; e < RPB * 2 * (16 * ELEM / 16); e += 256) {
      const int rr = (int)(blockIdx.x % (32 / RPB)) * RPB + e / (2 * ELEM), fx = (e / ELEM) & 1, part_i = e % ELEM;
      ((u32x4 *)o)[(((rr >> 4) * 2 + fx) * 256 + (rr & 15) * 16) * ELEM / 16 + part_i] = u32x4{0, 0, 0, 0};
    }
    __syncthreads();
    if (j == 0 && row_ok) {
      int64_t off = ((r >> 4) * 2) * 256 + (r & 15) * 16;
      if (ELEM == 2) ((uint16_t *)o)[off] = ttm_f32_to_bf16(stat);
      else ((float *)o)[off] = stat;
    }
    return;
  }

  uint8_t *o = (uint8_t *)p.out + trow * p.ct * 1024 * ELEM;
  if (MODE == RW_RMSNORM) {
    const float rs = 1.0f / sqrtf(stat / (float)cols + p.eps);
    #pragma unroll 4
  for (int q = j; q < nq; q += J) {
      ChunkPos<ELEM> cp = chunk_pos<ELEM>(r, q);
      float f[EPC], w[EPC], b[EPC];
      load_vals<ELEM>(x, cp.off, f);
      if (p.w) load_vec<ELEM>(p.w, p.w_tiled, cp.c0, w);
      if (p.b) load_vec<ELEM>(p.b, p.b_tiled, cp.c0, b);
#pragma unroll
      for (int i = 0; i < EPC; ++i) {
        float v = f[i] * rs;
        if (p.w) v *= w[i];
        if (p.b) v += b[i];
        f[i] = (row_ok && cp.c0 + i < cols) ? v : 0.0f;
      }
      store_vals<ELEM>(o, cp.off, f);
    }
  } else {  // softmax: second pass for the sum of exponentials, third pass writes
    const float mx = stat;
    float sum = 0.0f;
    #pragma unroll 4
  for (int q = j; q < nq; q += J) {
      ChunkPos<ELEM> cp = chunk_pos<ELEM>(r, q);
      float f[EPC];
      load_vals<ELEM>(x, cp.off, f);
#pragma unroll
      for (int i = 0; i < EPC; ++i) sum += cp.c0 + i < cols ? expf(f[i] - mx) : 0.0f;
    }
    part2[j][rl] = sum;
    __syncthreads();
    float tot = 0.0f;
#pragma unroll
    for (int k = 0; k < J; ++k) tot += part2[k][rl];
    const float inv = 1.0f / tot;
    #pragma unroll 4
  for (int q = j; q < nq; q += J) {
      ChunkPos<ELEM> cp = chunk_pos<ELEM>(r, q);
      float f[EPC];
      load_vals<ELEM>(x, cp.off, f);
#pragma unroll
      for (int i = 0; i < EPC; ++i) f[i] = (row_ok && cp.c0 + i < cols) ? expf(f[i] - mx) * inv : 0.0f;
      store_vals<ELEM>(o, cp.off, f);
    }
  }
}

// RMSNorm / softmax for rows of up to 16 chunks per lane (4096 bf16 or 2048 fp32 columns): 8 rows per workgroup,
// 32 lanes per row.  The row slice of a lane is read from global memory once and parked in LDS (64 KiB per
// workgroup, each lane reads back only what it wrote, so no barrier is involved) for the output pass.  The loops
// are kept rolled (8 loads in flight per lane): fully unrolled, the once-executed code ran at instruction-fetch speed.
template <int MODE, int ELEM>
__global__ __launch_bounds__(256) void ttm_rowwise_resident_k(RowArgs p) {
  constexpr int EPC = 16 / ELEM, RPB = 8, J = 32, NQ = 16;
  __shared__ u32x4 park[NQ * 256];
  __shared__ float part[J][RPB];
  __shared__ float part2[J][RPB];
  const int tid = threadIdx.x, j = tid / RPB, rl = tid % RPB;
  const int r = (int)(blockIdx.x % 4) * RPB + rl;
  const int trow = (int)(blockIdx.x / 4);
  const int row = (trow % p.rt) * 32 + r;
  const bool row_ok = row < p.rows;
  const int nq = p.ct * 2 * ELEM;
  const uint8_t *x = (const uint8_t *)p.x + (int64_t)trow * p.ct * 1024 * ELEM;
  uint8_t *o = (uint8_t *)p.out + (int64_t)trow * p.ct * 1024 * ELEM;
  const int cols = (int)p.cols;
  const int nk = (nq - j + J - 1) / J;   // chunks of this lane
  float acc = MODE == RW_SOFTMAX ? -INFINITY : 0.0f;
#pragma unroll 8
  for (int k = 0; k < nk; ++k) {
    const ChunkPos<ELEM> cp = chunk_pos<ELEM>(r, j + k * J);
    const u32x4 v = *(const u32x4 *)(x + cp.off * ELEM);
    park[k * 256 + tid] = v;
    float f[EPC];
    unpack_vals<ELEM>(v, f);
#pragma unroll
    for (int i = 0; i < EPC; ++i) {
      const bool ok = cp.c0 + i < cols;
      if (MODE == RW_RMSNORM) acc += ok ? f[i] * f[i] : 0.0f;
      else acc = ok ? ttm_max(acc, f[i]) : acc;
    }
  }
  part[j][rl] = acc;
  __syncthreads();
  float stat = part[0][rl];
#pragma unroll
  for (int k = 1; k < J; ++k) stat = MODE == RW_SOFTMAX ? ttm_max(stat, part[k][rl]) : stat + part[k][rl];
  float mul = 0.0f;
  if (MODE == RW_RMSNORM) mul = 1.0f / sqrtf(stat / (float)cols + p.eps);
  else {
    float sum = 0.0f;
#pragma unroll 4
    for (int k = 0; k < nk; ++k) {
      const int c0 = chunk_pos<ELEM>(r, j + k * J).c0;
      float f[EPC];
      unpack_vals<ELEM>(park[k * 256 + tid], f);
#pragma unroll
      for (int i = 0; i < EPC; ++i) sum += c0 + i < cols ? expf(f[i] - stat) : 0.0f;
    }
    part2[j][rl] = sum;
    __syncthreads();
    float tot = 0.0f;
#pragma unroll
    for (int k = 0; k < J; ++k) tot += part2[k][rl];
    mul = 1.0f / tot;
  }
#pragma unroll 4
  for (int k = 0; k < nk; ++k) {
    const ChunkPos<ELEM> cp = chunk_pos<ELEM>(r, j + k * J);
    float f[EPC], w[EPC], b[EPC];
    unpack_vals<ELEM>(park[k * 256 + tid], f);
    if (MODE == RW_RMSNORM) {
      if (p.w) load_vec<ELEM>(p.w, p.w_tiled, cp.c0, w);
      if (p.b) load_vec<ELEM>(p.b, p.b_tiled, cp.c0, b);
    }
#pragma unroll
    for (int i = 0; i < EPC; ++i) {
      float v;
      if (MODE == RW_RMSNORM) {
        v = f[i] * mul;
        if (p.w) v *= w[i];
        if (p.b) v += b[i];
      } else {
        v = expf(f[i] - stat) * mul;
      }
      f[i] = (row_ok && cp.c0 + i < cols) ? v : 0.0f;
    }
    store_vals<ELEM>(o, cp.off, f);
  }
}

// RMSNorm / softmax with one row per workgroup, for rows of up to NK = 2, 4 or 8 chunks per lane (at most 16384 bf16 or
// 8192 fp32 columns).
// The row stays in registers between the reduction and the output pass, weights are fetched while the reduction is in
// flight, and a workgroup issues all its loads at once: a [32, 4096] input is 32 short workgroups instead of 4 long ones.
// Consecutive rows of a face share 128-byte lines, so the row -> workgroup map gives every XCD (workgroup id mod 8)
// a contiguous range of rows and its L2 sees each line of that range whole.
template <int MODE, int ELEM, int NK, bool PRE = false>
__global__ __launch_bounds__(256) void ttm_rowwise_row_k(RowArgs p, int total_rows) {
  constexpr int EPC = 16 / ELEM;
  __shared__ float red[4], red2[4];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int per_xcd = total_rows / 8;                    // total_rows is a multiple of 32
  const int lrow = (int)(blockIdx.x % 8) * per_xcd + (int)(blockIdx.x / 8);
  const int r = lrow & 31, trow = lrow >> 5;
  const int row = (trow % p.rt) * 32 + r;
  const bool row_ok = row < p.rows;
  const int nq = p.ct * 2 * ELEM, cols = (int)p.cols;
  const uint8_t *x = (const uint8_t *)p.x + (int64_t)trow * p.ct * 1024 * ELEM;
  uint8_t *o = (uint8_t *)p.out + (int64_t)trow * p.ct * 1024 * ELEM;
  u32x4 v[NK];
#pragma unroll
  for (int k = 0; k < NK; ++k) {
    const int q = tid + k * 256;
    v[k] = u32x4{0, 0, 0, 0};
    if constexpr (PRE) {   // bf16 rows made from partial sums: the projection's rounding, then the residual add's
      static_assert(!PRE || ELEM == 2, "partial sums finish as bf16");
      if (q < nq) {
        const int64_t off = chunk_pos<ELEM>(r, q).off;
        if (row_ok) {
          f32x4 s0 = *(const f32x4 *)(p.partial + off), s1 = *(const f32x4 *)(p.partial + off + 4);
          for (int sl = 1; sl < p.slices; ++sl) {
            s0 += *(const f32x4 *)(p.partial + sl * p.per + off);
            s1 += *(const f32x4 *)(p.partial + sl * p.per + off + 4);
          }
          const u32x4 y = {ttm_pack_bf16x2(s0.x, s0.y), ttm_pack_bf16x2(s0.z, s0.w), ttm_pack_bf16x2(s1.x, s1.y), ttm_pack_bf16x2(s1.z, s1.w)};
          const u32x4 t = *(const u32x4 *)((const uint8_t *)p.residual + off * 2);
#pragma unroll
          for (int i = 0; i < 4; ++i)
            v[k][i] = ttm_pack_bf16x2(__uint_as_float(y[i] << 16) + __uint_as_float(t[i] << 16),
                                      __uint_as_float(y[i] & 0xFFFF0000u) + __uint_as_float(t[i] & 0xFFFF0000u));
        }
        *(u32x4 *)((uint8_t *)p.sum_out + off * 2) = v[k];
      }
    } else if (q < nq && row_ok) v[k] = *(const u32x4 *)(x + chunk_pos<ELEM>(r, q).off * ELEM);
  }
  u32x4 wraw[NK], braw[NK];   // weight / bias chunks, still packed
  if (MODE == RW_RMSNORM) {
#pragma unroll
    for (int k = 0; k < NK; ++k) {
      const int q = tid + k * 256;
      if (q < nq) {
        const int c0 = chunk_pos<ELEM>(r, q).c0;
        const int64_t tiled = (int64_t)(c0 >> 5) * 1024 + ((c0 >> 4) & 1) * 256 + (c0 & 15);
        if (p.w) wraw[k] = *(const u32x4 *)((const uint8_t *)p.w + (p.w_tiled ? tiled : c0) * ELEM);
        if (p.b) braw[k] = *(const u32x4 *)((const uint8_t *)p.b + (p.b_tiled ? tiled : c0) * ELEM);
      }
    }
  }
  float acc = MODE == RW_SOFTMAX ? -INFINITY : 0.0f;
#pragma unroll
  for (int k = 0; k < NK; ++k) {
    const int q = tid + k * 256;
    if (q < nq) {
      const int c0 = chunk_pos<ELEM>(r, q).c0;
      float f[EPC];
      unpack_vals<ELEM>(v[k], f);
#pragma unroll
      for (int i = 0; i < EPC; ++i) {
        const bool ok = c0 + i < cols;
        if (MODE == RW_RMSNORM) acc += ok ? f[i] * f[i] : 0.0f;
        else acc = ok ? ttm_max(acc, f[i]) : acc;
      }
    }
  }
#pragma unroll
  for (int s = 32; s > 0; s >>= 1) acc = MODE == RW_SOFTMAX ? ttm_max(acc, __shfl_xor(acc, s)) : acc + __shfl_xor(acc, s);
  if (lane == 0) red[wave] = acc;
  __syncthreads();
  const float stat = MODE == RW_SOFTMAX ? ttm_max(ttm_max(red[0], red[1]), ttm_max(red[2], red[3])) : red[0] + red[1] + red[2] + red[3];
  float mul;
  if (MODE == RW_RMSNORM) {
    mul = 1.0f / sqrtf(stat / (float)cols + p.eps);
  } else {
    float sum = 0.0f;
#pragma unroll
    for (int k = 0; k < NK; ++k) {
      const int q = tid + k * 256;
      if (q < nq) {
        const int c0 = chunk_pos<ELEM>(r, q).c0;
        float f[EPC];
        unpack_vals<ELEM>(v[k], f);
#pragma unroll
        for (int i = 0; i < EPC; ++i) sum += c0 + i < cols ? expf(f[i] - stat) : 0.0f;
      }
    }
#pragma unroll
    for (int s = 32; s > 0; s >>= 1) sum += __shfl_xor(sum, s);
    if (lane == 0) red2[wave] = sum;
    __syncthreads();
    mul = 1.0f / (red2[0] + red2[1] + red2[2] + red2[3]);
  }
#pragma unroll
  for (int k = 0; k < NK; ++k) {
    const int q = tid + k * 256;
    if (q < nq) {
      const ChunkPos<ELEM> cp = chunk_pos<ELEM>(r, q);
      float f[EPC], w[EPC], b[EPC];
      unpack_vals<ELEM>(v[k], f);
      if (MODE == RW_RMSNORM) {
        if (p.w) unpack_vals<ELEM>(wraw[k], w);
        if (p.b) unpack_vals<ELEM>(braw[k], b);
      }
#pragma unroll
      for (int i = 0; i < EPC; ++i) {
        float y;
        if (MODE == RW_RMSNORM) {
          y = f[i] * mul;
          if (p.w) y *= w[i];
          if (p.b) y += b[i];
        } else {
          y = expf(f[i] - stat) * mul;
        }
        f[i] = (row_ok && cp.c0 + i < cols) ? y : 0.0f;
      }
      store_vals<ELEM>(o, cp.off, f);
    }
  }
}

// All six modes with four consecutive rows per workgroup, for large row counts.  Four rows of a face are one run of whole
// 128-byte lines (128 bytes of bf16, 256 of fp32) in every tile, so a workgroup reads and writes nothing but whole lines
// that no other workgroup touches; consecutive lanes take consecutive 16-byte chunks of those runs.  A lane keeps its NK
// chunks (the same row in each: 256 is a multiple of the chunks per run) in registers from the single read to the write,
// and every load of the workgroup is in flight before the first use: 4 KiB x NK per workgroup, which is what keeps HBM
// busy when each workgroup lives only a few microseconds.  Row statistics: shuffles over the lanes of a wavefront that
// hold the same row, then four values per row through LDS.
#ifndef TTM_BAND_EXP
#define TTM_BAND_EXP expf
#endif
// Workgroups per CU by mode and band size (NK x 4 KiB per workgroup), measured at 65536 rows: reductions 4 at 16 KiB
// (44 -> 40 us for 1024 fp32 columns) and 3 from 32 KiB up (89 -> 82 us for 2048); fp32 softmax 4 at 16 KiB (94 -> 88 us)
// and 2 from 32 KiB up (195 -> 185 us); RMSNorm 3 at 16 KiB (96 -> 90 us); everything else runs best without a cap.
template <int MODE, int ELEM, int NK>
constexpr int band_max_waves() {
  if (MODE == RW_SUM || MODE == RW_MEAN || MODE == RW_MAX || MODE == RW_MIN) return NK == 4 ? 4 : (NK >= 8 ? 3 : 8);
  if (MODE == RW_SOFTMAX && ELEM == 4) return NK == 4 ? 4 : (NK >= 8 ? 2 : 8);
  if (MODE == RW_RMSNORM) return NK == 4 ? 3 : 8;
  return 8;
}
// NT = 512 lanes take bands of up to 32 chunks per 256 lanes (16384 bf16 or 8192 fp32 columns) with sixteen chunks per lane:
// one such workgroup per CU (128 KiB).
template <int MODE, int ELEM, int NK, int NT = 256>
__global__ __launch_bounds__(NT) TTM_MAX_WAVES((NT == 512 ? 2 : band_max_waves<MODE, ELEM, NK>())) void ttm_rowwise_band_k(RowArgs p) {
  constexpr int EPC = 16 / ELEM, RUN = 4 * ELEM;         // chunks per run of four face rows
  constexpr bool IS_MAX = MODE == RW_SOFTMAX || MODE == RW_MAX;
  constexpr bool REDUCE = MODE == RW_SUM || MODE == RW_MEAN || MODE == RW_MAX || MODE == RW_MIN;
  constexpr int NW = NT / 64;
  __shared__ float red[NW][4], red2[NW][4];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int g4 = (int)(blockIdx.x & 7);                  // group of four rows inside the tile row
  const int64_t trow = blockIdx.x >> 3;                  // tile row over all batch entries
  const int rl = (tid % RUN) / ELEM, part = tid % ELEM;
  const int r = g4 * 4 + rl;
  const int64_t row = (trow % p.rt) * 32 + r;
  const bool row_ok = row < p.rows;
  const int nruns = p.ct * 2, cols = (int)p.cols;        // runs per band: one per (tile, face column)
  const uint8_t *x = (const uint8_t *)p.x + trow * p.ct * 1024 * ELEM;
  // chunk k of this lane: run tid / RUN + k * (NT / RUN)
  auto run_of = [&](int k) { return tid / RUN + k * (NT / RUN); };
  auto off_of = [&](int run) { return (int64_t)(run >> 1) * 1024 + ((r >> 4) * 2 + (run & 1)) * 256 + (r & 15) * 16 + part * EPC; };
  auto col_of = [&](int run) { return (run >> 1) * 32 + (run & 1) * 16 + part * EPC; };
  u32x4 v[NK];
#pragma unroll
  for (int k = 0; k < NK; ++k) {
    // unconditional (a run past the end repeats the last one and is masked where it is used): a branch around a load
    // makes the compiler wait for each load before it issues the next
    const int run = min(run_of(k), nruns - 1);
    v[k] = __builtin_nontemporal_load((const u32x4 *)(x + off_of(run) * ELEM));
  }
  // RMSNorm: the weight and bias chunks of this lane's columns.  Up to eight chunks per lane they are loaded up front, beside
  // the input; with sixteen that would take every register of a SIMD for a single wavefront (measured 3.2 TB/s at 8192 bf16
  // columns), so there they are loaded four chunks at a time where they are used (they come from the L2: every row shares them)
  constexpr bool WB_EARLY = MODE == RW_RMSNORM && NK <= 8;
  auto wb_load = [&](int k, u32x4 &wv, u32x4 &bv) {
    const int c0 = col_of(min(run_of(k), nruns - 1));
    const int64_t tiled = (int64_t)(c0 >> 5) * 1024 + ((c0 >> 4) & 1) * 256 + (c0 & 15);
    // a null vector reads the input instead (the value is not used): no branch around the loads
    const uint8_t *wsrc = p.w ? (const uint8_t *)p.w + (p.w_tiled ? tiled : c0) * ELEM : x;
    const uint8_t *bsrc = p.b ? (const uint8_t *)p.b + (p.b_tiled ? tiled : c0) * ELEM : x;
    wv = *(const u32x4 *)wsrc;
    bv = *(const u32x4 *)bsrc;
  };
  u32x4 wraw[WB_EARLY ? NK : 1], braw[WB_EARLY ? NK : 1];
  if constexpr (WB_EARLY) {
#pragma unroll
    for (int k = 0; k < NK; ++k) wb_load(k, wraw[k], braw[k]);
  }
  // the lanes of a wavefront that share a row differ in the chunk-part bits (below ELEM) and the run bits (RUN and up)
  auto wave_combine = [&](float a, bool is_max, bool is_min) {
#pragma unroll
    for (int sft = 1; sft < 64; sft <<= 1) {
      if (sft >= ELEM && sft < RUN) continue;            // the row bits
      const float o = __shfl_xor(a, sft);
      a = is_max ? ttm_max(a, o) : (is_min ? ttm_min(a, o) : a + o);
    }
    return a;
  };
  float acc = IS_MAX ? -INFINITY : (MODE == RW_MIN ? INFINITY : 0.0f);
#pragma unroll
  for (int k = 0; k < NK; ++k) {
    const int run = run_of(k);
    const int c0 = col_of(run);
    const int lim = run < nruns ? cols : 0;
    float f[EPC];
    unpack_vals<ELEM>(v[k], f);
#pragma unroll
    for (int i = 0; i < EPC; ++i) {
      const bool ok = c0 + i < lim;
      if (MODE == RW_RMSNORM) acc += ok ? f[i] * f[i] : 0.0f;
      else if (IS_MAX) acc = ok ? ttm_max(acc, f[i]) : acc;
      else if (MODE == RW_MIN) acc = ok ? ttm_min(acc, f[i]) : acc;
      else acc += ok ? f[i] : 0.0f;
    }
  }
  acc = wave_combine(acc, IS_MAX, MODE == RW_MIN);
  if ((lane & ~(RUN - ELEM)) == 0) red[wave][rl] = acc;  // one lane per row and wavefront
  __syncthreads();
  float stat;
  {
    auto four = [&](int w0) {
      const float a0 = red[w0][rl], a1 = red[w0 + 1][rl], a2 = red[w0 + 2][rl], a3 = red[w0 + 3][rl];
      return IS_MAX ? ttm_max(ttm_max(a0, a1), ttm_max(a2, a3)) : (MODE == RW_MIN ? ttm_min(ttm_min(a0, a1), ttm_min(a2, a3)) : (a0 + a1) + (a2 + a3));
    };
    stat = four(0);
    if constexpr (NW == 8) {
      const float hi = four(4);
      stat = IS_MAX ? ttm_max(stat, hi) : (MODE == RW_MIN ? ttm_min(stat, hi) : stat + hi);
    }
  }
  if constexpr (REDUCE) {
    // output [.., rows, 1] in tile order: one column tile per tile row; this workgroup owns its four rows of it, both faces
    if (MODE == RW_MEAN) stat = stat / (float)cols;
    if (tid < 2 * RUN) {
      const int fx = tid / RUN;
      u32x4 z = u32x4{0, 0, 0, 0};
      if (fx == 0 && part == 0 && row_ok) z.x = ELEM == 2 ? (uint32_t)ttm_f32_to_bf16(stat) : __float_as_uint(stat);
      uint8_t *o = (uint8_t *)p.out + trow * 1024 * ELEM;
      *(u32x4 *)(o + (int64_t)(((r >> 4) * 2 + fx) * 256 + (r & 15) * 16 + part * EPC) * ELEM) = z;
    }
    return;
  } else {
    uint8_t *o = (uint8_t *)p.out + trow * p.ct * 1024 * ELEM;
    float mul;
    float e[MODE == RW_SOFTMAX ? NK : 1][EPC];
    if constexpr (MODE == RW_RMSNORM) {
      mul = 1.0f / sqrtf(stat / (float)cols + p.eps);
    } else {
      float sum = 0.0f;
#pragma unroll
      for (int k = 0; k < NK; ++k) {
        const int run = run_of(k);
        const int c0 = col_of(run);
        float f[EPC];
        unpack_vals<ELEM>(v[k], f);
#pragma unroll
        for (int i = 0; i < EPC; ++i) {
          e[k][i] = (run < nruns && c0 + i < cols) ? TTM_BAND_EXP(f[i] - stat) : 0.0f;
          sum += e[k][i];
        }
      }
      sum = wave_combine(sum, false, false);
      if ((lane & ~(RUN - ELEM)) == 0) red2[wave][rl] = sum;
      __syncthreads();
      float den = (red2[0][rl] + red2[1][rl]) + (red2[2][rl] + red2[3][rl]);
      if constexpr (NW == 8) den += (red2[4][rl] + red2[5][rl]) + (red2[6][rl] + red2[7][rl]);
      mul = 1.0f / den;
    }
    u32x4 wlate[4], blate[4];
#pragma unroll
    for (int k = 0; k < NK; ++k) {
      if constexpr (MODE == RW_RMSNORM && !WB_EARLY) {
        if (k % 4 == 0) {
          __builtin_amdgcn_sched_barrier(0);   // the loads of one batch only: the scheduler would hoist all sixteen
#pragma unroll
          for (int u = 0; u < 4; ++u) wb_load(min(k + u, NK - 1), wlate[u], blate[u]);
          __builtin_amdgcn_sched_barrier(0);
        }
      }
      const int run = run_of(k);
      if (run < nruns) {
        const int c0 = col_of(run);
        float f[EPC];
        if constexpr (MODE == RW_RMSNORM) {
          float w[EPC], b[EPC];
          // bf16: unpacked again from the raw chunk; without the empty asm the compiler keeps the floats of the first pass
          // alive across the barrier, twice the registers of the raw chunks
          if constexpr (ELEM == 2 && NK >= 16) asm volatile("" : "+v"(v[k]));
          unpack_vals<ELEM>(v[k], f);
          if (p.w) unpack_vals<ELEM>(WB_EARLY ? wraw[WB_EARLY ? k : 0] : wlate[k % 4], w);
          if (p.b) unpack_vals<ELEM>(WB_EARLY ? braw[WB_EARLY ? k : 0] : blate[k % 4], b);
#pragma unroll
          for (int i = 0; i < EPC; ++i) {
            float y = f[i] * mul;
            if (p.w) y *= w[i];
            if (p.b) y += b[i];
            f[i] = (row_ok && c0 + i < cols) ? y : 0.0f;
          }
        } else {
#pragma unroll
          for (int i = 0; i < EPC; ++i) f[i] = row_ok ? e[k][i] * mul : 0.0f;
        }
        u32x4 ov;
        if (ELEM == 2) {
#pragma unroll
          for (int i = 0; i < 4; ++i) ov[i] = ttm_pack_bf16x2(f[2 * i], f[2 * i + 1]);
        } else {
#pragma unroll
          for (int i = 0; i < 4; ++i) ov[i] = __float_as_uint(f[i]);
        }
        __builtin_nontemporal_store(ov, (u32x4 *)(o + off_of(run) * ELEM));
      }
    }
  }
}

// ------------------------------------------------------------------------------------------------ few, very wide rows
// A vocabulary-sized row for a handful of tokens: too few tile rows to fill the device with one workgroup each.  grid
// (slices, tile rows): a workgroup takes a range of column tiles of one tile row (all 32 rows of it).  Lane t holds the
// same 16-byte chunk position in every tile it visits, hence one row; the eight lanes that share a row are combined
// through LDS.  Step one leaves per (row, slice) the statistics - (max, sum of exp relative to it) for softmax, the sum of
// squares for RMSNorm, the partial result for the reductions; step two forms each row's total from all slices and, for
// softmax and RMSNorm, reads the slice again and writes the output.  stats: [tile row][32][slices][2] floats.
template <int ELEM>
struct WideLane {
  static constexpr int EPC = 16 / ELEM, CPT = 1024 / EPC, TPI = 256 / CPT;   // chunks per tile, tiles per step of a workgroup
  int e, r, col_in, sub;
  __device__ __forceinline__ WideLane(int tid) {
    const int c = tid % CPT;
    sub = tid / CPT;
    e = c * EPC;
    const int face = e >> 8;
    r = (face >> 1) * 16 + ((e >> 4) & 15);
    col_in = (face & 1) * 16 + (e & 15);
  }
  // LDS slot of the i-th of the eight lanes that hold row rr
  static __device__ __forceinline__ int partner(int rr, int i) {
    const int q = i % ELEM, f1 = (i / ELEM) & 1, sb = i / (2 * ELEM);
    return sb * CPT + ((rr >> 4) * 2 + f1) * (16 * ELEM) + (rr & 15) * ELEM + q;
  }
};

template <int MODE, int ELEM>
__global__ __launch_bounds__(256) void ttm_rowwise_wide_stats_k(RowArgs p, float *__restrict__ stats, int slices, int tiles_per_slice) {
  using L = WideLane<ELEM>;
  constexpr int EPC = L::EPC;
  constexpr bool IS_MAX = MODE == RW_SOFTMAX || MODE == RW_MAX;
  __shared__ float sa[256], sb[256];
  const int tid = threadIdx.x, slice = blockIdx.x, cols = (int)p.cols;
  const int64_t trow = blockIdx.y;
  const L ln(tid);
  const uint8_t *x = (const uint8_t *)p.x + trow * p.ct * 1024 * ELEM;
  const int t0 = slice * tiles_per_slice, t1 = min(p.ct, t0 + tiles_per_slice);
  float a = IS_MAX ? -INFINITY : (MODE == RW_MIN ? INFINITY : 0.0f), l = 0.0f;
  constexpr int UN = 4;   // loads in flight per lane: unconditional, clamped to the slice (a branch around a load serialises them)
  for (int tb = t0 + ln.sub; tb < t1; tb += UN * L::TPI) {
    u32x4 raw[UN];
#pragma unroll
    for (int u = 0; u < UN; ++u) raw[u] = __builtin_nontemporal_load((const u32x4 *)(x + ((int64_t)min(tb + u * L::TPI, t1 - 1) * 1024 + ln.e) * ELEM));
#pragma unroll
    for (int u = 0; u < UN; ++u) {
    const int t = tb + u * L::TPI;
    if (t >= t1) break;
    float f[EPC];
    unpack_vals<ELEM>(raw[u], f);
    const int c0 = t * 32 + ln.col_in;
    if (MODE == RW_SOFTMAX) {
      float cm = -INFINITY;
#pragma unroll
      for (int i = 0; i < EPC; ++i) cm = c0 + i < cols ? ttm_max(cm, f[i]) : cm;
      if (cm > a || cm != cm) { l *= expf(a - cm); a = cm; }   // a = -inf at first: l is 0 and stays 0; a NaN maximum stays and makes l NaN
      if (a != -INFINITY) {
#pragma unroll
        for (int i = 0; i < EPC; ++i) l += c0 + i < cols ? expf(f[i] - a) : 0.0f;
      }
    } else {
#pragma unroll
      for (int i = 0; i < EPC; ++i) {
        const bool ok = c0 + i < cols;
        if (MODE == RW_RMSNORM) a += ok ? f[i] * f[i] : 0.0f;
        else if (MODE == RW_MAX) a = ok ? ttm_max(a, f[i]) : a;
        else if (MODE == RW_MIN) a = ok ? ttm_min(a, f[i]) : a;
        else a += ok ? f[i] : 0.0f;
      }
    }
    }
  }
  sa[tid] = a; sb[tid] = l;
  __syncthreads();
  if (tid < 32) {
    float A = IS_MAX ? -INFINITY : (MODE == RW_MIN ? INFINITY : 0.0f), Lsum = 0.0f;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const float v = sa[L::partner(tid, i)];
      A = IS_MAX ? ttm_max(A, v) : (MODE == RW_MIN ? ttm_min(A, v) : A + v);
    }
    if (MODE == RW_SOFTMAX) {
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const int k = L::partner(tid, i);
        Lsum += sa[k] == -INFINITY ? 0.0f : sb[k] * expf(sa[k] - A);
      }
    }
    float *o = stats + ((trow * 32 + tid) * slices + slice) * 2;
    o[0] = A; o[1] = Lsum;
  }
}

// row totals from the slices, by the whole workgroup: lane (row = tid % 32, part = tid / 32) folds every eighth slice of its
// row, the eight parts of a row meet in LDS.  Softmax folds (max, sum relative to that max) pairs.
template <int MODE>
__device__ __forceinline__ void wide_fold(float &A, float &Ls, float v, float w) {
  if (MODE == RW_SOFTMAX) {
    if (v > A) { Ls = Ls * expf(A - v) + w; A = v; }   // A = -inf: Ls is 0 and exp gives 0
    else if (v != -INFINITY) Ls += w * expf(v - A);
  } else if (MODE == RW_MAX) A = ttm_max(A, v);
  else if (MODE == RW_MIN) A = ttm_min(A, v);
  else A += v;
}
template <int MODE>
__device__ __forceinline__ void wide_totals(const float *st, int slices, float *ga, float *gb, float *ta, float *tb) {
  constexpr bool IS_MAX = MODE == RW_SOFTMAX || MODE == RW_MAX;
  const int tid = threadIdx.x, rr = tid & 31, part = tid >> 5;
  float A = IS_MAX ? -INFINITY : (MODE == RW_MIN ? INFINITY : 0.0f), Ls = 0.0f;
  for (int s = part; s < slices; s += 8) wide_fold<MODE>(A, Ls, st[((int64_t)rr * slices + s) * 2], st[((int64_t)rr * slices + s) * 2 + 1]);
  ta[tid] = A; tb[tid] = Ls;
  __syncthreads();
  if (tid < 32) {
    for (int k = 1; k < 8; ++k) wide_fold<MODE>(A, Ls, ta[tid + 32 * k], tb[tid + 32 * k]);
    ga[tid] = A; gb[tid] = Ls;
  }
  __syncthreads();
}

template <int MODE, int ELEM>   // softmax or RMSNorm
__global__ __launch_bounds__(256) void ttm_rowwise_wide_apply_k(RowArgs p, const float *__restrict__ stats, int slices, int tiles_per_slice) {
  using L = WideLane<ELEM>;
  constexpr int EPC = L::EPC;
  __shared__ float ga[32], gb[32], ta[256], tb[256];
  const int tid = threadIdx.x, slice = blockIdx.x, cols = (int)p.cols;
  const int64_t trow = blockIdx.y;
  wide_totals<MODE>(stats + trow * 32 * slices * 2, slices, ga, gb, ta, tb);
  const L ln(tid);
  const bool row_ok = (trow % p.rt) * 32 + ln.r < p.rows;
  const float A = ga[ln.r];
  const float mul = MODE == RW_RMSNORM ? 1.0f / sqrtf(A / (float)cols + p.eps) : 1.0f / gb[ln.r];
  const uint8_t *x = (const uint8_t *)p.x + trow * p.ct * 1024 * ELEM;
  uint8_t *o = (uint8_t *)p.out + trow * p.ct * 1024 * ELEM;
  const int t0 = slice * tiles_per_slice, t1 = min(p.ct, t0 + tiles_per_slice);
  constexpr int UN = 4;
  for (int tb = t0 + ln.sub; tb < t1; tb += UN * L::TPI) {
    u32x4 raw[UN];
#pragma unroll
    for (int u = 0; u < UN; ++u) raw[u] = __builtin_nontemporal_load((const u32x4 *)(x + ((int64_t)min(tb + u * L::TPI, t1 - 1) * 1024 + ln.e) * ELEM));
#pragma unroll
    for (int u = 0; u < UN; ++u) {
    const int t = tb + u * L::TPI;
    if (t >= t1) break;
    const int64_t off = (int64_t)t * 1024 + ln.e;
    float f[EPC];
    unpack_vals<ELEM>(raw[u], f);
    const int c0 = t * 32 + ln.col_in;
    if (MODE == RW_RMSNORM) {
      float w[EPC], b[EPC];
      const int cc = min(c0, ((cols + EPC - 1) / EPC - 1) * EPC);   // the padding of the last tile has no weight: reread a valid chunk
      if (p.w) load_vec<ELEM>(p.w, p.w_tiled, cc, w);
      if (p.b) load_vec<ELEM>(p.b, p.b_tiled, cc, b);
#pragma unroll
      for (int i = 0; i < EPC; ++i) {
        float y = f[i] * mul;
        if (p.w) y *= w[i];
        if (p.b) y += b[i];
        f[i] = (row_ok && c0 + i < cols) ? y : 0.0f;
      }
    } else {
#pragma unroll
      for (int i = 0; i < EPC; ++i) f[i] = (row_ok && c0 + i < cols) ? expf(f[i] - A) * mul : 0.0f;
    }
    store_vals<ELEM>(o, off, f);
    }
  }
}

template <int MODE, int ELEM>   // reductions: the [.., rows, 1] output tile of every tile row
__global__ __launch_bounds__(256) void ttm_rowwise_wide_finish_k(RowArgs p, const float *__restrict__ stats, int slices) {
  using L = WideLane<ELEM>;
  __shared__ float ga[32], gb[32], ta[256], tb[256];
  const int tid = threadIdx.x;
  const int64_t trow = blockIdx.x;
  wide_totals<MODE>(stats + trow * 32 * slices * 2, slices, ga, gb, ta, tb);
  if (tid < L::CPT) {
    const L ln(tid);
    u32x4 z = {0, 0, 0, 0};
    const float total = MODE == RW_MEAN ? ga[ln.r] / (float)p.cols : ga[ln.r];
    if (ln.col_in == 0 && (trow % p.rt) * 32 + ln.r < p.rows) z.x = ELEM == 2 ? (uint32_t)ttm_f32_to_bf16(total) : __float_as_uint(total);
    *(u32x4 *)((uint8_t *)p.out + (trow * 1024 + ln.e) * ELEM) = z;
  }
}

template <int MODE>
static int launch_rowwise(const RowArgs &p, int dtype, int64_t trows, hipStream_t s) {
  TTM_REQUIRE(trows < (1ll << 29), "row-wise kernel: tensor too large");
  {
    // four rows per workgroup, whole lines, the band in registers: from one workgroup per CU upwards, rows of up to 16
    // chunks per lane (16384 bf16 or 8192 fp32 columns).  rowwise_variant: 2 forces it, 1 and 3 exclude it.
    const int elem = dtype == TTM_BF16 ? 2 : 4, variant = ttm_option("rowwise_variant");
    const int nk = (int)ttm_cdiv((int64_t)p.ct * 2 * 4 * elem, 256);
    if (nk > 16 && nk <= 32 && trows * 8 < (1ll << 31) && (variant == 2 || (variant == 0 && trows * 8 >= 256))) {
      // twice the lanes for bands of 17 - 32 chunks per 256 lanes
      const dim3 grid((unsigned)(trows * 8)), block(512);
      if (dtype == TTM_BF16) hipLaunchKernelGGL((ttm_rowwise_band_k<MODE, 2, 16, 512>), grid, block, 0, s, p);
      else hipLaunchKernelGGL((ttm_rowwise_band_k<MODE, 4, 16, 512>), grid, block, 0, s, p);
      TTM_LAUNCH_CHECK();
      return TTM_OK;
    }
    if (nk <= 16 && trows * 8 < (1ll << 31) && (variant == 2 || (variant == 0 && trows * 8 >= 256))) {
      const dim3 grid((unsigned)(trows * 8)), block(256);
#define TTM_BAND_LAUNCH(E, N) hipLaunchKernelGGL((ttm_rowwise_band_k<MODE, E, N>), grid, block, 0, s, p)
#define TTM_BAND_NK(E) \
      do { if (nk <= 1) TTM_BAND_LAUNCH(E, 1); else if (nk <= 2) TTM_BAND_LAUNCH(E, 2); else if (nk <= 4) TTM_BAND_LAUNCH(E, 4); \
           else if (nk <= 8) TTM_BAND_LAUNCH(E, 8); else TTM_BAND_LAUNCH(E, 16); } while (0)
      if (dtype == TTM_BF16) TTM_BAND_NK(2); else TTM_BAND_NK(4);
#undef TTM_BAND_NK
#undef TTM_BAND_LAUNCH
      TTM_LAUNCH_CHECK();
      return TTM_OK;
    }
  }
  // few tile rows of very wide rows: slices of at least eight column tiles, enough of them for about 512 workgroups
  const bool row_kernel_fits = (MODE == RW_RMSNORM || MODE == RW_SOFTMAX) && p.ct * 2 * (dtype == TTM_BF16 ? 2 : 4) <= 8 * 256;
  if (p.ct >= 256 && !row_kernel_fits && trows * 2 <= 256 && ttm_option("rowwise_variant") == 0) {
    int slices = (int)(512 / trows);
    if (slices > p.ct / 8) slices = p.ct / 8;
    if (slices > 256) slices = 256;
    if (slices < 1) slices = 1;
    const int tps = (int)ttm_cdiv(p.ct, slices);
    slices = (int)ttm_cdiv(p.ct, tps);
    void *ws = nullptr;
    if (int rc = ttm_stream_workspace(s, (size_t)(trows * 32 * slices * 2) * sizeof(float), &ws)) return rc;
    const dim3 grid((unsigned)slices, (unsigned)trows);
    if (trows <= 65535) {
      if (dtype == TTM_BF16) hipLaunchKernelGGL((ttm_rowwise_wide_stats_k<MODE, 2>), grid, dim3(256), 0, s, p, (float *)ws, slices, tps);
      else hipLaunchKernelGGL((ttm_rowwise_wide_stats_k<MODE, 4>), grid, dim3(256), 0, s, p, (float *)ws, slices, tps);
      TTM_LAUNCH_CHECK();
      if constexpr (MODE == RW_RMSNORM || MODE == RW_SOFTMAX) {
        if (dtype == TTM_BF16) hipLaunchKernelGGL((ttm_rowwise_wide_apply_k<MODE, 2>), grid, dim3(256), 0, s, p, (const float *)ws, slices, tps);
        else hipLaunchKernelGGL((ttm_rowwise_wide_apply_k<MODE, 4>), grid, dim3(256), 0, s, p, (const float *)ws, slices, tps);
      } else {
        if (dtype == TTM_BF16) hipLaunchKernelGGL((ttm_rowwise_wide_finish_k<MODE, 2>), dim3((unsigned)trows), dim3(256), 0, s, p, (const float *)ws, slices);
        else hipLaunchKernelGGL((ttm_rowwise_wide_finish_k<MODE, 4>), dim3((unsigned)trows), dim3(256), 0, s, p, (const float *)ws, slices);
      }
      TTM_LAUNCH_CHECK();
      return TTM_OK;
    }
  }
  if constexpr (MODE == RW_RMSNORM || MODE == RW_SOFTMAX) {
    const int elem = dtype == TTM_BF16 ? 2 : 4;
    if (p.ct * 2 * elem <= 8 * 256 && trows * 32 < (1 << 24) && ttm_option("rowwise_variant") != 1) {   // one row per workgroup
      const int total = (int)(trows * 32), nq = p.ct * 2 * elem;
      const dim3 grid((unsigned)total), block(256);
#define TTM_ROW_LAUNCH(E, N) hipLaunchKernelGGL((ttm_rowwise_row_k<MODE, E, N>), grid, block, 0, s, p, total)
      if (dtype == TTM_BF16) {
        if (nq <= 512) TTM_ROW_LAUNCH(2, 2);
        else if (nq <= 1024) TTM_ROW_LAUNCH(2, 4);
        else TTM_ROW_LAUNCH(2, 8);
      } else {
        if (nq <= 512) TTM_ROW_LAUNCH(4, 2);
        else if (nq <= 1024) TTM_ROW_LAUNCH(4, 4);
        else TTM_ROW_LAUNCH(4, 8);
      }
#undef TTM_ROW_LAUNCH
      TTM_LAUNCH_CHECK();
      return TTM_OK;
    }
    if (p.ct * 2 * elem <= 16 * 32) {   // a lane's share of the row fits in registers
      if (dtype == TTM_BF16) hipLaunchKernelGGL((ttm_rowwise_resident_k<MODE, 2>), dim3((unsigned)trows * 4), dim3(256), 0, s, p);
      else hipLaunchKernelGGL((ttm_rowwise_resident_k<MODE, 4>), dim3((unsigned)trows * 4), dim3(256), 0, s, p);
      TTM_LAUNCH_CHECK();
      return TTM_OK;
    }
  }
  if (trows >= 1024) {   // enough tile rows to fill the device with one workgroup each
    if (dtype == TTM_BF16) hipLaunchKernelGGL((ttm_rowwise_k<MODE, 2, 32>), dim3((unsigned)trows), dim3(256), 0, s, p);
    else hipLaunchKernelGGL((ttm_rowwise_k<MODE, 4, 32>), dim3((unsigned)trows), dim3(256), 0, s, p);
  } else {
    if (dtype == TTM_BF16) hipLaunchKernelGGL((ttm_rowwise_k<MODE, 2, 8>), dim3((unsigned)trows * 4), dim3(256), 0, s, p);
    else hipLaunchKernelGGL((ttm_rowwise_k<MODE, 4, 8>), dim3((unsigned)trows * 4), dim3(256), 0, s, p);
  }
  TTM_LAUNCH_CHECK();
  return TTM_OK;
}

static int fill_args(RowArgs &p, const void *x, void *out, int dtype, int64_t batch, int64_t rows, int64_t cols,
                     const char *who) {
  TTM_REQUIRE(dtype == TTM_BF16 || dtype == TTM_F32, "%s: dtype must be BFloat16 or Float32 (got %d)", who, dtype);
  TTM_REQUIRE(batch >= 0 && rows >= 0 && cols >= 0, "%s: negative dimension", who);
  TTM_REQUIRE(x && out, "%s: null pointer", who);
  TTM_REQUIRE(((uintptr_t)x & 15) == 0 && ((uintptr_t)out & 15) == 0, "%s: pointers must be 16-byte aligned", who);
  p.x = x; p.out = out; p.w = p.b = nullptr; p.w_tiled = p.b_tiled = 0;
  p.rows = rows; p.cols = cols;
  p.rt = (int)ttm_cdiv(rows, 32); p.ct = (int)ttm_cdiv(cols, 32);
  p.eps = 0.0f; p.out_ct = 1;
  p.partial = nullptr; p.slices = 0; p.per = 0; p.residual = nullptr; p.sum_out = nullptr;
  return TTM_OK;
}

// RMSNorm of x = bf16(bf16(sum of the partial sums) + residual) for one row tile ([rows <= 32, cols] bf16 tiles), x
// stored to sum_out on the way: what ttm_linear_reduce_k with an add tail followed by ttm_rms_norm computes, with the
// kernel ttm_rms_norm itself uses at this size, so the two agree bit for bit.
bool ttm_rowwise_partials_supported(int64_t rows, int64_t cols) {
  const int v = ttm_option("rowwise_variant");
  return rows >= 1 && rows <= 32 && cols >= 1 && ttm_cdiv(cols, 32) * 4 <= 8 * 256 && (v == 0 || v == 3);
}
int ttm_rowwise_rmsnorm_from_partials(const float *partial, int slices, int64_t per, const void *residual, void *sum_out,
                                      const void *weight, int weight_layout, const void *bias, int bias_layout, void *out,
                                      int64_t rows, int64_t cols, float eps, hipStream_t s) {
  TTM_REQUIRE(ttm_rowwise_partials_supported(rows, cols), "rms_norm from partial sums: at most 32 rows and 16384 columns");
  RowArgs p;
  if (int rc = fill_args(p, residual, out, TTM_BF16, 1, rows, cols, "ttm_linear_add_rms_norm")) return rc;
  TTM_REQUIRE(partial && sum_out && slices >= 1, "rms_norm from partial sums: null pointer");
  TTM_REQUIRE((((uintptr_t)weight | (uintptr_t)bias | (uintptr_t)sum_out) & 15) == 0, "ttm_linear_add_rms_norm: operands must be 16-byte aligned");
  p.w = weight; p.b = bias; p.w_tiled = weight_layout == TTM_TILE; p.b_tiled = bias_layout == TTM_TILE; p.eps = eps;
  p.partial = partial; p.slices = slices; p.per = per; p.residual = residual; p.sum_out = sum_out;
  const int nq = p.ct * 4;
  const dim3 grid(32), block(256);
  if (nq <= 512) hipLaunchKernelGGL((ttm_rowwise_row_k<RW_RMSNORM, 2, 2, true>), grid, block, 0, s, p, 32);
  else if (nq <= 1024) hipLaunchKernelGGL((ttm_rowwise_row_k<RW_RMSNORM, 2, 4, true>), grid, block, 0, s, p, 32);
  else hipLaunchKernelGGL((ttm_rowwise_row_k<RW_RMSNORM, 2, 8, true>), grid, block, 0, s, p, 32);
  TTM_LAUNCH_CHECK();
  return TTM_OK;
}

TTM_EXPORT int ttm_rms_norm(const void *x, const void *weight, int weight_layout, const void *bias, int bias_layout,
                            void *out, int dtype, int64_t batch, int64_t rows, int64_t cols, float eps, void *stream) {
  TTM_EXTENTS(rms_norm, x, weight, weight_layout, bias, bias_layout, out, dtype, batch, rows, cols);
  if (batch == 0 || rows == 0 || cols == 0) return TTM_OK;
  RowArgs p;
  int rc = fill_args(p, x, out, dtype, batch, rows, cols, "ttm_rms_norm");
  if (rc) return rc;
  TTM_REQUIRE((((uintptr_t)weight | (uintptr_t)bias) & 15) == 0, "ttm_rms_norm: weight/bias must be 16-byte aligned");
  p.w = weight; p.b = bias; p.w_tiled = weight_layout == TTM_TILE; p.b_tiled = bias_layout == TTM_TILE; p.eps = eps;
  return launch_rowwise<RW_RMSNORM>(p, dtype, batch * p.rt, (hipStream_t)stream);
}

TTM_EXPORT int ttm_softmax_lastdim(const void *x, void *out, int dtype, int64_t batch, int64_t rows, int64_t cols,
                                   void *stream) {
  TTM_EXTENTS(softmax, x, out, dtype, batch, rows, cols);
  if (batch == 0 || rows == 0 || cols == 0) return TTM_OK;
  RowArgs p;
  int rc = fill_args(p, x, out, dtype, batch, rows, cols, "ttm_softmax_lastdim");
  if (rc) return rc;
  return launch_rowwise<RW_SOFTMAX>(p, dtype, batch * p.rt, (hipStream_t)stream);
}

TTM_EXPORT int ttm_reduce_lastdim(int op, const void *x, void *out, int dtype, int64_t batch, int64_t rows, int64_t cols,
                                  void *stream) {
  TTM_EXTENTS(reduce, x, out, dtype, batch, rows, cols);
  TTM_REQUIRE(op >= 0 && op <= 3, "ttm_reduce_lastdim: op must be Sum(0), Mean(1), Max(2) or Min(3), got %d", op);
  if (batch == 0 || rows == 0 || cols == 0) return TTM_OK;
  RowArgs p;
  int rc = fill_args(p, x, out, dtype, batch, rows, cols, "ttm_reduce_lastdim");
  if (rc) return rc;
  hipStream_t s = (hipStream_t)stream;
  switch (op) {
  case 0: return launch_rowwise<RW_SUM>(p, dtype, batch * p.rt, s);
  case 1: return launch_rowwise<RW_MEAN>(p, dtype, batch * p.rt, s);
  case 2: return launch_rowwise<RW_MAX>(p, dtype, batch * p.rt, s);
  default: return launch_rowwise<RW_MIN>(p, dtype, batch * p.rt, s);
  }
}
