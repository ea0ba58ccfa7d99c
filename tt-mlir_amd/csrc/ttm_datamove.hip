// Generic data movement between tensors in row-major or tile order: one kernel covers reshape,
// permute / transpose, slice, concat, repeat_interleave and layout changes with padding.
//
// A copy is described by a view of `rank` (<= 8) extents.  View index v maps to a logical linear
// element index of the source, src_base + sum v[d] * src_stride[d], and of the destination,
// dst_base + sum v[d] * dst_stride[d].  Logical linear indices are row-major over the tensor's
// logical shape [batch, rows, cols]; the kernel converts them to physical offsets for the
// tensor's layout (row-major, or 32x32 tiles with 16x16 faces, zero padded).
#include "ttm_common.h"

struct ViewArgs {
  int rank;
  int64_t extent[8], sstride[8], dstride[8];
  int64_t sbase, dbase;
  int64_t srows, scols, drows, dcols;  // logical last-two dims of source / destination
  int stiled, dtiled;
  // optional position in device memory: the destination base advances by *index * istride; nothing is written when
  // *index lies outside [0, ilimit)
  const int32_t *index;
  int64_t istride, ilimit;
};

__device__ __forceinline__ bool view_position(const ViewArgs &p, int64_t &dbase) {
  dbase = p.dbase;
  if (!p.index) return true;
  const int64_t v = *p.index;
  if (v < 0 || v >= p.ilimit) return false;
  dbase += v * p.istride;
  return true;
}

// I is the index type of all logical and physical offsets: 32-bit when both tensors and every intermediate index fit
// (64-bit division costs several times as much as the copy itself)
template <typename I>
__device__ __forceinline__ I phys_offset(I lin, I rows, I cols, int tiled) {
  if (!tiled) return lin;
  I c = lin % cols, t = lin / cols;
  I r = t % rows, b = t / rows;
  I pr = (rows + 31) / 32 * 32, pc = (cols + 31) / 32 * 32;
  return b * pr * pc + (I)ttm_tiled_offset(r, c, pc / 32);
}

template <typename T, typename I>
__global__ __launch_bounds__(256) void ttm_copy_view_k(const T *__restrict__ src, T *__restrict__ dst, ViewArgs p,
                                                       int64_t total) {
  int64_t dbase;
  if (!view_position(p, dbase)) return;
  for (int64_t i0 = (int64_t)blockIdx.x * 256 + threadIdx.x; i0 < total; i0 += (int64_t)gridDim.x * 256) {
    I rem = (I)i0, ls = (I)p.sbase, ld = (I)dbase;
#pragma unroll 1
    for (int d = p.rank - 1; d >= 0; --d) {
      const I e = (I)p.extent[d];
      const I q = rem / e, v = rem - q * e;
      rem = q;
      ls += v * (I)p.sstride[d];
      ld += v * (I)p.dstride[d];
    }
    dst[phys_offset<I>(ld, (I)p.drows, (I)p.dcols, p.dtiled)] = src[phys_offset<I>(ls, (I)p.srows, (I)p.scols, p.stiled)];
  }
}

// 16 bytes per lane: the innermost view dimension is contiguous on both sides and everything that positions a
// group of V = 16 / elem_bytes elements is a multiple of V, so a group never leaves its row or its 16-wide face row.
// DPHYS: the destination is a tile-order tensor that the view covers densely in row-major order (reshape, permute, slice
// results).  Lanes then take the destination's 16-byte chunks in the order they lie in memory and find their view index
// from the chunk's position, so that a wavefront's stores are whole lines; in view order consecutive lanes would write
// one 32- or 64-byte face row each into a different line.  Chunks in the padding of the destination are left alone.
template <int ELEM, typename I, bool DPHYS>
__global__ __launch_bounds__(256) void ttm_copy_view_vec_k(const u32x4 *__restrict__ src, u32x4 *__restrict__ dst, ViewArgs p,
                                                           int64_t total) {
  constexpr int V = 16 / ELEM;
  int64_t dbase;
  if (!view_position(p, dbase)) return;
  for (int64_t i0 = (int64_t)blockIdx.x * 256 + threadIdx.x; i0 < total; i0 += (int64_t)gridDim.x * 256) {
    I rem = (I)i0, ls = (I)p.sbase, ld = (I)dbase;
    I dchunk = 0;
    if constexpr (DPHYS) {
      // chunk i0 of the destination's memory -> (matrix, row, first column) -> logical index = view index
      const I ph = (I)i0 * V, tile = ph >> 10, e = ph & 1023, face = e >> 8;
      const I ptc = ((I)p.dcols + 31) / 32, prt = ((I)p.drows + 31) / 32;
      const I m = tile / (prt * ptc), tin = tile - m * (prt * ptc), tr = tin / ptc, tc = tin - tr * ptc;
      const I row = tr * 32 + (face >> 1) * 16 + ((e >> 4) & 15), col = tc * 32 + (face & 1) * 16 + (e & 15);
      if (row >= (I)p.drows || col >= (I)p.dcols) continue;
      rem = ((m * (I)p.drows + row) * (I)p.dcols + col) / V;
      dchunk = (I)i0;
    }
    {
      const I e = (I)p.extent[p.rank - 1] / V;
      const I q = rem / e, v = rem - q * e;
      rem = q;
      ls += v * V;
      ld += v * V;
    }
#pragma unroll 1
    for (int d = p.rank - 2; d >= 0; --d) {
      const I e = (I)p.extent[d];
      const I q = rem / e, v = rem - q * e;
      rem = q;
      ls += v * (I)p.sstride[d];
      ld += v * (I)p.dstride[d];
    }
    if constexpr (!DPHYS) dchunk = phys_offset<I>(ld, (I)p.drows, (I)p.dcols, p.dtiled) / V;
    dst[dchunk] = src[phys_offset<I>(ls, (I)p.srows, (I)p.scols, p.stiled) / V];
  }
}

// Transpose of the last two dims between tile-order tensors whose extents are multiples of 32: tile (i, j) of the source is
// tile (j, i) of the destination with its 32 x 32 elements transposed, so every access is a whole tile (2 or 4 KiB
// contiguous).  One wavefront per tile: every load and store instruction of the wavefront covers 1 KiB contiguous (lane l
// takes 16-byte chunk 64 i + l of the tile), the elements cross through the wavefront's own 32 x 33-word area of LDS.
template <typename T>
__global__ __launch_bounds__(256) void ttm_transpose_tiles_k(const T *__restrict__ src, T *__restrict__ dst, int64_t tiles, int rt, int ct) {
  __shared__ uint32_t lds[4][32 * 33];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int64_t t = (int64_t)blockIdx.x * 4 + wave;
  if (t >= tiles) return;   // wavefront-uniform; no barrier below
  const int64_t per = (int64_t)rt * ct, b = t / per, rem = t - b * per;
  const int tr = (int)(rem / ct), tc = (int)(rem - (int64_t)tr * ct);
  const u32x4 *sp = (const u32x4 *)(src + (b * per + (int64_t)tr * ct + tc) * 1024);
  u32x4 *dp = (u32x4 *)(dst + (b * per + (int64_t)tc * rt + tr) * 1024);
  constexpr int V = 16 / sizeof(T), NCH = 1024 / V / 64;   // elements per chunk, chunks per lane
  uint32_t *w = lds[wave];
  u32x4 q[NCH];
#pragma unroll
  for (int i = 0; i < NCH; ++i) q[i] = __builtin_nontemporal_load(sp + i * 64 + lane);
#pragma unroll
  for (int i = 0; i < NCH; ++i) {
    const int e0 = (i * 64 + lane) * V, f = e0 >> 8, r = (e0 >> 4) & 15, c0 = e0 & 15;
    uint32_t *row = w + (16 * (f >> 1) + r) * 33 + 16 * (f & 1) + c0;
#pragma unroll
    for (int j = 0; j < V; ++j) row[j] = sizeof(T) == 2 ? (q[i][j / 2] >> (16 * (j & 1))) & 0xFFFFu : q[i][j];
  }
#pragma unroll
  for (int i = 0; i < NCH; ++i) {
    // chunk of the transposed tile: face (fr, fc), row r, columns c0 .. c0 + V - 1 = source elements (16 fc + c0 + j, 16 fr + r)
    const int e0 = (i * 64 + lane) * V, f = e0 >> 8, r = (e0 >> 4) & 15, c0 = e0 & 15;
    const uint32_t *col = w + (16 * (f & 1) + c0) * 33 + 16 * (f >> 1) + r;
    uint32_t e[V];
#pragma unroll
    for (int j = 0; j < V; ++j) e[j] = col[j * 33];
    u32x4 o;
    if (sizeof(T) == 2) {
#pragma unroll
      for (int j = 0; j < 4; ++j) o[j] = e[2 * j] | (e[2 * j + 1] << 16);
    } else {
#pragma unroll
      for (int j = 0; j < 4; ++j) o[j] = e[j];
    }
    __builtin_nontemporal_store(o, dp + i * 64 + lane);
  }
}

// whether a view is the transpose of the last two dims of a dense tile-order tensor (either way of writing it: view dims
// in source order with a transposed destination, or in destination order with a transposed source); *batches = the rest
static bool is_tile_transpose(const ViewArgs &p, int elem_bytes, int64_t *batches) {
  if (p.rank < 2 || !p.stiled || !p.dtiled || p.index || (elem_bytes != 2 && elem_bytes != 4) || p.sbase != 0 || p.dbase != 0) return false;
  const int64_t R = p.srows, C = p.scols;
  if (R % 32 != 0 || C % 32 != 0 || p.drows != C || p.dcols != R) return false;
  const int a = p.rank - 2, b = p.rank - 1;
  const bool src_order = p.extent[a] == R && p.extent[b] == C && p.sstride[a] == C && p.sstride[b] == 1 && p.dstride[a] == 1 && p.dstride[b] == R;
  const bool dst_order = p.extent[a] == C && p.extent[b] == R && p.sstride[a] == 1 && p.sstride[b] == C && p.dstride[a] == R && p.dstride[b] == 1;
  if (!src_order && !dst_order) return false;
  int64_t n = 1;   // the leading dims must number the matrices densely and alike on both sides
  for (int d = p.rank - 3; d >= 0; --d) {
    if (p.extent[d] != 1 && (p.sstride[d] != n * R * C || p.dstride[d] != n * R * C)) return false;
    n *= p.extent[d];
  }
  *batches = n;
  return true;
}

template <typename I>
static void launch_copy_view(const void *src, void *dst, const ViewArgs &p, int elem_bytes, bool vec, int64_t dphys_chunks, int64_t total,
                             hipStream_t s) {
  if (vec && dphys_chunks > 0) {   // in the order of the destination's memory: every chunk of it, padding included
    int64_t vblocks = ttm_cdiv(dphys_chunks, 256);
    unsigned vgrid = (unsigned)(vblocks > 262144 ? 262144 : vblocks);
    if (elem_bytes == 4) hipLaunchKernelGGL((ttm_copy_view_vec_k<4, I, true>), dim3(vgrid), dim3(256), 0, s, (const u32x4 *)src, (u32x4 *)dst, p, dphys_chunks);
    else if (elem_bytes == 2) hipLaunchKernelGGL((ttm_copy_view_vec_k<2, I, true>), dim3(vgrid), dim3(256), 0, s, (const u32x4 *)src, (u32x4 *)dst, p, dphys_chunks);
    else hipLaunchKernelGGL((ttm_copy_view_vec_k<1, I, true>), dim3(vgrid), dim3(256), 0, s, (const u32x4 *)src, (u32x4 *)dst, p, dphys_chunks);
    return;
  }
  if (vec) {
    const int64_t groups = total / (16 / elem_bytes);
    int64_t vblocks = ttm_cdiv(groups, 256);
    unsigned vgrid = (unsigned)(vblocks > 262144 ? 262144 : vblocks);
    if (elem_bytes == 4) hipLaunchKernelGGL((ttm_copy_view_vec_k<4, I, false>), dim3(vgrid), dim3(256), 0, s, (const u32x4 *)src, (u32x4 *)dst, p, groups);
    else if (elem_bytes == 2) hipLaunchKernelGGL((ttm_copy_view_vec_k<2, I, false>), dim3(vgrid), dim3(256), 0, s, (const u32x4 *)src, (u32x4 *)dst, p, groups);
    else hipLaunchKernelGGL((ttm_copy_view_vec_k<1, I, false>), dim3(vgrid), dim3(256), 0, s, (const u32x4 *)src, (u32x4 *)dst, p, groups);
    return;
  }
  int64_t blocks = ttm_cdiv(total, 256);
  unsigned grid = (unsigned)(blocks > 262144 ? 262144 : blocks);
  if (elem_bytes == 4) hipLaunchKernelGGL((ttm_copy_view_k<uint32_t, I>), dim3(grid), dim3(256), 0, s, (const uint32_t *)src, (uint32_t *)dst, p, total);
  else if (elem_bytes == 2) hipLaunchKernelGGL((ttm_copy_view_k<uint16_t, I>), dim3(grid), dim3(256), 0, s, (const uint16_t *)src, (uint16_t *)dst, p, total);
  else hipLaunchKernelGGL((ttm_copy_view_k<uint8_t, I>), dim3(grid), dim3(256), 0, s, (const uint8_t *)src, (uint8_t *)dst, p, total);
}

static int copy_view_entry(const void *src, int64_t src_rows, int64_t src_cols, int src_layout, void *dst, int64_t dst_rows,
                           int64_t dst_cols, int dst_layout, int elem_bytes, int rank, const int64_t *extent,
                           const int64_t *src_stride, int64_t src_base, const int64_t *dst_stride, int64_t dst_base,
                           const int32_t *index, int64_t index_stride, int64_t index_limit, void *stream) {
  TTM_REQUIRE(rank >= 0 && rank <= 8, "ttm_copy_view: rank must be 0..8 (got %d)", rank);
  TTM_REQUIRE(elem_bytes == 1 || elem_bytes == 2 || elem_bytes == 4, "ttm_copy_view: elem_bytes must be 1, 2 or 4");
  TTM_REQUIRE(rank == 0 || (extent && src_stride && dst_stride), "ttm_copy_view: null view description");
  TTM_REQUIRE(src_rows > 0 && src_cols > 0 && dst_rows > 0 && dst_cols > 0, "ttm_copy_view: empty tensor shape");
  ViewArgs p;
  p.rank = rank;
  int64_t total = 1;
  for (int d = 0; d < rank; ++d) {
    TTM_REQUIRE(extent[d] >= 0, "ttm_copy_view: negative extent");
    p.extent[d] = extent[d]; p.sstride[d] = src_stride[d]; p.dstride[d] = dst_stride[d];
    total *= extent[d];
  }
  if (total == 0) return TTM_OK;
  TTM_REQUIRE(src && dst, "ttm_copy_view: null pointer");
  p.sbase = src_base; p.dbase = dst_base;
  p.srows = src_rows; p.scols = src_cols; p.drows = dst_rows; p.dcols = dst_cols;
  p.stiled = src_layout == TTM_TILE; p.dtiled = dst_layout == TTM_TILE;
  p.index = index; p.istride = index_stride; p.ilimit = index_limit;
  if (index) TTM_REQUIRE(index_stride >= 0 && index_limit >= 1, "ttm_copy_view_at: index stride must be >= 0 and the limit >= 1");
  hipStream_t s = (hipStream_t)stream;
  int64_t matrices = 0;
  if (is_tile_transpose(p, elem_bytes, &matrices) && ((uintptr_t)src & 15) == 0 && ((uintptr_t)dst & 15) == 0 &&
      matrices * (src_rows / 32) * (src_cols / 32) < ((int64_t)1 << 32)) {
    const int rt = (int)(src_rows / 32), ct = (int)(src_cols / 32);
    const int64_t tiles = matrices * rt * ct;
    if (elem_bytes == 2) hipLaunchKernelGGL(ttm_transpose_tiles_k<uint16_t>, dim3((unsigned)ttm_cdiv(tiles, 4)), dim3(256), 0, s, (const uint16_t *)src, (uint16_t *)dst, tiles, rt, ct);
    else hipLaunchKernelGGL(ttm_transpose_tiles_k<uint32_t>, dim3((unsigned)ttm_cdiv(tiles, 4)), dim3(256), 0, s, (const uint32_t *)src, (uint32_t *)dst, tiles, rt, ct);
    TTM_LAUNCH_CHECK();
    return TTM_OK;
  }
  const int64_t V = 16 / elem_bytes;
  bool vec = rank >= 1 && src_stride[rank - 1] == 1 && dst_stride[rank - 1] == 1 && extent[rank - 1] % V == 0 &&
             src_base % V == 0 && dst_base % V == 0 && src_cols % V == 0 && dst_cols % V == 0 &&
             ((uintptr_t)src & 15) == 0 && ((uintptr_t)dst & 15) == 0;
  for (int d = 0; vec && d < rank - 1; ++d) vec = src_stride[d] % V == 0 && dst_stride[d] % V == 0;
  if (index) vec = vec && index_stride % V == 0;
  // 32-bit index arithmetic when no logical index, no physical (padded) offset and no partial sum can reach 2^31:
  // bases and strides non-negative, and the largest reachable logical index of either side, rounded up to whole padded
  // tiles per row, stays below the limit
  bool narrow = total < (int64_t)1 << 31 && src_base >= 0 && dst_base >= 0;
  int64_t smax = src_base, dmax = dst_base + (index ? (index_limit - 1) * index_stride : 0);
  narrow = narrow && dmax < ((int64_t)1 << 29);
  for (int d = 0; narrow && d < rank; ++d) {
    narrow = src_stride[d] >= 0 && dst_stride[d] >= 0;
    smax += (extent[d] - 1) * src_stride[d];
    dmax += (extent[d] - 1) * dst_stride[d];
    narrow = narrow && smax < ((int64_t)1 << 29) && dmax < ((int64_t)1 << 29);
  }
  auto padded_reach = [](int64_t lin_max, int64_t rows, int64_t cols) {
    const int64_t batches = lin_max / (rows * cols) + 1;
    return batches * ttm_round_up32(rows) * ttm_round_up32(cols);
  };
  narrow = narrow && padded_reach(smax, src_rows, src_cols) < ((int64_t)1 << 31) && padded_reach(dmax, dst_rows, dst_cols) < ((int64_t)1 << 31);
  // destination in tile order, covered densely and in row-major order by the view, from its first element on: the vector
  // kernel may walk the destination's memory instead of the view
  int64_t dphys_chunks = 0;
  if (vec && p.dtiled && !index && dst_base == 0 && total % (dst_rows * dst_cols) == 0) {
    bool dense = true;
    int64_t acc = 1;
    for (int d = rank - 1; d >= 0 && dense; --d) {
      dense = extent[d] == 1 || dst_stride[d] == acc;
      acc *= extent[d];
    }
    if (dense) dphys_chunks = total / (dst_rows * dst_cols) * ttm_round_up32(dst_rows) * ttm_round_up32(dst_cols) / V;
  }
  if (narrow) launch_copy_view<uint32_t>(src, dst, p, elem_bytes, vec, dphys_chunks, total, s);
  else launch_copy_view<int64_t>(src, dst, p, elem_bytes, vec, dphys_chunks, total, s);
  TTM_LAUNCH_CHECK();
  return TTM_OK;
}

TTM_EXPORT int ttm_copy_view(const void *src, int64_t src_rows, int64_t src_cols, int src_layout, void *dst,
                             int64_t dst_rows, int64_t dst_cols, int dst_layout, int elem_bytes, int rank,
                             const int64_t *extent, const int64_t *src_stride, int64_t src_base,
                             const int64_t *dst_stride, int64_t dst_base, void *stream) {
  if (rank >= 0 && rank <= 8 && (rank == 0 || (extent && src_stride && dst_stride)))
    TTM_EXTENTS_VIEW(src, src_rows, src_cols, src_layout, dst, dst_rows, dst_cols, dst_layout, elem_bytes, rank, extent, src_stride, src_base, dst_stride, dst_base, 0);
  return copy_view_entry(src, src_rows, src_cols, src_layout, dst, dst_rows, dst_cols, dst_layout, elem_bytes, rank, extent, src_stride,
                         src_base, dst_stride, dst_base, nullptr, 0, 0, stream);
}

TTM_EXPORT int ttm_copy_view_at(const void *src, int64_t src_rows, int64_t src_cols, int src_layout, void *dst,
                                int64_t dst_rows, int64_t dst_cols, int dst_layout, int elem_bytes, int rank,
                                const int64_t *extent, const int64_t *src_stride, int64_t src_base,
                                const int64_t *dst_stride, int64_t dst_base, const int32_t *index, int64_t index_stride,
                                int64_t index_limit, void *stream) {
  if (rank >= 0 && rank <= 8 && (rank == 0 || (extent && src_stride && dst_stride))) {
    TTM_EXTENTS_SPAN("index", index, 4);
    TTM_EXTENTS_VIEW(src, src_rows, src_cols, src_layout, dst, dst_rows, dst_cols, dst_layout, elem_bytes, rank, extent, src_stride, src_base, dst_stride, dst_base,
                     index_limit > 0 ? (index_limit - 1) * index_stride : 0);
  }
  TTM_REQUIRE(index, "ttm_copy_view_at: null index pointer");
  return copy_view_entry(src, src_rows, src_cols, src_layout, dst, dst_rows, dst_cols, dst_layout, elem_bytes, rank, extent, src_stride,
                         src_base, dst_stride, dst_base, index, index_stride, index_limit, stream);
}
