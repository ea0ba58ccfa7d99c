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
// group of V = 16 / elem_bytes elements is a multiple of V, so a group never leaves its row or its 16-wide face row
template <int ELEM, typename I>
__global__ __launch_bounds__(256) void ttm_copy_view_vec_k(const u32x4 *__restrict__ src, u32x4 *__restrict__ dst, ViewArgs p,
                                                           int64_t total) {
  constexpr int V = 16 / ELEM;
  int64_t dbase;
  if (!view_position(p, dbase)) return;
  for (int64_t i0 = (int64_t)blockIdx.x * 256 + threadIdx.x; i0 < total; i0 += (int64_t)gridDim.x * 256) {
    I rem = (I)i0, ls = (I)p.sbase, ld = (I)dbase;
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
    dst[phys_offset<I>(ld, (I)p.drows, (I)p.dcols, p.dtiled) / V] = src[phys_offset<I>(ls, (I)p.srows, (I)p.scols, p.stiled) / V];
  }
}

template <typename I>
static void launch_copy_view(const void *src, void *dst, const ViewArgs &p, int elem_bytes, bool vec, int64_t total, hipStream_t s) {
  if (vec) {
    const int64_t groups = total / (16 / elem_bytes);
    int64_t vblocks = ttm_cdiv(groups, 256);
    unsigned vgrid = (unsigned)(vblocks > 262144 ? 262144 : vblocks);
    if (elem_bytes == 4) hipLaunchKernelGGL((ttm_copy_view_vec_k<4, I>), dim3(vgrid), dim3(256), 0, s, (const u32x4 *)src, (u32x4 *)dst, p, groups);
    else if (elem_bytes == 2) hipLaunchKernelGGL((ttm_copy_view_vec_k<2, I>), dim3(vgrid), dim3(256), 0, s, (const u32x4 *)src, (u32x4 *)dst, p, groups);
    else hipLaunchKernelGGL((ttm_copy_view_vec_k<1, I>), dim3(vgrid), dim3(256), 0, s, (const u32x4 *)src, (u32x4 *)dst, p, groups);
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
  if (narrow) launch_copy_view<uint32_t>(src, dst, p, elem_bytes, vec, total, s);
  else launch_copy_view<int64_t>(src, dst, p, elem_bytes, vec, total, s);
  TTM_LAUNCH_CHECK();
  return TTM_OK;
}

TTM_EXPORT int ttm_copy_view(const void *src, int64_t src_rows, int64_t src_cols, int src_layout, void *dst,
                             int64_t dst_rows, int64_t dst_cols, int dst_layout, int elem_bytes, int rank,
                             const int64_t *extent, const int64_t *src_stride, int64_t src_base,
                             const int64_t *dst_stride, int64_t dst_base, void *stream) {
  return copy_view_entry(src, src_rows, src_cols, src_layout, dst, dst_rows, dst_cols, dst_layout, elem_bytes, rank, extent, src_stride,
                         src_base, dst_stride, dst_base, nullptr, 0, 0, stream);
}

TTM_EXPORT int ttm_copy_view_at(const void *src, int64_t src_rows, int64_t src_cols, int src_layout, void *dst,
                                int64_t dst_rows, int64_t dst_cols, int dst_layout, int elem_bytes, int rank,
                                const int64_t *extent, const int64_t *src_stride, int64_t src_base,
                                const int64_t *dst_stride, int64_t dst_base, const int32_t *index, int64_t index_stride,
                                int64_t index_limit, void *stream) {
  TTM_REQUIRE(index, "ttm_copy_view_at: null index pointer");
  return copy_view_entry(src, src_rows, src_cols, src_layout, dst, dst_rows, dst_cols, dst_layout, elem_bytes, rank, extent, src_stride,
                         src_base, dst_stride, dst_base, index, index_stride, index_limit, stream);
}
