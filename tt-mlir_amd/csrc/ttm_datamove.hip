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
};

__device__ __forceinline__ int64_t phys_offset(int64_t lin, int64_t rows, int64_t cols, int tiled) {
  if (!tiled) return lin;
  int64_t c = lin % cols, t = lin / cols;
  int64_t r = t % rows, b = t / rows;
  int64_t pr = (rows + 31) / 32 * 32, pc = (cols + 31) / 32 * 32;
  return b * pr * pc + ttm_tiled_offset(r, c, pc / 32);
}

template <typename T>
__global__ __launch_bounds__(256) void ttm_copy_view_k(const T *__restrict__ src, T *__restrict__ dst, ViewArgs p,
                                                       int64_t total) {
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
    int64_t rem = i, ls = p.sbase, ld = p.dbase;
#pragma unroll 1
    for (int d = p.rank - 1; d >= 0; --d) {
      int64_t v = rem % p.extent[d];
      rem /= p.extent[d];
      ls += v * p.sstride[d];
      ld += v * p.dstride[d];
    }
    dst[phys_offset(ld, p.drows, p.dcols, p.dtiled)] = src[phys_offset(ls, p.srows, p.scols, p.stiled)];
  }
}

// 16 bytes per lane: the innermost view dimension is contiguous on both sides and everything that positions a
// group of V = 16 / elem_bytes elements is a multiple of V, so a group never leaves its row or its 16-wide face row
template <int ELEM>
__global__ __launch_bounds__(256) void ttm_copy_view_vec_k(const u32x4 *__restrict__ src, u32x4 *__restrict__ dst, ViewArgs p,
                                                           int64_t total) {
  constexpr int V = 16 / ELEM;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
    int64_t rem = i, ls = p.sbase, ld = p.dbase;
    {
      const int64_t e = p.extent[p.rank - 1] / V;
      const int64_t v = rem % e;
      rem /= e;
      ls += v * V;
      ld += v * V;
    }
#pragma unroll 1
    for (int d = p.rank - 2; d >= 0; --d) {
      int64_t v = rem % p.extent[d];
      rem /= p.extent[d];
      ls += v * p.sstride[d];
      ld += v * p.dstride[d];
    }
    dst[phys_offset(ld, p.drows, p.dcols, p.dtiled) / V] = src[phys_offset(ls, p.srows, p.scols, p.stiled) / V];
  }
}

TTM_EXPORT int ttm_copy_view(const void *src, int64_t src_rows, int64_t src_cols, int src_layout, void *dst,
                             int64_t dst_rows, int64_t dst_cols, int dst_layout, int elem_bytes, int rank,
                             const int64_t *extent, const int64_t *src_stride, int64_t src_base,
                             const int64_t *dst_stride, int64_t dst_base, void *stream) {
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
  hipStream_t s = (hipStream_t)stream;
  {
    const int64_t V = 16 / elem_bytes;
    bool vec = rank >= 1 && src_stride[rank - 1] == 1 && dst_stride[rank - 1] == 1 && extent[rank - 1] % V == 0 &&
               src_base % V == 0 && dst_base % V == 0 && src_cols % V == 0 && dst_cols % V == 0 &&
               ((uintptr_t)src & 15) == 0 && ((uintptr_t)dst & 15) == 0;
    for (int d = 0; vec && d < rank - 1; ++d) vec = src_stride[d] % V == 0 && dst_stride[d] % V == 0;
    if (vec) {
      const int64_t groups = total / V;
      int64_t vblocks = ttm_cdiv(groups, 256);
      unsigned vgrid = (unsigned)(vblocks > 262144 ? 262144 : vblocks);
      if (elem_bytes == 4) hipLaunchKernelGGL(ttm_copy_view_vec_k<4>, dim3(vgrid), dim3(256), 0, s, (const u32x4 *)src, (u32x4 *)dst, p, groups);
      else if (elem_bytes == 2) hipLaunchKernelGGL(ttm_copy_view_vec_k<2>, dim3(vgrid), dim3(256), 0, s, (const u32x4 *)src, (u32x4 *)dst, p, groups);
      else hipLaunchKernelGGL(ttm_copy_view_vec_k<1>, dim3(vgrid), dim3(256), 0, s, (const u32x4 *)src, (u32x4 *)dst, p, groups);
      TTM_LAUNCH_CHECK();
      return TTM_OK;
    }
  }
  int64_t blocks = ttm_cdiv(total, 256);
  unsigned grid = (unsigned)(blocks > 262144 ? 262144 : blocks);
  if (elem_bytes == 4) hipLaunchKernelGGL(ttm_copy_view_k<uint32_t>, dim3(grid), dim3(256), 0, s, (const uint32_t *)src, (uint32_t *)dst, p, total);
  else if (elem_bytes == 2) hipLaunchKernelGGL(ttm_copy_view_k<uint16_t>, dim3(grid), dim3(256), 0, s, (const uint16_t *)src, (uint16_t *)dst, p, total);
  else hipLaunchKernelGGL(ttm_copy_view_k<uint8_t>, dim3(grid), dim3(256), 0, s, (const uint8_t *)src, (uint8_t *)dst, p, total);
  TTM_LAUNCH_CHECK();
  return TTM_OK;
}
