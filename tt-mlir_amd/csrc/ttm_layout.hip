// Tilize / untilize for Tenstorrent's 32x32 tile layout with 16x16 faces, plus the plain copy
// kernel used as the measured HBM ceiling.  All kernels move 16 bytes per lane per access.
//
// Two formulations of each direction, selected with ttm_set_option("tilize_variant"/"untilize_variant"):
//   0  LDS-staged: a workgroup owns a strip of 32 rows x 512 bytes (16/elem tiles).  Global reads
//      and writes are both fully contiguous (512 B per row segment on the row-major side, 16 KiB
//      on the tiled side); the face permutation happens between a padded LDS image and registers.
//   1  direct: one lane per 16-byte chunk of the tiled side, the row-major side is touched in
//      face-row segments (16 elements).  No LDS; used when a strip does not divide the row.
// A scalar kernel covers shapes that are not multiples of 32 (zero padding).
#include "ttm_common.h"

typedef u32x4 chunk_t;  // 16 bytes

// ------------------------------------------------------------------------------------ copy
// five workgroups of 16 KiB per CU: 256 MiB 84.4 -> 82.7 us, 64 MiB 25.6 -> 24.1 us against no cap
__global__ __launch_bounds__(256) TTM_MAX_WAVES(5) void ttm_copy_kernel_k(const chunk_t *__restrict__ src,
                                                         chunk_t *__restrict__ dst, size_t nchunks) {
  size_t base = (size_t)blockIdx.x * (256 * 4) + threadIdx.x;
  chunk_t v[4];
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    size_t i = base + u * 256;
    if (i < nchunks) v[u] = __builtin_nontemporal_load(&src[i]);
  }
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    size_t i = base + u * 256;
    if (i < nchunks) __builtin_nontemporal_store(v[u], &dst[i]);
  }
}

TTM_EXPORT int ttm_copy_kernel(const void *src, void *dst, size_t bytes, void *stream) {
  TTM_EXTENTS(copy_kernel, src, dst, bytes);
  if (bytes == 0) return TTM_OK;
  TTM_REQUIRE(src && dst, "ttm_copy_kernel: null pointer");
  TTM_REQUIRE(bytes % 16 == 0 && ((uintptr_t)src & 15) == 0 && ((uintptr_t)dst & 15) == 0,
              "ttm_copy_kernel: size and pointers must be multiples of 16 bytes");
  size_t n = bytes / 16;
  size_t blocks = (n + 1023) / 1024;
  TTM_REQUIRE(blocks < (1ull << 31), "ttm_copy_kernel: too large");
  hipLaunchKernelGGL(ttm_copy_kernel_k, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream,
                     (const chunk_t *)src, (chunk_t *)dst, n);
  TTM_LAUNCH_CHECK();
  return TTM_OK;
}

// ------------------------------------------------------------------------------------ direct
// ELEM = element bytes.  A face row (16 elements) is ELEM chunks; a tile is 64*ELEM chunks.
template <int ELEM, bool TILIZE>
__global__ __launch_bounds__(256) void ttm_tile_direct_k(const chunk_t *__restrict__ src,
                                                         chunk_t *__restrict__ dst, int64_t yt, int64_t xt,
                                                         int64_t total_chunks) {
  constexpr int CPT = 64 * ELEM;  // chunks per tile
  const int64_t row_chunks = xt * 2 * ELEM;  // chunks per row-major row
  int64_t base = (int64_t)blockIdx.x * (256 * 4) + threadIdx.x;
  chunk_t v[4];
  int64_t rm[4];
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    int64_t o = base + u * 256;  // chunk index on the tiled side
    if (o < total_chunks) {
      int64_t tile = o / CPT;
      int w = (int)(o % CPT);
      int face = w / (16 * ELEM), dy = (w / ELEM) % 16, q = w % ELEM;
      int64_t tx = tile % xt, tyb = tile / xt;  // tyb = batch * yt + ty (rows are multiples of 32)
      int64_t r = tyb * 32 + (face >> 1) * 16 + dy;
      rm[u] = r * row_chunks + tx * 2 * ELEM + (face & 1) * ELEM + q;
      v[u] = TILIZE ? __builtin_nontemporal_load(&src[rm[u]]) : __builtin_nontemporal_load(&src[o]);
    }
  }
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    int64_t o = base + u * 256;
    if (o < total_chunks) {
      if (TILIZE) __builtin_nontemporal_store(v[u], &dst[o]);
      else __builtin_nontemporal_store(v[u], &dst[rm[u]]);
    }
  }
  (void)yt;
}

// ------------------------------------------------------------------------------------ LDS staged
// Strip = 32 rows x 32 chunks (512 B).  LDS image is row-major with a 33-chunk pitch.
// Three (tilize) / four (untilize) workgroups per CU: 8192 x 8192 fp32 84.0 -> 80 / 81 us, the same 3 - 5 % for bf16 and for
// [16384, 4096], [2048, 14336], [65536, 2048].
template <int ELEM, bool TILIZE>
__global__ __launch_bounds__(256) TTM_MAX_WAVES(TILIZE ? 3 : 4) void ttm_tile_strip_k(const chunk_t *__restrict__ src,
                                                        chunk_t *__restrict__ dst, int64_t xt,
                                                        int64_t strips_per_row) {
  constexpr int CPT = 64 * ELEM;
  constexpr int PITCH = 33;
  __shared__ chunk_t lds[32 * PITCH];
  const int tid = threadIdx.x;
  const int64_t strip = blockIdx.x;                 // over (batch*yt) x strips_per_row
  const int64_t tyb = strip / strips_per_row;       // tile-row index over batch
  const int64_t sx = strip % strips_per_row;
  const int64_t row_chunks = xt * 2 * ELEM;
  const chunk_t *rm_base = (TILIZE ? src : dst) + tyb * 32 * row_chunks + sx * 32;  // unused const-ness below
  const int64_t tiled_base = (tyb * xt + sx * (16 / ELEM)) * CPT;

  chunk_t v[4];
  if (TILIZE) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      int r = i * 8 + (tid >> 5), j = tid & 31;
      v[i] = __builtin_nontemporal_load(&rm_base[r * row_chunks + j]);
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      int r = i * 8 + (tid >> 5), j = tid & 31;
      lds[r * PITCH + j] = v[i];
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      int oc = i * 256 + tid;
      int tl = oc / CPT, w = oc % CPT;
      int face = w / (16 * ELEM), dy = (w / ELEM) % 16, q = w % ELEM;
      int r = (face >> 1) * 16 + dy, j = tl * 2 * ELEM + (face & 1) * ELEM + q;
      __builtin_nontemporal_store(lds[r * PITCH + j], &dst[tiled_base + oc]);
    }
  } else {
#pragma unroll
    for (int i = 0; i < 4; ++i) v[i] = __builtin_nontemporal_load(&src[tiled_base + i * 256 + tid]);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      int oc = i * 256 + tid;
      int tl = oc / CPT, w = oc % CPT;
      int face = w / (16 * ELEM), dy = (w / ELEM) % 16, q = w % ELEM;
      int r = (face >> 1) * 16 + dy, j = tl * 2 * ELEM + (face & 1) * ELEM + q;
      lds[r * PITCH + j] = v[i];
    }
    __syncthreads();
    chunk_t *out = dst + tyb * 32 * row_chunks + sx * 32;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      int r = i * 8 + (tid >> 5), j = tid & 31;
      __builtin_nontemporal_store(lds[r * PITCH + j], &out[r * row_chunks + j]);
    }
  }
}

// ------------------------------------------------------------------------------------ scalar (padding)
template <typename T, bool TILIZE>
__global__ __launch_bounds__(256) void ttm_tile_scalar_k(const T *__restrict__ src, T *__restrict__ dst,
                                                         int64_t batch, int64_t rows, int64_t cols,
                                                         int64_t pr, int64_t pc) {
  int64_t n = batch * pr * pc;
  int64_t ct = pc / 32;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (int64_t)gridDim.x * 256) {
    // i enumerates the tiled side
    int64_t b = i / (pr * pc), w = i % (pr * pc);
    int64_t tile = w / 1024;
    int e = (int)(w % 1024);
    int face = e >> 8, dy = (e >> 4) & 15, dx = e & 15;
    int64_t r = (tile / ct) * 32 + (face >> 1) * 16 + dy, c = (tile % ct) * 32 + (face & 1) * 16 + dx;
    bool in = r < rows && c < cols;
    if (TILIZE) dst[i] = in ? src[(b * rows + r) * cols + c] : T(0);
    else if (in) dst[(b * rows + r) * cols + c] = src[i];
  }
}

// ------------------------------------------------------------------------------------ ragged shapes, 16 bytes at a time
// Rows or columns that are not multiples of 32.  Lanes walk the tile-order side in 16-byte chunks (V elements of one face
// row: one row, V consecutive columns), so that side is read or written in whole lines; the row-major side of a chunk is
// one 16-byte access when it lies inside the row and its address allows it, else up to V element accesses.  grid.y numbers
// the matrices.  Tilize writes zeros into the padding; untilize skips it.
template <typename T, bool TILIZE>
__global__ __launch_bounds__(256) void ttm_tile_ragged_k(const T *__restrict__ src, T *__restrict__ dst, uint32_t rows, uint32_t cols,
                                                         uint32_t pr, uint32_t pc) {
  constexpr uint32_t V = 16 / sizeof(T);
  const uint32_t chunks = pr / V * pc, ct = pc / 32;
  const int64_t b = blockIdx.y;
  const T *rm_src = src + b * rows * (int64_t)cols;
  T *rm_dst = dst + b * rows * (int64_t)cols;
  const chunk_t *t_src = (const chunk_t *)(src + b * pr * (int64_t)pc);
  chunk_t *t_dst = (chunk_t *)(dst + b * pr * (int64_t)pc);
  for (uint32_t ch = blockIdx.x * 256 + threadIdx.x; ch < chunks; ch += gridDim.x * 256) {
    const uint32_t e0 = ch * V, tile = e0 >> 10, e = e0 & 1023, face = e >> 8;
    const uint32_t tr = tile / ct, tc = tile - tr * ct;
    const uint32_t r = tr * 32 + (face >> 1) * 16 + ((e >> 4) & 15), c0 = tc * 32 + (face & 1) * 16 + (e & 15);
    const bool row_in = r < rows;
    const int64_t off = (int64_t)r * cols + c0;
    if (TILIZE) {
      chunk_t v = {0, 0, 0, 0};
      if (row_in && c0 < cols) {
        const T *p = rm_src + off;
        if (c0 + V <= cols && ((uintptr_t)p & 15) == 0) {
          v = __builtin_nontemporal_load((const chunk_t *)p);
        } else {
          T t[V];
#pragma unroll
          for (uint32_t j = 0; j < V; ++j) t[j] = c0 + j < cols ? p[j] : T(0);
          v = *(const chunk_t *)t;
        }
      }
      __builtin_nontemporal_store(v, t_dst + ch);
    } else if (row_in && c0 < cols) {
      const chunk_t v = __builtin_nontemporal_load(t_src + ch);
      T *p = rm_dst + off;
      if (c0 + V <= cols && ((uintptr_t)p & 15) == 0) {
        __builtin_nontemporal_store(v, (chunk_t *)p);
      } else {
        T t[V];
        *(chunk_t *)t = v;
#pragma unroll
        for (uint32_t j = 0; j < V; ++j)
          if (c0 + j < cols) p[j] = t[j];
      }
    }
  }
}

// Untilize of a ragged shape whose rows are whole 16-byte chunks (cols a multiple of V, destination 16-byte aligned): lanes
// walk the row-major destination, so the stores are whole lines, and fetch each chunk from its face row on the tile side.
template <typename T>
__global__ __launch_bounds__(256) void ttm_untilize_rows_k(const T *__restrict__ src, T *__restrict__ dst, uint32_t rows, uint32_t cols,
                                                           uint32_t pr, uint32_t pc) {
  constexpr uint32_t V = 16 / sizeof(T);
  const uint32_t cpr = cols / V, chunks = rows * cpr, ct = pc / 32;
  const int64_t b = blockIdx.y;
  const chunk_t *t_src = (const chunk_t *)(src + b * pr * (int64_t)pc);
  chunk_t *o = (chunk_t *)(dst + b * rows * (int64_t)cols);
  for (uint32_t i = blockIdx.x * 256 + threadIdx.x; i < chunks; i += gridDim.x * 256) {
    const uint32_t r = i / cpr, c0 = (i - r * cpr) * V;
    const uint32_t e = ((r >> 5) * ct + (c0 >> 5)) * 1024 + (((r >> 4) & 1) * 2 + ((c0 >> 4) & 1)) * 256 + (r & 15) * 16 + (c0 & 15);
    __builtin_nontemporal_store(__builtin_nontemporal_load(t_src + e / V), o + i);
  }
}

template <bool TILIZE>
static int run_layout(const void *src, void *dst, int64_t batch, int64_t rows, int64_t cols, int elem,
                      void *stream, const char *who) {
  TTM_REQUIRE(batch >= 0 && rows >= 0 && cols >= 0, "%s: negative dimension", who);
  TTM_REQUIRE(elem == 1 || elem == 2 || elem == 4, "%s: elem_bytes must be 1, 2 or 4 (got %d)", who, elem);
  if (batch == 0 || rows == 0 || cols == 0) return TTM_OK;
  TTM_REQUIRE(src && dst, "%s: null pointer", who);
  TTM_REQUIRE(src != dst, "%s: in-place conversion is not supported", who);
  hipStream_t s = (hipStream_t)stream;
  const int64_t pr = ttm_round_up32(rows), pc = ttm_round_up32(cols);
  const bool aligned = rows == pr && cols == pc && ((uintptr_t)src & 15) == 0 && ((uintptr_t)dst & 15) == 0;
  if (!aligned && batch <= 65535 && pr * pc < ((int64_t)1 << 31) && rows * cols < ((int64_t)1 << 31) &&
      ((uintptr_t)(TILIZE ? dst : src) & 15) == 0 &&   // the tile-order side moves in whole 16-byte chunks
      (TILIZE || elem > 1 || cols % 16 == 0)) {       // bytes into rows that are not whole chunks: the element-wise kernel is faster
    if (!TILIZE && cols % (16 / elem) == 0 && ((uintptr_t)dst & 15) == 0) {
      const int64_t rchunks = rows * cols * elem / 16;
      const dim3 rgrid((unsigned)(ttm_cdiv(rchunks, 256) > 262144 ? 262144 : ttm_cdiv(rchunks, 256)), (unsigned)batch);
#define ROWS(T) \
  hipLaunchKernelGGL((ttm_untilize_rows_k<T>), rgrid, dim3(256), 0, s, (const T *)src, (T *)dst, (uint32_t)rows, (uint32_t)cols, (uint32_t)pr, \
                     (uint32_t)pc)
      if (elem == 4) ROWS(uint32_t);
      else if (elem == 2) ROWS(uint16_t);
      else ROWS(uint8_t);
#undef ROWS
      TTM_LAUNCH_CHECK();
      return TTM_OK;
    }
    const int64_t chunks = pr * pc * elem / 16;
    const dim3 grid((unsigned)(ttm_cdiv(chunks, 256) > 262144 ? 262144 : ttm_cdiv(chunks, 256)), (unsigned)batch);
#define RAGGED(T) \
  hipLaunchKernelGGL((ttm_tile_ragged_k<T, TILIZE>), grid, dim3(256), 0, s, (const T *)src, (T *)dst, (uint32_t)rows, (uint32_t)cols, \
                     (uint32_t)pr, (uint32_t)pc)
    if (elem == 4) RAGGED(uint32_t);
    else if (elem == 2) RAGGED(uint16_t);
    else RAGGED(uint8_t);
#undef RAGGED
    TTM_LAUNCH_CHECK();
    return TTM_OK;
  }
  if (!aligned) {
    int64_t n = batch * pr * pc;
    unsigned blocks = (unsigned)(ttm_cdiv(n, 256) > 1048576 ? 1048576 : ttm_cdiv(n, 256));
#define SCALAR(T) \
  hipLaunchKernelGGL((ttm_tile_scalar_k<T, TILIZE>), dim3(blocks), dim3(256), 0, s, (const T *)src, (T *)dst, \
                     batch, rows, cols, pr, pc)
    if (elem == 4) SCALAR(uint32_t);
    else if (elem == 2) SCALAR(uint16_t);
    else SCALAR(uint8_t);
#undef SCALAR
    TTM_LAUNCH_CHECK();
    return TTM_OK;
  }
  const int64_t yt = batch * (pr / 32), xt = pc / 32;
  const int64_t total_chunks = yt * xt * 64 * elem;
  const int variant = ttm_option(TILIZE ? "tilize_variant" : "untilize_variant");
  const int64_t row_bytes = cols * elem;
  if (variant == 0 && row_bytes % 512 == 0) {
    int64_t strips_per_row = row_bytes / 512;
    int64_t blocks = yt * strips_per_row;
    TTM_REQUIRE(blocks < (1ll << 31), "%s: tensor too large", who);
#define STRIP(E) \
  hipLaunchKernelGGL((ttm_tile_strip_k<E, TILIZE>), dim3((unsigned)blocks), dim3(256), 0, s, \
                     (const chunk_t *)src, (chunk_t *)dst, xt, strips_per_row)
    if (elem == 4) STRIP(4);
    else if (elem == 2) STRIP(2);
    else STRIP(1);
#undef STRIP
  } else {
    int64_t blocks = ttm_cdiv(total_chunks, 1024);
    TTM_REQUIRE(blocks < (1ll << 31), "%s: tensor too large", who);
#define DIRECT(E) \
  hipLaunchKernelGGL((ttm_tile_direct_k<E, TILIZE>), dim3((unsigned)blocks), dim3(256), 0, s, \
                     (const chunk_t *)src, (chunk_t *)dst, yt, xt, total_chunks)
    if (elem == 4) DIRECT(4);
    else if (elem == 2) DIRECT(2);
    else DIRECT(1);
#undef DIRECT
  }
  TTM_LAUNCH_CHECK();
  return TTM_OK;
}

TTM_EXPORT int ttm_tilize(const void *src, void *dst, int64_t batch, int64_t rows, int64_t cols,
                          int elem_bytes, void *stream) {
  TTM_EXTENTS(tilize, src, dst, batch, rows, cols, elem_bytes);
  return run_layout<true>(src, dst, batch, rows, cols, elem_bytes, stream, "ttm_tilize");
}

TTM_EXPORT int ttm_untilize(const void *src, void *dst, int64_t batch, int64_t rows, int64_t cols,
                            int elem_bytes, void *stream) {
  TTM_EXTENTS(untilize, src, dst, batch, rows, cols, elem_bytes);
  return run_layout<false>(src, dst, batch, rows, cols, elem_bytes, stream, "ttm_untilize");
}
