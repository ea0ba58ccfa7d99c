// Index-driven ops around the attention / MLP path of a decoder layer: embedding lookup, argmax over rows, arange.
// All three are row-major on both sides (what ::ttnn::embedding, ::ttnn::argmax and ::ttnn::arange take and give on the
// host side of the reference); the caller converts layouts around them.
#include "ttm_common.h"

namespace {

// out[r, :] = weight[clamp(idx[r], 0, vocab - 1), :]; a lane moves `VEC` bytes
template <typename V>
__global__ __launch_bounds__(256) void ttm_embedding_k(const int32_t *__restrict__ idx, const V *__restrict__ weight, V *__restrict__ out,
                                                       int64_t rows, int64_t vocab, int64_t row_vecs, int idx_unsigned) {
  const int64_t total = rows * row_vecs;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
    const int64_t r = i / row_vecs, c = i % row_vecs;
    int64_t t = idx_unsigned ? (int64_t)(uint32_t)idx[r] : (int64_t)idx[r];
    t = t < 0 ? 0 : (t >= vocab ? vocab - 1 : t);
    out[i] = weight[t * row_vecs + c];
  }
}

// one wavefront per row: index of the first largest element; NaN counts as the largest value, as in torch.argmax
template <bool BF16>
__global__ __launch_bounds__(256) void ttm_argmax_k(const void *__restrict__ in, int32_t *__restrict__ out, int64_t rows, int64_t cols) {
  const int lane = threadIdx.x & 63;
  const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= rows) return;
  float best = -INFINITY;
  int64_t at = INT64_MAX;
  bool best_nan = false;
  for (int64_t c = lane; c < cols; c += 64) {
    const float x = BF16 ? __uint_as_float((uint32_t)((const uint16_t *)in)[row * cols + c] << 16) : ((const float *)in)[row * cols + c];
    const bool nan = x != x;
    // strictly better, or the first element seen (at == INT64_MAX): columns are visited in increasing order per lane
    if (at == INT64_MAX || (!best_nan && (nan || x > best))) { best = x; at = c; best_nan = nan; }
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    const float ob = __shfl_xor(best, o);
    const int64_t oa = __shfl_xor((long long)at, o);
    const bool on = __shfl_xor((int)best_nan, o) != 0;
    bool take;
    if (oa == INT64_MAX) take = false;
    else if (at == INT64_MAX) take = true;
    else if (on != best_nan) take = on;                 // NaN beats a number
    else if (on) take = oa < at;                        // both NaN: the earlier one
    else take = ob > best || (ob == best && oa < at);
    if (take) { best = ob; at = oa; best_nan = on; }
  }
  if (lane == 0) out[row] = (int32_t)(at == INT64_MAX ? 0 : at);
}

// Long rows (a vocabulary) in two steps: grid (parts, rows) workgroups each scan one slice of a row, 16 bytes per load where
// the row starts allow it, and leave (value, index) of their first largest element; a second kernel merges the parts of a
// row.  Candidates compare as in the one-wavefront kernel: NaN beats numbers, equal values go to the smaller index.
struct ArgBest {
  float v;
  int32_t at;     // -1: nothing seen yet
};
__device__ __forceinline__ void arg_take(ArgBest &b, float x, int32_t c) {
  const bool bnan = b.v != b.v, xnan = x != x;
  if (b.at < 0 || (!bnan && (xnan || x > b.v))) { b.v = x; b.at = c; }   // strictly better: columns come in increasing order
}
__device__ __forceinline__ void arg_merge(ArgBest &b, float ov, int32_t oa) {
  if (oa < 0) return;
  const bool bnan = b.v != b.v, onan = ov != ov;
  bool take;
  if (b.at < 0) take = true;
  else if (onan != bnan) take = onan;
  else if (onan) take = oa < b.at;
  else take = ov > b.v || (ov == b.v && oa < b.at);
  if (take) { b.v = ov; b.at = oa; }
}
__device__ __forceinline__ void arg_wave_merge(ArgBest &b) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    const float ov = __shfl_xor(b.v, o);
    const int32_t oa = __shfl_xor(b.at, o);
    arg_merge(b, ov, oa);
  }
}

template <bool BF16, bool VEC>
__global__ __launch_bounds__(256) void ttm_argmax_part_k(const void *__restrict__ in, float *__restrict__ part_v, int32_t *__restrict__ part_at,
                                                         int64_t cols, int64_t slice) {
  __shared__ float sv[4];
  __shared__ int32_t sa[4];
  constexpr int V = BF16 ? 8 : 4;
  const int64_t row = blockIdx.y, c0 = (int64_t)blockIdx.x * slice, c1 = min(c0 + slice, cols);
  ArgBest b = {0.0f, -1};
  if (VEC) {   // slice and row starts are multiples of V elements
    const u32x4 *base = (const u32x4 *)((const uint8_t *)in + (row * cols + c0) * (BF16 ? 2 : 4));
    const int64_t nv = (c1 - c0) / V;
    for (int64_t g0 = threadIdx.x; g0 < nv; g0 += 1024) {   // four loads in flight per lane
      u32x4 q[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) q[u] = __builtin_nontemporal_load(base + min(g0 + 256 * u, nv - 1));
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int64_t g = g0 + 256 * u;
        if (g < nv) {
          const int32_t c = (int32_t)(c0 + g * V);
#pragma unroll
          for (int j = 0; j < V; ++j) {
            const float x = BF16 ? __uint_as_float((j & 1) ? (q[u][j / 2] & 0xFFFF0000u) : (q[u][j / 2] << 16)) : __uint_as_float(q[u][j]);
            arg_take(b, x, c + j);
          }
        }
      }
    }
    for (int64_t c = c0 + nv * V + threadIdx.x; c < c1; c += 256) {   // the last, partial group of the row
      const float x = BF16 ? __uint_as_float((uint32_t)((const uint16_t *)in)[row * cols + c] << 16) : ((const float *)in)[row * cols + c];
      arg_merge(b, x, (int32_t)c);
    }
  } else {
    for (int64_t c = c0 + threadIdx.x; c < c1; c += 256) {
      const float x = BF16 ? __uint_as_float((uint32_t)((const uint16_t *)in)[row * cols + c] << 16) : ((const float *)in)[row * cols + c];
      arg_take(b, x, (int32_t)c);
    }
  }
  arg_wave_merge(b);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  if (lane == 0) { sv[wave] = b.v; sa[wave] = b.at; }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < 4; ++w) arg_merge(b, sv[w], sa[w]);
    part_v[row * gridDim.x + blockIdx.x] = b.v;
    part_at[row * gridDim.x + blockIdx.x] = b.at;
  }
}

// one wavefront per row over its parts
__global__ __launch_bounds__(256) void ttm_argmax_merge_k(const float *__restrict__ part_v, const int32_t *__restrict__ part_at, int32_t *__restrict__ out,
                                                          int64_t rows, int parts) {
  const int lane = threadIdx.x & 63;
  const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= rows) return;
  ArgBest b = {0.0f, -1};
  for (int i = lane; i < parts; i += 64) arg_merge(b, part_v[row * parts + i], part_at[row * parts + i]);
  arg_wave_merge(b);
  if (lane == 0) out[row] = b.at < 0 ? 0 : b.at;
}

template <int DT>
__global__ __launch_bounds__(256) void ttm_arange_k(void *__restrict__ out, int64_t n, double start, double step) {
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (int64_t)gridDim.x * 256) {
    // torch.arange in float32 (start + i * step, computed wide and rounded once), then the cast to the result type
    const float f = (float)(start + (double)i * step);
    if (DT == TTM_F32) ((float *)out)[i] = f;
    else if (DT == TTM_BF16) ((uint16_t *)out)[i] = ttm_f32_to_bf16(f);
    else if (DT == TTM_I32) ((int32_t *)out)[i] = (int32_t)f;
    else ((uint32_t *)out)[i] = f <= 0.0f ? 0u : (uint32_t)f;
  }
}

unsigned grid_of(int64_t items) {
  int64_t g = (items + 255) / 256;
  return (unsigned)(g < 1 ? 1 : (g > 65536 ? 65536 : g));
}

}  // namespace

TTM_EXPORT int ttm_embedding(const void *indices, int index_dtype, const void *weight, void *out, int elem_bytes, int64_t rows,
                             int64_t vocab, int64_t dim, void *stream) {
  TTM_EXTENTS(embedding, indices, weight, out, elem_bytes, rows, vocab, dim);
  TTM_REQUIRE(index_dtype == TTM_I32 || index_dtype == TTM_U32, "ttm_embedding: indices must be Int32 or UInt32 (got %d)", index_dtype);
  TTM_REQUIRE(elem_bytes == 2 || elem_bytes == 4, "ttm_embedding: element size must be 2 or 4 bytes");
  TTM_REQUIRE(rows >= 0 && vocab > 0 && dim > 0, "ttm_embedding: bad extents");
  if (rows == 0) return TTM_OK;
  TTM_REQUIRE(indices && weight && out, "ttm_embedding: null pointer");
  const int64_t row_bytes = dim * elem_bytes;
  const bool wide = row_bytes % 16 == 0 && (((uintptr_t)weight | (uintptr_t)out) & 15) == 0;
  hipStream_t s = (hipStream_t)stream;
  const int uns = index_dtype == TTM_U32;
  if (wide)
    hipLaunchKernelGGL(ttm_embedding_k<u32x4>, dim3(grid_of(rows * (row_bytes / 16))), dim3(256), 0, s, (const int32_t *)indices,
                       (const u32x4 *)weight, (u32x4 *)out, rows, vocab, row_bytes / 16, uns);
  else if (elem_bytes == 4)
    hipLaunchKernelGGL(ttm_embedding_k<uint32_t>, dim3(grid_of(rows * dim)), dim3(256), 0, s, (const int32_t *)indices,
                       (const uint32_t *)weight, (uint32_t *)out, rows, vocab, dim, uns);
  else
    hipLaunchKernelGGL(ttm_embedding_k<uint16_t>, dim3(grid_of(rows * dim)), dim3(256), 0, s, (const int32_t *)indices,
                       (const uint16_t *)weight, (uint16_t *)out, rows, vocab, dim, uns);
  TTM_LAUNCH_CHECK();
  return TTM_OK;
}

TTM_EXPORT int ttm_argmax(const void *in, int dtype, int32_t *out, int64_t rows, int64_t cols, void *stream) {
  TTM_EXTENTS(argmax, in, dtype, out, rows, cols);
  TTM_REQUIRE(dtype == TTM_BF16 || dtype == TTM_F32, "ttm_argmax: dtype must be BFloat16 or Float32 (got %d)", dtype);
  TTM_REQUIRE(rows >= 0 && cols > 0 && cols <= INT32_MAX, "ttm_argmax: bad extents");
  if (rows == 0) return TTM_OK;
  TTM_REQUIRE(in && out, "ttm_argmax: null pointer");
  TTM_REQUIRE((rows + 3) / 4 <= 0x7FFFFFFF, "ttm_argmax: too many rows");
  // rows too long for one wavefront each: slices of at least 2048 columns, enough of them for about 2048 workgroups
  if (cols >= 8192 && rows <= 65535) {
    const int es = dtype == TTM_BF16 ? 2 : 4, V = 16 / es;
    int64_t parts = ttm_cdiv(2048, rows);
    if (parts > cols / 2048) parts = cols / 2048;
    if (parts < 1) parts = 1;
    int64_t slice = ttm_cdiv(ttm_cdiv(cols, parts), V) * V;
    parts = ttm_cdiv(cols, slice);
    void *ws = nullptr;
    if (int rc = ttm_stream_workspace((hipStream_t)stream, (size_t)(rows * parts) * 8, &ws)) return rc;
    float *pv = (float *)ws;
    int32_t *pa = (int32_t *)(pv + rows * parts);
    const bool vec = ((uintptr_t)in & 15) == 0 && (cols * es) % 16 == 0;
    const dim3 pgrid((unsigned)parts, (unsigned)rows);
    hipStream_t s = (hipStream_t)stream;
    if (dtype == TTM_BF16) {
      if (vec) hipLaunchKernelGGL((ttm_argmax_part_k<true, true>), pgrid, dim3(256), 0, s, in, pv, pa, cols, slice);
      else hipLaunchKernelGGL((ttm_argmax_part_k<true, false>), pgrid, dim3(256), 0, s, in, pv, pa, cols, slice);
    } else {
      if (vec) hipLaunchKernelGGL((ttm_argmax_part_k<false, true>), pgrid, dim3(256), 0, s, in, pv, pa, cols, slice);
      else hipLaunchKernelGGL((ttm_argmax_part_k<false, false>), pgrid, dim3(256), 0, s, in, pv, pa, cols, slice);
    }
    TTM_LAUNCH_CHECK();
    hipLaunchKernelGGL(ttm_argmax_merge_k, dim3((unsigned)((rows + 3) / 4)), dim3(256), 0, s, pv, pa, out, rows, (int)parts);
    TTM_LAUNCH_CHECK();
    return TTM_OK;
  }
  const dim3 grid((unsigned)((rows + 3) / 4));
  if (dtype == TTM_BF16) hipLaunchKernelGGL(ttm_argmax_k<true>, grid, dim3(256), 0, (hipStream_t)stream, in, out, rows, cols);
  else hipLaunchKernelGGL(ttm_argmax_k<false>, grid, dim3(256), 0, (hipStream_t)stream, in, out, rows, cols);
  TTM_LAUNCH_CHECK();
  return TTM_OK;
}

TTM_EXPORT int ttm_arange(void *out, int dtype, int64_t n, double start, double step, void *stream) {
  TTM_EXTENTS(arange, out, dtype, n);
  TTM_REQUIRE(n >= 0, "ttm_arange: negative length");
  if (n == 0) return TTM_OK;
  TTM_REQUIRE(out != nullptr, "ttm_arange: null pointer");
  hipStream_t s = (hipStream_t)stream;
  const dim3 grid(grid_of(n));
  switch (dtype) {
  case TTM_F32: hipLaunchKernelGGL(ttm_arange_k<TTM_F32>, grid, dim3(256), 0, s, out, n, start, step); break;
  case TTM_BF16: hipLaunchKernelGGL(ttm_arange_k<TTM_BF16>, grid, dim3(256), 0, s, out, n, start, step); break;
  case TTM_I32: hipLaunchKernelGGL(ttm_arange_k<TTM_I32>, grid, dim3(256), 0, s, out, n, start, step); break;
  case TTM_U32: hipLaunchKernelGGL(ttm_arange_k<TTM_U32>, grid, dim3(256), 0, s, out, n, start, step); break;
  default: return ttm_set_error(TTM_ERR_INVALID, "ttm_arange: dtype must be Float32, BFloat16, Int32 or UInt32 (got %d)", dtype);
  }
  TTM_LAUNCH_CHECK();
  return TTM_OK;
}
