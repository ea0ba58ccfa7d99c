// Bandwidth-bound elementwise kernels: unary, binary (with broadcasting), typecast.
// Values are computed in fp32 and stored in the tensor dtype (the CPU path converts to f32,
// computes, and casts back).  Kernels that do not need coordinates run over the flat padded buffer
// 16 bytes per lane; broadcasting binaries decode tile coordinates per element.
#include <hip/hip_fp16.h>

#include <initializer_list>
#include <type_traits>

#include "ttm_common.h"
#include "ttm_math.h"

// op codes = EltwiseUnaryOpType / EltwiseBinaryOpType values of the TTNN flatbuffer schema
enum { U_ABS = 0, U_CEIL, U_COS, U_FLOOR, U_GELU, U_ISFINITE, U_LOGICALNOT, U_NEG, U_RELU, U_SQRT,
       U_RSQRT, U_SIGMOID, U_SIN, U_RECIPROCAL, U_SIGN, U_TAN, U_TANH, U_ATAN, U_EXP, U_ERF, U_ERFC,
       U_LOG, U_EXPM1, U_LEAKYRELU, U_BITWISENOT, U_RELU6, U_SILU, U_HARDSIGMOID, U_MISH, U_ACOS, U_ASIN, U_ASINH,
       // 100 + EltwiseUnaryCompositeOpType (ClampTensor, 102, is a ternary and has no kernel here)
       U_CBRT = 100, U_CLAMP = 101, U_LOG1P = 103 };
enum { B_ADD = 0, B_MUL = 1, B_SUB = 3, B_EQ = 4, B_NE = 5, B_GE = 6, B_GT = 7, B_LE = 8, B_LT = 9, B_DIV = 10,
       B_AND = 11, B_OR = 12, B_XOR = 13,
       // 100 + EltwiseBinaryCompositeOpType
       B_MAXIMUM = 100, B_MINIMUM = 101, B_REMAINDER = 102, B_POW = 103, B_ATAN2 = 104 };

template <int OP>
__device__ __forceinline__ float unary_op(float x, float p, float p2 = 0.0f) {
  switch (OP) {
  case U_ABS: return fabsf(x);
  case U_CEIL: return ceilf(x);
  case U_COS: return cosf(x);
  case U_FLOOR: return floorf(x);
  case U_GELU: return ttm_gelu_erf(x);
  case U_ISFINITE: return isfinite(x) ? 1.0f : 0.0f;
  case U_LOGICALNOT: return x == 0.0f ? 1.0f : 0.0f;
  case U_NEG: return -x;
  case U_RELU: return x > 0.0f ? x : (x != x ? x : 0.0f);   // NaN stays NaN, as arith.maximumf and torch.relu have it
  case U_SQRT: return sqrtf(x);
  case U_RSQRT: return 1.0f / sqrtf(x);
  case U_SIGMOID: return 1.0f / (1.0f + expf(-x));
  case U_SIN: return sinf(x);
  case U_RECIPROCAL: return 1.0f / x;
  case U_SIGN: return (float)((x > 0.0f) - (x < 0.0f));
  case U_TAN: return tanf(x);
  case U_TANH: return tanhf(x);
  case U_ATAN: return atanf(x);
  case U_EXP: return expf(x);
  case U_ERF: return erff(x);
  case U_ERFC: return erfcf(x);
  case U_LOG: return logf(x);
  case U_EXPM1: return expm1f(x);
  case U_LEAKYRELU: return x > 0.0f ? x : p * x;
  case U_RELU6: return fminf(fmaxf(x, 0.0f), 6.0f);
  case U_SILU: return x * (1.0f / (1.0f + expf(-x)));
  case U_HARDSIGMOID: return fminf(fmaxf(x + 3.0f, 0.0f), 6.0f) * (1.0f / 6.0f) + (x != x ? x : 0.0f);   // relu6(x + 3) / 6
  case U_MISH: return x * tanhf(x > 20.0f ? x : log1pf(expf(x)));                                       // x tanh(softplus(x))
  case U_ACOS: return acosf(x);
  case U_ASIN: return asinf(x);
  case U_ASINH: return asinhf(x);
  case U_CBRT: return cbrtf(x);
  case U_CLAMP: return x != x ? x : fminf(fmaxf(x, p), p2);                                               // torch.clamp: NaN stays
  case U_LOG1P: return log1pf(x);
  default: return x;
  }
}

__device__ __forceinline__ float binary_op(int op, float a, float b) {
  switch (op) {
  case B_ADD: return a + b;
  case B_MUL: return a * b;
  case B_SUB: return a - b;
  case B_EQ: return a == b ? 1.0f : 0.0f;
  case B_NE: return a != b ? 1.0f : 0.0f;
  case B_GE: return a >= b ? 1.0f : 0.0f;
  case B_GT: return a > b ? 1.0f : 0.0f;
  case B_LE: return a <= b ? 1.0f : 0.0f;
  case B_LT: return a < b ? 1.0f : 0.0f;
  case B_DIV: return a / b;
  case B_AND: return (a != 0.0f && b != 0.0f) ? 1.0f : 0.0f;
  case B_OR: return (a != 0.0f || b != 0.0f) ? 1.0f : 0.0f;
  case B_XOR: return ((a != 0.0f) != (b != 0.0f)) ? 1.0f : 0.0f;
  case B_MAXIMUM: return (a != a || b != b) ? NAN : fmaxf(a, b);   // NaN propagates, as in torch.maximum
  case B_MINIMUM: return (a != a || b != b) ? NAN : fminf(a, b);
  case B_REMAINDER: {   // sign of the divisor, as torch.remainder
    const float r = fmodf(a, b);
    return (r != 0.0f && ((r < 0.0f) != (b < 0.0f))) ? r + b : r;
  }
  case B_POW: return powf(a, b);
  case B_ATAN2: return atan2f(a, b);
  default: return a;
  }
}

template <bool BF16>
__device__ __forceinline__ void chunk_load(const void *p, int64_t chunk, float (&f)[BF16 ? 8 : 4]) {
  u32x4 v = ((const u32x4 *)p)[chunk];
  if (BF16) {
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
template <bool BF16>
__device__ __forceinline__ void chunk_store(void *p, int64_t chunk, const float (&f)[BF16 ? 8 : 4]) {
  u32x4 v;
  if (BF16) {
#pragma unroll
    for (int i = 0; i < 4; ++i) v[i] = ttm_pack_bf16x2(f[2 * i], f[2 * i + 1]);
  } else {
#pragma unroll
    for (int i = 0; i < 4; ++i) v[i] = __float_as_uint(f[i]);
  }
  ((u32x4 *)p)[chunk] = v;
}

template <int OP, bool BF16>
__global__ __launch_bounds__(256) void ttm_unary_k(const void *__restrict__ in, void *__restrict__ out, int64_t nchunks,
                                                   int64_t n, float param, float param2) {
  constexpr int EPC = BF16 ? 8 : 4;
  for (int64_t c = (int64_t)blockIdx.x * 256 + threadIdx.x; c < nchunks; c += (int64_t)gridDim.x * 256) {
    if ((c + 1) * EPC <= n) {
      float f[EPC];
      chunk_load<BF16>(in, c, f);
#pragma unroll
      for (int i = 0; i < EPC; ++i) f[i] = unary_op<OP>(f[i], param, param2);
      chunk_store<BF16>(out, c, f);
    } else {  // ragged tail
      for (int64_t i = c * EPC; i < n; ++i) {
        float x = BF16 ? ttm_bf16_to_f32(((const uint16_t *)in)[i]) : ((const float *)in)[i];
        float y = unary_op<OP>(x, param, param2);
        if (BF16) ((uint16_t *)out)[i] = ttm_f32_to_bf16(y);
        else ((float *)out)[i] = y;
      }
    }
  }
}

// ragged tile-order tensors: padding must stay zero (it feeds later contractions), so decode coordinates
template <int OP, bool BF16>
__global__ __launch_bounds__(256) void ttm_unary_masked_k(const void *__restrict__ in, void *__restrict__ out,
                                                          int64_t total, int64_t rows, int64_t cols, float param, float param2) {
  const int64_t pr = (rows + 31) / 32 * 32, pc = (cols + 31) / 32 * 32;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
    int64_t w = i % (pr * pc), tile = w >> 10;
    int e = (int)(w & 1023), face = e >> 8;
    int64_t r = (tile / (pc / 32)) * 32 + (face >> 1) * 16 + ((e >> 4) & 15);
    int64_t c = (tile % (pc / 32)) * 32 + (face & 1) * 16 + (e & 15);
    float y = 0.0f;
    if (r < rows && c < cols) {
      float x = BF16 ? ttm_bf16_to_f32(((const uint16_t *)in)[i]) : ((const float *)in)[i];
      y = unary_op<OP>(x, param, param2);
    }
    if (BF16) ((uint16_t *)out)[i] = ttm_f32_to_bf16(y);
    else ((float *)out)[i] = y;
  }
}

typedef void (*unary_fn)(const void *, void *, int64_t, int64_t, float, float);
typedef void (*unary_masked_fn)(const void *, void *, int64_t, int64_t, int64_t, float, float);

template <bool BF16>
static unary_fn pick_unary(int op) {
#define U(OP) case OP: return ttm_unary_k<OP, BF16>;
  switch (op) {
    U(U_ABS) U(U_CEIL) U(U_COS) U(U_FLOOR) U(U_GELU) U(U_ISFINITE) U(U_LOGICALNOT) U(U_NEG) U(U_RELU) U(U_SQRT)
    U(U_RSQRT) U(U_SIGMOID) U(U_SIN) U(U_RECIPROCAL) U(U_SIGN) U(U_TAN) U(U_TANH) U(U_ATAN) U(U_EXP) U(U_ERF)
    U(U_ERFC) U(U_LOG) U(U_EXPM1) U(U_LEAKYRELU) U(U_RELU6) U(U_SILU) U(U_HARDSIGMOID) U(U_MISH) U(U_ACOS) U(U_ASIN)
    U(U_ASINH) U(U_CBRT) U(U_CLAMP) U(U_LOG1P)
  default: return nullptr;
  }
#undef U
}
template <bool BF16>
static unary_masked_fn pick_unary_masked(int op) {
#define U(OP) case OP: return ttm_unary_masked_k<OP, BF16>;
  switch (op) {
    U(U_ABS) U(U_CEIL) U(U_COS) U(U_FLOOR) U(U_GELU) U(U_ISFINITE) U(U_LOGICALNOT) U(U_NEG) U(U_RELU) U(U_SQRT)
    U(U_RSQRT) U(U_SIGMOID) U(U_SIN) U(U_RECIPROCAL) U(U_SIGN) U(U_TAN) U(U_TANH) U(U_ATAN) U(U_EXP) U(U_ERF)
    U(U_ERFC) U(U_LOG) U(U_EXPM1) U(U_LEAKYRELU) U(U_RELU6) U(U_SILU) U(U_HARDSIGMOID) U(U_MISH) U(U_ACOS) U(U_ASIN)
    U(U_ASINH) U(U_CBRT) U(U_CLAMP) U(U_LOG1P)
  default: return nullptr;
  }
#undef U
}

// the same in 16-byte chunks: a chunk lies in one face row, so one (row, first column) decides which of its elements are
// padding; grid.y numbers the matrices
template <int OP, bool BF16>
__global__ __launch_bounds__(256) void ttm_unary_masked_chunk_k(const void *__restrict__ in, void *__restrict__ out, uint32_t chunks_per_plane,
                                                                uint32_t rows, uint32_t cols, float param, float param2) {
  constexpr int EPC = BF16 ? 8 : 4;
  const uint32_t tcols = (cols + 31) >> 5;
  const int64_t base = (int64_t)blockIdx.y * chunks_per_plane;
  for (uint32_t ci = blockIdx.x * 256 + threadIdx.x; ci < chunks_per_plane; ci += gridDim.x * 256) {
    const uint32_t w = ci * EPC, tile = w >> 10, e = w & 1023, face = e >> 8;
    const uint32_t r = (tile / tcols) * 32 + (face >> 1) * 16 + ((e >> 4) & 15), c0 = (tile % tcols) * 32 + (face & 1) * 16 + (e & 15);
    float f[EPC];
#pragma unroll
    for (int i = 0; i < EPC; ++i) f[i] = 0.0f;
    if (r < rows && c0 < cols) {
      chunk_load<BF16>(in, base + ci, f);
#pragma unroll
      for (int i = 0; i < EPC; ++i) f[i] = c0 + i < cols ? unary_op<OP>(f[i], param, param2) : 0.0f;
    }
    chunk_store<BF16>(out, base + ci, f);
  }
}
typedef void (*unary_chunk_fn)(const void *, void *, uint32_t, uint32_t, uint32_t, float, float);
template <bool BF16>
static unary_chunk_fn pick_unary_masked_chunk(int op) {
#define U(OP) case OP: return ttm_unary_masked_chunk_k<OP, BF16>;
  switch (op) {
    U(U_ABS) U(U_CEIL) U(U_COS) U(U_FLOOR) U(U_GELU) U(U_ISFINITE) U(U_LOGICALNOT) U(U_NEG) U(U_RELU) U(U_SQRT)
    U(U_RSQRT) U(U_SIGMOID) U(U_SIN) U(U_RECIPROCAL) U(U_SIGN) U(U_TAN) U(U_TANH) U(U_ATAN) U(U_EXP) U(U_ERF)
    U(U_ERFC) U(U_LOG) U(U_EXPM1) U(U_LEAKYRELU) U(U_RELU6) U(U_SILU) U(U_HARDSIGMOID) U(U_MISH) U(U_ACOS) U(U_ASIN)
    U(U_ASINH) U(U_CBRT) U(U_CLAMP) U(U_LOG1P)
  default: return nullptr;
  }
#undef U
}

static unsigned grid_for(int64_t nchunks) {
  int64_t b = ttm_cdiv(nchunks, 256);
  return (unsigned)(b > 262144 ? 262144 : (b < 1 ? 1 : b));
}

static int unary_entry(int op, const void *in, void *out, int dtype, int layout, int64_t batch, int64_t rows, int64_t cols, float param,
                       float param2, void *stream) {
  TTM_REQUIRE(dtype == TTM_BF16 || dtype == TTM_F32, "ttm_eltwise_unary: dtype must be BFloat16 or Float32 (got %d)", dtype);
  TTM_REQUIRE(layout == TTM_ROW_MAJOR || layout == TTM_TILE, "ttm_eltwise_unary: bad layout");
  TTM_REQUIRE(batch >= 0 && rows >= 0 && cols >= 0, "ttm_eltwise_unary: negative dimension");
  const bool tiled = layout == TTM_TILE;
  const int64_t pr = tiled ? ttm_round_up32(rows) : rows, pc = tiled ? ttm_round_up32(cols) : cols;
  const int64_t n = batch * pr * pc;
  if (n == 0) return TTM_OK;
  TTM_REQUIRE(in && out, "ttm_eltwise_unary: null pointer");
  if (tiled && (pr != rows || pc != cols) && batch <= 65535 && pr * pc < ((int64_t)1 << 31) &&
      (((uintptr_t)in | (uintptr_t)out) & 15) == 0) {
    unary_chunk_fn fn = dtype == TTM_BF16 ? pick_unary_masked_chunk<true>(op) : pick_unary_masked_chunk<false>(op);
    if (!fn) return ttm_set_error(TTM_ERR_UNSUPPORTED, "ttm_eltwise_unary: unsupported op %d", op);
    const uint32_t cpp = (uint32_t)(pr * pc * (dtype == TTM_BF16 ? 2 : 4) / 16);
    hipLaunchKernelGGL(fn, dim3(grid_for(cpp), (unsigned)batch), dim3(256), 0, (hipStream_t)stream, in, out, cpp, (uint32_t)rows, (uint32_t)cols,
                       param, param2);
    TTM_LAUNCH_CHECK();
    return TTM_OK;
  }
  if (tiled && (pr != rows || pc != cols)) {
    unary_masked_fn fn = dtype == TTM_BF16 ? pick_unary_masked<true>(op) : pick_unary_masked<false>(op);
    if (!fn) return ttm_set_error(TTM_ERR_UNSUPPORTED, "ttm_eltwise_unary: unsupported op %d", op);
    hipLaunchKernelGGL(fn, dim3(grid_for(n)), dim3(256), 0, (hipStream_t)stream, in, out, n, rows, cols, param, param2);
    TTM_LAUNCH_CHECK();
    return TTM_OK;
  }
  TTM_REQUIRE(((uintptr_t)in & 15) == 0 && ((uintptr_t)out & 15) == 0, "ttm_eltwise_unary: pointers must be 16-byte aligned");
  unary_fn fn = dtype == TTM_BF16 ? pick_unary<true>(op) : pick_unary<false>(op);
  if (!fn) return ttm_set_error(TTM_ERR_UNSUPPORTED, "ttm_eltwise_unary: unsupported op %d", op);
  const int epc = dtype == TTM_BF16 ? 8 : 4;
  int64_t nchunks = ttm_cdiv(n, epc);
  hipLaunchKernelGGL(fn, dim3(grid_for(nchunks)), dim3(256), 0, (hipStream_t)stream, in, out, nchunks, n, param, param2);
  TTM_LAUNCH_CHECK();
  return TTM_OK;
}

TTM_EXPORT int ttm_eltwise_unary(int op, const void *in, void *out, int dtype, int layout, int64_t batch, int64_t rows,
                                 int64_t cols, float param, void *stream) {
  TTM_EXTENTS(unary, in, out, dtype, layout, batch, rows, cols);
  TTM_REQUIRE(op != U_CLAMP, "ttm_eltwise_unary: clamp takes two bounds, use ttm_clamp");
  return unary_entry(op, in, out, dtype, layout, batch, rows, cols, param, 0.0f, stream);
}

TTM_EXPORT int ttm_clamp(const void *in, void *out, int dtype, int layout, int64_t batch, int64_t rows, int64_t cols, float lo, float hi,
                         void *stream) {
  TTM_EXTENTS(unary, in, out, dtype, layout, batch, rows, cols);
  return unary_entry(U_CLAMP, in, out, dtype, layout, batch, rows, cols, lo, hi, stream);
}

// ---- binary, same shape: flat
template <bool BF16>
__global__ __launch_bounds__(256) void ttm_binary_flat_k(int op, const void *__restrict__ a, const void *__restrict__ b,
                                                         void *__restrict__ out, int64_t nchunks) {
  constexpr int EPC = BF16 ? 8 : 4;
  for (int64_t c = (int64_t)blockIdx.x * 256 + threadIdx.x; c < nchunks; c += (int64_t)gridDim.x * 256) {
    float x[EPC], y[EPC];
    chunk_load<BF16>(a, c, x);
    chunk_load<BF16>(b, c, y);
#pragma unroll
    for (int i = 0; i < EPC; ++i) x[i] = binary_op(op, x[i], y[i]);
    chunk_store<BF16>(out, c, x);
  }
}

// ---- binary with broadcasting: shapes right-aligned to rank 4 as [d0, d1, R, C]
struct BcastArgs {
  int64_t oshape[4], ashape[4], bshape[4];
  int tiled;
};

__device__ __forceinline__ int64_t bcast_offset(const int64_t (&shape)[4], int64_t i0, int64_t i1, int64_t r, int64_t c,
                                                int tiled) {
  i0 = shape[0] == 1 ? 0 : i0; i1 = shape[1] == 1 ? 0 : i1;
  r = shape[2] == 1 ? 0 : r; c = shape[3] == 1 ? 0 : c;
  int64_t batch = i0 * shape[1] + i1;
  if (tiled) {
    int64_t pr = (shape[2] + 31) / 32 * 32, pc = (shape[3] + 31) / 32 * 32;
    return batch * pr * pc + ttm_tiled_offset(r, c, pc / 32);
  }
  return (batch * shape[2] + r) * shape[3] + c;
}

template <bool BF16>
__global__ __launch_bounds__(256) void ttm_binary_bcast_k(int op, const void *__restrict__ a, const void *__restrict__ b,
                                                          void *__restrict__ out, BcastArgs p, int64_t total) {
  const int64_t R = p.oshape[2], C = p.oshape[3];
  const int64_t pr = p.tiled ? (R + 31) / 32 * 32 : R, pc = p.tiled ? (C + 31) / 32 * 32 : C;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
    int64_t batch = i / (pr * pc), w = i % (pr * pc), r, c;
    if (p.tiled) {
      int64_t tile = w >> 10;
      int e = (int)(w & 1023);
      int face = e >> 8;
      r = (tile / (pc / 32)) * 32 + (face >> 1) * 16 + ((e >> 4) & 15);
      c = (tile % (pc / 32)) * 32 + (face & 1) * 16 + (e & 15);
    } else {
      r = w / pc; c = w % pc;
    }
    float y = 0.0f;
    if (r < R && c < C) {
      int64_t i0 = batch / p.oshape[1], i1 = batch % p.oshape[1];
      int64_t oa = bcast_offset(p.ashape, i0, i1, r, c, p.tiled), ob = bcast_offset(p.bshape, i0, i1, r, c, p.tiled);
      float x0 = BF16 ? ttm_bf16_to_f32(((const uint16_t *)a)[oa]) : ((const float *)a)[oa];
      float x1 = BF16 ? ttm_bf16_to_f32(((const uint16_t *)b)[ob]) : ((const float *)b)[ob];
      y = binary_op(op, x0, x1);
    }
    if (BF16) ((uint16_t *)out)[i] = ttm_f32_to_bf16(y);
    else ((float *)out)[i] = y;
  }
}

// Broadcasting in 16-byte chunks, for outputs whose chunks never straddle a row: tile layout (ragged extents included: the
// columns of a chunk that lie in the padding are written as zeros), row-major with a multiple of the chunk width.  A chunk is EPC consecutive columns of one row (inside a tile: part of one
// face row), so per chunk one (row, first column) is decoded and every operand is read either as the 16 bytes at its own
// offset for that position (its last dim is the output's) or as one element for the whole chunk (its last dim is 1).
// grid.y numbers the batch entries; rows past R (tile padding) are written as zeros.
struct ChunkPos {
  int64_t i0, i1, r, c0, out_chunk;
  bool live;    // the chunk holds at least one element of the tensor
  int valid;    // how many of its EPC columns do (fewer than EPC only in the last tile column of a ragged tile tensor)
};
template <int EPC>
__device__ __forceinline__ ChunkPos chunk_pos(const int64_t (&oshape)[4], int tiled, uint32_t ci, uint32_t chunks_per_plane) {
  const uint32_t R = (uint32_t)oshape[2], C = (uint32_t)oshape[3];
  ChunkPos q;
  const uint32_t batch = blockIdx.y;
  q.i0 = batch / (uint32_t)oshape[1]; q.i1 = batch % (uint32_t)oshape[1];
  uint32_t r, c0;
  if (tiled) {
    const uint32_t w = ci * EPC, tile = w >> 10, e = w & 1023, face = e >> 8, tcols = (C + 31) >> 5;
    r = (tile / tcols) * 32 + (face >> 1) * 16 + ((e >> 4) & 15);
    c0 = (tile % tcols) * 32 + (face & 1) * 16 + (e & 15);
  } else {
    const uint32_t cpr = C / EPC;
    r = ci / cpr; c0 = (ci % cpr) * EPC;
  }
  q.r = r; q.c0 = c0;
  q.live = r < R && c0 < C;
  q.valid = q.live ? (int)min(C - c0, (uint32_t)EPC) : 0;
  q.out_chunk = (int64_t)batch * chunks_per_plane + ci;
  return q;
}
template <bool BF16, typename F>
__device__ __forceinline__ void operand_chunk(const void *base, const int64_t (&shape)[4], const ChunkPos &q, int tiled, F (&v)[BF16 ? 8 : 4]) {
  constexpr int EPC = BF16 ? 8 : 4;
  const int64_t off = bcast_offset(shape, q.i0, q.i1, q.r, q.c0, tiled);
  if (shape[3] != 1) {
    const u32x4 raw = *(const u32x4 *)((const uint8_t *)base + off * (BF16 ? 2 : 4));
    if constexpr (std::is_same<F, float>::value) {
      if (BF16) {
#pragma unroll
        for (int i = 0; i < 4; ++i) { v[2 * i] = __uint_as_float(raw[i] << 16); v[2 * i + 1] = __uint_as_float(raw[i] & 0xFFFF0000u); }
      } else {
#pragma unroll
        for (int i = 0; i < 4; ++i) v[i] = __uint_as_float(raw[i]);
      }
    } else {   // raw bits, one element per entry
      if (BF16) {
#pragma unroll
        for (int i = 0; i < 4; ++i) { v[2 * i] = raw[i] & 0xFFFFu; v[2 * i + 1] = raw[i] >> 16; }
      } else {
#pragma unroll
        for (int i = 0; i < 4; ++i) v[i] = raw[i];
      }
    }
  } else {
    F one;
    if constexpr (std::is_same<F, float>::value) one = BF16 ? ttm_bf16_to_f32(((const uint16_t *)base)[off]) : ((const float *)base)[off];
    else one = BF16 ? (F)((const uint16_t *)base)[off] : (F)((const uint32_t *)base)[off];
#pragma unroll
    for (int i = 0; i < EPC; ++i) v[i] = one;
  }
}

template <bool BF16>
__global__ __launch_bounds__(256) void ttm_binary_chunk_k(int op, const void *__restrict__ a, const void *__restrict__ b,
                                                          void *__restrict__ out, BcastArgs p, uint32_t chunks_per_plane) {
  constexpr int EPC = BF16 ? 8 : 4;
  for (uint32_t ci = blockIdx.x * 256 + threadIdx.x; ci < chunks_per_plane; ci += gridDim.x * 256) {
    const ChunkPos q = chunk_pos<EPC>(p.oshape, p.tiled, ci, chunks_per_plane);
    float x[EPC], y[EPC];
#pragma unroll
    for (int i = 0; i < EPC; ++i) x[i] = 0.0f;
    if (q.live) {
      operand_chunk<BF16>(a, p.ashape, q, p.tiled, x);
      operand_chunk<BF16>(b, p.bshape, q, p.tiled, y);
#pragma unroll
      for (int i = 0; i < EPC; ++i) x[i] = i < q.valid ? binary_op(op, x[i], y[i]) : 0.0f;
    }
    chunk_store<BF16>(out, q.out_chunk, x);
  }
}

// whether the chunked kernels apply: chunks inside rows, everything 16-byte aligned, plane and batch counts within 32 bits
static bool chunkable(const int64_t (&oshape)[4], int tiled, int es, std::initializer_list<const void *> ptrs) {
  const int64_t R = oshape[2], C = oshape[3], epc = 16 / es;
  if (!tiled && C % epc != 0) return false;   // tile order: any extents, a chunk lies in one face row whatever they are
  const int64_t pr = tiled ? ttm_round_up32(R) : R, pcc = tiled ? ttm_round_up32(C) : C;
  if (pr * pcc >= ((int64_t)1 << 31) || oshape[0] * oshape[1] > 65535 || oshape[0] * oshape[1] < 1) return false;
  for (const void *q : ptrs)
    if (((uintptr_t)q & 15) != 0) return false;
  return true;
}

TTM_EXPORT int ttm_eltwise_binary(int op, const void *a, const int64_t *a_shape, const void *b, const int64_t *b_shape,
                                  void *out, const int64_t *out_shape, int rank, int dtype, int layout, void *stream) {
  if (rank >= 0 && rank <= 8 && a_shape && b_shape && out_shape) TTM_EXTENTS(binary, a, a_shape, b, b_shape, out, out_shape, rank, dtype, layout);
  TTM_REQUIRE(dtype == TTM_BF16 || dtype == TTM_F32, "ttm_eltwise_binary: dtype must be BFloat16 or Float32 (got %d)", dtype);
  TTM_REQUIRE(layout == TTM_ROW_MAJOR || layout == TTM_TILE, "ttm_eltwise_binary: bad layout");
  TTM_REQUIRE(rank >= 0 && rank <= 8 && a_shape && b_shape && out_shape, "ttm_eltwise_binary: bad rank or null shape");
  TTM_REQUIRE(((op >= B_ADD && op <= B_XOR) && op != 2) || (op >= B_MAXIMUM && op <= B_ATAN2), "ttm_eltwise_binary: unsupported op %d", op);
  // right-align to rank 4: leading dims beyond the last three are folded into d0 when both operands
  // agree with the output there (no broadcasting across them)
  BcastArgs p;
  int64_t *shapes[3] = {p.oshape, p.ashape, p.bshape};
  const int64_t *src[3] = {out_shape, a_shape, b_shape};
  for (int t = 0; t < 3; ++t) {
    for (int d = 0; d < 4; ++d) shapes[t][d] = 1;
    for (int d = 0; d < rank; ++d) {
      int64_t v = src[t][rank - 1 - d];
      TTM_REQUIRE(v >= 0, "ttm_eltwise_binary: negative dimension");
      if (d < 3) shapes[t][3 - d] = v;
      else shapes[t][0] *= v;
    }
  }
  bool same = true, lead_ok = true;
  for (int d = 0; d < rank; ++d) {
    int64_t o = out_shape[d], x = a_shape[d], y = b_shape[d];
    TTM_REQUIRE((x == o || x == 1) && (y == o || y == 1), "ttm_eltwise_binary: shapes do not broadcast at dim %d", d);
    if (x != o || y != o) {
      same = false;
      if (rank - 1 - d >= 3) lead_ok = false;
    }
  }
  TTM_REQUIRE(lead_ok || rank <= 4, "ttm_eltwise_binary: broadcasting across more than the last three dims of a rank>4 tensor");
  p.tiled = layout == TTM_TILE;
  int64_t R = p.oshape[2], C = p.oshape[3];
  int64_t pr = p.tiled ? ttm_round_up32(R) : R, pc = p.tiled ? ttm_round_up32(C) : C;
  int64_t total = p.oshape[0] * p.oshape[1] * pr * pc;
  if (total == 0) return TTM_OK;
  TTM_REQUIRE(a && b && out, "ttm_eltwise_binary: null pointer");
  hipStream_t s = (hipStream_t)stream;
  const int es = dtype == TTM_BF16 ? 2 : 4;
  const bool al = (((uintptr_t)a | (uintptr_t)b | (uintptr_t)out) & 15) == 0 && (total * es) % 16 == 0;
  const bool ragged = p.tiled && (pr != R || pc != C);
  if (same && al && !ragged) {
    int64_t nchunks = total * es / 16;
    if (dtype == TTM_BF16)
      hipLaunchKernelGGL(ttm_binary_flat_k<true>, dim3(grid_for(nchunks)), dim3(256), 0, s, op, a, b, out, nchunks);
    else
      hipLaunchKernelGGL(ttm_binary_flat_k<false>, dim3(grid_for(nchunks)), dim3(256), 0, s, op, a, b, out, nchunks);
  } else if (chunkable(p.oshape, p.tiled, es, {a, b, out})) {
    const uint32_t cpp = (uint32_t)(pr * pc * es / 16);
    const dim3 grid(grid_for(cpp), (unsigned)(p.oshape[0] * p.oshape[1]));
    if (dtype == TTM_BF16) hipLaunchKernelGGL(ttm_binary_chunk_k<true>, grid, dim3(256), 0, s, op, a, b, out, p, cpp);
    else hipLaunchKernelGGL(ttm_binary_chunk_k<false>, grid, dim3(256), 0, s, op, a, b, out, p, cpp);
  } else {
    if (dtype == TTM_BF16)
      hipLaunchKernelGGL(ttm_binary_bcast_k<true>, dim3(grid_for(total)), dim3(256), 0, s, op, a, b, out, p, total);
    else
      hipLaunchKernelGGL(ttm_binary_bcast_k<false>, dim3(grid_for(total)), dim3(256), 0, s, op, a, b, out, p, total);
  }
  TTM_LAUNCH_CHECK();
  return TTM_OK;
}

// ---- where(cond, a, b): cond != 0 selects a; the three operands broadcast to the output like the binaries
struct WhereArgs {
  int64_t oshape[4], cshape[4], ashape[4], bshape[4];
  int tiled;
};

template <bool BF16>
__global__ __launch_bounds__(256) void ttm_where_k(const void *__restrict__ cond, const void *__restrict__ a, const void *__restrict__ b,
                                                   void *__restrict__ out, WhereArgs p, int64_t total) {
  const int64_t R = p.oshape[2], C = p.oshape[3];
  const int64_t pr = p.tiled ? (R + 31) / 32 * 32 : R, pc = p.tiled ? (C + 31) / 32 * 32 : C;
  typedef typename std::conditional<BF16, uint16_t, uint32_t>::type T;   // values move as bits: no rounding, NaN payloads kept
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
    int64_t batch = i / (pr * pc), w = i % (pr * pc), r, c;
    if (p.tiled) {
      int64_t tile = w >> 10;
      int e = (int)(w & 1023);
      int face = e >> 8;
      r = (tile / (pc / 32)) * 32 + (face >> 1) * 16 + ((e >> 4) & 15);
      c = (tile % (pc / 32)) * 32 + (face & 1) * 16 + (e & 15);
    } else {
      r = w / pc; c = w % pc;
    }
    T y = 0;
    if (r < R && c < C) {
      const int64_t i0 = batch / p.oshape[1], i1 = batch % p.oshape[1];
      const T cv = ((const T *)cond)[bcast_offset(p.cshape, i0, i1, r, c, p.tiled)];
      const bool take = BF16 ? (cv & 0x7FFFu) != 0 : (cv & 0x7FFFFFFFu) != 0;   // +-0 is false, NaN is true
      y = take ? ((const T *)a)[bcast_offset(p.ashape, i0, i1, r, c, p.tiled)] : ((const T *)b)[bcast_offset(p.bshape, i0, i1, r, c, p.tiled)];
    }
    ((T *)out)[i] = y;
  }
}

template <bool BF16>
__global__ __launch_bounds__(256) void ttm_where_chunk_k(const void *__restrict__ cond, const void *__restrict__ a, const void *__restrict__ b,
                                                         void *__restrict__ out, WhereArgs p, uint32_t chunks_per_plane) {
  constexpr int EPC = BF16 ? 8 : 4;
  for (uint32_t ci = blockIdx.x * 256 + threadIdx.x; ci < chunks_per_plane; ci += gridDim.x * 256) {
    const ChunkPos q = chunk_pos<EPC>(p.oshape, p.tiled, ci, chunks_per_plane);
    uint32_t cv[EPC], av[EPC], bv[EPC];
#pragma unroll
    for (int i = 0; i < EPC; ++i) av[i] = 0u;
    if (q.live) {
      operand_chunk<BF16>(cond, p.cshape, q, p.tiled, cv);
      operand_chunk<BF16>(a, p.ashape, q, p.tiled, av);
      operand_chunk<BF16>(b, p.bshape, q, p.tiled, bv);
#pragma unroll
      for (int i = 0; i < EPC; ++i)   // +-0 is false, NaN is true; columns in the padding stay zero
        av[i] = i >= q.valid ? 0u : ((cv[i] & (BF16 ? 0x7FFFu : 0x7FFFFFFFu)) != 0 ? av[i] : bv[i]);
    }
    u32x4 o;
    if (BF16) {
#pragma unroll
      for (int i = 0; i < 4; ++i) o[i] = av[2 * i] | (av[2 * i + 1] << 16);
    } else {
#pragma unroll
      for (int i = 0; i < 4; ++i) o[i] = av[i];
    }
    ((u32x4 *)out)[q.out_chunk] = o;
  }
}

TTM_EXPORT int ttm_where(const void *cond, const int64_t *cond_shape, const void *a, const int64_t *a_shape, const void *b,
                         const int64_t *b_shape, void *out, const int64_t *out_shape, int rank, int dtype, int layout, void *stream) {
  if (rank >= 0 && rank <= 4 && cond_shape && a_shape && b_shape && out_shape)
    TTM_EXTENTS(where, cond, cond_shape, a, a_shape, b, b_shape, out, out_shape, rank, dtype, layout);
  TTM_REQUIRE(dtype == TTM_BF16 || dtype == TTM_F32, "ttm_where: dtype must be BFloat16 or Float32 (got %d)", dtype);
  TTM_REQUIRE(layout == TTM_ROW_MAJOR || layout == TTM_TILE, "ttm_where: bad layout");
  TTM_REQUIRE(rank >= 0 && rank <= 4 && cond_shape && a_shape && b_shape && out_shape, "ttm_where: rank must be at most 4, shapes non-null");
  WhereArgs p;
  int64_t *shapes[4] = {p.oshape, p.cshape, p.ashape, p.bshape};
  const int64_t *src[4] = {out_shape, cond_shape, a_shape, b_shape};
  for (int t = 0; t < 4; ++t) {
    for (int d = 0; d < 4; ++d) shapes[t][d] = 1;
    for (int d = 0; d < rank; ++d) {
      const int64_t v = src[t][rank - 1 - d];
      TTM_REQUIRE(v >= 0, "ttm_where: negative dimension");
      shapes[t][3 - d] = v;
      TTM_REQUIRE(t == 0 || v == out_shape[rank - 1 - d] || v == 1, "ttm_where: shapes do not broadcast at dim %d", rank - 1 - d);
    }
  }
  p.tiled = layout == TTM_TILE;
  const int64_t R = p.oshape[2], C = p.oshape[3];
  const int64_t pr = p.tiled ? ttm_round_up32(R) : R, pc = p.tiled ? ttm_round_up32(C) : C;
  const int64_t total = p.oshape[0] * p.oshape[1] * pr * pc;
  if (total == 0) return TTM_OK;
  TTM_REQUIRE(cond && a && b && out, "ttm_where: null pointer");
  const int es = dtype == TTM_BF16 ? 2 : 4;
  if (chunkable(p.oshape, p.tiled, es, {cond, a, b, out})) {
    const uint32_t cpp = (uint32_t)(pr * pc * es / 16);
    const dim3 grid(grid_for(cpp), (unsigned)(p.oshape[0] * p.oshape[1]));
    if (dtype == TTM_BF16) hipLaunchKernelGGL(ttm_where_chunk_k<true>, grid, dim3(256), 0, (hipStream_t)stream, cond, a, b, out, p, cpp);
    else hipLaunchKernelGGL(ttm_where_chunk_k<false>, grid, dim3(256), 0, (hipStream_t)stream, cond, a, b, out, p, cpp);
    TTM_LAUNCH_CHECK();
    return TTM_OK;
  }
  if (dtype == TTM_BF16)
    hipLaunchKernelGGL(ttm_where_k<true>, dim3(grid_for(total)), dim3(256), 0, (hipStream_t)stream, cond, a, b, out, p, total);
  else
    hipLaunchKernelGGL(ttm_where_k<false>, dim3(grid_for(total)), dim3(256), 0, (hipStream_t)stream, cond, a, b, out, p, total);
  TTM_LAUNCH_CHECK();
  return TTM_OK;
}

// ---- typecast between plain dtypes (layout preserved; block formats go through ttm_bfp_pack/unpack)
template <int SRC, int DST>
__global__ __launch_bounds__(256) void ttm_typecast_k(const void *__restrict__ in, void *__restrict__ out, int64_t n) {
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (int64_t)gridDim.x * 256) {
    float f; int64_t iv; bool is_int = false;
    if (SRC == TTM_F32) f = ((const float *)in)[i];
    else if (SRC == TTM_BF16) f = ttm_bf16_to_f32(((const uint16_t *)in)[i]);
    else if (SRC == TTM_F16) f = __half2float(((const __half *)in)[i]);
    else { is_int = true; f = 0.0f; }
    if (SRC == TTM_U32) iv = ((const uint32_t *)in)[i];
    else if (SRC == TTM_I32) iv = ((const int32_t *)in)[i];
    else if (SRC == TTM_U16) iv = ((const uint16_t *)in)[i];
    else if (SRC == TTM_U8) iv = ((const uint8_t *)in)[i];
    else iv = 0;
    if (DST == TTM_F32) ((float *)out)[i] = is_int ? (float)iv : f;
    else if (DST == TTM_BF16) ((uint16_t *)out)[i] = ttm_f32_to_bf16(is_int ? (float)iv : f);
    else if (DST == TTM_F16) ((__half *)out)[i] = __float2half(is_int ? (float)iv : f);
    else {
      // float -> integer truncates toward zero and saturates; integer -> integer saturates
      if (DST == TTM_I32) {
        ((int32_t *)out)[i] = is_int ? (int32_t)min(max(iv, (int64_t)INT32_MIN), (int64_t)INT32_MAX)
                                     : (f != f ? 0 : (f >= 2147483648.0f ? INT32_MAX : (f <= -2147483648.0f ? INT32_MIN : (int32_t)f)));
      } else {
        const int64_t hi = DST == TTM_U32 ? 4294967295ll : (DST == TTM_U16 ? 65535ll : 255ll);
        int64_t v = is_int ? iv : (f != f ? 0 : (f <= 0.0f ? 0 : (f >= 4294967296.0f ? 4294967295ll : (int64_t)f)));
        v = min(max(v, (int64_t)0), hi);
        if (DST == TTM_U32) ((uint32_t *)out)[i] = (uint32_t)v;
        else if (DST == TTM_U16) ((uint16_t *)out)[i] = (uint16_t)v;
        else ((uint8_t *)out)[i] = (uint8_t)v;
      }
    }
  }
}

// bf16 <-> fp32 in groups of four elements per lane: 8 bytes of bf16 against 16 of fp32, every instruction of a wavefront
// touching one contiguous run (the element-wise kernel above moves 2 + 4 bytes per lane and reaches half the bandwidth)
template <bool WIDEN>
__global__ __launch_bounds__(256) void ttm_typecast4_k(const void *__restrict__ in, void *__restrict__ out, int64_t groups) {
  for (int64_t g = (int64_t)blockIdx.x * 256 + threadIdx.x; g < groups; g += (int64_t)gridDim.x * 256) {
    if (WIDEN) {
      const u32x2 v = __builtin_nontemporal_load((const u32x2 *)in + g);
      const u32x4 w = {v.x << 16, v.x & 0xFFFF0000u, v.y << 16, v.y & 0xFFFF0000u};
      __builtin_nontemporal_store(w, (u32x4 *)out + g);
    } else {
      const u32x4 w = __builtin_nontemporal_load((const u32x4 *)in + g);
      const u32x2 v = {ttm_pack_bf16x2(__uint_as_float(w.x), __uint_as_float(w.y)), ttm_pack_bf16x2(__uint_as_float(w.z), __uint_as_float(w.w))};
      __builtin_nontemporal_store(v, (u32x2 *)out + g);
    }
  }
}

typedef void (*cast_fn)(const void *, void *, int64_t);
template <int SRC>
static cast_fn pick_cast_dst(int dst) {
  switch (dst) {
  case TTM_F32: return ttm_typecast_k<SRC, TTM_F32>;
  case TTM_BF16: return ttm_typecast_k<SRC, TTM_BF16>;
  case TTM_F16: return ttm_typecast_k<SRC, TTM_F16>;
  case TTM_U32: return ttm_typecast_k<SRC, TTM_U32>;
  case TTM_I32: return ttm_typecast_k<SRC, TTM_I32>;
  case TTM_U16: return ttm_typecast_k<SRC, TTM_U16>;
  case TTM_U8: return ttm_typecast_k<SRC, TTM_U8>;
  default: return nullptr;
  }
}

TTM_EXPORT int ttm_typecast(const void *in, int src_dtype, void *out, int dst_dtype, int64_t n, void *stream) {
  TTM_EXTENTS(typecast, in, src_dtype, out, dst_dtype, n);
  TTM_REQUIRE(n >= 0, "ttm_typecast: negative size");
  cast_fn fn = nullptr;
  switch (src_dtype) {
  case TTM_F32: fn = pick_cast_dst<TTM_F32>(dst_dtype); break;
  case TTM_BF16: fn = pick_cast_dst<TTM_BF16>(dst_dtype); break;
  case TTM_F16: fn = pick_cast_dst<TTM_F16>(dst_dtype); break;
  case TTM_U32: fn = pick_cast_dst<TTM_U32>(dst_dtype); break;
  case TTM_I32: fn = pick_cast_dst<TTM_I32>(dst_dtype); break;
  case TTM_U16: fn = pick_cast_dst<TTM_U16>(dst_dtype); break;
  case TTM_U8: fn = pick_cast_dst<TTM_U8>(dst_dtype); break;
  default: break;
  }
  if (!fn) return ttm_set_error(TTM_ERR_UNSUPPORTED, "ttm_typecast: unsupported conversion %d -> %d", src_dtype, dst_dtype);
  if (n == 0) return TTM_OK;
  TTM_REQUIRE(in && out, "ttm_typecast: null pointer");
  const bool widen = src_dtype == TTM_BF16 && dst_dtype == TTM_F32, narrow = src_dtype == TTM_F32 && dst_dtype == TTM_BF16;
  if ((widen || narrow) && n % 4 == 0 && (((uintptr_t)in | (uintptr_t)out) & 15) == 0) {
    if (widen) hipLaunchKernelGGL(ttm_typecast4_k<true>, dim3(grid_for(n / 4)), dim3(256), 0, (hipStream_t)stream, in, out, n / 4);
    else hipLaunchKernelGGL(ttm_typecast4_k<false>, dim3(grid_for(n / 4)), dim3(256), 0, (hipStream_t)stream, in, out, n / 4);
    TTM_LAUNCH_CHECK();
    return TTM_OK;
  }
  hipLaunchKernelGGL(fn, dim3(grid_for(n)), dim3(256), 0, (hipStream_t)stream, in, out, n);
  TTM_LAUNCH_CHECK();
  return TTM_OK;
}
