/*
 * ttm_oracle.c -- CPU restatement of the tt-mlir hot path.  TEST INFRASTRUCTURE ONLY.
 *
 * This file is the checker, never the product: only tests, the smoke check and the
 * cpu_baseline leg of the benchmark may build or call it.  Every function follows a
 * file in the reference tree (paths relative to the tt-mlir checkout):
 *
 *   tilize / untilize      tools/golden/mapping.py:3453-3549 (same loop in
 *                          test/python/golden/d2m/test_tilize.py:45-97)
 *   bfp8_b / bfp4_b        size contract lib/Dialect/TTCore/IR/TTCoreOpsTypes.cpp:1875-1887,
 *                          field widths include/ttmlir/Dialect/TTCore/IR/TTCoreOpsTypes.h:321-361,
 *                          face/row prose lib/Dialect/TTNN/Transforms/TTNNCollectPerfMetrics.cpp:459-464.
 *                          The arithmetic itself lives in tt-metal (pinned d5f9bc4a, un-vendored):
 *                          PARITY UNPINNED against tt-metal's packer; pinned here by hand-worked
 *                          vectors, an independent float-arithmetic model and format invariants.
 *   f16<->bf16, int casts  runtime/include/tt/runtime/utils.h:17-180, known answers in
 *                          runtime/test/common/gtest/test_handle_float_bfloat_buffer_cast.cpp:8-46
 *   matmul / linear        lib/Conversion/TTIRToLinalg/TTIRToLinalg.cpp:318-572, 1647-1912;
 *                          tools/golden/mapping.py:2359-2414, 7749-7797 (bias, then activation)
 *   f32 compute, cast back lib/Dialect/TTIR/Transforms/HoistCPUOps/HoistCPUOps.cpp:76-93, 219-245
 *   gelu / silu / unary    lib/Conversion/TTIRToLinalg/EltwiseUnary.cpp:251-326
 *   softmax                lib/Conversion/TTIRToLinalg/TTIRToLinalg.cpp:944-1017 (max-subtracted)
 *   reductions             lib/Conversion/TTIRToLinalg/Reduction.cpp:101-220 (mean = sum / N)
 *   rms_norm               lib/Dialect/TTIR/Transforms/DecomposeComposites.cpp:47-111
 *                          (x*x -> mean -> +eps -> rsqrt -> x*r -> *w -> +b), golden mapping.py:1221-1288
 *   sdpa                   tools/golden/mapping.py:8398-8500 (GQA by repeat_interleave, causal triu)
 *
 * The reference CPU path is a single-threaded scalar f32 loop nest
 * (lib/Target/LLVM/LLVMToDynamicLib.cpp:83-99: "generic" cpu, no vector features); the loops
 * below keep that shape.  orc_set_threads(n>1) runs the same loops over rows with OpenMP for
 * the "all cores" baseline column.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

static int g_threads = 1;
void orc_set_threads(int n) { g_threads = n > 0 ? n : 1; }
int orc_get_threads(void) { return g_threads; }
int orc_max_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}

#define TILE 32
#define FACE 16

static inline int64_t round_up32(int64_t v) { return (v + 31) / 32 * 32; }

/* ------------------------------------------------------------------ tilize / untilize
 * out_flat[idx++] = in[ty*32 + fy*16 + dy, tx*32 + fx*16 + dx], loops ty,tx,fy,fx,dy,dx.
 * Rows/cols that are not multiples of 32 are zero-padded to the next tile boundary
 * (runtime/include/tt/runtime/detail/ttnn/types/types.h:205).  Higher ranks tile the last
 * two dims per batch entry (lib/Dialect/TTCore/IR/TTCoreOpsTypes.cpp:1857-1865).           */
void orc_tilize(const void *in_, void *out_, int64_t batch, int64_t rows, int64_t cols, int elem) {
  const uint8_t *in = (const uint8_t *)in_;
  uint8_t *out = (uint8_t *)out_;
  int64_t pr = round_up32(rows), pc = round_up32(cols);
  int64_t yt = pr / TILE, xt = pc / TILE;
  for (int64_t b = 0; b < batch; ++b) {
    const uint8_t *src = in + b * rows * cols * elem;
    uint8_t *dst = out + b * pr * pc * elem;
    int64_t idx = 0;
    for (int64_t ty = 0; ty < yt; ++ty)
      for (int64_t tx = 0; tx < xt; ++tx)
        for (int fy = 0; fy < 2; ++fy)
          for (int fx = 0; fx < 2; ++fx)
            for (int dy = 0; dy < FACE; ++dy)
              for (int dx = 0; dx < FACE; ++dx) {
                int64_t r = dy + ty * TILE + fy * FACE;
                int64_t c = dx + tx * TILE + fx * FACE;
                if (r < rows && c < cols)
                  memcpy(dst + idx * elem, src + (r * cols + c) * elem, elem);
                else
                  memset(dst + idx * elem, 0, elem);
                ++idx;
              }
  }
}

void orc_untilize(const void *in_, void *out_, int64_t batch, int64_t rows, int64_t cols, int elem) {
  const uint8_t *in = (const uint8_t *)in_;
  uint8_t *out = (uint8_t *)out_;
  int64_t pr = round_up32(rows), pc = round_up32(cols);
  int64_t yt = pr / TILE, xt = pc / TILE;
  for (int64_t b = 0; b < batch; ++b) {
    const uint8_t *src = in + b * pr * pc * elem;
    uint8_t *dst = out + b * rows * cols * elem;
    int64_t idx = 0;
    for (int64_t ty = 0; ty < yt; ++ty)
      for (int64_t tx = 0; tx < xt; ++tx)
        for (int fy = 0; fy < 2; ++fy)
          for (int fx = 0; fx < 2; ++fx)
            for (int dy = 0; dy < FACE; ++dy)
              for (int dx = 0; dx < FACE; ++dx) {
                int64_t r = dy + ty * TILE + fy * FACE;
                int64_t c = dx + tx * TILE + fx * FACE;
                if (r < rows && c < cols)
                  memcpy(dst + (r * cols + c) * elem, src + idx * elem, elem);
                ++idx;
              }
  }
}

/* ------------------------------------------------------------------ block float
 * fmt 8 = bfp8_b (7 magnitude bits), fmt 4 = bfp4_b (3 magnitude bits).
 * Tile bytes: [0,64) exponents (face-major, one per 16-element face row), then mantissas
 * in the same face/row order; bfp8 one byte per element (sign<<7 | mag), bfp4 two elements
 * per byte, even column in the low nibble (sign<<3 | mag).                                 */
int64_t orc_bfp_tile_bytes(int fmt) { return fmt == 8 ? 1088 : (fmt == 4 ? 576 : -1); }

static inline uint32_t f32_bits(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static inline float bits_f32(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }

static inline uint32_t bfp_encode(uint32_t bits, uint32_t E, int W) {
  if ((bits & 0x7FFFFFFFu) == 0) return 0;
  uint32_t e = (bits >> 23) & 0xFF;
  uint32_t sign = bits >> 31;
  uint32_t m = 0x800000u | (bits & 0x7FFFFFu); /* hidden bit added, denormals not special-cased */
  uint32_t shift = E - e;
  m = shift >= 32 ? 0 : (m >> shift);
  /* round to nearest, ties to even, on the bits below the kept W */
  int drop = 24 - W;
  uint32_t keep = m >> drop;
  uint32_t rem = m & ((1u << drop) - 1);
  uint32_t half = 1u << (drop - 1);
  if (rem > half || (rem == half && (keep & 1))) keep += 1;
  uint32_t maxv = (1u << W) - 1;
  if (keep > maxv) keep = maxv;
  if (keep == 0) sign = 0;
  return (sign << W) | keep;
}

static inline float bfp_decode(uint32_t code, uint32_t E, int W) {
  uint32_t mag = code & ((1u << W) - 1);
  uint32_t sign = (code >> W) & 1;
  if (mag == 0) return 0.0f;
  /* mag * 2^(E - 127 - (W-1)); ldexp keeps it exact, including subnormal results */
  float v = ldexpf((float)mag, (int)E - 127 - (W - 1));
  return sign ? -v : v;
}

static void bfp_pack_tile(const float *t, uint8_t *out, int fmt) {
  int W = fmt == 8 ? 7 : 3;
  uint8_t *ex = out, *mant = out + 64;
  for (int f = 0; f < 4; ++f)
    for (int r = 0; r < FACE; ++r) {
      const float *row = t + f * 256 + r * 16;
      uint32_t E = 0;
      for (int c = 0; c < 16; ++c) {
        uint32_t e = (f32_bits(row[c]) >> 23) & 0xFF;
        if (e > E) E = e;
      }
      ex[f * 16 + r] = (uint8_t)E;
      if (fmt == 8) {
        for (int c = 0; c < 16; ++c)
          mant[f * 256 + r * 16 + c] = (uint8_t)bfp_encode(f32_bits(row[c]), E, W);
      } else {
        for (int c = 0; c < 16; c += 2) {
          uint32_t lo = bfp_encode(f32_bits(row[c]), E, W);
          uint32_t hi = bfp_encode(f32_bits(row[c + 1]), E, W);
          mant[f * 128 + r * 8 + c / 2] = (uint8_t)(lo | (hi << 4));
        }
      }
    }
}

static void bfp_unpack_tile(const uint8_t *in, float *t, int fmt) {
  int W = fmt == 8 ? 7 : 3;
  const uint8_t *ex = in, *mant = in + 64;
  for (int f = 0; f < 4; ++f)
    for (int r = 0; r < FACE; ++r) {
      uint32_t E = ex[f * 16 + r];
      float *row = t + f * 256 + r * 16;
      for (int c = 0; c < 16; ++c) {
        uint32_t code;
        if (fmt == 8) code = mant[f * 256 + r * 16 + c];
        else {
          uint8_t b = mant[f * 128 + r * 8 + c / 2];
          code = (c & 1) ? (b >> 4) : (b & 0xF);
        }
        row[c] = bfp_decode(code, E, W);
      }
    }
}

/* tiled fp32 (tile/face order) -> packed tiles */
void orc_bfp_pack_tiles(const float *tiled, uint8_t *out, int64_t ntiles, int fmt) {
  int64_t tb = orc_bfp_tile_bytes(fmt);
#pragma omp parallel for num_threads(g_threads) schedule(static) if (g_threads > 1)
  for (int64_t t = 0; t < ntiles; ++t) bfp_pack_tile(tiled + t * 1024, out + t * tb, fmt);
}

void orc_bfp_unpack_tiles(const uint8_t *in, float *tiled, int64_t ntiles, int fmt) {
  int64_t tb = orc_bfp_tile_bytes(fmt);
#pragma omp parallel for num_threads(g_threads) schedule(static) if (g_threads > 1)
  for (int64_t t = 0; t < ntiles; ++t) bfp_unpack_tile(in + t * tb, tiled + t * 1024, fmt);
}

/* row-major fp32 [batch, rows, cols] -> packed tiles (tilize fused, zero padded) */
void orc_bfp_pack_rm(const float *rm, uint8_t *out, int64_t batch, int64_t rows, int64_t cols, int fmt) {
  int64_t pr = round_up32(rows), pc = round_up32(cols);
  int64_t yt = pr / TILE, xt = pc / TILE, tb = orc_bfp_tile_bytes(fmt);
#pragma omp parallel for num_threads(g_threads) schedule(static) if (g_threads > 1)
  for (int64_t bt = 0; bt < batch * yt; ++bt) {
    int64_t b = bt / yt, ty = bt % yt;
    float tile[1024];
    for (int64_t tx = 0; tx < xt; ++tx) {
      for (int f = 0; f < 4; ++f)
        for (int r = 0; r < FACE; ++r)
          for (int c = 0; c < FACE; ++c) {
            int64_t rr = ty * TILE + (f >> 1) * FACE + r, cc = tx * TILE + (f & 1) * FACE + c;
            tile[f * 256 + r * 16 + c] = (rr < rows && cc < cols) ? rm[(b * rows + rr) * cols + cc] : 0.0f;
          }
      bfp_pack_tile(tile, out + ((b * yt + ty) * xt + tx) * tb, fmt);
    }
  }
}

void orc_bfp_unpack_rm(const uint8_t *in, float *rm, int64_t batch, int64_t rows, int64_t cols, int fmt) {
  int64_t pr = round_up32(rows), pc = round_up32(cols);
  int64_t yt = pr / TILE, xt = pc / TILE, tb = orc_bfp_tile_bytes(fmt);
#pragma omp parallel for num_threads(g_threads) schedule(static) if (g_threads > 1)
  for (int64_t bt = 0; bt < batch * yt; ++bt) {
    int64_t b = bt / yt, ty = bt % yt;
    float tile[1024];
    for (int64_t tx = 0; tx < xt; ++tx) {
      bfp_unpack_tile(in + ((b * yt + ty) * xt + tx) * tb, tile, fmt);
      for (int f = 0; f < 4; ++f)
        for (int r = 0; r < FACE; ++r)
          for (int c = 0; c < FACE; ++c) {
            int64_t rr = ty * TILE + (f >> 1) * FACE + r, cc = tx * TILE + (f & 1) * FACE + c;
            if (rr < rows && cc < cols) rm[(b * rows + rr) * cols + cc] = tile[f * 256 + r * 16 + c];
          }
    }
  }
}

/* ------------------------------------------------------------------ scalar casts */
static inline uint16_t f32_to_bf16_bits(float f) {
  uint32_t u = f32_bits(f);
  if ((u & 0x7FFFFFFFu) > 0x7F800000u) return (uint16_t)((u >> 16) | 0x40); /* quiet NaN */
  u += 0x7FFFu + ((u >> 16) & 1);                                          /* RNE */
  return (uint16_t)(u >> 16);
}
static inline float bf16_bits_to_f32(uint16_t h) { return bits_f32((uint32_t)h << 16); }

void orc_f32_to_bf16(const float *in, uint16_t *out, int64_t n) {
  for (int64_t i = 0; i < n; ++i) out[i] = f32_to_bf16_bits(in[i]);
}
void orc_bf16_to_f32(const uint16_t *in, float *out, int64_t n) {
  for (int64_t i = 0; i < n; ++i) out[i] = bf16_bits_to_f32(in[i]);
}

static float f16_bits_to_f32(uint16_t h) {
  uint32_t sign = (uint32_t)(h & 0x8000) << 16;
  uint32_t e = (h >> 10) & 0x1F, m = h & 0x3FF;
  if (e == 0) {
    if (m == 0) return bits_f32(sign);
    float v = ldexpf((float)m, -24);
    return sign ? -v : v;
  }
  if (e == 31) return bits_f32(sign | 0x7F800000u | (m << 13));
  return bits_f32(sign | ((e + 112) << 23) | (m << 13));
}
static uint16_t f32_to_f16_bits(float f) {
  uint32_t u = f32_bits(f), sign = (u >> 16) & 0x8000;
  uint32_t a = u & 0x7FFFFFFFu;
  if (a > 0x7F800000u) return (uint16_t)(sign | 0x7E00);
  if (a >= 0x477FF000u) return (uint16_t)(sign | 0x7C00); /* rounds to inf */
  if (a < 0x33000001u) return (uint16_t)sign;             /* below half the smallest subnormal */
  int e = (int)(a >> 23) - 127;
  uint32_t m = (a & 0x7FFFFFu) | 0x800000u;
  int shift = e < -14 ? (13 + (-14 - e)) : 13;
  uint32_t keep = m >> shift, rem = m & ((1u << shift) - 1), half = 1u << (shift - 1);
  if (rem > half || (rem == half && (keep & 1))) keep++;
  uint32_t out = e < -14 ? keep : (((uint32_t)(e + 15) << 10) + (keep - 0x400));
  return (uint16_t)(sign | out);
}
/* runtime/include/tt/runtime/utils.h:152-158 (handleFloat16ToBFloat16 / handleBFloat16ToFloat16) */
void orc_f16_to_bf16(const uint16_t *in, uint16_t *out, int64_t n) {
  for (int64_t i = 0; i < n; ++i) out[i] = f32_to_bf16_bits(f16_bits_to_f32(in[i]));
}
void orc_bf16_to_f16(const uint16_t *in, uint16_t *out, int64_t n) {
  for (int64_t i = 0; i < n; ++i) out[i] = f32_to_f16_bits(bf16_bits_to_f32(in[i]));
}

/* ------------------------------------------------------------------ eltwise (f32 compute)
 * op codes follow EltwiseUnaryOpType / EltwiseBinaryOpType in
 * include/ttmlir/Target/TTNN/operations/eltwise.fbs                                        */
enum { U_ABS = 0, U_CEIL, U_COS, U_FLOOR, U_GELU, U_ISFINITE, U_LOGICALNOT, U_NEG, U_RELU, U_SQRT,
       U_RSQRT, U_SIGMOID, U_SIN, U_RECIPROCAL, U_SIGN, U_TAN, U_TANH, U_ATAN, U_EXP, U_ERF, U_ERFC,
       U_LOG, U_EXPM1, U_LEAKYRELU, U_BITWISENOT, U_RELU6, U_SILU, U_HARDSIGMOID, U_MISH, U_ACOS, U_ASIN, U_ASINH,
       U_CBRT = 100, U_LOG1P = 103 };

static inline float unary_f32(int op, float x, float p) {
  switch (op) {
  case U_ABS: return fabsf(x);
  case U_CEIL: return ceilf(x);
  case U_COS: return cosf(x);
  case U_FLOOR: return floorf(x);
  case U_GELU: return (0.5f * x) * (1.0f + erff(x * 0.70710678118654752f));
  case U_ISFINITE: return isfinite(x) ? 1.0f : 0.0f;
  case U_LOGICALNOT: return x == 0.0f ? 1.0f : 0.0f;
  case U_NEG: return -x;
  /* max(x, 0) with NaN kept, as linalg.max / arith.maximumf (lib/Conversion/TTIRToLinalg/EltwiseUnary.cpp:508-541) and
   * torch.relu (tools/golden/mapping.py:7437, 9052) have it; -0.0 gives +0.0 as maximumf does (torch keeps -0.0) */
  case U_RELU: return x > 0.0f ? x : (x != x ? x : 0.0f);
  case U_SQRT: return sqrtf(x);
  case U_RSQRT: return 1.0f / sqrtf(x);
  case U_SIGMOID: return 1.0f / (1.0f + expf(-x));
  case U_SIN: return sinf(x);
  case U_RECIPROCAL: return 1.0f / x;
  case U_SIGN: return (x > 0.0f) - (x < 0.0f);
  case U_TAN: return tanf(x);
  case U_TANH: return tanhf(x);
  case U_ATAN: return atanf(x);
  case U_EXP: return expf(x);
  case U_ERF: return erff(x);
  case U_ERFC: return erfcf(x);
  case U_LOG: return logf(x);
  case U_EXPM1: return expm1f(x);
  case U_LEAKYRELU: return x > 0.0f ? x : p * x;
  case U_RELU6: return x < 0.0f ? 0.0f : (x > 6.0f ? 6.0f : x);
  case U_SILU: return x * (1.0f / (1.0f + expf(-x)));
  /* torch.nn.functional.hardsigmoid = relu6(x + 3) / 6, mish = x tanh(softplus(x)) (tools/golden/mapping.py:5544-5548 and
   * the torch definitions the other goldens call) */
  case U_HARDSIGMOID: { float t = x + 3.0f; t = t < 0.0f ? 0.0f : (t > 6.0f ? 6.0f : t); return x != x ? x : t / 6.0f; }
  case U_MISH: return x * tanhf(x > 20.0f ? x : log1pf(expf(x)));
  case U_ACOS: return acosf(x);
  case U_ASIN: return asinf(x);
  case U_ASINH: return asinhf(x);
  case U_CBRT: return cbrtf(x);
  case U_LOG1P: return log1pf(x);
  default: return NAN;
  }
}

void orc_unary_f32(int op, const float *in, float *out, int64_t n, float param) {
#pragma omp parallel for num_threads(g_threads) schedule(static) if (g_threads > 1)
  for (int64_t i = 0; i < n; ++i) out[i] = unary_f32(op, in[i], param);
}

enum { B_ADD = 0, B_MUL = 1, B_SUB = 3, B_EQ = 4, B_NE = 5, B_GE = 6, B_GT = 7, B_LE = 8, B_LT = 9, B_DIV = 10 };

static inline float binary_f32(int op, float a, float b) {
  switch (op) {
  case B_ADD: return a + b;
  case B_MUL: return a * b;
  case B_SUB: return a - b;
  case B_EQ: return a == b;
  case B_NE: return a != b;
  case B_GE: return a >= b;
  case B_GT: return a > b;
  case B_LE: return a <= b;
  case B_LT: return a < b;
  case B_DIV: return a / b;
  default: return NAN;
  }
}

/* numpy-style broadcasting over up to 8 dims; shapes are right-aligned by the caller */
void orc_binary_f32(int op, const float *a, const int64_t *ashape, const float *b, const int64_t *bshape,
                    float *out, const int64_t *oshape, int rank) {
  int64_t n = 1, astr[8], bstr[8];
  int64_t sa = 1, sb = 1;
  for (int d = rank - 1; d >= 0; --d) {
    astr[d] = ashape[d] == 1 ? 0 : sa; sa *= ashape[d];
    bstr[d] = bshape[d] == 1 ? 0 : sb; sb *= bshape[d];
    n *= oshape[d];
  }
#pragma omp parallel for num_threads(g_threads) schedule(static) if (g_threads > 1)
  for (int64_t i = 0; i < n; ++i) {
    int64_t rem = i, ia = 0, ib = 0;
    for (int d = rank - 1; d >= 0; --d) {
      int64_t c = rem % oshape[d]; rem /= oshape[d];
      ia += c * astr[d]; ib += c * bstr[d];
    }
    out[i] = binary_f32(op, a[ia], b[ib]);
  }
}

/* ------------------------------------------------------------------ matmul / linear
 * C[M,N] = act(A[M,K] . B[K,N] + bias[N]); transposes swap the last two dims of the stored
 * operand.  Accumulation is sequential in k, f32.  act: 0 none, 1 gelu, 2 silu, 3 sigmoid,
 * 4 relu (activation strings, lib/Dialect/TTNN/Transforms/TTNNFusing.cpp:155-159).          */
static inline float act_f32(int act, float x) {
  switch (act) {
  case 1: return unary_f32(U_GELU, x, 0);
  case 2: return unary_f32(U_SILU, x, 0);
  case 3: return unary_f32(U_SIGMOID, x, 0);
  case 4: return unary_f32(U_RELU, x, 0);
  default: return x;
  }
}

void orc_linear_f32(const float *A, const float *B, const float *bias, float *C, int64_t M, int64_t N,
                    int64_t K, int transA, int transB, int act) {
#pragma omp parallel for num_threads(g_threads) schedule(static) if (g_threads > 1)
  for (int64_t m = 0; m < M; ++m)
    for (int64_t n = 0; n < N; ++n) {
      float acc = 0.0f;
      for (int64_t k = 0; k < K; ++k) {
        float a = transA ? A[k * M + m] : A[m * K + k];
        float b = transB ? B[n * K + k] : B[k * N + n];
        acc += a * b;
      }
      if (bias) acc += bias[n];
      C[m * N + n] = act_f32(act, acc);
    }
}

/* Same result as orc_linear_f32 without transposes, loop order m,k,n so the inner loop
 * streams B rows; per-(m,n) accumulation order over k is unchanged (bit-identical).
 * Used only to keep large baseline samples affordable.                                     */
void orc_linear_f32_rowstream(const float *A, const float *B, const float *bias, float *C, int64_t M,
                              int64_t N, int64_t K, int act) {
#pragma omp parallel for num_threads(g_threads) schedule(static) if (g_threads > 1)
  for (int64_t m = 0; m < M; ++m) {
    float *c = C + m * N;
    for (int64_t n = 0; n < N; ++n) c[n] = 0.0f;
    for (int64_t k = 0; k < K; ++k) {
      float a = A[m * K + k];
      const float *b = B + k * N;
      for (int64_t n = 0; n < N; ++n) c[n] += a * b[n];
    }
    for (int64_t n = 0; n < N; ++n) c[n] = act_f32(act, bias ? c[n] + bias[n] : c[n]);
  }
}

/* batched matmul, batch of B broadcast when bbatch == 1 */
void orc_bmm_f32(const float *A, const float *B, float *C, int64_t batch, int64_t bbatch, int64_t M,
                 int64_t N, int64_t K, int transA, int transB) {
  for (int64_t b = 0; b < batch; ++b)
    orc_linear_f32(A + b * M * K, B + (bbatch == 1 ? 0 : b) * K * N, NULL, C + b * M * N, M, N, K, transA,
                   transB, 0);
}

/* ------------------------------------------------------------------ rms_norm over the last dim */
void orc_rmsnorm_f32(const float *x, const float *w, const float *b, float *out, int64_t rows, int64_t cols,
                     float eps) {
#pragma omp parallel for num_threads(g_threads) schedule(static) if (g_threads > 1)
  for (int64_t r = 0; r < rows; ++r) {
    const float *xr = x + r * cols;
    float s = 0.0f;
    for (int64_t c = 0; c < cols; ++c) s += xr[c] * xr[c];
    float mean = s / (float)cols;
    float rs = 1.0f / sqrtf(mean + eps);
    for (int64_t c = 0; c < cols; ++c) {
      float v = xr[c] * rs;
      if (w) v *= w[c];
      if (b) v += b[c];
      out[r * cols + c] = v;
    }
  }
}

/* ------------------------------------------------------------------ softmax / reduce over one dim
 * tensor viewed as [outer, dim, inner]                                                       */
void orc_softmax_f32(const float *x, float *out, int64_t outer, int64_t dim, int64_t inner) {
#pragma omp parallel for num_threads(g_threads) schedule(static) if (g_threads > 1)
  for (int64_t o = 0; o < outer; ++o)
    for (int64_t i = 0; i < inner; ++i) {
      const float *p = x + o * dim * inner + i;
      float *q = out + o * dim * inner + i;
      float mx = -INFINITY;
      for (int64_t d = 0; d < dim; ++d) mx = p[d * inner] > mx ? p[d * inner] : mx;
      float s = 0.0f;
      for (int64_t d = 0; d < dim; ++d) { float e = expf(p[d * inner] - mx); q[d * inner] = e; s += e; }
      float inv = 1.0f / s;
      for (int64_t d = 0; d < dim; ++d) q[d * inner] *= inv;
    }
}

/* op: 0 sum, 1 mean, 2 max, 3 min (ReductionOpType, operations/reduction.fbs:6-11) */
void orc_reduce_f32(int op, const float *x, float *out, int64_t outer, int64_t dim, int64_t inner) {
#pragma omp parallel for num_threads(g_threads) schedule(static) if (g_threads > 1)
  for (int64_t o = 0; o < outer; ++o)
    for (int64_t i = 0; i < inner; ++i) {
      const float *p = x + o * dim * inner + i;
      float acc = (op == 2) ? -INFINITY : (op == 3 ? INFINITY : 0.0f);
      for (int64_t d = 0; d < dim; ++d) {
        float v = p[d * inner];
        /* a NaN anywhere gives NaN: torch.max / torch.min of the goldens (tools/golden/mapping.py:5189-5220, 2815-2856) and
         * tosa.reduce_max / reduce_min of the CPU lowering (lib/Conversion/TTIRToLinalg/Reduction.cpp:133-136), whose
         * default is to propagate */
        if (op == 2) acc = (v > acc || v != v) ? v : acc;
        else if (op == 3) acc = (v < acc || v != v) ? v : acc;
        else acc += v;
      }
      if (op == 1) acc = acc / (float)dim;
      out[o * inner + i] = acc;
    }
}

/* ------------------------------------------------------------------ scaled dot product attention
 * q [B,Hq,Sq,D], k/v [B,Hkv,Sk,D]; query head h reads kv head h / (Hq/Hkv); mask (optional)
 * is additive, [B,1,Sq,Sk] or [B,Hq,Sq,Sk] (mask_heads = 1 or Hq); causal adds -inf above the
 * diagonal; scale <= 0 means 1/sqrt(D).  Softmax in f32.
 * window >= 0 (tools/golden/mapping.py:8450-8467): query i sees key j when 0 <= i - j < window under is_causal, when
 * |i - j| <= window / 2 otherwise; the window replaces the causal mask and a given mask is added on top.
 * sink (optional, one value per query head; mapping.py:8476-8494): one more logit per head in the softmax, with no
 * value row.  The value here is the operand of the TTNN op, which the kernel multiplies by scale like the scores
 * (lib/Conversion/TTIRToTTNN/TTIRToTTNN.cpp:3507-3533: the lowering divides the source graph's logit by scale to
 * compensate), so the golden on logit x equals this function on x / scale.
 * A query that sees nothing gives a row of zeros (the golden's softmax gives NaN there).                      */
void orc_sdpa_f32(const float *q, const float *k, const float *v, const float *mask, int mask_heads,
                  float *out, int64_t B, int64_t Hq, int64_t Hkv, int64_t Sq, int64_t Sk, int64_t D,
                  int is_causal, float scale, int64_t window, const float *sink) {
  if (!(scale > 0.0f)) scale = 1.0f / sqrtf((float)D);
  int64_t rep = Hq / Hkv;
#pragma omp parallel for num_threads(g_threads) schedule(dynamic, 4) if (g_threads > 1)
  for (int64_t bhs = 0; bhs < B * Hq * Sq; ++bhs) {
    int64_t b = bhs / (Hq * Sq), h = (bhs / Sq) % Hq, i = bhs % Sq;
    int64_t hk = h / rep;
    const float *qi = q + ((b * Hq + h) * Sq + i) * D;
    float *s = (float *)malloc(sizeof(float) * Sk);
    float mx = -INFINITY;
    for (int64_t j = 0; j < Sk; ++j) {
      const float *kj = k + ((b * Hkv + hk) * Sk + j) * D;
      float acc = 0.0f;
      for (int64_t d = 0; d < D; ++d) acc += qi[d] * kj[d];
      acc *= scale;
      if (mask) acc += mask[((b * mask_heads + (mask_heads == 1 ? 0 : h)) * Sq + i) * Sk + j];
      if (window >= 0) {
        int64_t diff = i - j, half = window / 2;
        if (is_causal ? (diff < 0 || diff >= window) : (diff < -half || diff > half)) acc = -INFINITY;
      } else if (is_causal && j > i) acc = -INFINITY;
      s[j] = acc;
      mx = acc > mx ? acc : mx;
    }
    float sink_logit = sink ? sink[h] * scale : -INFINITY;
    mx = sink_logit > mx ? sink_logit : mx;
    float sum = sink ? expf(sink_logit - mx) : 0.0f;
    for (int64_t j = 0; j < Sk; ++j) { s[j] = mx == -INFINITY ? 0.0f : expf(s[j] - mx); sum += s[j]; }
    float inv = sum > 0.0f ? 1.0f / sum : 0.0f;
    float *o = out + ((b * Hq + h) * Sq + i) * D;
    for (int64_t d = 0; d < D; ++d) o[d] = 0.0f;
    for (int64_t j = 0; j < Sk; ++j) {
      float p = s[j] * inv;
      const float *vj = v + ((b * Hkv + hk) * Sk + j) * D;
      for (int64_t d = 0; d < D; ++d) o[d] += p * vj[d];
    }
    free(s);
  }
}

/* ------------------------------------------------------------------ decode path
 * Rotary embedding: out = x * cos + rotate_half(x) * sin, rotate_half(x) = concat(-x[D/2:], x[:D/2])
 * (include/ttmlir/Dialect/TTNN/IR/TTNNOps.td:4002-4016; test/python/golden/ttir_ops/fusing/test_rope_fusing.py:24-33).
 * x [batch, rows, D]; cos / sin [cache_rows, D]; row s reads cache row s, or row token_index when token_index >= 0. */
void orc_rotary_embedding_f32(const float *x, const float *cosc, const float *sinc, float *out, int64_t batch,
                              int64_t rows, int64_t D, int64_t token_index) {
  const int64_t half = D / 2;
  for (int64_t b = 0; b < batch; ++b)
    for (int64_t s = 0; s < rows; ++s) {
      const float *xr = x + (b * rows + s) * D;
      const int64_t cr = token_index >= 0 ? token_index : s;
      const float *c = cosc + cr * D, *sn = sinc + cr * D;
      float *o = out + (b * rows + s) * D;
      for (int64_t d = 0; d < D; ++d) {
        const float rot = d < half ? -xr[d + half] : xr[d - half];
        o[d] = xr[d] * c[d] + rot * sn[d];
      }
    }
}

/* update_cache (tools/golden/mapping.py:3614-3671): cache [U,H,S,D] in place;
 * cache[batch_offset + b, h, idx, :] = input[0, h, b, :], input [1,H,Bin,D]. */
void orc_update_cache_f32(float *cache, const float *input, int64_t H, int64_t S, int64_t D, int64_t Bin,
                          int64_t idx, int64_t batch_offset) {
  for (int64_t b = 0; b < Bin; ++b)
    for (int64_t h = 0; h < H; ++h)
      memcpy(cache + (((batch_offset + b) * H + h) * S + idx) * D, input + (h * Bin + b) * D, sizeof(float) * D);
}

/* fill_cache (tools/golden/mapping.py:3582-3611 with the runner's batch_offset, operations/kv_cache/fill_cache.cpp:
 * 12-18): cache[batch_offset, :, :seq, :] = input[0]; rows seq .. round_up(seq, 32) become 0 when they exist. */
void orc_fill_cache_f32(float *cache, const float *input, int64_t H, int64_t S, int64_t D, int64_t seq,
                        int64_t batch_offset) {
  int64_t padded = (seq + 31) / 32 * 32;
  for (int64_t h = 0; h < H; ++h) {
    float *dst = cache + ((batch_offset * H + h) * S) * D;
    memcpy(dst, input + h * seq * D, sizeof(float) * seq * D);
    if (seq < padded && padded <= S) memset(dst + seq * D, 0, sizeof(float) * (padded - seq) * D);
  }
}

/* Attention of one new token (tools/golden/mapping.py:2417-2481): q [1,B,H,D], k / v [B,Hkv,S,D], mask (optional)
 * [B,1,mask_heads,S] additive BEFORE the scale, cur_pos (optional, with is_causal) excludes keys j > cur_pos[b];
 * scale <= 0 means 1/sqrt(D), the op's documented default (include/ttmlir/Dialect/TTNN/IR/TTNNOps.td:4130); the golden
 * leaves the logits unscaled when `scale is None` (mapping.py:2472), a deviation from it taken on purpose, since the
 * runtime passes the absent attribute on to the kernel, which applies the default.  out [1,B,H,D].
 * window >= 0: of the keys up to the decode position p only the last `window` are visible, [max(0, p - window + 1), p]
 * (mapping.py:8814-8824, the paged golden); p = cur_pos[b], or S - 1 without cur_pos, as the op's description has it
 * (include/ttmlir/Dialect/TTNN/IR/TTNNOps.td:4131-4134; the golden leaves the window out when cur_pos is absent).
 * sink (optional, one value per head = column 0 of the op's [H, 32] operand): one more logit per head, sink * scale, in the
 * softmax, with no value row - the prefill op's meaning (mapping.py:8476-8494) and what the lowering's comment says of
 * both kernels (TTIRToTTNN.cpp:3507-3508).  PARITY UNPINNED against the decode goldens for the sink: mapping.py:2417-2481
 * ignores the operand and mapping.py:8826-8829 only unmasks the first column, neither of which is the op.          */
void orc_sdpa_decode_f32(const float *q, const float *k, const float *v, const int32_t *cur_pos, const float *mask,
                         int mask_heads, float *out, int64_t B, int64_t H, int64_t Hkv, int64_t S, int64_t D,
                         int is_causal, float scale, int64_t window, const float *sink) {
  if (!(scale > 0.0f)) scale = 1.0f / sqrtf((float)D);
  int64_t rep = H / Hkv;
  float *s = (float *)malloc(sizeof(float) * S);
  for (int64_t b = 0; b < B; ++b)
    for (int64_t h = 0; h < H; ++h) {
      const float *qi = q + (b * H + h) * D;
      int64_t hk = h / rep;
      float mx = -INFINITY;
      for (int64_t j = 0; j < S; ++j) {
        const float *kj = k + ((b * Hkv + hk) * S + j) * D;
        float acc = 0.0f;
        for (int64_t d = 0; d < D; ++d) acc += qi[d] * kj[d];
        if (mask) acc += mask[(b * mask_heads + (mask_heads == 1 ? 0 : h)) * S + j];
        else if (is_causal && cur_pos && j > cur_pos[b]) acc = -INFINITY;
        if (window >= 0) {
          int64_t p = cur_pos ? cur_pos[b] : S - 1;
          if (j < p - window + 1) acc = -INFINITY;
        }
        acc *= scale;
        s[j] = acc;
        mx = acc > mx ? acc : mx;
      }
      float sink_logit = sink ? sink[h] * scale : -INFINITY;
      mx = sink_logit > mx ? sink_logit : mx;
      float sum = sink ? expf(sink_logit - mx) : 0.0f;
      for (int64_t j = 0; j < S; ++j) { s[j] = mx == -INFINITY ? 0.0f : expf(s[j] - mx); sum += s[j]; }
      if (!(sum > 0.0f)) sum = 1.0f;
      float *o = out + (b * H + h) * D;
      for (int64_t d = 0; d < D; ++d) o[d] = 0.0f;
      for (int64_t j = 0; j < S; ++j) {
        float p = s[j] / sum;
        const float *vj = v + ((b * Hkv + hk) * S + j) * D;
        for (int64_t d = 0; d < D; ++d) o[d] += p * vj[d];
      }
    }
  free(s);
}
