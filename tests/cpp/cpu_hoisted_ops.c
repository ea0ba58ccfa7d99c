/* Hand-written stand-in for a CPU-hoisted function library, with the ABI the compiler's wrappers have
 * (lib/Dialect/LLVM/Transforms/EmitWrapperFuncs.cpp:54-76; runtime/include/tt/runtime/detail/common/dylib.h:35-42, 128-175):
 *   WrappedTensor *<name>_helper(WrappedTensor *inputs)
 * dense row-major tensors; the callee mallocs the output array, one sizes-and-strides block shared by all outputs and
 * every data buffer; the runtime frees them.  Built by the test with `gcc -shared -fPIC`. */
#include <stdint.h>
#include <stdlib.h>

typedef struct {
  void *start;
  void *alignedStart;
  int64_t startIdx;
  int64_t *sizesAndStrides;
} WrappedTensor;

/* out0 = a + b (f32, same shape), out1 = row sums of out0 as int32 (truncated), shape [rows] */
WrappedTensor *cpu_hoisted_add_rowsum_0a1b2c3d_helper(WrappedTensor *in) {
  const int64_t rows = in[0].sizesAndStrides[0], cols = in[0].sizesAndStrides[1];
  const float *a = (const float *)in[0].alignedStart + in[0].startIdx;
  const float *b = (const float *)in[1].alignedStart + in[1].startIdx;
  WrappedTensor *out = (WrappedTensor *)malloc(2 * sizeof(WrappedTensor));
  int64_t *ss = (int64_t *)malloc(6 * sizeof(int64_t));
  ss[0] = rows; ss[1] = cols; ss[2] = cols; ss[3] = 1;   /* out0: sizes, strides */
  ss[4] = rows; ss[5] = 1;                               /* out1 */
  float *sum = (float *)malloc(sizeof(float) * rows * cols);
  int32_t *rs = (int32_t *)malloc(sizeof(int32_t) * rows);
  for (int64_t r = 0; r < rows; ++r) {
    float acc = 0.0f;
    for (int64_t c = 0; c < cols; ++c) {
      sum[r * cols + c] = a[r * cols + c] + b[r * cols + c];
      acc += sum[r * cols + c];
    }
    rs[r] = (int32_t)acc;
  }
  out[0].start = out[0].alignedStart = sum; out[0].startIdx = 0; out[0].sizesAndStrides = ss;
  out[1].start = out[1].alignedStart = rs; out[1].startIdx = 0; out[1].sizesAndStrides = ss + 4;
  return out;
}

/* two outputs that alias one buffer: the runtime must free it once */
WrappedTensor *cpu_hoisted_alias_helper(WrappedTensor *in) {
  const int64_t n = in[0].sizesAndStrides[0];
  const float *a = (const float *)in[0].alignedStart + in[0].startIdx;
  WrappedTensor *out = (WrappedTensor *)malloc(2 * sizeof(WrappedTensor));
  int64_t *ss = (int64_t *)malloc(2 * sizeof(int64_t));
  float *buf = (float *)malloc(sizeof(float) * n);
  ss[0] = n; ss[1] = 1;
  for (int64_t i = 0; i < n; ++i) buf[i] = 2.0f * a[i];
  for (int k = 0; k < 2; ++k) { out[k].start = out[k].alignedStart = buf; out[k].startIdx = 0; out[k].sizesAndStrides = ss; }
  return out;
}
