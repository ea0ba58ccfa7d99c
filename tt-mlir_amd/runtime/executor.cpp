// Program executor: walks the operations of one TTNN program and runs each through the gfx950
// kernel library.  Structure follows runtime/lib/ttnn/program_executor.cpp:146-266 (tensor pool keyed
// by global_id, pre/post hooks around every op, outputs gathered at the end) with one runner per
// flatbuffer op table (runtime/lib/ttnn/operations/**).  Ops outside the supported subset fail with
// the op name, like the reference's LOG_FATAL("Unsupported operation type").
#include <algorithm>
#include <set>
#include <cmath>
#include <cstring>
#include <map>
#include <sstream>

#include <dlfcn.h>
#include <sys/syscall.h>
#include <unistd.h>

#include "runtime_impl.h"

namespace tt::runtime {

using namespace ::ttmlir_amd;
using schema::OpType;

namespace {

int ttmDtype(DataType dt) { return static_cast<int>(dt); }
int ttmLayout(TensorLayout l) { return static_cast<int>(l); }

struct ProgramContext {
  std::shared_ptr<DeviceState> dev;
  Binary binary;
  std::uint32_t programIndex = 0;
  std::unordered_map<std::uint32_t, Tensor> pool;  // global_id -> live tensor
  // reshape / permute fusion (only when no hooks are registered): a reshape whose single consumer is the next permute is
  // not materialised, nor is a permute whose single consumer is the next update_cache (`deferred` keeps the source, the
  // logical shape of the result and, per result dimension, the stride in the source's row-major element order); a
  // permute whose single consumer is the next reshape writes the reshaped tensor directly (the reshape's index goes
  // into `skip`)
  struct DeferredView {
    Tensor source;
    std::vector<std::uint32_t> shape;
    std::vector<std::int64_t> strides;
  };
  std::vector<fb::Table> ops;
  std::uint32_t opIndex = 0;
  bool fuseViews = false;
  std::unordered_map<std::uint32_t, int> uses;      // consumers of a tensor (deallocations not counted; program outputs are)
  std::unordered_map<std::uint32_t, DeferredView> deferred;
  // head splits that feed scaled_dot_product_attention only: tensor id -> the [B, S, H * D] tensor it is the
  // [B, H, S, D] view of.  The id is not in the pool; the attention kernel reads the source in place.
  std::unordered_map<std::uint32_t, Tensor> headViews;
  std::set<std::uint32_t> skip;

  Tensor &get(const fb::Table &ref, const char *what) {
    TTRT_ASSERT(static_cast<bool>(ref), std::string("missing tensor reference: ") + what);
    std::uint32_t id = ref.scalar<std::uint32_t>(schema::TensorRef::f_global_id, 0);
    auto it = pool.find(id);
    TTRT_ASSERT(it != pool.end(), std::string("tensor ") + std::to_string(id) + " (" + what + ") is not in the tensor pool");
    TTRT_ASSERT(isTensorAllocated(it->second), std::string("tensor ") + std::to_string(id) + " (" + what + ") was deallocated");
    return it->second;
  }
  void put(const fb::Table &ref, Tensor t);

  void *stream() const { return dev->stream; }
};

// Tensor operands of an operation as the flatbuffer names them: `ins` in operand order (absent optional operands are
// skipped), `outs` in result order.  Ops outside the supported subset report nothing.
struct OpRefs {
  std::vector<fb::Table> ins, outs;
};

OpRefs opRefs(const fb::Table &operation) {
  auto type = static_cast<OpType>(operation.scalar<std::uint8_t>(schema::Operation::f_type_type, 0));
  fb::Table op = operation.table(schema::Operation::f_type);
  OpRefs r;
  auto in = [&](int slot) { if (fb::Table t = op.table(slot)) r.ins.push_back(t); };
  auto out = [&](int slot) { if (fb::Table t = op.table(slot)) r.outs.push_back(t); };
  auto inVec = [&](int slot) {
    auto v = op.tables(slot);
    for (std::uint32_t i = 0; i < v.size(); ++i) r.ins.push_back(v[i]);
  };
  auto outVec = [&](int slot) {
    auto v = op.tables(slot);
    for (std::uint32_t i = 0; i < v.size(); ++i) r.outs.push_back(v[i]);
  };
  switch (type) {
  case OpType::ToLayoutOp: in(schema::ToLayoutOp::f_in); out(schema::ToLayoutOp::f_out); break;
  case OpType::TypecastOp: in(schema::TypecastOp::f_in); out(schema::TypecastOp::f_out); break;
  case OpType::ToDeviceOp: in(schema::ToDeviceOp::f_in); out(schema::ToDeviceOp::f_out); break;
  case OpType::FromDeviceOp: in(schema::FromDeviceOp::f_in); out(schema::FromDeviceOp::f_out); break;
  case OpType::ToMemoryConfigOp: in(schema::ToMemoryConfigOp::f_in0); out(schema::ToMemoryConfigOp::f_out); break;
  case OpType::MatmulOp: in(schema::MatmulOp::f_a); in(schema::MatmulOp::f_b); out(schema::MatmulOp::f_out); break;
  case OpType::LinearOp:
    in(schema::LinearOp::f_a); in(schema::LinearOp::f_b); in(schema::LinearOp::f_bias); out(schema::LinearOp::f_out);
    break;
  case OpType::EltwiseUnaryOp: in(schema::EltwiseUnaryOp::f_in); out(schema::EltwiseUnaryOp::f_out); break;
  case OpType::EltwiseBinaryOp:
    in(schema::EltwiseBinaryOp::f_lhs); in(schema::EltwiseBinaryOp::f_rhs); out(schema::EltwiseBinaryOp::f_out);
    break;
  case OpType::RMSNormOp:
    in(schema::RMSNormOp::f_input); in(schema::RMSNormOp::f_weight); in(schema::RMSNormOp::f_bias); out(schema::RMSNormOp::f_out);
    break;
  case OpType::SoftmaxOp: in(schema::SoftmaxOp::f_in); out(schema::SoftmaxOp::f_out); break;
  case OpType::ReductionOp: in(schema::ReductionOp::f_in); out(schema::ReductionOp::f_out); break;
  case OpType::ScaledDotProductAttentionOp:
    in(schema::ScaledDotProductAttentionOp::f_query); in(schema::ScaledDotProductAttentionOp::f_key);
    in(schema::ScaledDotProductAttentionOp::f_value); in(schema::ScaledDotProductAttentionOp::f_attention_mask);
    in(schema::ScaledDotProductAttentionOp::f_attention_sink);
    out(schema::ScaledDotProductAttentionOp::f_out);
    break;
  case OpType::ReshapeOp: in(schema::ReshapeOp::f_in); out(schema::ReshapeOp::f_out); break;
  case OpType::PermuteOp: in(schema::PermuteOp::f_in); out(schema::PermuteOp::f_out); break;
  case OpType::TransposeOp: in(schema::TransposeOp::f_in); out(schema::TransposeOp::f_out); break;
  case OpType::ConcatOp: inVec(schema::ConcatOp::f_inputs); out(schema::ConcatOp::f_out); break;
  case OpType::SliceOp: in(schema::SliceOp::f_in); out(schema::SliceOp::f_out); break;
  case OpType::RepeatInterleaveOp: in(schema::RepeatInterleaveOp::f_input); out(schema::RepeatInterleaveOp::f_out); break;
  case OpType::RepeatOp: in(schema::RepeatOp::f_in); out(schema::RepeatOp::f_out); break;
  case OpType::ConcatenateHeadsOp: in(schema::ConcatenateHeadsOp::f_in); out(schema::ConcatenateHeadsOp::f_out); break;
  case OpType::NLPConcatHeadsOp: in(schema::NLPConcatHeadsOp::f_in); out(schema::NLPConcatHeadsOp::f_out); break;
  case OpType::NLPConcatHeadsDecodeOp: in(schema::NLPConcatHeadsDecodeOp::f_in); out(schema::NLPConcatHeadsDecodeOp::f_out); break;
  case OpType::NLPCreateQKVHeadsDecodeOp: {
    using S = schema::NLPCreateQKVHeadsDecodeOp;
    in(S::f_input); out(S::f_q_out); out(S::f_k_out); out(S::f_v_out);
    break;
  }
  case OpType::SplitQueryKeyValueAndSplitHeadsOp: {
    using S = schema::SplitQueryKeyValueAndSplitHeadsOp;
    in(S::f_in); in(S::f_kv_input); out(S::f_q_out); out(S::f_k_out); out(S::f_v_out);
    break;
  }
  case OpType::EltwiseUnaryCompositeOp: in(schema::EltwiseUnaryCompositeOp::f_in); out(schema::EltwiseUnaryCompositeOp::f_out); break;
  case OpType::EltwiseBinaryCompositeOp:
    in(schema::EltwiseBinaryCompositeOp::f_lhs); in(schema::EltwiseBinaryCompositeOp::f_rhs); out(schema::EltwiseBinaryCompositeOp::f_out);
    break;
  case OpType::EltwiseTernaryWhereOp:
    in(schema::EltwiseTernaryWhereOp::f_first); in(schema::EltwiseTernaryWhereOp::f_second); in(schema::EltwiseTernaryWhereOp::f_third);
    out(schema::EltwiseTernaryWhereOp::f_out);
    break;
  case OpType::EmbeddingOp: in(schema::EmbeddingOp::f_input); in(schema::EmbeddingOp::f_weight); out(schema::EmbeddingOp::f_out); break;
  case OpType::ReductionArgMaxOp: in(schema::ReductionArgMaxOp::f_in); out(schema::ReductionArgMaxOp::f_out); break;
  case OpType::ArangeOp: out(schema::ArangeOp::f_out); break;
  case OpType::ConstantOp: out(schema::ConstantOp::f_out); break;
  case OpType::FullOp: out(schema::FullOp::f_out); break;
  case OpType::NamedFullOp: out(schema::NamedFullOp::f_out); break;
  case OpType::EmptyOp: out(schema::EmptyOp::f_out); break;
  case OpType::DeallocateOp: in(schema::DeallocateOp::f_in); break;
  case OpType::LoadCachedOp: inVec(schema::LoadCachedOp::f_inputs); outVec(schema::LoadCachedOp::f_outputs); break;
  case OpType::FuncCallOp: inVec(schema::FuncCallOp::f_inputs); outVec(schema::FuncCallOp::f_outputs); break;
  case OpType::CpuOp: inVec(schema::CpuOp::f_ins); outVec(schema::CpuOp::f_outs); break;
  case OpType::RotaryEmbeddingLlamaOp:
    in(schema::RotaryEmbeddingLlamaOp::f_input); in(schema::RotaryEmbeddingLlamaOp::f_cos_cache);
    in(schema::RotaryEmbeddingLlamaOp::f_sin_cache); in(schema::RotaryEmbeddingLlamaOp::f_trans_mat);
    out(schema::RotaryEmbeddingLlamaOp::f_out);
    break;
  case OpType::ChunkedScaledDotProductAttentionOp:
    in(schema::ChunkedScaledDotProductAttentionOp::f_query); in(schema::ChunkedScaledDotProductAttentionOp::f_key);
    in(schema::ChunkedScaledDotProductAttentionOp::f_value); in(schema::ChunkedScaledDotProductAttentionOp::f_page_table);
    in(schema::ChunkedScaledDotProductAttentionOp::f_chunk_start_idx); out(schema::ChunkedScaledDotProductAttentionOp::f_out);
    break;
  case OpType::RotaryEmbeddingOp:
    in(schema::RotaryEmbeddingOp::f_input); in(schema::RotaryEmbeddingOp::f_cos_cache); in(schema::RotaryEmbeddingOp::f_sin_cache);
    out(schema::RotaryEmbeddingOp::f_out);
    break;
  case OpType::UpdateCacheOp:
    in(schema::UpdateCacheOp::f_cache); in(schema::UpdateCacheOp::f_input); in(schema::UpdateCacheOp::f_update_index);
    break;
  case OpType::FillCacheOp: in(schema::FillCacheOp::f_cache); in(schema::FillCacheOp::f_input); break;
  case OpType::PagedUpdateCacheOp: {
    using S = schema::PagedUpdateCacheOp;
    in(S::f_cache); in(S::f_input); in(S::f_update_index); in(S::f_page_table);
    break;
  }
  case OpType::PagedFillCacheOp: {
    using S = schema::PagedFillCacheOp;
    in(S::f_cache); in(S::f_input); in(S::f_page_table); in(S::f_batch_idx_tensor);
    break;
  }
  case OpType::ScaledDotProductAttentionDecodeOp: {
    using S = schema::ScaledDotProductAttentionDecodeOp;
    in(S::f_query); in(S::f_key); in(S::f_value); in(S::f_attention_mask); in(S::f_cur_pos_tensor); in(S::f_attention_sink); out(S::f_out);
    break;
  }
  case OpType::PagedScaledDotProductAttentionDecodeOp: {
    using S = schema::PagedScaledDotProductAttentionDecodeOp;
    in(S::f_query); in(S::f_key); in(S::f_value); in(S::f_page_table); in(S::f_attention_mask); in(S::f_cur_pos_tensor); in(S::f_attention_sink); out(S::f_out);
    break;
  }
  case OpType::CaptureOrExecuteTraceOp:
    inVec(schema::CaptureOrExecuteTraceOp::f_inputs); outVec(schema::CaptureOrExecuteTraceOp::f_outputs);
    break;
  case OpType::WriteTensorOp: in(schema::WriteTensorOp::f_host_tensor); in(schema::WriteTensorOp::f_device_tensor); break;
  case OpType::CopyOp: in(schema::CopyOp::f_src); in(schema::CopyOp::f_dst); break;
  case OpType::BeginTraceCaptureOp: out(schema::BeginTraceCaptureOp::f_trace_id); break;
  case OpType::EndTraceCaptureOp: in(schema::EndTraceCaptureOp::f_trace_id); break;
  case OpType::ExecuteTraceOp: in(schema::ExecuteTraceOp::f_trace_id); break;
  default: break;
  }
  return r;
}


// ---- helpers
Tensor onDevice(ProgramContext &ctx, const Tensor &t) { return t.handle->storage == StorageType::Device ? t : toDevice(t, ctx.dev); }

// a device tensor in (layout, dtype); never frees its argument
Tensor as(ProgramContext &ctx, const Tensor &t, TensorLayout layout, DataType dtype) { return convertOnDevice(onDevice(ctx, t), layout, dtype); }

Tensor convertTo(ProgramContext &ctx, const Tensor &t, const Layout &target) {
  Tensor cur = t;
  const bool change = cur.handle->layout != target.layout || cur.handle->dtype != target.dataType;
  if (change || target.storageType == StorageType::Device) cur = as(ctx, cur, target.layout, target.dataType);
  if (target.storageType == StorageType::Host && cur.handle->storage == StorageType::Device) cur = fromDevice(cur);
  return cur;
}

std::vector<std::int64_t> rowMajorStrides(const std::vector<std::uint32_t> &shape) {
  std::vector<std::int64_t> s(shape.size(), 1);
  for (int i = static_cast<int>(shape.size()) - 2; i >= 0; --i) s[i] = s[i + 1] * shape[i + 1];
  return s;
}

bool hasPadding(const std::vector<std::uint32_t> &shape) {
  Dims3 d = dims3(shape);
  return d.rows % 32 != 0 || d.cols % 32 != 0;
}

// zero a freshly made tile tensor whose padding the producing kernel does not write
void zeroIfPadded(ProgramContext &ctx, const Tensor &t) {
  if (t.handle->layout == TensorLayout::Tile && hasPadding(t.handle->shape))
    TTM_CALL(ttm_fill_u32(t.handle->data.get(), 0, (t.handle->bytes + 3) / 4, ctx.stream()));
}

// generic strided copy between two device tensors (any layouts) through ttm_copy_view
void copyView(ProgramContext &ctx, const Tensor &src, const Tensor &dst, const std::vector<std::int64_t> &extent,
              const std::vector<std::int64_t> &sstride, std::int64_t sbase, const std::vector<std::int64_t> &dstride,
              std::int64_t dbase) {
  TTRT_ASSERT(src.handle->dtype == dst.handle->dtype, "copyView: dtype mismatch");
  TTRT_ASSERT(!utils::isBlockFormatDataType(src.handle->dtype), "data movement on block-float tensors is not supported");
  // collapse to at most 8 view dims by merging leading ones when needed
  std::vector<std::int64_t> e = extent, ss = sstride, ds = dstride;
  TTRT_ASSERT(e.size() <= 8, "copyView: rank above 8");
  Dims3 sd = dims3(src.handle->shape), dd = dims3(dst.handle->shape);
  debug::Stats::get().incrementStat("CopyViewLaunch");
  TTM_CALL(ttm_copy_view(src.handle->data.get(), sd.rows, sd.cols, ttmLayout(src.handle->layout), dst.handle->data.get(), dd.rows,
                         dd.cols, ttmLayout(dst.handle->layout), static_cast<int>(utils::dataTypeElementSize(src.handle->dtype)),
                         static_cast<int>(e.size()), e.data(), ss.data(), sbase, ds.data(), dbase, ctx.stream()));
}

std::vector<std::int64_t> toI64(const std::vector<std::uint32_t> &v) { return std::vector<std::int64_t>(v.begin(), v.end()); }

Tensor makeOut(ProgramContext &ctx, const fb::Table &outRef, DataType dtype, TensorLayout layout) {
  return makeDeviceTensor(ctx.dev, shapeFromTensorRef(outRef), dtype, layout);
}

std::string shapeText(const std::vector<std::uint32_t> &s);
// A tensor enters the pool under the reference the program declares for it.  Its shape must be the declared one: later
// operations size their launches from the tensors they find here, and a program whose declarations do not agree with
// what its operations produce is refused at the first such result rather than run on shapes it did not state.
void ProgramContext::put(const fb::Table &ref, Tensor t) {
  std::uint32_t id = ref.scalar<std::uint32_t>(schema::TensorRef::f_global_id, 0);
  if (t.handle) {
    const std::vector<std::uint32_t> declared = shapeFromTensorRef(ref);
    TTRT_ASSERT(t.handle->shape == declared, "tensor " + std::to_string(id) + ": the program declares the shape " + shapeText(declared) +
                                                 ", the operation produced " + shapeText(t.handle->shape));
  }
  pool[id] = std::move(t);
}
std::string shapeText(const std::vector<std::uint32_t> &s) {
  std::string t = "[";
  for (size_t i = 0; i < s.size(); ++i) t += (i ? ", " : "") + std::to_string(s[i]);
  return t + "]";
}
// The kernels are launched from the operands' extents while the result is allocated from the shape the program declares
// for it: a program that declares another shape than its operands give must be refused here, before a launch writes past
// the allocation.
void requireResultShape(const fb::Table &outRef, const std::vector<std::uint32_t> &want, const char *op) {
  const std::vector<std::uint32_t> declared = shapeFromTensorRef(outRef);
  TTRT_ASSERT(declared == want, std::string(op) + ": the program declares the result as " + shapeText(declared) + ", the operands give " +
                                    shapeText(want));
}
// the same when only the extent the kernel writes is known: [batch, rows, cols] in the tile layout
void requireResultExtent(const Tensor &out, std::int64_t batch, std::int64_t rows, std::int64_t cols, const char *op) {
  const auto r32 = [](std::int64_t n) { return (n + 31) / 32 * 32; };
  TTRT_ASSERT(paddedVolume(out.handle->shape) == batch * r32(rows) * r32(cols),
              std::string(op) + ": the program declares the result as " + shapeText(out.handle->shape) + ", the operands give a [" +
                  std::to_string(batch) + ", " + std::to_string(rows) + ", " + std::to_string(cols) + "] product");
}

// final cast of an op result to what the program's TensorRef declares (dtype and layout)
Tensor finish(ProgramContext &ctx, const Tensor &t, const fb::Table &outRef) {
  Layout want = layoutFromTensorRef(outRef);
  if (want.storageType == StorageType::Host) return convertTo(ctx, t, want);
  return as(ctx, t, want.layout, want.dataType);
}

int activationCode(std::string_view s) {
  if (s.empty()) return TTM_ACT_NONE;
  if (s == "gelu") return TTM_ACT_GELU;
  if (s == "silu") return TTM_ACT_SILU;
  if (s == "sigmoid") return TTM_ACT_SIGMOID;
  if (s == "relu") return TTM_ACT_RELU;
  fatal("unsupported fused activation '" + std::string(s) + "'");
}

// The activation a matmul / linear op applies (runtime/lib/ttnn/operations/matmul/matmul.cpp:17-44, 64-66, 116-119): the
// multicast program configs carry a fused_activation of their own, and when one is present it is the one that runs; the
// op's `activation` string counts only without it.
std::string matmulActivation(const fb::Table &op, int configTypeSlot, int configSlot, int activationSlot) {
  const auto kind = static_cast<schema::MatmulProgramConfig>(op.scalar<std::uint8_t>(configTypeSlot, 0));
  int fusedSlot = -1;
  switch (kind) {
  case schema::MatmulProgramConfig::MatmulMultiCoreReuseMultiCastProgramConfig:
    fusedSlot = schema::MatmulMultiCoreReuseMultiCastProgramConfig::f_fused_activation; break;
  case schema::MatmulProgramConfig::MatmulMultiCoreReuseMultiCast1DProgramConfig:
    fusedSlot = schema::MatmulMultiCoreReuseMultiCast1DProgramConfig::f_fused_activation; break;
  case schema::MatmulProgramConfig::MatmulMultiCoreReuseMultiCastDRAMShardedProgramConfig:
    fusedSlot = schema::MatmulMultiCoreReuseMultiCastDRAMShardedProgramConfig::f_fused_activation; break;
  default: break;
  }
  if (fusedSlot >= 0) {
    if (fb::Table config = op.table(configSlot)) {
      if (fb::Table fused = config.table(fusedSlot)) {
        const auto type = static_cast<schema::UnaryOpType>(fused.scalar<std::uint32_t>(schema::UnaryWithParam::f_op_type, 0));
        switch (type) {
        case schema::UnaryOpType::Gelu: return "gelu";
        case schema::UnaryOpType::Relu: return "relu";
        case schema::UnaryOpType::Sigmoid: return "sigmoid";
        case schema::UnaryOpType::Silu: return "silu";
        default: fatal("unsupported fused activation in the matmul program config: UnaryOpType " + std::to_string(static_cast<std::uint32_t>(type)));
        }
      }
    }
  }
  return std::string(op.string(activationSlot));
}

// ---- layout ops (runtime/lib/ttnn/operations/layout/*.cpp)
void runToLayout(const fb::Table &op, ProgramContext &ctx) {
  Tensor in = ctx.get(op.table(schema::ToLayoutOp::f_in), "to_layout in");
  auto outRef = op.table(schema::ToLayoutOp::f_out);
  Layout want = layoutFromTensorRef(outRef);
  want.layout = static_cast<TensorLayout>(op.scalar<std::uint16_t>(schema::ToLayoutOp::f_layout, 0));
  if (op.has(schema::ToLayoutOp::f_dtype)) want.dataType = static_cast<DataType>(op.scalar<std::uint16_t>(schema::ToLayoutOp::f_dtype, 0));
  ctx.put(outRef, convertTo(ctx, in, want));
}
void runTypecast(const fb::Table &op, ProgramContext &ctx) {
  Tensor in = ctx.get(op.table(schema::TypecastOp::f_in), "typecast in");
  DataType dt = static_cast<DataType>(op.scalar<std::uint16_t>(schema::TypecastOp::f_dtype, 0));
  TensorLayout l = utils::isBlockFormatDataType(dt) ? TensorLayout::Tile : in.handle->layout;
  Tensor out = as(ctx, in, l, dt);
  auto outRef = op.table(schema::TypecastOp::f_out);
  if (layoutFromTensorRef(outRef).storageType == StorageType::Host) out = fromDevice(out);
  ctx.put(outRef, out);
}
void runToDevice(const fb::Table &op, ProgramContext &ctx) {
  Tensor in = ctx.get(op.table(schema::ToDeviceOp::f_in), "to_device in");
  ctx.put(op.table(schema::ToDeviceOp::f_out), onDevice(ctx, in));
}
void runFromDevice(const fb::Table &op, ProgramContext &ctx) {
  Tensor in = ctx.get(op.table(schema::FromDeviceOp::f_in), "from_device in");
  ctx.put(op.table(schema::FromDeviceOp::f_out), in.handle->storage == StorageType::Device ? fromDevice(in) : in);
}
void runToMemoryConfig(const fb::Table &op, ProgramContext &ctx) {
  // one memory space on this device: the tensor is passed through
  ctx.put(op.table(schema::ToMemoryConfigOp::f_out), ctx.get(op.table(schema::ToMemoryConfigOp::f_in0), "to_memory_config in"));
}

std::uint32_t refId(const fb::Table &ref);
Tensor materialiseView(ProgramContext &ctx, const ProgramContext::DeferredView &v, const std::vector<std::uint32_t> *finalShape);
fb::Table fusableNext(ProgramContext &ctx, OpType type, int inSlot, int outSlot, const fb::Table &produced, const Tensor &like);

// ---- matmul / linear (runtime/lib/ttnn/operations/matmul/matmul.cpp:47-125)
Tensor transposeLast2(ProgramContext &ctx, const Tensor &t) {
  std::vector<std::uint32_t> shape = t.handle->shape;
  TTRT_ASSERT(shape.size() >= 2, "transpose needs rank >= 2");
  std::vector<std::uint32_t> oshape = shape;
  std::swap(oshape[oshape.size() - 1], oshape[oshape.size() - 2]);
  Tensor out = makeDeviceTensor(ctx.dev, oshape, t.handle->dtype, t.handle->layout);
  zeroIfPadded(ctx, out);
  auto ss = rowMajorStrides(shape);
  std::swap(ss[ss.size() - 1], ss[ss.size() - 2]);
  copyView(ctx, t, out, toI64(oshape), ss, 0, rowMajorStrides(oshape), 0);
  return out;
}

// TTMLIR_RUNTIME_NO_DECODE_FUSION=1 keeps the decode-step fusions below off (the ops then run as the smaller fusions or
// one by one): for measurements and for telling a fusion's fault from a kernel's
bool decodeFusionEnabled() {
  static const bool on = [] { const char *e = std::getenv("TTMLIR_RUNTIME_NO_DECODE_FUSION"); return !(e && e[0] == '1'); }();
  return on;
}

// The op that consumes tensor `id` after op `from`, when the tensor has exactly one consumer (deallocations aside); else 0
std::uint32_t soleConsumer(ProgramContext &ctx, std::uint32_t id, std::uint32_t from) {
  auto u = ctx.uses.find(id);
  if (u == ctx.uses.end() || u->second != 1) return 0;
  for (std::uint32_t j = from + 1; j < ctx.ops.size(); ++j) {
    if (static_cast<OpType>(ctx.ops[j].scalar<std::uint8_t>(schema::Operation::f_type_type, 0)) == OpType::DeallocateOp) continue;
    for (const auto &ref : opRefs(ctx.ops[j]).ins)
      if (refId(ref) == id) return j;
  }
  return 0;
}

// A traced function ends by copying each result into the trace's output slot
// (lib/Dialect/TTNN/Transforms/TTNNTraceHoistTransform.cpp:452).  When the `copy` that is the only reader of tensor
// `produced` follows op `from` with nothing but deallocations of other tensors between, and its destination is a live
// device tensor of the same shape in the plain bf16 tile layout whose buffer is none of `operands`, the producer can write
// into the destination and the copy be skipped: returns the destination and the copy's index, or an empty tensor.
Tensor copyDestinationOf(ProgramContext &ctx, std::uint32_t from, const fb::Table &produced, const std::vector<const Tensor *> &operands,
                         std::uint32_t *copyIndex) {
  if (!ctx.fuseViews || !decodeFusionEnabled()) return Tensor();
  const Layout plain{StorageType::Device, TensorLayout::Tile, DataType::BFloat16};
  if (!(layoutFromTensorRef(produced) == plain)) return Tensor();
  const std::uint32_t id = refId(produced);
  auto u = ctx.uses.find(id);
  if (u == ctx.uses.end() || u->second != 1) return Tensor();
  std::vector<std::uint32_t> freed;
  std::uint32_t j = from + 1;
  auto typeOf = [&](std::uint32_t i) { return static_cast<OpType>(ctx.ops[i].scalar<std::uint8_t>(schema::Operation::f_type_type, 0)); };
  for (; j < ctx.ops.size() && typeOf(j) == OpType::DeallocateOp; ++j)
    freed.push_back(refId(ctx.ops[j].table(schema::Operation::f_type).table(schema::DeallocateOp::f_in)));
  if (j >= ctx.ops.size() || typeOf(j) != OpType::CopyOp || ctx.skip.count(j)) return Tensor();
  fb::Table cop = ctx.ops[j].table(schema::Operation::f_type);
  fb::Table src = cop.table(schema::CopyOp::f_src), dst = cop.table(schema::CopyOp::f_dst);
  if (!src || !dst || refId(src) != id || refId(dst) == id) return Tensor();
  if (std::find(freed.begin(), freed.end(), id) != freed.end() || std::find(freed.begin(), freed.end(), refId(dst)) != freed.end())
    return Tensor();
  auto it = ctx.pool.find(refId(dst));
  if (it == ctx.pool.end() || !isTensorAllocated(it->second) || !(getTensorLayout(it->second) == plain) ||
      it->second.handle->shape != shapeFromTensorRef(produced))
    return Tensor();
  for (const Tensor *t : operands)
    if (t && t->handle && t->handle->data.get() == it->second.handle->data.get()) return Tensor();
  *copyIndex = j;
  return it->second;
}

// The front of a decode step's attention block: three projections of the same <= 32 tokens (block-float weights) whose
// results go, each through its own chain of single-consumer ops, to
//   q: reshape [1, users, heads, D] -> rotary_embedding(token_index)                       -> whoever reads q
//   k: reshape [1, users, kv, D]    -> rotary_embedding(token_index) -> permute(0, 2, 1, 3) -> update_cache(k cache)
//   v: reshape [1, users, kv, D]                                     -> permute(0, 2, 1, 3) -> update_cache(v cache)
// (test/ttmlir/models/single_blocks_and_layers/llama_3_8b_decode_layer.mlir:51-82 after RoPE and cache fusing) run as one
// projection launch whose partial sums a second kernel turns into q and the two cache rows.  Nothing else may sit between
// the first projection and the last cache update except deallocations, so running the cache writes early is not observable.
// members: (op index, out ref, weight) of the three projections.  Returns false, with nothing changed, when the pattern or a
// shape does not fit.
struct QkvMember { std::uint32_t index; fb::Table out; Tensor weight; };
bool tryQkvDecode(ProgramContext &ctx, const Tensor &a, std::int64_t users, std::int64_t K, const std::vector<QkvMember> &members) {
  if (!decodeFusionEnabled() || members.size() != 3 || users > 32 || a.handle->shape.size() != 2) return false;
  auto typeOf = [&](std::uint32_t i) { return static_cast<OpType>(ctx.ops[i].scalar<std::uint8_t>(schema::Operation::f_type_type, 0)); };
  auto body = [&](std::uint32_t i) { return ctx.ops[i].table(schema::Operation::f_type); };
  const Layout plain{StorageType::Device, TensorLayout::Tile, DataType::BFloat16};
  struct Chain { int member = -1; std::uint32_t reshape = 0, rotary = 0, permute = 0, update = 0; std::uint32_t nh = 0; };
  Chain q, k, v;
  std::set<std::uint32_t> chainOps;
  std::uint32_t D = 0, last = 0;
  for (int mi = 0; mi < 3; ++mi) {
    Chain c;
    c.member = mi;
    chainOps.insert(members[mi].index);
    c.reshape = soleConsumer(ctx, refId(members[mi].out), members[mi].index);
    if (!c.reshape || typeOf(c.reshape) != OpType::ReshapeOp || ctx.skip.count(c.reshape)) return false;
    fb::Table rs = body(c.reshape).table(schema::ReshapeOp::f_out);
    const std::vector<std::uint32_t> shape = shapeFromTensorRef(rs);
    if (!rs || !(layoutFromTensorRef(rs) == plain) || shape.size() != 4 || shape[0] != 1 || shape[1] != users || shape[3] % 32 != 0) return false;
    if (D && D != shape[3]) return false;
    D = shape[3];
    c.nh = shape[2];
    if (static_cast<std::int64_t>(c.nh) * D != members[mi].weight.handle->shape[1]) return false;
    std::uint32_t next = soleConsumer(ctx, refId(rs), c.reshape);
    if (!next || ctx.skip.count(next)) return false;
    std::uint32_t produced = refId(rs), after = c.reshape;
    if (typeOf(next) == OpType::RotaryEmbeddingOp) {
      using R = schema::RotaryEmbeddingOp;
      fb::Table rop = body(next);
      if (!rop.table(R::f_input) || refId(rop.table(R::f_input)) != produced || !rop.has(R::f_token_index) || !rop.table(R::f_out) ||
          !(layoutFromTensorRef(rop.table(R::f_out)) == plain) || shapeFromTensorRef(rop.table(R::f_out)) != shape)
        return false;
      c.rotary = next;
      produced = refId(rop.table(R::f_out));
      after = next;
      next = soleConsumer(ctx, produced, after);   // 0 when q has several readers: fine for q
    }
    if (next && !ctx.skip.count(next) && typeOf(next) == OpType::PermuteOp) {
      fb::Table pop = body(next);
      auto pv = pop.scalars<std::int64_t>(schema::PermuteOp::f_permutation);
      fb::Table pout = pop.table(schema::PermuteOp::f_out);
      if (pv.size() == 4 && pv[0] == 0 && pv[1] == 2 && pv[2] == 1 && pv[3] == 3 && pout && refId(pop.table(schema::PermuteOp::f_in)) == produced) {
        const std::uint32_t upd = soleConsumer(ctx, refId(pout), next);
        if (upd && !ctx.skip.count(upd) && typeOf(upd) == OpType::UpdateCacheOp &&
            refId(body(upd).table(schema::UpdateCacheOp::f_input)) == refId(pout)) {
          c.permute = next;
          c.update = upd;
        }
      }
    }
    if (c.rotary && !c.update) { if (q.member >= 0) return false; q = c; }
    else if (c.rotary && c.update) { if (k.member >= 0) return false; k = c; }
    else if (c.update) { if (v.member >= 0) return false; v = c; }
    else return false;
    for (std::uint32_t o : {c.reshape, c.rotary, c.permute, c.update})
      if (o) { chainOps.insert(o); last = std::max(last, o); }
  }
  if (q.member < 0 || k.member < 0 || v.member < 0 || k.nh != v.nh || q.nh % k.nh != 0) return false;
  // only the chains and deallocations between the first projection and the last cache update
  for (std::uint32_t j = ctx.opIndex; j <= last; ++j)
    if (!chainOps.count(j) && typeOf(j) != OpType::DeallocateOp) return false;
  using R = schema::RotaryEmbeddingOp;
  using U = schema::UpdateCacheOp;
  fb::Table rq = body(q.rotary), rk = body(k.rotary), uk = body(k.update), uv = body(v.update);
  if (refId(rq.table(R::f_cos_cache)) != refId(rk.table(R::f_cos_cache)) || refId(rq.table(R::f_sin_cache)) != refId(rk.table(R::f_sin_cache)) ||
      rq.scalar<std::uint32_t>(R::f_token_index, 0) != rk.scalar<std::uint32_t>(R::f_token_index, 0) ||
      refId(uk.table(U::f_update_index)) != refId(uv.table(U::f_update_index)) ||
      uk.scalar<std::uint32_t>(U::f_batch_offset, 0) != uv.scalar<std::uint32_t>(U::f_batch_offset, 0) ||
      refId(uk.table(U::f_cache)) == refId(uv.table(U::f_cache)))
    return false;
  auto live = [&](const fb::Table &ref) {
    auto it = ref ? ctx.pool.find(refId(ref)) : ctx.pool.end();
    return it != ctx.pool.end() && isTensorAllocated(it->second) ? &it->second : nullptr;
  };
  Tensor *cosT = live(rq.table(R::f_cos_cache)), *sinT = live(rq.table(R::f_sin_cache)), *idxT = live(uk.table(U::f_update_index));
  Tensor *kc = live(uk.table(U::f_cache)), *vc = live(uv.table(U::f_cache));
  if (!cosT || !sinT || !idxT || !kc || !vc) return false;
  const Layout cl = getTensorLayout(*cosT);
  if (!(cl == plain) || !(getTensorLayout(*sinT) == plain) || !(getTensorLayout(*kc) == plain) || !(getTensorLayout(*vc) == plain)) return false;
  const auto &cs = cosT->handle->shape, &ks = kc->handle->shape;
  const std::uint32_t token = rq.scalar<std::uint32_t>(R::f_token_index, 0), offset = uk.scalar<std::uint32_t>(U::f_batch_offset, 0);
  if (cs.size() != 4 || sinT->handle->shape != cs || cs[0] != 1 || cs[1] != 1 || cs[3] != D || token >= cs[2]) return false;
  if (ks.size() != 4 || vc->handle->shape != ks || ks[1] != k.nh || ks[3] != D || offset + users > ks[0]) return false;
  if (idxT->handle->storage != StorageType::Device || idxT->handle->layout != TensorLayout::RowMajor ||
      (idxT->handle->dtype != DataType::Int32 && idxT->handle->dtype != DataType::UInt32) || volume(idxT->handle->shape) < 1)
    return false;
  const int wdt = ttmDtype(members[0].weight.handle->dtype);
  if (!ttm_linear_qkv_decode_supported(wdt, users, K, q.nh, k.nh, D)) return false;

  fb::Table qRef = rq.table(R::f_out);
  Tensor qOut = makeOut(ctx, qRef, DataType::BFloat16, TensorLayout::Tile);
  TTM_CALL(ttm_linear_qkv_decode(a.handle->data.get(), members[q.member].weight.handle->data.get(), members[k.member].weight.handle->data.get(),
                                 members[v.member].weight.handle->data.get(), wdt, users, K, q.nh, k.nh, D, cosT->handle->data.get(),
                                 sinT->handle->data.get(), cs[2], token, qOut.handle->data.get(), kc->handle->data.get(), vc->handle->data.get(),
                                 ks[0], ks[2], static_cast<const std::int32_t *>(idxT->handle->data.get()), offset, ctx.stream()));
  ctx.put(qRef, finish(ctx, qOut, qRef));
  kc->handle->version = nextTensorVersion();
  vc->handle->version = nextTensorVersion();
  for (std::uint32_t o : chainOps)
    if (o != ctx.opIndex) ctx.skip.insert(o);
  debug::Stats::get().incrementStat("FusedQkvDecode");
  return true;
}

void runMatmulLike(ProgramContext &ctx, const fb::Table &aRef, const fb::Table &bRef, const fb::Table &biasRef, const fb::Table &outRef,
                   bool transposeA, bool transposeB, std::string_view activation) {
  Tensor a = as(ctx, ctx.get(aRef, "matmul a"), TensorLayout::Tile, DataType::BFloat16);
  Tensor b = onDevice(ctx, ctx.get(bRef, "matmul b"));
  if (!utils::isBlockFormatDataType(b.handle->dtype)) b = as(ctx, b, TensorLayout::Tile, DataType::BFloat16);
  TTRT_ASSERT(b.handle->layout == TensorLayout::Tile, "matmul: weights must be in tile layout");
  if (transposeA) a = transposeLast2(ctx, a);
  if (transposeB && utils::isBlockFormatDataType(b.handle->dtype)) {
    // block-float rows share exponents along n: transpose through bf16
    b = transposeLast2(ctx, as(ctx, b, TensorLayout::Tile, DataType::BFloat16));
    transposeB = false;
  }
  const auto &as_ = a.handle->shape, &bs = b.handle->shape;
  TTRT_ASSERT(!as_.empty() && !bs.empty(), "matmul: scalar operands are not supported");
  Dims3 ad = dims3(as_), bd = dims3(bs);
  std::int64_t M = ad.rows, K = ad.cols;
  std::int64_t Kb = transposeB ? bd.cols : bd.rows, N = transposeB ? bd.rows : bd.cols;
  if (as_.size() == 1) { M = 1; K = as_[0]; }
  TTRT_ASSERT(K == Kb, "matmul: inner dimensions differ (" + std::to_string(K) + " vs " + std::to_string(Kb) + ")");
  std::int64_t batch = ad.batch, wbatch = bd.batch;
  TTRT_ASSERT(wbatch == 1 || wbatch == batch, "matmul: RHS batch must be 1 or match the LHS batch");
  // shared weights: fold the LHS batch into M when that does not cross tile padding
  if (wbatch == 1 && batch > 1 && M % 32 == 0) { M *= batch; batch = 1; }
  const void *biasPtr = nullptr;
  int biasLayout = TTM_TILE;
  Tensor bias;
  if (biasRef) {
    bias = as(ctx, ctx.get(biasRef, "linear bias"), TensorLayout::Tile, DataType::BFloat16);
    TTRT_ASSERT(volume(bias.handle->shape) == N, "linear: bias must have N elements");
    biasPtr = bias.handle->data.get();
  }
  Tensor out = makeOut(ctx, outRef, DataType::BFloat16, TensorLayout::Tile);
  requireResultExtent(out, batch, M, N, "matmul");
  // an `add` or `multiply` that is the only consumer of this result and comes next runs in the kernel's epilogue
  // (residual connections, SiLU(gate) * up); its output takes this op's place
  Tensor tail;
  int tailOp = TTM_TAIL_NONE;
  fb::Table finalRef = outRef;
  // deallocations of other tensors may sit between the two ops (the compiler frees the matmul's operand right after it)
  std::uint32_t nextIdx = ctx.opIndex + 1;
  auto opType = [&](std::uint32_t i) { return static_cast<OpType>(ctx.ops[i].scalar<std::uint8_t>(schema::Operation::f_type_type, 0)); };
  std::vector<std::uint32_t> freedBetween;
  while (ctx.fuseViews && nextIdx < ctx.ops.size() && opType(nextIdx) == OpType::DeallocateOp) {
    freedBetween.push_back(refId(ctx.ops[nextIdx].table(schema::Operation::f_type).table(schema::DeallocateOp::f_in)));
    ++nextIdx;
  }
  if (ctx.fuseViews && nextIdx < ctx.ops.size()) {
    const fb::Table &next = ctx.ops[nextIdx];
    if (opType(nextIdx) == OpType::EltwiseBinaryOp) {
      using B = schema::EltwiseBinaryOp;
      fb::Table bop = next.table(schema::Operation::f_type);
      const std::uint32_t kind = bop.scalar<std::uint32_t>(B::f_type, 0);
      fb::Table lhs = bop.table(B::f_lhs), rhs = bop.table(B::f_rhs), bout = bop.table(B::f_out);
      const std::uint32_t mine = refId(outRef);
      auto uses = ctx.uses.find(mine);
      const Layout plain{StorageType::Device, TensorLayout::Tile, DataType::BFloat16};
      if ((kind == 0 || kind == 1) && lhs && rhs && bout && (refId(lhs) == mine) != (refId(rhs) == mine) && uses != ctx.uses.end() &&
          uses->second == 1 && layoutFromTensorRef(outRef) == plain && layoutFromTensorRef(bout) == plain &&
          shapeFromTensorRef(bout) == shapeFromTensorRef(outRef)) {
        const std::uint32_t otherId = refId(refId(lhs) == mine ? rhs : lhs);
        const bool freed = std::find(freedBetween.begin(), freedBetween.end(), otherId) != freedBetween.end() ||
                           std::find(freedBetween.begin(), freedBetween.end(), mine) != freedBetween.end();
        auto it = ctx.pool.find(otherId);
        if (!freed && it != ctx.pool.end() && isTensorAllocated(it->second) && getTensorLayout(it->second) == plain &&
            it->second.handle->shape == out.handle->shape) {
          tail = it->second;
          tailOp = kind == 0 ? TTM_TAIL_ADD : TTM_TAIL_MUL;
          finalRef = bout;
          ctx.skip.insert(nextIdx);
          debug::Stats::get().incrementStat("FusedLinearTail");
        }
      }
    }
  }
  // Further matmuls / bias-free linears of the same activations with block-float weights of the same format a few ops
  // further on (the Q, K and V projections; the gate and up projections of an MLP) run in this launch, each with its own
  // activation; only reshapes, permutes, rotary embeddings and deallocations of other tensors may lie between.  A follower
  // that has an add / multiply of its own to fuse is left alone, unless the token count is one where a projection alone
  // would split K to fill the device (64 < M <= 1024): there one unsplit launch for all members wins and the follower's
  // element-wise op runs by itself.
  if (ctx.fuseViews && tailOp == TTM_TAIL_NONE && !biasRef && !transposeA && !transposeB && batch == 1 &&
      utils::isBlockFormatDataType(b.handle->dtype) && layoutFromTensorRef(outRef) == Layout{StorageType::Device, TensorLayout::Tile, DataType::BFloat16}) {
    struct Follower { std::uint32_t index; fb::Table out; Tensor weight; std::int64_t n; int act; };
    std::vector<Follower> followers;
    const std::vector<std::uint32_t> outShape = shapeFromTensorRef(outRef);
    const bool midM = M > 64 && M <= 1024;
    for (std::uint32_t j = ctx.opIndex + 1; j < ctx.ops.size() && j <= ctx.opIndex + 10 && followers.size() < 3; ++j) {
      const OpType t = opType(j);
      fb::Table nop = ctx.ops[j].table(schema::Operation::f_type);
      if (t == OpType::ReshapeOp || t == OpType::PermuteOp || t == OpType::RotaryEmbeddingOp) continue;   // touch neither operand
      if (t == OpType::DeallocateOp) {
        const std::uint32_t freed = refId(nop.table(schema::DeallocateOp::f_in));
        if (freed == refId(aRef) || freed == refId(outRef)) break;
        continue;
      }
      if ((t != OpType::MatmulOp && t != OpType::LinearOp) || ctx.skip.count(j)) break;
      fb::Table a2, b2, out2;
      bool plainOperands;
      std::string act2;
      if (t == OpType::MatmulOp) {
        using M2 = schema::MatmulOp;
        a2 = nop.table(M2::f_a); b2 = nop.table(M2::f_b); out2 = nop.table(M2::f_out);
        plainOperands = !nop.scalar<std::uint8_t>(M2::f_transpose_a, 0) && !nop.scalar<std::uint8_t>(M2::f_transpose_b, 0);
        act2 = matmulActivation(nop, M2::f_matmul_program_config_type, M2::f_matmul_program_config, M2::f_activation);
      } else {
        using L2 = schema::LinearOp;
        a2 = nop.table(L2::f_a); b2 = nop.table(L2::f_b); out2 = nop.table(L2::f_out);
        plainOperands = !nop.scalar<std::uint8_t>(L2::f_transpose_a, 0) && !nop.scalar<std::uint8_t>(L2::f_transpose_b, 0) &&
                        !nop.table(L2::f_bias);
        act2 = matmulActivation(nop, L2::f_matmul_program_config_type, L2::f_matmul_program_config, L2::f_activation);
      }
      if (!a2 || !b2 || !out2 || refId(a2) != refId(aRef) || !plainOperands) break;
      auto wit = ctx.pool.find(refId(b2));
      if (wit == ctx.pool.end() || !isTensorAllocated(wit->second) || wit->second.handle->storage != StorageType::Device ||
          wit->second.handle->dtype != b.handle->dtype || wit->second.handle->shape.size() != 2 || b.handle->shape.size() != 2 ||
          wit->second.handle->shape[0] != b.handle->shape[0] || !(layoutFromTensorRef(out2) == layoutFromTensorRef(outRef)))
        break;
      const std::vector<std::uint32_t> shape2 = shapeFromTensorRef(out2);
      if (shape2.size() != outShape.size() || shape2.empty() || !std::equal(shape2.begin(), shape2.end() - 1, outShape.begin()) ||
          shape2.back() != wit->second.handle->shape[1])
        break;
      {   // its own element-wise tail, if it has one, is worth more than the shared launch (not at the middle token counts)
        std::uint32_t after = j + 1;
        while (after < ctx.ops.size() && opType(after) == OpType::DeallocateOp) ++after;
        if (after < ctx.ops.size() && opType(after) == OpType::EltwiseBinaryOp) {
          fb::Table bop = ctx.ops[after].table(schema::Operation::f_type);
          fb::Table l = bop.table(schema::EltwiseBinaryOp::f_lhs), r = bop.table(schema::EltwiseBinaryOp::f_rhs);
          if ((l && refId(l) == refId(out2)) || (r && refId(r) == refId(out2))) {
            // ... unless that op multiplies the follower's result with this one's (SiLU(gate) * up of a decode step's MLP):
            // both projections and the multiply are one launch whose workgroups stream the same columns of both matrices
            fb::Table bout = bop.table(schema::EltwiseBinaryOp::f_out);
            const std::uint32_t mine = refId(outRef), theirs = refId(out2);
            auto usesOf = [&](std::uint32_t id) { auto u = ctx.uses.find(id); return u == ctx.uses.end() ? 0u : u->second; };
            const Layout plain{StorageType::Device, TensorLayout::Tile, DataType::BFloat16};
            if ((decodeFusionEnabled() || M > 32) && followers.empty() && as_.size() >= 2 && bop.scalar<std::uint32_t>(schema::EltwiseBinaryOp::f_type, 0) == 1 && l && r && bout &&
                ((refId(l) == mine && refId(r) == theirs) || (refId(l) == theirs && refId(r) == mine)) && usesOf(mine) == 1 &&
                usesOf(theirs) == 1 && shape2 == outShape && shapeFromTensorRef(bout) == outShape && layoutFromTensorRef(bout) == plain &&
                wit->second.handle->shape[1] == b.handle->shape[1] && wit->second.handle->data.get() != b.handle->data.get() &&
                ttm_linear_glu_supported(ttmDtype(b.handle->dtype), M, N, K)) {
              Tensor gated = makeOut(ctx, bout, DataType::BFloat16, TensorLayout::Tile);
              TTM_CALL(ttm_linear_glu(a.handle->data.get(), b.handle->data.get(), wit->second.handle->data.get(), ttmDtype(b.handle->dtype),
                                      gated.handle->data.get(), M, N, K, activationCode(activation), activationCode(act2), ctx.stream()));
              ctx.put(bout, finish(ctx, gated, bout));
              ctx.skip.insert(j);
              ctx.skip.insert(after);
              debug::Stats::get().incrementStat("FusedLinearGlu");
              return;
            }
            if (!midM) break;
          }
        }
      }
      bool distinct = wit->second.handle->data.get() != b.handle->data.get();
      for (const Follower &f : followers) distinct = distinct && f.weight.handle->data.get() != wit->second.handle->data.get();
      if (!distinct) break;
      followers.push_back(Follower{j, out2, wit->second, static_cast<std::int64_t>(shape2.back()), activationCode(act2)});
    }
    if (followers.size() == 2 && M <= 32 && activationCode(activation) == TTM_ACT_NONE && followers[0].act == TTM_ACT_NONE &&
        followers[1].act == TTM_ACT_NONE &&
        tryQkvDecode(ctx, a, M, K, {QkvMember{ctx.opIndex, outRef, b}, QkvMember{followers[0].index, followers[0].out, followers[0].weight},
                                    QkvMember{followers[1].index, followers[1].out, followers[1].weight}}))
      return;
    if (!followers.empty()) {
      std::vector<const void *> ws{b.handle->data.get()};
      std::vector<void *> outs{out.handle->data.get()};
      std::vector<std::int64_t> ns{N};
      std::vector<int> acts{activationCode(activation)};
      std::vector<Tensor> outTensors;
      for (const Follower &f : followers) {
        outTensors.push_back(makeOut(ctx, f.out, DataType::BFloat16, TensorLayout::Tile));
        ws.push_back(f.weight.handle->data.get());
        outs.push_back(outTensors.back().handle->data.get());
        ns.push_back(f.n);
        acts.push_back(f.act);
      }
      TTM_CALL(ttm_linear_group(a.handle->data.get(), static_cast<int>(ws.size()), ws.data(), ttmDtype(b.handle->dtype), outs.data(), ns.data(),
                                acts.data(), M, K, ctx.stream()));
      ctx.put(outRef, out);
      for (size_t i = 0; i < followers.size(); ++i) {
        ctx.put(followers[i].out, outTensors[i]);
        ctx.skip.insert(followers[i].index);
      }
      debug::Stats::get().incrementStat("GroupedMatmul");
      debug::Stats::get().incrementStat("GroupedMatmulMembers", static_cast<std::int64_t>(ws.size()));
      return;
    }
  }
  // residual + projection followed at once by the RMSNorm of that sum (the end of a decode step's attention block): the
  // projection leaves partial sums and the RMSNorm kernel starts from them, one launch fewer and no pass over the sum
  if (decodeFusionEnabled() && tailOp == TTM_TAIL_ADD && !biasRef && !transposeB && batch == 1 && as_.size() == 2 && activationCode(activation) == TTM_ACT_NONE &&
      utils::isBlockFormatDataType(b.handle->dtype) && ttm_linear_add_rms_norm_supported(ttmDtype(b.handle->dtype), M, N, K)) {
    std::uint32_t j = nextIdx + 1;
    while (j < ctx.ops.size() && opType(j) == OpType::DeallocateOp) {
      const std::uint32_t freed = refId(ctx.ops[j].table(schema::Operation::f_type).table(schema::DeallocateOp::f_in));
      if (freed == refId(finalRef)) break;
      ++j;
    }
    if (j < ctx.ops.size() && opType(j) == OpType::RMSNormOp && !ctx.skip.count(j)) {
      using R = schema::RMSNormOp;
      fb::Table nop = ctx.ops[j].table(schema::Operation::f_type);
      fb::Table nin = nop.table(R::f_input), nout = nop.table(R::f_out), wr = nop.table(R::f_weight), br = nop.table(R::f_bias);
      const Layout plain{StorageType::Device, TensorLayout::Tile, DataType::BFloat16};
      auto vec = [&](const fb::Table &ref) -> const Tensor * {   // a [N] bf16 tile tensor that is live now
        auto it = ctx.pool.find(refId(ref));
        if (it == ctx.pool.end() || !isTensorAllocated(it->second) || !(getTensorLayout(it->second) == plain) ||
            static_cast<std::int64_t>(volume(it->second.handle->shape)) != N)
          return nullptr;
        return &it->second;
      };
      const Tensor *wT = wr ? vec(wr) : nullptr, *bT = br ? vec(br) : nullptr;
      if (nin && nout && refId(nin) == refId(finalRef) && layoutFromTensorRef(nout) == plain &&
          shapeFromTensorRef(nout) == shapeFromTensorRef(finalRef) && (!wr || wT) && (!br || bT)) {
        Tensor normOut = makeDeviceTensor(ctx.dev, out.handle->shape, DataType::BFloat16, TensorLayout::Tile);
        TTM_CALL(ttm_linear_add_rms_norm(a.handle->data.get(), b.handle->data.get(), ttmDtype(b.handle->dtype), tail.handle->data.get(),
                                         out.handle->data.get(), wT ? wT->handle->data.get() : nullptr, TTM_TILE,
                                         bT ? bT->handle->data.get() : nullptr, TTM_TILE, nop.scalar<float>(R::f_epsilon, 0.0f),
                                         normOut.handle->data.get(), M, N, K, ctx.stream()));
        ctx.put(finalRef, finish(ctx, out, finalRef));
        ctx.put(nout, finish(ctx, normOut, nout));
        ctx.skip.insert(j);
        debug::Stats::get().incrementStat("FusedLinearAddNorm");
        return;
      }
    }
  }
  // the last projection of a traced function writes straight into the trace's output slot
  std::uint32_t copyIndex = 0;
  if (Tensor slot = copyDestinationOf(ctx, tailOp == TTM_TAIL_NONE ? ctx.opIndex : nextIdx, finalRef, {&a, &b, &bias, &tail}, &copyIndex)) {
    out = slot;
    ctx.skip.insert(copyIndex);
    debug::Stats::get().incrementStat("FusedCopyIntoSlot");
  }
  TTM_CALL(ttm_linear_tail(a.handle->data.get(), TTM_BF16, b.handle->data.get(), ttmDtype(b.handle->dtype), transposeB ? 1 : 0, biasPtr,
                           TTM_BF16, biasLayout, out.handle->data.get(), TTM_BF16, batch, wbatch == 1 ? 1 : batch, M, N, K,
                           activationCode(activation), tailOp, tail ? tail.handle->data.get() : nullptr, ctx.stream()));
  ctx.put(finalRef, finish(ctx, out, finalRef));
}
void runMatmul(const fb::Table &op, ProgramContext &ctx) {
  runMatmulLike(ctx, op.table(schema::MatmulOp::f_a), op.table(schema::MatmulOp::f_b), fb::Table(), op.table(schema::MatmulOp::f_out),
                op.scalar<std::uint8_t>(schema::MatmulOp::f_transpose_a, 0) != 0,
                op.scalar<std::uint8_t>(schema::MatmulOp::f_transpose_b, 0) != 0,
                matmulActivation(op, schema::MatmulOp::f_matmul_program_config_type, schema::MatmulOp::f_matmul_program_config,
                                 schema::MatmulOp::f_activation));
}
void runLinear(const fb::Table &op, ProgramContext &ctx) {
  runMatmulLike(ctx, op.table(schema::LinearOp::f_a), op.table(schema::LinearOp::f_b), op.table(schema::LinearOp::f_bias),
                op.table(schema::LinearOp::f_out), op.scalar<std::uint8_t>(schema::LinearOp::f_transpose_a, 0) != 0,
                op.scalar<std::uint8_t>(schema::LinearOp::f_transpose_b, 0) != 0,
                matmulActivation(op, schema::LinearOp::f_matmul_program_config_type, schema::LinearOp::f_matmul_program_config,
                                 schema::LinearOp::f_activation));
}

// ---- eltwise (runtime/lib/ttnn/operations/eltwise/{unary,binary}/*.cpp)
DataType computeDtype(DataType dt) { return dt == DataType::Float32 ? DataType::Float32 : DataType::BFloat16; }

void runEltwiseUnary(const fb::Table &op, ProgramContext &ctx) {
  Tensor in0 = ctx.get(op.table(schema::EltwiseUnaryOp::f_in), "unary in");
  auto outRef = op.table(schema::EltwiseUnaryOp::f_out);
  Layout want = layoutFromTensorRef(outRef);
  DataType dt = computeDtype(want.dataType);
  Tensor in = as(ctx, in0, in0.handle->layout, dt);
  std::uint32_t type = op.scalar<std::uint32_t>(schema::EltwiseUnaryOp::f_type, 0);
  float param = 0.0f;
  if (auto prm = op.table(schema::EltwiseUnaryOp::f_params)) param = prm.scalar<float>(schema::EltwiseOpWithFloatParams::f_parameter, 0.0f);
  Tensor out = makeDeviceTensor(ctx.dev, in.handle->shape, dt, in.handle->layout);
  Dims3 d = dims3(in.handle->shape);
  TTM_CALL(ttm_eltwise_unary(static_cast<int>(type), in.handle->data.get(), out.handle->data.get(), ttmDtype(dt),
                             ttmLayout(in.handle->layout), d.batch, d.rows, d.cols, param, ctx.stream()));
  ctx.put(outRef, finish(ctx, out, outRef));
}

// the type element-wise ops with several operands compute in: fp32 as soon as an operand or the result is Float32 or a
// 32-bit integer (positions and token ids compared against each other must stay exact; bf16 holds 8 bits), bf16 otherwise
DataType computeDtypeOf(std::initializer_list<DataType> types) {
  for (DataType t : types)
    if (t == DataType::Float32 || t == DataType::Int32 || t == DataType::UInt32) return DataType::Float32;
  return DataType::BFloat16;
}

void binaryImpl(ProgramContext &ctx, const fb::Table &lhsRef, const fb::Table &rhsRef, const fb::Table &outRef, int code) {
  Tensor l0 = ctx.get(lhsRef, "binary lhs"), r0 = ctx.get(rhsRef, "binary rhs");
  Layout want = layoutFromTensorRef(outRef);
  DataType dt = computeDtypeOf({want.dataType, l0.handle->dtype, r0.handle->dtype});
  TensorLayout lay = want.storageType == StorageType::Device ? want.layout : onDevice(ctx, l0).handle->layout;
  Tensor l = as(ctx, l0, lay, dt), r = as(ctx, r0, lay, dt);
  std::vector<std::uint32_t> oshape = shapeFromTensorRef(outRef);
  size_t rank = std::max<size_t>(1, oshape.size());
  auto pad = [&](const std::vector<std::uint32_t> &s) {
    std::vector<std::int64_t> o(rank, 1);
    for (size_t i = 0; i < s.size(); ++i) o[rank - s.size() + i] = s[i];
    return o;
  };
  TTRT_ASSERT(l.handle->shape.size() <= rank && r.handle->shape.size() <= rank, "binary: operand rank exceeds the output rank");
  auto ls = pad(l.handle->shape), rs = pad(r.handle->shape), os = pad(oshape);
  Tensor out = makeDeviceTensor(ctx.dev, oshape, dt, lay);
  TTM_CALL(ttm_eltwise_binary(code, l.handle->data.get(), ls.data(), r.handle->data.get(), rs.data(),
                              out.handle->data.get(), os.data(), static_cast<int>(rank), ttmDtype(dt), ttmLayout(lay), ctx.stream()));
  ctx.put(outRef, finish(ctx, out, outRef));
}
// runtime/lib/ttnn/operations/eltwise/unary/unary_composite.cpp:104-135: cbrt, log1p, clamp with scalar bounds
void runEltwiseUnaryComposite(const fb::Table &op, ProgramContext &ctx) {
  using S = schema::EltwiseUnaryCompositeOp;
  const std::uint32_t type = op.scalar<std::uint32_t>(S::f_type, 0);
  TTRT_ASSERT(type != static_cast<std::uint32_t>(schema::EltwiseUnaryCompositeOpType::ClampTensor), "clamp with tensor bounds is not supported");
  Tensor in0 = ctx.get(op.table(S::f_in), "unary composite in");
  auto outRef = op.table(S::f_out);
  const DataType dt = computeDtypeOf({layoutFromTensorRef(outRef).dataType, in0.handle->dtype});
  Tensor in = as(ctx, in0, in0.handle->layout, dt);
  Tensor out = makeDeviceTensor(ctx.dev, in.handle->shape, dt, in.handle->layout);
  const Dims3 d = dims3(in.handle->shape);
  if (type == static_cast<std::uint32_t>(schema::EltwiseUnaryCompositeOpType::ClampScalar)) {
    auto prm = op.table(S::f_params);
    TTRT_ASSERT(static_cast<bool>(prm), "clamp: bounds missing");
    auto number = [&](int typeSlot, int slot) {
      const auto kind = static_cast<schema::NumberType>(prm.scalar<std::uint8_t>(typeSlot, 0));
      auto t = prm.table(slot);
      TTRT_ASSERT(static_cast<bool>(t), "clamp: bound missing");
      return kind == schema::NumberType::I32 ? static_cast<float>(t.scalar<std::int32_t>(schema::IntegralType::f_value, 0))
                                             : t.scalar<float>(schema::FloatingPointType::f_value, 0.0f);
    };
    using P = schema::ClampScalarOpParams;
    TTM_CALL(ttm_clamp(in.handle->data.get(), out.handle->data.get(), ttmDtype(dt), ttmLayout(in.handle->layout), d.batch, d.rows, d.cols,
                       number(P::f_min_type, P::f_min), number(P::f_max_type, P::f_max), ctx.stream()));
  } else {
    TTM_CALL(ttm_eltwise_unary(100 + static_cast<int>(type), in.handle->data.get(), out.handle->data.get(), ttmDtype(dt),
                               ttmLayout(in.handle->layout), d.batch, d.rows, d.cols, 0.0f, ctx.stream()));
  }
  ctx.put(outRef, finish(ctx, out, outRef));
}
void runEltwiseBinary(const fb::Table &op, ProgramContext &ctx) {
  using S = schema::EltwiseBinaryOp;
  binaryImpl(ctx, op.table(S::f_lhs), op.table(S::f_rhs), op.table(S::f_out), static_cast<int>(op.scalar<std::uint32_t>(S::f_type, 0)));
}
// runtime/lib/ttnn/operations/eltwise/binary/binary_composite.cpp: maximum, minimum, remainder, pow, atan2 (the bitwise and
// shift members work on integers and have no kernel here)
void runEltwiseBinaryComposite(const fb::Table &op, ProgramContext &ctx) {
  using S = schema::EltwiseBinaryCompositeOp;
  const std::uint32_t type = op.scalar<std::uint32_t>(S::f_type, 0);
  TTRT_ASSERT(type <= 4, "binary composite: bitwise and shift ops are not supported");
  binaryImpl(ctx, op.table(S::f_lhs), op.table(S::f_rhs), op.table(S::f_out), 100 + static_cast<int>(type));
}
// runtime/lib/ttnn/operations/eltwise/ternary/where.cpp:14-33
void runWhere(const fb::Table &op, ProgramContext &ctx) {
  using S = schema::EltwiseTernaryWhereOp;
  Tensor c0 = ctx.get(op.table(S::f_first), "where condition"), a0 = ctx.get(op.table(S::f_second), "where true value"),
         b0 = ctx.get(op.table(S::f_third), "where false value");
  auto outRef = op.table(S::f_out);
  Layout want = layoutFromTensorRef(outRef);
  const DataType dt = computeDtypeOf({want.dataType, c0.handle->dtype, a0.handle->dtype, b0.handle->dtype});
  const TensorLayout lay = want.storageType == StorageType::Device ? want.layout : onDevice(ctx, a0).handle->layout;
  Tensor c = as(ctx, c0, lay, dt), a = as(ctx, a0, lay, dt), b = as(ctx, b0, lay, dt);
  const std::vector<std::uint32_t> oshape = shapeFromTensorRef(outRef);
  const size_t rank = std::max<size_t>(1, oshape.size());
  TTRT_ASSERT(rank <= 4 && c.handle->shape.size() <= rank && a.handle->shape.size() <= rank && b.handle->shape.size() <= rank,
              "where: ranks above 4, or an operand of higher rank than the result, are not supported");
  auto pad = [&](const std::vector<std::uint32_t> &s) {
    std::vector<std::int64_t> o(rank, 1);
    for (size_t i = 0; i < s.size(); ++i) o[rank - s.size() + i] = s[i];
    return o;
  };
  auto cs = pad(c.handle->shape), as_ = pad(a.handle->shape), bs = pad(b.handle->shape), os = pad(oshape);
  Tensor out = makeDeviceTensor(ctx.dev, oshape, dt, lay);
  TTM_CALL(ttm_where(c.handle->data.get(), cs.data(), a.handle->data.get(), as_.data(), b.handle->data.get(), bs.data(),
                     out.handle->data.get(), os.data(), static_cast<int>(rank), ttmDtype(dt), ttmLayout(lay), ctx.stream()));
  ctx.put(outRef, finish(ctx, out, outRef));
}

// ---- normalization / reduction (runtime/lib/ttnn/operations/normalization/*.cpp, reduction/reduction.cpp)
void runRmsNorm(const fb::Table &op, ProgramContext &ctx) {
  auto outRef = op.table(schema::RMSNormOp::f_out);
  DataType dt = computeDtype(layoutFromTensorRef(outRef).dataType);
  Tensor x = as(ctx, ctx.get(op.table(schema::RMSNormOp::f_input), "rms_norm input"), TensorLayout::Tile, dt);
  Tensor w, b;
  Dims3 d = dims3(x.handle->shape);
  if (auto wr = op.table(schema::RMSNormOp::f_weight)) {
    w = as(ctx, ctx.get(wr, "rms_norm weight"), TensorLayout::Tile, dt);
    TTRT_ASSERT(volume(w.handle->shape) == d.cols, "rms_norm: weight must have as many elements as the last dim");
  }
  if (auto br = op.table(schema::RMSNormOp::f_bias)) {
    b = as(ctx, ctx.get(br, "rms_norm bias"), TensorLayout::Tile, dt);
    TTRT_ASSERT(volume(b.handle->shape) == d.cols, "rms_norm: bias must have as many elements as the last dim");
  }
  float eps = op.scalar<float>(schema::RMSNormOp::f_epsilon, 0.0f);
  Tensor out = makeDeviceTensor(ctx.dev, x.handle->shape, dt, TensorLayout::Tile);
  TTM_CALL(ttm_rms_norm(x.handle->data.get(), w ? w.handle->data.get() : nullptr, TTM_TILE, b ? b.handle->data.get() : nullptr, TTM_TILE,
                        out.handle->data.get(), ttmDtype(dt), d.batch, d.rows, d.cols, eps, ctx.stream()));
  ctx.put(outRef, finish(ctx, out, outRef));
}

// move dimension `dim` to the end (or back) with one strided copy
Tensor moveDimLast(ProgramContext &ctx, const Tensor &t, int dim, bool inverse, const std::vector<std::uint32_t> &origShape) {
  const int rank = static_cast<int>(origShape.size());
  std::vector<int> perm;  // perm[i] = source dim of output dim i for the forward move
  for (int i = 0; i < rank; ++i) if (i != dim) perm.push_back(i);
  perm.push_back(dim);
  std::vector<std::uint32_t> moved(rank);
  for (int i = 0; i < rank; ++i) moved[i] = origShape[perm[i]];
  const std::vector<std::uint32_t> &srcShape = inverse ? moved : origShape, &dstShape = inverse ? origShape : moved;
  Tensor out = makeDeviceTensor(ctx.dev, dstShape, t.handle->dtype, t.handle->layout);
  zeroIfPadded(ctx, out);
  auto ss = rowMajorStrides(srcShape), ds = rowMajorStrides(dstShape);
  std::vector<std::int64_t> extent(rank), sst(rank), dst(rank);
  for (int i = 0; i < rank; ++i) {  // iterate in the order of `moved`
    extent[i] = moved[i];
    sst[i] = inverse ? ss[i] : ss[perm[i]];
    dst[i] = inverse ? ds[perm[i]] : ds[i];
  }
  copyView(ctx, t, out, extent, sst, 0, dst, 0);
  return out;
}

void runSoftmax(const fb::Table &op, ProgramContext &ctx) {
  auto outRef = op.table(schema::SoftmaxOp::f_out);
  DataType dt = computeDtype(layoutFromTensorRef(outRef).dataType);
  Tensor x = as(ctx, ctx.get(op.table(schema::SoftmaxOp::f_in), "softmax in"), TensorLayout::Tile, dt);
  const int rank = static_cast<int>(x.handle->shape.size());
  int dim = op.scalar<std::int32_t>(schema::SoftmaxOp::f_dimension, 0);
  if (dim < 0) dim += rank;
  TTRT_ASSERT(dim >= 0 && dim < rank, "softmax: dimension out of range");
  const std::vector<std::uint32_t> orig = x.handle->shape;
  if (dim != rank - 1) x = moveDimLast(ctx, x, dim, false, orig);
  Dims3 d = dims3(x.handle->shape);
  Tensor out = makeDeviceTensor(ctx.dev, x.handle->shape, dt, TensorLayout::Tile);
  TTM_CALL(ttm_softmax_lastdim(x.handle->data.get(), out.handle->data.get(), ttmDtype(dt), d.batch, d.rows, d.cols, ctx.stream()));
  if (dim != rank - 1) out = moveDimLast(ctx, out, dim, true, orig);
  ctx.put(outRef, finish(ctx, out, outRef));
}

void runReduction(const fb::Table &op, ProgramContext &ctx) {
  auto outRef = op.table(schema::ReductionOp::f_out);
  DataType dt = computeDtype(layoutFromTensorRef(outRef).dataType);
  Tensor x = as(ctx, ctx.get(op.table(schema::ReductionOp::f_in), "reduction in"), TensorLayout::Tile, dt);
  const int rank = static_cast<int>(x.handle->shape.size());
  auto dims = op.scalars<std::int32_t>(schema::ReductionOp::f_dim_arg);
  std::uint32_t type = op.scalar<std::uint32_t>(schema::ReductionOp::f_type, 0);
  std::vector<int> rd;
  for (std::uint32_t i = 0; i < dims.size(); ++i) rd.push_back(dims[i] < 0 ? dims[i] + rank : dims[i]);
  if (rd.empty()) for (int i = 0; i < rank; ++i) rd.push_back(i);
  std::sort(rd.begin(), rd.end(), std::greater<int>());
  // reduce one dim at a time, innermost first; the reduced dim is kept as size 1.  A mean over several
  // dims is a mean of means (equal group sizes), so every op applies dim by dim.
  for (int dim : rd) {
    TTRT_ASSERT(dim >= 0 && dim < rank, "reduction: dimension out of range");
    const std::vector<std::uint32_t> orig = x.handle->shape;
    Tensor cur = dim != rank - 1 ? moveDimLast(ctx, x, dim, false, orig) : x;
    Dims3 d = dims3(cur.handle->shape);
    std::vector<std::uint32_t> rshape = cur.handle->shape;
    rshape.back() = 1;
    Tensor red = makeDeviceTensor(ctx.dev, rshape, dt, TensorLayout::Tile);
    TTM_CALL(ttm_reduce_lastdim(static_cast<int>(type), cur.handle->data.get(), red.handle->data.get(), ttmDtype(dt), d.batch, d.rows,
                                d.cols, ctx.stream()));
    if (dim != rank - 1) {
      std::vector<std::uint32_t> back = orig;
      back[dim] = 1;
      red = moveDimLast(ctx, red, dim, true, back);
    }
    x = red;
  }
  // keep_dim = false only changes the logical shape; relayout through a strided copy
  std::vector<std::uint32_t> oshape = shapeFromTensorRef(outRef);
  if (oshape != x.handle->shape) {
    TTRT_ASSERT(volume(oshape) == volume(x.handle->shape), "reduction: output shape does not match");
    Tensor out = makeDeviceTensor(ctx.dev, oshape, dt, TensorLayout::Tile);
    zeroIfPadded(ctx, out);
    std::vector<std::int64_t> e{volume(oshape)}, one{1};
    copyView(ctx, x, out, e, one, 0, one, 0);
    x = out;
  }
  ctx.put(outRef, finish(ctx, x, outRef));
}

// ---- attention (runtime/lib/ttnn/operations/transformer/scaled_dot_product_attention.cpp:14-55)
void runSdpa(const fb::Table &op, ProgramContext &ctx) {
  using S = schema::ScaledDotProductAttentionOp;
  // an operand may be a head split that was never materialised (ctx.headViews): then the tensor at hand is the
  // [B, S, H * D] source and the kernel is told so; shapes come from the program's tensor refs
  int inner = 0;
  auto operand = [&](const fb::Table &ref, int bit, const char *what) {
    auto hv = ctx.headViews.find(refId(ref));
    if (hv != ctx.headViews.end()) {
      Tensor t = hv->second;
      ctx.headViews.erase(hv);
      inner |= bit;
      return t;
    }
    return as(ctx, ctx.get(ref, what), TensorLayout::Tile, DataType::BFloat16);
  };
  Tensor q = operand(op.table(S::f_query), 1, "sdpa query");
  Tensor k = operand(op.table(S::f_key), 2, "sdpa key");
  Tensor v = operand(op.table(S::f_value), 4, "sdpa value");
  const std::vector<std::uint32_t> qs = (inner & 1) ? shapeFromTensorRef(op.table(S::f_query)) : q.handle->shape;
  const std::vector<std::uint32_t> ks = (inner & 2) ? shapeFromTensorRef(op.table(S::f_key)) : k.handle->shape;
  const std::vector<std::uint32_t> vs = (inner & 4) ? shapeFromTensorRef(op.table(S::f_value)) : v.handle->shape;
  TTRT_ASSERT(qs.size() == 4 && ks.size() == 4 && vs.size() == 4, "sdpa: q, k, v must be rank 4");
  const std::int64_t window = op.has(S::f_sliding_window_size) ? static_cast<std::int64_t>(op.scalar<std::uint32_t>(S::f_sliding_window_size, 0)) : std::int64_t(-1);
  Tensor sink;
  if (auto sr = op.table(S::f_attention_sink)) {
    sink = as(ctx, ctx.get(sr, "sdpa attention sink"), TensorLayout::Tile, DataType::BFloat16);
    const auto &ss = sink.handle->shape;
    TTRT_ASSERT(ss.size() == 4 && ss[0] == 1 && ss[1] == qs[1] && ss[2] == 1 && ss[3] == 1, "sdpa: attention sink must be [1, Hq, 1, 1]");
  }
  TTRT_ASSERT(ks == vs && qs[0] == ks[0] && qs[3] == ks[3], "sdpa: q/k/v shapes do not agree");
  Tensor mask;
  int maskHeads = 1;
  std::int64_t maskBatch = 1;
  if (auto mr = op.table(S::f_attention_mask)) {
    mask = as(ctx, ctx.get(mr, "sdpa mask"), TensorLayout::Tile, DataType::BFloat16);
    const auto &ms = mask.handle->shape;
    TTRT_ASSERT(ms.size() == 4 && (ms[0] == 1 || ms[0] == qs[0]) && ms[2] == qs[2] && ms[3] == ks[2] && (ms[1] == 1 || ms[1] == qs[1]),
                "sdpa: mask must be [1|B, 1|Hq, Sq, Sk]");
    maskHeads = static_cast<int>(ms[1]);
    maskBatch = ms[0];
  }
  bool causal = op.scalar<std::uint8_t>(S::f_is_causal, 0) != 0;
  TTRT_ASSERT(!(causal && mask), "sdpa: is_causal and an explicit mask are mutually exclusive");
  float scale = op.has(S::f_scale) ? op.scalar<float>(S::f_scale, 0.0f) : 0.0f;
  auto outRef = op.table(S::f_out);
  // The head merge behind the attention - permute (0, 2, 1, 3) and reshape to [.., Sq, Hq * D], each the only consumer of
  // what precedes it, deallocations of other tensors between them allowed - is folded in: the kernel writes that layout.
  fb::Table mergedRef;
  std::vector<std::uint32_t> skipped;
  if (ctx.fuseViews && qs[3] % 32 == 0) {
    auto opType = [&](std::uint32_t i) { return static_cast<OpType>(ctx.ops[i].scalar<std::uint8_t>(schema::Operation::f_type_type, 0)); };
    auto soleUse = [&](const fb::Table &r) { auto u = ctx.uses.find(refId(r)); return u != ctx.uses.end() && u->second == 1; };
    auto nextReal = [&](std::uint32_t i, std::uint32_t avoid) {   // first op after i that is not a deallocation of another tensor
      for (++i; i < ctx.ops.size() && opType(i) == OpType::DeallocateOp; ++i)
        if (refId(ctx.ops[i].table(schema::Operation::f_type).table(schema::DeallocateOp::f_in)) == avoid) return static_cast<std::uint32_t>(ctx.ops.size());
      return i;
    };
    const Layout plain{StorageType::Device, TensorLayout::Tile, DataType::BFloat16};
    const std::uint32_t pi = nextReal(ctx.opIndex, refId(outRef));
    if (pi < ctx.ops.size() && opType(pi) == OpType::PermuteOp && soleUse(outRef) && layoutFromTensorRef(outRef) == plain) {
      fb::Table pop = ctx.ops[pi].table(schema::Operation::f_type);
      fb::Table pin = pop.table(schema::PermuteOp::f_in), pout = pop.table(schema::PermuteOp::f_out);
      auto pv = pop.scalars<std::int64_t>(schema::PermuteOp::f_permutation);
      const bool swaps = pv.size() == 4 && pv[0] == 0 && pv[1] == 2 && pv[2] == 1 && pv[3] == 3;
      if (pin && pout && refId(pin) == refId(outRef) && swaps && soleUse(pout) && layoutFromTensorRef(pout) == plain) {
        const std::uint32_t ri = nextReal(pi, refId(pout));
        if (ri < ctx.ops.size() && opType(ri) == OpType::ReshapeOp) {
          fb::Table rop = ctx.ops[ri].table(schema::Operation::f_type);
          fb::Table rin = rop.table(schema::ReshapeOp::f_in), rout = rop.table(schema::ReshapeOp::f_out);
          if (rin && rout && refId(rin) == refId(pout) && layoutFromTensorRef(rout) == plain) {
            const Dims3 fd = dims3(shapeFromTensorRef(rout));
            if (fd.batch == qs[0] && fd.rows == qs[2] && fd.cols == static_cast<std::int64_t>(qs[1]) * qs[3]) {
              mergedRef = rout;
              skipped = {pi, ri};
            }
          }
        }
      }
    }
  }
  if (mergedRef) inner |= 8;
  Tensor out = makeDeviceTensor(ctx.dev, mergedRef ? shapeFromTensorRef(mergedRef) : qs, DataType::BFloat16, TensorLayout::Tile);
  if (inner) debug::Stats::get().incrementStat("SdpaHeadsInner");
  TTM_CALL(ttm_sdpa_windowed(q.handle->data.get(), k.handle->data.get(), v.handle->data.get(), mask ? mask.handle->data.get() : nullptr,
                             maskHeads, maskBatch, out.handle->data.get(), TTM_BF16, qs[0], qs[1], ks[1], qs[2], ks[2], qs[3], causal ? 1 : 0, scale,
                             inner, window, sink ? sink.handle->data.get() : nullptr, ctx.stream()));
  if (mergedRef) {
    ctx.put(mergedRef, out);
    for (std::uint32_t i : skipped) ctx.skip.insert(i);
    return;
  }
  ctx.put(outRef, finish(ctx, out, outRef));
}

// ---- decode path (runtime/lib/ttnn/operations/transformer/rotary_embedding.cpp, scaled_dot_product_attention_decode.cpp,
// paged_scaled_dot_product_attention_decode.cpp; operations/kv_cache/{update_cache,fill_cache}.cpp)
int floatCode(DataType dt, const char *what) {
  if (dt == DataType::BFloat16) return TTM_BF16;
  if (dt == DataType::Float32) return TTM_F32;
  fatal(std::string(what) + ": tensors must be BFloat16 or Float32");
}
// positions (update index, current positions, page table) as 32-bit integers in device memory, row-major
Tensor devicePositions(ProgramContext &ctx, const Tensor &t, const char *what) {
  TTRT_ASSERT(t.handle->dtype == DataType::Int32 || t.handle->dtype == DataType::UInt32,
              std::string(what) + " must be a 32-bit integer tensor");
  return as(ctx, t, TensorLayout::RowMajor, t.handle->dtype);
}

void runRotaryEmbedding(const fb::Table &op, ProgramContext &ctx) {
  using S = schema::RotaryEmbeddingOp;
  if (auto d = ctx.deferred.find(refId(op.table(S::f_input))); d != ctx.deferred.end()) {
    // the input is the head split [users, heads * head_dim] -> [1, users, heads, head_dim] of a projection, not
    // materialised (runReshape checked the shapes and that this is decode mode): the kernel splits on the way in
    const ProgramContext::DeferredView v = d->second;
    ctx.deferred.erase(d);
    const DataType dt = v.source.handle->dtype;
    Tensor cosc = as(ctx, ctx.get(op.table(S::f_cos_cache), "rotary_embedding cos"), TensorLayout::Tile, dt);
    Tensor sinc = as(ctx, ctx.get(op.table(S::f_sin_cache), "rotary_embedding sin"), TensorLayout::Tile, dt);
    const auto &cs = cosc.handle->shape;
    TTRT_ASSERT(cs.size() == 4 && sinc.handle->shape == cs && cs[0] == 1 && cs[1] == 1 && cs[3] == v.shape[3],
                "rotary_embedding: cos / sin caches must be [1, 1, positions, head_dim]");
    auto outRef = op.table(S::f_out);
    Tensor out = makeDeviceTensor(ctx.dev, v.shape, dt, TensorLayout::Tile);
    debug::Stats::get().incrementStat("FusedHeadSplit");
    TTM_CALL(ttm_rotary_embedding_split_heads(v.source.handle->data.get(), cosc.handle->data.get(), sinc.handle->data.get(),
                                              out.handle->data.get(), floatCode(dt, "rotary_embedding"), v.shape[1], v.shape[2], v.shape[3],
                                              cs[2], op.scalar<std::uint32_t>(S::f_token_index, 0), ctx.stream()));
    ctx.put(outRef, finish(ctx, out, outRef));
    return;
  }
  Tensor &in = ctx.get(op.table(S::f_input), "rotary_embedding input");
  const DataType dt = in.handle->dtype == DataType::Float32 ? DataType::Float32 : DataType::BFloat16;
  Tensor x = as(ctx, in, TensorLayout::Tile, dt);
  Tensor cosc = as(ctx, ctx.get(op.table(S::f_cos_cache), "rotary_embedding cos"), TensorLayout::Tile, dt);
  Tensor sinc = as(ctx, ctx.get(op.table(S::f_sin_cache), "rotary_embedding sin"), TensorLayout::Tile, dt);
  const auto &xs = x.handle->shape, &cs = cosc.handle->shape;
  TTRT_ASSERT(xs.size() == 4 && cs.size() == 4 && sinc.handle->shape == cs, "rotary_embedding: all tensors must be 4D, cos and sin of one shape");
  TTRT_ASSERT(cs[0] == 1 && cs[1] == 1 && cs[3] == xs[3], "rotary_embedding: cos / sin caches must be [1, 1, positions, head_dim]");
  // (both arms as int64: with an unsigned arm the -1 would arrive as 4294967295)
  const std::int64_t token = op.has(S::f_token_index) ? static_cast<std::int64_t>(op.scalar<std::uint32_t>(S::f_token_index, 0)) : std::int64_t{-1};
  auto outRef = op.table(S::f_out);
  Tensor out = makeDeviceTensor(ctx.dev, xs, dt, TensorLayout::Tile);
  TTM_CALL(ttm_rotary_embedding(x.handle->data.get(), cosc.handle->data.get(), sinc.handle->data.get(), out.handle->data.get(),
                                floatCode(dt, "rotary_embedding"), static_cast<std::int64_t>(xs[0]) * xs[1], xs[2], xs[3], cs[2], token,
                                ctx.stream()));
  ctx.put(outRef, finish(ctx, out, outRef));
}

// ::ttnn::experimental::rotary_embedding_llama (runtime/lib/ttnn/operations/transformer/rotary_embedding_llama.cpp:11-34):
// out = x * cos + (x T) * sin with the 32 x 32 transformation matrix applied per 32-column tile.  Prefill: x
// [1, heads, seq, head_dim], cos / sin [1, 1, seq, head_dim]; decode: x [1, users, heads, head_dim], cos / sin
// [1, users, 1 | heads, head_dim] (lib/Dialect/TTNN/IR/TTNNOps.cpp:6293-6380 fixes dtype, layout and the matrix shape).
void runRotaryEmbeddingLlama(const fb::Table &op, ProgramContext &ctx) {
  using S = schema::RotaryEmbeddingLlamaOp;
  Tensor x = as(ctx, ctx.get(op.table(S::f_input), "rotary_embedding_llama input"), TensorLayout::Tile, DataType::BFloat16);
  Tensor cosc = as(ctx, ctx.get(op.table(S::f_cos_cache), "rotary_embedding_llama cos"), TensorLayout::Tile, DataType::BFloat16);
  Tensor sinc = as(ctx, ctx.get(op.table(S::f_sin_cache), "rotary_embedding_llama sin"), TensorLayout::Tile, DataType::BFloat16);
  Tensor tm = as(ctx, ctx.get(op.table(S::f_trans_mat), "rotary_embedding_llama trans_mat"), TensorLayout::Tile, DataType::BFloat16);
  const auto &xs = x.handle->shape, &cs = cosc.handle->shape, &ts = tm.handle->shape;
  TTRT_ASSERT(xs.size() == 4 && cs.size() == 4, "rotary_embedding_llama: input and caches must be 4D");
  TTRT_ASSERT(sinc.handle->shape == cs, "rotary_embedding_llama: cos and sin tensors must have the same shape.");
  TTRT_ASSERT(ts.size() == 4 && ts[0] == 1 && ts[1] == 1 && ts[2] == 32 && ts[3] == 32,
              "rotary_embedding_llama: transformation matrix must have shape (1,1,32,32)");
  TTRT_ASSERT(xs[3] <= 256 && cs[3] == xs[3], "rotary_embedding_llama: head dimension must be <= 256 and match the caches'");
  TTRT_ASSERT(cs[0] == 1 && (cs[1] == 1 || cs[1] == xs[1]) && (cs[2] == xs[2] || cs[2] == 1),
              "rotary_embedding_llama: cos / sin must be [1, 1 | dim1, dim2 | 1, head_dim]");
  auto outRef = op.table(S::f_out);
  Tensor out = makeDeviceTensor(ctx.dev, xs, DataType::BFloat16, TensorLayout::Tile);
  TTM_CALL(ttm_rotary_embedding_llama(x.handle->data.get(), cosc.handle->data.get(), sinc.handle->data.get(), tm.handle->data.get(),
                                      out.handle->data.get(), TTM_BF16, static_cast<std::int64_t>(xs[0]) * xs[1], xs[2], xs[3], cs[1], cs[2],
                                      ctx.stream()));
  ctx.put(outRef, finish(ctx, out, outRef));
}

// ::ttnn::transformer::chunked_scaled_dot_product_attention (runtime/lib/ttnn/operations/transformer/
// chunked_scaled_dot_product_attention.cpp:11-58; golden tools/golden/mapping.py:8847-8913): a prefill chunk
// [users, heads, chunk_len, head_dim] attends causally over the prefix held in a paged cache; query row j stands at position
// chunk_start_idx + j.  The pages are gathered, the mask is written and the attention kernel runs, all from device-resident
// operands: like the reference's "flexible" overload the op keeps no host state and can be recorded into a trace.
void runChunkedSdpa(const fb::Table &op, ProgramContext &ctx) {
  using S = schema::ChunkedScaledDotProductAttentionOp;
  Tensor q = as(ctx, ctx.get(op.table(S::f_query), "chunked sdpa query"), TensorLayout::Tile, DataType::BFloat16);
  Tensor k = as(ctx, ctx.get(op.table(S::f_key), "chunked sdpa key"), TensorLayout::Tile, DataType::BFloat16);
  Tensor v = as(ctx, ctx.get(op.table(S::f_value), "chunked sdpa value"), TensorLayout::Tile, DataType::BFloat16);
  Tensor table = devicePositions(ctx, ctx.get(op.table(S::f_page_table), "chunked sdpa page table"), "chunked sdpa: page_table");
  Tensor start = devicePositions(ctx, ctx.get(op.table(S::f_chunk_start_idx), "chunked sdpa chunk start"), "chunked sdpa: chunk_start_idx");
  const auto &qs = q.handle->shape, &ks = k.handle->shape, &ts = table.handle->shape;
  TTRT_ASSERT(qs.size() == 4, "Query must be a 4D tensor.");
  TTRT_ASSERT(ks.size() == 4 && v.handle->shape == ks, "Key and value must be 4D tensors of the same shape.");
  TTRT_ASSERT(ts.size() == 2 && ts[0] == qs[0], "Page table number of users must match query number of users.");
  TTRT_ASSERT(volume(start.handle->shape) == 1, "Chunk start index must have shape [1]");
  TTRT_ASSERT(qs[3] == ks[3], "Query head size must match key/value head size.");
  TTRT_ASSERT(ks[1] != 0 && qs[1] % ks[1] == 0, "Query num heads must be divisible by key/value num heads.");
  TTRT_ASSERT(ks[2] % 32 == 0, "Key/value block size must be divisible by 32.");
  const std::int64_t B = qs[0], H = qs[1], Sq = qs[2], D = qs[3], Hkv = ks[1], block = ks[2], pages = ts[1], Sk = pages * block;
  Tensor kc = makeDeviceTensor(ctx.dev, {static_cast<std::uint32_t>(B), static_cast<std::uint32_t>(Hkv), static_cast<std::uint32_t>(Sk),
                                         static_cast<std::uint32_t>(D)}, DataType::BFloat16, TensorLayout::Tile);
  Tensor vc = makeDeviceTensor(ctx.dev, kc.handle->shape, DataType::BFloat16, TensorLayout::Tile);
  const auto *tp = static_cast<const std::int32_t *>(table.handle->data.get());
  TTM_CALL(ttm_paged_gather(k.handle->data.get(), tp, kc.handle->data.get(), TTM_BF16, ks[0], Hkv, block, D, B, pages, ctx.stream()));
  TTM_CALL(ttm_paged_gather(v.handle->data.get(), tp, vc.handle->data.get(), TTM_BF16, ks[0], Hkv, block, D, B, pages, ctx.stream()));
  Tensor mask = makeDeviceTensor(ctx.dev, {1, 1, static_cast<std::uint32_t>(Sq), static_cast<std::uint32_t>(Sk)}, DataType::BFloat16,
                                 TensorLayout::Tile);
  TTM_CALL(ttm_chunk_causal_mask(mask.handle->data.get(), static_cast<const std::int32_t *>(start.handle->data.get()), Sq, Sk, ctx.stream()));
  auto outRef = op.table(S::f_out);
  Tensor out = makeDeviceTensor(ctx.dev, qs, DataType::BFloat16, TensorLayout::Tile);
  TTM_CALL(ttm_sdpa_windowed(q.handle->data.get(), kc.handle->data.get(), vc.handle->data.get(), mask.handle->data.get(), 1, 1,
                             out.handle->data.get(), TTM_BF16, B, H, Hkv, Sq, Sk, D, 0, op.has(S::f_scale) ? op.scalar<float>(S::f_scale, 0.0f) : 0.0f,
                             0, -1, nullptr, ctx.stream()));
  ctx.put(outRef, finish(ctx, out, outRef));
}

// the cache operand of the in-place cache ops: it must already be what the kernels write into
Tensor &cacheOperand(ProgramContext &ctx, const fb::Table &ref, const char *what) {
  Tensor &cache = ctx.get(ref, what);
  TTRT_ASSERT(cache.handle->storage == StorageType::Device && cache.handle->layout == TensorLayout::Tile && cache.handle->shape.size() == 4,
              std::string(what) + " must be a 4D device tensor in tile layout");
  return cache;
}
void runUpdateCache(const fb::Table &op, ProgramContext &ctx) {
  using S = schema::UpdateCacheOp;
  Tensor &cache = cacheOperand(ctx, op.table(S::f_cache), "update_cache cache");
  const auto &cs = cache.handle->shape;
  if (auto d = ctx.deferred.find(refId(op.table(S::f_input))); d != ctx.deferred.end()) {
    // the input is a permuted / reshaped view that was not materialised: one strided copy from its source into the cache
    // row of the position.  cache[batch_offset + b, h, *index, :] = view[0, h, b, :]
    const ProgramContext::DeferredView v = d->second;
    ctx.deferred.erase(d);
    const auto &is = v.shape;
    TTRT_ASSERT(is.size() == 4 && is[0] == 1 && is[1] == cs[1] && is[3] == cs[3],
                "update_cache: input must be [1, heads, users, head_dim] matching the cache");
    const std::int64_t users = cs[0], heads = cs[1], maxSeq = cs[2], hd = cs[3];
    const std::int64_t offset = op.scalar<std::uint32_t>(S::f_batch_offset, 0);
    TTRT_ASSERT(offset + is[2] <= users, "update_cache: batch_offset + input users exceeds the cache");
    TTRT_ASSERT(v.source.handle->dtype == cache.handle->dtype, "update_cache: fused input has another element type than the cache");
    Tensor index = devicePositions(ctx, ctx.get(op.table(S::f_update_index), "update_cache index"), "update_cache: update_index");
    const std::int64_t extent[3] = {heads, static_cast<std::int64_t>(is[2]), hd};
    const std::int64_t sst[3] = {v.strides[1], v.strides[2], v.strides[3]};
    const std::int64_t dst[3] = {maxSeq * hd, heads * maxSeq * hd, 1};
    Dims3 sd = dims3(v.source.handle->shape), dd = dims3(cs);
    debug::Stats::get().incrementStat("CopyViewLaunch");
    debug::Stats::get().incrementStat("FusedCacheUpdate");
    TTM_CALL(ttm_copy_view_at(v.source.handle->data.get(), sd.rows, sd.cols, ttmLayout(v.source.handle->layout), cache.handle->data.get(),
                              dd.rows, dd.cols, TTM_TILE, static_cast<int>(utils::dataTypeElementSize(cache.handle->dtype)), 3, extent,
                              sst, 0, dst, offset * heads * maxSeq * hd, static_cast<const std::int32_t *>(index.handle->data.get()), hd,
                              maxSeq, ctx.stream()));
    cache.handle->version = nextTensorVersion();
    return;
  }
  Tensor in = as(ctx, ctx.get(op.table(S::f_input), "update_cache input"), TensorLayout::Tile, cache.handle->dtype);
  const auto &is = in.handle->shape;
  TTRT_ASSERT(is.size() == 4 && is[0] == 1 && is[1] == cs[1] && is[3] == cs[3],
              "update_cache: input must be [1, heads, users, head_dim] matching the cache");
  Tensor index = devicePositions(ctx, ctx.get(op.table(S::f_update_index), "update_cache index"), "update_cache: update_index");
  TTM_CALL(ttm_update_cache(cache.handle->data.get(), in.handle->data.get(), static_cast<const std::int32_t *>(index.handle->data.get()),
                            floatCode(cache.handle->dtype, "update_cache"), cs[0], cs[1], cs[2], cs[3], is[2],
                            op.scalar<std::uint32_t>(S::f_batch_offset, 0), ctx.stream()));
  cache.handle->version = nextTensorVersion();
}
void runFillCache(const fb::Table &op, ProgramContext &ctx) {
  using S = schema::FillCacheOp;
  Tensor &cache = cacheOperand(ctx, op.table(S::f_cache), "fill_cache cache");
  const auto &cs = cache.handle->shape;
  Tensor in = as(ctx, ctx.get(op.table(S::f_input), "fill_cache input"), TensorLayout::Tile, cache.handle->dtype);
  const auto &is = in.handle->shape;
  // lib/Dialect/TTNN/IR/TTNNOps.cpp:4896-4946
  TTRT_ASSERT(is.size() == 4 && is[1] == cs[1] && is[3] == cs[3], "fill_cache: cache and input must agree on dims 1 and 3");
  TTRT_ASSERT(is[2] <= cs[2], "fill_cache: input has more positions than the cache");
  TTRT_ASSERT(is[0] == 1, "fill_cache: input must hold one user");
  TTM_CALL(ttm_fill_cache(cache.handle->data.get(), in.handle->data.get(), floatCode(cache.handle->dtype, "fill_cache"), cs[0], cs[1], cs[2],
                          cs[3], is[2], op.scalar<std::uint32_t>(S::f_batch_offset, 0), ctx.stream()));
  cache.handle->version = nextTensorVersion();
}

// runtime/lib/ttnn/operations/kv_cache/paged_update_cache.cpp:14-57; shapes lib/Dialect/TTNN/IR/TTNNOps.cpp:4719-4820
void runPagedUpdateCache(const fb::Table &op, ProgramContext &ctx) {
  using S = schema::PagedUpdateCacheOp;
  Tensor &cache = cacheOperand(ctx, op.table(S::f_cache), "paged_update_cache cache");
  const auto &cs = cache.handle->shape;
  Tensor in = as(ctx, ctx.get(op.table(S::f_input), "paged_update_cache input"), TensorLayout::Tile, cache.handle->dtype);
  const auto &is = in.handle->shape;
  Tensor index = devicePositions(ctx, ctx.get(op.table(S::f_update_index), "paged_update_cache index"), "paged_update_cache: update_index");
  TTRT_ASSERT(index.handle->shape.size() == 1, "paged_update_cache: update_index must be 1D");
  const std::int64_t users = index.handle->shape[0];
  TTRT_ASSERT(is.size() == 4 && is[0] == 1 && is[1] == users && is[2] == cs[1] && is[3] == cs[3],
              "paged_update_cache: input must be [1, users, heads, head_dim] matching the cache and the update index");
  const bool shared = op.scalar<std::uint8_t>(S::f_share_cache, 0) != 0;
  Tensor table;
  std::int64_t pages = 0;
  if (fb::Table tref = op.table(S::f_page_table)) {
    table = devicePositions(ctx, ctx.get(tref, "paged_update_cache page table"), "paged_update_cache: page_table");
    const auto &ts = table.handle->shape;
    TTRT_ASSERT(ts.size() == 2 && ts[0] == users, "paged_update_cache: page table must be [users, pages]");
    TTRT_ASSERT(cs[2] % 32 == 0, "paged_update_cache: block size must be divisible by 32");
    pages = ts[1];
  } else {
    TTRT_ASSERT(shared ? cs[0] == 1 : users <= static_cast<std::int64_t>(cs[0]), "paged_update_cache: more users than cache entries");
  }
  TTM_CALL(ttm_paged_update_cache(cache.handle->data.get(), in.handle->data.get(), static_cast<const std::int32_t *>(index.handle->data.get()),
                                  table.handle ? static_cast<const std::int32_t *>(table.handle->data.get()) : nullptr,
                                  floatCode(cache.handle->dtype, "paged_update_cache"), cs[0], cs[1], cs[2], cs[3], users, pages,
                                  shared ? 1 : 0, ctx.stream()));
  cache.handle->version = nextTensorVersion();
}
// runtime/lib/ttnn/operations/kv_cache/paged_fill_cache.cpp; golden tools/golden/mapping.py:8966-9008
void runPagedFillCache(const fb::Table &op, ProgramContext &ctx) {
  using S = schema::PagedFillCacheOp;
  Tensor &cache = cacheOperand(ctx, op.table(S::f_cache), "paged_fill_cache cache");
  const auto &cs = cache.handle->shape;
  Tensor in = as(ctx, ctx.get(op.table(S::f_input), "paged_fill_cache input"), TensorLayout::Tile, cache.handle->dtype);
  const auto &is = in.handle->shape;
  TTRT_ASSERT(is.size() == 4 && is[1] == cs[1] && is[3] == cs[3], "paged_fill_cache: input must be [batch, heads, seq, head_dim] matching the cache");
  Tensor table = devicePositions(ctx, ctx.get(op.table(S::f_page_table), "paged_fill_cache page table"), "paged_fill_cache: page_table");
  const auto &ts = table.handle->shape;
  TTRT_ASSERT(ts.size() == 2, "paged_fill_cache: page table must be [users, pages]");
  Tensor rows;
  if (fb::Table bref = op.table(S::f_batch_idx_tensor)) {
    rows = devicePositions(ctx, ctx.get(bref, "paged_fill_cache batch index"), "paged_fill_cache: batch_idx_tensor");
    TTRT_ASSERT(volume(rows.handle->shape) >= is[0], "paged_fill_cache: one batch index per input batch entry is needed");
  }
  TTM_CALL(ttm_paged_fill_cache(cache.handle->data.get(), in.handle->data.get(), static_cast<const std::int32_t *>(table.handle->data.get()),
                                rows.handle ? static_cast<const std::int32_t *>(rows.handle->data.get()) : nullptr,
                                floatCode(cache.handle->dtype, "paged_fill_cache"), cs[0], cs[1], cs[2], cs[3], is[0], is[2], ts[0], ts[1],
                                ctx.stream()));
  cache.handle->version = nextTensorVersion();
}

void sdpaDecode(ProgramContext &ctx, const fb::Table &qRef, const fb::Table &kRef, const fb::Table &vRef, const fb::Table &pageRef,
                const fb::Table &maskRef, const fb::Table &posRef, bool causal, float scale, std::int64_t window,
                const fb::Table &sinkRef, const fb::Table &outRef) {
  Tensor q = as(ctx, ctx.get(qRef, "sdpa_decode query"), TensorLayout::Tile, DataType::BFloat16);
  Tensor k = as(ctx, ctx.get(kRef, "sdpa_decode key"), TensorLayout::Tile, DataType::BFloat16);
  Tensor v = as(ctx, ctx.get(vRef, "sdpa_decode value"), TensorLayout::Tile, DataType::BFloat16);
  const auto &qs = q.handle->shape, &ks = k.handle->shape;
  TTRT_ASSERT(qs.size() == 4 && ks.size() == 4 && v.handle->shape == ks && qs[0] == 1 && qs[3] == ks[3],
              "sdpa_decode: query must be [1, batch, heads, head_dim], key / value 4D with the same head_dim");
  const std::int64_t B = qs[1], H = qs[2], Hkv = ks[1], D = qs[3];
  Tensor table;
  std::int64_t pages = 0, block = 0, cacheBlocks = 0, S = ks[2];
  if (pageRef) {
    table = devicePositions(ctx, ctx.get(pageRef, "sdpa_decode page table"), "sdpa_decode: page_table");
    const auto &ts = table.handle->shape;
    TTRT_ASSERT(ts.size() == 2 && ts[0] == B, "sdpa_decode: page table must be [batch, blocks per user]");
    pages = ts[1]; block = ks[2]; cacheBlocks = ks[0]; S = pages * block;
  } else {
    TTRT_ASSERT(ks[0] == B, "sdpa_decode: key / value batch differs from the query's");
  }
  Tensor mask, pos, sink;
  int maskHeads = 1;
  std::int64_t maskBatch = 1;
  if (sinkRef) {
    sink = as(ctx, ctx.get(sinkRef, "sdpa_decode attention sink"), TensorLayout::Tile, DataType::BFloat16);
    const auto &ss = sink.handle->shape;
    TTRT_ASSERT(ss.size() == 2 && ss[0] == H && ss[1] == 32, "sdpa_decode: attention sink must be [heads, 32]");
  }
  const void *sinkPtr = sink ? sink.handle->data.get() : nullptr;
  if (maskRef) {
    mask = as(ctx, ctx.get(maskRef, "sdpa_decode mask"), TensorLayout::Tile, DataType::BFloat16);
    const auto &ms = mask.handle->shape;
    TTRT_ASSERT(ms.size() == 4 && (ms[0] == 1 || ms[0] == B) && ms[1] == 1 && (ms[2] == 1 || ms[2] == H) && ms[3] == S,
                "sdpa_decode: mask must be [1|batch, 1, 1|heads, positions]");
    maskHeads = static_cast<int>(ms[2]);
    maskBatch = ms[0];
  }
  if (posRef) {
    pos = devicePositions(ctx, ctx.get(posRef, "sdpa_decode cur_pos"), "sdpa_decode: cur_pos_tensor");
    TTRT_ASSERT(volume(pos.handle->shape) == B, "sdpa_decode: cur_pos_tensor must hold one position per user");
  }
  // a reshape to [users, heads * head_dim] that is the only consumer of the result (the head merge in front of the output
  // projection) is folded in: the merge kernel writes that layout directly
  if (fb::Table rs = fusableNext(ctx, OpType::ReshapeOp, schema::ReshapeOp::f_in, schema::ReshapeOp::f_out, outRef, q)) {
    auto finalRef = rs.table(schema::ReshapeOp::f_out);
    const std::vector<std::uint32_t> finalShape = shapeFromTensorRef(finalRef);
    const Dims3 fd = dims3(finalShape);
    if (fd.batch == 1 && fd.rows == B && fd.cols == H * D) {
      Tensor merged = makeDeviceTensor(ctx.dev, finalShape, DataType::BFloat16, TensorLayout::Tile);
      debug::Stats::get().incrementStat("FusedHeadConcat");
      TTM_CALL(ttm_sdpa_decode_windowed(q.handle->data.get(), k.handle->data.get(), v.handle->data.get(),
                                        pos ? static_cast<const std::int32_t *>(pos.handle->data.get()) : nullptr,
                                        mask ? mask.handle->data.get() : nullptr, maskHeads, maskBatch,
                                        table ? static_cast<const std::int32_t *>(table.handle->data.get()) : nullptr, pages, block, cacheBlocks,
                                        merged.handle->data.get(), TTM_BF16, B, H, Hkv, S, D, causal ? 1 : 0, scale, 1, window, sinkPtr,
                                        ctx.stream()));
      ctx.put(finalRef, merged);
      ctx.skip.insert(ctx.opIndex + 1);
      return;
    }
  }
  Tensor out = makeDeviceTensor(ctx.dev, qs, DataType::BFloat16, TensorLayout::Tile);
  TTM_CALL(ttm_sdpa_decode_windowed(q.handle->data.get(), k.handle->data.get(), v.handle->data.get(),
                                    pos ? static_cast<const std::int32_t *>(pos.handle->data.get()) : nullptr,
                                    mask ? mask.handle->data.get() : nullptr, maskHeads, maskBatch,
                                    table ? static_cast<const std::int32_t *>(table.handle->data.get()) : nullptr, pages, block, cacheBlocks,
                                    out.handle->data.get(), TTM_BF16, B, H, Hkv, S, D, causal ? 1 : 0, scale, 0, window, sinkPtr,
                                    ctx.stream()));
  ctx.put(outRef, finish(ctx, out, outRef));
}
void runSdpaDecode(const fb::Table &op, ProgramContext &ctx) {
  using S = schema::ScaledDotProductAttentionDecodeOp;
  sdpaDecode(ctx, op.table(S::f_query), op.table(S::f_key), op.table(S::f_value), fb::Table(), op.table(S::f_attention_mask),
             op.table(S::f_cur_pos_tensor), op.scalar<std::uint8_t>(S::f_is_causal, 0) != 0,
             op.has(S::f_scale) ? op.scalar<float>(S::f_scale, 0.0f) : 0.0f,
             op.has(S::f_sliding_window_size) ? static_cast<std::int64_t>(op.scalar<std::uint32_t>(S::f_sliding_window_size, 0)) : std::int64_t(-1), op.table(S::f_attention_sink),
             op.table(S::f_out));
}
void runPagedSdpaDecode(const fb::Table &op, ProgramContext &ctx) {
  using S = schema::PagedScaledDotProductAttentionDecodeOp;
  TTRT_ASSERT(static_cast<bool>(op.table(S::f_page_table)), "paged sdpa_decode: page table missing");
  sdpaDecode(ctx, op.table(S::f_query), op.table(S::f_key), op.table(S::f_value), op.table(S::f_page_table), op.table(S::f_attention_mask),
             op.table(S::f_cur_pos_tensor), op.scalar<std::uint8_t>(S::f_is_causal, 0) != 0,
             op.has(S::f_scale) ? op.scalar<float>(S::f_scale, 0.0f) : 0.0f,
             op.has(S::f_sliding_window_size) ? static_cast<std::int64_t>(op.scalar<std::uint32_t>(S::f_sliding_window_size, 0)) : std::int64_t(-1), op.table(S::f_attention_sink),
             op.table(S::f_out));
}

// ---- data movement (runtime/lib/ttnn/operations/data_movement/*.cpp)
bool sameTiling(const std::vector<std::uint32_t> &a, const std::vector<std::uint32_t> &b) {
  // physical tile order is unchanged when the last dim is kept and no padding is involved
  if (a.empty() || b.empty() || a.back() != b.back()) return false;
  Dims3 da = dims3(a), db = dims3(b);
  return da.rows % 32 == 0 && db.rows % 32 == 0 && da.cols % 32 == 0 && a.size() >= 2 && b.size() >= 2;
}

Tensor reshapeTo(ProgramContext &ctx, const Tensor &in, const std::vector<std::uint32_t> &oshape) {
  TTRT_ASSERT(volume(in.handle->shape) == volume(oshape), "reshape: element count differs");
  if (in.handle->layout == TensorLayout::RowMajor || sameTiling(in.handle->shape, oshape)) {
    auto t = std::make_shared<TensorImpl>();  // alias: same buffer, new logical shape
    t->shape = oshape; t->dtype = in.handle->dtype; t->layout = in.handle->layout; t->storage = in.handle->storage;
    t->data = in.handle->data; t->bytes = in.handle->bytes; t->device = in.handle->device; t->version = in.handle->version;
    return Tensor{t};
  }
  Tensor out = makeDeviceTensor(ctx.dev, oshape, in.handle->dtype, in.handle->layout);
  zeroIfPadded(ctx, out);
  std::vector<std::int64_t> e{volume(oshape)}, one{1};
  copyView(ctx, in, out, e, one, 0, one, 0);
  return out;
}

std::uint32_t refId(const fb::Table &ref) { return ref.scalar<std::uint32_t>(schema::TensorRef::f_global_id, 0); }

// the operation after the current one, if it is of `type`, consumes `produced` as its first operand, and is the only
// consumer of it; its output must keep the producer's layout so that no conversion hides between the two
fb::Table fusableNext(ProgramContext &ctx, OpType type, int inSlot, int outSlot, const fb::Table &produced, const Tensor &like) {
  if (!ctx.fuseViews || ctx.opIndex + 1 >= ctx.ops.size()) return fb::Table();
  const fb::Table &next = ctx.ops[ctx.opIndex + 1];
  if (static_cast<OpType>(next.scalar<std::uint8_t>(schema::Operation::f_type_type, 0)) != type) return fb::Table();
  fb::Table nop = next.table(schema::Operation::f_type);
  fb::Table in = nop.table(inSlot), out = nop.table(outSlot);
  if (!in || !out || refId(in) != refId(produced)) return fb::Table();
  auto u = ctx.uses.find(refId(produced));
  if (u == ctx.uses.end() || u->second != 1) return fb::Table();
  Layout a = layoutFromTensorRef(produced), b = layoutFromTensorRef(out);
  if (!(a == b) || a.storageType != StorageType::Device || a.layout != like.handle->layout || a.dataType != like.handle->dtype)
    return fb::Table();
  return nop;
}

void runReshape(const fb::Table &op, ProgramContext &ctx) {
  Tensor in = onDevice(ctx, ctx.get(op.table(schema::ReshapeOp::f_in), "reshape in"));
  auto outRef = op.table(schema::ReshapeOp::f_out);
  std::vector<std::uint32_t> oshape = shapeFromTensorRef(outRef);
  const bool copies = in.handle->layout == TensorLayout::Tile && !sameTiling(in.handle->shape, oshape);
  if (copies && !utils::isBlockFormatDataType(in.handle->dtype) &&
      fusableNext(ctx, OpType::PermuteOp, schema::PermuteOp::f_in, schema::PermuteOp::f_out, outRef, in)) {
    TTRT_ASSERT(volume(in.handle->shape) == volume(oshape), "reshape: element count differs");
    ctx.deferred[refId(outRef)] = ProgramContext::DeferredView{in, oshape, rowMajorStrides(oshape)};   // the permute reads the source directly
    return;
  }
  // the head split of a projection in front of a decode-mode rotary embedding: [users, heads * head_dim] ->
  // [1, users, heads, head_dim]; the rotary kernel reads the projection's layout directly
  if (copies && ctx.fuseViews && ctx.opIndex + 1 < ctx.ops.size() && oshape.size() == 4 && oshape[0] == 1 && oshape[3] % 32 == 0 &&
      (in.handle->dtype == DataType::BFloat16 || in.handle->dtype == DataType::Float32)) {
    const fb::Table &next = ctx.ops[ctx.opIndex + 1];
    const Dims3 sd = dims3(in.handle->shape);
    if (static_cast<OpType>(next.scalar<std::uint8_t>(schema::Operation::f_type_type, 0)) == OpType::RotaryEmbeddingOp && sd.batch == 1 &&
        sd.rows == oshape[1] && sd.cols == static_cast<std::int64_t>(oshape[2]) * oshape[3]) {
      using R = schema::RotaryEmbeddingOp;
      fb::Table rop = next.table(schema::Operation::f_type);
      fb::Table rin = rop.table(R::f_input), rout = rop.table(R::f_out);
      auto u = ctx.uses.find(refId(outRef));
      const Layout a = layoutFromTensorRef(outRef);
      if (rin && rout && refId(rin) == refId(outRef) && rop.has(R::f_token_index) && u != ctx.uses.end() && u->second == 1 &&
          a.storageType == StorageType::Device && a.layout == TensorLayout::Tile && a.dataType == in.handle->dtype &&
          layoutFromTensorRef(rout) == a) {
        ctx.deferred[refId(outRef)] = ProgramContext::DeferredView{in, oshape, rowMajorStrides(oshape)};
        return;
      }
    }
  }
  ctx.put(outRef, finish(ctx, reshapeTo(ctx, in, oshape), outRef));
}

// A strided view of `source` written out as a tensor of its own: element v of the view (row-major over `shape`) is
// the source element with row-major index sum v[d] * strides[d].  `finalShape` gives the output another logical shape
// of the same volume (a reshape is the identity on flat indices).
Tensor materialiseView(ProgramContext &ctx, const ProgramContext::DeferredView &v, const std::vector<std::uint32_t> *finalShape) {
  if (finalShape) TTRT_ASSERT(volume(*finalShape) == volume(v.shape), "reshape: element count differs");
  Tensor out = makeDeviceTensor(ctx.dev, finalShape ? *finalShape : v.shape, v.source.handle->dtype, v.source.handle->layout);
  zeroIfPadded(ctx, out);
  copyView(ctx, v.source, out, toI64(v.shape), v.strides, 0, rowMajorStrides(v.shape), 0);
  return out;
}
// out[i0, i1, ...] = in[i_perm...] as a view of the input (or of the view `in` already is)
ProgramContext::DeferredView permutedView(const ProgramContext::DeferredView &in, const std::vector<int> &perm) {
  const size_t rank = in.shape.size();
  TTRT_ASSERT(perm.size() == rank, "permute: permutation rank differs from the tensor rank");
  ProgramContext::DeferredView out{in.source, std::vector<std::uint32_t>(rank), std::vector<std::int64_t>(rank)};
  for (size_t i = 0; i < rank; ++i) {
    TTRT_ASSERT(perm[i] >= 0 && static_cast<size_t>(perm[i]) < rank, "permute: index out of range");
    out.shape[i] = in.shape[perm[i]];
    out.strides[i] = in.strides[perm[i]];
  }
  return out;
}
Tensor permuteTo(ProgramContext &ctx, const Tensor &in, const std::vector<int> &perm) {
  return materialiseView(ctx, permutedView(ProgramContext::DeferredView{in, in.handle->shape, rowMajorStrides(in.handle->shape)}, perm), nullptr);
}
// the next operation is an update_cache that is the only consumer of `produced` (as its input) and whose cache holds
// the element type of `like`: it can read the view directly
bool feedsUpdateCache(ProgramContext &ctx, const fb::Table &produced, const Tensor &like) {
  if (!ctx.fuseViews || ctx.opIndex + 1 >= ctx.ops.size()) return false;
  const fb::Table &next = ctx.ops[ctx.opIndex + 1];
  if (static_cast<OpType>(next.scalar<std::uint8_t>(schema::Operation::f_type_type, 0)) != OpType::UpdateCacheOp) return false;
  fb::Table nop = next.table(schema::Operation::f_type);
  fb::Table in = nop.table(schema::UpdateCacheOp::f_input), cache = nop.table(schema::UpdateCacheOp::f_cache);
  if (!in || !cache || refId(in) != refId(produced)) return false;
  auto u = ctx.uses.find(refId(produced));
  if (u == ctx.uses.end() || u->second != 1) return false;
  Layout a = layoutFromTensorRef(produced);
  if (a.storageType != StorageType::Device || a.layout != TensorLayout::Tile || a.dataType != like.handle->dtype ||
      like.handle->layout != TensorLayout::Tile)
    return false;
  auto c = ctx.pool.find(refId(cache));
  return c != ctx.pool.end() && isTensorAllocated(c->second) && c->second.handle->storage == StorageType::Device &&
         c->second.handle->layout == TensorLayout::Tile && c->second.handle->dtype == like.handle->dtype;
}
// `view` is the head split [B, S, H * D] -> [B, H, S, D] of a tile tensor (whole tiles move, nothing inside them), and
// the only consumer of `produced` is a scaled_dot_product_attention that takes it as query, key or value
bool headSplitForSdpa(ProgramContext &ctx, const fb::Table &produced, const ProgramContext::DeferredView &view) {
  if (!ctx.fuseViews || view.shape.size() != 4) return false;
  const Tensor &src = view.source;
  const std::int64_t B = view.shape[0], H = view.shape[1], Sq = view.shape[2], D = view.shape[3];
  if (src.handle->dtype != DataType::BFloat16 || src.handle->layout != TensorLayout::Tile || src.handle->storage != StorageType::Device) return false;
  if (D % 32 != 0 || !(D == 32 || D == 64 || D == 128 || D == 256)) return false;
  const Dims3 sd = dims3(src.handle->shape);
  if (sd.batch != B || sd.rows != Sq || sd.cols != H * D) return false;
  if (view.strides[3] != 1 || view.strides[2] != H * D || view.strides[1] != D || (B > 1 && view.strides[0] != Sq * H * D)) return false;
  if (!(layoutFromTensorRef(produced) == Layout{StorageType::Device, TensorLayout::Tile, DataType::BFloat16})) return false;
  const std::uint32_t id = refId(produced);
  auto u = ctx.uses.find(id);
  if (u == ctx.uses.end() || u->second != 1) return false;
  for (std::uint32_t j = ctx.opIndex + 1; j < ctx.ops.size(); ++j) {
    const OpType t = static_cast<OpType>(ctx.ops[j].scalar<std::uint8_t>(schema::Operation::f_type_type, 0));
    if (t == OpType::DeallocateOp) continue;
    bool reads = false;
    for (const auto &ref : opRefs(ctx.ops[j]).ins) reads = reads || refId(ref) == id;
    if (!reads) continue;
    if (t != OpType::ScaledDotProductAttentionOp) return false;
    using S = schema::ScaledDotProductAttentionOp;
    fb::Table sop = ctx.ops[j].table(schema::Operation::f_type);
    int named = 0;
    for (int slot : {int(S::f_query), int(S::f_key), int(S::f_value)}) named += sop.table(slot) && refId(sop.table(slot)) == id;
    return named == 1;   // not the mask, and not two operands at once
  }
  return false;
}
void runPermute(const fb::Table &op, ProgramContext &ctx) {
  auto inRef = op.table(schema::PermuteOp::f_in);
  auto pv = op.scalars<std::int64_t>(schema::PermuteOp::f_permutation);
  std::vector<int> perm;
  for (std::uint32_t i = 0; i < pv.size(); ++i) perm.push_back(static_cast<int>(pv[i] < 0 ? pv[i] + pv.size() : pv[i]));
  auto outRef = op.table(schema::PermuteOp::f_out);
  ProgramContext::DeferredView in;
  auto d = ctx.deferred.find(refId(inRef));
  if (d != ctx.deferred.end()) {
    in = d->second;
    ctx.deferred.erase(d);
  } else {
    Tensor t = onDevice(ctx, ctx.get(inRef, "permute in"));
    in = ProgramContext::DeferredView{t, t.handle->shape, rowMajorStrides(t.handle->shape)};
  }
  ProgramContext::DeferredView view = permutedView(in, perm);
  const Tensor &src = in.source;
  if (src.handle->layout == TensorLayout::Tile && !utils::isBlockFormatDataType(src.handle->dtype)) {
    if (feedsUpdateCache(ctx, outRef, src)) {
      ctx.deferred[refId(outRef)] = view;   // the cache write reads the source directly
      return;
    }
    if (headSplitForSdpa(ctx, outRef, view)) {
      ctx.headViews[refId(outRef)] = src;   // the attention kernel reads the projection's layout in place
      return;
    }
    if (fb::Table rs = fusableNext(ctx, OpType::ReshapeOp, schema::ReshapeOp::f_in, schema::ReshapeOp::f_out, outRef, src)) {
      auto finalRef = rs.table(schema::ReshapeOp::f_out);
      std::vector<std::uint32_t> finalShape = shapeFromTensorRef(finalRef);
      ctx.put(finalRef, materialiseView(ctx, view, &finalShape));
      ctx.skip.insert(ctx.opIndex + 1);
      return;
    }
  }
  ctx.put(outRef, finish(ctx, materialiseView(ctx, view, nullptr), outRef));
}
void runTranspose(const fb::Table &op, ProgramContext &ctx) {
  Tensor in = onDevice(ctx, ctx.get(op.table(schema::TransposeOp::f_in), "transpose in"));
  int rank = static_cast<int>(in.handle->shape.size());
  int d0 = op.scalar<std::int32_t>(schema::TransposeOp::f_dim0, 0), d1 = op.scalar<std::int32_t>(schema::TransposeOp::f_dim1, 0);
  if (d0 < 0) d0 += rank;
  if (d1 < 0) d1 += rank;
  std::vector<int> perm(rank);
  for (int i = 0; i < rank; ++i) perm[i] = i;
  TTRT_ASSERT(d0 >= 0 && d0 < rank && d1 >= 0 && d1 < rank, "transpose: dim out of range");
  std::swap(perm[d0], perm[d1]);
  auto outRef = op.table(schema::TransposeOp::f_out);
  ctx.put(outRef, finish(ctx, permuteTo(ctx, in, perm), outRef));
}
void runConcat(const fb::Table &op, ProgramContext &ctx) {
  auto ins = op.tables(schema::ConcatOp::f_inputs);
  TTRT_ASSERT(ins.size() >= 1, "concat: no inputs");
  auto outRef = op.table(schema::ConcatOp::f_out);
  std::vector<std::uint32_t> oshape = shapeFromTensorRef(outRef);
  Tensor first = onDevice(ctx, ctx.get(ins[0], "concat in"));
  int rank = static_cast<int>(oshape.size());
  int dim = op.scalar<std::int32_t>(schema::ConcatOp::f_dim, 0);
  if (dim < 0) dim += rank;
  TTRT_ASSERT(dim >= 0 && dim < rank, "concat: dim out of range");
  {
    // the copies below address the result by the inputs' extents: the declared shape must be what the inputs add up to
    std::vector<std::uint32_t> want = first.handle->shape;
    TTRT_ASSERT(static_cast<int>(want.size()) == rank, "concat: rank mismatch");
    want[dim] = 0;
    for (std::uint32_t i = 0; i < ins.size(); ++i) {
      const std::vector<std::uint32_t> &si = ctx.get(ins[i], "concat in").handle->shape;
      TTRT_ASSERT(static_cast<int>(si.size()) == rank, "concat: rank mismatch");
      for (int d = 0; d < rank; ++d)
        TTRT_ASSERT(d == dim || si[d] == first.handle->shape[d], "concat: inputs differ in a dimension other than the concatenated one");
      want[dim] += si[dim];
    }
    requireResultShape(outRef, want, "concat");
  }
  Tensor out = makeDeviceTensor(ctx.dev, oshape, first.handle->dtype, first.handle->layout);
  zeroIfPadded(ctx, out);
  auto os = rowMajorStrides(oshape);
  std::int64_t at = 0;
  for (std::uint32_t i = 0; i < ins.size(); ++i) {
    Tensor t = as(ctx, ctx.get(ins[i], "concat in"), first.handle->layout, first.handle->dtype);
    TTRT_ASSERT(static_cast<int>(t.handle->shape.size()) == rank, "concat: rank mismatch");
    copyView(ctx, t, out, toI64(t.handle->shape), rowMajorStrides(t.handle->shape), 0, os, at * os[dim]);
    at += t.handle->shape[dim];
  }
  TTRT_ASSERT(at == oshape[dim], "concat: inputs do not add up to the output extent");
  ctx.put(outRef, finish(ctx, out, outRef));
}
void runSlice(const fb::Table &op, ProgramContext &ctx) {
  Tensor in = onDevice(ctx, ctx.get(op.table(schema::SliceOp::f_in), "slice in"));
  TTRT_ASSERT(op.scalar<std::uint8_t>(schema::SliceOp::f_params_type, 0) == static_cast<std::uint8_t>(schema::SliceOpParams::SliceStaticOpParams),
              "slice: only static begins/ends are supported");
  auto prm = op.table(schema::SliceOp::f_params);
  auto begins = prm.scalars<std::int64_t>(schema::SliceStaticOpParams::f_begins), ends = prm.scalars<std::int64_t>(schema::SliceStaticOpParams::f_ends);
  auto steps = op.scalars<std::int64_t>(schema::SliceOp::f_step);
  const auto &shape = in.handle->shape;
  const size_t rank = shape.size();
  TTRT_ASSERT(begins.size() == rank && ends.size() == rank, "slice: begins/ends rank mismatch");
  auto ss = rowMajorStrides(shape);
  std::vector<std::uint32_t> oshape(rank);
  std::vector<std::int64_t> sst(rank);
  std::int64_t base = 0;
  for (size_t i = 0; i < rank; ++i) {
    std::int64_t b = begins[i], e = ends[i], st = i < steps.size() ? steps[i] : 1;
    if (b < 0) b += shape[i];
    if (e < 0) e += shape[i];
    TTRT_ASSERT(st > 0 && b >= 0 && e <= static_cast<std::int64_t>(shape[i]) && b <= e, "slice: bad range");
    oshape[i] = static_cast<std::uint32_t>((e - b + st - 1) / st);
    sst[i] = ss[i] * st;
    base += b * ss[i];
  }
  Tensor out = makeDeviceTensor(ctx.dev, oshape, in.handle->dtype, in.handle->layout);
  zeroIfPadded(ctx, out);
  copyView(ctx, in, out, toI64(oshape), sst, base, rowMajorStrides(oshape), 0);
  auto outRef = op.table(schema::SliceOp::f_out);
  ctx.put(outRef, finish(ctx, out, outRef));
}
void runRepeatInterleave(const fb::Table &op, ProgramContext &ctx) {
  Tensor in = onDevice(ctx, ctx.get(op.table(schema::RepeatInterleaveOp::f_input), "repeat_interleave in"));
  const auto &shape = in.handle->shape;
  int rank = static_cast<int>(shape.size());
  int dim = op.scalar<std::int32_t>(schema::RepeatInterleaveOp::f_dim, 0);
  if (dim < 0) dim += rank;
  std::uint32_t rep = op.scalar<std::uint32_t>(schema::RepeatInterleaveOp::f_repeats, 1);
  TTRT_ASSERT(dim >= 0 && dim < rank && rep >= 1, "repeat_interleave: bad arguments");
  std::vector<std::uint32_t> oshape = shape;
  oshape[dim] *= rep;
  // view [.., shape[dim], rep, ..]: the rep axis has source stride 0
  std::vector<std::int64_t> extent, sst, dstv;
  auto ss = rowMajorStrides(shape), os = rowMajorStrides(oshape);
  for (int i = 0; i < rank; ++i) {
    extent.push_back(shape[i]);
    sst.push_back(ss[i]);
    dstv.push_back(i == dim ? os[i] * rep : os[i]);
    if (i == dim) { extent.push_back(rep); sst.push_back(0); dstv.push_back(os[i]); }
  }
  Tensor out = makeDeviceTensor(ctx.dev, oshape, in.handle->dtype, in.handle->layout);
  zeroIfPadded(ctx, out);
  copyView(ctx, in, out, extent, sst, 0, dstv, 0);
  auto outRef = op.table(schema::RepeatInterleaveOp::f_out);
  ctx.put(outRef, finish(ctx, out, outRef));
}

// ---- head splits and merges around the attention ops (runtime/lib/ttnn/operations/transformer/{concatenate_heads,
// split_query_key_value_and_split_heads,nlp_concat_heads,nlp_concat_heads_decode,nlp_create_qkv_heads_decode}.cpp): each
// result is a strided view of its operand, written out by one copy.  (Where the compiler emits reshape + permute instead,
// the attention runners fold them away; these ops are materialised as they stand.)
// a tensor of `shape` whose element v (row-major) is the source's row-major element base + sum v[d] * strides[d]
Tensor stridedCopy(ProgramContext &ctx, const Tensor &src, const std::vector<std::uint32_t> &shape, const std::vector<std::int64_t> &strides,
                   std::int64_t base, const std::vector<std::uint32_t> &finalShape) {
  TTRT_ASSERT(volume(finalShape) == volume(shape), "head split / merge: output shape does not match");
  Tensor out = makeDeviceTensor(ctx.dev, finalShape, src.handle->dtype, src.handle->layout);
  zeroIfPadded(ctx, out);
  copyView(ctx, src, out, toI64(shape), strides, base, rowMajorStrides(shape), 0);
  return out;
}
Tensor plainOperand(ProgramContext &ctx, const fb::Table &ref, const char *what) {
  Tensor t = onDevice(ctx, ctx.get(ref, what));
  TTRT_ASSERT(!utils::isBlockFormatDataType(t.handle->dtype), std::string(what) + ": block-float tensors are not supported here");
  return t;
}
// [B, H, S, D] -> [B, S, H * D] (ConcatenateHeadsOp) or [B, 1, S, H * D] (NLPConcatHeadsOp)
void concatHeads(ProgramContext &ctx, const fb::Table &inRef, const fb::Table &outRef, const char *what) {
  Tensor in = plainOperand(ctx, inRef, what);
  const auto &s = in.handle->shape;
  TTRT_ASSERT(s.size() == 4, std::string(what) + ": input must be [batch, heads, seq, head_dim]");
  const std::int64_t H = s[1], S = s[2], D = s[3];
  Tensor out = stridedCopy(ctx, in, {s[0], s[2], s[1], s[3]}, {H * S * D, D, S * D, 1}, 0, shapeFromTensorRef(outRef));
  ctx.put(outRef, finish(ctx, out, outRef));
}
void runConcatenateHeads(const fb::Table &op, ProgramContext &ctx) {
  concatHeads(ctx, op.table(schema::ConcatenateHeadsOp::f_in), op.table(schema::ConcatenateHeadsOp::f_out), "concatenate_heads");
}
void runNlpConcatHeads(const fb::Table &op, ProgramContext &ctx) {
  concatHeads(ctx, op.table(schema::NLPConcatHeadsOp::f_in), op.table(schema::NLPConcatHeadsOp::f_out), "nlp_concat_heads");
}
// [1, B, Hpad, D] -> [1, 1, B, num_heads * D]: the first num_heads heads of every user, side by side
void runNlpConcatHeadsDecode(const fb::Table &op, ProgramContext &ctx) {
  using S = schema::NLPConcatHeadsDecodeOp;
  Tensor in = plainOperand(ctx, op.table(S::f_in), "nlp_concat_heads_decode");
  const auto &s = in.handle->shape;
  const std::uint32_t heads = op.scalar<std::uint32_t>(S::f_num_heads, 0);
  TTRT_ASSERT(s.size() == 4 && s[0] == 1 && heads >= 1 && heads <= s[2], "nlp_concat_heads_decode: input must be [1, users, heads (padded), head_dim]");
  auto outRef = op.table(S::f_out);
  Tensor out = stridedCopy(ctx, in, {s[1], heads, s[3]}, {static_cast<std::int64_t>(s[2]) * s[3], s[3], 1}, 0, shapeFromTensorRef(outRef));
  ctx.put(outRef, finish(ctx, out, outRef));
}
// [1, 1, B, (H + 2 Hkv) * D] -> q [1, B, H, D], k and v [1, B, Hkv, D]
void runNlpCreateQkvHeadsDecode(const fb::Table &op, ProgramContext &ctx) {
  using S = schema::NLPCreateQKVHeadsDecodeOp;
  TTRT_ASSERT(!op.table(S::f_batch_offset) && !op.has(S::f_slice_size), "nlp_create_qkv_heads_decode: batch_offset / slice_size are not supported");
  Tensor in = plainOperand(ctx, op.table(S::f_input), "nlp_create_qkv_heads_decode");
  const auto &s = in.handle->shape;
  const std::int64_t H = op.scalar<std::uint32_t>(S::f_num_heads, 0);
  const std::int64_t Hkv = op.has(S::f_num_kv_heads) ? op.scalar<std::uint32_t>(S::f_num_kv_heads, 0) : H;
  TTRT_ASSERT(s.size() == 4 && s[0] == 1 && s[1] == 1 && H >= 1 && Hkv >= 1 && s[3] % (H + 2 * Hkv) == 0,
              "nlp_create_qkv_heads_decode: input must be [1, 1, users, (heads + 2 kv_heads) * head_dim]");
  const std::int64_t W = s[3], D = W / (H + 2 * Hkv);
  const std::uint32_t B = s[2], d = static_cast<std::uint32_t>(D);
  auto part = [&](const fb::Table &ref, std::int64_t heads, std::int64_t base) {
    Tensor t = stridedCopy(ctx, in, {B, static_cast<std::uint32_t>(heads), d}, {W, D, 1}, base, shapeFromTensorRef(ref));
    ctx.put(ref, finish(ctx, t, ref));
  };
  part(op.table(S::f_q_out), H, 0);
  part(op.table(S::f_k_out), Hkv, H * D);
  part(op.table(S::f_v_out), Hkv, (H + Hkv) * D);
}
// fused [B, S, (H + 2 Hkv) * D], or q [B, S, H * D] and kv [B, S, 2 Hkv * D] -> q [B, H, S, D], k [B, Hkv, S, D] (or
// [B, Hkv, D, S] with transpose_key), v [B, Hkv, S, D]; golden tools/golden/mapping.py:5084-5186
void runSplitQkvAndSplitHeads(const fb::Table &op, ProgramContext &ctx) {
  using S = schema::SplitQueryKeyValueAndSplitHeadsOp;
  Tensor in = plainOperand(ctx, op.table(S::f_in), "split_query_key_value_and_split_heads");
  const auto &s = in.handle->shape;
  const std::int64_t H = op.scalar<std::uint32_t>(S::f_num_heads, 0);
  const std::int64_t Hkv = op.has(S::f_num_kv_heads) ? op.scalar<std::uint32_t>(S::f_num_kv_heads, 0) : H;
  const bool transposeKey = op.scalar<std::uint8_t>(S::f_transpose_key, 0) != 0;
  TTRT_ASSERT(s.size() == 3 && H >= 1 && Hkv >= 1, "split_query_key_value_and_split_heads: input must be [batch, seq, hidden]");
  const std::uint32_t B = s[0], Sq = s[1];
  Tensor kv;
  std::int64_t D, Wq = s[2], Wkv, kBase, vBase;
  if (auto kr = op.table(S::f_kv_input)) {
    kv = plainOperand(ctx, kr, "split_query_key_value_and_split_heads kv");
    const auto &ks = kv.handle->shape;
    TTRT_ASSERT(ks.size() == 3 && ks[0] == B && ks[1] == Sq && Wq % H == 0 && ks[2] == 2 * Hkv * (Wq / H),
                "split_query_key_value_and_split_heads: kv input must be [batch, seq, 2 * kv_heads * head_dim]");
    D = Wq / H; Wkv = ks[2]; kBase = 0; vBase = Hkv * D;
  } else {
    TTRT_ASSERT(Wq % (H + 2 * Hkv) == 0, "split_query_key_value_and_split_heads: hidden size must be (heads + 2 kv_heads) * head_dim");
    kv = in;
    D = Wq / (H + 2 * Hkv); Wkv = Wq; kBase = H * D; vBase = (H + Hkv) * D;
  }
  const std::uint32_t d = static_cast<std::uint32_t>(D), h = static_cast<std::uint32_t>(H), hk = static_cast<std::uint32_t>(Hkv);
  auto qRef = op.table(S::f_q_out), kRef = op.table(S::f_k_out), vRef = op.table(S::f_v_out);
  Tensor q = stridedCopy(ctx, in, {B, h, Sq, d}, {Sq * Wq, D, Wq, 1}, 0, shapeFromTensorRef(qRef));
  Tensor k = transposeKey ? stridedCopy(ctx, kv, {B, hk, d, Sq}, {Sq * Wkv, D, 1, Wkv}, kBase, shapeFromTensorRef(kRef))
                          : stridedCopy(ctx, kv, {B, hk, Sq, d}, {Sq * Wkv, D, Wkv, 1}, kBase, shapeFromTensorRef(kRef));
  Tensor v = stridedCopy(ctx, kv, {B, hk, Sq, d}, {Sq * Wkv, D, Wkv, 1}, vBase, shapeFromTensorRef(vRef));
  ctx.put(qRef, finish(ctx, q, qRef));
  ctx.put(kRef, finish(ctx, k, kRef));
  ctx.put(vRef, finish(ctx, v, vRef));
}

// runtime/lib/ttnn/operations/data_movement/repeat.cpp:12-22: the input tiled repeat_dims[i] times along dim i
void runRepeat(const fb::Table &op, ProgramContext &ctx) {
  Tensor in = onDevice(ctx, ctx.get(op.table(schema::RepeatOp::f_in), "repeat in"));
  const auto &shape = in.handle->shape;
  const int rank = static_cast<int>(shape.size());
  auto reps = op.scalars<std::int64_t>(schema::RepeatOp::f_repeat_dims);
  TTRT_ASSERT(static_cast<int>(reps.size()) == rank, "repeat: one repeat count per dimension expected");
  std::vector<std::uint32_t> oshape = shape;
  for (int i = 0; i < rank; ++i) {
    TTRT_ASSERT(reps[i] >= 1, "repeat: counts must be positive");
    oshape[i] = static_cast<std::uint32_t>(shape[i] * reps[i]);
  }
  // view [.., rep_i, shape_i, ..]: the rep axes have source stride 0
  std::vector<std::int64_t> extent, sst, dstv;
  auto ss = rowMajorStrides(shape), os = rowMajorStrides(oshape);
  for (int i = 0; i < rank; ++i) {
    if (reps[i] > 1) { extent.push_back(reps[i]); sst.push_back(0); dstv.push_back(os[i] * shape[i]); }
    extent.push_back(shape[i]); sst.push_back(ss[i]); dstv.push_back(os[i]);
  }
  TTRT_ASSERT(extent.size() <= 8, "repeat: more than 8 view dimensions");
  Tensor out = makeDeviceTensor(ctx.dev, oshape, in.handle->dtype, in.handle->layout);
  zeroIfPadded(ctx, out);
  copyView(ctx, in, out, extent, sst, 0, dstv, 0);
  auto outRef = op.table(schema::RepeatOp::f_out);
  ctx.put(outRef, finish(ctx, out, outRef));
}

// runtime/lib/ttnn/operations/embedding/embedding.cpp:14-43: rows of the table picked by index
void runEmbedding(const fb::Table &op, ProgramContext &ctx) {
  using S = schema::EmbeddingOp;
  Tensor idx0 = ctx.get(op.table(S::f_input), "embedding indices");
  const DataType it = idx0.handle->dtype == DataType::UInt32 ? DataType::UInt32 : DataType::Int32;
  Tensor idx = as(ctx, idx0, TensorLayout::RowMajor, it);
  Tensor w0 = onDevice(ctx, ctx.get(op.table(S::f_weight), "embedding weight"));
  TTRT_ASSERT(!utils::isBlockFormatDataType(w0.handle->dtype), "embedding: block-float tables are not supported");
  const DataType wt = w0.handle->dtype == DataType::Float32 ? DataType::Float32 : DataType::BFloat16;
  Tensor w = as(ctx, w0, TensorLayout::RowMajor, wt);
  const auto &ws = w.handle->shape;
  TTRT_ASSERT(ws.size() >= 2 && volume(ws) == static_cast<std::int64_t>(ws[ws.size() - 2]) * ws.back(),
              "embedding: the table must be [.., vocab, dim] with leading ones");
  auto outRef = op.table(S::f_out);
  const std::vector<std::uint32_t> oshape = shapeFromTensorRef(outRef);
  const std::int64_t rows = volume(idx.handle->shape), vocab = ws[ws.size() - 2], dim = ws.back();
  TTRT_ASSERT(!oshape.empty() && oshape.back() == dim && volume(oshape) == rows * dim, "embedding: output shape must be indices x dim");
  Tensor out = makeDeviceTensor(ctx.dev, oshape, wt, TensorLayout::RowMajor);
  TTM_CALL(ttm_embedding(idx.handle->data.get(), ttmDtype(it), w.handle->data.get(), out.handle->data.get(),
                         static_cast<int>(utils::dataTypeElementSize(wt)), rows, vocab, dim, ctx.stream()));
  ctx.put(outRef, finish(ctx, out, outRef));
}

// runtime/lib/ttnn/operations/reduction/argmax.cpp:14-28: index of the largest element along `dim`, or of the whole tensor
void runArgMax(const fb::Table &op, ProgramContext &ctx) {
  using S = schema::ReductionArgMaxOp;
  Tensor x0 = onDevice(ctx, ctx.get(op.table(S::f_in), "argmax in"));
  const DataType dt = computeDtypeOf({x0.handle->dtype});
  Tensor x = as(ctx, x0, x0.handle->layout, dt);
  const int rank = static_cast<int>(x.handle->shape.size());
  std::int64_t rows = 1, cols = volume(x.handle->shape);
  if (op.has(S::f_dim) && rank > 0) {
    int dim = op.scalar<std::int32_t>(S::f_dim, 0);
    if (dim < 0) dim += rank;
    TTRT_ASSERT(dim >= 0 && dim < rank, "argmax: dimension out of range");
    if (dim != rank - 1) x = moveDimLast(ctx, x, dim, false, x.handle->shape);
    cols = x.handle->shape.back();
    rows = volume(x.handle->shape) / std::max<std::int64_t>(cols, 1);
  }
  TTRT_ASSERT(cols > 0, "argmax: empty reduction");
  x = as(ctx, x, TensorLayout::RowMajor, dt);
  auto outRef = op.table(S::f_out);
  const std::vector<std::uint32_t> oshape = shapeFromTensorRef(outRef);
  TTRT_ASSERT(volume(oshape) == rows, "argmax: output shape does not match");
  Tensor out = makeDeviceTensor(ctx.dev, oshape, DataType::Int32, TensorLayout::RowMajor);
  TTM_CALL(ttm_argmax(x.handle->data.get(), ttmDtype(dt), static_cast<std::int32_t *>(out.handle->data.get()), rows, cols, ctx.stream()));
  ctx.put(outRef, finish(ctx, out, outRef));
}

// ---- creation (runtime/lib/ttnn/operations/creation/*.cpp)
// arange.cpp:14-42: start, start + step, ... below end
void runArange(const fb::Table &op, ProgramContext &ctx) {
  using S = schema::ArangeOp;
  const double start = op.scalar<float>(S::f_start, 0.0f), end = op.scalar<float>(S::f_end, 0.0f), step = op.scalar<float>(S::f_step, 0.0f);
  TTRT_ASSERT(step != 0.0, "arange: step must not be zero");
  auto outRef = op.table(S::f_out);
  const std::vector<std::uint32_t> oshape = shapeFromTensorRef(outRef);
  const std::int64_t n = std::max<std::int64_t>(0, static_cast<std::int64_t>(std::ceil((end - start) / step)));
  TTRT_ASSERT(volume(oshape) == n, "arange: output holds " + std::to_string(volume(oshape)) + " elements, the range " + std::to_string(n));
  Layout want = layoutFromTensorRef(outRef);
  DataType dt = want.dataType;
  if (dt != DataType::Float32 && dt != DataType::BFloat16 && dt != DataType::Int32 && dt != DataType::UInt32) dt = DataType::Float32;
  Tensor out = makeDeviceTensor(ctx.dev, oshape, dt, TensorLayout::RowMajor);
  TTM_CALL(ttm_arange(out.handle->data.get(), ttmDtype(dt), n, start, step, ctx.stream()));
  ctx.put(outRef, finish(ctx, out, outRef));
}
void runConstant(const fb::Table &op, ProgramContext &ctx) {
  auto outRef = op.table(schema::ConstantOp::f_out);
  auto bytes = op.scalars<std::uint8_t>(schema::ConstantOp::f_input);
  DataType in = static_cast<DataType>(op.scalar<std::uint16_t>(schema::ConstantOp::f_input_dtype, 0));
  std::vector<std::uint32_t> shape = shapeFromTensorRef(outRef);
  TTRT_ASSERT(static_cast<std::int64_t>(bytes.size()) == volume(shape) * utils::dataTypeElementSize(in), "constant: payload size does not match the shape");
  Tensor h = createOwnedHostTensor(bytes.data(), shape, {}, utils::dataTypeElementSize(in), in);
  ctx.put(outRef, convertTo(ctx, h, layoutFromTensorRef(outRef)));
}
void fillTensor(ProgramContext &ctx, const fb::Table &outRef, double value) {
  Layout want = layoutFromTensorRef(outRef);
  std::vector<std::uint32_t> shape = shapeFromTensorRef(outRef);
  std::int64_t n = volume(shape);
  std::vector<float> host(static_cast<size_t>(n), static_cast<float>(value));
  Tensor h = createOwnedHostTensor(host.data(), shape, {}, 4, DataType::Float32);
  ctx.put(outRef, convertTo(ctx, h, want));
}
void runFull(const fb::Table &op, ProgramContext &ctx) {
  double v = 0.0;
  auto fv = op.table(schema::FullOp::f_fill_value);
  auto kind = op.scalar<std::uint8_t>(schema::FullOp::f_fill_value_type, 0);
  if (kind == static_cast<std::uint8_t>(schema::NumberType::FP)) v = fv.scalar<float>(schema::FloatingPointType::f_value, 0.0f);
  else if (kind == static_cast<std::uint8_t>(schema::NumberType::I32)) v = fv.scalar<std::int32_t>(schema::IntegralType::f_value, 0);
  fillTensor(ctx, op.table(schema::FullOp::f_out), v);
}
void runNamedFull(const fb::Table &op, ProgramContext &ctx) {
  auto t = op.scalar<std::uint32_t>(schema::NamedFullOp::f_type, 0);
  fillTensor(ctx, op.table(schema::NamedFullOp::f_out), t == static_cast<std::uint32_t>(schema::NamedFullOpType::Ones) ? 1.0 : 0.0);
}
void runEmpty(const fb::Table &op, ProgramContext &ctx) {
  auto outRef = op.table(schema::EmptyOp::f_out);
  Layout want = layoutFromTensorRef(outRef);
  Tensor t = makeDeviceTensor(ctx.dev, shapeFromTensorRef(outRef), want.dataType, want.layout);
  TTM_CALL(ttm_fill_u32(t.handle->data.get(), 0, (t.handle->bytes + 3) / 4, ctx.stream()));
  ctx.put(outRef, t);
}

void runDeallocate(const fb::Table &op, ProgramContext &ctx) {
  auto ref = op.table(schema::DeallocateOp::f_in);
  std::uint32_t id = ref.scalar<std::uint32_t>(schema::TensorRef::f_global_id, 0);
  ctx.headViews.erase(id);
  auto it = ctx.pool.find(id);
  if (it == ctx.pool.end()) return;
  if (getTensorRetain(it->second)) return;  // runtime/lib/ttnn/operations/deletion/deallocate.cpp:16-18
  ctx.pool.erase(it);                        // other aliases (reshape views) keep the buffer alive
}

// ---- const-eval (runtime/lib/ttnn/operations/cache/load_cached.cpp:20-90)
void runLoadCached(const fb::Table &op, ProgramContext &ctx) {
  auto ins = op.tables(schema::LoadCachedOp::f_inputs), outs = op.tables(schema::LoadCachedOp::f_outputs);
  std::uint32_t prog = op.scalar<std::uint32_t>(schema::LoadCachedOp::f_program_idx, 0);
  std::vector<Tensor> inputs;
  std::vector<std::uint64_t> versions;
  for (std::uint32_t i = 0; i < ins.size(); ++i) {
    inputs.push_back(ctx.get(ins[i], "load_cached in"));
    versions.push_back(inputs.back().handle->version);
  }
  const ConstEvalKey key{ctx.binary.id(), prog, versions};
  {
    std::vector<Tensor> cached;
    {
      std::lock_guard<std::mutex> g(ctx.dev->constEvalMu);
      auto it = ctx.dev->constEval.find(key);
      if (it != ctx.dev->constEval.end()) cached = it->second.outputs;
    }
    if (!cached.empty()) {
      debug::Stats::get().incrementStat("ConstEvalCacheHit");
      for (std::uint32_t i = 0; i < outs.size(); ++i) ctx.put(outs[i], cached.at(i));
      return;
    }
  }
  debug::Stats::get().incrementStat("ConstEvalCacheMiss");
  std::vector<Tensor> results = executeProgram(ctx.dev, ctx.binary, prog, inputs);
  TTRT_ASSERT(results.size() == outs.size(), "load_cached: callee returned a different number of outputs");
  for (auto &t : results) setTensorRetain(t, true);
  {
    ConstEvalEntry replaced;   // destroyed after the lock is released
    std::lock_guard<std::mutex> g(ctx.dev->constEvalMu);
    ConstEvalEntry &slot = ctx.dev->constEval[key];
    replaced = std::move(slot);
    slot = ConstEvalEntry{versions, results};
  }
  // The entry can be asked for only while all the tensors it was computed from exist (a version belongs to one tensor):
  // when one of them is destroyed the entry goes with it, as in the reference (global_tensor_cache.cpp, store()).
  std::weak_ptr<DeviceState> device = ctx.dev;
  for (Tensor &in : inputs) {
    std::lock_guard<std::mutex> g(in.handle->destroyMu);
    in.handle->onDestroy.push_back([device, key] {
      auto d = device.lock();
      if (!d) return;
      ConstEvalEntry dropped;   // destroyed after the lock is released
      {
        std::lock_guard<std::mutex> g2(d->constEvalMu);
        auto it = d->constEval.find(key);
        if (it == d->constEval.end()) return;
        dropped = std::move(it->second);
        d->constEval.erase(it);
      }
      debug::Stats::get().incrementStat("ConstEvalCacheEvicted");
    });
  }
  for (std::uint32_t i = 0; i < outs.size(); ++i) ctx.put(outs[i], results[i]);
}
void runFuncCall(const fb::Table &op, ProgramContext &ctx) {
  auto ins = op.tables(schema::FuncCallOp::f_inputs), outs = op.tables(schema::FuncCallOp::f_outputs);
  std::vector<Tensor> inputs;
  for (std::uint32_t i = 0; i < ins.size(); ++i) inputs.push_back(ctx.get(ins[i], "func_call in"));
  std::vector<Tensor> results = executeProgram(ctx.dev, ctx.binary, op.scalar<std::uint32_t>(schema::FuncCallOp::f_program_id, 0), inputs);
  TTRT_ASSERT(results.size() == outs.size(), "func_call: callee returned a different number of outputs");
  for (std::uint32_t i = 0; i < outs.size(); ++i) ctx.put(outs[i], results[i]);
}

// ---- CPU-hoisted ops (runtime/lib/ttnn/operations/cpu/cpu.cpp:215-238, runtime/lib/common/dylib.cpp:13-38,
// runtime/include/tt/runtime/detail/common/dylib.h:35-175).  A program carries its dynamic libraries as byte vectors
// (Program.dylibs); each is loaded once per binary from an in-memory file.  The callee takes an array of WrappedTensor
// (dense row-major host data: start, aligned start, start index, sizes then strides) and returns a malloc'ed array of
// outputs whose data buffers, shared sizes / strides block and the array itself the runtime frees.
struct WrappedTensor {
  void *start;
  void *alignedStart;
  std::int64_t startIdx;
  std::int64_t *sizesAndStrides;
};
using WrappedFunc = WrappedTensor *(*)(WrappedTensor *);

void *loadLibraryFromMemory(const std::uint8_t *data, size_t size) {
  const int fd = static_cast<int>(::syscall(SYS_memfd_create, "dylib", 1u /* MFD_CLOEXEC */));
  TTRT_ASSERT(fd >= 0, "CpuOp: memfd_create failed");
  size_t done = 0;
  while (done < size) {
    const ssize_t n = ::write(fd, data + done, size - done);
    if (n <= 0) break;
    done += static_cast<size_t>(n);
  }
  void *handle = done == size ? ::dlopen(("/proc/self/fd/" + std::to_string(fd)).c_str(), RTLD_LAZY | RTLD_LOCAL) : nullptr;
  const std::string err = handle ? "" : (done == size ? std::string(::dlerror()) : "short write");
  ::close(fd);   // the mapping stays
  TTRT_ASSERT(handle != nullptr, "CpuOp: failed to open the program's dynamic library: " + err);
  return handle;
}

// handles by (binary id, program index, dylib id); a binary's libraries stay loaded for the life of the process (the
// reference unloads them with the program executor; code pages of a few KiB are not worth the unload hazards)
WrappedFunc cpuFunction(const Binary &binary, std::uint32_t programIndex, std::uint32_t dylibId, const std::string &name) {
  static std::mutex mu;
  static auto *handles = new std::map<std::tuple<std::uint64_t, std::uint32_t, std::uint32_t>, void *>;
  std::lock_guard<std::mutex> g(mu);
  const auto key = std::make_tuple(binary.id(), programIndex, dylibId);
  auto it = handles->find(key);
  if (it == handles->end()) {
    fb::Table program = binary.handle->root.tables(schema::TTNNBinary::f_programs)[programIndex];
    auto libs = program.tables(schema::Program::f_dylibs);
    void *h = nullptr;
    for (std::uint32_t i = 0; i < libs.size() && !h; ++i) {
      if (libs[i].scalar<std::uint32_t>(schema::DynamicLib::f_dylib_id, 0) != dylibId) continue;
      auto raw = libs[i].scalars<std::uint8_t>(schema::DynamicLib::f_raw_file);
      h = loadLibraryFromMemory(raw.data(), raw.size());
    }
    TTRT_ASSERT(h != nullptr, "could not find dylib corresponding to id: " + std::to_string(dylibId));
    it = handles->emplace(key, h).first;
  }
  auto fn = reinterpret_cast<WrappedFunc>(::dlsym(it->second, name.c_str()));
  TTRT_ASSERT(fn != nullptr, "could not find requested op: \"" + name + "\" in dylib with id: " + std::to_string(dylibId));
  return fn;
}

// the function of a CpuOp on the given host tensors (runtime/lib/ttnn/operations/cpu/cpu.cpp:240-300): needs the binary
// for the program's libraries, nothing else of a running program
std::vector<Tensor> callCpuFunction(const Binary &binary, std::uint32_t programIndex, const fb::Table &op, const std::vector<Tensor> &inputs) {
  auto ins = op.tables(schema::CpuOp::f_ins), outs = op.tables(schema::CpuOp::f_outs);
  TTRT_ASSERT(inputs.size() == ins.size(),
              "CpuOp: input count mismatch: got " + std::to_string(inputs.size()) + ", expected " + std::to_string(ins.size()));
  WrappedFunc fn = cpuFunction(binary, programIndex, op.scalar<std::uint32_t>(schema::CpuOp::f_dylib_id, 0), std::string(op.string(schema::CpuOp::f_func_name)));
  std::vector<std::vector<std::int64_t>> sizesAndStrides;
  std::vector<WrappedTensor> packed;
  sizesAndStrides.reserve(ins.size());
  for (std::uint32_t i = 0; i < ins.size(); ++i) {
    const Tensor &t = inputs[i];
    TTRT_ASSERT(isTensorAllocated(t), "CpuOp: input " + std::to_string(i) + " is deallocated");
    // the compiler brings operands of a hoisted function to the host as dense row-major f32 / i32 / u32
    // (lib/Dialect/TTIR/Transforms/HoistCPUOps/HoistCPUOps.cpp:76-108); anything else here is a malformed program
    TTRT_ASSERT(t.handle->storage == StorageType::Host && t.handle->layout == TensorLayout::RowMajor,
                "CpuOp: input " + std::to_string(i) + " must be a row-major host tensor");
    TTRT_ASSERT(utils::dataTypeElementSize(t.handle->dtype) == 4, "CpuOp: input " + std::to_string(i) + " must have 4-byte elements");
    TTRT_ASSERT(t.handle->dtype == layoutFromTensorRef(ins[i]).dataType, "CpuOp: input " + std::to_string(i) + " has the wrong data type");
    const std::vector<std::uint32_t> shape = shapeFromTensorRef(ins[i]);
    TTRT_ASSERT(shape == t.handle->shape, "CpuOp: input " + std::to_string(i) + " has the wrong shape");
    std::vector<std::int64_t> ss(2 * shape.size());
    std::int64_t stride = 1;
    for (size_t d = shape.size(); d-- > 0;) {
      ss[d] = shape[d];
      ss[shape.size() + d] = stride;
      stride *= shape[d];
    }
    sizesAndStrides.push_back(std::move(ss));
    void *data = t.handle->data.get();
    packed.push_back(WrappedTensor{data, data, 0, sizesAndStrides.back().data()});
  }
  WrappedTensor *result = fn(packed.data());
  TTRT_ASSERT(result != nullptr || outs.size() == 0, "CpuOp: the function returned no outputs");
  std::vector<Tensor> outputs;
  std::map<void *, std::shared_ptr<void>> seen;   // outputs that alias one buffer share its owner
  for (std::uint32_t i = 0; i < outs.size(); ++i) {
    const WrappedTensor &w = result[i];
    const Layout lay = layoutFromTensorRef(outs[i]);
    TTRT_ASSERT(lay.dataType == DataType::Float32 || lay.dataType == DataType::UInt32 || lay.dataType == DataType::Int32,
                "Unsupported data type for CPU op output");
    auto t = std::make_shared<TensorImpl>();
    t->shape = shapeFromTensorRef(outs[i]);
    t->dtype = lay.dataType; t->layout = TensorLayout::RowMajor; t->storage = StorageType::Host;
    t->bytes = tensorBytes(t->shape, t->dtype, t->layout);
    auto it = seen.find(w.start);
    if (it == seen.end()) it = seen.emplace(w.start, std::shared_ptr<void>(w.alignedStart, [start = w.start](void *) { std::free(start); })).first;
    t->data = it->second;
    t->version = nextTensorVersion();
    outputs.push_back(Tensor{t});
  }
  if (outs.size() > 0) std::free(result[0].sizesAndStrides);   // one block for all outputs
  std::free(result);
  return outputs;
}

void runCpu(const fb::Table &op, ProgramContext &ctx) {
  auto ins = op.tables(schema::CpuOp::f_ins), outs = op.tables(schema::CpuOp::f_outs);
  std::vector<Tensor> inputs;   // held over the call
  for (std::uint32_t i = 0; i < ins.size(); ++i) inputs.push_back(ctx.get(ins[i], "cpu op input"));
  std::vector<Tensor> outputs = callCpuFunction(ctx.binary, ctx.programIndex, op, inputs);
  for (std::uint32_t i = 0; i < outs.size(); ++i) ctx.put(outs[i], outputs[i]);
}

// ---- traces (runtime/lib/ttnn/operations/trace/*.cpp): a trace is a HIP graph recorded on the device's stream
Tensor makeTraceIdTensor(std::uint32_t id) {
  Tensor t = makeHostTensor({}, DataType::UInt32, TensorLayout::RowMajor);
  std::memcpy(t.handle->data.get(), &id, sizeof(id));
  return t;
}
std::uint32_t traceIdOf(const Tensor &t) {
  TTRT_ASSERT(t.handle->storage == StorageType::Host && t.handle->dtype == DataType::UInt32 && t.handle->bytes >= 4,
              "Trace ID must be a UINT32 host scalar");
  std::uint32_t id = 0;
  std::memcpy(&id, t.handle->data.get(), sizeof(id));
  return id;
}
void runBeginTraceCapture(const fb::Table &op, ProgramContext &ctx) {
  std::uint32_t id = ctx.dev->nextTraceId++;
  beginTraceCapture(ctx.dev, id);
  ctx.put(op.table(schema::BeginTraceCaptureOp::f_trace_id), makeTraceIdTensor(id));
}
void runEndTraceCapture(const fb::Table &op, ProgramContext &ctx) {
  endTraceCapture(ctx.dev, traceIdOf(ctx.get(op.table(schema::EndTraceCaptureOp::f_trace_id), "end_trace_capture trace id")));
}
void runExecuteTrace(const fb::Table &op, ProgramContext &ctx) {
  executeTrace(ctx.dev, traceIdOf(ctx.get(op.table(schema::ExecuteTraceOp::f_trace_id), "execute_trace trace id")),
               op.scalar<std::uint8_t>(schema::ExecuteTraceOp::f_blocking, 0) != 0);
}

// dst <- src for tensors of one shape; src is brought to dst's layout and dtype first (on the device)
void overwriteTensor(ProgramContext &ctx, Tensor &dst, const Tensor &src, const char *what) {
  TTRT_ASSERT(dst.handle->shape == src.handle->shape, std::string(what) + ": shape mismatch");
  Tensor conv = src;
  if (conv.handle->layout != dst.handle->layout || conv.handle->dtype != dst.handle->dtype)
    conv = as(ctx, conv, dst.handle->layout, dst.handle->dtype);
  TTRT_ASSERT(conv.handle->bytes == dst.handle->bytes, std::string(what) + ": size mismatch");
  if (conv.handle->storage == StorageType::Device && dst.handle->storage == StorageType::Device)
    TTM_CALL(ttm_copy_kernel(conv.handle->data.get(), dst.handle->data.get(), dst.handle->bytes, ctx.stream()));
  else
    memcpy(dst, conv);
}
void runWriteTensor(const fb::Table &op, ProgramContext &ctx) {
  Tensor &host = ctx.get(op.table(schema::WriteTensorOp::f_host_tensor), "write_tensor host");
  Tensor &dev = ctx.get(op.table(schema::WriteTensorOp::f_device_tensor), "write_tensor device");
  TTRT_ASSERT(host.handle->storage == StorageType::Host && dev.handle->storage == StorageType::Device,
              "write_tensor: source must be on host and destination on device");
  overwriteTensor(ctx, dev, host, "write_tensor");
  dev.handle->version = host.handle->version;
}
void runCopy(const fb::Table &op, ProgramContext &ctx) {
  Tensor &src = ctx.get(op.table(schema::CopyOp::f_src), "copy src");
  Tensor &dst = ctx.get(op.table(schema::CopyOp::f_dst), "copy dst");
  overwriteTensor(ctx, dst, src, "copy");
}

bool inDeviceMemory(const fb::Table &ref) { return layoutFromTensorRef(ref).storageType == StorageType::Device; }

// Copies the current values of the op's inputs into the persistent input slots.  A slot that is its input's own memory
// (device-resident inputs pass through the allocation program) needs nothing; any other slot belongs to the trace and is
// overwritten when its version is not its input's.
void updateTraceInputSlots(const fb::Table &op, ProgramContext &ctx, std::vector<Tensor> &slots, bool deviceResidentOnly) {
  auto ins = op.tables(schema::CaptureOrExecuteTraceOp::f_inputs);
  TTRT_ASSERT(ins.size() == slots.size(), "capture_or_execute_trace: mismatched number of input slots");
  for (std::uint32_t i = 0; i < ins.size(); ++i) {
    const bool resident = inDeviceMemory(ins[i]);
    if (deviceResidentOnly && !resident) continue;
    Tensor &in = ctx.get(ins[i], "trace input");
    if (in.handle->data.get() == slots[i].handle->data.get()) continue;
    if (in.handle->version == slots[i].handle->version) continue;
    overwriteTensor(ctx, slots[i], in, "trace input slot");
    slots[i].handle->version = in.handle->version;
  }
}
void publishTraceOutputs(const fb::Table &op, ProgramContext &ctx, const std::vector<Tensor> &slots) {
  auto outs = op.tables(schema::CaptureOrExecuteTraceOp::f_outputs);
  TTRT_ASSERT(outs.size() == slots.size(), "capture_or_execute_trace: mismatched number of output slots");
  for (std::uint32_t i = 0; i < outs.size(); ++i) ctx.put(outs[i], slots[i]);
}
void runCaptureOrExecuteTrace(const fb::Table &op, ProgramContext &ctx) {
  const std::uint32_t captureId = op.scalar<std::uint32_t>(schema::CaptureOrExecuteTraceOp::f_capture_program_id, 0);
  const std::uint32_t executeId = op.scalar<std::uint32_t>(schema::CaptureOrExecuteTraceOp::f_execute_program_id, 0);
  const std::uint32_t allocateId = op.scalar<std::uint32_t>(schema::CaptureOrExecuteTraceOp::f_allocate_slots_program_id, 0);
  auto ins = op.tables(schema::CaptureOrExecuteTraceOp::f_inputs);
  auto outs = op.tables(schema::CaptureOrExecuteTraceOp::f_outputs);
  std::vector<const void *> residentAddresses;
  for (std::uint32_t i = 0; i < ins.size(); ++i)
    if (inDeviceMemory(ins[i])) residentAddresses.push_back(ctx.get(ins[i], "trace input").handle->data.get());
  TraceKey key{ctx.binary.id(), ctx.programIndex, captureId, executeId, residentAddresses};
  auto hit = ctx.dev->traceCache.find(key);
  if (hit == ctx.dev->traceCache.end()) {
    // allocate the persistent slots once: the allocation program takes the device-resident inputs (their own slots)
    // and returns the input slots followed by the output slots
    std::vector<Tensor> resident;
    for (std::uint32_t i = 0; i < ins.size(); ++i)
      if (inDeviceMemory(ins[i])) resident.push_back(ctx.get(ins[i], "trace input"));
    std::vector<Tensor> slots = executeProgram(ctx.dev, ctx.binary, allocateId, resident);
    TTRT_ASSERT(slots.size() == ins.size() + outs.size(), "capture_or_execute_trace: mismatched number of trace slots, expected " +
                                                              std::to_string(ins.size() + outs.size()) + " got " + std::to_string(slots.size()));
    for (Tensor &t : slots) setTensorRetain(t, true);
    std::vector<Tensor> inputSlots(slots.begin(), slots.begin() + ins.size()), outputSlots(slots.begin() + ins.size(), slots.end());
    updateTraceInputSlots(op, ctx, inputSlots, /*deviceResidentOnly=*/true);
    // capture program arguments: host-staged inputs, input slots, output slots; it returns the new trace id
    std::vector<Tensor> args;
    for (std::uint32_t i = 0; i < ins.size(); ++i)
      if (!inDeviceMemory(ins[i])) args.push_back(ctx.get(ins[i], "trace input"));
    args.insert(args.end(), inputSlots.begin(), inputSlots.end());
    args.insert(args.end(), outputSlots.begin(), outputSlots.end());
    std::vector<Tensor> ret = executeProgram(ctx.dev, ctx.binary, captureId, args);
    TTRT_ASSERT(ret.size() == 1, "Capture program must return exactly the new trace id");
    const std::uint32_t traceId = traceIdOf(ret[0]);
    auto it = ctx.dev->traces.find(traceId);
    TTRT_ASSERT(it != ctx.dev->traces.end(), "capture program returned a trace id that was not captured");
    // the capture program wrote the host inputs into their slots itself
    for (std::uint32_t i = 0; i < ins.size(); ++i)
      if (!inDeviceMemory(ins[i])) inputSlots[i].handle->version = ctx.get(ins[i], "trace input").handle->version;
    it->second.inputSlots = std::move(inputSlots);
    it->second.outputSlots = std::move(outputSlots);
    it->second.lastUse = ++ctx.dev->traceClock;
    ctx.dev->traceCache[key] = traceId;
    publishTraceOutputs(op, ctx, it->second.outputSlots);  // the capture program replayed the trace once
    debug::Stats::get().incrementStat("TraceCacheMiss");
    debug::Stats::get().incrementStat("CapturedTrace");
    // traces of this op recorded on other resident tensors: the caller may come back to them (weight sets that alternate),
    // but each keeps its slots and intermediates alive, so only the most recently used ones stay
    for (;;) {
      std::uint32_t oldest = 0, count = 0;
      std::uint64_t oldestUse = ~std::uint64_t(0);
      for (const auto &kv : ctx.dev->traceCache) {
        const TraceKey &k = kv.first;
        if (std::get<0>(k) != std::get<0>(key) || std::get<1>(k) != std::get<1>(key) || std::get<2>(k) != std::get<2>(key) ||
            std::get<3>(k) != std::get<3>(key))
          continue;
        ++count;
        const std::uint64_t use = ctx.dev->traces.at(kv.second).lastUse;
        if (use < oldestUse) { oldestUse = use; oldest = kv.second; }
      }
      if (count <= kMaxTracesPerOp) break;
      releaseTrace(ctx.dev, oldest);
      debug::Stats::get().incrementStat("ReleasedTrace");
    }
    return;
  }
  TraceData &td = ctx.dev->traces.at(hit->second);
  td.lastUse = ++ctx.dev->traceClock;
  updateTraceInputSlots(op, ctx, td.inputSlots, /*deviceResidentOnly=*/false);
  std::vector<Tensor> idArg{makeTraceIdTensor(td.traceId)};
  executeProgram(ctx.dev, ctx.binary, executeId, idArg);
  publishTraceOutputs(op, ctx, td.outputSlots);
  debug::Stats::get().incrementStat("ExecutedTrace");
}

void runOperation(const fb::Table &operation, ProgramContext &ctx) {
  auto type = static_cast<OpType>(operation.scalar<std::uint8_t>(schema::Operation::f_type_type, 0));
  fb::Table op = operation.table(schema::Operation::f_type);
  switch (type) {
  case OpType::GetDeviceOp: return;
  case OpType::ToLayoutOp: return runToLayout(op, ctx);
  case OpType::TypecastOp: return runTypecast(op, ctx);
  case OpType::ToDeviceOp: return runToDevice(op, ctx);
  case OpType::FromDeviceOp: return runFromDevice(op, ctx);
  case OpType::ToMemoryConfigOp: return runToMemoryConfig(op, ctx);
  case OpType::MatmulOp: return runMatmul(op, ctx);
  case OpType::LinearOp: return runLinear(op, ctx);
  case OpType::EltwiseUnaryOp: return runEltwiseUnary(op, ctx);
  case OpType::EltwiseBinaryOp: return runEltwiseBinary(op, ctx);
  case OpType::RMSNormOp: return runRmsNorm(op, ctx);
  case OpType::SoftmaxOp: return runSoftmax(op, ctx);
  case OpType::ReductionOp: return runReduction(op, ctx);
  case OpType::ScaledDotProductAttentionOp: return runSdpa(op, ctx);
  case OpType::ReshapeOp: return runReshape(op, ctx);
  case OpType::PermuteOp: return runPermute(op, ctx);
  case OpType::TransposeOp: return runTranspose(op, ctx);
  case OpType::ConcatOp: return runConcat(op, ctx);
  case OpType::SliceOp: return runSlice(op, ctx);
  case OpType::RepeatInterleaveOp: return runRepeatInterleave(op, ctx);
  case OpType::RepeatOp: return runRepeat(op, ctx);
  case OpType::ConcatenateHeadsOp: return runConcatenateHeads(op, ctx);
  case OpType::NLPConcatHeadsOp: return runNlpConcatHeads(op, ctx);
  case OpType::NLPConcatHeadsDecodeOp: return runNlpConcatHeadsDecode(op, ctx);
  case OpType::NLPCreateQKVHeadsDecodeOp: return runNlpCreateQkvHeadsDecode(op, ctx);
  case OpType::SplitQueryKeyValueAndSplitHeadsOp: return runSplitQkvAndSplitHeads(op, ctx);
  case OpType::EltwiseBinaryCompositeOp: return runEltwiseBinaryComposite(op, ctx);
  case OpType::EltwiseUnaryCompositeOp: return runEltwiseUnaryComposite(op, ctx);
  case OpType::EltwiseTernaryWhereOp: return runWhere(op, ctx);
  case OpType::EmbeddingOp: return runEmbedding(op, ctx);
  case OpType::ReductionArgMaxOp: return runArgMax(op, ctx);
  case OpType::ArangeOp: return runArange(op, ctx);
  case OpType::ConstantOp: return runConstant(op, ctx);
  case OpType::FullOp: return runFull(op, ctx);
  case OpType::NamedFullOp: return runNamedFull(op, ctx);
  case OpType::EmptyOp: return runEmpty(op, ctx);
  case OpType::DeallocateOp: return runDeallocate(op, ctx);
  case OpType::LoadCachedOp: return runLoadCached(op, ctx);
  case OpType::FuncCallOp: return runFuncCall(op, ctx);
  case OpType::CpuOp: return runCpu(op, ctx);
  case OpType::RotaryEmbeddingOp: return runRotaryEmbedding(op, ctx);
  case OpType::RotaryEmbeddingLlamaOp: return runRotaryEmbeddingLlama(op, ctx);
  case OpType::ChunkedScaledDotProductAttentionOp: return runChunkedSdpa(op, ctx);
  case OpType::UpdateCacheOp: return runUpdateCache(op, ctx);
  case OpType::PagedUpdateCacheOp: return runPagedUpdateCache(op, ctx);
  case OpType::PagedFillCacheOp: return runPagedFillCache(op, ctx);
  case OpType::FillCacheOp: return runFillCache(op, ctx);
  case OpType::ScaledDotProductAttentionDecodeOp: return runSdpaDecode(op, ctx);
  case OpType::PagedScaledDotProductAttentionDecodeOp: return runPagedSdpaDecode(op, ctx);
  case OpType::BeginTraceCaptureOp: return runBeginTraceCapture(op, ctx);
  case OpType::EndTraceCaptureOp: return runEndTraceCapture(op, ctx);
  case OpType::ExecuteTraceOp: return runExecuteTrace(op, ctx);
  case OpType::CaptureOrExecuteTraceOp: return runCaptureOrExecuteTrace(op, ctx);
  case OpType::WriteTensorOp: return runWriteTensor(op, ctx);
  case OpType::CopyOp: return runCopy(op, ctx);
  default: fatal(std::string("Unsupported operation type: ") + schema::opTypeName(type));
  }
}

// Per-operation profiler ranges: the reference opens a tracy zone per operation and sends its MLIR location as a message
// (runtime/lib/ttnn/program_executor.cpp:223-237); here each operation is a roctx range named "<OpType> <loc_info>", which
// rocprofv3 --marker-trace shows around the kernels the operation launched.  TTMLIR_RUNTIME_PROFILE_OPS=1 switches the
// ranges on (the marker library is loaded on first use); TTMLIR_RUNTIME_SYNC_AFTER_OP=1 also waits for the device at the
// end of every operation, which makes a range's duration the operation's own (the reference's TT_RUNTIME_SYNC_AFTER_OP).
struct Roctx {
  int (*push)(const char *) = nullptr;
  int (*pop)() = nullptr;
  bool ranges = false, sync = false;
  static Roctx &get() {
    static Roctx r = [] {
      Roctx x;
      const char *on = std::getenv("TTMLIR_RUNTIME_PROFILE_OPS"), *sy = std::getenv("TTMLIR_RUNTIME_SYNC_AFTER_OP");
      x.sync = sy && sy[0] == '1';
      if (on && on[0] == '1') {
        for (const char *name : {"libroctx64.so", "libroctx64.so.4", "librocprofiler-sdk-roctx.so"}) {
          if (void *h = ::dlopen(name, RTLD_LAZY | RTLD_GLOBAL)) {
            x.push = reinterpret_cast<int (*)(const char *)>(::dlsym(h, "roctxRangePushA"));
            x.pop = reinterpret_cast<int (*)()>(::dlsym(h, "roctxRangePop"));
            if (x.push && x.pop) break;
          }
        }
        x.ranges = x.push && x.pop;
        if (!x.ranges) std::fprintf(stderr, "[tt::runtime] TTMLIR_RUNTIME_PROFILE_OPS: no roctx library found, ranges are off\n");
      }
      return x;
    }();
    return r;
  }
};
struct OpRange {
  bool open = false;
  explicit OpRange(const fb::Table &op) {
    Roctx &r = Roctx::get();
    if (!r.ranges) return;
    const auto type = static_cast<OpType>(op.scalar<std::uint8_t>(schema::Operation::f_type_type, 0));
    const std::string name = std::string(schema::opTypeName(type)) + " " + std::string(op.string(schema::Operation::f_loc_info));
    r.push(name.c_str());
    open = true;
    debug::Stats::get().incrementStat("ProfiledOpRange");
  }
  void close(ProgramContext &ctx) {
    Roctx &r = Roctx::get();
    if (r.sync && !ctx.dev->capturing) TTM_CALL(ttm_stream_sync(ctx.stream()));
    if (open) r.pop();
    open = false;
  }
  ~OpRange() {
    if (open) Roctx::get().pop();   // an operation that threw
  }
};

}  // namespace

std::vector<Tensor> executeProgram(const std::shared_ptr<DeviceState> &dev, const Binary &binary, std::uint32_t programIndex,
                                   std::vector<Tensor> &inputs) {
  auto programs = binary.handle->root.tables(schema::TTNNBinary::f_programs);
  TTRT_ASSERT(programIndex < programs.size(), "submit: program index out of range");
  fb::Table program = programs[programIndex];
  ProgramContext ctx;
  ctx.dev = dev; ctx.binary = binary; ctx.programIndex = programIndex;
  auto ins = program.tables(schema::Program::f_inputs);
  TTRT_ASSERT(ins.size() == inputs.size(), "submit: program '" + std::string(program.string(schema::Program::f_name)) + "' expects " +
                                               std::to_string(ins.size()) + " inputs, got " + std::to_string(inputs.size()));
  for (std::uint32_t i = 0; i < ins.size(); ++i) {
    TTRT_ASSERT(isTensorAllocated(inputs[i]), "submit: input " + std::to_string(i) + " is deallocated");
    std::vector<std::uint32_t> want = shapeFromTensorRef(ins[i]);
    TTRT_ASSERT(want == inputs[i].handle->shape, "submit: input " + std::to_string(i) + " has the wrong shape");
    // callers must bring every input to the layout in the flatbuffer (docs/src/specs/runtime-stitching.md:50-66)
    TTRT_ASSERT(getTensorLayout(inputs[i]) == layoutFromTensorRef(ins[i]),
                "submit: input " + std::to_string(i) + " is not in the layout the program expects (use toLayout(getLayout(...)))");
    ctx.put(ins[i], inputs[i]);
  }
  auto ops = program.tables(schema::Program::f_operations);
  auto &hooks = debug::Hooks::get();
  // with callbacks registered every operation must leave its own output in the pool: no fusion then
  ctx.fuseViews = !hooks.preOperatorCallback && !hooks.postOperatorCallback;
  if (ctx.fuseViews) {
    for (std::uint32_t i = 0; i < ops.size(); ++i) {
      ctx.ops.push_back(ops[i]);
      if (static_cast<OpType>(ops[i].scalar<std::uint8_t>(schema::Operation::f_type_type, 0)) == OpType::DeallocateOp) continue;
      for (const auto &ref : opRefs(ops[i]).ins) ++ctx.uses[refId(ref)];
    }
    auto pouts = program.tables(schema::Program::f_outputs);
    for (std::uint32_t i = 0; i < pouts.size(); ++i) ++ctx.uses[refId(pouts[i])];
  }
  CallbackContext cc{&ctx};
  if (hooks.preProgramCallback) (*hooks.preProgramCallback)(binary, cc);
  for (std::uint32_t i = 0; i < ops.size(); ++i) {
    if (ctx.skip.count(i)) continue;   // folded into the operation before it
    ctx.opIndex = i;
    OpContext oc{ops[i], i};
    if (hooks.preOperatorCallback) (*hooks.preOperatorCallback)(binary, cc, oc);
    OpRange range(ops[i]);
    runOperation(ops[i], ctx);
    range.close(ctx);
    if (hooks.postOperatorCallback) (*hooks.postOperatorCallback)(binary, cc, oc);
  }
  if (hooks.postProgramCallback) (*hooks.postProgramCallback)(binary, cc);
  std::vector<Tensor> outputs;
  auto outs = program.tables(schema::Program::f_outputs);
  for (std::uint32_t i = 0; i < outs.size(); ++i) outputs.push_back(ctx.get(outs[i], "program output"));
  return outputs;
}

// ---- hook-side access to the running program (runtime/include/tt/runtime/runtime.h:246-297)
namespace {
std::vector<TensorRef> wrapRefs(const std::vector<fb::Table> &tables) {
  std::vector<TensorRef> out;
  for (const auto &t : tables) out.push_back(TensorRef{t});
  return out;
}
}  // namespace

std::vector<TensorRef> getOpOutputRefs(OpContext oc) { return wrapRefs(opRefs(oc.op).outs); }
std::vector<TensorRef> getOpInputRefs(OpContext oc) { return wrapRefs(opRefs(oc.op).ins); }
std::vector<std::uint32_t> getTensorRefShape(TensorRef ref) { return shapeFromTensorRef(ref.table); }
::tt::target::DataType getTensorRefDataType(TensorRef ref) { return layoutFromTensorRef(ref.table).dataType; }
std::uint32_t getTensorRefGlobalId(TensorRef ref) { return ref.table.scalar<std::uint32_t>(schema::TensorRef::f_global_id, 0); }
void walkProgram(Binary binary, std::uint32_t programIndex, const OpWalkFn &callback) {
  TTRT_ASSERT(binary.handle != nullptr, "walkProgram: null binary");
  auto programs = binary.handle->root.tables(schema::TTNNBinary::f_programs);
  TTRT_ASSERT(programIndex < programs.size(), "walkProgram: program index out of range");
  auto ops = programs[programIndex].tables(schema::Program::f_operations);
  for (std::uint32_t i = 0; i < ops.size(); ++i) callback(OpContext{ops[i], i});
}
std::vector<Tensor> invokeCpuOpOf(const Binary &binary, std::uint32_t programIndex, OpContext oc, const std::vector<Tensor> &inputs) {
  TTRT_ASSERT(binary.handle != nullptr, "invokeCpuOp: null binary");
  TTRT_ASSERT(programIndex < binary.handle->root.tables(schema::TTNNBinary::f_programs).size(), "invokeCpuOp: program index out of range");
  const auto type = static_cast<OpType>(oc.op.scalar<std::uint8_t>(schema::Operation::f_type_type, 0));
  TTRT_ASSERT(type == OpType::CpuOp, std::string("invokeCpuOp: opContext must wrap a CpuOp, got ") + schema::opTypeName(type));
  return callCpuFunction(binary, programIndex, oc.op.table(schema::Operation::f_type), inputs);
}
std::vector<Tensor> invokeCpuOp(CallbackContext cc, OpContext oc, const std::vector<Tensor> &inputs) {
  auto *ctx = static_cast<ProgramContext *>(cc.programContext);
  TTRT_ASSERT(ctx != nullptr, "invokeCpuOp: no program context");
  return invokeCpuOpOf(ctx->binary, static_cast<std::uint32_t>(ctx->programIndex), oc, inputs);
}
size_t getProgramIndex(CallbackContext cc) {
  auto *ctx = static_cast<ProgramContext *>(cc.programContext);
  TTRT_ASSERT(ctx != nullptr, "getProgramIndex: no program context");
  return ctx->programIndex;
}

std::unordered_map<std::uint32_t, Tensor> getOpOutputTensor(OpContext oc, CallbackContext cc) {
  std::unordered_map<std::uint32_t, Tensor> out;
  auto *ctx = static_cast<ProgramContext *>(cc.programContext);
  OpRefs refs = opRefs(oc.op);
  if (refs.outs.empty() || !ctx) return out;
  std::uint32_t id = refs.outs.front().scalar<std::uint32_t>(schema::TensorRef::f_global_id, 0);
  auto it = ctx->pool.find(id);
  if (it == ctx->pool.end() || !isTensorAllocated(it->second)) return out;
  out[0] = toHost(it->second, /*untilize=*/true)[0];
  return out;
}

std::optional<Tensor> retrieveTensorFromPool(CallbackContext cc, TensorRef ref, bool untilize) {
  return retrieveTensorFromPool(cc, getTensorRefGlobalId(ref), untilize);
}
void updateTensorInPool(CallbackContext cc, TensorRef ref, Tensor src) { updateTensorInPool(cc, getTensorRefGlobalId(ref), src); }

std::optional<Tensor> retrieveTensorFromPool(CallbackContext cc, std::uint32_t globalId, bool untilize) {
  auto *ctx = static_cast<ProgramContext *>(cc.programContext);
  if (!ctx) return std::nullopt;
  auto it = ctx->pool.find(globalId);
  if (it == ctx->pool.end() || !isTensorAllocated(it->second)) return std::nullopt;
  return toHost(it->second, untilize)[0];
}

void updateTensorInPool(CallbackContext cc, std::uint32_t globalId, Tensor src) {
  auto *ctx = static_cast<ProgramContext *>(cc.programContext);
  TTRT_ASSERT(ctx != nullptr, "updateTensorInPool: no program context");
  auto it = ctx->pool.find(globalId);
  TTRT_ASSERT(it != ctx->pool.end(), "updateTensorInPool: tensor is not in the pool");
  Tensor &dst = it->second;
  TTRT_ASSERT(dst.handle->shape == src.handle->shape, "updateTensorInPool: shape mismatch");
  // normalise the source to the destination's layout, then overwrite the payload in place
  Layout want = getTensorLayout(dst);
  Tensor conv = src;
  if (want.storageType == StorageType::Device || conv.handle->layout != want.layout || conv.handle->dtype != want.dataType)
    conv = convertOnDevice(conv.handle->storage == StorageType::Device ? conv : toDevice(conv, ctx->dev), want.layout, want.dataType);
  if (want.storageType == StorageType::Host && conv.handle->storage == StorageType::Device) conv = fromDevice(conv);
  memcpy(dst, conv);
  // new contents, new version (runtime/lib/ttnn/runtime.cpp:2588): a const-eval result or a trace slot computed from the
  // old contents no longer matches
  dst.handle->version = nextTensorVersion();
}

}  // namespace tt::runtime
