#include "program_builder.h"

#include <cmath>
#include <algorithm>

namespace ttmlir_amd {

using namespace schema;
using Off = fb::Builder::Off;
using ::tt::runtime::fatal;

ProgramBuilder::Id ProgramBuilder::newTensor(const Desc &d) {
  tensors_.push_back(d);
  if (declaredShape_) {
    tensors_.back().shape = *declaredShape_;
    declaredShape_.reset();
  }
  return static_cast<Id>(tensors_.size() - 1);
}

const ProgramBuilder::Desc &ProgramBuilder::desc(Id t) const {
  if (t == 0 || t >= tensors_.size()) fatal("ProgramBuilder: unknown tensor id " + std::to_string(t));
  return tensors_[t];
}

Off ProgramBuilder::memoryConfig(StorageType storage) {
  b_.startTable(MemoryConfig::kNumFields);
  b_.addScalarDefault<std::uint16_t>(MemoryConfig::f_tensor_memory_layout, static_cast<std::uint16_t>(TensorMemoryLayout::Interleaved), 0);
  b_.addScalarDefault<std::uint16_t>(MemoryConfig::f_buffer_type,
                                     static_cast<std::uint16_t>(storage == StorageType::Device ? BufferType::DRAM : BufferType::SystemMemory), 0);
  return b_.endTable();
}

Off ProgramBuilder::tensorRef(Id t) {
  const Desc &d = desc(t);
  std::vector<std::int32_t> shape(d.shape.begin(), d.shape.end());
  Off shapeOff = b_.createScalarVector(shape);
  Off memcfg = memoryConfig(d.storage);
  b_.startTable(MemoryDesc::kNumFields);
  b_.addScalarDefault<std::uint16_t>(MemoryDesc::f_storage_type, static_cast<std::uint16_t>(d.storage), 0);
  std::int32_t tile[2] = {d.layout == TensorLayout::Tile ? 32 : 1, d.layout == TensorLayout::Tile ? 32 : 1};
  b_.addStruct(MemoryDesc::f_tile_shape, tile, sizeof(tile), 4);
  b_.addScalarDefault<std::uint16_t>(MemoryDesc::f_data_type, static_cast<std::uint16_t>(d.dtype), 0);
  b_.addOffset(MemoryDesc::f_memory_config, memcfg);
  Off md = b_.endTable();
  b_.startTable(LayoutDesc::kNumFields);
  b_.addScalarDefault<std::uint16_t>(LayoutDesc::f_oob_val, static_cast<std::uint16_t>(OOBVal::Undef), 0);
  b_.addOffset(LayoutDesc::f_memory_desc, md);
  Off ld = b_.endTable();
  b_.startTable(TensorDesc::kNumFields);
  b_.addOffset(TensorDesc::f_shape, shapeOff);
  b_.addOffset(TensorDesc::f_layout, ld);
  b_.addScalarDefault<std::uint32_t>(TensorDesc::f_shard_status, static_cast<std::uint32_t>(ShardStatus::Unsharded), 0);
  Off td = b_.endTable();
  b_.startTable(TensorRef::kNumFields);
  b_.addScalarDefault<std::uint32_t>(TensorRef::f_global_id, t, 0);
  b_.addOffset(TensorRef::f_desc, td);
  return b_.endTable();
}

void ProgramBuilder::addOp(OpType type, Off table, const std::string &debug) {
  if (!open_) fatal("ProgramBuilder: no program is open");
  cur_.ops.push_back(OpRec{static_cast<std::uint8_t>(type), table, debug});
}

static std::string opLoc(const std::string &program, std::uint32_t index) {
  return "loc(\"" + program + "\"(\"op" + std::to_string(index) + "\"))";
}

std::string ProgramBuilder::lastOpLoc() const {
  if (!open_ || cur_.ops.empty()) fatal("ProgramBuilder: no operation to name");
  return opLoc(cur_.name, static_cast<std::uint32_t>(cur_.ops.size() - 1));
}

void ProgramBuilder::golden(const std::string &loc, const std::string &name, const void *data, size_t bytes,
                            const std::vector<std::int64_t> &shape, DataType dtype) {
  if (!open_) fatal("ProgramBuilder: no program is open");
  std::uint64_t volume = 1;
  for (std::int64_t d : shape) {
    if (d < 0) fatal("ProgramBuilder: golden tensor has a negative dimension");
    volume *= static_cast<std::uint64_t>(d);
  }
  if (::tt::runtime::utils::isBlockFormatDataType(dtype))
    fatal("ProgramBuilder: golden tensors hold plain element types, not block-float tiles");
  const std::uint32_t elem = ::tt::runtime::utils::dataTypeElementSize(dtype);
  if (volume * elem != bytes)
    fatal("ProgramBuilder: golden tensor of " + std::to_string(bytes) + " bytes does not match its shape and dtype (" +
          std::to_string(volume * elem) + " bytes)");
  std::vector<std::int64_t> stride(shape.size(), 1);
  for (int d = static_cast<int>(shape.size()) - 2; d >= 0; --d) stride[d] = stride[d + 1] * shape[d + 1];
  Off nameOff = b_.createString(name);
  Off shapeOff = b_.createScalarVector(shape), strideOff = b_.createScalarVector(stride);
  Off dataOff = b_.createScalarVector(static_cast<const std::uint8_t *>(data), bytes);
  b_.startTable(GoldenTensor::kNumFields);
  b_.addOffset(GoldenTensor::f_name, nameOff);
  b_.addOffset(GoldenTensor::f_shape, shapeOff);
  b_.addOffset(GoldenTensor::f_stride, strideOff);
  b_.addScalar<std::uint16_t>(GoldenTensor::f_dtype, static_cast<std::uint16_t>(dtype));
  b_.addOffset(GoldenTensor::f_data, dataOff);
  Off gt = b_.endTable();
  b_.startTable(GoldenDeviceTensor::kNumFields);
  b_.addScalarDefault<std::uint32_t>(GoldenDeviceTensor::f_device, 0, 0);
  b_.addOffset(GoldenDeviceTensor::f_value, gt);
  cur_.goldens.emplace_back(loc, b_.endTable());
}

void ProgramBuilder::beginProgram(const std::string &name, bool isPrivate) {
  if (open_) fatal("ProgramBuilder: a program is already open");
  cur_ = ProgramRec{};
  cur_.name = name;
  cur_.isPrivate = isPrivate;
  open_ = true;
}

ProgramBuilder::Id ProgramBuilder::input(const std::vector<std::uint32_t> &shape, DataType dtype, TensorLayout layout, StorageType storage) {
  Id t = newTensor(Desc{shape, dtype, layout, storage});
  cur_.inputs.push_back(t);
  return t;
}
void ProgramBuilder::output(Id t) {
  desc(t);
  cur_.outputs.push_back(t);
}

std::uint32_t ProgramBuilder::endProgram() {
  if (!open_) fatal("ProgramBuilder: no program is open");
  std::vector<Off> ops;
  std::uint32_t opIndex = 0;
  for (const OpRec &r : cur_.ops) {
    Off dbg = b_.createString(r.debug);
    Off loc = b_.createString(opLoc(cur_.name, opIndex++));
    b_.startTable(Operation::kNumFields);
    b_.addScalar<std::uint8_t>(Operation::f_type_type, r.type);
    b_.addOffset(Operation::f_type, r.table);
    b_.addOffset(Operation::f_debug_info, dbg);
    b_.addOffset(Operation::f_loc_info, loc);
    ops.push_back(b_.endTable());
  }
  std::vector<Off> ins, outs;
  for (Id t : cur_.inputs) ins.push_back(tensorRef(t));
  for (Id t : cur_.outputs) outs.push_back(tensorRef(t));
  Off opsV = b_.createOffsetVector(ops), insV = b_.createOffsetVector(ins), outsV = b_.createOffsetVector(outs);
  Off name = b_.createString(cur_.name);
  Off debugInfo = 0;
  if (!cur_.goldens.empty()) {
    // one GoldenKV per location, each with the single device-0 tensor
    std::vector<Off> kvs;
    for (const auto &g : cur_.goldens) {
      Off key = b_.createString(g.first);
      Off vals = b_.createOffsetVector(std::vector<Off>{g.second});
      b_.startTable(GoldenKV::kNumFields);
      b_.addOffset(GoldenKV::f_key, key);
      b_.addOffset(GoldenKV::f_value, vals);
      kvs.push_back(b_.endTable());
    }
    Off map = b_.createOffsetVector(kvs);
    b_.startTable(GoldenInfo::kNumFields);
    b_.addOffset(GoldenInfo::f_golden_map, map);
    Off info = b_.endTable();
    b_.startTable(DebugInfo::kNumFields);
    b_.addOffset(DebugInfo::f_golden_info, info);
    debugInfo = b_.endTable();
  }
  Off dylibsV = cur_.dylibs.empty() ? 0 : b_.createOffsetVector(cur_.dylibs);
  b_.startTable(Program::kNumFields);
  if (debugInfo) b_.addOffset(Program::f_debug_info, debugInfo);
  if (dylibsV) b_.addOffset(Program::f_dylibs, dylibsV);
  b_.addOffset(Program::f_name, name);
  b_.addOffset(Program::f_inputs, insV);
  b_.addOffset(Program::f_outputs, outsV);
  b_.addOffset(Program::f_operations, opsV);
  b_.addScalarDefault<std::uint8_t>(Program::f_private, cur_.isPrivate ? 1 : 0, 0);
  std::int32_t mesh[2] = {1, 1};
  b_.addStruct(Program::f_mesh_shape, mesh, sizeof(mesh), 4);
  finishedPrograms_.push_back(b_.endTable());
  open_ = false;
  return static_cast<std::uint32_t>(finishedPrograms_.size() - 1);
}

std::vector<std::uint8_t> ProgramBuilder::finish() {
  if (open_) fatal("ProgramBuilder: a program is still open");
  Off programs = b_.createOffsetVector(finishedPrograms_);
  Off hash = b_.createString("mi355x-native-writer");  // not reproducible without flatc; readers here never enforce it
  Off git = b_.createString("0000000000000000000000000000000000000000");
  b_.startTable(TTNNBinary::kNumFields);
  struct { std::uint16_t major, minor; std::uint32_t patch; } ver{0, 1, 0};
  b_.addStruct(TTNNBinary::f_version, &ver, sizeof(ver), 4);
  b_.addOffset(TTNNBinary::f_schema_hash, hash);
  b_.addOffset(TTNNBinary::f_ttmlir_git_hash, git);
  b_.addOffset(TTNNBinary::f_programs, programs);
  Off root = b_.endTable();
  return b_.finishSizePrefixed(root, "TTNN");
}

// ------------------------------------------------------------------------------------ ops
static std::string shapeStr(const std::vector<std::uint32_t> &s) {
  std::string o = "[";
  for (size_t i = 0; i < s.size(); ++i) o += (i ? "x" : "") + std::to_string(s[i]);
  return o + "]";
}

ProgramBuilder::Id ProgramBuilder::toLayout(Id in, TensorLayout layout, int dtype, StorageType storage) {
  Desc d = desc(in);
  d.layout = layout;
  d.storage = storage;
  if (dtype >= 0) d.dtype = static_cast<DataType>(dtype);
  Id out = newTensor(d);
  Off i = tensorRef(in), o = tensorRef(out), mc = memoryConfig(storage);
  b_.startTable(ToLayoutOp::kNumFields);
  b_.addOffset(ToLayoutOp::f_in, i);
  b_.addScalarDefault<std::uint16_t>(ToLayoutOp::f_layout, static_cast<std::uint16_t>(layout), 0);
  if (dtype >= 0) b_.addScalar<std::uint16_t>(ToLayoutOp::f_dtype, static_cast<std::uint16_t>(dtype));
  b_.addOffset(ToLayoutOp::f_memcfg, mc);
  b_.addOffset(ToLayoutOp::f_out, o);
  addOp(OpType::ToLayoutOp, b_.endTable(), "ttnn.to_layout " + shapeStr(d.shape));
  return out;
}
ProgramBuilder::Id ProgramBuilder::typecast(Id in, DataType dtype) {
  Desc d = desc(in);
  d.dtype = dtype;
  if (::tt::runtime::utils::isBlockFormatDataType(dtype)) d.layout = TensorLayout::Tile;
  Id out = newTensor(d);
  Off i = tensorRef(in), o = tensorRef(out);
  b_.startTable(TypecastOp::kNumFields);
  b_.addOffset(TypecastOp::f_in, i);
  b_.addScalarDefault<std::uint16_t>(TypecastOp::f_dtype, static_cast<std::uint16_t>(dtype), 0);
  b_.addOffset(TypecastOp::f_out, o);
  addOp(OpType::TypecastOp, b_.endTable(), std::string("ttnn.typecast -> ") + ::tt::runtime::utils::dataTypeName(dtype));
  return out;
}
ProgramBuilder::Id ProgramBuilder::toDevice(Id in) {
  Desc d = desc(in);
  d.storage = StorageType::Device;
  Id out = newTensor(d);
  Off i = tensorRef(in), o = tensorRef(out);
  b_.startTable(DeviceRef::kNumFields);
  Off dev = b_.endTable();
  b_.startTable(ToDeviceOp::kNumFields);
  b_.addOffset(ToDeviceOp::f_in, i);
  b_.addOffset(ToDeviceOp::f_device, dev);
  b_.addOffset(ToDeviceOp::f_out, o);
  addOp(OpType::ToDeviceOp, b_.endTable(), "ttnn.to_device");
  return out;
}
ProgramBuilder::Id ProgramBuilder::fromDevice(Id in) {
  Desc d = desc(in);
  d.storage = StorageType::Host;
  Id out = newTensor(d);
  Off i = tensorRef(in), o = tensorRef(out);
  b_.startTable(FromDeviceOp::kNumFields);
  b_.addOffset(FromDeviceOp::f_in, i);
  b_.addOffset(FromDeviceOp::f_out, o);
  addOp(OpType::FromDeviceOp, b_.endTable(), "ttnn.from_device");
  return out;
}

static std::vector<std::uint32_t> matmulShape(const std::vector<std::uint32_t> &a, const std::vector<std::uint32_t> &b, bool ta, bool tb) {
  if (a.size() < 2 || b.size() < 2) fatal("ProgramBuilder: matmul operands must have rank >= 2");
  std::uint32_t M = ta ? a[a.size() - 1] : a[a.size() - 2], K = ta ? a[a.size() - 2] : a[a.size() - 1];
  std::uint32_t Kb = tb ? b[b.size() - 1] : b[b.size() - 2], N = tb ? b[b.size() - 2] : b[b.size() - 1];
  if (K != Kb) fatal("ProgramBuilder: matmul inner dimensions differ");
  std::vector<std::uint32_t> out(a.begin(), a.end() - 2);
  if (b.size() > a.size()) out.assign(b.begin(), b.end() - 2);
  out.push_back(M);
  out.push_back(N);
  return out;
}

void ProgramBuilder::setMatmulProgramConfig(int kind, int fusedActivation) {
  if (kind < 0 || kind > static_cast<int>(MatmulProgramConfig::MatmulMultiCoreReuseMultiCastDRAMShardedProgramConfig))
    fatal("ProgramBuilder: unknown matmul program config kind " + std::to_string(kind));
  pendingMatmulConfig_ = kind;
  pendingFusedActivation_ = fusedActivation;
}

// the program config table of the next matmul / linear (include/ttmlir/Target/TTNN/operations/matmul.fbs:5-62); only the
// fields the runtime reads are written: the fused activation
Off ProgramBuilder::takeMatmulProgramConfig(std::uint8_t *kindOut) {
  const auto kind = static_cast<MatmulProgramConfig>(pendingMatmulConfig_);
  *kindOut = static_cast<std::uint8_t>(pendingMatmulConfig_);
  const int fused = pendingFusedActivation_;
  pendingMatmulConfig_ = 0;
  pendingFusedActivation_ = -1;
  if (kind == MatmulProgramConfig::NONE) return 0;
  int numFields = MatmulMultiCoreReuseProgramConfig::kNumFields, fusedSlot = -1;
  switch (kind) {
  case MatmulProgramConfig::MatmulMultiCoreReuseMultiCastProgramConfig:
    numFields = MatmulMultiCoreReuseMultiCastProgramConfig::kNumFields;
    fusedSlot = MatmulMultiCoreReuseMultiCastProgramConfig::f_fused_activation; break;
  case MatmulProgramConfig::MatmulMultiCoreReuseMultiCast1DProgramConfig:
    numFields = MatmulMultiCoreReuseMultiCast1DProgramConfig::kNumFields;
    fusedSlot = MatmulMultiCoreReuseMultiCast1DProgramConfig::f_fused_activation; break;
  case MatmulProgramConfig::MatmulMultiCoreReuseMultiCastDRAMShardedProgramConfig:
    numFields = MatmulMultiCoreReuseMultiCastDRAMShardedProgramConfig::kNumFields;
    fusedSlot = MatmulMultiCoreReuseMultiCastDRAMShardedProgramConfig::f_fused_activation; break;
  default: break;
  }
  Off unary = 0;
  if (fused >= 0 && fusedSlot >= 0) {
    b_.startTable(UnaryWithParam::kNumFields);
    b_.addScalar<std::uint32_t>(UnaryWithParam::f_op_type, static_cast<std::uint32_t>(fused));
    unary = b_.endTable();
  }
  b_.startTable(numFields);
  if (unary) b_.addOffset(fusedSlot, unary);
  return b_.endTable();
}

ProgramBuilder::Id ProgramBuilder::matmul(Id a, Id b, bool ta, bool tb, const std::string &activation, DataType outDtype) {
  Desc d{matmulShape(desc(a).shape, desc(b).shape, ta, tb), outDtype, TensorLayout::Tile, StorageType::Device};
  Id out = newTensor(d);
  Off ar = tensorRef(a), br = tensorRef(b), orf = tensorRef(out);
  Off act = activation.empty() ? 0 : b_.createString(activation);
  std::uint8_t configKind = 0;
  Off config = takeMatmulProgramConfig(&configKind);
  b_.startTable(MatmulOp::kNumFields);
  b_.addOffset(MatmulOp::f_a, ar);
  b_.addOffset(MatmulOp::f_b, br);
  b_.addOffset(MatmulOp::f_out, orf);
  b_.addScalarDefault<std::uint8_t>(MatmulOp::f_transpose_a, ta, 0);
  b_.addScalarDefault<std::uint8_t>(MatmulOp::f_transpose_b, tb, 0);
  b_.addScalarDefault<std::uint8_t>(MatmulOp::f_matmul_program_config_type, configKind, 0);
  b_.addOffset(MatmulOp::f_matmul_program_config, config);
  b_.addOffset(MatmulOp::f_activation, act);
  addOp(OpType::MatmulOp, b_.endTable(), "ttnn.matmul " + shapeStr(desc(a).shape) + " x " + shapeStr(desc(b).shape));
  return out;
}
ProgramBuilder::Id ProgramBuilder::linear(Id a, Id b, Id bias, bool ta, bool tb, const std::string &activation, DataType outDtype) {
  Desc d{matmulShape(desc(a).shape, desc(b).shape, ta, tb), outDtype, TensorLayout::Tile, StorageType::Device};
  Id out = newTensor(d);
  Off ar = tensorRef(a), br = tensorRef(b), bi = bias ? tensorRef(bias) : 0, orf = tensorRef(out);
  Off act = activation.empty() ? 0 : b_.createString(activation);
  b_.startTable(DeviceComputeKernelConfig::kNumFields);
  b_.addScalar<std::uint8_t>(DeviceComputeKernelConfig::f_math_fidelity, static_cast<std::uint8_t>(MathFidelity::HiFi4));
  b_.addScalar<std::uint8_t>(DeviceComputeKernelConfig::f_fp32_dest_acc_en, 1);
  Off cc = b_.endTable();
  std::uint8_t configKind = 0;
  Off config = takeMatmulProgramConfig(&configKind);
  b_.startTable(LinearOp::kNumFields);
  b_.addOffset(LinearOp::f_a, ar);
  b_.addOffset(LinearOp::f_b, br);
  b_.addOffset(LinearOp::f_bias, bi);
  b_.addOffset(LinearOp::f_out, orf);
  b_.addScalarDefault<std::uint8_t>(LinearOp::f_transpose_a, ta, 0);
  b_.addScalarDefault<std::uint8_t>(LinearOp::f_transpose_b, tb, 0);
  b_.addScalarDefault<std::uint8_t>(LinearOp::f_matmul_program_config_type, configKind, 0);
  b_.addOffset(LinearOp::f_matmul_program_config, config);
  b_.addOffset(LinearOp::f_activation, act);
  b_.addOffset(LinearOp::f_compute_config, cc);
  addOp(OpType::LinearOp, b_.endTable(), "ttnn.linear " + shapeStr(desc(a).shape) + " x " + shapeStr(desc(b).shape) + (activation.empty() ? "" : " + " + activation));
  return out;
}

ProgramBuilder::Id ProgramBuilder::unary(std::uint32_t type, Id in, bool hasParam, float param) {
  Desc d = desc(in);
  d.storage = StorageType::Device;
  Id out = newTensor(d);
  Off i = tensorRef(in), o = tensorRef(out), prm = 0;
  if (hasParam) {
    b_.startTable(EltwiseOpWithFloatParams::kNumFields);
    b_.addScalar<float>(EltwiseOpWithFloatParams::f_parameter, param);
    prm = b_.endTable();
  }
  b_.startTable(EltwiseUnaryOp::kNumFields);
  b_.addScalarDefault<std::uint32_t>(EltwiseUnaryOp::f_type, type, 0);
  b_.addOffset(EltwiseUnaryOp::f_in, i);
  b_.addOffset(EltwiseUnaryOp::f_out, o);
  if (prm) {
    b_.addScalar<std::uint8_t>(EltwiseUnaryOp::f_params_type, static_cast<std::uint8_t>(EltwiseUnaryOpParams::EltwiseOpWithFloatParams));
    b_.addOffset(EltwiseUnaryOp::f_params, prm);
  }
  addOp(OpType::EltwiseUnaryOp, b_.endTable(), "ttnn.unary#" + std::to_string(type));
  return out;
}

ProgramBuilder::Id ProgramBuilder::unaryComposite(std::uint32_t type, Id in, float lo, float hi, bool intBounds) {
  Desc d = desc(in);
  d.storage = StorageType::Device;
  Id out = newTensor(d);
  Off i = tensorRef(in), o = tensorRef(out), prm = 0;
  if (type == static_cast<std::uint32_t>(EltwiseUnaryCompositeOpType::ClampScalar)) {
    auto number = [&](float v) {
      if (intBounds) {
        b_.startTable(IntegralType::kNumFields);
        b_.addScalar<std::int32_t>(IntegralType::f_value, static_cast<std::int32_t>(v));
      } else {
        b_.startTable(FloatingPointType::kNumFields);
        b_.addScalar<float>(FloatingPointType::f_value, v);
      }
      return b_.endTable();
    };
    Off mn = number(lo), mx = number(hi);
    const std::uint8_t kind = static_cast<std::uint8_t>(intBounds ? NumberType::I32 : NumberType::FP);
    b_.startTable(ClampScalarOpParams::kNumFields);
    b_.addScalar<std::uint8_t>(ClampScalarOpParams::f_min_type, kind);
    b_.addOffset(ClampScalarOpParams::f_min, mn);
    b_.addScalar<std::uint8_t>(ClampScalarOpParams::f_max_type, kind);
    b_.addOffset(ClampScalarOpParams::f_max, mx);
    prm = b_.endTable();
  }
  b_.startTable(EltwiseUnaryCompositeOp::kNumFields);
  b_.addScalarDefault<std::uint32_t>(EltwiseUnaryCompositeOp::f_type, type, 0);
  b_.addOffset(EltwiseUnaryCompositeOp::f_in, i);
  b_.addOffset(EltwiseUnaryCompositeOp::f_out, o);
  if (prm) {
    b_.addScalar<std::uint8_t>(EltwiseUnaryCompositeOp::f_params_type, static_cast<std::uint8_t>(EltwiseUnaryCompositeOpParams::ClampScalarOpParams));
    b_.addOffset(EltwiseUnaryCompositeOp::f_params, prm);
  }
  addOp(OpType::EltwiseUnaryCompositeOp, b_.endTable(), "ttnn.unary_composite#" + std::to_string(type));
  return out;
}

ProgramBuilder::Id ProgramBuilder::binary(std::uint32_t type, Id lhs, Id rhs) {
  const auto &a = desc(lhs).shape, &b = desc(rhs).shape;
  size_t rank = std::max(a.size(), b.size());
  std::vector<std::uint32_t> shape(rank);
  for (size_t i = 0; i < rank; ++i) {
    std::uint32_t x = i < rank - a.size() ? 1 : a[i - (rank - a.size())], y = i < rank - b.size() ? 1 : b[i - (rank - b.size())];
    if (x != y && x != 1 && y != 1) fatal("ProgramBuilder: binary operands do not broadcast");
    shape[i] = std::max(x, y);
  }
  Desc d{shape, desc(lhs).dtype, desc(lhs).layout, StorageType::Device};
  Id out = newTensor(d);
  Off l = tensorRef(lhs), r = tensorRef(rhs), o = tensorRef(out);
  b_.startTable(EltwiseBinaryOp::kNumFields);
  b_.addScalarDefault<std::uint32_t>(EltwiseBinaryOp::f_type, type, 0);
  b_.addOffset(EltwiseBinaryOp::f_lhs, l);
  b_.addOffset(EltwiseBinaryOp::f_rhs, r);
  b_.addOffset(EltwiseBinaryOp::f_out, o);
  addOp(OpType::EltwiseBinaryOp, b_.endTable(), "ttnn.binary#" + std::to_string(type));
  return out;
}

ProgramBuilder::Id ProgramBuilder::rmsNorm(Id in, Id weight, Id bias, float eps) {
  Desc d = desc(in);
  d.storage = StorageType::Device;
  d.layout = TensorLayout::Tile;
  Id out = newTensor(d);
  Off i = tensorRef(in), w = weight ? tensorRef(weight) : 0, bi = bias ? tensorRef(bias) : 0, o = tensorRef(out);
  b_.startTable(RMSNormOp::kNumFields);
  b_.addOffset(RMSNormOp::f_input, i);
  b_.addOffset(RMSNormOp::f_weight, w);
  b_.addOffset(RMSNormOp::f_bias, bi);
  b_.addScalar<float>(RMSNormOp::f_epsilon, eps);
  b_.addOffset(RMSNormOp::f_out, o);
  addOp(OpType::RMSNormOp, b_.endTable(), "ttnn.rms_norm " + shapeStr(d.shape));
  return out;
}

ProgramBuilder::Id ProgramBuilder::softmax(Id in, int dim) {
  Desc d = desc(in);
  d.storage = StorageType::Device;
  d.layout = TensorLayout::Tile;
  Id out = newTensor(d);
  Off i = tensorRef(in), o = tensorRef(out);
  b_.startTable(SoftmaxOp::kNumFields);
  b_.addOffset(SoftmaxOp::f_in, i);
  b_.addOffset(SoftmaxOp::f_out, o);
  b_.addScalarDefault<std::int32_t>(SoftmaxOp::f_dimension, dim, 0);
  b_.addScalarDefault<std::uint8_t>(SoftmaxOp::f_numeric_stable, 1, 0);
  addOp(OpType::SoftmaxOp, b_.endTable(), "ttnn.softmax dim=" + std::to_string(dim));
  return out;
}

ProgramBuilder::Id ProgramBuilder::reduction(std::uint32_t type, Id in, const std::vector<int> &dims, bool keepDim) {
  Desc d = desc(in);
  int rank = static_cast<int>(d.shape.size());
  std::vector<bool> red(rank, dims.empty());
  for (int x : dims) red.at(x < 0 ? x + rank : x) = true;
  std::vector<std::uint32_t> shape;
  for (int i = 0; i < rank; ++i) {
    if (!red[i]) shape.push_back(d.shape[i]);
    else if (keepDim) shape.push_back(1);
  }
  Desc od{shape, d.dtype, TensorLayout::Tile, StorageType::Device};
  Id out = newTensor(od);
  Off i = tensorRef(in), o = tensorRef(out);
  std::vector<std::int32_t> dv(dims.begin(), dims.end());
  Off dimsOff = b_.createScalarVector(dv);
  b_.startTable(ReductionOp::kNumFields);
  b_.addScalarDefault<std::uint32_t>(ReductionOp::f_type, type, 0);
  b_.addOffset(ReductionOp::f_in, i);
  b_.addOffset(ReductionOp::f_out, o);
  b_.addOffset(ReductionOp::f_dim_arg, dimsOff);
  b_.addScalarDefault<std::uint8_t>(ReductionOp::f_keep_dim, keepDim, 0);
  addOp(OpType::ReductionOp, b_.endTable(), "ttnn.reduction#" + std::to_string(type));
  return out;
}

ProgramBuilder::Id ProgramBuilder::sdpa(Id q, Id k, Id v, Id mask, bool causal, bool hasScale, float scale, std::int64_t slidingWindow,
                                        Id sink) {
  Desc d = desc(q);
  d.storage = StorageType::Device;
  d.layout = TensorLayout::Tile;
  Id out = newTensor(d);
  using S = ScaledDotProductAttentionOp;
  Off qr = tensorRef(q), kr = tensorRef(k), vr = tensorRef(v), mr = mask ? tensorRef(mask) : 0, o = tensorRef(out);
  Off sr = sink ? tensorRef(sink) : 0;
  b_.startTable(S::kNumFields);
  b_.addOffset(S::f_query, qr);
  b_.addOffset(S::f_key, kr);
  b_.addOffset(S::f_value, vr);
  b_.addScalarDefault<std::uint8_t>(S::f_is_causal, causal, 0);
  b_.addOffset(S::f_attention_mask, mr);
  if (hasScale) b_.addScalar<float>(S::f_scale, scale);
  if (slidingWindow >= 0) b_.addScalar<std::uint32_t>(S::f_sliding_window_size, static_cast<std::uint32_t>(slidingWindow));
  b_.addOffset(S::f_attention_sink, sr);
  b_.addOffset(S::f_out, o);
  addOp(OpType::ScaledDotProductAttentionOp, b_.endTable(), "ttnn.scaled_dot_product_attention " + shapeStr(d.shape));
  return out;
}

ProgramBuilder::Id ProgramBuilder::rotaryEmbedding(Id in, Id cosCache, Id sinCache, bool hasTokenIndex, std::uint32_t tokenIndex) {
  Desc d = desc(in);
  d.storage = StorageType::Device;
  d.layout = TensorLayout::Tile;
  Id out = newTensor(d);
  using S = RotaryEmbeddingOp;
  Off i = tensorRef(in), c = tensorRef(cosCache), sn = tensorRef(sinCache), o = tensorRef(out);
  b_.startTable(S::kNumFields);
  b_.addOffset(S::f_input, i);
  b_.addOffset(S::f_cos_cache, c);
  b_.addOffset(S::f_sin_cache, sn);
  if (hasTokenIndex) b_.addScalar<std::uint32_t>(S::f_token_index, tokenIndex);
  b_.addOffset(S::f_out, o);
  addOp(OpType::RotaryEmbeddingOp, b_.endTable(), "ttnn.rotary_embedding " + shapeStr(d.shape));
  return out;
}
void ProgramBuilder::updateCache(Id cache, Id in, Id updateIndex, std::uint32_t batchOffset) {
  Off c = tensorRef(cache), i = tensorRef(in), u = tensorRef(updateIndex);
  b_.startTable(UpdateCacheOp::kNumFields);
  b_.addOffset(UpdateCacheOp::f_cache, c);
  b_.addOffset(UpdateCacheOp::f_input, i);
  b_.addOffset(UpdateCacheOp::f_update_index, u);
  b_.addScalarDefault<std::uint32_t>(UpdateCacheOp::f_batch_offset, batchOffset, 0);
  addOp(OpType::UpdateCacheOp, b_.endTable(), "ttnn.update_cache");
}
void ProgramBuilder::fillCache(Id cache, Id in, std::uint32_t batchOffset) {
  Off c = tensorRef(cache), i = tensorRef(in);
  b_.startTable(FillCacheOp::kNumFields);
  b_.addOffset(FillCacheOp::f_cache, c);
  b_.addOffset(FillCacheOp::f_input, i);
  b_.addScalarDefault<std::uint32_t>(FillCacheOp::f_batch_offset, batchOffset, 0);
  addOp(OpType::FillCacheOp, b_.endTable(), "ttnn.fill_cache");
}
void ProgramBuilder::pagedUpdateCache(Id cache, Id in, Id updateIndex, Id pageTable, bool shareCache) {
  using S = PagedUpdateCacheOp;
  Off c = tensorRef(cache), i = tensorRef(in), u = tensorRef(updateIndex), t = pageTable ? tensorRef(pageTable) : 0;
  b_.startTable(S::kNumFields);
  b_.addOffset(S::f_cache, c);
  b_.addOffset(S::f_input, i);
  b_.addOffset(S::f_update_index, u);
  b_.addScalarDefault<std::uint8_t>(S::f_share_cache, shareCache ? 1 : 0, 0);
  if (pageTable) b_.addOffset(S::f_page_table, t);
  addOp(OpType::PagedUpdateCacheOp, b_.endTable(), "ttnn.paged_update_cache");
}
void ProgramBuilder::pagedFillCache(Id cache, Id in, Id pageTable, Id batchIdx) {
  using S = PagedFillCacheOp;
  Off c = tensorRef(cache), i = tensorRef(in), t = tensorRef(pageTable), bi = batchIdx ? tensorRef(batchIdx) : 0;
  b_.startTable(S::kNumFields);
  b_.addOffset(S::f_cache, c);
  b_.addOffset(S::f_input, i);
  b_.addOffset(S::f_page_table, t);
  if (batchIdx) b_.addOffset(S::f_batch_idx_tensor, bi);
  addOp(OpType::PagedFillCacheOp, b_.endTable(), "ttnn.paged_fill_cache");
}
ProgramBuilder::Id ProgramBuilder::sdpaDecode(Id q, Id k, Id v, Id pageTable, Id mask, Id curPos, bool causal, bool hasScale, float scale,
                                              std::int64_t slidingWindow, Id sink) {
  Desc d = desc(q);
  d.storage = StorageType::Device;
  d.layout = TensorLayout::Tile;
  Id out = newTensor(d);
  Off qr = tensorRef(q), kr = tensorRef(k), vr = tensorRef(v), pt = pageTable ? tensorRef(pageTable) : 0, mr = mask ? tensorRef(mask) : 0,
      cp = curPos ? tensorRef(curPos) : 0, o = tensorRef(out), sr = sink ? tensorRef(sink) : 0;
  if (pageTable) {
    using S = PagedScaledDotProductAttentionDecodeOp;
    b_.startTable(S::kNumFields);
    b_.addOffset(S::f_query, qr); b_.addOffset(S::f_key, kr); b_.addOffset(S::f_value, vr); b_.addOffset(S::f_page_table, pt);
    b_.addScalarDefault<std::uint8_t>(S::f_is_causal, causal, 0);
    b_.addOffset(S::f_attention_mask, mr); b_.addOffset(S::f_cur_pos_tensor, cp);
    if (hasScale) b_.addScalar<float>(S::f_scale, scale);
    if (slidingWindow >= 0) b_.addScalar<std::uint32_t>(S::f_sliding_window_size, static_cast<std::uint32_t>(slidingWindow));
    b_.addOffset(S::f_attention_sink, sr);
    b_.addOffset(S::f_out, o);
    addOp(OpType::PagedScaledDotProductAttentionDecodeOp, b_.endTable(), "ttnn.paged_scaled_dot_product_attention_decode " + shapeStr(d.shape));
  } else {
    using S = ScaledDotProductAttentionDecodeOp;
    b_.startTable(S::kNumFields);
    b_.addOffset(S::f_query, qr); b_.addOffset(S::f_key, kr); b_.addOffset(S::f_value, vr);
    b_.addScalarDefault<std::uint8_t>(S::f_is_causal, causal, 0);
    b_.addOffset(S::f_attention_mask, mr); b_.addOffset(S::f_cur_pos_tensor, cp);
    if (hasScale) b_.addScalar<float>(S::f_scale, scale);
    if (slidingWindow >= 0) b_.addScalar<std::uint32_t>(S::f_sliding_window_size, static_cast<std::uint32_t>(slidingWindow));
    b_.addOffset(S::f_attention_sink, sr);
    b_.addOffset(S::f_out, o);
    addOp(OpType::ScaledDotProductAttentionDecodeOp, b_.endTable(), "ttnn.scaled_dot_product_attention_decode " + shapeStr(d.shape));
  }
  return out;
}

ProgramBuilder::Id ProgramBuilder::reshape(Id in, const std::vector<std::uint32_t> &shape) {
  Desc d = desc(in);
  d.shape = shape;
  Id out = newTensor(d);
  Off i = tensorRef(in), o = tensorRef(out);
  std::vector<std::int32_t> sv(shape.begin(), shape.end());
  Off s = b_.createScalarVector(sv);
  b_.startTable(ReshapeOp::kNumFields);
  b_.addOffset(ReshapeOp::f_in, i);
  b_.addOffset(ReshapeOp::f_out, o);
  b_.addOffset(ReshapeOp::f_shape, s);
  addOp(OpType::ReshapeOp, b_.endTable(), "ttnn.reshape -> " + shapeStr(shape));
  return out;
}
ProgramBuilder::Id ProgramBuilder::permute(Id in, const std::vector<std::int64_t> &perm) {
  Desc d = desc(in);
  std::vector<std::uint32_t> shape(perm.size());
  for (size_t i = 0; i < perm.size(); ++i) shape[i] = d.shape.at(static_cast<size_t>(perm[i]));
  d.shape = shape;
  Id out = newTensor(d);
  Off i = tensorRef(in), o = tensorRef(out), p = b_.createScalarVector(perm);
  b_.startTable(PermuteOp::kNumFields);
  b_.addOffset(PermuteOp::f_in, i);
  b_.addOffset(PermuteOp::f_permutation, p);
  b_.addOffset(PermuteOp::f_out, o);
  addOp(OpType::PermuteOp, b_.endTable(), "ttnn.permute -> " + shapeStr(shape));
  return out;
}
ProgramBuilder::Id ProgramBuilder::transpose(Id in, int dim0, int dim1) {
  Desc d = desc(in);
  int rank = static_cast<int>(d.shape.size());
  std::swap(d.shape.at(dim0 < 0 ? dim0 + rank : dim0), d.shape.at(dim1 < 0 ? dim1 + rank : dim1));
  Id out = newTensor(d);
  Off i = tensorRef(in), o = tensorRef(out);
  b_.startTable(TransposeOp::kNumFields);
  b_.addOffset(TransposeOp::f_in, i);
  b_.addOffset(TransposeOp::f_out, o);
  b_.addScalarDefault<std::int32_t>(TransposeOp::f_dim0, dim0, 0);
  b_.addScalarDefault<std::int32_t>(TransposeOp::f_dim1, dim1, 0);
  addOp(OpType::TransposeOp, b_.endTable(), "ttnn.transpose");
  return out;
}
ProgramBuilder::Id ProgramBuilder::concat(const std::vector<Id> &ins, int dim) {
  Desc d = desc(ins.at(0));
  int rank = static_cast<int>(d.shape.size());
  int ax = dim < 0 ? dim + rank : dim;
  std::uint32_t total = 0;
  for (Id t : ins) total += desc(t).shape.at(ax);
  d.shape[ax] = total;
  Id out = newTensor(d);
  std::vector<Off> refs;
  for (Id t : ins) refs.push_back(tensorRef(t));
  Off iv = b_.createOffsetVector(refs), o = tensorRef(out);
  b_.startTable(ConcatOp::kNumFields);
  b_.addOffset(ConcatOp::f_inputs, iv);
  b_.addOffset(ConcatOp::f_out, o);
  b_.addScalarDefault<std::int32_t>(ConcatOp::f_dim, dim, 0);
  addOp(OpType::ConcatOp, b_.endTable(), "ttnn.concat dim=" + std::to_string(dim));
  return out;
}
ProgramBuilder::Id ProgramBuilder::slice(Id in, const std::vector<std::int64_t> &begins, const std::vector<std::int64_t> &ends,
                                         const std::vector<std::int64_t> &steps) {
  Desc d = desc(in);
  for (size_t i = 0; i < d.shape.size(); ++i) {
    std::int64_t st = i < steps.size() ? steps[i] : 1;
    d.shape[i] = static_cast<std::uint32_t>((ends.at(i) - begins.at(i) + st - 1) / st);
  }
  Id out = newTensor(d);
  Off i = tensorRef(in), o = tensorRef(out);
  Off bv = b_.createScalarVector(begins), ev = b_.createScalarVector(ends), sv = b_.createScalarVector(steps);
  b_.startTable(SliceStaticOpParams::kNumFields);
  b_.addOffset(SliceStaticOpParams::f_begins, bv);
  b_.addOffset(SliceStaticOpParams::f_ends, ev);
  Off prm = b_.endTable();
  b_.startTable(SliceOp::kNumFields);
  b_.addScalarDefault<std::uint32_t>(SliceOp::f_type, static_cast<std::uint32_t>(SliceOpType::SliceStaticOp), 0);
  b_.addOffset(SliceOp::f_in, i);
  b_.addOffset(SliceOp::f_out, o);
  b_.addOffset(SliceOp::f_step, sv);
  b_.addScalar<std::uint8_t>(SliceOp::f_params_type, static_cast<std::uint8_t>(SliceOpParams::SliceStaticOpParams));
  b_.addOffset(SliceOp::f_params, prm);
  addOp(OpType::SliceOp, b_.endTable(), "ttnn.slice_static -> " + shapeStr(d.shape));
  return out;
}
ProgramBuilder::Id ProgramBuilder::repeatInterleave(Id in, std::uint32_t repeats, int dim) {
  Desc d = desc(in);
  int rank = static_cast<int>(d.shape.size());
  d.shape.at(dim < 0 ? dim + rank : dim) *= repeats;
  Id out = newTensor(d);
  Off i = tensorRef(in), o = tensorRef(out);
  b_.startTable(RepeatInterleaveOp::kNumFields);
  b_.addOffset(RepeatInterleaveOp::f_input, i);
  b_.addOffset(RepeatInterleaveOp::f_out, o);
  b_.addScalarDefault<std::uint32_t>(RepeatInterleaveOp::f_repeats, repeats, 0);
  b_.addScalarDefault<std::int32_t>(RepeatInterleaveOp::f_dim, dim, 0);
  addOp(OpType::RepeatInterleaveOp, b_.endTable(), "ttnn.repeat_interleave x" + std::to_string(repeats));
  return out;
}
ProgramBuilder::Id ProgramBuilder::repeat(Id in, const std::vector<std::int64_t> &repeats) {
  Desc d = desc(in);
  if (repeats.size() != d.shape.size()) fatal("ProgramBuilder: repeat needs one count per dimension");
  for (size_t i = 0; i < repeats.size(); ++i) d.shape[i] = static_cast<std::uint32_t>(d.shape[i] * repeats[i]);
  Id out = newTensor(d);
  Off i = tensorRef(in), o = tensorRef(out), r = b_.createScalarVector(repeats);
  b_.startTable(RepeatOp::kNumFields);
  b_.addOffset(RepeatOp::f_in, i);
  b_.addOffset(RepeatOp::f_out, o);
  b_.addOffset(RepeatOp::f_repeat_dims, r);
  addOp(OpType::RepeatOp, b_.endTable(), "ttnn.repeat -> " + shapeStr(d.shape));
  return out;
}
ProgramBuilder::Id ProgramBuilder::concatHeads(int kind, Id in, std::uint32_t numHeads) {
  Desc d = desc(in);
  const auto s = d.shape;
  if (s.size() != 4) fatal("ProgramBuilder: head merge needs a rank-4 input");
  if (kind == 0) d.shape = {s[0], s[2], s[1] * s[3]};
  else if (kind == 1) d.shape = {s[0], 1, s[2], s[1] * s[3]};
  else d.shape = {1, 1, s[1], numHeads * s[3]};
  d.storage = StorageType::Device;
  Id out = newTensor(d);
  Off i = tensorRef(in), o = tensorRef(out);
  if (kind == 0) {
    b_.startTable(ConcatenateHeadsOp::kNumFields);
    b_.addOffset(ConcatenateHeadsOp::f_in, i);
    b_.addOffset(ConcatenateHeadsOp::f_out, o);
    addOp(OpType::ConcatenateHeadsOp, b_.endTable(), "ttnn.concatenate_heads " + shapeStr(d.shape));
  } else if (kind == 1) {
    b_.startTable(NLPConcatHeadsOp::kNumFields);
    b_.addOffset(NLPConcatHeadsOp::f_in, i);
    b_.addOffset(NLPConcatHeadsOp::f_out, o);
    addOp(OpType::NLPConcatHeadsOp, b_.endTable(), "ttnn.nlp_concat_heads " + shapeStr(d.shape));
  } else {
    b_.startTable(NLPConcatHeadsDecodeOp::kNumFields);
    b_.addOffset(NLPConcatHeadsDecodeOp::f_in, i);
    b_.addOffset(NLPConcatHeadsDecodeOp::f_out, o);
    b_.addScalarDefault<std::uint32_t>(NLPConcatHeadsDecodeOp::f_num_heads, numHeads, 0);
    addOp(OpType::NLPConcatHeadsDecodeOp, b_.endTable(), "ttnn.nlp_concat_heads_decode " + shapeStr(d.shape));
  }
  return out;
}
std::array<ProgramBuilder::Id, 3> ProgramBuilder::nlpCreateQkvHeadsDecode(Id in, std::uint32_t numHeads, std::uint32_t numKvHeads) {
  Desc d = desc(in);
  const auto s = d.shape;
  if (s.size() != 4 || s[3] % (numHeads + 2 * numKvHeads) != 0) fatal("ProgramBuilder: nlp_create_qkv_heads_decode input must be [1, 1, users, (heads + 2 kv) * dim]");
  const std::uint32_t dim = s[3] / (numHeads + 2 * numKvHeads);
  d.storage = StorageType::Device;
  d.shape = {1, s[2], numHeads, dim};
  Id q = newTensor(d);
  d.shape = {1, s[2], numKvHeads, dim};
  Id k = newTensor(d), v = newTensor(d);
  using S = NLPCreateQKVHeadsDecodeOp;
  Off i = tensorRef(in), qo = tensorRef(q), ko = tensorRef(k), vo = tensorRef(v);
  b_.startTable(S::kNumFields);
  b_.addOffset(S::f_input, i);
  b_.addOffset(S::f_q_out, qo);
  b_.addOffset(S::f_k_out, ko);
  b_.addOffset(S::f_v_out, vo);
  b_.addScalarDefault<std::uint32_t>(S::f_num_heads, numHeads, 0);
  b_.addScalar<std::uint32_t>(S::f_num_kv_heads, numKvHeads);
  addOp(OpType::NLPCreateQKVHeadsDecodeOp, b_.endTable(), "ttnn.nlp_create_qkv_heads_decode");
  return {q, k, v};
}
std::array<ProgramBuilder::Id, 3> ProgramBuilder::splitQkvAndSplitHeads(Id in, Id kvInput, std::uint32_t numHeads, std::uint32_t numKvHeads,
                                                                        bool transposeKey) {
  Desc d = desc(in);
  const auto s = d.shape;
  if (s.size() != 3) fatal("ProgramBuilder: split_query_key_value_and_split_heads input must be [batch, seq, hidden]");
  const std::uint32_t dim = kvInput ? s[2] / numHeads : s[2] / (numHeads + 2 * numKvHeads);
  d.storage = StorageType::Device;
  d.shape = {s[0], numHeads, s[1], dim};
  Id q = newTensor(d);
  d.shape = transposeKey ? std::vector<std::uint32_t>{s[0], numKvHeads, dim, s[1]} : std::vector<std::uint32_t>{s[0], numKvHeads, s[1], dim};
  Id k = newTensor(d);
  d.shape = {s[0], numKvHeads, s[1], dim};
  Id v = newTensor(d);
  using S = SplitQueryKeyValueAndSplitHeadsOp;
  Off i = tensorRef(in), kv = kvInput ? tensorRef(kvInput) : 0, qo = tensorRef(q), ko = tensorRef(k), vo = tensorRef(v);
  b_.startTable(S::kNumFields);
  b_.addOffset(S::f_in, i);
  b_.addOffset(S::f_kv_input, kv);
  b_.addOffset(S::f_q_out, qo);
  b_.addOffset(S::f_k_out, ko);
  b_.addOffset(S::f_v_out, vo);
  b_.addScalarDefault<std::uint32_t>(S::f_num_heads, numHeads, 0);
  b_.addScalar<std::uint32_t>(S::f_num_kv_heads, numKvHeads);
  b_.addScalarDefault<std::uint8_t>(S::f_transpose_key, transposeKey, 0);
  addOp(OpType::SplitQueryKeyValueAndSplitHeadsOp, b_.endTable(), "ttnn.split_query_key_value_and_split_heads");
  return {q, k, v};
}
ProgramBuilder::Id ProgramBuilder::binaryComposite(std::uint32_t type, Id lhs, Id rhs) {
  const auto &a = desc(lhs).shape, &b = desc(rhs).shape;
  size_t rank = std::max(a.size(), b.size());
  std::vector<std::uint32_t> shape(rank);
  for (size_t i = 0; i < rank; ++i) {
    std::uint32_t x = i < rank - a.size() ? 1 : a[i - (rank - a.size())], y = i < rank - b.size() ? 1 : b[i - (rank - b.size())];
    if (x != y && x != 1 && y != 1) fatal("ProgramBuilder: binary operands do not broadcast");
    shape[i] = std::max(x, y);
  }
  Id out = newTensor(Desc{shape, desc(lhs).dtype, desc(lhs).layout, StorageType::Device});
  Off l = tensorRef(lhs), r = tensorRef(rhs), o = tensorRef(out);
  b_.startTable(EltwiseBinaryCompositeOp::kNumFields);
  b_.addScalarDefault<std::uint32_t>(EltwiseBinaryCompositeOp::f_type, type, 0);
  b_.addOffset(EltwiseBinaryCompositeOp::f_lhs, l);
  b_.addOffset(EltwiseBinaryCompositeOp::f_rhs, r);
  b_.addOffset(EltwiseBinaryCompositeOp::f_out, o);
  addOp(OpType::EltwiseBinaryCompositeOp, b_.endTable(), "ttnn.binary_composite#" + std::to_string(type));
  return out;
}
ProgramBuilder::Id ProgramBuilder::where(Id cond, Id a, Id b) {
  const auto &cs = desc(cond).shape, &as = desc(a).shape, &bs = desc(b).shape;
  size_t rank = std::max({cs.size(), as.size(), bs.size()});
  std::vector<std::uint32_t> shape(rank, 1);
  for (const auto *s : {&cs, &as, &bs})
    for (size_t i = 0; i < s->size(); ++i) {
      std::uint32_t &o = shape[rank - s->size() + i], v = (*s)[i];
      if (o != v && o != 1 && v != 1) fatal("ProgramBuilder: where operands do not broadcast");
      o = std::max(o, v);
    }
  Id out = newTensor(Desc{shape, desc(a).dtype, desc(a).layout, StorageType::Device});
  Off c = tensorRef(cond), x = tensorRef(a), y = tensorRef(b), o = tensorRef(out);
  b_.startTable(EltwiseTernaryWhereOp::kNumFields);
  b_.addOffset(EltwiseTernaryWhereOp::f_first, c);
  b_.addOffset(EltwiseTernaryWhereOp::f_second, x);
  b_.addOffset(EltwiseTernaryWhereOp::f_third, y);
  b_.addOffset(EltwiseTernaryWhereOp::f_out, o);
  addOp(OpType::EltwiseTernaryWhereOp, b_.endTable(), "ttnn.where " + shapeStr(shape));
  return out;
}
ProgramBuilder::Id ProgramBuilder::embedding(Id indices, Id weight) {
  Desc d = desc(weight);
  std::vector<std::uint32_t> shape = desc(indices).shape;
  shape.push_back(d.shape.back());
  d.shape = shape;
  d.storage = StorageType::Device;
  Id out = newTensor(d);
  Off i = tensorRef(indices), w = tensorRef(weight), o = tensorRef(out);
  b_.startTable(EmbeddingOp::kNumFields);
  b_.addOffset(EmbeddingOp::f_input, i);
  b_.addOffset(EmbeddingOp::f_weight, w);
  b_.addOffset(EmbeddingOp::f_out, o);
  addOp(OpType::EmbeddingOp, b_.endTable(), "ttnn.embedding " + shapeStr(shape));
  return out;
}
ProgramBuilder::Id ProgramBuilder::argmax(Id in, bool hasDim, int dim, bool keepDim, DataType outDtype) {
  Desc d = desc(in);
  const int rank = static_cast<int>(d.shape.size());
  std::vector<std::uint32_t> shape;
  if (hasDim) {
    const int dd = dim < 0 ? dim + rank : dim;
    for (int i = 0; i < rank; ++i) {
      if (i != dd) shape.push_back(d.shape[i]);
      else if (keepDim) shape.push_back(1);
    }
  } else if (keepDim) {
    shape.assign(rank, 1);
  }
  if (shape.empty()) shape.push_back(1);
  Id out = newTensor(Desc{shape, outDtype, TensorLayout::RowMajor, StorageType::Device});
  Off i = tensorRef(in), o = tensorRef(out);
  b_.startTable(ReductionArgMaxOp::kNumFields);
  b_.addOffset(ReductionArgMaxOp::f_in, i);
  b_.addOffset(ReductionArgMaxOp::f_out, o);
  if (hasDim) b_.addScalar<std::int32_t>(ReductionArgMaxOp::f_dim, dim);
  b_.addScalarDefault<std::uint8_t>(ReductionArgMaxOp::f_keep_dim, keepDim, 0);
  addOp(OpType::ReductionArgMaxOp, b_.endTable(), "ttnn.argmax " + shapeStr(shape));
  return out;
}
ProgramBuilder::Id ProgramBuilder::arange(float start, float end, float step, DataType dtype, TensorLayout layout) {
  const double n = std::ceil((static_cast<double>(end) - start) / step);
  std::vector<std::uint32_t> shape{static_cast<std::uint32_t>(n > 0 ? n : 0)};
  Id out = newTensor(Desc{shape, dtype, layout, StorageType::Device});
  Off o = tensorRef(out);
  b_.startTable(ArangeOp::kNumFields);
  b_.addScalarDefault<float>(ArangeOp::f_start, start, 0.0f);
  b_.addScalarDefault<float>(ArangeOp::f_end, end, 0.0f);
  b_.addScalarDefault<float>(ArangeOp::f_step, step, 0.0f);
  b_.addScalar<std::uint16_t>(ArangeOp::f_dtype, static_cast<std::uint16_t>(dtype));
  b_.addScalar<std::uint16_t>(ArangeOp::f_layout, static_cast<std::uint16_t>(layout));
  b_.addOffset(ArangeOp::f_out, o);
  addOp(OpType::ArangeOp, b_.endTable(), "ttnn.arange " + shapeStr(shape));
  return out;
}
ProgramBuilder::Id ProgramBuilder::constant(const void *data, size_t bytes, DataType inDtype, const std::vector<std::uint32_t> &shape,
                                            DataType dtype, TensorLayout layout, StorageType storage) {
  Id out = newTensor(Desc{shape, dtype, layout, storage});
  Off payload = b_.createScalarVector(static_cast<const std::uint8_t *>(data), bytes), o = tensorRef(out);
  b_.startTable(ConstantOp::kNumFields);
  b_.addOffset(ConstantOp::f_input, payload);
  b_.addScalarDefault<std::uint16_t>(ConstantOp::f_input_dtype, static_cast<std::uint16_t>(inDtype), 0);
  b_.addScalar<std::uint16_t>(ConstantOp::f_dtype, static_cast<std::uint16_t>(dtype));
  b_.addScalar<std::uint16_t>(ConstantOp::f_layout, static_cast<std::uint16_t>(layout));
  b_.addOffset(ConstantOp::f_out, o);
  addOp(OpType::ConstantOp, b_.endTable(), "ttnn.constant " + shapeStr(shape));
  return out;
}
ProgramBuilder::Id ProgramBuilder::full(const std::vector<std::uint32_t> &shape, float value, DataType dtype, TensorLayout layout) {
  Id out = newTensor(Desc{shape, dtype, layout, StorageType::Device});
  std::vector<std::int64_t> sv(shape.begin(), shape.end());
  Off s = b_.createScalarVector(sv), o = tensorRef(out);
  b_.startTable(FloatingPointType::kNumFields);
  b_.addScalar<float>(FloatingPointType::f_value, value);
  Off fv = b_.endTable();
  b_.startTable(FullOp::kNumFields);
  b_.addOffset(FullOp::f_shape, s);
  b_.addScalar<std::uint8_t>(FullOp::f_fill_value_type, static_cast<std::uint8_t>(NumberType::FP));
  b_.addOffset(FullOp::f_fill_value, fv);
  b_.addScalar<std::uint16_t>(FullOp::f_dtype, static_cast<std::uint16_t>(dtype));
  b_.addScalar<std::uint16_t>(FullOp::f_layout, static_cast<std::uint16_t>(layout));
  b_.addOffset(FullOp::f_out, o);
  addOp(OpType::FullOp, b_.endTable(), "ttnn.full " + shapeStr(shape));
  return out;
}
ProgramBuilder::Id ProgramBuilder::empty(const std::vector<std::uint32_t> &shape, DataType dtype, TensorLayout layout) {
  Id out = newTensor(Desc{shape, dtype, layout, StorageType::Device});
  std::vector<std::int64_t> sv(shape.begin(), shape.end());
  Off s = b_.createScalarVector(sv), o = tensorRef(out);
  b_.startTable(EmptyOp::kNumFields);
  b_.addOffset(EmptyOp::f_shape, s);
  b_.addScalar<std::uint16_t>(EmptyOp::f_dtype, static_cast<std::uint16_t>(dtype));
  b_.addScalar<std::uint16_t>(EmptyOp::f_layout, static_cast<std::uint16_t>(layout));
  b_.addOffset(EmptyOp::f_out, o);
  addOp(OpType::EmptyOp, b_.endTable(), "ttnn.empty " + shapeStr(shape));
  return out;
}
void ProgramBuilder::copy(Id src, Id dst) {
  Off s = tensorRef(src), d = tensorRef(dst);
  b_.startTable(CopyOp::kNumFields);
  b_.addOffset(CopyOp::f_src, s);
  b_.addOffset(CopyOp::f_dst, d);
  addOp(OpType::CopyOp, b_.endTable(), "ttnn.copy");
}
void ProgramBuilder::writeTensor(Id host, Id device) {
  Off h = tensorRef(host), d = tensorRef(device);
  b_.startTable(WriteTensorOp::kNumFields);
  b_.addOffset(WriteTensorOp::f_host_tensor, h);
  b_.addOffset(WriteTensorOp::f_device_tensor, d);
  b_.addScalarDefault<std::uint8_t>(WriteTensorOp::f_blocking, 1, 0);
  addOp(OpType::WriteTensorOp, b_.endTable(), "ttnn.write_tensor");
}
ProgramBuilder::Id ProgramBuilder::beginTraceCapture() {
  Id out = newTensor(Desc{{}, DataType::UInt32, TensorLayout::RowMajor, StorageType::Host});
  Off o = tensorRef(out);
  b_.startTable(BeginTraceCaptureOp::kNumFields);
  b_.addOffset(BeginTraceCaptureOp::f_trace_id, o);
  addOp(OpType::BeginTraceCaptureOp, b_.endTable(), "ttnn.begin_trace_capture");
  return out;
}
void ProgramBuilder::endTraceCapture(Id traceId) {
  Off t = tensorRef(traceId);
  b_.startTable(EndTraceCaptureOp::kNumFields);
  b_.addOffset(EndTraceCaptureOp::f_trace_id, t);
  addOp(OpType::EndTraceCaptureOp, b_.endTable(), "ttnn.end_trace_capture");
}
void ProgramBuilder::executeTrace(Id traceId, bool blocking) {
  Off t = tensorRef(traceId);
  b_.startTable(ExecuteTraceOp::kNumFields);
  b_.addOffset(ExecuteTraceOp::f_trace_id, t);
  b_.addScalarDefault<std::uint8_t>(ExecuteTraceOp::f_blocking, blocking, 0);
  addOp(OpType::ExecuteTraceOp, b_.endTable(), "ttnn.execute_trace");
}
std::vector<ProgramBuilder::Id> ProgramBuilder::captureOrExecuteTrace(std::uint32_t captureProgram, std::uint32_t executeProgram,
                                                                      std::uint32_t allocateSlotsProgram, const std::vector<Id> &ins,
                                                                      const std::vector<Desc> &outs) {
  std::vector<Id> ids;
  std::vector<Off> ir, orf;
  for (Id t : ins) ir.push_back(tensorRef(t));
  for (const Desc &d : outs) {
    ids.push_back(newTensor(d));
    orf.push_back(tensorRef(ids.back()));
  }
  Off iv = b_.createOffsetVector(ir), ov = b_.createOffsetVector(orf);
  b_.startTable(CaptureOrExecuteTraceOp::kNumFields);
  b_.addScalarDefault<std::uint32_t>(CaptureOrExecuteTraceOp::f_capture_program_id, captureProgram, 0);
  b_.addScalarDefault<std::uint32_t>(CaptureOrExecuteTraceOp::f_execute_program_id, executeProgram, 0);
  b_.addScalarDefault<std::uint32_t>(CaptureOrExecuteTraceOp::f_allocate_slots_program_id, allocateSlotsProgram, 0);
  b_.addOffset(CaptureOrExecuteTraceOp::f_inputs, iv);
  b_.addOffset(CaptureOrExecuteTraceOp::f_outputs, ov);
  addOp(OpType::CaptureOrExecuteTraceOp, b_.endTable(),
        "ttnn.capture_or_execute_trace capture #" + std::to_string(captureProgram) + " execute #" + std::to_string(executeProgram));
  return ids;
}
void ProgramBuilder::deallocate(Id in, bool force) {
  Off i = tensorRef(in);
  b_.startTable(DeallocateOp::kNumFields);
  b_.addOffset(DeallocateOp::f_in, i);
  b_.addScalarDefault<std::uint8_t>(DeallocateOp::f_force, force, 0);
  addOp(OpType::DeallocateOp, b_.endTable(), "ttnn.deallocate");
}
std::vector<ProgramBuilder::Id> ProgramBuilder::loadCached(std::uint32_t programIdx, const std::string &callee, const std::vector<Id> &ins,
                                                           const std::vector<Desc> &outs) {
  std::vector<Id> ids;
  std::vector<Off> ir, orf;
  for (Id t : ins) ir.push_back(tensorRef(t));
  for (const Desc &d : outs) {
    ids.push_back(newTensor(d));
    orf.push_back(tensorRef(ids.back()));
  }
  Off iv = b_.createOffsetVector(ir), ov = b_.createOffsetVector(orf), name = b_.createString(callee);
  Off hash = b_.createString(callee + "#" + std::to_string(programIdx));
  b_.startTable(LoadCachedOp::kNumFields);
  b_.addOffset(LoadCachedOp::f_inputs, iv);
  b_.addOffset(LoadCachedOp::f_callee_name, name);
  b_.addScalarDefault<std::uint32_t>(LoadCachedOp::f_program_idx, programIdx, 0);
  b_.addOffset(LoadCachedOp::f_outputs, ov);
  b_.addOffset(LoadCachedOp::f_program_hash, hash);
  addOp(OpType::LoadCachedOp, b_.endTable(), "ttcore.load_cached @" + callee);
  return ids;
}
std::vector<ProgramBuilder::Id> ProgramBuilder::funcCall(std::uint32_t programIdx, const std::vector<Id> &ins, const std::vector<Desc> &outs) {
  std::vector<Id> ids;
  std::vector<Off> ir, orf;
  for (Id t : ins) ir.push_back(tensorRef(t));
  for (const Desc &d : outs) {
    ids.push_back(newTensor(d));
    orf.push_back(tensorRef(ids.back()));
  }
  Off iv = b_.createOffsetVector(ir), ov = b_.createOffsetVector(orf);
  b_.startTable(FuncCallOp::kNumFields);
  b_.addScalarDefault<std::uint32_t>(FuncCallOp::f_program_id, programIdx, 0);
  b_.addOffset(FuncCallOp::f_inputs, iv);
  b_.addOffset(FuncCallOp::f_outputs, ov);
  addOp(OpType::FuncCallOp, b_.endTable(), "func.call #" + std::to_string(programIdx));
  return ids;
}

ProgramBuilder::Id ProgramBuilder::rotaryEmbeddingLlama(Id in, Id cosCache, Id sinCache, Id transMat, bool decodeMode) {
  const Desc d = desc(in);
  Id out = newTensor(Desc{d.shape, d.dtype, TensorLayout::Tile, StorageType::Device});
  Off i = tensorRef(in), c = tensorRef(cosCache), s = tensorRef(sinCache), t = tensorRef(transMat), o = tensorRef(out);
  using S = RotaryEmbeddingLlamaOp;
  b_.startTable(S::kNumFields);
  b_.addOffset(S::f_input, i);
  b_.addOffset(S::f_cos_cache, c);
  b_.addOffset(S::f_sin_cache, s);
  b_.addOffset(S::f_trans_mat, t);
  b_.addScalarDefault<std::uint8_t>(S::f_is_decode_mode, decodeMode ? 1 : 0, 0);
  b_.addOffset(S::f_out, o);
  addOp(OpType::RotaryEmbeddingLlamaOp, b_.endTable(), "ttnn.rotary_embedding_llama " + shapeStr(d.shape));
  return out;
}

ProgramBuilder::Id ProgramBuilder::chunkedSdpa(Id q, Id k, Id v, Id pageTable, Id chunkStart, bool hasScale, float scale) {
  const Desc d = desc(q);
  Id out = newTensor(Desc{d.shape, DataType::BFloat16, TensorLayout::Tile, StorageType::Device});
  Off qr = tensorRef(q), kr = tensorRef(k), vr = tensorRef(v), pr = tensorRef(pageTable), sr = tensorRef(chunkStart), o = tensorRef(out);
  using S = ChunkedScaledDotProductAttentionOp;
  b_.startTable(S::kNumFields);
  b_.addOffset(S::f_query, qr);
  b_.addOffset(S::f_key, kr);
  b_.addOffset(S::f_value, vr);
  b_.addOffset(S::f_page_table, pr);
  b_.addOffset(S::f_chunk_start_idx, sr);
  if (hasScale) b_.addScalar<float>(S::f_scale, scale);
  b_.addOffset(S::f_out, o);
  addOp(OpType::ChunkedScaledDotProductAttentionOp, b_.endTable(), "ttnn.chunked_scaled_dot_product_attention " + shapeStr(d.shape));
  return out;
}

void ProgramBuilder::addDylib(std::uint32_t dylibId, const void *data, size_t bytes) {
  if (!open_) fatal("ProgramBuilder: no program is open");
  Off raw = b_.createScalarVector(static_cast<const std::uint8_t *>(data), bytes);
  b_.startTable(DynamicLib::kNumFields);
  b_.addScalarDefault<std::uint32_t>(DynamicLib::f_dylib_id, dylibId, 0);
  b_.addOffset(DynamicLib::f_raw_file, raw);
  cur_.dylibs.push_back(b_.endTable());
}

std::vector<ProgramBuilder::Id> ProgramBuilder::cpuOp(std::uint32_t dylibId, const std::string &funcName, const std::vector<Id> &ins,
                                                      const std::vector<Desc> &outs) {
  std::vector<Id> ids;
  std::vector<Off> ir, orf;
  for (Id t : ins) ir.push_back(tensorRef(t));
  for (const Desc &d : outs) {
    ids.push_back(newTensor(d));
    orf.push_back(tensorRef(ids.back()));
  }
  Off iv = b_.createOffsetVector(ir), ov = b_.createOffsetVector(orf), name = b_.createString(funcName);
  b_.startTable(CpuOp::kNumFields);
  b_.addOffset(CpuOp::f_ins, iv);
  b_.addOffset(CpuOp::f_outs, ov);
  b_.addOffset(CpuOp::f_func_name, name);
  b_.addScalarDefault<std::uint32_t>(CpuOp::f_dylib_id, dylibId, 0);
  addOp(OpType::CpuOp, b_.endTable(), "ttnn.cpu " + funcName);
  return ids;
}

}  // namespace ttmlir_amd
