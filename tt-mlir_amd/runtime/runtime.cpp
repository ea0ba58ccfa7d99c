// Host runtime: dtype utilities, binary loading, device and tensor handles, layout conversion
// (toLayout / toHost / memcpy).  Program execution lives in executor.cpp.
#include <algorithm>
#include <cmath>
#include <cstdio>
#include <cstring>
#include <fstream>
#include <limits>
#include <map>
#include <mutex>
#include <set>
#include <sstream>
#include <thread>

#include "device_pool.h"
#include "runtime_impl.h"

namespace tt::runtime {

using namespace ::ttmlir_amd;

void fatal(const std::string &msg) {
  const char *quiet = std::getenv("TTMLIR_RUNTIME_LOGGER_LEVEL");
  if (!quiet || std::string(quiet) != "FATAL_SILENT") std::fprintf(stderr, "[tt::runtime] FATAL: %s\n", msg.c_str());
  throw std::runtime_error("Fatal error: " + msg);
}

void hipCheck(int status, const char *what) {
  if (status != 0) fatal(std::string(what) + " -> " + ttm_last_error());
}

// ============================================================================ utils
namespace utils {

std::uint32_t dataTypeElementSize(DataType dt) {
  switch (dt) {
  case DataType::Float64: case DataType::Int64: case DataType::UInt64: return 8;
  case DataType::Float32: case DataType::UInt32: case DataType::Int32: return 4;
  case DataType::Float16: case DataType::BFloat16: case DataType::UInt16: case DataType::Int16: return 2;
  case DataType::UInt8: case DataType::Int8: case DataType::Bool: return 1;
  default: fatal("Unsupported element size for data type");
  }
}

bool isBlockFormatDataType(DataType dt) {
  switch (dt) {
  case DataType::BFP_Float8: case DataType::BFP_BFloat8: case DataType::BFP_Float4: case DataType::BFP_BFloat4:
  case DataType::BFP_Float2: case DataType::BFP_BFloat2: return true;
  default: return false;
  }
}

std::uint64_t blockFormatTileSizeBytes(DataType dt) {
  // one shared-exponent byte per 16 elements of a 32x32 tile, then the mantissas
  auto tileBytes = [](std::uint64_t bits) { return (1024 * bits) / 8 + 1024 / 16; };
  switch (dt) {
  case DataType::BFP_Float8: case DataType::BFP_BFloat8: return tileBytes(8);
  case DataType::BFP_Float4: case DataType::BFP_BFloat4: return tileBytes(4);
  case DataType::BFP_Float2: case DataType::BFP_BFloat2: return tileBytes(2);
  default: fatal("Not a block format data type");
  }
}

bool isSupportedDataType(DataType dt) {
  switch (dt) {
  case DataType::Float16: case DataType::Float64: case DataType::Int64: case DataType::UInt64: case DataType::Int16:
  case DataType::Int8: case DataType::Bool: return false;
  default: return true;
  }
}

DataType getUnsupportedDataTypeAlias(DataType dt) {
  switch (dt) {
  case DataType::Float64: return DataType::Float32;
  case DataType::Int64: return DataType::Int32;
  case DataType::UInt64: return DataType::UInt32;
  case DataType::Int16: return DataType::UInt16;
  case DataType::Int8: return DataType::UInt8;
  case DataType::Bool: return DataType::BFloat16;
  case DataType::Float16: return DataType::BFloat16;
  default: fatal(std::string("data type ") + dataTypeName(dt) + " needs no alias");
  }
}

const char *dataTypeName(DataType dt) {
  static const char *names[] = {"Float32", "Float16", "BFloat16", "BFP_Float8", "BFP_BFloat8", "BFP_Float4", "BFP_BFloat4",
                                "BFP_Float2", "BFP_BFloat2", "UInt32", "UInt16", "UInt8", "Int32", "Float64", "Int64",
                                "UInt64", "Int16", "Int8", "Bool"};
  auto i = static_cast<unsigned>(dt);
  return i < sizeof(names) / sizeof(names[0]) ? names[i] : "?";
}

// saturating integer casts (runtime/include/tt/runtime/utils.h:26-150)
template <typename From, typename To>
static void intCast(const void *src, void *dst, std::int64_t n) {
  const From *s = static_cast<const From *>(src);
  To *d = static_cast<To *>(dst);
  for (std::int64_t i = 0; i < n; ++i) {
    From v = s[i];
    if constexpr (std::is_signed_v<From> && std::is_unsigned_v<To>) {
      if (v < 0) { d[i] = 0; continue; }
      if (static_cast<std::make_unsigned_t<From>>(v) > std::numeric_limits<To>::max()) { d[i] = std::numeric_limits<To>::max(); continue; }
    } else if constexpr (std::is_unsigned_v<From> && std::is_signed_v<To>) {
      if (v > static_cast<std::make_unsigned_t<To>>(std::numeric_limits<To>::max())) { d[i] = std::numeric_limits<To>::max(); continue; }
    } else if constexpr (sizeof(To) < sizeof(From)) {
      if (v < static_cast<From>(std::numeric_limits<To>::min())) { d[i] = std::numeric_limits<To>::min(); continue; }
      if (v > static_cast<From>(std::numeric_limits<To>::max())) { d[i] = std::numeric_limits<To>::max(); continue; }
    }
    d[i] = static_cast<To>(v);
  }
}

static std::uint16_t f32ToBf16(float f) {
  std::uint32_t u;
  std::memcpy(&u, &f, 4);
  if ((u & 0x7FFFFFFFu) > 0x7F800000u) return static_cast<std::uint16_t>((u >> 16) | 0x40);
  u += 0x7FFFu + ((u >> 16) & 1);
  return static_cast<std::uint16_t>(u >> 16);
}
static float bf16ToF32(std::uint16_t h) {
  std::uint32_t u = static_cast<std::uint32_t>(h) << 16;
  float f;
  std::memcpy(&f, &u, 4);
  return f;
}
static float f16ToF32(std::uint16_t h) {
  std::uint32_t sign = static_cast<std::uint32_t>(h & 0x8000) << 16, e = (h >> 10) & 0x1F, m = h & 0x3FF, u;
  if (e == 0) {
    float v = std::ldexp(static_cast<float>(m), -24);
    return sign ? -v : v;
  }
  u = e == 31 ? (sign | 0x7F800000u | (m << 13)) : (sign | ((e + 112) << 23) | (m << 13));
  float f;
  std::memcpy(&f, &u, 4);
  return f;
}
static std::uint16_t f32ToF16(float f) {
  std::uint32_t u;
  std::memcpy(&u, &f, 4);
  std::uint32_t sign = (u >> 16) & 0x8000, a = u & 0x7FFFFFFFu;
  if (a > 0x7F800000u) return static_cast<std::uint16_t>(sign | 0x7E00);
  if (a >= 0x477FF000u) return static_cast<std::uint16_t>(sign | 0x7C00);
  if (a < 0x33000001u) return static_cast<std::uint16_t>(sign);
  int e = static_cast<int>(a >> 23) - 127;
  std::uint32_t m = (a & 0x7FFFFFu) | 0x800000u;
  int shift = e < -14 ? (13 + (-14 - e)) : 13;
  std::uint32_t keep = m >> shift, rem = m & ((1u << shift) - 1), half = 1u << (shift - 1);
  if (rem > half || (rem == half && (keep & 1))) keep++;
  std::uint32_t out = e < -14 ? keep : ((static_cast<std::uint32_t>(e + 15) << 10) + (keep - 0x400));
  return static_cast<std::uint16_t>(sign | out);
}

void handleBufferCast(const void *src, void *dst, DataType from, DataType to, std::int64_t n) {
  if (!src || !dst) throw std::runtime_error("Buffer pointers must not be null");
  if (from == to) {
    std::memcpy(dst, src, static_cast<size_t>(n) * dataTypeElementSize(from));
    return;
  }
  auto is = [&](DataType a, DataType b) { return from == a && to == b; };
  if (is(DataType::Int64, DataType::Int32)) intCast<std::int64_t, std::int32_t>(src, dst, n);
  else if (is(DataType::Int32, DataType::Int64)) intCast<std::int32_t, std::int64_t>(src, dst, n);
  else if (is(DataType::UInt64, DataType::UInt32)) intCast<std::uint64_t, std::uint32_t>(src, dst, n);
  else if (is(DataType::UInt32, DataType::UInt64)) intCast<std::uint32_t, std::uint64_t>(src, dst, n);
  else if (is(DataType::UInt32, DataType::Int64)) intCast<std::uint32_t, std::int64_t>(src, dst, n);
  else if (is(DataType::Int16, DataType::UInt16)) intCast<std::int16_t, std::uint16_t>(src, dst, n);
  else if (is(DataType::UInt16, DataType::Int16)) intCast<std::uint16_t, std::int16_t>(src, dst, n);
  else if (is(DataType::Int8, DataType::UInt8)) intCast<std::int8_t, std::uint8_t>(src, dst, n);
  else if (is(DataType::UInt8, DataType::Int8)) intCast<std::uint8_t, std::int8_t>(src, dst, n);
  else if (is(DataType::Float32, DataType::Float64)) {
    for (std::int64_t i = 0; i < n; ++i) static_cast<double *>(dst)[i] = static_cast<const float *>(src)[i];
  } else if (is(DataType::Float64, DataType::Float32)) {
    for (std::int64_t i = 0; i < n; ++i) static_cast<float *>(dst)[i] = static_cast<float>(static_cast<const double *>(src)[i]);
  } else if (is(DataType::BFloat16, DataType::Bool)) {
    for (std::int64_t i = 0; i < n; ++i) static_cast<bool *>(dst)[i] = (static_cast<const std::uint16_t *>(src)[i] & 0x7FFF) != 0;
  } else if (is(DataType::Bool, DataType::BFloat16)) {
    for (std::int64_t i = 0; i < n; ++i) static_cast<std::uint16_t *>(dst)[i] = static_cast<const std::uint8_t *>(src)[i] ? 0x3F80 : 0;
  } else if (is(DataType::Float16, DataType::BFloat16)) {
    for (std::int64_t i = 0; i < n; ++i) static_cast<std::uint16_t *>(dst)[i] = f32ToBf16(f16ToF32(static_cast<const std::uint16_t *>(src)[i]));
  } else if (is(DataType::BFloat16, DataType::Float16)) {
    for (std::int64_t i = 0; i < n; ++i) static_cast<std::uint16_t *>(dst)[i] = f32ToF16(bf16ToF32(static_cast<const std::uint16_t *>(src)[i]));
  } else {
    throw std::runtime_error(std::string("Unhandled buffer cast case: From ") + dataTypeName(from) + " to " + dataTypeName(to));
  }
}

std::vector<std::int64_t> calculateStride(const std::vector<std::uint32_t> &shape) {
  std::vector<std::int64_t> s(shape.size(), 1);
  for (int i = static_cast<int>(shape.size()) - 2; i >= 0; --i) s[i] = s[i + 1] * shape[i + 1];
  return s;
}

}  // namespace utils

// ============================================================================ shapes and sizes
Dims3 dims3(const std::vector<std::uint32_t> &shape) {
  Dims3 d;
  if (shape.empty()) return d;
  d.cols = shape.back();
  if (shape.size() >= 2) d.rows = shape[shape.size() - 2];
  for (size_t i = 0; i + 2 < shape.size(); ++i) d.batch *= shape[i];
  return d;
}
std::int64_t volume(const std::vector<std::uint32_t> &shape) {
  std::int64_t v = 1;
  for (auto s : shape) v *= s;
  return v;
}
std::int64_t paddedVolume(const std::vector<std::uint32_t> &shape) {
  Dims3 d = dims3(shape);
  return d.batch * ((d.rows + 31) / 32 * 32) * ((d.cols + 31) / 32 * 32);
}
// Every allocation is sized here.  Extents come from the binary or the caller: their padded product is formed with a check
// at every step, so that an absurd shape (a damaged binary) is an error and not an overflow that allocates a few bytes for
// a tensor the kernels would then be launched on.
static void requireRepresentableShape(const std::vector<std::uint32_t> &shape) {
  TTRT_ASSERT(shape.size() <= 8, "tensor rank above 8");
  constexpr std::uint64_t kMaxElements = std::uint64_t{1} << 40;   // 1 Ti elements: beyond any device
  std::uint64_t v = 1;
  for (size_t i = 0; i < shape.size(); ++i) {
    const bool tiled = i + 2 >= shape.size();   // the last two extents may be padded to 32
    const std::uint64_t e = tiled ? (static_cast<std::uint64_t>(shape[i]) + 31) / 32 * 32 : shape[i];
    if (e == 0) return;                          // an empty tensor
    TTRT_ASSERT(v <= kMaxElements / e, "tensor shape is too large to allocate");
    v *= e;
  }
}
size_t tensorBytes(const std::vector<std::uint32_t> &shape, DataType dtype, TensorLayout layout) {
  requireRepresentableShape(shape);
  if (utils::isBlockFormatDataType(dtype)) {
    TTRT_ASSERT(layout == TensorLayout::Tile, "block-float tensors must be in tile layout");
    return static_cast<size_t>(paddedVolume(shape) / 1024) * utils::blockFormatTileSizeBytes(dtype);
  }
  std::int64_t n = layout == TensorLayout::Tile ? paddedVolume(shape) : volume(shape);
  return static_cast<size_t>(n) * utils::dataTypeElementSize(dtype);
}

// ============================================================================ binary
static std::atomic<std::uint64_t> g_binaryId{1};

// Devices that may hold cached results of a binary.  Leaked on purpose: binaries and devices may be destroyed from static
// destructors in any order.
namespace {
struct DeviceRegistry {
  std::mutex mu;
  std::vector<std::weak_ptr<DeviceState>> devices;
};
DeviceRegistry &deviceRegistry() {
  static DeviceRegistry *r = new DeviceRegistry;
  return *r;
}
}  // namespace

TensorImpl::~TensorImpl() {
  for (auto &f : onDestroy) {
    try { f(); } catch (...) { /* a destructor must not throw */ }
  }
}

BinaryImpl::~BinaryImpl() {
  std::vector<std::shared_ptr<DeviceState>> devs;
  {
    std::lock_guard<std::mutex> g(deviceRegistry().mu);
    auto &v = deviceRegistry().devices;
    for (auto it = v.begin(); it != v.end();) {
      if (auto d = it->lock()) { devs.push_back(d); ++it; } else it = v.erase(it);
    }
  }
  for (auto &d : devs) {
    std::vector<ConstEvalEntry> dropped;   // their tensors return to the pool outside the lock
    {
      std::lock_guard<std::mutex> g(d->constEvalMu);
      for (auto it = d->constEval.begin(); it != d->constEval.end();) {
        if (std::get<0>(it->first) == id) { dropped.push_back(std::move(it->second)); it = d->constEval.erase(it); } else ++it;
      }
    }
    if (!d->open) continue;
    // traces recorded for this binary: nobody can replay them once the binary is gone
    std::lock_guard<std::recursive_mutex> g(d->mu);
    if (d->capturing) continue;
    std::vector<std::uint32_t> ids;
    for (const auto &kv : d->traceCache)
      if (std::get<0>(kv.first) == id) ids.push_back(kv.second);
    for (std::uint32_t t : ids) {
      try { releaseTrace(d, t); } catch (const std::exception &) { /* a destructor must not throw */ }
    }
  }
}

static Binary makeBinary(std::vector<std::uint8_t> &&bytes) {
  auto impl = std::make_shared<BinaryImpl>();
  impl->bytes = std::move(bytes);
  try {
    impl->root = fb::sizePrefixedRoot(impl->bytes.data(), impl->bytes.size(), "TTNN");
  } catch (const std::exception &e) {
    fatal(std::string("Binary: not a TTNN flatbuffer: ") + e.what());
  }
  impl->id = g_binaryId++;
  return Binary{impl};
}

Binary Binary::loadFromPath(const std::string &path) {
  std::ifstream f(path, std::ios::binary | std::ios::ate);
  if (!f) fatal("Binary::loadFromPath: cannot open " + path);
  std::streamsize n = f.tellg();
  f.seekg(0);
  std::vector<std::uint8_t> bytes(static_cast<size_t>(n));
  f.read(reinterpret_cast<char *>(bytes.data()), n);
  return makeBinary(std::move(bytes));
}
Binary Binary::loadFromMemory(const void *data, size_t size) {
  TTRT_ASSERT(data != nullptr, "Binary::loadFromMemory: null buffer");
  const auto *p = static_cast<const std::uint8_t *>(data);
  return makeBinary(std::vector<std::uint8_t>(p, p + size));
}
void Binary::store(const std::string &path) const {
  std::ofstream f(path, std::ios::binary);
  if (!f) fatal("Binary::store: cannot open " + path);
  f.write(reinterpret_cast<const char *>(handle->bytes.data()), static_cast<std::streamsize>(handle->bytes.size()));
}
std::string Binary::getFileIdentifier() const { return std::string(reinterpret_cast<const char *>(handle->bytes.data() + 8), 4); }
std::string Binary::getVersion() const {
  const std::uint8_t *v = handle->root.structPtr(schema::TTNNBinary::f_version, 8);
  if (!v) return "0.0.0";
  std::ostringstream os;
  os << fb::readScalar<std::uint16_t>(v) << "." << fb::readScalar<std::uint16_t>(v + 2) << "." << fb::readScalar<std::uint32_t>(v + 4);
  return os.str();
}
std::string Binary::getSchemaHash() const { return std::string(handle->root.string(schema::TTNNBinary::f_schema_hash)); }
std::uint64_t Binary::id() const { return handle->id; }

static fb::Table programAt(const Binary &b, std::uint32_t idx) {
  auto programs = b.handle->root.tables(schema::TTNNBinary::f_programs);
  TTRT_ASSERT(idx < programs.size(), "program index " + std::to_string(idx) + " out of range (binary has " +
                                         std::to_string(programs.size()) + " programs)");
  return programs[idx];
}
std::uint32_t Binary::getNumPrograms() const { return handle->root.tables(schema::TTNNBinary::f_programs).size(); }
std::string Binary::getProgramName(std::uint32_t i) const { return std::string(programAt(*this, i).string(schema::Program::f_name)); }
bool Binary::isProgramPrivate(std::uint32_t i) const { return programAt(*this, i).scalar<std::uint8_t>(schema::Program::f_private, 0) != 0; }
std::uint32_t Binary::getNumOps(std::uint32_t i) const { return programAt(*this, i).tables(schema::Program::f_operations).size(); }

std::vector<std::uint32_t> shapeFromTensorRef(const fb::Table &ref) {
  auto desc = ref.table(schema::TensorRef::f_desc);
  auto shp = desc.scalars<std::int32_t>(schema::TensorDesc::f_shape);
  std::vector<std::uint32_t> out(shp.size());
  for (std::uint32_t i = 0; i < shp.size(); ++i) {
    TTRT_ASSERT(shp[i] >= 0, "the binary declares a tensor with a negative extent");
    out[i] = static_cast<std::uint32_t>(shp[i]);
  }
  requireRepresentableShape(out);   // every shape a binary declares passes here before anything is computed from it
  return out;
}

Layout layoutFromTensorRef(const fb::Table &ref) {
  auto md = ref.table(schema::TensorRef::f_desc).table(schema::TensorDesc::f_layout).table(schema::LayoutDesc::f_memory_desc);
  Layout l;
  l.storageType = static_cast<StorageType>(md.scalar<std::uint16_t>(schema::MemoryDesc::f_storage_type, 0));
  l.dataType = static_cast<DataType>(md.scalar<std::uint16_t>(schema::MemoryDesc::f_data_type, 0));
  // tile layout is encoded as tile_shape == 32x32 (runtime/lib/ttnn/utils/utils.cpp:57-60)
  const std::uint8_t *ts = md.structPtr(schema::MemoryDesc::f_tile_shape, 8);
  bool tile = ts && fb::readScalar<std::int32_t>(ts) == 32 && fb::readScalar<std::int32_t>(ts + 4) == 32;
  l.layout = tile ? TensorLayout::Tile : TensorLayout::RowMajor;
  return l;
}

static std::vector<TensorRefInfo> refInfos(const fb::TableVector &v) {
  std::vector<TensorRefInfo> out;
  for (std::uint32_t i = 0; i < v.size(); ++i) {
    TensorRefInfo r;
    r.globalId = v[i].scalar<std::uint32_t>(schema::TensorRef::f_global_id, 0);
    r.shape = shapeFromTensorRef(v[i]);
    r.layout = layoutFromTensorRef(v[i]);
    out.push_back(std::move(r));
  }
  return out;
}
std::vector<TensorRefInfo> Binary::getProgramInputs(std::uint32_t i) const { return refInfos(programAt(*this, i).tables(schema::Program::f_inputs)); }
std::vector<TensorRefInfo> Binary::getProgramOutputs(std::uint32_t i) const { return refInfos(programAt(*this, i).tables(schema::Program::f_outputs)); }

std::string Binary::getProgramOpsAsText(std::uint32_t i) const {
  auto ops = programAt(*this, i).tables(schema::Program::f_operations);
  std::ostringstream os;
  for (std::uint32_t k = 0; k < ops.size(); ++k) {
    auto t = static_cast<schema::OpType>(ops[k].scalar<std::uint8_t>(schema::Operation::f_type_type, 0));
    os << k << ": " << schema::opTypeName(t) << "  " << ops[k].string(schema::Operation::f_debug_info) << "\n";
  }
  return os.str();
}

// ---- JSON views and embedded goldens
static std::string jsonEscape(std::string_view in) {
  std::string o;
  for (char c : in) {
    switch (c) {
    case '"': o += "\\\""; break;
    case '\\': o += "\\\\"; break;
    case '\n': o += "\\n"; break;
    case '\t': o += "\\t"; break;
    default:
      if (static_cast<unsigned char>(c) < 0x20) { char b[8]; snprintf(b, sizeof(b), "\\u%04x", c); o += b; }
      else o += c;
    }
  }
  return o;
}
static std::string tensorRefJson(const fb::Table &ref) {
  std::ostringstream os;
  Layout l = layoutFromTensorRef(ref);
  os << "{\"global_id\": " << ref.scalar<std::uint32_t>(schema::TensorRef::f_global_id, 0) << ", \"desc\": {\"shape\": [";
  auto shp = shapeFromTensorRef(ref);
  for (size_t i = 0; i < shp.size(); ++i) os << (i ? ", " : "") << shp[i];
  os << "], \"layout\": {\"memory_desc\": {\"storage_type\": \"" << (l.storageType == StorageType::Device ? "DRAM" : "System")
     << "\", \"tile_shape\": " << (l.layout == TensorLayout::Tile ? "{\"y\": 32, \"x\": 32}" : "{\"y\": 1, \"x\": 1}")
     << ", \"data_type\": \"" << utils::dataTypeName(l.dataType) << "\"}}}}";
  return os.str();
}
static std::string refsJson(const fb::TableVector &v) {
  std::string o = "[";
  for (std::uint32_t k = 0; k < v.size(); ++k) o += (k ? ", " : "") + tensorRefJson(v[k]);
  return o + "]";
}
std::string Binary::getProgramInputsAsJson(std::uint32_t i) const { return refsJson(programAt(*this, i).tables(schema::Program::f_inputs)); }
std::string Binary::getProgramOutputsAsJson(std::uint32_t i) const { return refsJson(programAt(*this, i).tables(schema::Program::f_outputs)); }
std::string Binary::getProgramOpsAsJson(std::uint32_t i) const {
  auto ops = programAt(*this, i).tables(schema::Program::f_operations);
  std::ostringstream os;
  os << "[";
  for (std::uint32_t k = 0; k < ops.size(); ++k) {
    auto t = static_cast<schema::OpType>(ops[k].scalar<std::uint8_t>(schema::Operation::f_type_type, 0));
    os << (k ? ", " : "") << "{\"type_type\": \"" << schema::opTypeName(t) << "\", \"debug_info\": \""
       << jsonEscape(ops[k].string(schema::Operation::f_debug_info)) << "\", \"loc_info\": \""
       << jsonEscape(ops[k].string(schema::Operation::f_loc_info)) << "\"}";
  }
  os << "]";
  return os.str();
}
std::unordered_map<std::uint32_t, GoldenTensorInfo> Binary::getDebugInfoGolden(const std::string &loc) const {
  std::unordered_map<std::uint32_t, GoldenTensorInfo> out;
  for (std::uint32_t pi = 0; pi < getNumPrograms(); ++pi) {
    auto dbg = programAt(*this, pi).table(schema::Program::f_debug_info);
    if (!dbg) continue;
    auto info = dbg.table(schema::DebugInfo::f_golden_info);
    if (!info) continue;
    auto kvs = info.tables(schema::GoldenInfo::f_golden_map);
    for (std::uint32_t k = 0; k < kvs.size(); ++k) {
      if (kvs[k].string(schema::GoldenKV::f_key) != loc) continue;
      auto vals = kvs[k].tables(schema::GoldenKV::f_value);
      for (std::uint32_t v = 0; v < vals.size(); ++v) {
        auto gt = vals[v].table(schema::GoldenDeviceTensor::f_value);
        if (!gt) continue;
        GoldenTensorInfo g;
        g.name = std::string(gt.string(schema::GoldenTensor::f_name));
        auto shp = gt.scalars<std::int64_t>(schema::GoldenTensor::f_shape);
        auto str = gt.scalars<std::int64_t>(schema::GoldenTensor::f_stride);
        for (std::uint32_t q = 0; q < shp.size(); ++q) g.shape.push_back(shp[q]);
        for (std::uint32_t q = 0; q < str.size(); ++q) g.stride.push_back(str[q]);
        g.dataType = static_cast<::tt::target::DataType>(gt.scalar<std::uint16_t>(schema::GoldenTensor::f_dtype, 0));
        auto data = gt.scalars<std::uint8_t>(schema::GoldenTensor::f_data);
        g.data = data.data();
        g.size = data.size();
        out[vals[v].scalar<std::uint32_t>(schema::GoldenDeviceTensor::f_device, 0)] = g;
      }
    }
  }
  return out;
}

Layout getLayout(Binary binary, std::uint32_t programIndex, std::uint32_t inputIndex) {
  auto inputs = programAt(binary, programIndex).tables(schema::Program::f_inputs);
  TTRT_ASSERT(inputIndex < inputs.size(), "getLayout: input index out of range");
  return layoutFromTensorRef(inputs[inputIndex]);
}

// ============================================================================ device
// Caching allocator: blocks are kept per rounded size and reused; all work of a device is ordered
// on one stream, so reuse by a later launch is safe.  Freed to the driver at closeMeshDevice.
namespace {
DevicePool &pool() {
  // never destroyed: tensors held by other statics (the const-eval cache) return their blocks here
  // during process teardown, after function-local statics would already be gone
  static DevicePool *p = new DevicePool(PoolBackend{
      [](void **ptr, size_t bytes) { return ttm_malloc(ptr, bytes); }, [](void *ptr) { return ttm_free(ptr); },
      []() { return ttm_device_sync(); }});
  return *p;
}
}  // namespace

DeviceState::~DeviceState() {
  if (open && stream) ttm_stream_destroy(stream);
}

size_t getNumAvailableDevices() {
  int n = 0;
  ttm_device_count(&n);
  return static_cast<size_t>(n);
}

Device openMeshDevice(const MeshDeviceOptions &options) {
  TTRT_ASSERT(options.meshShape.size() == 2 && options.meshShape[0] * options.meshShape[1] == 1,
              "openMeshDevice: this backend drives one GPU; mesh shape must be 1x1");
  TTRT_ASSERT(getNumAvailableDevices() >= 1, "openMeshDevice: no GPU visible");
  auto st = std::make_shared<DeviceState>();
  st->deviceId = options.deviceIds.empty() ? 0 : options.deviceIds[0];
  TTM_CALL(ttm_set_device(st->deviceId));
  TTM_CALL(ttm_stream_create(&st->stream));
  st->open = true;
  {
    std::lock_guard<std::mutex> g(deviceRegistry().mu);
    deviceRegistry().devices.push_back(st);
  }
  return Device{st};
}

void requireNotCapturing(const std::shared_ptr<DeviceState> &dev, const char *what) {
  TTRT_ASSERT(!(dev && dev->capturing), std::string(what) + " is not possible while a trace is being captured: "
                                           "host transfers and waits cannot be recorded");
}

void beginTraceCapture(const std::shared_ptr<DeviceState> &dev, std::uint32_t traceId) {
  TTRT_ASSERT(dev && dev->open, "begin_trace_capture: device is not open");
  TTRT_ASSERT(!dev->capturing, "begin_trace_capture: a capture is already in progress on this device");
  pool().beginRecording();
  int rc = ttm_graph_begin_capture(dev->stream);
  if (rc != 0) {
    pool().unpin(pool().endRecording());
    hipCheck(rc, "ttm_graph_begin_capture");
  }
  dev->capturing = true;
  dev->capturingTraceId = traceId;
}

void endTraceCapture(const std::shared_ptr<DeviceState> &dev, std::uint32_t traceId) {
  TTRT_ASSERT(dev && dev->capturing, "end_trace_capture: no capture is in progress");
  TTRT_ASSERT(dev->capturingTraceId == traceId, "end_trace_capture: trace id does not match the capture in progress");
  dev->capturing = false;
  TraceData td;
  td.traceId = traceId;
  td.blocks = pool().endRecording();
  int rc = ttm_graph_end_capture(dev->stream, &td.graphExec, &td.numNodes);
  if (rc != 0) {
    pool().unpin(td.blocks);
    hipCheck(rc, "ttm_graph_end_capture");
  }
  dev->traces[traceId] = std::move(td);
}

void abortTraceCapture(const std::shared_ptr<DeviceState> &dev) {
  if (!dev || !dev->capturing) return;
  dev->capturing = false;
  auto blocks = pool().endRecording();
  void *exec = nullptr;
  size_t nodes = 0;
  if (ttm_graph_end_capture(dev->stream, &exec, &nodes) == 0 && exec) ttm_graph_destroy(exec);
  pool().unpin(blocks);
}

void executeTrace(const std::shared_ptr<DeviceState> &dev, std::uint32_t traceId, bool blocking) {
  TTRT_ASSERT(dev && dev->open, "execute_trace: device is not open");
  TTRT_ASSERT(!dev->capturing, "execute_trace: a capture is in progress");
  auto it = dev->traces.find(traceId);
  TTRT_ASSERT(it != dev->traces.end(), "execute_trace: unknown trace id " + std::to_string(traceId));
  TTM_CALL(ttm_graph_launch(it->second.graphExec, dev->stream));
  if (blocking) TTM_CALL(ttm_stream_sync(dev->stream));
}

void releaseTrace(const std::shared_ptr<DeviceState> &dev, std::uint32_t traceId) {
  auto it = dev->traces.find(traceId);
  if (it == dev->traces.end()) return;
  TTM_CALL(ttm_stream_sync(dev->stream));
  TTM_CALL(ttm_graph_destroy(it->second.graphExec));
  pool().unpin(it->second.blocks);
  for (auto kv = dev->traceCache.begin(); kv != dev->traceCache.end();)
    kv = kv->second == traceId ? dev->traceCache.erase(kv) : std::next(kv);
  dev->traces.erase(it);
}

void closeMeshDevice(Device d) {
  TTRT_ASSERT(d.handle && d.handle->open, "closeMeshDevice: device is not open");
  TTRT_ASSERT(!d.handle->capturing, "closeMeshDevice: a trace capture is in progress");
  TTM_CALL(ttm_stream_sync(d.handle->stream));
  while (!d.handle->traces.empty()) releaseTrace(d.handle, d.handle->traces.begin()->first);
  d.handle->traceCache.clear();
  {
    // const-eval results are memory of this device: they go back to the pool before the pool returns it to the driver
    std::map<ConstEvalKey, ConstEvalEntry> dropped;   // destroyed after the lock is released
    {
      std::lock_guard<std::mutex> g(d.handle->constEvalMu);
      dropped.swap(d.handle->constEval);
    }
  }
  pool().release();
  TTM_CALL(ttm_stream_destroy(d.handle->stream));
  d.handle->stream = nullptr;
  d.handle->open = false;
}

std::string getDeviceName(Device) {
  char buf[256];
  TTM_CALL(ttm_device_name(buf, sizeof(buf)));
  return buf;
}

// ============================================================================ tensors
static std::atomic<std::uint64_t> g_tensorVersion{1};
std::uint64_t nextTensorVersion() { return g_tensorVersion++; }

Tensor makeHostTensor(const std::vector<std::uint32_t> &shape, DataType dtype, TensorLayout layout) {
  auto t = std::make_shared<TensorImpl>();
  t->shape = shape; t->dtype = dtype; t->layout = layout; t->storage = StorageType::Host;
  t->bytes = tensorBytes(shape, dtype, layout);
  t->data = std::shared_ptr<void>(std::malloc(std::max<size_t>(t->bytes, 1)), std::free);
  TTRT_ASSERT(t->data != nullptr, "host allocation failed");
  t->version = g_tensorVersion++;
  return Tensor{t};
}

Tensor makeDeviceTensor(const std::shared_ptr<DeviceState> &dev, const std::vector<std::uint32_t> &shape, DataType dtype,
                        TensorLayout layout) {
  TTRT_ASSERT(dev && dev->open, "device is not open");
  auto t = std::make_shared<TensorImpl>();
  t->shape = shape; t->dtype = dtype; t->layout = layout; t->storage = StorageType::Device;
  t->bytes = tensorBytes(shape, dtype, layout);
  size_t bytes = t->bytes;
  void *p = pool().alloc(bytes);
  t->data = std::shared_ptr<void>(p, [bytes](void *q) { pool().free(q, bytes); });
  t->device = dev;
  t->version = g_tensorVersion++;
  return Tensor{t};
}

static bool isContiguous(const std::vector<std::uint32_t> &shape, const std::vector<std::int64_t> &stride) {
  if (stride.empty()) return true;
  return stride == utils::calculateStride(shape);
}

// gather a strided host buffer into contiguous bytes (runtime/lib/ttnn/runtime.cpp:105-162)
static std::vector<std::uint8_t> gatherContiguous(const void *data, const std::vector<std::uint32_t> &shape,
                                                 const std::vector<std::int64_t> &stride, std::uint32_t itemsize) {
  std::int64_t n = volume(shape);
  std::vector<std::uint8_t> out(static_cast<size_t>(n) * itemsize);
  std::vector<std::uint32_t> idx(shape.size(), 0);
  const auto *src = static_cast<const std::uint8_t *>(data);
  for (std::int64_t i = 0; i < n; ++i) {
    std::int64_t off = 0;
    for (size_t d = 0; d < shape.size(); ++d) off += static_cast<std::int64_t>(idx[d]) * stride[d];
    std::memcpy(out.data() + static_cast<size_t>(i) * itemsize, src + off * itemsize, itemsize);
    for (int d = static_cast<int>(shape.size()) - 1; d >= 0; --d) {
      if (++idx[d] < shape[d]) break;
      idx[d] = 0;
    }
  }
  return out;
}

Tensor createOwnedHostTensor(const void *data, const std::vector<std::uint32_t> &shape, const std::vector<std::int64_t> &stride,
                             std::uint32_t itemsize, DataType dataType) {
  TTRT_ASSERT(!utils::isBlockFormatDataType(dataType), "host tensors cannot be created in a block-float type");
  TTRT_ASSERT(itemsize == utils::dataTypeElementSize(dataType), "createOwnedHostTensor: itemsize does not match the data type");
  TTRT_ASSERT(stride.empty() || stride.size() == shape.size(), "createOwnedHostTensor: stride rank differs from shape rank");
  const void *src = data;
  std::vector<std::uint8_t> gathered;
  if (data && !isContiguous(shape, stride)) {
    gathered = gatherContiguous(data, shape, stride, itemsize);
    src = gathered.data();
  }
  DataType use = dataType;
  if (!utils::isSupportedDataType(dataType)) use = utils::getUnsupportedDataTypeAlias(dataType);
  Tensor t = makeHostTensor(shape, use, TensorLayout::RowMajor);
  if (src) utils::handleBufferCast(src, t.handle->data.get(), dataType, use, volume(shape));
  return t;
}

Tensor createBorrowedHostTensor(void *data, const std::vector<std::uint32_t> &shape, const std::vector<std::int64_t> &stride,
                                std::uint32_t itemsize, DataType dataType) {
  TTRT_ASSERT(data != nullptr, "Cannot create borrowed tensor with null data");
  TTRT_ASSERT(isContiguous(shape, stride), "Cannot create borrowed tensor from non-contiguous data");
  if (!utils::isSupportedDataType(dataType)) return createOwnedHostTensor(data, shape, stride, itemsize, dataType);
  TTRT_ASSERT(itemsize == utils::dataTypeElementSize(dataType), "createBorrowedHostTensor: itemsize does not match the data type");
  auto t = std::make_shared<TensorImpl>();
  t->shape = shape; t->dtype = dataType; t->layout = TensorLayout::RowMajor; t->storage = StorageType::Host;
  t->bytes = tensorBytes(shape, dataType, TensorLayout::RowMajor);
  t->data = std::shared_ptr<void>(data, [](void *) {});
  t->borrowed = true;
  t->version = g_tensorVersion++;
  return Tensor{t};
}

Tensor createUnsafeBorrowedHostTensor(Tensor owned) {
  TTRT_ASSERT(isTensorAllocated(owned) && owned.handle->storage == StorageType::Host, "createUnsafeBorrowedHostTensor requires a host tensor");
  TTRT_ASSERT(owned.handle->layout == TensorLayout::RowMajor, "createUnsafeBorrowedHostTensor requires ROW_MAJOR layout");
  const TensorDesc desc = getTensorDesc(owned);
  return createBorrowedHostTensor(owned.handle->data.get(), desc.shape, desc.stride, utils::dataTypeElementSize(desc.dataType), desc.dataType);
}

Tensor createEmptyTensor(Device device, Layout layout, const std::vector<std::uint32_t> &shape, const std::vector<std::int64_t> &,
                         std::uint32_t) {
  if (layout.storageType == StorageType::Device) return makeDeviceTensor(device.handle, shape, layout.dataType, layout.layout);
  return makeHostTensor(shape, layout.dataType, layout.layout);
}

bool isTensorAllocated(Tensor t) { return t.handle && t.handle->data != nullptr; }
DataType getTensorDataType(Tensor t) { return t.handle->dtype; }
std::uint32_t getTensorElementSize(Tensor t) {
  return utils::isBlockFormatDataType(t.handle->dtype) ? 1 : utils::dataTypeElementSize(t.handle->dtype);
}
// physical volume: the elements the storage holds, the tile layout's padding included (runtime/lib/ttnn/runtime.cpp:542-552)
std::uint32_t getTensorVolume(Tensor t) {
  return static_cast<std::uint32_t>(t.handle->layout == TensorLayout::Tile ? paddedVolume(t.handle->shape) : volume(t.handle->shape));
}
std::uint32_t getTensorLogicalVolume(Tensor t) { return static_cast<std::uint32_t>(volume(t.handle->shape)); }
std::vector<std::uint32_t> getTensorShape(Tensor t) { return t.handle->shape; }
std::vector<std::int64_t> getTensorStride(Tensor t) { return utils::calculateStride(t.handle->shape); }
TensorDesc getTensorDesc(Tensor t) { return TensorDesc{t.handle->shape, getTensorStride(t), t.handle->dtype}; }
bool getTensorRetain(Tensor t) { return t.handle->retain.load(); }
void setTensorRetain(Tensor t, bool r) { t.handle->retain.store(r); }
Layout getTensorLayout(Tensor t) { return Layout{t.handle->storage, t.handle->layout, t.handle->dtype}; }
bool hasLayout(Tensor t, Layout l) { return getTensorLayout(t) == l; }

std::vector<std::byte> getTensorDataBuffer(Tensor t) {
  TTRT_ASSERT(isTensorAllocated(t), "getTensorDataBuffer: tensor is deallocated");
  Tensor h = t;
  if (t.handle->storage == StorageType::Device) h = toHost(t, /*untilize=*/true)[0];
  std::vector<std::byte> out(h.handle->bytes);
  std::memcpy(out.data(), h.handle->data.get(), h.handle->bytes);
  return out;
}

void wait(Event) {}
void wait(Tensor t, std::optional<std::uint8_t>) {
  TTRT_ASSERT(t.handle != nullptr, "wait: null tensor");
  if (t.handle->storage == StorageType::Device && t.handle->device && t.handle->device->open) {
    std::lock_guard<std::recursive_mutex> g(t.handle->device->mu);
    requireNotCapturing(t.handle->device, "wait");
    TTM_CALL(ttm_stream_sync(t.handle->device->stream));
  }
}
void wait(const std::vector<Tensor> &ts, std::optional<std::uint8_t> cq) {
  for (const auto &t : ts) wait(t, cq);
}

void deallocateTensor(Tensor &t, bool force) {
  if (!t.handle) return;
  if (t.handle->retain.load() && !force) return;  // runtime/lib/ttnn/operations/deletion/deallocate.cpp:16-18
  TTRT_ASSERT(!t.handle->borrowed || t.handle->storage != StorageType::Host || force,
              "Cannot deallocate host tensors with borrowed storage");
  t.handle->data.reset();
  t.handle->bytes = 0;
}

// ---------------------------------------------------------------------------- conversions
static int ttmDtype(DataType dt) { return static_cast<int>(dt); }  // same numbering as the C ABI

Tensor toDevice(const Tensor &h, const std::shared_ptr<DeviceState> &dev) {
  TTRT_ASSERT(h.handle->storage == StorageType::Host, "toDevice: tensor is not on the host");
  requireNotCapturing(dev, "a host to device transfer");
  Tensor d = makeDeviceTensor(dev, h.handle->shape, h.handle->dtype, h.handle->layout);
  TTM_CALL(ttm_memcpy_h2d(d.handle->data.get(), h.handle->data.get(), h.handle->bytes, dev->stream));
  TTM_CALL(ttm_stream_sync(dev->stream));  // the host buffer may be borrowed: do not outlive the call
  return d;
}

Tensor fromDevice(const Tensor &d) {
  TTRT_ASSERT(d.handle->storage == StorageType::Device, "fromDevice: tensor is not on the device");
  TTRT_ASSERT(d.handle->device && d.handle->device->open, "the tensor belongs to a device that has been closed");
  requireNotCapturing(d.handle->device, "a device to host transfer");
  Tensor h = makeHostTensor(d.handle->shape, d.handle->dtype, d.handle->layout);
  TTM_CALL(ttm_memcpy_d2h(h.handle->data.get(), d.handle->data.get(), d.handle->bytes, d.handle->device->stream));
  TTM_CALL(ttm_stream_sync(d.handle->device->stream));
  return h;
}

// ---- dumpTensor / loadTensor (runtime/include/tt/runtime/runtime.h:304-308; runtime/lib/ttnn/runtime.cpp:2613-2633).
// The reference passes the tensor to its device library's flatbuffer tensor writer, whose format is not part of the
// reference's sources.  The container here: "TTMT", version, data type, layout, rank, the extents, the payload size (all
// little-endian, 32 bits except the 64-bit size), then the payload in the tensor's own layout, so tile order and
// block-float bytes come back exactly as they were.
namespace {
constexpr char kTensorFileMagic[4] = {'T', 'T', 'M', 'T'};
constexpr std::uint32_t kTensorFileVersion = 1;
}  // namespace

void dumpTensor(Tensor tensor, const std::string &filePath) {
  TTRT_ASSERT(isTensorAllocated(tensor), "dumpTensor: tensor is deallocated");
  Tensor h = tensor.handle->storage == StorageType::Device ? fromDevice(tensor) : tensor;
  const TensorImpl &t = *h.handle;
  TTRT_ASSERT(t.shape.size() <= 8, "dumpTensor: tensor rank above 8");
  std::ofstream f(filePath, std::ios::binary | std::ios::trunc);
  TTRT_ASSERT(f.good(), "dumpTensor: cannot open '" + filePath + "' for writing");
  auto put32 = [&](std::uint32_t v) { f.write(reinterpret_cast<const char *>(&v), 4); };
  f.write(kTensorFileMagic, 4);
  put32(kTensorFileVersion);
  put32(static_cast<std::uint32_t>(t.dtype));
  put32(static_cast<std::uint32_t>(t.layout));
  put32(static_cast<std::uint32_t>(t.shape.size()));
  for (std::uint32_t e : t.shape) put32(e);
  const std::uint64_t bytes = t.bytes;
  f.write(reinterpret_cast<const char *>(&bytes), 8);
  f.write(static_cast<const char *>(t.data.get()), static_cast<std::streamsize>(t.bytes));
  f.flush();
  TTRT_ASSERT(f.good(), "dumpTensor: writing '" + filePath + "' failed");
}

Tensor loadTensor(const std::string &filePath, std::optional<Device> device) {
  std::ifstream f(filePath, std::ios::binary);
  TTRT_ASSERT(f.good(), "loadTensor: cannot open '" + filePath + "'");
  auto get32 = [&]() {
    std::uint32_t v = 0;
    f.read(reinterpret_cast<char *>(&v), 4);
    TTRT_ASSERT(f.gcount() == 4, "loadTensor: '" + filePath + "' ends inside its header");
    return v;
  };
  char magic[4] = {};
  f.read(magic, 4);
  TTRT_ASSERT(f.gcount() == 4 && std::memcmp(magic, kTensorFileMagic, 4) == 0, "loadTensor: '" + filePath + "' is not a tensor file");
  const std::uint32_t version = get32();
  TTRT_ASSERT(version == kTensorFileVersion, "loadTensor: unknown tensor file version " + std::to_string(version));
  const std::uint32_t dtype = get32(), layout = get32(), rank = get32();
  TTRT_ASSERT(dtype <= static_cast<std::uint32_t>(DataType::Bool), "loadTensor: unknown data type " + std::to_string(dtype));
  TTRT_ASSERT(layout <= static_cast<std::uint32_t>(TensorLayout::Tile), "loadTensor: unknown layout " + std::to_string(layout));
  TTRT_ASSERT(rank <= 8, "loadTensor: tensor rank above 8");
  std::vector<std::uint32_t> shape(rank);
  for (auto &e : shape) e = get32();
  std::uint64_t bytes = 0;
  f.read(reinterpret_cast<char *>(&bytes), 8);
  TTRT_ASSERT(f.gcount() == 8, "loadTensor: '" + filePath + "' ends inside its header");
  const DataType dt = static_cast<DataType>(dtype);
  const TensorLayout lay = static_cast<TensorLayout>(layout);
  TTRT_ASSERT(utils::isSupportedDataType(dt), "loadTensor: the file holds a data type tensors are never stored in");
  TTRT_ASSERT(!utils::isBlockFormatDataType(dt) || lay == TensorLayout::Tile, "loadTensor: block-float data outside the tile layout");
  TTRT_ASSERT(bytes == tensorBytes(shape, dt, lay), "loadTensor: the payload size does not match the shape, data type and layout");
  Tensor t = makeHostTensor(shape, dt, lay);
  f.read(static_cast<char *>(t.handle->data.get()), static_cast<std::streamsize>(bytes));
  TTRT_ASSERT(static_cast<std::uint64_t>(f.gcount()) == bytes, "loadTensor: '" + filePath + "' ends inside its payload");
  if (device.has_value()) return toDevice(t, device->handle);
  return t;
}

// Device-side change of layout and/or dtype; the order mirrors LayoutConverter
// (runtime/lib/ttnn/types/layout_converter.cpp:196-215, 363-379): tilize / untilize and typecast are
// separate steps except for block-float targets, where the pack kernel tilizes on the fly.
Tensor convertOnDevice(const Tensor &src, TensorLayout layout, DataType dtype) {
  const TensorImpl &s = *src.handle;
  TTRT_ASSERT(s.storage == StorageType::Device, "convertOnDevice: tensor is not on the device");
  if (s.layout == layout && s.dtype == dtype) return src;
  TTRT_ASSERT(s.device && s.device->open, "the tensor belongs to a device that has been closed");
  void *stream = s.device->stream;
  Dims3 d = dims3(s.shape);
  const bool srcBfp = utils::isBlockFormatDataType(s.dtype), dstBfp = utils::isBlockFormatDataType(dtype);
  auto plainOk = [](DataType t) { return t == DataType::Float32 || t == DataType::BFloat16; };
  if (srcBfp) {
    TTRT_ASSERT(s.dtype == DataType::BFP_BFloat8 || s.dtype == DataType::BFP_BFloat4, "only bfp8_b / bfp4_b block formats are supported");
    DataType mid = plainOk(dtype) ? dtype : DataType::Float32;
    TensorLayout midLayout = dstBfp ? TensorLayout::Tile : layout;
    Tensor t = makeDeviceTensor(s.device, s.shape, mid, midLayout);
    TTM_CALL(ttm_bfp_unpack(s.data.get(), ttmDtype(s.dtype), t.handle->data.get(), ttmDtype(mid), static_cast<int>(midLayout),
                            d.batch, d.rows, d.cols, stream));
    return convertOnDevice(t, layout, dtype);
  }
  if (dstBfp) {
    TTRT_ASSERT(dtype == DataType::BFP_BFloat8 || dtype == DataType::BFP_BFloat4, "only bfp8_b / bfp4_b block formats are supported");
    TTRT_ASSERT(layout == TensorLayout::Tile, "block-float tensors must be in tile layout");
    Tensor plain = plainOk(s.dtype) ? src : convertOnDevice(src, s.layout, DataType::Float32);
    Tensor t = makeDeviceTensor(s.device, s.shape, dtype, TensorLayout::Tile);
    TTM_CALL(ttm_bfp_pack(plain.handle->data.get(), ttmDtype(plain.handle->dtype), static_cast<int>(plain.handle->layout),
                          t.handle->data.get(), ttmDtype(dtype), d.batch, d.rows, d.cols, stream));
    return t;
  }
  Tensor cur = src;
  if (cur.handle->layout != layout) {
    Tensor t = makeDeviceTensor(s.device, s.shape, cur.handle->dtype, layout);
    int es = static_cast<int>(utils::dataTypeElementSize(cur.handle->dtype));
    if (layout == TensorLayout::Tile)
      TTM_CALL(ttm_tilize(cur.handle->data.get(), t.handle->data.get(), d.batch, d.rows, d.cols, es, stream));
    else
      TTM_CALL(ttm_untilize(cur.handle->data.get(), t.handle->data.get(), d.batch, d.rows, d.cols, es, stream));
    cur = t;
  }
  if (cur.handle->dtype != dtype) {
    Tensor t = makeDeviceTensor(s.device, s.shape, dtype, layout);
    std::int64_t n = layout == TensorLayout::Tile ? paddedVolume(s.shape) : volume(s.shape);
    TTM_CALL(ttm_typecast(cur.handle->data.get(), ttmDtype(cur.handle->dtype), t.handle->data.get(), ttmDtype(dtype), n, stream));
    cur = t;
  }
  return cur;
}

Tensor toLayout(Tensor tensor, Device device, Layout layout, std::optional<bool> retain) {
  TTRT_ASSERT(isTensorAllocated(tensor), "toLayout: tensor is deallocated");
  TTRT_ASSERT(device.handle && device.handle->open, "toLayout: device is not open");
  std::lock_guard<std::recursive_mutex> g(device.handle->mu);
  Tensor cur = tensor;
  const bool needsDevice = layout.storageType == StorageType::Device || cur.handle->layout != layout.layout ||
                           cur.handle->dtype != layout.dataType;
  if (cur.handle->storage == StorageType::Host && needsDevice) cur = toDevice(cur, device.handle);
  if (cur.handle->storage == StorageType::Device) cur = convertOnDevice(cur, layout.layout, layout.dataType);
  if (layout.storageType == StorageType::Host && cur.handle->storage == StorageType::Device) cur = fromDevice(cur);
  // one decision for both sides, as in runtime/lib/ttnn/runtime.cpp:906-932: the result carries the flag, and the input is
  // consumed exactly when the flag is off
  const bool shouldRetain = retain.value_or(getTensorRetain(tensor));
  if (cur.handle == tensor.handle) {
    // already in the requested layout: hand back the same tensor, nothing to free
    setTensorRetain(cur, shouldRetain);
    return cur;
  }
  setTensorRetain(cur, shouldRetain);
  if (!shouldRetain && !tensor.handle->borrowed) {   // borrowed host memory is the caller's
    Tensor t = tensor;
    deallocateTensor(t, false);
  }
  return cur;
}

std::vector<Tensor> toHost(Tensor tensor, bool untilize, bool /*blocking*/) {
  TTRT_ASSERT(isTensorAllocated(tensor), "toHost: tensor is deallocated");
  if (tensor.handle->storage == StorageType::Host) return {tensor};
  std::unique_lock<std::recursive_mutex> g;
  if (tensor.handle->device) g = std::unique_lock<std::recursive_mutex>(tensor.handle->device->mu);
  Tensor cur = tensor;
  if (untilize) {
    // block-float tensors read back as float32 (runtime/lib/ttnn/runtime.cpp:450-466)
    DataType dt = utils::isBlockFormatDataType(cur.handle->dtype) ? DataType::Float32 : cur.handle->dtype;
    cur = convertOnDevice(cur, TensorLayout::RowMajor, dt);
  }
  return {fromDevice(cur)};
}

void memcpy(void *dst, Tensor src, std::optional<DataType> target) {
  TTRT_ASSERT(dst != nullptr, "memcpy: null destination");
  TTRT_ASSERT(isTensorAllocated(src), "memcpy: source tensor is deallocated");
  TTRT_ASSERT(src.handle->storage == StorageType::Host, "memcpy: source must be a host tensor");
  if (target.has_value() && *target != src.handle->dtype) {
    TTRT_ASSERT(!utils::isBlockFormatDataType(src.handle->dtype), "memcpy: cannot cast a block-float tensor");
    utils::handleBufferCast(src.handle->data.get(), dst, src.handle->dtype, *target, volume(src.handle->shape));
    return;
  }
  std::memcpy(dst, src.handle->data.get(), src.handle->bytes);
}

void memcpy(Tensor dst, Tensor src) {
  TTRT_ASSERT(isTensorAllocated(dst) && isTensorAllocated(src), "memcpy: tensor is deallocated");
  TTRT_ASSERT(dst.handle->bytes == src.handle->bytes, "memcpy: tensors differ in size");
  const bool dDev = dst.handle->storage == StorageType::Device, sDev = src.handle->storage == StorageType::Device;
  std::unique_lock<std::recursive_mutex> g;
  if (dDev && dst.handle->device) g = std::unique_lock<std::recursive_mutex>(dst.handle->device->mu);
  else if (sDev && src.handle->device) g = std::unique_lock<std::recursive_mutex>(src.handle->device->mu);
  if (!dDev && !sDev) {
    std::memcpy(dst.handle->data.get(), src.handle->data.get(), src.handle->bytes);
  } else if (dDev && !sDev) {
    requireNotCapturing(dst.handle->device, "a host to device copy");
    TTM_CALL(ttm_memcpy_h2d(dst.handle->data.get(), src.handle->data.get(), src.handle->bytes, dst.handle->device->stream));
    TTM_CALL(ttm_stream_sync(dst.handle->device->stream));
  } else if (!dDev && sDev) {
    requireNotCapturing(src.handle->device, "a device to host copy");
    TTM_CALL(ttm_memcpy_d2h(dst.handle->data.get(), src.handle->data.get(), src.handle->bytes, src.handle->device->stream));
    TTM_CALL(ttm_stream_sync(src.handle->device->stream));
  } else {
    TTM_CALL(ttm_memcpy_d2d(dst.handle->data.get(), src.handle->data.get(), src.handle->bytes, dst.handle->device->stream));
  }
}

std::vector<Tensor> submit(Device device, Binary binary, std::uint32_t programIndex, std::vector<Tensor> &inputs) {
  TTRT_ASSERT(device.handle && device.handle->open, "submit: device is not open");
  TTRT_ASSERT(binary.handle != nullptr, "submit: null binary");
  // one program at a time per device: its launches share one stream, one workspace and, while a trace is being captured,
  // one recording.  Threads that drive different devices do not meet here (test/python/.../test_data_parallel.py:58-75).
  std::lock_guard<std::recursive_mutex> programLock(device.handle->mu);
  try {
    return executeProgram(device.handle, binary, programIndex, inputs);
  } catch (...) {
    abortTraceCapture(device.handle);  // an op that failed while a trace was being recorded must not leave the stream capturing
    throw;
  }
}

// ---------------------------------------------------------------------------- debug
namespace debug {
Hooks &Hooks::get(std::optional<CallbackFn> pre, std::optional<CallbackFn> post, std::optional<ProgramCallbackFn> preProgram,
                  std::optional<ProgramCallbackFn> postProgram) {
  static Hooks h;
  if (pre.has_value()) h.preOperatorCallback = pre;
  if (post.has_value()) h.postOperatorCallback = post;
  if (preProgram.has_value()) h.preProgramCallback = preProgram;
  if (postProgram.has_value()) h.postProgramCallback = postProgram;
  return h;
}
void Hooks::unregisterHooks() {
  preOperatorCallback.reset();
  postOperatorCallback.reset();
  preProgramCallback.reset();
  postProgramCallback.reset();
}
static std::mutex g_statsMu;
Stats &Stats::get() {
  static Stats s;
  return s;
}
void Stats::incrementStat(const std::string &stat, std::int64_t value) {
  std::lock_guard<std::mutex> g(g_statsMu);
  counters[stat] += value;
}
std::int64_t Stats::getStat(const std::string &stat) const {
  std::lock_guard<std::mutex> g(g_statsMu);
  auto it = counters.find(stat);
  return it == counters.end() ? 0 : it->second;
}
void Stats::clear() {
  std::lock_guard<std::mutex> g(g_statsMu);
  counters.clear();
}
}  // namespace debug

std::string getOpDebugString(OpContext c) { return std::string(c.op.string(schema::Operation::f_debug_info)); }
std::string getOpLocInfo(OpContext c) { return std::string(c.op.string(schema::Operation::f_loc_info)); }

}  // namespace tt::runtime
