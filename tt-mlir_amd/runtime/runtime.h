// tt::runtime-style host API of the MI355X backend.  Names, argument meaning and error behaviour
// follow runtime/include/tt/runtime/runtime.h:31-308 and types.h:112-150, 392-481 of tt-mlir, for the
// subset a `.ttnn` program needs on one device: load a binary, create host tensors, convert them to
// the layout the program expects, submit, wait, read back.  Errors throw std::runtime_error, like
// the reference's LOG_FATAL (runtime/include/tt/runtime/detail/common/logger.h:301-320).
#pragma once
#include <cstddef>
#include <cstdint>
#include <functional>
#include <memory>
#include <optional>
#include <string>
#include <string_view>
#include <unordered_map>
#include <vector>

#include "flatbuffer.h"
#include "schema_generated.h"

namespace tt::target {
using DataType = ::ttmlir_amd::schema::DataType;
using TensorLayout = ::ttmlir_amd::schema::TensorLayout;
using StorageType = ::ttmlir_amd::schema::StorageType;
}  // namespace tt::target

namespace tt::runtime {

namespace fb = ::ttmlir_amd::fb;

[[noreturn]] void fatal(const std::string &msg);
#define TTRT_ASSERT(cond, msg)                 \
  do {                                         \
    if (!(cond)) ::tt::runtime::fatal(msg);    \
  } while (0)

// ---- dtype helpers (runtime/lib/common/utils.cpp:140-290)
namespace utils {
std::uint32_t dataTypeElementSize(::tt::target::DataType dataType);
bool isBlockFormatDataType(::tt::target::DataType dataType);
std::uint64_t blockFormatTileSizeBytes(::tt::target::DataType dataType);
bool isSupportedDataType(::tt::target::DataType dataType);
::tt::target::DataType getUnsupportedDataTypeAlias(::tt::target::DataType unsupportedDataType);
void handleBufferCast(const void *oldBuffer, void *newBuffer, ::tt::target::DataType oldDataType,
                      ::tt::target::DataType newDataType, std::int64_t numElements);
std::vector<std::int64_t> calculateStride(const std::vector<std::uint32_t> &shape);
const char *dataTypeName(::tt::target::DataType dataType);
}  // namespace utils

struct TensorDesc {
  std::vector<std::uint32_t> shape;
  std::vector<std::int64_t> stride;
  ::tt::target::DataType dataType = ::tt::target::DataType::Float32;
  std::uint32_t elementSize() const { return utils::dataTypeElementSize(dataType); }
};

// Layout of a tensor as a program sees it (runtime/include/tt/runtime/detail/ttnn/types/types.h:112-135)
struct Layout {
  ::tt::target::StorageType storageType = ::tt::target::StorageType::Host;
  ::tt::target::TensorLayout layout = ::tt::target::TensorLayout::RowMajor;
  ::tt::target::DataType dataType = ::tt::target::DataType::Float32;
  bool operator==(const Layout &o) const { return storageType == o.storageType && layout == o.layout && dataType == o.dataType; }
};

struct DeviceState;
struct TensorImpl;
struct BinaryImpl;

struct Device {
  std::shared_ptr<DeviceState> handle;
};
struct Tensor {
  std::shared_ptr<TensorImpl> handle;
  explicit operator bool() const { return handle != nullptr; }
};
struct Event {
  std::shared_ptr<void> handle;
};

struct MeshDeviceOptions {
  std::vector<std::uint32_t> meshShape{1, 1};
  std::vector<int> deviceIds;
};

// ---- binary (runtime/lib/binary.cpp)
struct TensorRefInfo {
  std::uint32_t globalId = 0;
  std::vector<std::uint32_t> shape;
  Layout layout;
};
// golden tensor embedded in a program's debug info (include/ttmlir/Target/Common/debug_info.fbs:5-27)
struct GoldenTensorInfo {
  std::string name;
  std::vector<std::int64_t> shape, stride;
  ::tt::target::DataType dataType = ::tt::target::DataType::Float32;
  const std::uint8_t *data = nullptr;   // points into the binary; valid while the Binary is alive
  std::size_t size = 0;
};
struct Binary {
  std::shared_ptr<BinaryImpl> handle;
  static Binary loadFromPath(const std::string &path);
  static Binary loadFromMemory(const void *data, size_t size);  // copies
  void store(const std::string &path) const;
  std::string getFileIdentifier() const;
  std::string getVersion() const;
  std::string getSchemaHash() const;
  std::uint32_t getNumPrograms() const;
  std::string getProgramName(std::uint32_t programIndex) const;
  bool isProgramPrivate(std::uint32_t programIndex) const;
  std::vector<TensorRefInfo> getProgramInputs(std::uint32_t programIndex) const;
  std::vector<TensorRefInfo> getProgramOutputs(std::uint32_t programIndex) const;
  std::uint32_t getNumOps(std::uint32_t programIndex) const;
  std::string getProgramOpsAsText(std::uint32_t programIndex) const;
  // JSON views of one program (runtime/lib/binary.cpp:197-224) and the goldens keyed by op location (:233-253)
  std::string getProgramOpsAsJson(std::uint32_t programIndex) const;
  std::string getProgramInputsAsJson(std::uint32_t programIndex) const;
  std::string getProgramOutputsAsJson(std::uint32_t programIndex) const;
  std::unordered_map<std::uint32_t, GoldenTensorInfo> getDebugInfoGolden(const std::string &loc) const;
  std::uint64_t id() const;
};

// ---- debug hooks (runtime/include/tt/runtime/debug.h:77-157)
struct OpContext {
  fb::Table op;  // the Operation table
  std::uint32_t index = 0;
};
struct CallbackContext {
  void *programContext = nullptr;
};
// a TensorRef table of the binary, as hooks see an operation's operands (runtime/include/tt/runtime/types.h TensorRef)
struct TensorRef {
  fb::Table table;
};
namespace debug {
using CallbackFn = std::function<void(Binary, CallbackContext, OpContext)>;
using ProgramCallbackFn = std::function<void(Binary, CallbackContext)>;
struct Hooks {
  static Hooks &get(std::optional<CallbackFn> preOperator = std::nullopt, std::optional<CallbackFn> postOperator = std::nullopt,
                    std::optional<ProgramCallbackFn> preProgram = std::nullopt,
                    std::optional<ProgramCallbackFn> postProgram = std::nullopt);
  std::optional<CallbackFn> preOperatorCallback, postOperatorCallback;
  std::optional<ProgramCallbackFn> preProgramCallback, postProgramCallback;
  void unregisterHooks();
};
struct Stats {
  static Stats &get();
  void incrementStat(const std::string &stat, std::int64_t value = 1);
  std::int64_t getStat(const std::string &stat) const;
  void clear();
  std::unordered_map<std::string, std::int64_t> counters;
};
}  // namespace debug

// ---- API
size_t getNumAvailableDevices();
Device openMeshDevice(const MeshDeviceOptions &options = {});
void closeMeshDevice(Device parentMesh);
std::string getDeviceName(Device device);

Tensor createBorrowedHostTensor(void *data, const std::vector<std::uint32_t> &shape, const std::vector<std::int64_t> &stride,
                                std::uint32_t itemsize, ::tt::target::DataType dataType);
Tensor createOwnedHostTensor(const void *data, const std::vector<std::uint32_t> &shape, const std::vector<std::int64_t> &stride,
                             std::uint32_t itemsize, ::tt::target::DataType dataType);
// borrowed host tensor over the buffer of an owned row-major host tensor, no copy; it must not outlive the owner's buffer
// (runtime.h:70-76; runtime/lib/ttnn/runtime.cpp:283-304)
Tensor createUnsafeBorrowedHostTensor(Tensor ownedHostTensor);
Tensor createEmptyTensor(Device device, Layout layout, const std::vector<std::uint32_t> &shape,
                         const std::vector<std::int64_t> &stride, std::uint32_t itemsize);

bool isTensorAllocated(Tensor tensor);
::tt::target::DataType getTensorDataType(Tensor tensor);
std::vector<std::byte> getTensorDataBuffer(Tensor tensor);
std::uint32_t getTensorElementSize(Tensor tensor);
std::uint32_t getTensorVolume(Tensor tensor);          // elements in storage, tile padding included
std::uint32_t getTensorLogicalVolume(Tensor tensor);   // product of the shape
std::vector<std::uint32_t> getTensorShape(Tensor tensor);
std::vector<std::int64_t> getTensorStride(Tensor tensor);
TensorDesc getTensorDesc(Tensor tensor);
bool getTensorRetain(Tensor tensor);
void setTensorRetain(Tensor tensor, bool retain);
Layout getTensorLayout(Tensor tensor);
bool hasLayout(Tensor tensor, Layout layout);

void wait(Event event);
void wait(Tensor tensor, std::optional<std::uint8_t> cqId = std::nullopt);
void wait(const std::vector<Tensor> &tensors, std::optional<std::uint8_t> cqId = std::nullopt);

std::vector<Tensor> toHost(Tensor tensor, bool untilize = false, bool blocking = true);
Tensor toLayout(Tensor tensor, Device device, Layout layout, std::optional<bool> retain = std::nullopt);
Layout getLayout(Binary executableHandle, std::uint32_t programIndex, std::uint32_t inputIndex);
void memcpy(void *dst, Tensor src, std::optional<::tt::target::DataType> targetDataType = std::nullopt);
void memcpy(Tensor dst, Tensor src);
void deallocateTensor(Tensor &tensor, bool force = false);

std::string getOpDebugString(OpContext opContextHandle);
std::string getOpLocInfo(OpContext opContextHandle);
std::unordered_map<std::uint32_t, Tensor> getOpOutputTensor(OpContext opContextHandle, CallbackContext programContextHandle);
std::vector<TensorRef> getOpOutputRefs(OpContext opContextHandle);
std::vector<TensorRef> getOpInputRefs(OpContext opContextHandle);
std::vector<std::uint32_t> getTensorRefShape(TensorRef tensorRef);
::tt::target::DataType getTensorRefDataType(TensorRef tensorRef);
std::uint32_t getTensorRefGlobalId(TensorRef tensorRef);
std::optional<Tensor> retrieveTensorFromPool(CallbackContext programContextHandle, TensorRef tensorRef, bool untilize);
std::optional<Tensor> retrieveTensorFromPool(CallbackContext programContextHandle, std::uint32_t globalId, bool untilize);
void updateTensorInPool(CallbackContext programContextHandle, TensorRef tensorRef, Tensor srcTensor);
void updateTensorInPool(CallbackContext programContextHandle, std::uint32_t globalId, Tensor srcTensor);
size_t getProgramIndex(CallbackContext programContextHandle);
// the function behind a CpuOp on caller-supplied host tensors, which must match the op's declared inputs in number, shape
// and data type (runtime.h:285-292; runtime/lib/ttnn/runtime.cpp:2598-2611)
std::vector<Tensor> invokeCpuOp(CallbackContext programContextHandle, OpContext opContextHandle, const std::vector<Tensor> &inputs);

// every operation of a program in its order, nothing is run (runtime.h:294-297; runtime/lib/ttnn/runtime.cpp:2530-2540):
// the OpContext answers getOpDebugString / getOpLocInfo / getOpInputRefs / getOpOutputRefs
using OpWalkFn = std::function<void(OpContext)>;
void walkProgram(Binary executableHandle, std::uint32_t programIndex, const OpWalkFn &callback);

std::vector<Tensor> submit(Device deviceHandle, Binary executableHandle, std::uint32_t programIndex, std::vector<Tensor> &inputs);

// a tensor to a file and back (runtime.h:304-308).  The file keeps the tensor's own layout: tile order and block-float
// bytes are stored as they are.  loadTensor gives a host tensor, or a device tensor when a device is passed.
void dumpTensor(Tensor tensor, const std::string &filePath);
Tensor loadTensor(const std::string &filePath, std::optional<Device> device = std::nullopt);

}  // namespace tt::runtime
