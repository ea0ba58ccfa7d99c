// Internal state behind the opaque handles of runtime.h.
#pragma once
#include <atomic>
#include <mutex>

#include "runtime.h"
#include "ttmlir_amd_hip.h"

namespace tt::runtime {

using ::tt::target::DataType;
using ::tt::target::StorageType;
using ::tt::target::TensorLayout;

void hipCheck(int status, const char *what);
#define TTM_CALL(expr) ::tt::runtime::hipCheck((expr), #expr)

struct DeviceState {
  int deviceId = 0;
  void *stream = nullptr;  // hipStream_t: all work of this device is ordered on it
  bool open = false;
  std::mutex mu;           // submit is re-entrant per device, one program at a time per stream
  ~DeviceState();
};

struct TensorImpl {
  std::vector<std::uint32_t> shape;  // logical shape
  DataType dtype = DataType::Float32;
  TensorLayout layout = TensorLayout::RowMajor;
  StorageType storage = StorageType::Host;
  std::shared_ptr<void> data;        // host bytes or device allocation
  size_t bytes = 0;
  bool borrowed = false;
  std::atomic<bool> retain{false};
  std::shared_ptr<DeviceState> device;  // for device tensors
  std::uint64_t version = 0;
};

struct BinaryImpl {
  std::vector<std::uint8_t> bytes;
  fb::Table root;
  std::uint64_t id = 0;
};

// [.., R, C] -> (batch, rows, cols); rank 0/1 tensors are a single row
struct Dims3 {
  std::int64_t batch = 1, rows = 1, cols = 1;
};
Dims3 dims3(const std::vector<std::uint32_t> &shape);
std::int64_t volume(const std::vector<std::uint32_t> &shape);
std::int64_t paddedVolume(const std::vector<std::uint32_t> &shape);
size_t tensorBytes(const std::vector<std::uint32_t> &shape, DataType dtype, TensorLayout layout);

Tensor makeDeviceTensor(const std::shared_ptr<DeviceState> &dev, const std::vector<std::uint32_t> &shape, DataType dtype,
                        TensorLayout layout);
Tensor makeHostTensor(const std::vector<std::uint32_t> &shape, DataType dtype, TensorLayout layout);

// layout / dtype / storage conversion used by toLayout, toHost and the layout op runners
Tensor convertOnDevice(const Tensor &src, TensorLayout layout, DataType dtype);
Tensor toDevice(const Tensor &hostTensor, const std::shared_ptr<DeviceState> &dev);
Tensor fromDevice(const Tensor &deviceTensor);

Layout layoutFromTensorRef(const fb::Table &tensorRef);
std::vector<std::uint32_t> shapeFromTensorRef(const fb::Table &tensorRef);

// program execution (executor.cpp)
std::vector<Tensor> executeProgram(const std::shared_ptr<DeviceState> &dev, const Binary &binary, std::uint32_t programIndex,
                                   std::vector<Tensor> &inputs);

}  // namespace tt::runtime
