// Internal state behind the opaque handles of runtime.h.
#pragma once
#include <atomic>
#include <functional>
#include <map>
#include <mutex>
#include <tuple>
#include <utility>
#include <vector>

#include "runtime.h"
#include "ttmlir_amd_hip.h"

namespace tt::runtime {

using ::tt::target::DataType;
using ::tt::target::StorageType;
using ::tt::target::TensorLayout;

void hipCheck(int status, const char *what);
#define TTM_CALL(expr) ::tt::runtime::hipCheck((expr), #expr)

// One captured trace: an executable HIP graph plus everything its recorded launches name.  The slots are the
// persistent tensors the trace reads and writes (TraceData, runtime/include/tt/runtime/detail/ttnn/types/trace_cache.h);
// `blocks` are the device allocations that held intermediates while the trace was recorded - they stay out of
// circulation until the trace is released, so a replay can never write into memory that was handed to someone else.
struct TraceData {
  std::uint32_t traceId = 0;
  void *graphExec = nullptr;
  size_t numNodes = 0;
  std::vector<Tensor> inputSlots, outputSlots;
  std::vector<std::pair<void *, size_t>> blocks;
  std::uint64_t lastUse = 0;   // DeviceState::traceClock at the last capture or replay
};

// (binary id, main program, capture program, execute program): MainProgramKey + CaptureExecuteProgramKey of the reference,
// then the device addresses of the device-resident inputs.  A recorded graph names those addresses (resident inputs are
// their own slots), so a call with other resident tensors is another trace: nothing is ever copied into, or re-versioned
// in, a tensor the trace does not own (a caller's parameter, a const-eval result that the const-eval cache still serves).
using TraceKey = std::tuple<std::uint64_t, std::uint32_t, std::uint32_t, std::uint32_t, std::vector<const void *>>;
// traces kept per capture_or_execute_trace op; the least recently used one is released beyond that
constexpr size_t kMaxTracesPerOp = 4;

// Results of a const-eval program (runtime/lib/ttnn/operations/cache/load_cached.cpp:20-90): valid while the versions of
// the tensors it was run on are those of the current inputs.
struct ConstEvalEntry {
  std::vector<std::uint64_t> inputVersions;
  std::vector<Tensor> outputs;
};
// binary id, const-eval program, versions of the tensors it ran on
using ConstEvalKey = std::tuple<std::uint64_t, std::uint32_t, std::vector<std::uint64_t>>;

struct DeviceState {
  int deviceId = 0;
  void *stream = nullptr;  // hipStream_t: all work of this device is ordered on it
  bool open = false;
  // Work on the stream of a device is issued by one thread at a time: submit, toLayout, toHost, wait and device copies
  // take this lock (recursive: a hook running inside submit may call toHost).  A capture in progress is thereby never
  // interleaved with the launches or the synchronisation of another thread.
  std::recursive_mutex mu;
  // trace state
  bool capturing = false;                         // between begin_trace_capture and end_trace_capture
  std::uint32_t capturingTraceId = 0;
  std::uint32_t nextTraceId = 1;
  std::map<std::uint32_t, TraceData> traces;      // by trace id: graphs recorded on this device
  std::map<TraceKey, std::uint32_t> traceCache;   // capture_or_execute_trace on these resident tensors -> trace id
  std::uint64_t traceClock = 0;
  // const-eval results by (binary id, program index, input versions), one entry per combination as in the reference's
  // GlobalTensorCache (device id, function hash, input versions; runtime/lib/ttnn/operations/cache/load_cached.cpp:24-38).
  // They are device memory of this device, so they live and die with it: dropped at closeMeshDevice, per binary when the
  // binary is destroyed, and singly when one of the tensors an entry was computed from is destroyed (nobody can ask for
  // it again).  Entries are always destroyed outside the lock: their tensors may carry such callbacks themselves.
  std::mutex constEvalMu;
  std::map<ConstEvalKey, ConstEvalEntry> constEval;
  ~DeviceState();
};

// trace capture on a device's stream (runtime.cpp): device allocations made or released between begin and end belong to
// the trace afterwards
void beginTraceCapture(const std::shared_ptr<DeviceState> &dev, std::uint32_t traceId);
void endTraceCapture(const std::shared_ptr<DeviceState> &dev, std::uint32_t traceId);
void executeTrace(const std::shared_ptr<DeviceState> &dev, std::uint32_t traceId, bool blocking);
void releaseTrace(const std::shared_ptr<DeviceState> &dev, std::uint32_t traceId);
void abortTraceCapture(const std::shared_ptr<DeviceState> &dev);  // no-op when no capture is in progress
// fails with `what` in the message when the device's stream is recording a trace (host transfers and waits are not
// recordable)
void requireNotCapturing(const std::shared_ptr<DeviceState> &dev, const char *what);

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
  // run when the tensor is destroyed: const-eval results computed from it are dropped with it
  // (runtime/lib/ttnn/operations/cache/global_tensor_cache.cpp, registerOnDestroyCallback)
  std::mutex destroyMu;
  std::vector<std::function<void()>> onDestroy;
  ~TensorImpl();
};

struct BinaryImpl {
  std::vector<std::uint8_t> bytes;
  fb::Table root;
  std::uint64_t id = 0;
  ~BinaryImpl();   // drops what open devices cached for this binary (const-eval results, traces)
};

// [.., R, C] -> (batch, rows, cols); rank 0/1 tensors are a single row
struct Dims3 {
  std::int64_t batch = 1, rows = 1, cols = 1;
};
Dims3 dims3(const std::vector<std::uint32_t> &shape);
std::int64_t volume(const std::vector<std::uint32_t> &shape);
std::int64_t paddedVolume(const std::vector<std::uint32_t> &shape);
size_t tensorBytes(const std::vector<std::uint32_t> &shape, DataType dtype, TensorLayout layout);

std::uint64_t nextTensorVersion();  // a tensor written in place takes a new version
Tensor makeDeviceTensor(const std::shared_ptr<DeviceState> &dev, const std::vector<std::uint32_t> &shape, DataType dtype,
                        TensorLayout layout);
Tensor makeHostTensor(const std::vector<std::uint32_t> &shape, DataType dtype, TensorLayout layout);

// layout / dtype / storage conversion used by toLayout, toHost and the layout op runners
Tensor convertOnDevice(const Tensor &src, TensorLayout layout, DataType dtype);
// invokeCpuOp without a running program: all it needs of one is the binary whose program carries the library
std::vector<Tensor> invokeCpuOpOf(const Binary &binary, std::uint32_t programIndex, OpContext opContext, const std::vector<Tensor> &inputs);
Tensor toDevice(const Tensor &hostTensor, const std::shared_ptr<DeviceState> &dev);
Tensor fromDevice(const Tensor &deviceTensor);

Layout layoutFromTensorRef(const fb::Table &tensorRef);
std::vector<std::uint32_t> shapeFromTensorRef(const fb::Table &tensorRef);

// program execution (executor.cpp)
std::vector<Tensor> executeProgram(const std::shared_ptr<DeviceState> &dev, const Binary &binary, std::uint32_t programIndex,
                                   std::vector<Tensor> &inputs);

}  // namespace tt::runtime
