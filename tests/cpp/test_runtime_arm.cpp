// The integration sketch for the reference's runtime dispatch, compiled: a fourth arm of that dispatch that forwards to the C ABI.
// The three structs below are stand-ins with the two properties the arm needs of the reference's handle types
// (runtime/include/tt/runtime/types.h:112-135): a shared_ptr<void> member `handle` and construction from
// (handle, ..., DeviceRuntime).  Runs on the host: it loads a binary that the Python side wrote and walks its metadata;
// nothing here touches a GPU.
#include <cstdio>
#include <cstring>

#include "ttmlir_amd_runtime_arm.hpp"

namespace tt::runtime {
enum class DeviceRuntime { Disabled, TTNN, TTMetal, MI355X };
struct Device {
  std::shared_ptr<void> handle;
  DeviceRuntime rt;
  Device(std::shared_ptr<void> h, DeviceRuntime r) : handle(std::move(h)), rt(r) {}
};
struct Tensor {
  std::shared_ptr<void> handle, event;
  DeviceRuntime rt;
  Tensor(std::shared_ptr<void> h, std::shared_ptr<void> e, DeviceRuntime r) : handle(std::move(h)), event(std::move(e)), rt(r) {}
};
struct Binary {
  std::shared_ptr<void> handle;
};

// runtime/lib/runtime.cpp:1285-1303 with the fourth lambda
std::vector<Tensor> submit(Device device, Binary executable, std::uint32_t programIndex, std::vector<Tensor> &inputs) {
  switch (device.rt) {
  case DeviceRuntime::MI355X:
    return ::tt::runtime::mi355x::submit(DeviceRuntime::MI355X, device, executable, programIndex, inputs);
  default:
    throw std::runtime_error("Fatal error: Device runtime not enabled.");
  }
}
}  // namespace tt::runtime

int main(int argc, char **argv) {
  using namespace tt::runtime;
  if (argc < 2) return 2;
  Binary bin{mi355x::loadBinary(argv[1])};
  std::uint32_t programs = 0, inputs = 0;
  mi355x::check(ttrt_binary_num_programs(mi355x::raw<ttrt_binary>(bin.handle), &programs), "num_programs");
  mi355x::check(ttrt_binary_num_inputs(mi355x::raw<ttrt_binary>(bin.handle), 0, &inputs), "num_inputs");
  const ttrt_layout lay = mi355x::getLayout(bin.handle, 0, 0);
  // host tensors work without a device: create, read back, free
  const float data[6] = {1, 2, 3, 4, 5, 6};
  float back[6] = {};
  Tensor t = mi355x::createHostTensor<Tensor>(DeviceRuntime::MI355X, data, {2, 3}, {3, 1}, 4, /*Float32*/ 0, false);
  mi355x::memcpy(back, t);
  if (std::memcmp(data, back, sizeof(data)) != 0) return 1;
  // errors arrive as exceptions with the library's message
  bool threw = false;
  try { mi355x::loadBinary("/nonexistent.ttnn"); } catch (const std::runtime_error &e) { threw = std::strstr(e.what(), "Fatal error") != nullptr; }
  if (!threw) return 1;
  std::printf("programs=%u inputs=%u layout=(%d,%d,%d)\n", programs, inputs, lay.storage, lay.layout, lay.dtype);
  return 0;
}
