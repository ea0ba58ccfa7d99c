/*
 * ttmlir_amd_runtime_arm.hpp -- header-only C++ arm over the C ABI of libttmlir_amd_rt.so, for the dispatch switch of
 * tt::runtime (runtime/lib/runtime.cpp:63-90).
 *
 * The reference's handle types (Tensor, Device, Binary, Layout: runtime/include/tt/runtime/types.h:112-135, 302-420) are
 * objects that carry a std::shared_ptr<void> named `handle` and are constructible from (shared_ptr<void>, DeviceRuntime).
 * This arm keeps the C ABI's opaque pointers inside those shared_ptrs, with the matching ttrt_*_free as the deleter, so it
 * needs nothing of the reference but those two properties: every function is a template over the handle types and the
 * value of the new DeviceRuntime enumerator.  It lives in its own namespace (tt::runtime::mi355x), so it can be compiled
 * into the reference next to tt::runtime::ttnn without clashing with it, and it links against the C symbols (ttrt_*) only,
 * which are the only symbols the library exports.  Errors become std::runtime_error("Fatal error: ..."), what LOG_FATAL
 * throws in the reference (runtime/include/tt/runtime/detail/common/logger.h:301-320).
 */
#ifndef TTMLIR_AMD_RUNTIME_ARM_HPP
#define TTMLIR_AMD_RUNTIME_ARM_HPP

#include <cstdint>
#include <memory>
#include <optional>
#include <stdexcept>
#include <string>
#include <vector>

#include "ttmlir_amd_runtime.h"

namespace tt::runtime::mi355x {

inline void check(int status, const char *what) {
  if (status != 0) throw std::runtime_error(std::string("Fatal error: ") + what + ": " + ttrt_last_error());
}

template <typename T>
inline T *raw(const std::shared_ptr<void> &handle) {
  return static_cast<T *>(handle.get());
}

inline std::shared_ptr<void> own(ttrt_tensor *t) {
  return std::shared_ptr<void>(t, [](void *p) { ttrt_tensor_free(static_cast<ttrt_tensor *>(p)); });
}

// tt::runtime::openMeshDevice / closeMeshDevice (runtime.h:155-157) for a 1x1 mesh
template <typename Device, typename RuntimeTag>
Device openMeshDevice(RuntimeTag tag) {
  ttrt_device *d = nullptr;
  check(ttrt_device_open(&d), "openMeshDevice");
  // closing is explicit in the reference's API; the deleter only drops the handle
  return Device(std::shared_ptr<void>(d, [](void *) {}), tag);
}
template <typename Device>
void closeMeshDevice(Device device) {
  check(ttrt_device_close(raw<ttrt_device>(device.handle)), "closeMeshDevice");
}

// Binary::loadFromPath (runtime/include/tt/runtime/types.h:336-360): the same .ttnn file
inline std::shared_ptr<void> loadBinary(const std::string &path) {
  ttrt_binary *b = nullptr;
  check(ttrt_binary_load_file(path.c_str(), &b), "Binary::loadFromPath");
  return std::shared_ptr<void>(b, [](void *p) { ttrt_binary_free(static_cast<ttrt_binary *>(p)); });
}

// createOwnedHostTensor / createBorrowedHostTensor (runtime.h:56-69)
template <typename Tensor, typename RuntimeTag>
Tensor createHostTensor(RuntimeTag tag, const void *data, const std::vector<std::uint32_t> &shape,
                        const std::vector<std::uint32_t> &stride, std::uint32_t itemsize, int dataType, bool borrowed) {
  std::vector<std::int64_t> st(stride.begin(), stride.end());
  ttrt_tensor *t = nullptr;
  check(ttrt_tensor_create_host(data, shape.data(), static_cast<int>(shape.size()), st.empty() ? nullptr : st.data(), itemsize,
                                dataType, borrowed ? 1 : 0, &t),
        "createHostTensor");
  return Tensor(own(t), nullptr, tag);
}

// getLayout (runtime.h:234-235) and toLayout (runtime.h:227-228)
inline ttrt_layout getLayout(const std::shared_ptr<void> &binary, std::uint32_t programIndex, std::uint32_t inputIndex) {
  ttrt_layout l{};
  check(ttrt_get_layout(raw<ttrt_binary>(binary), programIndex, inputIndex, &l), "getLayout");
  return l;
}
template <typename Tensor, typename Device, typename RuntimeTag>
Tensor toLayout(RuntimeTag tag, Tensor tensor, Device device, const ttrt_layout &layout, std::optional<bool> retain) {
  ttrt_tensor *out = nullptr;
  check(ttrt_to_layout(raw<ttrt_tensor>(tensor.handle), raw<ttrt_device>(device.handle), &layout,
                       retain.has_value() ? (*retain ? 1 : 0) : -1, &out),
        "toLayout");
  return Tensor(own(out), nullptr, tag);
}

// submit (runtime.h:299-301)
template <typename Tensor, typename Device, typename Binary, typename RuntimeTag>
std::vector<Tensor> submit(RuntimeTag tag, Device device, Binary executable, std::uint32_t programIndex, std::vector<Tensor> &inputs) {
  std::vector<ttrt_tensor *> in;
  for (auto &t : inputs) in.push_back(raw<ttrt_tensor>(t.handle));
  std::uint32_t n = 0;
  check(ttrt_binary_num_outputs(raw<ttrt_binary>(executable.handle), programIndex, &n), "submit");
  std::vector<ttrt_tensor *> out(n, nullptr);
  std::uint32_t got = 0;
  check(ttrt_submit(raw<ttrt_device>(device.handle), raw<ttrt_binary>(executable.handle), programIndex, in.data(),
                    static_cast<std::uint32_t>(in.size()), out.data(), n, &got),
        "submit");
  std::vector<Tensor> res;
  for (std::uint32_t i = 0; i < got; ++i) res.push_back(Tensor(own(out[i]), nullptr, tag));
  return res;
}

// wait (runtime.h:212-217), toHost (runtime.h:221-222), memcpy (runtime.h:237-240), deallocateTensor (runtime.h:244)
template <typename Tensor>
void wait(Tensor tensor) {
  check(ttrt_wait(raw<ttrt_tensor>(tensor.handle)), "wait");
}
template <typename Tensor, typename RuntimeTag>
std::vector<Tensor> toHost(RuntimeTag tag, Tensor tensor, bool untilize) {
  ttrt_tensor *out = nullptr;
  check(ttrt_to_host(raw<ttrt_tensor>(tensor.handle), untilize ? 1 : 0, &out), "toHost");
  return {Tensor(own(out), nullptr, tag)};
}
template <typename Tensor>
void memcpy(void *dst, Tensor src, std::optional<int> targetDataType = std::nullopt) {
  check(ttrt_memcpy_out(dst, raw<ttrt_tensor>(src.handle), targetDataType.value_or(-1)), "memcpy");
}
template <typename Tensor>
void deallocateTensor(Tensor &tensor, bool force) {
  check(ttrt_tensor_deallocate(raw<ttrt_tensor>(tensor.handle), force ? 1 : 0), "deallocateTensor");
}

}  // namespace tt::runtime::mi355x
#endif
