// Threads hammering the host runtime through its C ABI on the null device (tests/cpp/null_device.cpp): submits of a program
// with a const-eval part from several threads on one device, each thread creating and destroying its own weight tensors
// (const-eval entries come and go with them), while another thread opens hooks and reads statistics.  Built with
// -fsanitize=thread by tests/test_null_device.py: the device lock, the caching allocator, the const-eval cache with its
// destroy callbacks and the statistics must be free of data races and deadlocks.
#include <atomic>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <thread>
#include <vector>

#include "ttmlir_amd_runtime.h"

#define CK(call) do { if ((call) != 0) { std::fprintf(stderr, "%s failed: %s\n", #call, ttrt_last_error()); std::exit(2); } } while (0)

static const int kBF16 = 2, kBFP8 = 4, kTile = 1, kRowMajor = 0, kDevice = 1, kHost = 0;

int main() {
  // x [64, 128] @ bfp8(w [128, 160]) with the weights packed by a private const-eval program behind load_cached
  ttrt_builder *pb = nullptr;
  CK(ttrt_pb_create(&pb));
  uint32_t wshape[2] = {128, 160}, xshape[2] = {64, 128}, w0 = 0, wq = 0, prep = 0, x = 0, w = 0, y = 0, main_prog = 0;
  ttrt_layout dev_bf16{kDevice, kTile, kBF16}, dev_bfp8{kDevice, kTile, kBFP8};
  CK(ttrt_pb_begin_program(pb, "pack", 1));
  CK(ttrt_pb_input(pb, wshape, 2, &dev_bf16, &w0));
  CK(ttrt_pb_typecast(pb, w0, kBFP8, &wq));
  CK(ttrt_pb_output(pb, wq));
  CK(ttrt_pb_end_program(pb, &prep));
  CK(ttrt_pb_begin_program(pb, "main", 0));
  CK(ttrt_pb_input(pb, xshape, 2, &dev_bf16, &x));
  CK(ttrt_pb_input(pb, wshape, 2, &dev_bf16, &w));
  uint32_t cached = 0;
  const int wrank = 2;
  CK(ttrt_pb_load_cached(pb, prep, "pack", &w, 1, wshape, &wrank, &dev_bfp8, 1, &cached));
  CK(ttrt_pb_matmul(pb, x, cached, 0, 0, "", kBF16, &y));
  CK(ttrt_pb_output(pb, y));
  CK(ttrt_pb_end_program(pb, &main_prog));
  uint8_t *bytes = nullptr;
  size_t size = 0;
  CK(ttrt_pb_finish(pb, &bytes, &size));
  ttrt_binary *bin = nullptr;
  CK(ttrt_binary_load_memory(bytes, size, &bin));
  ttrt_free_bytes(bytes);
  ttrt_pb_destroy(pb);

  ttrt_device *dev = nullptr;
  CK(ttrt_device_open(&dev));
  std::vector<uint16_t> xdata(64 * 128, 0x3f80), wdata(128 * 160, 0x3c00);
  auto device_tensor = [&](const std::vector<uint16_t> &data, const uint32_t *shape) {
    ttrt_tensor *host = nullptr, *out = nullptr;
    CK(ttrt_tensor_create_host(data.data(), shape, 2, nullptr, 2, kBF16, 0, &host));
    CK(ttrt_to_layout(host, dev, &dev_bf16, 1, &out));
    ttrt_tensor_free(host);
    return out;
  };
  ttrt_tensor *shared_w = device_tensor(wdata, wshape);
  std::atomic<long> submits{0};
  std::atomic<bool> stop{false};
  auto worker = [&](int id) {
    ttrt_tensor *xt = device_tensor(xdata, xshape);
    for (int it = 0; it < 60; ++it) {
      // every third round on a weight tensor of its own, destroyed right after: an entry comes and goes
      ttrt_tensor *own = (it + id) % 3 == 0 ? device_tensor(wdata, wshape) : nullptr;
      ttrt_tensor *ins[2] = {xt, own ? own : shared_w}, *outs[4] = {};
      uint32_t n = 0;
      CK(ttrt_submit(dev, bin, main_prog, ins, 2, outs, 4, &n));
      CK(ttrt_wait(outs[0]));
      ttrt_tensor *host = nullptr;
      CK(ttrt_to_host(outs[0], 1, &host));
      ttrt_tensor_free(host);
      for (uint32_t i = 0; i < n; ++i) ttrt_tensor_free(outs[i]);
      if (own) ttrt_tensor_free(own);
      ++submits;
    }
    ttrt_tensor_free(xt);
  };
  std::thread reader([&] {
    while (!stop.load()) {
      int64_t v = 0;
      CK(ttrt_stat("ConstEvalCacheHit", &v));
      CK(ttrt_stat("ConstEvalCacheEvicted", &v));
      std::this_thread::yield();
    }
  });
  std::vector<std::thread> threads;
  for (int i = 0; i < 6; ++i) threads.emplace_back(worker, i);
  for (auto &t : threads) t.join();
  stop = true;
  reader.join();
  int64_t miss = 0, hit = 0, evicted = 0;
  CK(ttrt_stat("ConstEvalCacheMiss", &miss));
  CK(ttrt_stat("ConstEvalCacheHit", &hit));
  CK(ttrt_stat("ConstEvalCacheEvicted", &evicted));
  ttrt_tensor_free(shared_w);
  CK(ttrt_stat("ConstEvalCacheEvicted", &evicted));
  CK(ttrt_device_close(dev));
  ttrt_binary_free(bin);
  std::printf("submits %ld miss %lld hit %lld evicted %lld\n", submits.load(), (long long)miss, (long long)hit, (long long)evicted);
  return submits.load() == 360 && miss + hit == 360 && evicted == miss ? 0 : 1;
}
