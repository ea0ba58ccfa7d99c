// Damaged programs through the whole host runtime on the null device, under AddressSanitizer: each program file named on
// the command line is loaded, its inputs are created as zeroed device tensors of the shapes the intact program declares,
// and then copies of the file with a few bytes flipped are loaded and submitted.  Every outcome but one is fine - the
// reader refusing the binary, the executor refusing the program, the null device refusing a launch, or the program
// running: the process must not touch memory it does not own (built by tests/test_null_device.py with
// -fsanitize=address,undefined).
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <fstream>
#include <iterator>
#include <random>
#include <string>
#include <vector>

#include "ttmlir_amd_runtime.h"

int main(int argc, char **argv) {
  if (argc < 3) return 2;
  const int rounds = std::atoi(argv[1]);
  ttrt_device *dev = nullptr;
  if (ttrt_device_open(&dev) != 0) { std::fprintf(stderr, "device: %s\n", ttrt_last_error()); return 2; }
  long loaded = 0, ran = 0, refused = 0, out_of_bounds = 0;
  for (int f = 2; f < argc; ++f) {
    std::ifstream in(argv[f], std::ios::binary);
    std::vector<uint8_t> good((std::istreambuf_iterator<char>(in)), std::istreambuf_iterator<char>());
    ttrt_binary *bin = nullptr;
    if (ttrt_binary_load_memory(good.data(), good.size(), &bin) != 0) { std::fprintf(stderr, "%s: %s\n", argv[f], ttrt_last_error()); return 2; }
    uint32_t programs = 0, nin = 0;
    ttrt_binary_num_programs(bin, &programs);
    const uint32_t prog = programs - 1;
    ttrt_binary_num_inputs(bin, prog, &nin);
    std::vector<std::vector<uint32_t>> shapes(nin);
    std::vector<ttrt_layout> layouts(nin);
    for (uint32_t i = 0; i < nin; ++i) {
      uint32_t shape[8];
      int rank = 0;
      if (ttrt_binary_tensor_desc(bin, prog, 0, i, shape, &rank, &layouts[i]) != 0) return 2;
      shapes[i].assign(shape, shape + rank);
    }
    ttrt_binary_free(bin);
    std::mt19937 rng(1234 + f);
    for (int round = 0; round <= rounds; ++round) {
      std::vector<uint8_t> data = good;
      if (round > 0) {
        const int flips = 1 + (int)(rng() % 4);
        for (int k = 0; k < flips; ++k) {
          const size_t pos = 8 + rng() % (data.size() - 8);   // the size prefix and root offset stay: the reader checks them first
          switch (rng() % 3) {
          case 0: data[pos] ^= (uint8_t)(1u << (rng() % 8)); break;
          case 1: data[pos] = (uint8_t)rng(); break;
          default: data[pos] = (rng() & 1) ? 0 : 0xff; break;
          }
        }
      }
      ttrt_binary *b = nullptr;
      if (ttrt_binary_load_memory(data.data(), data.size(), &b) != 0) { ++refused; continue; }
      ++loaded;
      std::vector<ttrt_tensor *> ins;
      bool ok = true;
      for (uint32_t i = 0; i < nin && ok; ++i) {
        ttrt_tensor *t = nullptr;
        ok = ttrt_tensor_create_empty(dev, &layouts[i], shapes[i].data(), (int)shapes[i].size(), &t) == 0;
        if (ok) ins.push_back(t);
      }
      if (ok) {
        ttrt_tensor *outs[16] = {};
        uint32_t n = 0;
        const bool submitted = ttrt_submit(dev, b, prog, ins.data(), (uint32_t)ins.size(), outs, 16, &n) == 0;
        if (submitted) {
          ++ran;
          for (uint32_t i = 0; i < n; ++i) ttrt_tensor_free(outs[i]);
        } else {
          ++refused;
          if (std::string(ttrt_last_error()).find("null device: out of bounds") != std::string::npos) {   // a launch past a buffer
            ++out_of_bounds;
            std::fprintf(stderr, "%s round %d: %s\n", argv[f], round, ttrt_last_error());
          }
        }
        if (round == 0 && !submitted) { std::fprintf(stderr, "%s: the intact program does not run: %s\n", argv[f], ttrt_last_error()); return 2; }
      }
      for (ttrt_tensor *t : ins) ttrt_tensor_free(t);
      ttrt_binary_free(b);
    }
  }
  ttrt_device_close(dev);
  std::printf("loaded %ld ran %ld refused %ld out_of_bounds %ld\n", loaded, ran, refused, out_of_bounds);
  return 0;
}
