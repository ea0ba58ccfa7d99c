// Host-side checks of the device pool's bookkeeping with malloc / free standing in for the driver.
// Build: g++ -std=c++17 -I tt-mlir_amd/runtime tests/cpp/test_device_pool.cpp -o <exe>; exit status 0 = all checks passed.
#include <cstdio>
#include <cstdlib>
#include <set>

#include "device_pool.h"

using tt::runtime::DevicePool;
using tt::runtime::PoolBackend;

static std::set<void *> g_driver;   // blocks the "driver" has handed out and not taken back
static int g_syncs = 0, g_fail_next = 0;

static int mockMalloc(void **p, size_t n) {
  if (g_fail_next > 0) { --g_fail_next; *p = nullptr; return 1; }
  *p = std::malloc(n);
  g_driver.insert(*p);
  return 0;
}
static int mockFree(void *p) {
  if (!g_driver.erase(p)) { std::fprintf(stderr, "double free or foreign pointer %p\n", p); std::abort(); }
  std::free(p);
  return 0;
}
static int mockSync() { ++g_syncs; return 0; }

#define CHECK(cond)                                                          \
  do {                                                                       \
    if (!(cond)) { std::fprintf(stderr, "%s:%d: CHECK(%s) failed\n", __FILE__, __LINE__, #cond); return 1; } \
  } while (0)

static int reuse() {
  DevicePool pool(PoolBackend{mockMalloc, mockFree, mockSync});
  void *a = pool.alloc(1000);
  CHECK(pool.liveBlocks() == 1 && pool.cached() == 0);
  pool.free(a, 1000);
  CHECK(pool.cached() == 1024 && pool.liveBlocks() == 0);
  void *b = pool.alloc(600);          // same rounded size: the cached block
  CHECK(b == a && pool.cached() == 0);
  pool.free(b, 600);
  pool.release();
  CHECK(g_driver.empty() && pool.cached() == 0);
  return 0;
}

// A tensor allocated while a trace was recorded (an output the caller keeps) outlives the trace and the device's release():
// its block must neither be handed to anyone else nor returned to the driver until the tensor's deleter gives it back.
static int tensorOutlivesItsTrace() {
  DevicePool pool(PoolBackend{mockMalloc, mockFree, mockSync});
  pool.beginRecording();
  void *scratch = pool.alloc(4096);   // intermediate of the traced region
  void *out = pool.alloc(4096);       // output the caller keeps
  pool.free(scratch, 4096);
  auto blocks = pool.endRecording();
  CHECK(blocks.size() == 2 && pool.pinnedBlocks() == 2);
  void *other = pool.alloc(4096);     // pinned blocks are out of circulation while the trace lives
  CHECK(other != scratch && other != out);
  pool.free(other, 4096);
  pool.unpin(blocks);                 // releaseTrace
  CHECK(pool.pinnedBlocks() == 0 && pool.liveBlocks() == 1);
  CHECK(pool.cached() == 2 * 4096);   // scratch and other, not out
  pool.release();                     // closeMeshDevice
  CHECK(g_driver.count(out) == 1 && g_driver.size() == 1);   // still the tensor's
  void *again = pool.alloc(4096);     // reopened device: must not alias the live tensor
  CHECK(again != out);
  pool.free(out, 4096);               // the tensor dies: only now the block is cached
  CHECK(pool.cached() == 4096);
  void *third = pool.alloc(4096);
  CHECK(third == out);
  pool.free(third, 4096);
  pool.free(again, 4096);
  pool.release();
  CHECK(g_driver.empty());
  return 0;
}

// A block that existed before the recording and is released inside it stays pinned (recorded launches read it), is reused
// by the recording itself, and returns to circulation when the trace is released.
static int releasedInsideARecording() {
  DevicePool pool(PoolBackend{mockMalloc, mockFree, mockSync});
  void *before = pool.alloc(2048);
  pool.beginRecording();
  pool.free(before, 2048);
  void *inside = pool.alloc(2048);
  CHECK(inside == before);            // the recording's own order makes the reuse safe
  pool.free(inside, 2048);
  auto blocks = pool.endRecording();
  CHECK(blocks.size() == 1);
  void *outside = pool.alloc(2048);
  CHECK(outside != before);
  pool.unpin(blocks);
  CHECK(pool.cached() == 2048);
  pool.free(outside, 2048);
  pool.release();
  CHECK(g_driver.empty());
  return 0;
}

// Two traces name one block (an output of the first, kept by the caller, is released inside the second recording): it
// returns to circulation only when both are released.
static int blockSharedByTwoTraces() {
  DevicePool pool(PoolBackend{mockMalloc, mockFree, mockSync});
  pool.beginRecording();
  void *out = pool.alloc(512);
  auto first = pool.endRecording();
  pool.beginRecording();
  pool.free(out, 512);
  auto second = pool.endRecording();
  pool.unpin(first);
  CHECK(pool.pinnedBlocks() == 1 && pool.cached() == 0);
  pool.unpin(second);
  CHECK(pool.pinnedBlocks() == 0 && pool.cached() == 512);
  pool.release();
  CHECK(g_driver.empty());
  return 0;
}

static int allocationFailureReleasesTheCacheFirst() {
  DevicePool pool(PoolBackend{mockMalloc, mockFree, mockSync});
  void *a = pool.alloc(8192);
  pool.free(a, 8192);
  g_fail_next = 1;
  const int syncs = g_syncs;
  void *b = pool.alloc(100000);       // first driver call fails, the cache is released, the second succeeds
  CHECK(b != nullptr && g_syncs == syncs + 1 && pool.cached() == 0 && g_driver.size() == 1);
  g_fail_next = 2;
  bool threw = false;
  try { pool.alloc(200000); } catch (const std::runtime_error &) { threw = true; }
  CHECK(threw);
  pool.free(b, 100000);
  pool.release();
  CHECK(g_driver.empty());
  return 0;
}

int main() {
  int rc = reuse() | tensorOutlivesItsTrace() | releasedInsideARecording() | blockSharedByTwoTraces() |
           allocationFailureReleasesTheCacheFirst();
  std::printf(rc ? "FAILED\n" : "ok\n");
  return rc;
}
