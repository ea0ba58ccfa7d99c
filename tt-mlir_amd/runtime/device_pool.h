// Caching allocator of device memory: blocks are kept per rounded size and reused; all work of a device is ordered on one
// stream, so reuse by a later launch is safe.  Blocks return to the driver at release().  The driver calls are injected, so
// the bookkeeping can be exercised on the host with malloc / free standing in for them.
#pragma once
#include <algorithm>
#include <cstddef>
#include <map>
#include <mutex>
#include <set>
#include <stdexcept>
#include <thread>
#include <utility>
#include <vector>

namespace tt::runtime {

struct PoolBackend {
  int (*malloc)(void **ptr, size_t bytes);   // 0 on success
  int (*free)(void *ptr);
  int (*sync)();                             // waits for all device work: called before blocks go back to the driver
};

class DevicePool {
public:
  using Blocks = std::vector<std::pair<void *, size_t>>;

  explicit DevicePool(PoolBackend backend) : be(backend) {}

  static size_t rounded(size_t bytes) { return std::max<size_t>(512, (bytes + 511) / 512 * 512); }

  void *alloc(size_t bytes) {
    const size_t sz = rounded(bytes);
    {
      std::lock_guard<std::mutex> g(mu);
      const bool rec = recordingHere();
      if (rec) {
        auto it = recordFree.find(sz);
        if (it != recordFree.end()) {
          void *p = it->second;
          recordFree.erase(it);
          live.insert(p);
          return p;
        }
      }
      auto it = freeBlocks.find(sz);
      if (it != freeBlocks.end()) {
        void *p = it->second;
        freeBlocks.erase(it);
        cachedBytes -= sz;
        if (rec) touch(p, sz);
        live.insert(p);
        return p;
      }
    }
    void *p = nullptr;
    if (be.malloc(&p, sz) != 0) {
      release();
      if (be.malloc(&p, sz) != 0) throw std::runtime_error("Fatal error: device allocation of " + std::to_string(sz) + " bytes failed");
    }
    std::lock_guard<std::mutex> g(mu);
    if (recordingHere()) touch(p, sz);
    live.insert(p);
    return p;
  }

  // called by the deleter of the tensor that owned the block
  void free(void *p, size_t bytes) {
    const size_t sz = rounded(bytes);
    std::lock_guard<std::mutex> g(mu);
    live.erase(p);
    if (recordingHere()) {
      // a block that existed before the recording and is released inside it may still be read by recorded launches; it
      // stays with the recording, whose later launches may reuse it (the graph keeps their order)
      touch(p, sz);
      recordFree.emplace(sz, p);
      return;
    }
    if (pinned.count(p)) return;  // a trace's launches name it; it comes back through unpin()
    freeBlocks.emplace(sz, p);
    cachedBytes += sz;
  }

  // While a trace is being recorded on this thread every block the recording allocates or releases is pinned: it does not
  // return to circulation before the trace is released, so a replay can never touch memory handed to another tensor.
  void beginRecording() {
    std::lock_guard<std::mutex> g(mu);
    if (recording) throw std::runtime_error("Fatal error: a trace is already being recorded");
    recording = true;
    recorder = std::this_thread::get_id();
    recordFree.clear();
    recordTouched.clear();
  }
  Blocks endRecording() {
    std::lock_guard<std::mutex> g(mu);
    Blocks out(recordTouched.begin(), recordTouched.end());
    recording = false;
    recordFree.clear();
    recordTouched.clear();
    return out;
  }
  // The blocks of a released trace go back into circulation, except those a tensor still owns (an output of the traced
  // region that the caller kept): such a block is only unpinned, and the tensor's deleter returns it through free().
  void unpin(const Blocks &blocks) {
    std::lock_guard<std::mutex> g(mu);
    for (const auto &b : blocks) {
      auto it = pinned.find(b.first);
      if (it == pinned.end()) continue;
      if (--it->second > 0) continue;         // another trace's launches name the block too
      pinned.erase(it);
      if (live.count(b.first)) continue;
      freeBlocks.emplace(b.second, b.first);
      cachedBytes += b.second;
    }
  }

  // cached blocks go back to the driver; blocks owned by tensors or pinned by traces are not touched
  void release() {
    std::lock_guard<std::mutex> g(mu);
    if (!freeBlocks.empty()) be.sync();
    for (auto &kv : freeBlocks) be.free(kv.second);
    freeBlocks.clear();
    cachedBytes = 0;
  }

  size_t cached() {
    std::lock_guard<std::mutex> g(mu);
    return cachedBytes;
  }
  size_t liveBlocks() {
    std::lock_guard<std::mutex> g(mu);
    return live.size();
  }
  size_t pinnedBlocks() {
    std::lock_guard<std::mutex> g(mu);
    return pinned.size();
  }

private:
  bool recordingHere() const { return recording && recorder == std::this_thread::get_id(); }
  void touch(void *p, size_t sz) {
    if (recordTouched.emplace(p, sz).second) ++pinned[p];
  }

  PoolBackend be;
  std::mutex mu;
  std::multimap<size_t, void *> freeBlocks;      // cached, owned by nobody
  size_t cachedBytes = 0;
  bool recording = false;
  std::thread::id recorder;
  std::multimap<size_t, void *> recordFree;      // released inside the current recording
  std::map<void *, size_t> recordTouched;        // every block the current recording allocated or released
  std::map<void *, int> pinned;                  // named by the launches of that many traces
  std::set<void *> live;                         // owned by a tensor
};

}  // namespace tt::runtime
