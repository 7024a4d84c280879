// Bookkeeping of the workspaces of the skinny quantized matmul that splits K: one entry per (device, stream).
//
// Rules it keeps, whatever the allocator behind it:
//   * a workspace that has been handed to a launch is never freed while its stream may still use it: when a wider
//     product needs a larger one, the old block is retired, not released - launches recorded earlier (a captured
//     graph replays with the pointer it was recorded with) keep a valid, all-zero workspace;
//   * growing needs an allocation, and the caller says whether one is allowed right now (not while the stream is
//     being captured): if not, acquire() reports kWouldAllocate and the caller takes a path without a workspace;
//   * an entry whose last launch did not go through is marked, and the next acquire() reports that the block must
//     be cleared on the stream before it is used again;
//   * release() gives back everything kept for one stream, forget-me-not for streams that are about to go away.
// Plain C++ (no GPU calls of its own): the allocator comes in as two functions, so the same code runs under a
// host-side test with a counting allocator.
#pragma once

#include <cstddef>
#include <mutex>
#include <unordered_map>
#include <vector>

namespace tfcc_rocm {
namespace gemv_ws {

constexpr int kOk = 0, kWouldAllocate = -1;

struct Lease {
  void* mem = nullptr;       // zero-filled when first handed out
  size_t blocks = 0;         // capacity in column blocks
  bool mustClear = false;    // the previous launch on this entry failed: clear `mem` on the stream first
};

class Registry {
 public:
  using AllocFn = int (*)(void** mem, size_t bytes);  // allocates and zero-fills; 0 on success, else an error code
  using FreeFn = void (*)(void* mem);

  // A workspace of at least `blocks` column blocks of `bytesPerBlock` for `key`.  Returns kOk, kWouldAllocate
  // (only when !mayAllocate) or the allocator's error code.
  int acquire(unsigned long long key, size_t blocks, size_t bytesPerBlock, bool mayAllocate, AllocFn alloc, Lease* out) {
    std::lock_guard<std::mutex> lock(mutex_);
    auto found = entries_.find(key);
    if (!mayAllocate && (found == entries_.end() || found->second.blocks < blocks)) return kWouldAllocate;
    Entry& e = found == entries_.end() ? entries_[key] : found->second;
    if (e.blocks < blocks) {
      size_t want = blocks > 2 * e.blocks ? blocks : 2 * e.blocks;  // geometric growth bounds what retired blocks hold
      void* mem = nullptr;
      if (int err = alloc(&mem, want * bytesPerBlock)) return err;
      if (e.mem) e.retired.push_back(e.mem);
      e.mem = mem;
      e.blocks = want;
      e.dirty = false;
    }
    out->mem = e.mem;
    out->blocks = e.blocks;
    out->mustClear = e.dirty;
    e.dirty = false;
    return kOk;
  }
  // the launch that was given key's workspace failed
  void mark_dirty(unsigned long long key) {
    std::lock_guard<std::mutex> lock(mutex_);
    auto it = entries_.find(key);
    if (it != entries_.end()) it->second.dirty = true;
  }
  // Frees every block kept for `key` (the caller has made sure the stream is idle); returns how many were freed.
  size_t release(unsigned long long key, FreeFn release_fn) {
    std::lock_guard<std::mutex> lock(mutex_);
    auto it = entries_.find(key);
    if (it == entries_.end()) return 0;
    size_t n = 0;
    for (void* m : it->second.retired) { release_fn(m); ++n; }
    if (it->second.mem) { release_fn(it->second.mem); ++n; }
    entries_.erase(it);
    return n;
  }
  size_t entries() {
    std::lock_guard<std::mutex> lock(mutex_);
    return entries_.size();
  }

 private:
  struct Entry {
    void* mem = nullptr;
    size_t blocks = 0;
    bool dirty = false;
    std::vector<void*> retired;
  };
  std::mutex mutex_;
  std::unordered_map<unsigned long long, Entry> entries_;
};

}  // namespace gemv_ws
}  // namespace tfcc_rocm
