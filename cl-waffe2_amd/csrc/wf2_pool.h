// wf2_pool.h -- the bookkeeping of the caching allocator: which block is idle, which is
// handed out, and which captured graphs still write into it.  No device call in here: the
// runtime performs the actual allocation and release, so this class also builds and runs
// on the host alone.
//
// cl-waffe2 allocates a compiled model's temporaries once and reuses them on every forward
// (maybe-allocate!, source/vm/allocation.lisp:121-145); a host that allocates per call gets
// the same steady state from this pool.
//
// A captured graph keeps the blocks its kernels were recorded with.  Every block handed out
// or freed during a capture gets that graph as one of its owners.  When a block with owners
// is freed -- during the capture or at any time after it, e.g. when the host's collector
// finalises a result it dropped -- it is parked in an owner's `held` list instead of the idle
// pool: every replay of every owner still writes into it, and an eager allocation that
// received it would be silently overwritten.  Blocks parked during a capture are re-usable
// by later allocations of the same capture (a replay preserves the recorded order).  A
// block returns to the idle pool when the last of its owners is destroyed.
#pragma once
#include <algorithm>
#include <cstddef>
#include <map>
#include <unordered_map>
#include <utility>
#include <vector>

namespace wf2 {

struct GraphBlocks {
  std::multimap<size_t, void*> held;  // size class -> parked block
};

class BlockPool {
 public:
  bool enabled = true;

  static size_t size_class(size_t bytes) {
    const size_t small = 512, large = (size_t)2 << 20;
    if (bytes < ((size_t)1 << 20)) return (bytes + small - 1) / small * small;
    return (bytes + large - 1) / large * large;
  }

  size_t idle_bytes() const { return idle_bytes_; }
  size_t blocks_known() const { return size_of_.size(); }
  bool knows(void* ptr) const { return size_of_.count(ptr) != 0; }
  size_t owners_of(void* ptr) const {
    auto it = owners_.find(ptr);
    return it == owners_.end() ? 0 : it->second.size();
  }

  // A block of this size class that may be handed out now, or nullptr: the caller then
  // allocates one and calls adopt() (never during a capture).
  void* take(size_t cls, GraphBlocks* capture) {
    if (capture) {
      auto held = capture->held.find(cls);
      if (held != capture->held.end()) {
        void* ptr = held->second;
        capture->held.erase(held);
        return ptr;
      }
    }
    if (!enabled) return nullptr;
    auto it = idle_.find(cls);
    if (it == idle_.end()) return nullptr;
    void* ptr = it->second;
    idle_.erase(it);
    idle_bytes_ -= cls;
    if (capture) add_owner(ptr, capture);
    return ptr;
  }

  void adopt(void* ptr, size_t cls) { size_of_[ptr] = cls; }

  enum Outcome { kUnknown, kKept, kRelease };

  // The host is done with ptr.  kRelease: no graph owns it and the pool is disabled -- the
  // caller releases the memory (the block is forgotten here).
  Outcome give_back(void* ptr, GraphBlocks* capture) {
    auto it = size_of_.find(ptr);
    if (it == size_of_.end()) return kUnknown;
    const size_t cls = it->second;
    if (capture) {
      // also a block from before the capture: its last use may be recorded
      add_owner(ptr, capture);
      capture->held.emplace(cls, ptr);
      return kKept;
    }
    auto owner = owners_.find(ptr);
    if (owner != owners_.end()) {
      owner->second.front()->held.emplace(cls, ptr);
      return kKept;
    }
    if (enabled) {
      idle_.emplace(cls, ptr);
      idle_bytes_ += cls;
      return kKept;
    }
    size_of_.erase(it);
    return kRelease;
  }

  // g is being destroyed.  Blocks nobody else owns go back to the idle pool, or into
  // `release` (to be freed by the caller) when the pool is disabled; blocks parked with g
  // that other graphs own as well move to one of those.
  void forget_graph(GraphBlocks* g, std::vector<void*>* release) {
    for (auto it = owners_.begin(); it != owners_.end();) {
      auto& v = it->second;
      v.erase(std::remove(v.begin(), v.end(), g), v.end());
      it = v.empty() ? owners_.erase(it) : std::next(it);
    }
    for (auto& kv : g->held) {
      auto owner = owners_.find(kv.second);
      if (owner != owners_.end()) {
        owner->second.front()->held.emplace(kv.first, kv.second);
      } else if (enabled) {
        idle_.emplace(kv.first, kv.second);
        idle_bytes_ += kv.first;
      } else {
        size_of_.erase(kv.second);
        release->push_back(kv.second);
      }
    }
    g->held.clear();
  }

  // Every idle block, forgotten here, for the caller to free.
  void drain_idle(std::vector<void*>* release) {
    for (auto& kv : idle_) {
      size_of_.erase(kv.second);
      release->push_back(kv.second);
    }
    idle_.clear();
    idle_bytes_ = 0;
  }

  bool has_idle() const { return !idle_.empty(); }

 private:
  void add_owner(void* ptr, GraphBlocks* g) {
    auto& v = owners_[ptr];
    if (std::find(v.begin(), v.end(), g) == v.end()) v.push_back(g);
  }

  std::multimap<size_t, void*> idle_;                          // size class -> block
  std::unordered_map<void*, size_t> size_of_;                  // every block handed out, parked or idle
  std::unordered_map<void*, std::vector<GraphBlocks*>> owners_;  // block -> the live graphs recorded with it
  size_t idle_bytes_ = 0;
};

}  // namespace wf2
