// Bookkeeping of a device context's allocation cache: which cached block serves a request, and
// where a released block may go while HIP graphs hold its address. No HIP call in here (the
// caller allocates and frees), so the rules are unit-tested on the CPU.
//
// Rules:
//   * a request takes the smallest cached block of at least its size and at most 1/8 more;
//   * a block released while the stream is being captured is not reused: the captured kernels
//     carry its address, so it is parked with the graph and returns to the cache when the graph
//     is released (this covers the temporaries a captured call allocates and frees inside);
//   * a block handed out during a capture and released later, while that graph is alive, is
//     parked with the graph in the same way;
//   * a workspace replaced by a larger one while a capture is open or graphs are alive is retired
//     instead of freed; retired workspaces are handed back for freeing once no graph is left.
#pragma once

#include <cstddef>
#include <map>
#include <set>
#include <utility>
#include <vector>

namespace bq {

struct GraphBlocks {
  std::vector<std::pair<size_t, void*>> parked;  // released, reusable once the graph is gone
  std::set<void*> owned;                         // handed out during the capture, still in use
};

class BlockCache {
 public:
  // A cached block for `bytes`, or false. *actual receives the block's real size.
  bool take(size_t bytes, void** ptr, size_t* actual) {
    auto it = free_.lower_bound(bytes);
    if (it == free_.end() || it->first > bytes + bytes / 8) return false;
    *ptr = it->second;
    *actual = it->first;
    cached_bytes_ -= it->first;
    free_.erase(it);
    note_handed_out(*ptr);
    return true;
  }

  // Every block handed to a tensor passes through here (cache hits and fresh allocations).
  void note_handed_out(void* ptr) {
    if (capturing_) capture_owned_.insert(ptr);
  }

  // A tensor gave `ptr` (of `size` bytes) back.
  void put(void* ptr, size_t size) {
    if (capturing_) {
      capture_owned_.erase(ptr);
      capture_parked_.emplace_back(size, ptr);
      return;
    }
    for (GraphBlocks* g : graphs_) {
      auto it = g->owned.find(ptr);
      if (it != g->owned.end()) {
        g->owned.erase(it);
        g->parked.emplace_back(size, ptr);
        return;
      }
    }
    free_.emplace(size, ptr);
    cached_bytes_ += size;
  }

  bool capturing() const { return capturing_; }
  size_t live_graphs() const { return graphs_.size(); }
  size_t cached_bytes() const { return cached_bytes_; }
  size_t cached_blocks() const { return free_.size(); }

  void begin_capture() {
    capturing_ = true;
    capture_owned_.clear();
    capture_parked_.clear();
  }

  // Ends the capture; `g` (owned by the caller's graph object) takes what the capture pinned.
  void end_capture(GraphBlocks* g) {
    capturing_ = false;
    if (g != nullptr) {
      g->parked.swap(capture_parked_);
      g->owned.swap(capture_owned_);
      graphs_.insert(g);
    } else {  // the capture failed: nothing will replay, the blocks are free again
      for (auto& b : capture_parked_) {
        free_.emplace(b.first, b.second);
        cached_bytes_ += b.first;
      }
    }
    capture_parked_.clear();
    capture_owned_.clear();
  }

  // The graph is gone (its last replay has finished): its parked blocks are reusable.
  void release_graph(GraphBlocks* g) {
    graphs_.erase(g);
    for (auto& b : g->parked) {
      free_.emplace(b.first, b.second);
      cached_bytes_ += b.first;
    }
    g->parked.clear();
    g->owned.clear();
  }

  // True when a replaced workspace must be kept (its address may be inside a graph).
  bool must_retire() const { return capturing_ || !graphs_.empty(); }
  void retire(void* ptr) { retired_.push_back(ptr); }
  // Retired workspaces that may be freed now (none while a graph could still use them).
  std::vector<void*> take_retired() {
    std::vector<void*> out;
    if (!must_retire()) out.swap(retired_);
    return out;
  }

  // Empties the cache: the caller frees what is returned. Parked and retired blocks stay.
  std::vector<void*> drain() {
    std::vector<void*> out;
    for (auto& kv : free_) out.push_back(kv.second);
    free_.clear();
    cached_bytes_ = 0;
    return out;
  }

 private:
  std::multimap<size_t, void*> free_;
  size_t cached_bytes_ = 0;
  bool capturing_ = false;
  std::set<void*> capture_owned_;
  std::vector<std::pair<size_t, void*>> capture_parked_;
  std::set<GraphBlocks*> graphs_;
  std::vector<void*> retired_;
};

}  // namespace bq
