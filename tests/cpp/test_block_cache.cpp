// CPU unit test of the allocation cache's graph-capture rules (burn_amd/csrc/block_cache.hpp).
// Pointers are plain tokens here: nothing is allocated on a device.
#include <cassert>
#include <cstdio>
#include <cstdint>

#include "block_cache.hpp"

using bq::BlockCache;
using bq::GraphBlocks;

static void* P(uintptr_t v) { return reinterpret_cast<void*>(v); }

int main() {
  BlockCache c;
  void* p = nullptr;
  size_t actual = 0;

  // exact and near fits: a cached block serves a request up to 1/8 smaller, never a larger one
  c.put(P(0x1000), 4096);
  c.put(P(0x2000), 8192);
  assert(c.cached_bytes() == 12288 && c.cached_blocks() == 2);
  assert(!c.take(16384, &p, &actual));
  assert(c.take(7680, &p, &actual) && p == P(0x2000) && actual == 8192);  // 7680 + 7680 / 8 >= 8192
  assert(!c.take(2048, &p, &actual));                                     // 4096 is more than 1/8 over
  assert(c.take(4096, &p, &actual) && p == P(0x1000) && actual == 4096);
  assert(c.cached_blocks() == 0 && c.cached_bytes() == 0);

  // a temporary allocated and released inside a capture is parked with the graph, not reused
  c.put(P(0x3000), 512);                      // cached before the capture (its work is already enqueued)
  c.begin_capture();
  assert(c.capturing() && c.must_retire());
  assert(c.take(512, &p, &actual) && p == P(0x3000));  // cache hit during the capture
  c.note_handed_out(P(0x4000));               // a fresh allocation during the capture (an output tensor)
  c.note_handed_out(P(0x5000));               // another fresh one: a temporary
  c.put(P(0x5000), 1024);                     // ... released inside the captured call
  c.put(P(0x3000), 512);                      // ... and so is the cache hit
  assert(!c.take(1024, &p, &actual) && !c.take(512, &p, &actual));
  GraphBlocks g;
  c.end_capture(&g);
  assert(!c.capturing() && c.live_graphs() == 1 && c.must_retire());
  assert(g.parked.size() == 2 && g.owned.size() == 1 && g.owned.count(P(0x4000)) == 1);
  assert(!c.take(1024, &p, &actual) && !c.take(512, &p, &actual));  // still pinned by the graph

  // a tensor created during the capture and released while the graph lives: parked too
  c.put(P(0x4000), 2048);
  assert(!c.take(2048, &p, &actual));
  assert(g.parked.size() == 3 && g.owned.empty());
  // an unrelated block is cached as usual
  c.put(P(0x6000), 2048);
  assert(c.take(2048, &p, &actual) && p == P(0x6000));

  // a workspace replaced while the graph lives is retired, and only handed back once no graph is left
  c.retire(P(0x9000));
  assert(c.take_retired().empty());
  c.release_graph(&g);
  assert(c.live_graphs() == 0 && !c.must_retire());
  auto retired = c.take_retired();
  assert(retired.size() == 1 && retired[0] == P(0x9000));
  assert(c.take_retired().empty());
  // the graph's blocks are reusable now
  assert(c.take(2048, &p, &actual) && p == P(0x4000));
  assert(c.take(1024, &p, &actual) && p == P(0x5000));
  assert(c.take(512, &p, &actual) && p == P(0x3000));

  // a failed capture gives its parked blocks straight back
  c.begin_capture();
  c.note_handed_out(P(0x7000));
  c.put(P(0x7000), 512);
  c.end_capture(nullptr);
  assert(c.live_graphs() == 0 && c.take(512, &p, &actual) && p == P(0x7000));

  // drain empties the cache and reports every block once
  c.put(P(0xA000), 512);
  c.put(P(0xB000), 512);
  assert(c.drain().size() == 2 && c.cached_blocks() == 0 && c.cached_bytes() == 0);
  std::puts("block cache: ok");
  return 0;
}
