// Host-side test of the bookkeeping behind the per-stream workspaces of the skinny quantized matmul
// (wechat-tfcc_amd/csrc/gemv_workspace.hpp) with a counting allocator: no GPU.
#include <cstdio>
#include <cstdlib>
#include <set>

#include "gemv_workspace.hpp"

using namespace tfcc_rocm::gemv_ws;

static int failures = 0;
#define EXPECT(cond)                                         \
  do {                                                       \
    if (!(cond)) {                                           \
      ++failures;                                            \
      std::printf("FAIL line %d: %s\n", __LINE__, #cond);    \
    }                                                        \
  } while (0)

static std::set<void*> live;
static int allocations = 0, failNext = 0;
static int test_alloc(void** mem, size_t bytes) {
  if (failNext) { failNext = 0; return 3; }
  *mem = std::calloc(1, bytes);
  live.insert(*mem);
  ++allocations;
  return 0;
}
static void test_free(void* mem) {
  EXPECT(live.count(mem) == 1);  // never a double free, never a pointer the allocator did not hand out
  live.erase(mem);
  std::free(mem);
}

int main() {
  Registry reg;
  Lease a, b, c;
  // first use allocates, zero-filled, and keeps
  EXPECT(reg.acquire(1, 43, 16384, true, test_alloc, &a) == kOk);
  EXPECT(a.mem != nullptr && a.blocks >= 43 && !a.mustClear && allocations == 1);
  EXPECT(reg.acquire(1, 43, 16384, true, test_alloc, &b) == kOk);
  EXPECT(b.mem == a.mem && allocations == 1);
  // a smaller product reuses it; another stream gets its own
  EXPECT(reg.acquire(1, 4, 16384, true, test_alloc, &b) == kOk && b.mem == a.mem);
  EXPECT(reg.acquire(2, 4, 16384, true, test_alloc, &c) == kOk && c.mem != a.mem && allocations == 2);
  // growing while allocation is not allowed (stream being recorded): refused, nothing changes
  EXPECT(reg.acquire(1, 500, 16384, false, test_alloc, &b) == kWouldAllocate);
  EXPECT(reg.acquire(1, 43, 16384, false, test_alloc, &b) == kOk && b.mem == a.mem);
  // an unknown stream while recording: refused too
  EXPECT(reg.acquire(3, 1, 16384, false, test_alloc, &b) == kWouldAllocate);
  // growing: a new block, the old one stays alive (a recorded launch may still use it)
  EXPECT(reg.acquire(1, 500, 16384, true, test_alloc, &b) == kOk);
  EXPECT(b.mem != a.mem && b.blocks >= 500 && allocations == 3);
  EXPECT(live.count(a.mem) == 1);
  // geometric growth: a slightly larger request after that does not allocate again until twice the size is passed
  size_t before = b.blocks;
  EXPECT(reg.acquire(1, 501, 16384, true, test_alloc, &c) == kOk);
  EXPECT(c.blocks >= 2 * before || c.mem == b.mem || c.blocks >= 501);
  // a failed allocation reports the allocator's code and leaves the entry as it was
  Lease d;
  failNext = 1;
  EXPECT(reg.acquire(1, 100000, 16384, true, test_alloc, &d) == 3);
  EXPECT(reg.acquire(1, 43, 16384, true, test_alloc, &d) == kOk && d.mem == c.mem);
  // a failed launch marks the entry; the next lease says so once
  reg.mark_dirty(1);
  EXPECT(reg.acquire(1, 43, 16384, true, test_alloc, &d) == kOk && d.mustClear);
  EXPECT(reg.acquire(1, 43, 16384, true, test_alloc, &d) == kOk && !d.mustClear);
  reg.mark_dirty(77);  // unknown key: ignored
  // release gives everything of one stream back, the other stream's block stays
  const size_t liveBefore = live.size();
  const size_t freed = reg.release(1, test_free);
  EXPECT(freed >= 2 && live.size() == liveBefore - freed);
  EXPECT(reg.entries() == 1);
  EXPECT(reg.release(1, test_free) == 0);
  EXPECT(reg.release(2, test_free) == 1 && live.empty());
  // after a release the stream starts afresh
  EXPECT(reg.acquire(1, 4, 16384, true, test_alloc, &d) == kOk && d.mem != nullptr);
  EXPECT(reg.release(1, test_free) == 1 && live.empty());
  if (failures) {
    std::printf("%d failures\n", failures);
    return 1;
  }
  std::printf("gemv workspace bookkeeping ok\n");
  return 0;
}
