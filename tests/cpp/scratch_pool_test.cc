// CPU exercise of the scratch buffer's lifetime rules (zero-tvm_amd/csrc/scratch_pool.h) with a
// counting allocator in place of hipMalloc / hipFree. Prints one line per check; exit code 0 = all hold.
#include "../../zero-tvm_amd/csrc/scratch_pool.h"

#include <cstdio>
#include <cstdlib>
#include <set>

struct CountingAlloc {
  std::set<void*>* live;
  size_t* fail_above;  // allocations larger than this fail
  void* allocate(size_t bytes) const {
    if (bytes > *fail_above) return nullptr;
    void* p = std::malloc(bytes ? bytes : 1);
    live->insert(p);
    return p;
  }
  void release(void* p) const {
    if (!live->erase(p)) { std::printf("FAIL double or foreign free\n"); std::exit(1); }
    std::free(p);
  }
};

static int failures = 0;
#define CHECK(cond)                                                 \
  do {                                                              \
    if (!(cond)) { std::printf("FAIL %s:%d %s\n", __FILE__, __LINE__, #cond); failures++; } \
    else std::printf("ok %s\n", #cond);                             \
  } while (0)

int main() {
  std::set<void*> live;
  size_t limit = ~(size_t)0;
  {
    ztvm::ScratchPool<CountingAlloc> pool(CountingAlloc{&live, &limit});
    CHECK(pool.reserve(4096) && pool.bytes() >= 4096 && live.size() == 1);
    void* first = pool.data();
    CHECK(pool.reserve(100) && pool.data() == first);  // smaller requests never move the buffer

    // no command buffer alive: growth frees the old buffer at once
    CHECK(pool.reserve(10000) && pool.data() != nullptr && live.size() == 1 && pool.retired() == 0);
    CHECK(pool.bytes() >= 10000);

    // a command buffer recorded now holds `held`; growth afterwards must keep it allocated
    void* held = pool.data();
    pool.pin();
    CHECK(pool.reserve(1 << 20) && pool.data() != held);
    CHECK(live.count(held) == 1 && pool.retired() == 1);
    void* held2 = pool.data();
    pool.pin();  // a second command buffer, recorded against the grown buffer
    CHECK(pool.reserve(4 << 20) && live.count(held) == 1 && live.count(held2) == 1 && pool.retired() == 2);
    pool.unpin();  // one of the two is destroyed: both addresses may still be referenced by the other
    CHECK(live.count(held) == 1 && live.count(held2) == 1);
    pool.unpin();  // the last one is gone: the retired buffers go, the current one stays
    CHECK(live.count(held) == 0 && live.count(held2) == 0 && pool.retired() == 0 && live.size() == 1);

    // growth at least doubles, so the retired buffers together stay below the current size
    const size_t before = pool.bytes();
    CHECK(pool.reserve(before + 1) && pool.bytes() >= 2 * before);

    // a failed allocation keeps the buffer that works
    void* good = pool.data();
    const size_t good_bytes = pool.bytes();
    limit = good_bytes;  // nothing larger can be had
    CHECK(!pool.reserve(good_bytes * 8) && pool.data() == good && pool.bytes() == good_bytes);
    limit = good_bytes * 3;  // the doubled size fails, the exact size fits
    CHECK(pool.reserve(good_bytes * 2 + 16) && pool.bytes() == good_bytes * 2 + 16);
    limit = ~(size_t)0;

    // destroying the context with a command buffer still alive frees everything once
    pool.pin();
    CHECK(pool.reserve(pool.bytes() * 2) && pool.retired() == 1);
    pool.release_all();
    CHECK(live.empty() && pool.data() == nullptr && pool.bytes() == 0);
    pool.unpin();  // the command buffer dies after its context: nothing left to free
    CHECK(live.empty());
  }
  std::printf(failures ? "FAILED %d\n" : "ALL OK\n", failures);
  return failures ? 1 : 0;
}
