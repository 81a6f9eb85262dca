// Host-only test shim: the pool's policy (pool.h) over a fake block source, so that
// best fit, coalescing, dedicated blocks, trim and the out-of-memory retry can be
// unit-tested on a machine without a GPU.  Not linked into the product library.
#include <cstdint>
#include <map>
#include <memory>
#include <string>

#include "limits.h"
#include "pool.h"

namespace {

struct FakeSource {
  uint64_t* capacity;  // bytes the fake device can still map
  uint64_t* next;
  std::map<uint64_t, uint64_t>* live;
  bool map(uint64_t bytes, uint64_t* address, std::string* err) {
    if (bytes > *capacity) {
      *err = "fake device out of memory";
      return false;
    }
    *capacity -= bytes;
    *address = *next;
    *next += vkt::round_up(bytes, 1ull << 21) + (1ull << 21);
    (*live)[*address] = bytes;
    return true;
  }
  void unmap(uint64_t address) {
    auto it = live->find(address);
    if (it != live->end()) {
      *capacity += it->second;
      live->erase(it);
    }
  }
};

struct TestPool {
  uint64_t capacity, next = 1ull << 32;
  std::map<uint64_t, uint64_t> live;
  std::unique_ptr<vkt::Pool<FakeSource>> pool;
  std::string err;
  int idle_calls = 0;
};

void idle(void* arg) { ++static_cast<TestPool*>(arg)->idle_calls; }

}  // namespace

extern "C" {

void* vkt_test_pool_new(uint64_t capacity, uint64_t block_bytes) {
  auto* t = new TestPool;
  t->capacity = capacity;
  t->pool = std::make_unique<vkt::Pool<FakeSource>>(FakeSource{&t->capacity, &t->next, &t->live}, block_bytes);
  t->pool->set_idle_hook(&idle, t);
  return t;
}

void vkt_test_pool_delete(void* p) { delete static_cast<TestPool*>(p); }

// out[0..2] = address, size, block.  Returns 0, or -1 (message via vkt_test_pool_error).
int vkt_test_pool_alloc(void* p, uint64_t nbytes, uint64_t* out) {
  auto* t = static_cast<TestPool*>(p);
  vkt::Allocation a;
  if (!t->pool->alloc(nbytes, &a, &t->err)) return -1;
  out[0] = a.address, out[1] = a.size, out[2] = a.block;
  return 0;
}

void vkt_test_pool_free(void* p, const uint64_t* a) {
  vkt::Allocation al;
  al.address = a[0], al.size = a[1], al.block = static_cast<uint32_t>(a[2]);
  static_cast<TestPool*>(p)->pool->free(al);
}

uint64_t vkt_test_pool_trim(void* p) { return static_cast<TestPool*>(p)->pool->trim(); }

void vkt_test_pool_stats(void* p, uint64_t* out) {
  auto* t = static_cast<TestPool*>(p);
  vkt::PoolStats s = t->pool->stats();
  out[0] = s.allocated, out[1] = s.reserved, out[2] = s.blocks, out[3] = t->live.size(),
  out[4] = static_cast<uint64_t>(t->idle_calls);
}

const char* vkt_test_pool_error(void* p) { return static_cast<TestPool*>(p)->err.c_str(); }

// the stride bound of the stream kernel's 32-bit operand offsets (kernels/limits.h)
int shim_mma_stream_strides_ok(uint64_t lda, uint64_t ldb) { return vkt::mma_stream_strides_ok(lda, ldb) ? 1 : 0; }

// the slices of K a launcher makes for `wanted` (kernels/limits.h): slices in the low word, chunks per slice above
uint64_t shim_k_slices(uint32_t chunks, uint32_t wanted) {
  const vkt::KSlices s = vkt::k_slices(chunks, wanted);
  return uint64_t(s.slices) | uint64_t(s.chunks_per_slice) << 32;
}

}  // extern "C"
