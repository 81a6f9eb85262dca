// Caching device-memory pool: a best-fit range allocator over large hipMalloc'd blocks.
//
// Policy follows the reference's pool (crates/vkcore/src/memory.rs:18-28,37-78,150-225):
// 256-byte alignment, requests carved out of shared blocks by best fit with coalescing
// on free, oversized requests in blocks of their own (2 MiB granule), freed ranges
// reusable immediately (every user is queued on one in-order stream, so a later kernel
// can never overtake an earlier user of the same bytes), trim() returns unused blocks,
// and an out-of-memory block request is retried once after a trim.
//
// Sized for 288 GB of HBM3E: shared blocks are 256 MiB (the reference, written for
// integrated GPUs, uses 64 MiB) so that a decode step's weights and temporaries sit in
// a handful of driver allocations.
//
// The block source is a template parameter so that the policy is unit-testable on a
// machine without a GPU.
#pragma once

#include <cstdint>
#include <map>
#include <memory>
#include <string>
#include <vector>

namespace vkt {

constexpr uint64_t kAlign = 256;
constexpr uint64_t kBlockBytes = 256ull << 20;
constexpr uint64_t kLargeGranule = 2ull << 20;

inline uint64_t round_up(uint64_t v, uint64_t a) { return (v + a - 1) / a * a; }

// Free ranges of one block, best fit, coalescing (memory.rs:37-78).
class RangeAllocator {
 public:
  explicit RangeAllocator(uint64_t size) : size_(size) { free_[0] = size; }

  // Offset of a range of `n` bytes (n a multiple of kAlign), or UINT64_MAX.
  uint64_t alloc(uint64_t n) {
    auto best = free_.end();
    for (auto it = free_.begin(); it != free_.end(); ++it) {
      if (it->second >= n && (best == free_.end() || it->second < best->second)) best = it;
    }
    if (best == free_.end()) return UINT64_MAX;
    uint64_t off = best->first, len = best->second;
    free_.erase(best);
    if (len > n) free_[off + n] = len - n;
    used_ += n;
    return off;
  }

  void free(uint64_t off, uint64_t n) {
    used_ -= n;
    auto next = free_.lower_bound(off);
    if (next != free_.begin()) {
      auto prev = std::prev(next);
      if (prev->first + prev->second == off) {
        off = prev->first;
        n += prev->second;
        free_.erase(prev);
      }
    }
    if (next != free_.end() && off + n == next->first) {
      n += next->second;
      free_.erase(next);
    }
    free_[off] = n;
  }

  bool unused() const { return used_ == 0; }
  uint64_t size() const { return size_; }
  uint64_t used() const { return used_; }
  size_t fragments() const { return free_.size(); }

 private:
  uint64_t size_, used_ = 0;
  std::map<uint64_t, uint64_t> free_;  // offset -> length
};

struct Allocation {
  uint64_t address = 0;
  uint64_t size = 0;
  uint32_t block = 0;  // index into the pool's block table
};

struct PoolStats {
  uint64_t allocated = 0, reserved = 0, blocks = 0;
};

// Source: struct with `bool map(uint64_t bytes, uint64_t* address, std::string* err)`
// and `void unmap(uint64_t address)`.
template <class Source>
class Pool {
 public:
  explicit Pool(Source src, uint64_t block_bytes = kBlockBytes) : src_(std::move(src)), block_bytes_(block_bytes) {}
  ~Pool() { release_all(); }

  bool alloc(uint64_t nbytes, Allocation* out, std::string* err) {
    uint64_t n = round_up(nbytes == 0 ? 1 : nbytes, kAlign);
    if (n < nbytes) {
      *err = "allocation size overflows";
      return false;
    }
    if (n <= block_bytes_ / 2) {
      // best fit over the shared blocks: the block whose chosen range is tightest is
      // approximated by first trying blocks in order of least free space
      for (uint32_t i = 0; i < blocks_.size(); ++i) {
        Block& b = blocks_[i];
        if (!b.live || b.dedicated) continue;
        uint64_t off = b.ranges->alloc(n);
        if (off != UINT64_MAX) return finish(i, off, n, out);
      }
      uint32_t i;
      if (!new_block(block_bytes_, false, &i, err)) return false;
      return finish(i, blocks_[i].ranges->alloc(n), n, out);
    }
    // oversized: reuse a cached dedicated block of sufficient size (tightest), else a new one
    uint64_t want = round_up(n, kLargeGranule);
    int best = -1;
    for (uint32_t i = 0; i < blocks_.size(); ++i) {
      Block& b = blocks_[i];
      if (b.live && b.dedicated && b.ranges->unused() && b.size >= n && b.size <= want + want / 4 &&
          (best < 0 || b.size < blocks_[best].size))
        best = static_cast<int>(i);
    }
    uint32_t i;
    if (best >= 0) {
      i = static_cast<uint32_t>(best);
    } else if (!new_block(want, true, &i, err)) {
      return false;
    }
    // a dedicated block is handed out whole, so its usable size is the block's
    return finish(i, blocks_[i].ranges->alloc(blocks_[i].size), blocks_[i].size, out);
  }

  void free(const Allocation& a) {
    if (a.block >= blocks_.size() || !blocks_[a.block].live) return;
    Block& b = blocks_[a.block];
    b.ranges->free(a.address - b.address, a.size);
    allocated_ -= a.size;
  }

  // Returns unused blocks to the driver (memory.rs trim).  The caller has made the
  // device idle.  Returns the bytes released.
  uint64_t trim() {
    uint64_t released = 0;
    for (Block& b : blocks_) {
      if (b.live && b.ranges->unused()) {
        src_.unmap(b.address);
        reserved_ -= b.size;
        released += b.size;
        b.live = false;
        b.ranges.reset();
        --live_blocks_;
      }
    }
    return released;
  }

  PoolStats stats() const { return PoolStats{allocated_, reserved_, live_blocks_}; }
  void set_idle_hook(void (*hook)(void*), void* arg) {
    idle_hook_ = hook;
    idle_arg_ = arg;
  }

 private:
  struct Block {
    uint64_t address = 0, size = 0;
    bool dedicated = false, live = false;
    std::unique_ptr<RangeAllocator> ranges;
  };

  bool finish(uint32_t i, uint64_t off, uint64_t n, Allocation* out) {
    out->address = blocks_[i].address + off;
    out->size = n;
    out->block = i;
    allocated_ += n;
    return true;
  }

  bool new_block(uint64_t bytes, bool dedicated, uint32_t* index, std::string* err) {
    uint64_t address = 0;
    if (!src_.map(bytes, &address, err)) {
      // out of memory: wait for the device, give cached blocks back, retry once (memory.rs:171-179)
      if (idle_hook_) idle_hook_(idle_arg_);
      if (trim() == 0 || !src_.map(bytes, &address, err)) return false;
    }
    Block b;
    b.address = address;
    b.size = bytes;
    b.dedicated = dedicated;
    b.live = true;
    b.ranges = std::make_unique<RangeAllocator>(bytes);
    uint32_t i = 0;
    for (; i < blocks_.size(); ++i)
      if (!blocks_[i].live) break;
    if (i == blocks_.size()) blocks_.emplace_back();
    blocks_[i] = std::move(b);
    reserved_ += bytes;
    ++live_blocks_;
    *index = i;
    return true;
  }

  void release_all() {
    for (Block& b : blocks_)
      if (b.live) src_.unmap(b.address);
    blocks_.clear();
  }

  Source src_;
  uint64_t block_bytes_;
  std::vector<Block> blocks_;
  uint64_t allocated_ = 0, reserved_ = 0, live_blocks_ = 0;
  void (*idle_hook_)(void*) = nullptr;
  void* idle_arg_ = nullptr;
};

}  // namespace vkt
