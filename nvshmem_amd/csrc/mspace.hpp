// Symmetric-space allocator: manages one PE's slice by address; every PE uses the same offsets.
//
// Behavioural contract (reference class mspace, src/host/mem/custom_malloc.cpp:74-237, declared in
// src/include/internal/host/custom_malloc.h:18-48): lowest-address first fit, requests rounded up
// to 512 bytes, the remainder of a split chunk stays free, a freed chunk merges with free
// neighbours on both sides, an aligned request over-allocates by `alignment` and gives the unused
// front back.  The bookkeeping here is one address-ordered free map plus a hash of live blocks.
#pragma once

#include <cstddef>
#include <cstdint>
#include <iterator>
#include <map>
#include <unordered_map>

namespace nvshmem_amd {

class SymmetricSpace {
  public:
    static constexpr uint64_t kGranule = 512;

    SymmetricSpace(uint64_t base, uint64_t capacity);

    // Each returns 0 when the request cannot be served.
    uint64_t allocate(uint64_t bytes);
    uint64_t allocate_aligned(uint64_t alignment, uint64_t bytes);
    // *moved_from receives the old address when the block had to move (caller copies the bytes).
    uint64_t reallocate(uint64_t addr, uint64_t bytes, uint64_t *moved_from);
    // false: addr is not the start of a live block.
    bool deallocate(uint64_t addr);

    uint64_t inuse_size(uint64_t addr) const;
    uint64_t free_bytes() const;
    uint64_t free_chunks() const { return free_.size(); }
    uint64_t live_blocks() const { return live_.size(); }
    uint64_t total_bytes() const { return total_; }

  private:
    void release(uint64_t addr, uint64_t bytes);

    std::map<uint64_t, uint64_t> free_;            // start -> length, address ordered
    std::unordered_map<uint64_t, uint64_t> live_;  // start -> length
    uint64_t total_ = 0;
};

}  // namespace nvshmem_amd
