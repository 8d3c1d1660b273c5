#include "mspace.hpp"

namespace nvshmem_amd {

namespace {
inline uint64_t round_up(uint64_t v, uint64_t a) { return (v + a - 1) / a * a; }
}  // namespace

SymmetricSpace::SymmetricSpace(uint64_t base, uint64_t capacity) {
    const uint64_t start = round_up(base, kGranule);
    const uint64_t skipped = start - base;
    if (capacity > skipped) {
        total_ = capacity - skipped;
        free_[start] = total_;
    }
}

// Insert [addr, addr+bytes) into the free map, fusing with the chunk that ends at addr and the
// chunk that starts at addr+bytes.
void SymmetricSpace::release(uint64_t addr, uint64_t bytes) {
    if (bytes == 0) return;
    auto next = free_.lower_bound(addr);
    if (next != free_.begin()) {
        auto prev = std::prev(next);
        if (prev->first + prev->second == addr) {
            addr = prev->first;
            bytes += prev->second;
            free_.erase(prev);
        }
    }
    if (next != free_.end() && next->first == addr + bytes) {
        bytes += next->second;
        free_.erase(next);
    }
    free_[addr] = bytes;
}

uint64_t SymmetricSpace::allocate(uint64_t bytes) {
    if (bytes == 0) return 0;
    if (bytes > UINT64_MAX - kGranule) return 0;
    bytes = round_up(bytes, kGranule);
    for (auto it = free_.begin(); it != free_.end(); ++it) {
        if (it->second < bytes) continue;
        const uint64_t addr = it->first;
        const uint64_t rest = it->second - bytes;
        free_.erase(it);
        if (rest) free_[addr + bytes] = rest;
        live_[addr] = bytes;
        return addr;
    }
    return 0;
}

uint64_t SymmetricSpace::allocate_aligned(uint64_t alignment, uint64_t bytes) {
    if (alignment == 0 || (alignment & (alignment - 1)) || (alignment % sizeof(void *))) return 0;
    if (bytes > UINT64_MAX - alignment) return 0;
    const uint64_t raw = allocate(bytes + alignment);
    if (!raw) return 0;
    const uint64_t addr = round_up(raw, alignment);
    if (addr != raw) {
        const uint64_t front = addr - raw;
        const uint64_t len = live_[raw];
        live_.erase(raw);
        live_[addr] = len - front;
        release(raw, front);
    }
    return addr;
}

uint64_t SymmetricSpace::reallocate(uint64_t addr, uint64_t bytes, uint64_t *moved_from) {
    if (moved_from) *moved_from = 0;
    auto it = live_.find(addr);
    if (it == live_.end()) return 0;
    bytes = round_up(bytes, kGranule);
    const uint64_t cur = it->second;
    if (bytes == cur) return addr;
    if (bytes < cur) {
        if (bytes == 0) return addr;
        it->second = bytes;
        release(addr + bytes, cur - bytes);
        return addr;
    }
    // Grow in place when the chunk right behind the block is free and large enough.  (The
    // reference's in-place branch returns `bytes - cur` of the consumed chunk to the free list
    // instead of the real remainder, custom_malloc.cpp:210-213; the remainder is used here.)
    auto nx = free_.find(addr + cur);
    if (nx != free_.end() && cur + nx->second >= bytes) {
        const uint64_t rest = cur + nx->second - bytes;
        free_.erase(nx);
        it->second = bytes;
        if (rest) free_[addr + bytes] = rest;
        return addr;
    }
    const uint64_t fresh = allocate(bytes);
    if (!fresh) return 0;
    live_.erase(addr);
    release(addr, cur);
    if (moved_from) *moved_from = addr;
    return fresh;
}

bool SymmetricSpace::deallocate(uint64_t addr) {
    auto it = live_.find(addr);
    if (it == live_.end()) return false;
    const uint64_t bytes = it->second;
    live_.erase(it);
    release(addr, bytes);
    return true;
}

uint64_t SymmetricSpace::inuse_size(uint64_t addr) const {
    auto it = live_.find(addr);
    return it == live_.end() ? 0 : it->second;
}

uint64_t SymmetricSpace::free_bytes() const {
    uint64_t s = 0;
    for (const auto &c : free_) s += c.second;
    return s;
}

}  // namespace nvshmem_amd
