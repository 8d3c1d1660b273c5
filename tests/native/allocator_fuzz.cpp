// Differential run of the product allocator (nvshmem_amd/csrc/mspace.cpp) against the oracle's independent
// model (oracle/nvshmem_oracle.c, which restates the reference's mspace, src/host/mem/custom_malloc.cpp:74-237),
// meant to be built with -fsanitize=address,undefined: random malloc / align / realloc / free sequences,
// every address, the free byte count and the number of free chunks compared after every operation.
// Usage: allocator_fuzz <seed> <operations>.  Prints "ok <operations> <live blocks at the end>".
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <vector>

#include "mspace.hpp"
extern "C" {
#include "nvshmem_oracle.h"
}

static uint64_t state;
static uint64_t rnd() {  // SplitMix64
    uint64_t z = (state += 0x9E3779B97F4A7C15ull);
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}

#define CHECK(cond, what)                                                               \
    do {                                                                                \
        if (!(cond)) {                                                                  \
            fprintf(stderr, "mismatch at operation %ld: %s\n", op, what);               \
            return 1;                                                                   \
        }                                                                               \
    } while (0)

int main(int argc, char **argv) {
    state = argc > 1 ? strtoull(argv[1], nullptr, 0) : 1;
    const long nops = argc > 2 ? atol(argv[2]) : 20000;
    const uint64_t base = 0x7f0000000000ull, capacity = (uint64_t)(1 + rnd() % 64) << 20;
    nvshmem_amd::SymmetricSpace mine(base, capacity);
    oracle_space_t *model = oracle_space_create(base, capacity);
    std::vector<uint64_t> live;
    long op = 0;
    for (; op < nops; ++op) {
        const unsigned kind = (unsigned)(rnd() % 100);
        const uint64_t size_class = rnd() % 4;
        const uint64_t bytes = size_class == 0 ? rnd() % 64 : size_class == 1 ? rnd() % 4096
                             : size_class == 2 ? rnd() % (256 << 10) : rnd() % (capacity / 2 + 1);
        if (kind < 35) {
            const uint64_t a = mine.allocate(bytes), b = oracle_space_alloc(model, bytes);
            CHECK(a == b, "allocate");
            if (a) live.push_back(a);
        } else if (kind < 50) {
            const uint64_t alignment = (uint64_t)8 << (rnd() % 14);
            const uint64_t a = mine.allocate_aligned(alignment, bytes), b = oracle_space_align(model, alignment, bytes);
            CHECK(a == b, "allocate_aligned");
            CHECK(a % (alignment < 512 ? 512 : alignment) == 0 || a == 0, "alignment");
            if (a) live.push_back(a);
        } else if (kind < 65 && !live.empty()) {
            const size_t i = rnd() % live.size();
            uint64_t from_a = 0, from_b = 0;
            const uint64_t a = mine.reallocate(live[i], bytes, &from_a);
            const uint64_t b = oracle_space_realloc(model, live[i], bytes, &from_b);
            CHECK(a == b && from_a == from_b, "reallocate");
            if (a) live[i] = a;
            else if (bytes == 0) { live[i] = live.back(); live.pop_back(); }
        } else if (!live.empty()) {
            const size_t i = rnd() % live.size();
            const bool a = mine.deallocate(live[i]);
            const int b = oracle_space_free(model, live[i]);
            CHECK(a && b == 0, "deallocate");
            live[i] = live.back();
            live.pop_back();
        } else {
            CHECK(!mine.deallocate(base + 512 * (rnd() % 1000)), "free of an address that is not live");
        }
        CHECK(mine.free_bytes() == oracle_space_free_bytes(model), "free bytes");
        CHECK(mine.free_chunks() == oracle_space_free_chunks(model), "free chunks");
        CHECK(mine.live_blocks() == live.size(), "live blocks");
    }
    while (!live.empty()) {
        CHECK(mine.deallocate(live.back()) && oracle_space_free(model, live.back()) == 0, "final free");
        live.pop_back();
    }
    CHECK(mine.free_chunks() == 1 && mine.free_bytes() == mine.total_bytes(), "everything coalesced");
    oracle_space_destroy(model);
    printf("ok %ld\n", nops);
    return 0;
}
