// Mixture-of-experts token shuffle, the workload of the reference's examples/moe_shuffle.cu: every PE
// holds `tokens` rows and sends each of them to the PEs that own its top-k experts (dispatch), where
// the rows land grouped by (expert, source PE, token order); combine fetches every copy back to the
// slot it came from.  Steps: exchange the per-expert counts and prefix-sum them into segment offsets
// (moe_shuffle.cu:204-234), push rows with non-blocking puts, announce the row counts with ADD
// signals and wait for the expected counts (the put_signal + signal_wait_until(GE) idiom of
// examples/ring-reduce.cu:111-127), then gather.  Checks: every receive buffer holds exactly the
// rows that were routed to it, in order, and combine(dispatch(x)) gives every row back k times.
#include <cstring>

#include "example_util.hpp"

constexpr int kMaxPes = 64;

// counts: rows this PE sends to each expert.  Afterwards seg[e * npes + s] on every PE is the first
// receive row of the segment (expert e, source PE s) and my_rows[0] the rows this PE receives.
__global__ void exchange_offsets(const int64_t *counts, int64_t *seg, int64_t *my_rows, int experts) {
    extern __shared__ int64_t table[];  // [expert][source PE]
    const int me = nvshmem_my_pe(), np = nvshmem_n_pes(), per_pe = experts / np;
    for (int i = threadIdx.x; i < experts * np; i += blockDim.x) table[i] = nvshmem_int64_g(counts + i / np, i % np);
    __syncthreads();
    int64_t *mine = (int64_t *)nvshmem_ptr(seg, me);
    for (int d = threadIdx.x; d < np; d += blockDim.x) {
        int64_t run = 0;  // segments restart at row 0 on every destination PE
        for (int i = d * per_pe * np; i < (d + 1) * per_pe * np; ++i) {
            mine[i] = run;
            run += table[i];
        }
        if (d == me) *(int64_t *)nvshmem_ptr(my_rows, me) = run;
    }
}

// One token per wavefront: k puts back to back, a tally per destination in LDS, one signal per
// destination and block once the block's puts are complete, then the receiver's wait.
__global__ void dispatch(char *recv, const char *send, const int *dest_pe, const int64_t *dest_row,
                         const uint64_t *expected, uint64_t *arrived, int tokens, int topk, size_t row_bytes) {
    __shared__ unsigned tally[kMaxPes];
    const int me = nvshmem_my_pe(), np = nvshmem_n_pes();
    const int *to_pe = (const int *)nvshmem_ptr(dest_pe, me);
    const int64_t *to_row = (const int64_t *)nvshmem_ptr(dest_row, me);
    for (int i = threadIdx.x; i < np; i += blockDim.x) tally[i] = 0;
    __syncthreads();
    const int waves = blockDim.x / 64, wave = blockIdx.x * waves + threadIdx.x / 64;
    for (int t = wave; t < tokens; t += gridDim.x * waves)
        for (int k = 0; k < topk; ++k) {
            const int pe = to_pe[t * topk + k];
            nvshmemx_putmem_nbi_warp(recv + to_row[t * topk + k] * row_bytes, send + (size_t)t * row_bytes, row_bytes, pe);
            if (threadIdx.x % 64 == 0) atomicAdd(&tally[pe], 1u);
        }
    nvshmemx_quiet_block();
    for (int pe = threadIdx.x; pe < np; pe += blockDim.x)
        if (tally[pe]) nvshmemx_signal_op(arrived + me, tally[pe], NVSHMEM_SIGNAL_ADD, pe);
    if (blockIdx.x == 0) {
        const uint64_t *want = (const uint64_t *)nvshmem_ptr(expected, me);
        for (int s = threadIdx.x; s < np; s += blockDim.x) nvshmem_signal_wait_until(arrived + s, NVSHMEM_CMP_GE, want[s]);
    }
}

__global__ void combine(char *out, const char *recv, const int *dest_pe, const int64_t *dest_row, int copies,
                        size_t row_bytes) {
    const int me = nvshmem_my_pe();
    const int *from_pe = (const int *)nvshmem_ptr(dest_pe, me);
    const int64_t *from_row = (const int64_t *)nvshmem_ptr(dest_row, me);
    const int waves = blockDim.x / 64, wave = blockIdx.x * waves + threadIdx.x / 64;
    for (int r = wave; r < copies; r += gridDim.x * waves)
        nvshmemx_getmem_nbi_warp(out + (size_t)r * row_bytes, recv + from_row[r] * row_bytes, row_bytes, from_pe[r]);
}

int main() {
    nvshmem_init();
    const int np = nvshmem_n_pes();
    const int tokens = 2048, topk = 4, experts = 8 * np, per_pe = experts / np;
    const size_t row_bytes = 2048;  // 1024 bf16
    const int copies = tokens * topk;

    // routing: distinct experts per token, skewed towards the low numbers
    uint64_t rng = 0x9E3779B97F4A7C15ull;
    auto next = [&] { rng ^= rng << 13; rng ^= rng >> 7; rng ^= rng << 17; return rng; };
    std::vector<std::vector<int>> expert(np, std::vector<int>(copies));
    std::vector<std::vector<int64_t>> counts(np, std::vector<int64_t>(experts, 0));
    for (int pe = 0; pe < np; ++pe)
        for (int t = 0; t < tokens; ++t)
            for (int k = 0; k < topk; ++k) {
                int e;
                bool dup;
                do {  // the duplicate rejection loop of moe_shuffle.cu:502-506
                    const uint64_t a = next() % experts, b = next() % experts;
                    e = (int)(a < b ? a : b);
                    dup = false;
                    for (int j = 0; j < k; ++j) dup |= expert[pe][t * topk + j] == e;
                } while (dup);
                expert[pe][t * topk + k] = e;
                ++counts[pe][e];
            }

    int64_t *d_counts = (int64_t *)nvshmem_malloc(experts * sizeof(int64_t));
    int64_t *d_seg = (int64_t *)nvshmem_malloc((size_t)experts * np * sizeof(int64_t));
    int64_t *d_rows = (int64_t *)nvshmem_malloc(sizeof(int64_t));
    for (int pe = 0; pe < np; ++pe) store(d_counts, counts[pe], pe);
    hipLaunchKernelGGL(exchange_offsets, dim3(1, 1, np), dim3(256), (size_t)experts * np * sizeof(int64_t), nullptr,
                       d_counts, d_seg, d_rows, experts);
    nvshmem_barrier_all();
    const std::vector<int64_t> seg = fetch(d_seg, (size_t)experts * np, 0);
    long errors = 0;
    int64_t cap = 0;
    std::vector<int64_t> recv_rows(np);
    for (int pe = 0; pe < np; ++pe) {
        errors += fetch(d_seg, (size_t)experts * np, pe) != seg;  // every PE derived the same table
        recv_rows[pe] = fetch(d_rows, 1, pe)[0];
        int64_t want = 0;
        for (int s = 0; s < np; ++s)
            for (int e = pe * per_pe; e < (pe + 1) * per_pe; ++e) want += counts[s][e];
        errors += recv_rows[pe] != want;
        cap = recv_rows[pe] > cap ? recv_rows[pe] : cap;
    }

    // destination of every copy: its expert's PE, the segment's base plus the copy's rank among this
    // PE's copies for that expert
    std::vector<std::vector<int>> dest_pe(np, std::vector<int>(copies));
    std::vector<std::vector<int64_t>> dest_row(np, std::vector<int64_t>(copies));
    std::vector<std::vector<uint64_t>> expected(np, std::vector<uint64_t>(np, 0));
    for (int pe = 0; pe < np; ++pe) {
        std::vector<int64_t> used(experts, 0);
        for (int r = 0; r < copies; ++r) {
            const int e = expert[pe][r];
            dest_pe[pe][r] = e / per_pe;
            dest_row[pe][r] = seg[(size_t)e * np + pe] + used[e]++;
            ++expected[e / per_pe][pe];
        }
    }

    char *send = (char *)nvshmem_malloc((size_t)tokens * row_bytes);
    char *recv = (char *)nvshmem_calloc((size_t)cap, row_bytes);
    char *out = (char *)nvshmem_calloc((size_t)copies, row_bytes);
    int *d_pe = (int *)nvshmem_malloc(copies * sizeof(int));
    int64_t *d_row = (int64_t *)nvshmem_malloc(copies * sizeof(int64_t));
    uint64_t *d_expected = (uint64_t *)nvshmem_malloc(np * sizeof(uint64_t));
    uint64_t *arrived = (uint64_t *)nvshmem_calloc(np, sizeof(uint64_t));
    std::vector<std::vector<char>> rows(np, std::vector<char>((size_t)tokens * row_bytes));
    for (int pe = 0; pe < np; ++pe) {
        for (char &c : rows[pe]) c = (char)next();
        store(send, rows[pe], pe);
        store(d_pe, dest_pe[pe], pe);
        store(d_row, dest_row[pe], pe);
        store(d_expected, expected[pe], pe);
    }

    void *dargs[] = {&recv, &send, &d_pe, &d_row, &d_expected, &arrived, (void *)&tokens, (void *)&topk, (void *)&row_bytes};
    NVSHMEM_CHECK(nvshmemx_collective_launch((const void *)dispatch, dim3(16), dim3(256), dargs, 0, nullptr));
    nvshmem_barrier_all();
    for (int src = 0; src < np; ++src)  // every row sits where the plan says
        for (int r = 0; r < copies; ++r) {
            char got[64];
            const char *at = (const char *)nvshmem_ptr(recv, dest_pe[src][r]) + dest_row[src][r] * row_bytes;
            if (r % 97 == 0 || r == copies - 1) {  // spot check: first 64 bytes of a sample of rows
                HIP_CHECK(hipMemcpy(got, at, sizeof got, hipMemcpyDeviceToHost));
                errors += memcmp(got, rows[src].data() + (size_t)(r / topk) * row_bytes, sizeof got) != 0;
            }
        }
    for (int pe = 0; pe < np; ++pe) errors += fetch(arrived, np, pe) != expected[pe];

    hipLaunchKernelGGL(combine, dim3(64, 1, np), dim3(256), 0, nullptr, out, recv, d_pe, d_row, copies, row_bytes);
    nvshmem_barrier_all();
    for (int pe = 0; pe < np; ++pe) {  // the round trip returns every row topk times
        const std::vector<char> got = fetch(out, (size_t)copies * row_bytes, pe);
        for (int r = 0; r < copies; ++r)
            errors += memcmp(got.data() + (size_t)r * row_bytes, rows[pe].data() + (size_t)(r / topk) * row_bytes, row_bytes) != 0;
    }
    for (void *p : {(void *)d_counts, (void *)d_seg, (void *)d_rows, (void *)send, (void *)recv, (void *)out, (void *)d_pe,
                    (void *)d_row, (void *)d_expected, (void *)arrived})
        nvshmem_free(p);
    return finish("moe_shuffle", errors);
}
