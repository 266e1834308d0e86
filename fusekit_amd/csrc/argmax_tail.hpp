// Greedy argmax over bf16 logits as packed 64-bit candidates, shared by the stand-alone argmax launch and by the
// LM-head GEMV that selects the token itself.
//
// A candidate is (order-preserving key of the logit << 32) | ~index: the maximum of the packed values is the largest
// logit with the LOWEST index, the reference's `v > max` scan order (argmax_logits_decode.rs:63-95; the direct head
// keeps (value, index) pairs per threadgroup and a finalize kernel, msl.rs:1674-1890).  NaN maps to key 0 and never
// wins; an all-NaN row yields token 0.
//
// Every block reduces what its threads hold to one candidate, stores it write-through, and counts itself in on an
// atomic counter; the block that counts last reduces all candidates, writes the token (and its history entry) and
// leaves the counter at zero for the next launch.
#pragma once
#include "fk_device.hpp"

namespace fk {

struct ArgmaxTail {
    uint32_t* next_token;
    uint32_t* history;  // optional: history[(*hist_counter)++] = token
    uint32_t* hist_counter;
    uint32_t hist_capacity;
    uint64_t* partial;  // [gridDim.x]
    uint32_t* counter;  // zero before the first launch
};

__device__ __forceinline__ uint32_t order_key(float v) {
    if (v != v) return 0u;
    const uint32_t u = __float_as_uint(v);
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

__device__ __forceinline__ uint64_t argmax_candidate(uint32_t bf16_bits, uint32_t index) {
    return ((uint64_t)order_key(bf16_bits_to_f32((uint16_t)bf16_bits)) << 32) | (uint32_t)(~index);
}

// Called by all BLOCK threads of every block of the launch, each with the best candidate it has seen (0: none).
// `sm` holds BLOCK / 64 entries of LDS, `is_last` one.
template <int BLOCK>
__device__ __forceinline__ void argmax_block_finish(const ArgmaxTail& t, uint64_t best, uint64_t* sm, uint32_t* is_last) {
    auto block_best = [&](uint64_t v) {
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) {
            const uint64_t other = __shfl_xor(v, o, kWave);
            v = other > v ? other : v;
        }
        if ((threadIdx.x & (kWave - 1)) == 0) sm[threadIdx.x / kWave] = v;
        __syncthreads();
        uint64_t r = sm[0];
#pragma unroll
        for (int w = 1; w < BLOCK / kWave; ++w) r = sm[w] > r ? sm[w] : r;
        __syncthreads();
        return r;
    };
    best = block_best(best);
    // The candidate is stored write-through (agent scope) and its arrival awaited before the block counts itself
    // in; the last block reads the candidates past the caches.  No device-wide fence (which would write back a
    // whole L2).
    if (threadIdx.x == 0) {
        __hip_atomic_store(&t.partial[blockIdx.x], best, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        wait_memory_ops_done();
        *is_last = (atomicAdd(t.counter, 1u) == gridDim.x - 1) ? 1u : 0u;
    }
    __syncthreads();
    if (!*is_last) return;
    // Eight candidates per thread are requested before the first is looked at (a grid of up to 2048 blocks is one
    // round trip to the L2 instead of eight in a row); indices past the grid repeat its last candidate.
    uint64_t fin = 0;
    constexpr int kAhead = 8;
    for (uint32_t base = threadIdx.x; base < gridDim.x; base += BLOCK * kAhead) {
        uint64_t c[kAhead];
#pragma unroll
        for (int u = 0; u < kAhead; ++u) {
            const uint32_t i = base + u * BLOCK;
            c[u] = __hip_atomic_load(&t.partial[i < gridDim.x ? i : gridDim.x - 1], __ATOMIC_RELAXED,
                                     __HIP_MEMORY_SCOPE_AGENT);
        }
#pragma unroll
        for (int u = 0; u < kAhead; ++u) fin = c[u] > fin ? c[u] : fin;
    }
    fin = block_best(fin);
    if (threadIdx.x == 0) {
        const uint32_t tok = (fin >> 32) ? ~(uint32_t)fin : 0u;
        *t.next_token = tok;
        if (t.history && t.hist_counter) {
            const uint32_t slot = *t.hist_counter;
            if (slot < t.hist_capacity) t.history[slot] = tok;
            *t.hist_counter = slot + 1;
        }
        __hip_atomic_store(t.counter, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
}

}  // namespace fk
