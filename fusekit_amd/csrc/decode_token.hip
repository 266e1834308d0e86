// Whole-token persistent decode kernel for gfx950.
//
// One launch runs the complete decode pipeline of one token -- embedding, every
// layer's [rmsnorm+qkv | head-norm/rope + KV append + sdpa | o_proj+residual |
// rmsnorm+gate/up+SwiGLU | down+residual], final norm + LM head, argmax -- with
// the same device functions as the one-kernel-per-task path (gemv_run,
// sdpa_block), so the arithmetic is identical.  The grid is exactly what is
// resident at once; phases are separated by a grid barrier (see grid_barrier).  What a kernel boundary cannot
// do and this can: before arriving at a barrier every block issues the 16-byte
// weight loads of its first batch of the NEXT phase, which do not depend on the
// activations, so HBM keeps streaming across the dependency.
#include "fk_host.hpp"
#include "decode_token.hpp"

namespace fk {

namespace {

// The per-phase argument blocks live in device memory and never change while
// the kernel runs; viewing them through the constant address space makes every
// field access a scalar load (as for kernel arguments).
typedef __attribute__((address_space(4))) GemvArgs ConstGemvArgs;
typedef __attribute__((address_space(4))) SdpaArgs ConstSdpaArgs;
__device__ __forceinline__ const ConstGemvArgs& gemv_args(const GemvArgs* base, uint32_t i) {
    return *(const ConstGemvArgs*)(base + i);
}
__device__ __forceinline__ const ConstSdpaArgs& sdpa_args(const SdpaArgs* base, uint32_t i) {
    return *(const ConstSdpaArgs*)(base + i);
}

// Grid barrier without device-wide fences.  A device-scope fence writes back and
// invalidates a whole L2 and costs ~30 ns per block per barrier on this part
// (30 us for 1024 blocks); instead every byte that crosses blocks inside this
// kernel moves through agent-scope accesses (ld_u16 / st_u16 and friends), so a
// barrier only has to (1) wait until this block's stores have completed
// (every wave waits for its own memory counter, then the block barrier), (2) count arrivals on two levels of counters -- one
// per group of kBarFan blocks, then one for the groups, so no address sees more
// than kBarFan atomics -- and (3) let the last arriver publish the epoch in a flag
// the others poll.  All counters are monotonic across launches.
constexpr uint32_t kBarFan = 32;

struct BarrierState {
    unsigned long long epoch;   // the barrier this block is about to pass
    unsigned long long first_epoch;
    uint32_t gsize, ngrp;
    unsigned long long* c1;     // this block's group counter
};

__device__ __forceinline__ void grid_barrier(const TokenArgs& t, BarrierState& b) {
    wait_memory_ops_done();  // this wave's write-through stores have landed
    __syncthreads();
    if (threadIdx.x == 0) {
        bool released = false;
        const unsigned long long prev = atomicAdd(b.c1, 1ull);
        if (prev + 1 == b.epoch * b.gsize) {
            const unsigned long long p2 = atomicAdd(t.bar_counter, 1ull);
            if (p2 + 1 == b.epoch * b.ngrp) {
                __hip_atomic_store(t.bar_flag, b.epoch, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                released = true;
            }
        }
        uint32_t spins = 0;
        while (!released && __hip_atomic_load(t.bar_flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < b.epoch) {
            ++spins;
            if ((spins & 63u) == 0u && __hip_atomic_load(t.abort_flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0u)
                break;
            if (spins > t.spin_limit) {
                __hip_atomic_store(t.abort_flag, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                break;
            }
            __builtin_amdgcn_s_sleep(1);
        }
    }
    __syncthreads();
    b.epoch += 1;
    if (t.trace && blockIdx.x == 0 && threadIdx.x == 0) {
        const uint32_t i = (uint32_t)(b.epoch - b.first_epoch);
        if (i < t.trace_capacity) t.trace[i] = wall_clock64();
    }
}

__device__ __forceinline__ uint32_t order_key(float v) {
    if (v != v) return 0u;
    const uint32_t u = __float_as_uint(v);
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

__device__ __forceinline__ unsigned long long block_best(unsigned long long v, unsigned long long* sm) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        const unsigned long long other = __shfl_xor(v, o, kWave);
        v = other > v ? other : v;
    }
    if ((threadIdx.x & (kWave - 1)) == 0) sm[threadIdx.x / kWave] = v;
    __syncthreads();
    unsigned long long r = sm[0];
#pragma unroll
    for (int w = 1; w < kGemvBlock / kWave; ++w) r = sm[w] > r ? sm[w] : r;
    __syncthreads();
    return r;
}

// The attention phase as a function of its own: its register needs (in-flight K/V
// rows, per-head accumulators, trigonometry) then do not merge with the streaming
// phases' allocation.
// Only blocks that own a work item call it (the caller tests bid < items): its
// prologue saves ~150 registers per lane, which 1000 idle blocks must not pay.
template <int GT>
__device__ __noinline__ void attention_phase(const SdpaArgs* sdpa, uint32_t l, uint32_t kv_len, uint32_t bid,
                                             uint32_t nb) {
    // named here, not passed in: a pointer parameter would be a generic pointer and
    // every LDS access in the phase would become a FLAT instruction
    extern __shared__ uint4 lds_raw[];
    float* lds = reinterpret_cast<float*>(lds_raw);
    const ConstSdpaArgs& s = sdpa_args(sdpa, l);
    const uint32_t G = s.n_heads / s.n_kv, gz_count = (G + GT - 1) / GT;
    const uint32_t n_active = (kv_len + s.chunk_len - 1) / s.chunk_len;
    const uint32_t items = n_active * s.n_kv * gz_count;
    for (uint32_t it = bid; it < items; it += nb) {
        const uint32_t split = it % n_active, rest = it / n_active;
        sdpa_block<GT, true, ConstSdpaArgs>(s, kv_len, split, rest % s.n_kv, rest / s.n_kv, gz_count, lds);
        __syncthreads();
    }
}

}  // namespace

template <WKind KIND, int GT>
__global__ __launch_bounds__(kGemvBlock) __attribute__((amdgpu_waves_per_eu(4, 8))) void decode_token_kernel(const TokenArgs t) {
    extern __shared__ uint4 lds_raw[];
    const uint32_t bid = blockIdx.x, nb = gridDim.x, tid = threadIdx.x;

    BarrierState bar;
    {
        const uint32_t grp = bid / kBarFan, g0 = grp * kBarFan;
        bar.ngrp = (nb + kBarFan - 1) / kBarFan;
        bar.gsize = (nb - g0) < kBarFan ? (nb - g0) : kBarFan;
        bar.c1 = t.bar_groups + grp * 16;  // one counter per 128-byte line
        bar.epoch = bar.first_epoch = *t.bar_base + 1;
        if (t.trace && bid == 0 && tid == 0) t.trace[0] = wall_clock64();
    }
    // every block reads the step counter before the first barrier; block 0 advances it after
    const uint32_t pos = *t.step_counter;
    const uint32_t kv_len = pos + 1;
    const uint32_t token_in = *t.token;

    uint4 wa[kGemvUnroll];
    uint32_t sa[kGemvUnroll], ba[kGemvUnroll];

    // ---- embedding: x0 = T(embed[token] * scale) (embed_lookup_decode.rs:74-99) ----
    {
        const ConstGemvArgs& g0 = gemv_args(t.gemv, 0);
        gemv_prefetch<KIND, 1>(g0, bid, wa, sa, ba);
        const uint32_t tok = token_in < t.vocab ? token_in : t.vocab - 1;
        if (bid == nb - 1 && tid < t.rope_dims / 2) {  // this token's rotary table, once for all layers
            float cs, sn;
            rope_cos_sin(tid, t.rope_dims / 2, pos, t.rope_base_log2, cs, sn);
            st_f32<true>(t.rope_tab + 2 * tid, cs);
            st_f32<true>(t.rope_tab + 2 * tid + 1, sn);
        }
        const uint32_t d = bid * kGemvBlock + tid;
        if (d < t.hidden)
            st_u16<true>(t.x0 + d, f32_to_bf16_bits(bf16_bits_to_f32(t.embed[(size_t)tok * t.hidden + d]) * t.embed_scale));
    }
    grid_barrier(t, bar);
    if (bid == 0 && tid == 0) {
        *t.step_counter = pos + 1;
        *t.offset = pos;
        *t.kv_len = kv_len;
    }

    for (uint32_t l = 0; l < t.n_layers; ++l) {
        // ---- rmsnorm + q/k/v projections ----
        gemv_run<KIND, 1, true>(gemv_args(t.gemv, 4 * l), bid, nb, lds_raw, wa, sa, ba);
        grid_barrier(t, bar);
        // ---- head norm / rope / KV append / attention ----
        {
            const ConstSdpaArgs& s = sdpa_args(t.sdpa, l);
            const uint32_t G = s.n_heads / s.n_kv, gz_count = (G + GT - 1) / GT;
            const uint32_t n_active = (kv_len + s.chunk_len - 1) / s.chunk_len;
            if (bid < n_active * s.n_kv * gz_count) attention_phase<GT>(t.sdpa, l, kv_len, bid, nb);
            gemv_prefetch<KIND, 1>(gemv_args(t.gemv, 4 * l + 1), bid, wa, sa, ba);
        }
        grid_barrier(t, bar);
        // ---- o_proj + residual ----
        gemv_run<KIND, 1, true>(gemv_args(t.gemv, 4 * l + 1), bid, nb, lds_raw, wa, sa, ba);
        gemv_prefetch<KIND, 2>(gemv_args(t.gemv, 4 * l + 2), bid, wa, sa, ba);
        grid_barrier(t, bar);
        // ---- rmsnorm + gate/up + SwiGLU ----
        gemv_run<KIND, 2, true>(gemv_args(t.gemv, 4 * l + 2), bid, nb, lds_raw, wa, sa, ba);
        gemv_prefetch<KIND, 1>(gemv_args(t.gemv, 4 * l + 3), bid, wa, sa, ba);
        grid_barrier(t, bar);
        // ---- down_proj + residual ----
        gemv_run<KIND, 1, true>(gemv_args(t.gemv, 4 * l + 3), bid, nb, lds_raw, wa, sa, ba);
        if (l + 1 < t.n_layers)
            gemv_prefetch<KIND, 1>(gemv_args(t.gemv, 4 * l + 4), bid, wa, sa, ba);
        else
            gemv_prefetch<W_BF16, 1>(gemv_args(t.gemv, 4 * l + 4), bid, wa, sa, ba);
        grid_barrier(t, bar);
    }

    // ---- final norm + LM head (dense bf16) ----
    gemv_run<W_BF16, 1, true>(gemv_args(t.gemv, 4 * t.n_layers), bid, nb, lds_raw, wa, sa, ba);
    grid_barrier(t, bar);

    // ---- greedy argmax, lowest index wins ties (argmax_logits_decode.rs:63-95) ----
    unsigned long long* sm = reinterpret_cast<unsigned long long*>(lds_raw);
    {
        unsigned long long best = 0;
        for (uint32_t i = bid * kGemvBlock + tid; i < t.vocab; i += nb * kGemvBlock) {
            const unsigned long long cand =
                ((unsigned long long)order_key(bf16_bits_to_f32(t.logits[i])) << 32) | (uint32_t)(~i);
            best = cand > best ? cand : best;
        }
        best = block_best(best, sm);
        if (tid == 0) __hip_atomic_store(&t.argmax_partial[bid], best, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    grid_barrier(t, bar);
    if (bid == 0) {
        unsigned long long fin = 0;
        for (uint32_t i = tid; i < nb; i += kGemvBlock) {
            const unsigned long long c = __hip_atomic_load(&t.argmax_partial[i], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            fin = c > fin ? c : fin;
        }
        fin = block_best(fin, sm);
        if (tid == 0) {
            const uint32_t tok = (fin >> 32) ? ~(uint32_t)fin : 0u;
            *t.token = tok;
            const uint32_t slot = *t.hist_counter;
            if (slot < t.hist_capacity) t.history[slot] = tok;
            *t.hist_counter = slot + 1;
            *t.bar_base = bar.epoch - 1;  // barriers passed so far; the next launch counts on from here
        }
    }
}

namespace {
template <WKind KIND>
const void* pick_gt(int gt) {
    switch (gt) {
        case 2: return reinterpret_cast<const void*>(&decode_token_kernel<KIND, 2>);
        case 4: return reinterpret_cast<const void*>(&decode_token_kernel<KIND, 4>);
        case 8: return reinterpret_cast<const void*>(&decode_token_kernel<KIND, 8>);
        default: return nullptr;
    }
}
const void* pick(int kind, int gt) {
    switch (kind) {
        case W_Q4: return pick_gt<W_Q4>(gt);
        case W_Q8: return pick_gt<W_Q8>(gt);
        case W_BF16: return pick_gt<W_BF16>(gt);
        default: return nullptr;
    }
}
}  // namespace

fk_status token_kernel_max_grid(int kind, int gt, uint32_t lds_bytes, uint32_t* grid) {
    const DeviceFacts* dev;
    FK_TRY(device_facts(&dev));
    const void* f = pick(kind, gt);
    if (!f) return set_error(FK_ERR_UNSUPPORTED, "token kernel: unsupported weight kind or GQA group size");
    if ((int)lds_bytes > dev->max_dyn_lds) return set_error(FK_ERR_UNSUPPORTED, "token kernel: LDS need exceeds the CU");
    if (lds_bytes > 48 * 1024) FK_HIP(hipFuncSetAttribute(f, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes));
    int per_cu = 0;
    FK_HIP(hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, f, kGemvBlock, lds_bytes));
    if (per_cu < 1) return set_error(FK_ERR_UNSUPPORTED, "token kernel: does not fit on a compute unit");
    *grid = (uint32_t)per_cu * (uint32_t)dev->cus;
    return FK_OK;
}

fk_status plan_token_kernel(const TokenKernelSpec& spec, uint32_t grid, Launch* out) {
    const void* f = pick(spec.kind, spec.gt);
    if (!f) return set_error(FK_ERR_UNSUPPORTED, "token kernel: unsupported weight kind or GQA group size");
    uint32_t max_grid = 0;
    FK_TRY(token_kernel_max_grid(spec.kind, spec.gt, spec.lds_bytes, &max_grid));
    // every block must be resident at once: the grid barrier waits for all of them
    if (grid == 0 || grid > max_grid) return set_error(FK_ERR_INVALID, "token kernel: grid exceeds what is resident at once");
    out->func = f;
    out->grid = dim3(grid, 1, 1);
    out->block = dim3(kGemvBlock, 1, 1);
    out->shmem = spec.lds_bytes;
    out->set_args(spec.args);
    return FK_OK;
}

}  // namespace fk
