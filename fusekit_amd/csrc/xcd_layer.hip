// XCD-resident decoder layer: the attention launch and the MLP launch (see xcd_layer.hpp for the scheme).
#include "xcd_layer.hpp"

// Timing probes (empty in the library build): launch k (0 attention, 1 MLP), boundary i, by the first thread of
// the block's first and last wave-pair.
#include "fk_probe.hpp"
FK_PROBE_DEFINE(xcd, 1024, 16)
#define FK_XCD_STAMP(k, i) FK_PROBE_STAMP(xcd, 1024, 16, (k) * 512 + blockIdx.x, threadIdx.x == 0 || threadIdx.x == 256, i)

#include "xcd_device.hpp"

namespace fk {

// =============================================================================================== MLP launch
constexpr int kMlpBlock = kBlock;

// One MLP phase of one block.  `sync` carries the block's XCD, slot and hand-over epoch; `xres_in` / `xres_out`:
// the residual row in LDS (token kernel only).
// EARLY: the caller has already issued input_request into `inr` (the stand-alone launch does so before anything
// else, from its leading parameters).
template <WKind KIND, int NLA, int NLB, bool TOKEN, bool EARLY, bool ONE = false, typename ARGS, typename LEAD>
__device__ __forceinline__ void xcd_mlp_phase(const ARGS& a, const LEAD& lead, InputRegs& inr, XcdSync& sync, uint4* lds_raw,
                                              const uint4* xres_in, uint4* xres_out) {
    const uint32_t cs_max = a.cs_max, work_floats = a.work_floats;
    constexpr int PIECES = ChunkTraits<KIND>::kPieces;
    uint4* xs = lds_raw;
    float* sx = reinterpret_cast<float*>(xs + PIECES * cs_max);
    float* work = sx + cs_max;
    constexpr uint32_t MW = meta_words<ONE>();
    uint32_t* meta = reinterpret_cast<uint32_t*>(work + work_floats);  // [3][MW]
    float* red = reinterpret_cast<float*>(meta + 3 * MW);              // [16]
    const uint32_t tid = threadIdx.x;
    constexpr bool streams = true;

    FK_XCD_STAMP(1, 0);
    const uint32_t per_xcd = a.inter / kXcds;
    const uint32_t gu0 = sync.slot * a.gu_rows;
    const uint32_t gu_n = gu0 < per_xcd ? ((per_xcd - gu0) < a.gu_rows ? (per_xcd - gu0) : a.gu_rows) : 0u;
    const Tile tg = make_tile(sync.xcd * per_xcd + gu0, gu_n, 0, a.gate.cpr);
    const uint32_t d0 = sync.slot * a.down_rows;
    const uint32_t d_n = d0 < a.in.hidden ? ((a.in.hidden - d0) < a.down_rows ? (a.in.hidden - d0) : a.down_rows) : 0u;
    const Tile td = make_tile(d0, d_n, sync.xcd * a.down_cs, a.down_cs);

    MetaRegs mg, mu, md;
    TileRegs<NLA> rg, ru;
    TileRegs<NLB> rd;
    TilePos<NLA> pg;
    TilePos<NLB> pd;
    // Requested now, behind the input: the groups' scales and biases and the first pass of gate / up -- a few
    // KiB per CU.  The later passes stream while the earlier ones are consumed; the down_proj slice is queued
    // behind the last of them.
    if constexpr (!EARLY) input_request<TOKEN>(lead, inr, xres_in);
    tile_pos_init<NLA, kBlock>(a.gate, tg, tid, pg);
    tile_pos_init<NLB, kBlock>(a.down, td, tid, pd);
    meta_fetch<KIND, kBlock, true, !ONE>(a.gate, tg, tid, mg);
    meta_fetch<KIND, kBlock, true, !ONE>(a.up, tg, tid, mu);
    // Only kGuAhead requests of the gate matrix go out ahead of the input's staging, the rest of the pass and the up
    // matrix's behind it: a wave cannot stage before it has ISSUED what stands in front, issue stalls once the CU's
    // request queue is full, and the block's staging waits for its slowest wave.  With all twelve in front the
    // median block had its activations staged 1.3 us later than the attention launch has; with none the stream
    // starts too late (4B int4, tok/s by requests in front: 12: 780, 6: 791, 4: 796, 3: 796, 2: 790, 1: 781, 0: 774; with the
    // down_proj slice requested behind the arithmetic: 6: 802, 4: 819, 3: 828, 2: 820).
    constexpr int GP = kGuAhead < NLA ? kGuAhead : NLA;
    tile_load<KIND, NLA, kBlock, 0, GP>(a.gate, tg, pg, rg);
    FK_XCD_STAMP(1, 1);
    input_pin(lead, inr);
    input_stage<KIND, 1>(a.in, inr, xs, sx, a.gate.cpr, red, xres_out);
    tile_load<KIND, NLA, kBlock, GP, NLA>(a.gate, tg, pg, rg);
    tile_load<KIND, NLA, kBlock>(a.up, tg, pg, ru);
    FK_XCD_STAMP(1, 5);
    input_clear<TOKEN>(a.in);
    meta_store<KIND, kBlock, true, !ONE>(mg, tid, meta);
    meta_store<KIND, kBlock, true, !ONE>(mu, tid, meta + MW);
    meta_fetch<KIND, kBlock, true, !ONE>(a.down, td, tid, md, sync.xcd);  // not needed before the hand-over: kept off the start-up path
    __syncthreads();

    // ---- gate / up rows of this XCD's slice, SwiGLU ----
    const uint32_t seg = (gu_n * a.gate.cpr + NLA * kBlock - 1) / (NLA * kBlock) * (NLA * kBlock);
    if (streams) {
        auto request_down = [&]() { tile_load<KIND, NLB, kBlock>(a.down, td, pd, rd); };
        if (gu_n)
            tile_run_pair<KIND, NLA, kBlock, ONE>(a.gate, a.up, tg, pg, rg, ru, xs, sx, meta, meta + MW, work, work + seg,
                                             request_down);
        else
            request_down();
    }
    FK_XCD_STAMP(1, 6);
    meta_store<KIND, kBlock, true, !ONE>(md, tid, meta + 2 * MW);
    __syncthreads();
    FK_XCD_STAMP(1, 12);
    if (streams && gu_n) {
        uint16_t* mid = a.mid + (size_t)sync.xcd * per_xcd + gu0;
        const int variant = a.swiglu_variant;
        tile_rows<true, ONE>(tg, work, work + seg,
                        [&](uint32_t r, float s0, float s1) { mid[r] = (uint16_t)swiglu_bits(s0, s1, variant, 1.0f); });

    }
    FK_XCD_STAMP(1, 7);
    uint32_t* okw = reinterpret_cast<uint32_t*>(red) + 8;
    xcd_barrier<0>(sync, okw);
    const bool ok = xcd_wait_ok(okw);  // tested in front of the additions into the sum row
    FK_XCD_STAMP(1, 8);

    // ---- down_proj over this XCD's K-slice: fp32 partial row ----
    if (streams) stage_vector<KIND>(a.mid + (size_t)sync.xcd * per_xcd, per_xcd >> 3, a.down_cs, xs, sx);
    __syncthreads();
    FK_XCD_STAMP(1, 9);
    if (streams && d_n) tile_run<KIND, NLB, kBlock, ONE>(a.down, td, pd, rd, xs, sx, meta + 2 * MW, work, []() {});
    __syncthreads();
    FK_XCD_STAMP(1, 10);
    if (streams && d_n && ok) {
        long long* out = a.out_sums;
        XcdControl* ctl = sync.ctl;
        tile_rows<false, ONE>(td, work, work, [&](uint32_t r, float s0, float) { xcd_sum_add(out, d0 + r, s0, ctl); });
    }
    FK_XCD_STAMP(1, 11);
}

template <WKind KIND, int NLA, int NLB, bool ONE>
__global__ __launch_bounds__(kMlpBlock, 2) void xcd_mlp_kernel(const long long* sums, const uint16_t* residual,
                                                               const uint16_t* norm_w, uint32_t hidden, const XcdMlpArgs a) {
    extern __shared__ uint4 lds_raw[];
    // The input is requested from the leading parameters before the argument block is touched.
    const XcdInputLead lead{sums, residual, norm_w, hidden};
    InputRegs inr;
    input_request<false>(lead, inr, nullptr);
    kernarg_warm<32 + (int)sizeof(XcdMlpArgs)>();
    XcdSync sync = xcd_sync_init(a.ctl, a.spin_limit);
    xcd_mlp_phase<KIND, NLA, NLB, false, true, ONE>(a, lead, inr, sync, lds_raw, nullptr, nullptr);
    xcd_mark_placement(sync, a.mark_placement);
}

// =============================================================================================== attention launch
constexpr int kAttnStream = kBlock;

template <WKind KIND, int NLA, int NLB, bool TOKEN, bool EARLY, bool ONE = false, typename ARGS, typename LEAD>
__device__ __forceinline__ void xcd_attn_phase(const ARGS& a, const LEAD& lead, InputRegs& inr, XcdSync& sync, uint4* lds_raw,
                                               const uint4* xres_in, uint4* xres_out) {
    const uint32_t cs_max = a.cs_max, work_floats = a.work_floats, att_elems = a.att_elems;
    (void)att_elems;
    constexpr int PIECES = ChunkTraits<KIND>::kPieces;
    uint4* xs = lds_raw;
    float* sx = reinterpret_cast<float*>(xs + PIECES * cs_max);
    float* work = sx + cs_max;
    constexpr uint32_t MW = meta_words<ONE>();
    uint32_t* meta = reinterpret_cast<uint32_t*>(work + work_floats);  // [3][MW]; two used
    uint16_t* att = reinterpret_cast<uint16_t*>(meta + 3 * MW);

    // Requested now, looked at only behind the start-up requests (the pin below): used at once, the wave would sit
    // out this load's trip to memory before it has asked for anything else.
    uint32_t kv_len_raw = *a.sdpa.kv_len_ptr;
    const uint32_t tid = threadIdx.x, ti = tid;
    constexpr bool streams = true;
    float* red = reinterpret_cast<float*>(att + ((att_elems + 7u) & ~7u));  // [16]

    FK_XCD_STAMP(0, 0);
    // tile of the q / k / v projections: the XCD's q rows first, then its k rows, then its v rows
    const uint32_t R = a.qkv_tile_rows, tix = sync.slot;
    const bool has_tile = tix < a.q_tiles + 2 * a.kv_tiles;
    const uint32_t part_id = tix < a.q_tiles ? 0u : (tix < a.q_tiles + a.kv_tiles ? 1u : 2u);
    const uint32_t tl = part_id == 0 ? tix : (part_id == 1 ? tix - a.q_tiles : tix - a.q_tiles - a.kv_tiles);
    const uint32_t part_rows = part_id == 0 ? a.q_rows : a.kv_rows;
    const uint32_t pr0 = tl * R;
    const uint32_t pr_n = has_tile ? ((part_rows - pr0) < R ? (part_rows - pr0) : R) : 0u;
    const auto& mq = part_id == 0 ? a.wq : (part_id == 1 ? a.wk : a.wv);
    const Tile tq = make_tile(sync.xcd * part_rows + pr0, pr_n, 0, a.wq.cpr);
    const uint32_t o0 = sync.slot * a.o_rows;
    const uint32_t o_n = o0 < a.in.hidden ? ((a.in.hidden - o0) < a.o_rows ? (a.in.hidden - o0) : a.o_rows) : 0u;
    const Tile to = make_tile(o0, o_n, sync.xcd * a.o_cs, a.o_cs);

    MetaRegs mmq, mmo;
    TileRegs<NLA> rq;
    TileRegs<NLB> ro;
    TilePos<NLA> pq;
    TilePos<NLB> po;
    if constexpr (!EARLY) input_request<TOKEN>(lead, inr, xres_in);
    tile_pos_init<NLA, kAttnStream>(mq, tq, ti, pq);
    tile_pos_init<NLB, kAttnStream>(a.wo, to, ti, po);
    meta_fetch<KIND, kAttnStream, true, !ONE>(mq, tq, ti, mmq);
    tile_load<KIND, NLA, kAttnStream>(mq, tq, pq, rq);  // all of it ahead of the staging: 2 or 3 of 5 were no faster here
    FK_XCD_STAMP(0, 1);
    asm volatile("" : "+v"(kv_len_raw));
    const uint32_t kv_len0 = __builtin_amdgcn_readfirstlane(kv_len_raw);
    input_pin(lead, inr);
    input_stage<KIND, 0>(a.in, inr, xs, sx, a.wq.cpr, red, xres_out);
    FK_XCD_STAMP(0, 5);
    input_clear<TOKEN>(a.in);
    meta_store<KIND, kAttnStream, true, !ONE>(mmq, ti, meta);
    meta_fetch<KIND, kAttnStream, true, !ONE>(a.wo, to, ti, mmo, sync.xcd);  // not needed before the attention is done
    __syncthreads();
    FK_XCD_STAMP(0, 13);

    // ---- q / k / v rows of this XCD's KV head; the o_proj slice is requested behind their last pass ----
    if (streams) {
        auto request_o = [&]() { tile_load<KIND, NLB, kAttnStream>(a.wo, to, po, ro); };
        if (pr_n)
            tile_run<KIND, NLA, kAttnStream, ONE>(mq, tq, pq, rq, xs, sx, meta, work, request_o);
        else
            request_o();
    }
    FK_XCD_STAMP(0, 14);
    __syncthreads();
    FK_XCD_STAMP(0, 15);
    if (pr_n) {
        uint16_t* dst = (part_id == 0 ? a.q : (part_id == 1 ? a.k : a.v)) + (size_t)sync.xcd * part_rows + pr0;
        tile_rows<false, ONE>(tq, work, work, [&](uint32_t r, float s0, float) { dst[r] = (uint16_t)f32_to_bf16_bits(s0); });
    }
    FK_XCD_STAMP(0, 6);
    uint32_t* okw = reinterpret_cast<uint32_t*>(red) + 8;
    xcd_barrier<0>(sync, okw);
    if (!xcd_wait_ok(okw)) return;  // the attention phase appends to the cache
    FK_XCD_STAMP(0, 7);

    // ---- head norm + RoPE + cache append + attention: block = (query head of the group, key range) ----
    const uint32_t G = a.sdpa.n_heads / a.sdpa.n_kv;
    {
        const uint32_t gz = sync.slot % G, split = sync.slot / G;
        if (split < a.sdpa.n_splits)
            sdpa_block<1, 2, std::remove_cv_t<std::remove_reference_t<decltype((a.sdpa))>>, 0, true, true>(a.sdpa, kv_len0, split, sync.xcd, gz, G, work);
    }
    FK_XCD_STAMP(0, 8);
    xcd_barrier<0>(sync, okw);
    const bool ok2 = xcd_wait_ok(okw);  // tested in front of the additions into the sum row
    FK_XCD_STAMP(0, 9);

    // ---- merge the ranges of each of the group's heads (range order), rows to LDS ----
    {
        const uint32_t span = a.sdpa.chunk_len * a.sdpa.chunks_per_block;
        const uint32_t covered = a.sdpa.n_splits * span < a.sdpa.capacity ? a.sdpa.n_splits * span : a.sdpa.capacity;
        const uint32_t kv_len = kv_len0 < 1u ? 1u : (kv_len0 > covered ? covered : kv_len0);
        const uint32_t n_active = (kv_len + span - 1) / span;
        const uint32_t row = a.sdpa.v_dim + 2;
        const uint32_t lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
        for (uint32_t h = wave; h < G; h += kBlock / kWave) {
            const float* ph = a.sdpa.partials + (size_t)(sync.xcd * G + h) * a.sdpa.n_splits * row;
            for (uint32_t d2 = lane; d2 < ((a.sdpa.v_dim >> 1) + kWave - 1) / kWave * kWave; d2 += kWave) {
                const bool live = d2 < (a.sdpa.v_dim >> 1);
                const float* pd = ph + 2 + 2 * (live ? d2 : 0u);
                float M = -INFINITY, L = 0.f, o0_ = 0.f, o1_ = 0.f;
                // all requests first (clamped indices: straight-line), then the fold in range order; up to 8 ranges
                // (a context of 8 x the range length) take half the requests.  The (maximum, sum) pair of range i is
                // fetched by lane i alone and handed to the wave through scalar registers: one request, not N.
                auto merge = [&](auto n_const) {
                    constexpr uint32_t N = decltype(n_const)::value;
                    float2 po[N];
                    const float2 mine = ld_f32x2<true>(ph + (size_t)(lane < n_active ? lane : 0u) * row);
#pragma unroll
                    for (uint32_t i = 0; i < N; ++i) po[i] = ld_f32x2<true>(pd + (size_t)(i < n_active ? i : 0u) * row);
                    float2 ml[N];
#pragma unroll
                    for (uint32_t i = 0; i < N; ++i) {
                        ml[i].x = __uint_as_float(__builtin_amdgcn_readlane(__float_as_uint(mine.x), i));
                        ml[i].y = __uint_as_float(__builtin_amdgcn_readlane(__float_as_uint(mine.y), i));
                    }
                    M = ml[0].x;
#pragma unroll
                    for (uint32_t i = 1; i < N; ++i) M = i < n_active ? fmaxf(M, ml[i].x) : M;
#pragma unroll
                    for (uint32_t i = 0; i < N; ++i) {
                        const float w = i < n_active ? expf(ml[i].x - M) : 0.f;
                        L = fmaf(ml[i].y, w, L);
                        o0_ = fmaf(po[i].x, w, o0_);
                        o1_ = fmaf(po[i].y, w, o1_);
                    }
                };
                if (n_active <= kXcdMaxRanges / 4)
                    merge(std::integral_constant<uint32_t, kXcdMaxRanges / 4>{});
                else if (n_active <= kXcdMaxRanges / 2)
                    merge(std::integral_constant<uint32_t, kXcdMaxRanges / 2>{});
                else
                    merge(std::integral_constant<uint32_t, kXcdMaxRanges>{});
                const float inv_l = 1.0f / L;
                if (live) {
                    att[h * a.sdpa.v_dim + 2 * d2] = (uint16_t)f32_to_bf16_bits(o0_ * inv_l);
                    att[h * a.sdpa.v_dim + 2 * d2 + 1] = (uint16_t)f32_to_bf16_bits(o1_ * inv_l);
                }
            }
        }
    }
    __syncthreads();
    FK_XCD_STAMP(0, 10);
    // ---- o_proj over this XCD's K-slice (its heads' columns): fp32 partial row ----
    {
        const uint32_t n8 = (G * a.sdpa.v_dim) >> 3, n8_up = (n8 + kWave - 1) / kWave * kWave;
        const uint4* a8 = reinterpret_cast<const uint4*>(att);
        for (uint32_t t = threadIdx.x; t < n8_up; t += kBlock) {
            const bool live = t < n8;
            const uint4 v = a8[live ? t : 0u];
            stage_emit<KIND>(xs, sx, a.o_cs, t, live, v, v, 1.0f, false);
        }
    }
    meta_store<KIND, kAttnStream, true, !ONE>(mmo, ti, meta + MW);
    __syncthreads();
    if (streams && o_n) tile_run<KIND, NLB, kAttnStream, ONE>(a.wo, to, po, ro, xs, sx, meta + MW, work, []() {});
    __syncthreads();
    FK_XCD_STAMP(0, 11);
    if (o_n && ok2) {
        long long* out = a.out_sums;
        XcdControl* ctl = sync.ctl;
        // (the one-round form was slower here: 835 against 837 tok/s; the o_proj slice has 16 chunks per row)
        tile_rows<false>(to, work, work, [&](uint32_t r, float s0, float) { xcd_sum_add(out, o0 + r, s0, ctl); });
    }
    FK_XCD_STAMP(0, 12);
}

template <WKind KIND, int NLA, int NLB, bool ONE>
__global__ __launch_bounds__(kBlock, 2) void xcd_attn_kernel(const long long* sums, const uint16_t* residual,
                                                             const uint16_t* norm_w, uint32_t hidden, const XcdAttnArgs a) {
    extern __shared__ uint4 lds_raw[];
    const XcdInputLead lead{sums, residual, norm_w, hidden};
    InputRegs inr;
    input_request<false>(lead, inr, nullptr);
    kernarg_warm<32 + (int)sizeof(XcdAttnArgs)>();
    XcdSync sync = xcd_sync_init(a.ctl, a.spin_limit);
    xcd_attn_phase<KIND, NLA, NLB, false, true, ONE>(a, lead, inr, sync, lds_raw, nullptr, nullptr);
    xcd_mark_placement(sync, a.mark_placement);
}

// ---- the whole token in one launch --------------------------------------------------------------------------
// Device-wide barrier in two levels: every block publishes its arrival word as in a hand-over; the leader block of
// each XCD (slot 0) waits for its 64 blocks, adds one to `arrivals` (a memory-side add) and waits until all eight
// leaders have (L1-bypassing loads see memory-side additions), then releases its XCD through `release[xcd]`, which
// the other 63 blocks poll.  Counters only grow; every wait is bounded.  Returns false after an abort.
struct XcdGlobalSync {
    uint32_t arrivals_base, release_base, k;
};
__device__ __forceinline__ XcdGlobalSync xcd_global_init(const XcdSync& s) {
    XcdGlobalSync g;
    // a fast leader may already have arrived at the first barrier: it completes only with all eight, so the count
    // read here lies within 7 of the last completed multiple of 8
    g.arrivals_base = __hip_atomic_load(&s.ctl->arrivals, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) & ~7u;
    g.release_base = __hip_atomic_load(&s.ctl->release[s.xcd], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    g.k = 0;
    return g;
}
__device__ __forceinline__ bool xcd_global_barrier(XcdSync& s, XcdGlobalSync& g) {
    s.epoch += 1;
    g.k += 1;
    wait_memory_ops_done();
    __syncthreads();
    if (threadIdx.x < (uint32_t)kWave) {
        const uint32_t lane = threadIdx.x;
        bool ok = true;
        if (s.slot == 0) {
            ok = xcd_publish_and_wait(s, lane);
            if (ok) {
                if (lane == 0) (void)__hip_atomic_fetch_add(&s.ctl->arrivals, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                const uint32_t target = g.arrivals_base + kXcds * g.k;
                uint32_t spins = 0;
                for (;;) {
                    const uint32_t v = __hip_atomic_load(&s.ctl->arrivals, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    if ((int32_t)(v - target) >= 0) break;
                    if (++spins > s.spin_limit || ((spins & 255u) == 0u &&
                                                   __hip_atomic_load(&s.ctl->abort_flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0u)) {
                        if (lane == 0) __hip_atomic_store(&s.ctl->abort_flag, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                        ok = false;
                        break;
                    }
                    __builtin_amdgcn_s_sleep(1);
                }
            }
            // released also after a failure, so that the XCD's blocks leave their wait at once and see the abort word
            if (lane == 0) __hip_atomic_store(&s.ctl->release[s.xcd], g.release_base + g.k, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
        } else {
            if (lane == 0) __hip_atomic_store(s.ctl->flags + s.xcd * kXcdSlots + s.slot, s.epoch, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
            const uint32_t target = g.release_base + g.k;
            uint32_t spins = 0;
            for (;;) {
                const uint32_t v = __hip_atomic_load(&s.ctl->release[s.xcd], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                if ((int32_t)(v - target) >= 0) break;
                if (++spins > s.spin_limit) {
                    if (lane == 0) __hip_atomic_store(&s.ctl->abort_flag, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    break;
                }
                __builtin_amdgcn_s_sleep(1);
            }
        }
    }
    __syncthreads();
    return __hip_atomic_load(&s.ctl->abort_flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == 0u;
}

template <WKind KIND, int NLQ, int NLO, int NLG, int NLD>
__global__ __launch_bounds__(kBlock, 2) void xcd_token_kernel(const XcdTokenArgs t) {
    extern __shared__ uint4 lds_raw[];
    uint4* xres = lds_raw + t.xres_off;
    XcdSync sync = xcd_sync_init(t.ctl, t.spin_limit);
    XcdGlobalSync gs = xcd_global_init(sync);
    // The argument blocks never change while the kernel runs: read through the constant address space, every field
    // is a scalar load, as for kernel arguments.
#if defined(__HIP_DEVICE_COMPILE__)
    typedef __attribute__((address_space(4))) XcdAttnArgs ConstAttn;
    typedef __attribute__((address_space(4))) XcdMlpArgs ConstMlp;
#else
    typedef XcdAttnArgs ConstAttn;
    typedef XcdMlpArgs ConstMlp;
#endif
    // The next phase's argument block is pulled into this XCD's L2 while the current phase runs (one request per
    // 64 bytes by a few lanes), so that its scalar loads do not start the phase with a trip to memory.
    auto touch = [&](const void* p, uint32_t bytes) {
        if (threadIdx.x * 64u < bytes) (void)*reinterpret_cast<const volatile uint32_t*>(reinterpret_cast<const char*>(p) + threadIdx.x * 64u);
    };
    for (uint32_t l = 0; l < t.n_layers; ++l) {
        touch(t.mlp + l, sizeof(XcdMlpArgs));
        {
            InputRegs inr;
            xcd_attn_phase<KIND, NLQ, NLO, true, false>(*(const ConstAttn*)(t.attn + l), ((const ConstAttn*)(t.attn + l))->in, inr, sync, lds_raw, l ? xres : nullptr, xres);
        }
        if (!xcd_global_barrier(sync, gs)) return;
        if (l + 1 < t.n_layers) touch(t.attn + l + 1, sizeof(XcdAttnArgs));
        {
            InputRegs inr;
            xcd_mlp_phase<KIND, NLG, NLD, true, false>(*(const ConstMlp*)(t.mlp + l), ((const ConstMlp*)(t.mlp + l))->in, inr, sync, lds_raw, xres, xres);
        }
        if (l + 1 < t.n_layers && !xcd_global_barrier(sync, gs)) return;
    }
    xcd_mark_placement(sync, t.mark_placement);
}

// ---- a whole layer in one launch ------------------------------------------------------------------------------
// Attention phase (the stand-alone launch's, input requested from the leading parameters), a device-wide barrier,
// MLP phase.  What crosses the barrier: the sum row the attention phase added into (memory-side additions, read with
// L1-bypassing loads), the residual row (every block holds its own copy in LDS) and the row the attention phase
// cleared for the MLP phase to add into (write-through stores).  Everything else is private to an XCD as in the
// separate launches.
template <WKind KIND, int NLQ, int NLO, int NLG, int NLD>
__global__ __launch_bounds__(kBlock, 2) void xcd_layer_kernel(const long long* sums, const uint16_t* residual,
                                                              const uint16_t* norm_w, uint32_t hidden, const XcdLayerArgs t) {
    extern __shared__ uint4 lds_raw[];
    const XcdInputLead lead{sums, residual, norm_w, hidden};
    InputRegs inr;
    input_request<false>(lead, inr, nullptr);
    kernarg_warm<768>();
    kernarg_warm<32 + (int)sizeof(XcdLayerArgs), 12>();
    uint4* xres = lds_raw + t.xres_off;
    XcdSync sync = xcd_sync_init(t.attn.ctl, t.attn.spin_limit);
    XcdGlobalSync gs = xcd_global_init(sync);
    xcd_attn_phase<KIND, NLQ, NLO, true, true, true>(t.attn, lead, inr, sync, lds_raw, nullptr, xres);
    if (!xcd_global_barrier(sync, gs)) return;
    {
        InputRegs inm;
        xcd_mlp_phase<KIND, NLG, NLD, true, false, true>(t.mlp, t.mlp.in, inm, sync, lds_raw, xres, nullptr);
    }
    xcd_mark_placement(sync, t.mark_placement);
}

__global__ __launch_bounds__(kBlock) void xcd_reduce_kernel(const XcdReduceArgs a) {
    const uint32_t i = blockIdx.x * kBlock + threadIdx.x;
    if (i >= a.hidden) return;
    const uint32_t at = xcd_sum_index(i);
    // every request first (a row that is not given repeats the first: no branch between the loads)
    const unsigned long long s = (unsigned long long)a.sums[at];
    const unsigned long long s2 = (unsigned long long)(a.sums2 ? a.sums2 : a.sums)[at];
    const uint16_t res = a.residual[i];
    float v = xcd_sum_to_f32((uint32_t)s, (uint32_t)(s >> 32));
    if (a.sums2) v = __fadd_rn(v, round_bf16(xcd_sum_to_f32((uint32_t)s2, (uint32_t)(s2 >> 32))));
    a.x[i] = (uint16_t)f32_to_bf16_bits(v + bf16_bits_to_f32(res));
    if (a.clear) a.clear[at] = 0;
    if (a.clear2) a.clear2[at] = 0;
    if (a.clear3) a.clear3[at] = 0;
}

// dst[(h * n + r) * gl + g] = src[r * groups + h * gl + g]: the scales (or biases) of a [n, groups] matrix, the
// K dimension cut into 8 slices of gl = groups / 8 groups, one contiguous copy per slice.
__global__ __launch_bounds__(kBlock) void xcd_kslice_meta_kernel(const uint16_t* src, uint16_t* dst, uint32_t n, uint32_t groups) {
    const uint32_t gl = groups / kXcds;
    const size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x;
    if (i >= (size_t)n * groups) return;
    const uint32_t g = (uint32_t)(i % gl), r = (uint32_t)((i / gl) % n), h = (uint32_t)(i / ((size_t)gl * n));
    dst[i] = src[(size_t)r * groups + h * gl + g];
}

// =============================================================================================== host side
fk_status xcd_kslice_meta(const uint16_t* src, uint32_t n, uint32_t groups, uint16_t* dst, hipStream_t stream) {
    const DeviceFacts* dev;
    FK_TRY(device_facts(&dev));
    if (!src || !dst || n == 0 || groups == 0 || groups % kXcds) return set_error(FK_ERR_INVALID, "xcd k-slice scales: null buffer, or groups per row not a multiple of 8");
    const size_t total = (size_t)n * groups;
    hipLaunchKernelGGL(xcd_kslice_meta_kernel, dim3((unsigned)((total + kBlock - 1) / kBlock)), dim3(kBlock), 0, stream, src, dst, n, groups);
    FK_HIP(hipGetLastError());
    return FK_OK;
}

namespace {

constexpr int kNlQkv = 5, kNlO = 3, kNlGu = 6, kNlDown = 6;  // 16-byte requests per streaming thread and pass
constexpr int kNlGuToken = 4;  // the whole-token launch holds both phases' registers: shallower gate / up passes
// Stand-alone attention launch with 8-bit weights: twice the chunks per tile, and passes deep enough that the
// 4B-class tiles are one pass there as well (18.5 -> 17.8 us).  The MLP launch keeps its depth: with 12 requests per
// matrix and thread in one go it was slower (24.0 -> 24.8 us) than two passes of 6.
struct PassDepth {
    int qkv, o, gu, down;
};
constexpr PassDepth depth_of(WKind k) {
    return k == W_Q8 ? PassDepth{9, 5, kNlGu, kNlDown} : PassDepth{kNlQkv, kNlO, kNlGu, kNlDown};
}
inline PassDepth depth_of_bits(uint32_t bits) { return depth_of(bits == 4 ? W_Q4 : (bits == 8 ? W_Q8 : W_BF16)); }



template <WKind KIND>
const void* mlp_func(bool one) {
    constexpr PassDepth d = depth_of(KIND);  // the deeper passes only where they make the launch one pass
    return one ? reinterpret_cast<const void*>(&xcd_mlp_kernel<KIND, d.gu, d.down, true>)
               : reinterpret_cast<const void*>(&xcd_mlp_kernel<KIND, kNlGu, kNlDown, false>);
}
template <WKind KIND>
const void* attn_func(bool one) {
    constexpr PassDepth d = depth_of(KIND);
    return one ? reinterpret_cast<const void*>(&xcd_attn_kernel<KIND, d.qkv, d.o, true>)
               : reinterpret_cast<const void*>(&xcd_attn_kernel<KIND, kNlQkv, kNlO, false>);
}

template <WKind KIND>
const void* layer_func() {
    constexpr PassDepth d = depth_of(KIND);
    return reinterpret_cast<const void*>(&xcd_layer_kernel<KIND, d.qkv, d.o, d.gu, d.down>);
}

uint32_t lds_for(uint32_t bits, const LdsPlan& p) {
    return bits == 4 ? xcd_lds_bytes<W_Q4>(p) : (bits == 8 ? xcd_lds_bytes<W_Q8>(p) : xcd_lds_bytes<W_BF16>(p));
}




// What a launch's shape decides: tiles, kernel flavour, LDS.
struct MlpGeometry {
    uint32_t gate_cpr, down_cpr, gu_rows, down_rows, down_cs;
    bool one;
    LdsPlan lp;
    uint32_t lds;
    const void* func;
};
MlpGeometry mlp_geometry(const XcdLayerShape& s, bool for_token) {
    MlpGeometry g;
    const uint32_t cv = chunk_values(s.bits);
    g.gate_cpr = s.hidden / cv;
    g.down_cpr = s.inter / cv;
    g.gu_rows = ceil_div(s.inter / kXcds, kXcdSlots);
    g.down_rows = ceil_div(s.hidden, kXcdSlots);
    g.down_cs = g.down_cpr / kXcds;
    auto padded = [](uint32_t chunks, int nl) { return ceil_div(chunks, nl * kBlock) * nl * kBlock; };
    g.lp.cs_max = g.gate_cpr > g.down_cs ? g.gate_cpr : g.down_cs;
    const PassDepth deep = depth_of_bits(s.bits);
    // every tile within one pass (the 4B-class shapes): the flavour compiled without the pass loop
    g.one = !for_token && g.gu_rows * g.gate_cpr <= (uint32_t)deep.gu * kBlock && g.down_rows * g.down_cs <= (uint32_t)deep.down * kBlock;
    const PassDepth depth = for_token ? PassDepth{kNlQkv, kNlO, kNlGuToken, kNlDown} : (g.one ? deep : PassDepth{kNlQkv, kNlO, kNlGu, kNlDown});
    const uint32_t gu = 2 * padded(g.gu_rows * g.gate_cpr, depth.gu), dn = padded(g.down_rows * g.down_cs, depth.down);
    g.lp.work_floats = gu > dn ? gu : dn;
    g.lp.att_elems = 0;
    g.lp.meta_words = g.one ? kMetaWords : kMetaWordsBig;
    g.lds = lds_for(s.bits, g.lp);
    g.func = s.bits == 4 ? mlp_func<W_Q4>(g.one) : (s.bits == 8 ? mlp_func<W_Q8>(g.one) : mlp_func<W_BF16>(g.one));
    return g;
}

struct AttnGeometry {
    uint32_t wq_cpr, wo_cpr, q_rows, kv_rows, R, q_tiles, kv_tiles, o_rows, o_cs;
    uint32_t chunk_len, chunks_per_block, n_splits;
    bool one;
    LdsPlan lp;
    uint32_t lds;
    const void* func;
};
AttnGeometry attn_geometry(const XcdLayerShape& s, bool for_token = false) {
    AttnGeometry g;
    const uint32_t cv = chunk_values(s.bits), G = s.n_heads / s.n_kv;
    g.wq_cpr = s.hidden / cv;
    g.wo_cpr = s.n_heads * s.head_dim / cv;
    g.q_rows = G * s.head_dim;
    g.kv_rows = s.head_dim;
    uint32_t R = 1;
    while (ceil_div(g.q_rows, R) + 2 * ceil_div(g.kv_rows, R) > kXcdSlots) ++R;
    g.R = R;
    g.q_tiles = ceil_div(g.q_rows, R);
    g.kv_tiles = ceil_div(g.kv_rows, R);
    g.o_rows = ceil_div(s.hidden, kXcdSlots);
    g.o_cs = g.wo_cpr / kXcds;
    // attention of one KV head per XCD: blocks = (query head of the group) x (key range)
    g.chunk_len = sdpa_chunk_len(s.head_dim, s.head_dim, false);
    uint32_t splits = kXcdSlots / G;
    if (splits > kXcdMaxRanges) splits = kXcdMaxRanges;
    const uint32_t n_chunks = ceil_div(s.capacity, g.chunk_len);
    g.chunks_per_block = ceil_div(n_chunks, splits);
    g.n_splits = ceil_div(n_chunks, g.chunks_per_block);
    auto padded = [](uint32_t chunks, int nl) { return ceil_div(chunks, nl * kAttnStream) * nl * kAttnStream; };
    g.lp.cs_max = g.wq_cpr > g.o_cs ? g.wq_cpr : g.o_cs;
    // partial rows padded to whole passes: of this launch's depths and of the whole-token launch's (it shares this plan)
    const PassDepth deep = depth_of_bits(s.bits);
    g.one = !for_token && R * g.wq_cpr <= (uint32_t)deep.qkv * kAttnStream && g.o_rows * g.o_cs <= (uint32_t)deep.o * kAttnStream;
    const PassDepth depth = g.one ? deep : PassDepth{kNlQkv, kNlO, kNlGu, kNlDown};
    auto larger = [](uint32_t x, uint32_t y) { return x > y ? x : y; };
    uint32_t wf = larger(padded(R * g.wq_cpr, depth.qkv), padded(R * g.wq_cpr, kNlQkv));
    const uint32_t wo_ = larger(padded(g.o_rows * g.o_cs, depth.o), padded(g.o_rows * g.o_cs, kNlO));
    wf = wf > wo_ ? wf : wo_;
    const uint32_t sf = sdpa_lds_floats(1, g.chunk_len, s.head_dim, s.head_dim, true);
    g.lp.work_floats = wf > sf ? wf : sf;
    g.lp.att_elems = G * s.head_dim;
    g.lp.meta_words = g.one ? kMetaWords : kMetaWordsBig;   // the whole-token launch runs the flavour with the pass loop
    g.lds = lds_for(s.bits, g.lp);
    g.func = s.bits == 4 ? attn_func<W_Q4>(g.one) : (s.bits == 8 ? attn_func<W_Q8>(g.one) : attn_func<W_BF16>(g.one));
    return g;
}

}  // namespace

// The shape rules and the LDS budget come first and need no device; the device's CU count and its occupancy answer for
// the two kernels come last.
fk_status xcd_layer_supported(const XcdLayerShape& s) {
    if (s.bits != 4 && s.bits != 8 && s.bits != 16) return set_error(FK_ERR_UNSUPPORTED, "xcd layer: bits must be 4, 8 or 16");
    const uint32_t cv = chunk_values(s.bits), unit = s.bits == 16 ? cv : (s.group > cv ? s.group : cv);
    if (s.bits != 16 && s.group != 32 && s.group != 64 && s.group != 128)
        return set_error(FK_ERR_UNSUPPORTED, "xcd layer: group size must be 32, 64 or 128");
    if (s.n_kv != kXcds) return set_error(FK_ERR_UNSUPPORTED, "xcd layer: needs exactly 8 KV heads (one per XCD)");
    if (s.n_heads % s.n_kv) return set_error(FK_ERR_INVALID, "xcd layer: n_heads must be a multiple of n_kv");
    const uint32_t G = s.n_heads / s.n_kv;
    if (G != 1 && G != 2 && G != 4 && G != 8) return set_error(FK_ERR_UNSUPPORTED, "xcd layer: 1, 2, 4 or 8 query heads per KV head");
    if (s.head_dim != 64 && s.head_dim != 128) return set_error(FK_ERR_UNSUPPORTED, "xcd layer: head_dim must be 64 or 128");
    if (s.hidden % 64 || s.hidden > (uint32_t)kInGroups * kBlock * 8) return set_error(FK_ERR_UNSUPPORTED, "xcd layer: hidden must be a multiple of 64, at most 4096");
    if (s.bits != 16 && (s.hidden / s.group) % 4) return set_error(FK_ERR_UNSUPPORTED, "xcd layer: hidden must hold a multiple of four quantisation groups");
    if ((G * s.head_dim) % unit) return set_error(FK_ERR_UNSUPPORTED, "xcd layer: a KV head's query columns must be whole quantisation groups");
    if (s.inter % (kXcds * unit) || s.inter % (kXcds * 8)) return set_error(FK_ERR_UNSUPPORTED, "xcd layer: intermediate / 8 must be whole quantisation groups");
    if (s.capacity == 0) return set_error(FK_ERR_INVALID, "xcd layer: zero cache capacity");
    const MlpGeometry mg = mlp_geometry(s, false);
    const AttnGeometry ag = attn_geometry(s);
    if (s.bits != 16) {
        // a tile's quantisation groups are fetched once per block: 768 per matrix in the one-pass flavour, 2048 in the
        // flavour with the pass loop
        const uint32_t n_q = s.n_heads * s.head_dim;
        const uint32_t budget_a = ag.lp.meta_words, budget_m = mg.lp.meta_words;
        uint32_t R = 1;
        while (ceil_div(G * s.head_dim, R) + 2 * ceil_div(s.head_dim, R) > kXcdSlots) ++R;
        if (R * (s.hidden / s.group) > budget_a || ceil_div(s.hidden, kXcdSlots) * (n_q / kXcds / s.group) > budget_a ||
            ceil_div(s.inter / kXcds, kXcdSlots) * (s.hidden / s.group) > budget_m ||
            ceil_div(s.hidden, kXcdSlots) * (s.inter / kXcds / s.group) > budget_m)
            return set_error(FK_ERR_UNSUPPORTED, "xcd layer: a block's tile holds more quantisation groups than the kernel fetches");
        // the groups of a block's o_proj / down_proj tile are fetched four per lane from the per-XCD copies
        const uint32_t rpb = ceil_div(s.hidden, kXcdSlots);
        if (s.hidden % kXcdSlots || (rpb * (n_q / kXcds / s.group)) % 4 || (rpb * (s.inter / kXcds / s.group)) % 4)
            return set_error(FK_ERR_UNSUPPORTED, "xcd layer: a block's o_proj / down_proj tile must hold a multiple of four quantisation groups");
    }
    if (2u * ((mg.lds + 1023u) & ~1023u) > kCuLdsBytes || 2u * ((ag.lds + 1023u) & ~1023u) > kCuLdsBytes)
        return set_error(FK_ERR_UNSUPPORTED, "xcd layer: two workgroups of a launch must fit the LDS of one CU (MLP launch " +
                                                 std::to_string(mg.lds) + " bytes, attention launch " + std::to_string(ag.lds) +
                                                 " bytes per workgroup): its 512 workgroups could not all be resident");
    const DeviceFacts* dev;
    FK_TRY(device_facts(&dev));
    if (dev->cus != (int)(kXcds * 32)) return set_error(FK_ERR_UNSUPPORTED, "xcd layer: needs 8 XCDs of 32 CUs");
    FK_TRY(require_two_blocks_per_cu(mg.func, mg.lds, "MLP"));
    FK_TRY(require_two_blocks_per_cu(ag.func, ag.lds, "attention"));
    return FK_OK;
}

size_t xcd_workspace_bytes() { return sizeof(XcdControl); }

fk_status xcd_check_control(void* workspace) {
    if (!workspace) return set_error(FK_ERR_INVALID, "xcd layer: null control block");
    static_assert(offsetof(XcdControl, abort_flag) == sizeof(uint32_t) * kXcds * kXcdSlots, "control block layout");
    // everything behind the arrival words in one copy
    constexpr size_t off = offsetof(XcdControl, abort_flag);
    alignas(8) unsigned char tail[sizeof(XcdControl) - off];
    FK_HIP(hipMemcpy(tail, reinterpret_cast<const char*>(workspace) + off, sizeof(tail), hipMemcpyDeviceToHost));
    auto word = [&](size_t o) {
        uint32_t v;
        memcpy(&v, tail + (o - off), 4);
        return v;
    };
    const char* what = nullptr;
    if (word(offsetof(XcdControl, abort_flag)))
        what = "a hand-over wait exceeded its spin limit";
    else if (word(offsetof(XcdControl, overflow)))
        what = "a contribution to a sum row was not finite or reached 2^27 in magnitude (the fixed-point range)";
    else
        for (uint32_t x = 0; x < kXcds; ++x) {
            unsigned long long bits;
            memcpy(&bits, tail + (offsetof(XcdControl, placement) + x * sizeof(XcdPlacement) - off), 8);
            if (bits != 0ull && bits != ~0ull) what = "two workgroups of a launch ran in the same (XCD, slot): the dispatch order is not the round-robin dealing the layer cut relies on";
        }
    if (!what) return FK_OK;
    // the arrival words of a failed launch are inconsistent: start over from zero
    FK_HIP(hipMemset(workspace, 0, sizeof(XcdControl)));
    return set_error(FK_ERR_HIP, std::string("xcd layer: ") + what +
                                     "; results are invalid (the control block was reset; zero the sum rows and decode the token again)");
}
size_t xcd_sum_row_bytes(uint32_t hidden) { return (size_t)xcd_sum_row_elems(hidden) * sizeof(long long); }

size_t xcd_attn_partials_bytes(const XcdLayerShape& s) {
    return (size_t)s.n_heads * kXcdMaxRanges * (s.head_dim + 2) * sizeof(float);
}

fk_status plan_xcd_mlp(const XcdMlpRequest& rq, Launch* out) {
    const XcdLayerShape& s = rq.shape;
    FK_TRY(xcd_layer_supported(s));
    if (!rq.mid || !rq.out_sums || !rq.workspace) return set_error(FK_ERR_INVALID, "xcd mlp: null mid, sum row or workspace");
    if (rq.swiglu_variant < 0 || rq.swiglu_variant > 2) return set_error(FK_ERR_INVALID, "xcd mlp: swiglu variant must be 0, 1 or 2");
    XcdMlpArgs a;
    memset(&a, 0, sizeof(a));
    FK_TRY(fill_input(s, rq.sums_in, rq.residual, rq.x_out, rq.clear, rq.out_sums, rq.norm_w, rq.eps, &a.in));
    FK_TRY(bind_mat(rq.wgate, s.inter, s.hidden, s, &a.gate, "gate_proj"));
    FK_TRY(bind_mat(rq.wup, s.inter, s.hidden, s, &a.up, "up_proj"));
    FK_TRY(bind_mat(rq.wdown, s.hidden, s.inter, s, &a.down, "down_proj"));
    const MlpGeometry g = mlp_geometry(s, rq.for_token);
    a.inter = s.inter;
    a.gu_rows = g.gu_rows;
    a.down_rows = g.down_rows;
    a.down_cs = g.down_cs;
    a.swiglu_variant = rq.swiglu_variant;
    a.mid = rq.mid;
    a.out_sums = rq.out_sums;
    a.ctl = reinterpret_cast<XcdControl*>(rq.workspace);
    a.spin_limit = rq.spin_limit ? rq.spin_limit : (1u << 20);
    a.mark_placement = rq.mark_placement ? 1u : 0u;
    const LdsPlan lp = g.lp;
    const uint32_t lds = g.lds;
    out->func = g.func;
    if (rq.for_token)
        FK_TRY(set_lds_limit(out->func, lds));  // an argument block for the whole-token launch, which is planned (and checked) as a whole
    else
        FK_TRY(require_two_blocks_per_cu(out->func, lds, "MLP"));
    out->grid = dim3(kXcdGrid, 1, 1);
    out->block = dim3(kMlpBlock, 1, 1);
    out->shmem = lds;
    a.cs_max = lp.cs_max;
    a.work_floats = lp.work_floats;
    out->set_args(a);
    out->n_lead = 0;
    out->add_lead(a.in.sums);
    out->add_lead(a.in.residual);
    out->add_lead(a.in.norm_w);
    out->add_lead(a.in.hidden);
    return FK_OK;
}

fk_status plan_xcd_attn(const XcdAttnRequest& rq, Launch* out) {
    const XcdLayerShape& s = rq.shape;
    FK_TRY(xcd_layer_supported(s));
    if (!rq.q || !rq.k || !rq.v || !rq.cache_k || !rq.cache_v || !rq.kv_len || !rq.rope_tab || !rq.att_partials ||
        !rq.out_sums || !rq.workspace)
        return set_error(FK_ERR_INVALID, "xcd attention: null buffer");
    if ((rq.q_norm == nullptr) != (rq.k_norm == nullptr)) return set_error(FK_ERR_INVALID, "xcd attention: q and k head norms come together");
    const uint32_t n_q = s.n_heads * s.head_dim, n_kvd = s.n_kv * s.head_dim;
    XcdAttnArgs a;
    memset(&a, 0, sizeof(a));
    FK_TRY(fill_input(s, rq.sums_in, rq.residual, rq.x_out, rq.clear, rq.out_sums, rq.norm_w, rq.eps, &a.in));
    FK_TRY(bind_mat(rq.wq, n_q, s.hidden, s, &a.wq, "q_proj"));
    FK_TRY(bind_mat(rq.wk, n_kvd, s.hidden, s, &a.wk, "k_proj"));
    FK_TRY(bind_mat(rq.wv, n_kvd, s.hidden, s, &a.wv, "v_proj"));
    FK_TRY(bind_mat(rq.wo, s.hidden, n_q, s, &a.wo, "o_proj"));
    const AttnGeometry g = attn_geometry(s, rq.for_token);
    a.q_rows = g.q_rows;
    a.kv_rows = g.kv_rows;
    a.qkv_tile_rows = g.R;
    a.q_tiles = g.q_tiles;
    a.kv_tiles = g.kv_tiles;
    a.o_rows = g.o_rows;
    a.o_cs = g.o_cs;
    a.q = rq.q;
    a.k = rq.k;
    a.v = rq.v;
    // attention of one KV head per XCD: blocks = (query head of the group) x (key range)
    SdpaArgs& sd = a.sdpa;
    sd.q = rq.q;
    sd.k = rq.cache_k;
    sd.v = rq.cache_v;
    sd.out = nullptr;
    sd.kv_len_ptr = rq.kv_len;
    sd.n_heads = s.n_heads;
    sd.n_kv = s.n_kv;
    sd.qk_dim = sd.v_dim = s.head_dim;
    sd.capacity = s.capacity;
    sd.chunk_len = g.chunk_len;
    sd.chunks_per_block = g.chunks_per_block;
    sd.n_splits = g.n_splits;
    sd.rows = 1;
    uint32_t lp_ = 1;
    while (lp_ < s.head_dim / 8) lp_ <<= 1;
    sd.lpk = sd.lpv = lp_;
    sd.scale = 1.0f / sqrtf((float)s.head_dim);
    sd.partials = rq.att_partials;
    sd.counters = nullptr;
    sd.k_new = rq.k;
    sd.v_new = rq.v;
    sd.q_norm = rq.q_norm;
    sd.k_norm = rq.k_norm;
    sd.cache_k_w = rq.cache_k;
    sd.cache_v_w = rq.cache_v;
    sd.rope_dims = s.head_dim;
    sd.eps = rq.eps;
    sd.base_log2 = (float)log2((double)rq.theta);
    sd.rope_tab = rq.rope_tab;
    sd.v_stride = s.head_dim;
    sd.k1_heads = 1;
    a.out_sums = rq.out_sums;
    a.ctl = reinterpret_cast<XcdControl*>(rq.workspace);
    a.spin_limit = rq.spin_limit ? rq.spin_limit : (1u << 20);
    a.mark_placement = rq.mark_placement ? 1u : 0u;
    const LdsPlan lp = g.lp;
    const uint32_t lds = g.lds;
    out->func = g.func;
    if (rq.for_token)
        FK_TRY(set_lds_limit(out->func, lds));  // an argument block for the whole-token launch, which is checked as a whole
    else
        FK_TRY(require_two_blocks_per_cu(out->func, lds, "attention"));
    out->grid = dim3(kXcdGrid, 1, 1);
    out->block = dim3(kBlock, 1, 1);
    out->shmem = lds;
    a.cs_max = lp.cs_max;
    a.work_floats = lp.work_floats;
    a.att_elems = lp.att_elems;
    out->set_args(a);
    out->n_lead = 0;
    out->add_lead(a.in.sums);
    out->add_lead(a.in.residual);
    out->add_lead(a.in.norm_w);
    out->add_lead(a.in.hidden);
    return FK_OK;
}

fk_status plan_xcd_layer(const Launch& la, const Launch& lm, Launch* out) {
    if (la.args_size != sizeof(XcdAttnArgs) || lm.args_size != sizeof(XcdMlpArgs))
        return set_error(FK_ERR_INVALID, "xcd layer launch: not an attention launch followed by an MLP launch");
    XcdLayerArgs t;
    memset(&t, 0, sizeof(t));
    memcpy(&t.attn, la.args, sizeof(XcdAttnArgs));
    memcpy(&t.mlp, lm.args, sizeof(XcdMlpArgs));
    const void* func = nullptr;
    if (la.func == attn_func<W_Q4>(true) && lm.func == mlp_func<W_Q4>(true)) func = layer_func<W_Q4>();
    if (la.func == attn_func<W_Q8>(true) && lm.func == mlp_func<W_Q8>(true)) func = layer_func<W_Q8>();
    if (la.func == attn_func<W_BF16>(true) && lm.func == mlp_func<W_BF16>(true)) func = layer_func<W_BF16>();
    if (!func) return set_error(FK_ERR_UNSUPPORTED, "xcd layer launch: both launches must take their one-pass flavour, same weight kind");
    if (t.attn.ctl != t.mlp.ctl) return set_error(FK_ERR_INVALID, "xcd layer launch: the two launches use different control blocks");
    if (!t.mlp.in.sums || t.mlp.in.sums != t.attn.out_sums || t.mlp.in.residual != t.attn.in.x_out ||
        t.mlp.in.hidden != t.attn.in.hidden)
        return set_error(FK_ERR_INVALID, "xcd layer launch: the MLP launch must read the sum row the attention launch adds into and the row it writes");
    if (t.attn.in.clear != t.mlp.out_sums)
        return set_error(FK_ERR_INVALID, "xcd layer launch: the attention launch must clear the row the MLP launch adds into");
    const uint32_t phase_lds = ((la.shmem > lm.shmem ? la.shmem : lm.shmem) + 15u) & ~15u;
    t.xres_off = phase_lds / 16u;
    t.mark_placement = (t.attn.mark_placement | t.mlp.mark_placement) ? 1u : 0u;
    const uint32_t lds = phase_lds + t.attn.in.hidden * 2u;
    out->func = func;
    FK_TRY(require_two_blocks_per_cu(out->func, lds, "whole-layer"));
    out->grid = dim3(kXcdGrid, 1, 1);
    out->block = dim3(kBlock, 1, 1);
    out->shmem = lds;
    out->set_args(t);
    out->n_lead = 0;
    out->add_lead(t.attn.in.sums);
    out->add_lead(t.attn.in.residual);
    out->add_lead(t.attn.in.norm_w);
    out->add_lead(t.attn.in.hidden);
    return FK_OK;
}

fk_status plan_xcd_token(const XcdAttnArgs* h_attn, const XcdMlpArgs* h_mlp, uint32_t n_layers, uint32_t bits,
                         const XcdAttnArgs* d_attn, const XcdMlpArgs* d_mlp, uint32_t attn_lds, uint32_t mlp_lds, Launch* out) {
    if (!h_attn || !h_mlp || !d_attn || !d_mlp || n_layers == 0) return set_error(FK_ERR_INVALID, "xcd token: empty layer list");
    for (uint32_t l = 0; l < n_layers; ++l) {
        if (h_attn[l].ctl != h_attn[0].ctl || h_mlp[l].ctl != h_attn[0].ctl)
            return set_error(FK_ERR_INVALID, "xcd token: every launch of the run must use the same control block");
        if (h_attn[l].in.hidden != h_attn[0].in.hidden || h_mlp[l].in.hidden != h_attn[0].in.hidden)
            return set_error(FK_ERR_INVALID, "xcd token: layers of different width");
        for (uint32_t m = 0; m < l; ++m)
            if (h_attn[l].q == h_attn[m].q || h_attn[l].k == h_attn[m].k || h_attn[l].v == h_attn[m].v)
                return set_error(FK_ERR_UNSUPPORTED, "xcd token: every layer needs its own q / k / v rows inside one launch");
    }
    XcdTokenArgs t;
    memset(&t, 0, sizeof(t));
    t.attn = d_attn;
    t.mlp = d_mlp;
    t.n_layers = n_layers;
    t.ctl = h_attn[0].ctl;
    t.spin_limit = h_attn[0].spin_limit;
    t.mark_placement = h_attn[0].mark_placement;
    const uint32_t phase_lds = ((attn_lds > mlp_lds ? attn_lds : mlp_lds) + 15u) & ~15u;
    t.xres_off = phase_lds / 16u;
    const uint32_t lds = phase_lds + h_attn[0].in.hidden * 2u;
    auto func = [&]() -> const void* {
        if (bits == 4) return reinterpret_cast<const void*>(&xcd_token_kernel<W_Q4, kNlQkv, kNlO, kNlGuToken, kNlDown>);
        if (bits == 8) return reinterpret_cast<const void*>(&xcd_token_kernel<W_Q8, kNlQkv, kNlO, kNlGuToken, kNlDown>);
        return reinterpret_cast<const void*>(&xcd_token_kernel<W_BF16, kNlQkv, kNlO, kNlGuToken, kNlDown>);
    };
    out->func = func();
    FK_TRY(require_two_blocks_per_cu(out->func, lds, "whole-token"));
    out->grid = dim3(kXcdGrid, 1, 1);
    out->block = dim3(kBlock, 1, 1);
    out->shmem = lds;
    out->set_args(t);
    return FK_OK;
}

fk_status plan_xcd_reduce(const long long* sums, const uint16_t* residual, uint16_t* x, long long* clear, uint32_t hidden,
                          Launch* out, const long long* sums2, long long* clear2, long long* clear3) {
    const DeviceFacts* dev;
    FK_TRY(device_facts(&dev));
    if (!sums || !residual || !x || hidden == 0) return set_error(FK_ERR_INVALID, "xcd reduce: null buffer or zero width");
    XcdReduceArgs a{sums, residual, x, clear, hidden, sums2, clear2, clear3};
    out->func = reinterpret_cast<const void*>(&xcd_reduce_kernel);
    out->grid = dim3(ceil_div(hidden, kBlock), 1, 1);
    out->block = dim3(kBlock, 1, 1);
    out->shmem = 0;
    out->set_args(a);
    return FK_OK;
}

}  // namespace fk
