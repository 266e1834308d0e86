// The attention half of a layer with low-rank keys (the mixture-of-experts benchmark architecture) as ONE XCD-resident
// launch (see XcdMlaArgs in xcd_layer.hpp for the cut): input row, RMSNorm, q and kv_a projections, latent norm + kv_b,
// rotation + cache append + attention, merge, o_proj into a sum row.  Reference semantics: rmsnorm_qkv.rs (both
// projection launches), rope_kv_cache_store_decode.rs / rope_q_decode.rs in their split-key form, sdpa_decode.rs,
// linear_residual.rs.
#include "xcd_layer.hpp"

// Timing probes (empty in the library build): boundary i of every block, by its first thread.
#include "fk_probe.hpp"
FK_PROBE_DEFINE(xcd_mla, 512, 16)
#define FK_XCD_STAMP(k, i) FK_PROBE_STAMP(xcd_mla, 512, 16, blockIdx.x, threadIdx.x == 0, i)

#include "xcd_device.hpp"

namespace fk {

constexpr int kMlaNlA = 5;   // 16-byte requests per thread: a q / kv_a tile holds at most 5 * 256 chunks
constexpr int kMlaNlB = 2;   // ... a kv_b tile
constexpr int kMlaNlO = 3;   // ... an o_proj tile

namespace {

// The second sum row of the input (the shared expert's dot products of the previous layer's expert launch): requested
// like the first.
struct InputRegs2 {
    uint4 sv[kInGroups][4];
};
__device__ __forceinline__ void mla_input_request2(const long long* sums2, uint32_t hidden, InputRegs2& r) {
    const uint32_t n8 = hidden >> 3, lane = threadIdx.x & (kWave - 1);
    const uint4* s16 = reinterpret_cast<const uint4*>(sums2);
#pragma unroll
    for (int i = 0; i < kInGroups; ++i) {
        const uint32_t t = threadIdx.x + i * kBlock, sec = t >> 6;
        if (sec * kWave < n8 && sums2) {
#pragma unroll
            for (int k = 0; k < 4; ++k) r.sv[i][k] = ld_u128<false>(s16 + (sec * 4 + k) * kWave + lane);
        }
    }
}
__device__ __forceinline__ void mla_input_pin2(const long long* sums2, uint32_t hidden, InputRegs2& r) {
    const uint32_t n8 = hidden >> 3;
#pragma unroll
    for (int i = 0; i < kInGroups; ++i) {
        const uint32_t t = threadIdx.x + i * kBlock, sec = t >> 6;
        if (sec * kWave < n8 && sums2) {
#pragma unroll
            for (int k = 0; k < 4; ++k) pin128(r.sv[i][k]);
        }
    }
}

// input_stage of the dense launches with the second row: x = T((f32(sums) + T(f32(sums2))) + residual) -- the order in
// which the reference's reduction adds the routes, the shared expert and the residual.
template <WKind KIND>
__device__ __forceinline__ void mla_input_stage(const XcdInput& in, const long long* sums2, const InputRegs& r, const InputRegs2& r2,
                                                uint4* xs, float* sx, uint32_t cs, float* red) {
    const uint32_t n8 = in.hidden >> 3;
    uint4 xv[kInGroups];
    float sq = 0.f;
#pragma unroll
    for (int i = 0; i < kInGroups; ++i) {
        const uint32_t t = threadIdx.x + i * kBlock, sec = t >> 6;
        if (sec * kWave < n8) {
            uint32_t xb[4] = {r.rv[i].x, r.rv[i].y, r.rv[i].z, r.rv[i].w};
            if (in.sums) {
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    float lo = xcd_sum_to_f32(r.sv[i][k].x, r.sv[i][k].y), hi = xcd_sum_to_f32(r.sv[i][k].z, r.sv[i][k].w);
                    if (sums2) {
                        lo = __fadd_rn(lo, round_bf16(xcd_sum_to_f32(r2.sv[i][k].x, r2.sv[i][k].y)));
                        hi = __fadd_rn(hi, round_bf16(xcd_sum_to_f32(r2.sv[i][k].z, r2.sv[i][k].w)));
                    }
                    xb[k] = pack_bf16(lo + bf16_lo(xb[k]), hi + bf16_hi(xb[k]));
                }
            }
            xv[i] = make_uint4(xb[0], xb[1], xb[2], xb[3]);
            if (t < n8) {
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    const float lo = bf16_lo(xb[k]), hi = bf16_hi(xb[k]);
                    sq = fmaf(lo, lo, sq);
                    sq = fmaf(hi, hi, sq);
                }
                if (blockIdx.x == 0) reinterpret_cast<uint4*>(in.x_out)[t] = xv[i];
            }
        }
    }
    sq = wave_sum(sq);
    if ((threadIdx.x & (kWave - 1)) == 0) red[threadIdx.x / kWave] = sq;
    __syncthreads();
    sq = (red[0] + red[1]) + (red[2] + red[3]);
    const float rr = 1.0f / sqrtf(sq / (float)in.hidden + in.eps);
#pragma unroll
    for (int i = 0; i < kInGroups; ++i) {
        const uint32_t t = threadIdx.x + i * kBlock, sec = t >> 6;
        if (sec * kWave < n8) stage_emit<KIND>(xs, sx, cs, t, t < n8, xv[i], r.nw[i], rr, true);
    }
    __syncthreads();
}

// Zeroes a second sum row (16-byte units spread over the grid), as input_clear does the first.
__device__ __forceinline__ void mla_clear2(long long* row, uint32_t row_elems) {
    if (!row) return;
    const uint32_t u = blockIdx.x * kBlock + threadIdx.x;
    if (u < row_elems / 2) reinterpret_cast<uint4*>(row)[u] = make_uint4(0, 0, 0, 0);
}

}  // namespace

template <WKind KIND>
__global__ __launch_bounds__(kBlock, 2) void xcd_mla_kernel(const long long* sums, const uint16_t* residual, const uint16_t* norm_w,
                                                            uint32_t hidden, const XcdMlaArgs a) {
    extern __shared__ uint4 lds_raw[];
    constexpr int NLA = kMlaNlA, NLB = kMlaNlB, NLO = kMlaNlO;
    const XcdInputLead lead{sums, residual, norm_w, hidden};
    InputRegs inr;
    InputRegs2 inr2;
    input_request<false>(lead, inr, nullptr);
    kernarg_warm<32 + (int)sizeof(XcdMlaArgs)>();
    const long long* sums2 = sums ? a.sums2 : nullptr;
    mla_input_request2(sums2, hidden, inr2);
    XcdSync sync = xcd_sync_init(a.ctl, a.spin_limit);
    uint32_t kv_len_raw = *a.sdpa.kv_len_ptr;   // looked at behind the start-up requests
    FK_XCD_STAMP(0, 0);

    const uint32_t cs_max = a.cs_max, work_floats = a.work_floats, att_elems = a.att_elems;
    constexpr int PIECES = ChunkTraits<KIND>::kPieces;
    uint4* xs = lds_raw;
    float* sx = reinterpret_cast<float*>(xs + PIECES * cs_max);
    float* work = sx + cs_max;
    constexpr uint32_t MW = kMetaWords;
    uint32_t* meta = reinterpret_cast<uint32_t*>(work + work_floats);  // [3][MW]
    uint16_t* att = reinterpret_cast<uint16_t*>(meta + 3 * MW);
    float* red = reinterpret_cast<float*>(att + ((att_elems + 7u) & ~7u));  // [16]
    const uint32_t tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
    const uint32_t xcd = sync.xcd, slot = sync.slot;

    // ---- this block's tiles ----
    // q / kv_a: the XCD's q rows (its heads') first, then ALL kv_a rows (every XCD forms the whole latent row itself:
    // no hand-over between XCDs)
    const uint32_t R = a.tile_rows;
    const bool has_tile = slot < a.q_tiles + a.a_tiles, is_q = slot < a.q_tiles;
    const uint32_t tl = is_q ? slot : slot - a.q_tiles;
    const uint32_t part_rows = is_q ? a.q_rows : a.a_rows;
    const uint32_t pr0 = tl * R;
    const uint32_t pr_n = has_tile ? ((part_rows - pr0) < R ? (part_rows - pr0) : R) : 0u;
    const XcdMat A = pick_mat(is_q, a.wq, a.wa);
    const Tile ta = make_tile((is_q ? xcd * a.q_rows : 0u) + pr0, pr_n, 0, A.cpr);
    // kv_b: the XCD's heads' rows ([k_nope | v] per head), all of the latent width
    // (the last 2 hl blocks of the XCD take no kv_b rows: they rotate q_pe / k_pe of its heads meanwhile)
    const uint32_t n_rot = 2u * a.hl;
    const bool is_rot = slot >= kXcdSlots - n_rot;
    const uint32_t b0 = slot * a.b_rows;
    const uint32_t b_n = (!is_rot && b0 < a.b_total) ? ((a.b_total - b0) < a.b_rows ? (a.b_total - b0) : a.b_rows) : 0u;
    const Tile tb = make_tile(xcd * a.b_total + b0, b_n, 0, a.wb.cpr);
    // o_proj: this block's output rows x the K-slice of the XCD's heads
    const uint32_t o0 = slot * a.o_rows;
    const uint32_t o_n = o0 < hidden ? ((hidden - o0) < a.o_rows ? (hidden - o0) : a.o_rows) : 0u;
    const Tile to = make_tile(o0, o_n, xcd * a.o_cs, a.o_cs);

    TileRegs<NLA> ra;
    TileRegs<NLB> rb;
    TileRegs<NLO> ro;
    MetaRegs ma, mb, mo;
    TilePos<NLA> pa;
    TilePos<NLB> pb;
    TilePos<NLO> po;
    tile_pos_init<NLA, kBlock>(A, ta, tid, pa);
    tile_pos_init<NLB, kBlock>(a.wb, tb, tid, pb);
    tile_pos_init<NLO, kBlock>(a.wo, to, tid, po);
    meta_fetch<KIND, kBlock, true>(A, ta, tid, ma);
    tile_load<KIND, NLA, kBlock>(A, ta, pa, ra);
    FK_XCD_STAMP(0, 1);
    asm volatile("" : "+v"(kv_len_raw));
    const uint32_t kv_len0 = __builtin_amdgcn_readfirstlane(kv_len_raw);
    input_pin(lead, inr);
    mla_input_pin2(sums2, hidden, inr2);
    mla_input_stage<KIND>(a.in, sums2, inr, inr2, xs, sx, A.cpr, red);
    FK_XCD_STAMP(0, 2);
    input_clear<false>(a.in);
    mla_clear2(a.clear2, a.in.row_elems);
    // the later projections' rows: requested now, used behind the hand-overs
    meta_fetch<KIND, kBlock, true>(a.wb, tb, tid, mb);
    tile_load<KIND, NLB, kBlock>(a.wb, tb, pb, rb);
    meta_fetch<KIND, kBlock, true>(a.wo, to, tid, mo, xcd);
    tile_load<KIND, NLO, kBlock>(a.wo, to, po, ro);
    meta_store<KIND, kBlock, true>(ma, tid, meta);
    __syncthreads();

    // ---- q rows of the XCD's heads, the latent row ----
    tile_partials<KIND, NLA, kBlock>(A, ta, pa, ra, xs, sx, meta, work);
    __syncthreads();
    if (pr_n) {
        uint16_t* dst = is_q ? a.q + (size_t)xcd * a.q_rows + pr0 : a.kva + (size_t)xcd * a.a_rows + pr0;
        tile_rows<false, true>(ta, work, work, [&](uint32_t r, float s0, float) { dst[r] = (uint16_t)f32_to_bf16_bits(s0); });
    }
    FK_XCD_STAMP(0, 3);
    meta_store<KIND, kBlock, true>(mb, tid, meta + MW);
    meta_store<KIND, kBlock, true>(mo, tid, meta + 2 * MW);
    uint32_t* okw = reinterpret_cast<uint32_t*>(red) + 8;
    xcd_barrier<0>(sync, okw);
    if (!xcd_wait_ok(okw)) return;
    FK_XCD_STAMP(0, 4);

    // position of the new token, as the attention blocks settle it
    const uint32_t span = a.sdpa.chunk_len * a.sdpa.chunks_per_block;
    const uint32_t covered = a.sdpa.n_splits * span < a.sdpa.capacity ? a.sdpa.n_splits * span : a.sdpa.capacity;
    const uint32_t kv_len = kv_len0 < 1u ? 1u : (kv_len0 > covered ? covered : kv_len0);
    const uint32_t pos = kv_len - 1, cache_row = pos % a.sdpa.capacity;
    if (is_rot) {
        // ---- rotations, one wave each: unit 2 h -> the head's q with its second part rotated, into the second half of
        // `q`; unit 2 h + 1 -> the rotated k_pe into the head's new cache row.  They run beside the other blocks' kv_b
        // rows and meet them at the hand-over. ----
        if (wave == 0) {
            const uint32_t unit = kXcdSlots - 1 - slot, head = xcd * a.hl + (unit >> 1);
            const uint32_t d0 = a.sdpa.q0_dim, d1 = a.sdpa.qk_dim - d0;
            if ((unit & 1u) == 0) {
                const uint16_t* qh = a.q + (size_t)head * a.sdpa.qk_dim;
                uint16_t* qr = a.q + (size_t)a.sdpa.n_heads * a.sdpa.qk_dim + (size_t)head * a.sdpa.qk_dim;
                split_head_transform(qh, qh + d0, qr, d0, d1, a.sdpa.rope_dims, a.sdpa.traditional != 0, pos, a.sdpa.base_log2, lane,
                                     a.sdpa.rope_tab);
            } else {
                const uint16_t* kpe = a.kva + (size_t)xcd * a.a_rows + a.rank;
                uint16_t* krow = a.sdpa.cache_k_w + ((size_t)head * a.sdpa.capacity + cache_row) * a.sdpa.qk_dim + d0;
                split_head_transform(kpe, kpe, krow, 0u, d1, a.sdpa.rope_dims, a.sdpa.traditional != 0, pos, a.sdpa.base_log2, lane,
                                     a.sdpa.rope_tab);
            }
        }
    } else {
        // ---- latent RMSNorm, kv_b rows of the XCD's heads ----
        {
            const uint32_t n8 = a.rank >> 3;   // at most 256 groups: one per thread
            const uint4* l8 = reinterpret_cast<const uint4*>(a.kva + (size_t)xcd * a.a_rows);
            const uint4* w8 = reinterpret_cast<const uint4*>(a.a_norm);
            const bool live = tid < n8;
            const bool wave_live = (tid & ~(kWave - 1u)) < n8;   // wave-uniform
            uint4 v = make_uint4(0, 0, 0, 0), wv = v;
            if (wave_live) {
                v = ld_u128<true>(l8 + (live ? tid : 0u));
                wv = w8[live ? tid : 0u];
            }
            float sq = 0.f;
            if (live) {
                const uint32_t xb[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    const float lo = bf16_lo(xb[k]), hi = bf16_hi(xb[k]);
                    sq = fmaf(lo, lo, sq);
                    sq = fmaf(hi, hi, sq);
                }
            }
            sq = wave_sum(sq);
            if (lane == 0) red[wave] = sq;
            __syncthreads();
            sq = (red[0] + red[1]) + (red[2] + red[3]);
            const float rr = 1.0f / sqrtf(sq / (float)a.rank + a.in.eps);
            if (wave_live) stage_emit<KIND>(xs, sx, a.wb.cpr, tid, live, v, wv, rr, true);
            __syncthreads();
        }
        tile_partials<KIND, NLB, kBlock>(a.wb, tb, pb, rb, xs, sx, meta + MW, work);
        __syncthreads();
        if (b_n) {   // [k_nope | v] of a head: into `kvb` and straight into the head's new cache rows
            uint16_t* dst = a.kvb + (size_t)xcd * a.b_total + b0;
            const uint32_t d0 = a.sdpa.q0_dim, packed = d0 + a.sdpa.v_dim, qkd = a.sdpa.qk_dim, vd = a.sdpa.v_dim, cap = a.sdpa.capacity;
            uint16_t* ck = a.sdpa.cache_k_w;
            uint16_t* cv = a.sdpa.cache_v_w;
            const uint32_t head0 = xcd * a.hl;
            tile_rows<false, true>(tb, work, work, [&](uint32_t r, float s0, float) {
                const uint16_t v16 = (uint16_t)f32_to_bf16_bits(s0);
                dst[r] = v16;
                const uint32_t rr_ = b0 + r, hl_ = rr_ / packed, w = rr_ - hl_ * packed;
                const size_t crow = (size_t)(head0 + hl_) * cap + cache_row;
                if (w < d0)
                    ck[crow * qkd + w] = v16;
                else
                    cv[crow * vd + (w - d0)] = v16;
            });
        }
    }
    FK_XCD_STAMP(0, 5);
    xcd_barrier<0>(sync, okw);
    if (!xcd_wait_ok(okw)) return;  // the attention phase appends to the cache
    FK_XCD_STAMP(0, 6);

    // ---- rotation + cache append + attention: block = (head of the XCD, key range) ----
    {
        const uint32_t head = slot % a.hl, split = slot / a.hl;
        if (split < a.sdpa.n_splits) {   // q rotated and the new rows cached by the phase before: plain attention
            SdpaArgs sd = a.sdpa;
            sd.q += (size_t)a.sdpa.n_heads * a.sdpa.qk_dim;   // the rotated copy
            sdpa_block<1, 0, SdpaArgs, 0, false, true>(sd, kv_len0, split, xcd * a.hl + head, 0u, 1u, work);
        }
    }
    FK_XCD_STAMP(0, 7);
    xcd_barrier<0>(sync, okw);
    const bool ok = xcd_wait_ok(okw);  // tested in front of the additions into the sum row
    FK_XCD_STAMP(0, 8);

    // ---- merge the ranges of each of the XCD's heads (range order), rows to LDS ----
    {
        const uint32_t n_active = (kv_len + span - 1) / span;
        const uint32_t row = a.sdpa.v_dim + 2;
        for (uint32_t h = wave; h < a.hl; h += kBlock / kWave) {
            const float* ph = a.sdpa.partials + (size_t)(xcd * a.hl + h) * a.sdpa.n_splits * row;
            for (uint32_t d2 = lane; d2 < ((a.sdpa.v_dim >> 1) + kWave - 1) / kWave * kWave; d2 += kWave) {
                const bool live = d2 < (a.sdpa.v_dim >> 1);
                const float* pd = ph + 2 + 2 * (live ? d2 : 0u);
                float M = -INFINITY, L = 0.f, o0_ = 0.f, o1_ = 0.f;
                // all requests first (clamped indices: straight-line), then the fold in range order; the (maximum, sum)
                // pair of range i is fetched by lane i alone and handed to the wave through scalar registers
                auto merge = [&](auto n_const) {
                    constexpr uint32_t N = decltype(n_const)::value;
                    float2 pp[N];
                    const float2 mine = ld_f32x2<true>(ph + (size_t)(lane < n_active ? lane : 0u) * row);
#pragma unroll
                    for (uint32_t i = 0; i < N; ++i) pp[i] = ld_f32x2<true>(pd + (size_t)(i < n_active ? i : 0u) * row);
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
                        o0_ = fmaf(pp[i].x, w, o0_);
                        o1_ = fmaf(pp[i].y, w, o1_);
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
    FK_XCD_STAMP(0, 9);
    // ---- o_proj over this XCD's K-slice (its heads' columns): fp32 partial row ----
    {
        const uint32_t n8 = (a.hl * a.sdpa.v_dim) >> 3, n8_up = (n8 + kWave - 1) / kWave * kWave;
        const uint4* a8 = reinterpret_cast<const uint4*>(att);
        for (uint32_t t = tid; t < n8_up; t += kBlock) {
            const bool live = t < n8;
            const uint4 v = a8[live ? t : 0u];
            stage_emit<KIND>(xs, sx, a.o_cs, t, live, v, v, 1.0f, false);
        }
    }
    __syncthreads();
    tile_partials<KIND, NLO, kBlock>(a.wo, to, po, ro, xs, sx, meta + 2 * MW, work);
    __syncthreads();
    FK_XCD_STAMP(0, 10);
    if (o_n && ok) {
        long long* out = a.out_sums;
        XcdControl* ctl = sync.ctl;
        tile_rows<false, true>(to, work, work, [&](uint32_t r, float s0, float) { xcd_sum_add(out, o0 + r, s0, ctl); });
    }
    FK_XCD_STAMP(0, 11);
    xcd_mark_placement(sync, a.mark_placement);
}

// ================================================================================================ host
namespace {

struct MlaGeometry {
    uint32_t hl, qk_dim, q_rows, a_rows, b_total, R, q_tiles, a_tiles, b_rows, o_rows, o_cs;
    uint32_t chunk_len, chunks_per_block, n_splits, lp;
    LdsPlan lp_;
    uint32_t lds;
};
MlaGeometry mla_geometry(const XcdMlaShape& s) {
    MlaGeometry g;
    const uint32_t cv = chunk_values(s.bits);
    g.hl = s.n_heads / kXcds;
    g.qk_dim = s.nope_dim + s.rope_dim;
    g.q_rows = g.hl * g.qk_dim;
    g.a_rows = s.rank + s.rope_dim;
    g.b_total = g.hl * (s.nope_dim + s.v_dim);
    uint32_t R = 1;
    while (ceil_div(g.q_rows, R) + ceil_div(g.a_rows, R) > kXcdSlots) ++R;
    g.R = R;
    g.q_tiles = ceil_div(g.q_rows, R);
    g.a_tiles = ceil_div(g.a_rows, R);
    // the last 2 hl blocks of an XCD rotate instead; a tile's quantisation groups are fetched four per lane, so its rows
    // are rounded up to a whole number of such runs
    g.b_rows = ceil_div(g.b_total, kXcdSlots - 2u * g.hl);
    {
        const uint32_t gb = s.group ? s.rank / s.group : 1u;
        const uint32_t unit = (gb % 4u == 0) ? 1u : ((gb % 2u == 0) ? 2u : 4u);
        g.b_rows = ceil_div(g.b_rows, unit) * unit;
    }
    g.o_rows = ceil_div(s.hidden, kXcdSlots);
    g.o_cs = s.n_heads * s.v_dim / cv / kXcds;
    g.chunk_len = sdpa_chunk_len(g.qk_dim, s.v_dim, false);
    uint32_t splits = kXcdSlots / (g.hl ? g.hl : 1u);
    if (splits > kXcdMaxRanges) splits = kXcdMaxRanges;
    const uint32_t n_chunks = ceil_div(s.capacity, g.chunk_len);
    g.chunks_per_block = ceil_div(n_chunks, splits);
    g.n_splits = ceil_div(n_chunks, g.chunks_per_block);
    uint32_t lpk = 1, lpv = 1;
    while (lpk < g.qk_dim / 8) lpk <<= 1;
    while (lpv < s.v_dim / 8) lpv <<= 1;
    g.lp = lpk > lpv ? lpk : lpv;
    const uint32_t wq_cpr = s.hidden / cv, wb_cpr = s.rank / cv;
    g.lp_.cs_max = wq_cpr > wb_cpr ? wq_cpr : wb_cpr;
    if (g.o_cs > g.lp_.cs_max) g.lp_.cs_max = g.o_cs;
    uint32_t wf = (uint32_t)kMlaNlA * kBlock;
    const uint32_t sf = sdpa_lds_floats(1, g.chunk_len, g.qk_dim, s.v_dim, true);
    g.lp_.work_floats = wf > sf ? wf : sf;
    g.lp_.att_elems = g.hl * s.v_dim;
    g.lp_.meta_words = kMetaWords;
    g.lds = xcd_lds_bytes<W_Q4>(g.lp_);
    return g;
}

}  // namespace

fk_status xcd_mla_supported(const XcdMlaShape& s) {
    if (s.bits != 4) return set_error(FK_ERR_UNSUPPORTED, "xcd mla: 4-bit weights only");
    if (s.group != 32 && s.group != 64 && s.group != 128) return set_error(FK_ERR_UNSUPPORTED, "xcd mla: group size must be 32, 64 or 128");
    if (s.hidden == 0 || s.n_heads == 0 || s.rank == 0 || s.rope_dim == 0 || s.nope_dim == 0 || s.v_dim == 0 || s.capacity == 0)
        return set_error(FK_ERR_INVALID, "xcd mla: shape parameters missing");
    if (s.n_heads % kXcds || s.n_heads / kXcds > 4) return set_error(FK_ERR_UNSUPPORTED, "xcd mla: 8, 16, 24 or 32 heads (1 to 4 per XCD)");
    if (s.hidden % 256 || s.hidden > (uint32_t)kInGroups * kBlock * 8) return set_error(FK_ERR_UNSUPPORTED, "xcd mla: hidden must be a multiple of 256, at most 4096");
    if (s.rank % 128 || s.rank > 2048) return set_error(FK_ERR_UNSUPPORTED, "xcd mla: the latent width must be a multiple of 128, at most 2048");
    if (s.rope_dim % 8 || s.nope_dim % 8 || s.v_dim % 8 || s.rope_dim % 2)
        return set_error(FK_ERR_UNSUPPORTED, "xcd mla: head parts must be multiples of 8");
    const MlaGeometry g = mla_geometry(s);
    const uint32_t cv = chunk_values(s.bits), unit = s.group > cv ? s.group : cv;
    if ((g.hl * s.v_dim) % unit) return set_error(FK_ERR_UNSUPPORTED, "xcd mla: an XCD's value columns must be whole quantisation groups");
    if (s.hidden % kXcdSlots) return set_error(FK_ERR_UNSUPPORTED, "xcd mla: hidden must be a multiple of 64");
    if (g.lp > (uint32_t)kWave) return set_error(FK_ERR_UNSUPPORTED, "xcd mla: a head row must fit one wave (at most 512 dims)");
    // tiles: one pass each; groups fetched four per lane as one aligned run
    const uint32_t wq_cpr = s.hidden / cv, wb_cpr = s.rank / cv;
    const uint32_t gq = s.hidden / s.group, gb = s.rank / s.group, go = (g.hl * s.v_dim) / s.group;
    if (g.R * wq_cpr > (uint32_t)kMlaNlA * kBlock || g.b_rows * wb_cpr > (uint32_t)kMlaNlB * kBlock ||
        g.o_rows * g.o_cs > (uint32_t)kMlaNlO * kBlock)
        return set_error(FK_ERR_UNSUPPORTED, "xcd mla: a block's tile holds more chunks than the kernel requests in one pass");
    if (g.R * gq > kMetaWords || g.b_rows * gb > kMetaWords || g.o_rows * go > kMetaWords)
        return set_error(FK_ERR_UNSUPPORTED, "xcd mla: a block's tile holds more than 768 quantisation groups");
    if (gq % 4 || (g.b_rows * gb) % 4 || (g.b_total * gb) % 4 || (g.o_rows * go) % 4)
        return set_error(FK_ERR_UNSUPPORTED, "xcd mla: a block's tile must hold a multiple of four quantisation groups");
    if (g.lp_.cs_max % 4 || g.lp_.cs_max > 160u) return set_error(FK_ERR_UNSUPPORTED, "xcd mla: rows of more than 160 chunks are not served");
    if (2u * ((g.lds + 1023u) & ~1023u) > kCuLdsBytes) return set_error(FK_ERR_UNSUPPORTED, "xcd mla: two workgroups must fit the LDS of one CU");
    const DeviceFacts* dev;
    FK_TRY(device_facts(&dev));
    if (dev->cus != (int)(kXcds * 32)) return set_error(FK_ERR_UNSUPPORTED, "xcd mla: needs 8 XCDs of 32 CUs");
    return require_two_blocks_per_cu(reinterpret_cast<const void*>(&xcd_mla_kernel<W_Q4>), g.lds, "low-rank attention");
}

size_t xcd_mla_partials_bytes(const XcdMlaShape& s) { return (size_t)s.n_heads * kXcdMaxRanges * (s.v_dim + 2) * sizeof(float); }
size_t xcd_mla_latent_bytes(const XcdMlaShape& s) { return (size_t)kXcds * (s.rank + s.rope_dim) * 2; }

fk_status plan_xcd_mla(const XcdMlaRequest& rq, Launch* out) {
    const XcdMlaShape& s = rq.shape;
    FK_TRY(xcd_mla_supported(s));
    if (!rq.q || !rq.kva || !rq.kvb || !rq.cache_k || !rq.cache_v || !rq.kv_len || !rq.rope_tab || !rq.att_partials ||
        !rq.out_sums || !rq.workspace || !rq.a_norm)
        return set_error(FK_ERR_INVALID, "xcd mla: null buffer");
    if (((uintptr_t)rq.q | (uintptr_t)rq.kva | (uintptr_t)rq.kvb | (uintptr_t)rq.a_norm) & 15u)
        return set_error(FK_ERR_INVALID, "xcd mla: rows must be 16-byte aligned");
    if ((rq.sums2_in != nullptr) && !rq.sums_in) return set_error(FK_ERR_INVALID, "xcd mla: a second sum row comes with a first");
    if (rq.sums2_in && (rq.sums2_in == rq.sums_in || rq.sums2_in == rq.out_sums || rq.sums2_in == rq.clear || rq.sums2_in == rq.clear2))
        return set_error(FK_ERR_INVALID, "xcd mla: the sum rows read, added into and cleared must be different rows");
    if (rq.clear2 && (rq.clear2 == rq.out_sums || rq.clear2 == rq.sums_in || rq.clear2 == rq.clear))
        return set_error(FK_ERR_INVALID, "xcd mla: the sum rows read, added into and cleared must be different rows");
    const MlaGeometry g = mla_geometry(s);
    XcdMlaArgs a;
    memset(&a, 0, sizeof(a));
    XcdLayerShape ls;
    memset(&ls, 0, sizeof(ls));
    ls.hidden = s.hidden;
    ls.bits = s.bits;
    ls.group = s.group;
    FK_TRY(fill_input(ls, rq.sums_in, rq.residual, rq.x_out, rq.clear, rq.out_sums, rq.norm_w, rq.eps, &a.in));
    a.sums2 = rq.sums2_in;
    a.clear2 = rq.clear2;
    FK_TRY(bind_mat(rq.wq, s.n_heads * g.qk_dim, s.hidden, ls, &a.wq, "q_proj"));
    FK_TRY(bind_mat(rq.wa, g.a_rows, s.hidden, ls, &a.wa, "kv_a_proj"));
    FK_TRY(bind_mat(rq.wb, s.n_heads * (s.nope_dim + s.v_dim), s.rank, ls, &a.wb, "kv_b_proj"));
    FK_TRY(bind_mat(rq.wo, s.hidden, s.n_heads * s.v_dim, ls, &a.wo, "o_proj"));
    a.a_norm = rq.a_norm;
    a.hl = g.hl;
    a.q_rows = g.q_rows;
    a.a_rows = g.a_rows;
    a.rank = s.rank;
    a.b_total = g.b_total;
    a.tile_rows = g.R;
    a.q_tiles = g.q_tiles;
    a.a_tiles = g.a_tiles;
    a.b_rows = g.b_rows;
    a.o_rows = g.o_rows;
    a.o_cs = g.o_cs;
    a.q = rq.q;
    a.kva = rq.kva;
    a.kvb = rq.kvb;
    SdpaArgs& sd = a.sdpa;
    sd.q = rq.q;
    sd.k = rq.cache_k;
    sd.v = rq.cache_v;
    sd.out = nullptr;
    sd.kv_len_ptr = rq.kv_len;
    sd.n_heads = s.n_heads;
    sd.n_kv = s.n_heads;
    sd.qk_dim = g.qk_dim;
    sd.v_dim = s.v_dim;
    sd.capacity = s.capacity;
    sd.chunk_len = g.chunk_len;
    sd.chunks_per_block = g.chunks_per_block;
    sd.n_splits = g.n_splits;
    sd.rows = 1;
    sd.lpk = sd.lpv = g.lp;
    sd.scale = rq.scale != 0.f ? rq.scale : 1.0f / sqrtf((float)g.qk_dim);
    sd.partials = rq.att_partials;
    sd.counters = nullptr;
    sd.k_new = rq.kvb;                      // [head][k_nope | v]
    sd.v_new = rq.kvb + s.nope_dim;
    sd.k1_new = rq.kva + s.rank;            // k_pe of the first XCD's copy of the latent row (every copy holds the same bits)
    sd.q0_dim = s.nope_dim;
    sd.k0_stride = s.nope_dim + s.v_dim;
    sd.v_stride = s.nope_dim + s.v_dim;
    sd.k1_heads = 1;
    sd.traditional = rq.traditional ? 1u : 0u;
    sd.cache_k_w = rq.cache_k;
    sd.cache_v_w = rq.cache_v;
    sd.rope_dims = s.rope_dim;
    sd.eps = rq.eps;
    sd.base_log2 = (float)log2((double)rq.theta);
    sd.rope_tab = rq.rope_tab;
    a.out_sums = rq.out_sums;
    a.ctl = reinterpret_cast<XcdControl*>(rq.workspace);
    a.spin_limit = rq.spin_limit ? rq.spin_limit : (1u << 20);
    a.cs_max = g.lp_.cs_max;
    a.work_floats = g.lp_.work_floats;
    a.att_elems = g.lp_.att_elems;
    a.mark_placement = rq.mark_placement ? 1u : 0u;
    out->func = reinterpret_cast<const void*>(&xcd_mla_kernel<W_Q4>);
    FK_TRY(require_two_blocks_per_cu(out->func, g.lds, "low-rank attention"));
    out->grid = dim3(kXcdGrid, 1, 1);
    out->block = dim3(kBlock, 1, 1);
    out->shmem = g.lds;
    out->set_args(a);
    out->n_lead = 0;
    out->add_lead(a.in.sums);
    out->add_lead(a.in.residual);
    out->add_lead(a.in.norm_w);
    out->add_lead(a.in.hidden);
    return FK_OK;
}

}  // namespace fk
