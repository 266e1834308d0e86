// The expert block of a mixture-of-experts layer as ONE XCD-resident launch (see XcdMoeArgs in xcd_layer.hpp for the cut):
// router, ranking, routed and shared gate / up + SwiGLU, routed and shared down_proj, weighted sum into the sum row.
// Reference semantics: SoftmaxTopKRoute (src/codegen/kernels/single.rs:2615-2760), routed_qmv_swiglu.rs:20-452,
// routed_qmv_reduce.rs:11-543.
#include "xcd_layer.hpp"

// Timing probes (empty in the library build): boundary i of every block, by the first thread of each wave pair.
#include "fk_probe.hpp"
FK_PROBE_DEFINE(xcd_moe, 512, 16)
#define FK_XCD_STAMP(k, i) FK_PROBE_STAMP(xcd_moe, 512, 16, blockIdx.x, threadIdx.x == 0, i)

#include "route_device.hpp"
#include "xcd_device.hpp"

namespace fk {

constexpr int kMoeNl = 6;        // 16-byte requests per thread and tile: a tile holds at most 6 * 256 chunks

namespace {

// T(w * T(x * r)) of one group of eight values: the arithmetic of stage_emit's NORM path, kept in registers so that
// the router's dot product can use the same values that are staged.
__device__ __forceinline__ uint4 normed_group(uint4 v, uint4 wv, float r) {
    uint32_t nb[4] = {v.x, v.y, v.z, v.w};
    const uint32_t q[4] = {wv.x, wv.y, wv.z, wv.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const uint32_t xr_ = pack_bf16(bf16_lo(nb[i]) * r, bf16_hi(nb[i]) * r);
        nb[i] = pack_bf16(bf16_lo(q[i]) * bf16_lo(xr_), bf16_hi(q[i]) * bf16_hi(xr_));
    }
    return make_uint4(nb[0], nb[1], nb[2], nb[3]);
}

__device__ __forceinline__ float dot8_bf16(uint4 w, uint4 x, float acc) {
    const uint32_t a[4] = {w.x, w.y, w.z, w.w}, b[4] = {x.x, x.y, x.z, x.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        acc = fmaf(bf16_lo(a[i]), bf16_lo(b[i]), acc);
        acc = fmaf(bf16_hi(a[i]), bf16_hi(b[i]), acc);
    }
    return acc;
}

// Scales and biases of a tile that may be a K-slice of the matrix's rows (MLX layout: [row][groups of the row]), one
// group per lane and request: group gi of the tile = (row gi / gpr, group gi % gpr of the slice).
template <WKind KIND, int SN, typename MAT>
__device__ __forceinline__ void meta_fetch_slice(const MAT& m, const Tile& t, uint32_t ti, MetaRegs& r) {
    const uint32_t gpr = t.cs >> m.gshift, total = t.rows * gpr, full = m.cpr >> m.gshift, g0 = t.col0 >> m.gshift;
    const float inv = 1.0f / (float)gpr;
#pragma unroll
    for (int k = 0; k < kMetaRegs; ++k) {
        const uint32_t gi = k * SN + ti;
        const uint32_t row = (uint32_t)(((float)gi + 0.5f) * inv);
        const size_t e = gi < total ? (size_t)(t.row0 + row) * full + g0 + (gi - row * gpr) : (size_t)t.row0 * full + g0;
        r.s[k] = m.sc[e];
        r.b[k] = m.bi[e];
    }
}

// input_stage of the dense launches, with the router's dot product taken on the way: x = T(sums + residual), its sum
// of squares, T(w * T(x * r)) staged, and -- when `rw` holds this block's router row -- the row's dot product with the
// normalised values (fp32, one partial per thread).  Whole block (two block barriers inside); red: 4 floats of LDS.
template <WKind KIND>
__device__ __forceinline__ float moe_input_stage(const XcdInput& in, const InputRegs& r, const uint4 (&rw)[kInGroups], bool with_router,
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
                    const float lo = xcd_sum_to_f32(r.sv[i][k].x, r.sv[i][k].y) + bf16_lo(xb[k]);
                    const float hi = xcd_sum_to_f32(r.sv[i][k].z, r.sv[i][k].w) + bf16_hi(xb[k]);
                    xb[k] = pack_bf16(lo, hi);
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
    float dot = 0.f;
#pragma unroll
    for (int i = 0; i < kInGroups; ++i) {
        const uint32_t t = threadIdx.x + i * kBlock, sec = t >> 6;
        if (sec * kWave < n8) {
            const uint4 nb = normed_group(xv[i], r.nw[i], rr);
            stage_emit<KIND>(xs, sx, cs, t, t < n8, nb, nb, 1.0f, false);
            if (with_router && t < n8) dot = dot8_bf16(rw[i], nb, dot);
        }
    }
    __syncthreads();
    return dot;
}

}  // namespace

template <WKind KIND>
__global__ __launch_bounds__(kBlock, 2) void xcd_moe_kernel(const long long* sums, const uint16_t* residual, const uint16_t* norm_w,
                                                            uint32_t hidden, const XcdMoeArgs a) {
    extern __shared__ uint4 lds_raw[];
    constexpr int NL = kMoeNl;
    const XcdInputLead lead{sums, residual, norm_w, hidden};
    InputRegs inr;
    input_request<false>(lead, inr, nullptr);
    kernarg_warm<32 + (int)sizeof(XcdMoeArgs)>();
    XcdSync sync = xcd_sync_init(a.ctl, a.spin_limit);
    FK_XCD_STAMP(0, 0);

    const uint32_t cs_max = a.cs_max, work_floats = a.work_floats;
    constexpr int PIECES = ChunkTraits<KIND>::kPieces;
    uint4* xs = lds_raw;
    float* sx = reinterpret_cast<float*>(xs + PIECES * cs_max);
    float* work = sx + cs_max;
    constexpr uint32_t MW = kMetaWords;
    uint32_t* meta = reinterpret_cast<uint32_t*>(work + work_floats);  // [3][MW]
    float* red = reinterpret_cast<float*>(meta + 3 * MW);              // [16]
    const uint32_t tid = threadIdx.x, lane = tid & (kWave - 1);

    const uint32_t unit = sync.xcd;
    const bool routed = unit < a.top_k;                   // block-uniform
    const bool idle = !routed && unit - a.top_k >= a.n_shared;   // an XCD without a unit (top_k + n_shared < 8)
    // shared unit; an idle XCD walks the same code with empty tiles, whose (clamped) requests must stay inside the
    // matrices: it addresses unit 0
    const uint32_t sh = (routed || idle) ? 0u : unit - a.top_k;
    XcdMat G = pick_mat(routed, a.gate, a.sgate), U = pick_mat(routed, a.up, a.sup), D = pick_mat(routed, a.down, a.sdown);

    // A shared unit is served like a route: unit h of the shared expert is its gate / up rows [h I, (h+1) I) and, in
    // down_proj, the K-slice of those rows' outputs -- a partial dot product per output row, added UNROUNDED into the
    // second sum row, whose finished element is the shared expert's full dot product (rounded to T where it is read).
    // Every XCD therefore streams the same number of bytes.
    TileRegs<NL> rg, ru, rd;
    MetaRegs mg, mu, md;
    TilePos<NL> pg, pd;

    // Tile geometry does not depend on the expert: positions are worked out now, relative to the unit's first row, and
    // the ranking only moves the matrices' base pointers to that row (scalar work).
    const uint32_t gu0 = sync.slot * a.gu_rows;
    const Tile tg = make_tile(gu0, idle ? 0u : a.gu_rows, 0, G.cpr);
    tile_pos_init<NL, kBlock>(G, tg, tid, pg);
    const uint32_t out0 = sync.slot * a.down_rows, dcs = a.down.cpr;
    const Tile td = make_tile(out0, idle ? 0u : a.down_rows, routed ? 0u : sh * dcs, dcs);
    tile_pos_init<NL, kBlock>(D, td, tid, pd);
    const bool with_router = routed && sync.slot < a.experts;
    uint4 rw[kInGroups];
    {
        const uint32_t n8 = hidden >> 3;
        const uint4* w8 = reinterpret_cast<const uint4*>(a.router_w) + (size_t)(with_router ? sync.slot : 0u) * n8;
#pragma unroll
        for (int i = 0; i < kInGroups; ++i) {
            const uint32_t t = tid + i * kBlock;
            rw[i] = make_uint4(0, 0, 0, 0);
            if (routed && (t >> 6) * kWave < n8) rw[i] = w8[t < n8 ? t : 0u];
        }
    }
    const float sc = bf16_bits_to_f32(a.route_scale[0]);
    FK_XCD_STAMP(0, 1);
    input_pin(lead, inr);
    float dot = moe_input_stage<KIND>(a.in, inr, rw, with_router, xs, sx, G.cpr, red);
    FK_XCD_STAMP(0, 2);
    input_clear<false>(a.in);

    uint32_t* okw = reinterpret_cast<uint32_t*>(red) + 8;
    uint32_t expert = 0;
    float route_w = 1.0f;
    if (routed) {
        // ---- router logit of expert `slot`, published inside the XCD ----
        dot = wave_sum(dot);
        if (lane == 0) red[4 + tid / kWave] = dot;
        __syncthreads();
        uint32_t* lg = a.logits_xcd + unit * kXcdSlots;
        if (tid == 0 && with_router) {
            const float logit = round_bf16((red[4] + red[5]) + (red[6] + red[7]));
            lg[sync.slot] = __float_as_uint(logit);
            if (unit == 0 && a.logits_out) a.logits_out[sync.slot] = (uint16_t)(__float_as_uint(logit) >> 16);
        }
        xcd_barrier<0>(sync, okw);
        if (!xcd_wait_ok(okw)) return;
        FK_XCD_STAMP(0, 3);
        // ---- every wave ranks the logits and takes winner `unit` ----
        // (route_candidates / route_take_best with one logit per lane: at most 64 experts here; same arithmetic)
        const bool has = lane < a.experts;
        const float xl = has ? __uint_as_float(__hip_atomic_load(lg + lane, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)) : -INFINITY;
        const float mx = wave_max(xl);
        FK_XCD_STAMP(0, 11);
        const float pl = has ? expf(xl - mx) : 0.f;
        const float inv = 1.0f / wave_sum(pl);
        uint32_t key = has ? (__float_as_uint(round_bf16(pl * inv)) | (256u - lane)) : 0u;
        // Rank of every lane's key = number of larger keys (keys of live lanes are distinct: the index is part of the
        // key): 64 independent compares instead of top_k dependent rounds of a wave-wide maximum.  The lane of rank
        // `unit` is the unit's expert -- the lane index IS the expert index.
        uint32_t c0 = 0, c1 = 0;
#pragma unroll
        for (int i = 0; i < (int)kWave; i += 2) {
            const uint32_t s0 = (uint32_t)__builtin_amdgcn_readlane((int)key, i), s1 = (uint32_t)__builtin_amdgcn_readlane((int)key, i + 1);
            c0 += s0 > key ? 1u : 0u;
            c1 += s1 > key ? 1u : 0u;
        }
        const uint32_t rank = c0 + c1;
        const uint32_t wbits = f32_to_bf16_bits(__uint_as_float(key & 0xffff0000u) * sc);
        const unsigned long long mine = __ballot(has && rank == unit);
        const uint32_t win = mine ? (uint32_t)__builtin_ctzll(mine) : 0u;   // (always one lane: top_k <= experts)
        expert = win;
        route_w = bf16_bits_to_f32((uint16_t)__builtin_amdgcn_readlane((int)wbits, win));
        if (unit == 0 && sync.slot == 0 && tid < kWave && has && rank < a.top_k) {   // the host's copy of the route
            if (a.idx_out) a.idx_out[rank] = lane;
            if (a.weight_out) a.weight_out[rank] = (uint16_t)wbits;
        }
        expert = __builtin_amdgcn_readfirstlane(expert);
        FK_XCD_STAMP(0, 12);
    }
    // ---- the unit's gate / up rows: the expert's (routed), rows [h I, (h+1) I) of the shared expert (shared) ----
    {
        const size_t urow = (size_t)(routed ? expert : sh) * a.inter;   // first gate / up row of the unit
        const uint32_t ggr = G.cpr >> G.gshift;
        G.w += urow * G.cpr;
        U.w += urow * U.cpr;
        G.sc += urow * ggr;
        G.bi += urow * ggr;
        U.sc += urow * ggr;
        U.bi += urow * ggr;
        if (routed) {   // an expert's down_proj rows; the shared units take a K-slice of the one shared matrix
            const size_t drow = (size_t)expert * hidden;
            D.w += drow * D.cpr;
            D.sc += drow * (D.cpr >> D.gshift);
            D.bi += drow * (D.cpr >> D.gshift);
        }
    }
    meta_fetch<KIND, kBlock, true>(G, tg, tid, mg);
    meta_fetch<KIND, kBlock, true>(U, tg, tid, mu);
    FK_XCD_STAMP(0, 13);
    tile_load<KIND, NL, kBlock>(G, tg, pg, rg);
    tile_load<KIND, NL, kBlock>(U, tg, pg, ru);
    FK_XCD_STAMP(0, 4);

    uint16_t* mid = a.mid + (size_t)unit * a.inter;
    const int variant = a.swiglu_variant;
    constexpr uint32_t seg = NL * kBlock;
    meta_store<KIND, kBlock, true>(mg, tid, meta);
    meta_store<KIND, kBlock, true>(mu, tid, meta + MW);
    __syncthreads();
    tile_partials<KIND, NL, kBlock>(G, tg, pg, rg, xs, sx, meta, work);
    tile_partials<KIND, NL, kBlock>(U, tg, pg, ru, xs, sx, meta + MW, work + seg);
    // the down_proj rows are requested behind the gate / up arithmetic: not needed before the hand-over
    meta_fetch_slice<KIND, kBlock>(D, td, tid, md);
    tile_load<KIND, NL, kBlock>(D, td, pd, rd);
    FK_XCD_STAMP(0, 5);
    __syncthreads();
    if (!idle)
        tile_rows<true, true>(tg, work, work + seg,
                              [&](uint32_t r, float s0, float s1) { mid[gu0 + r] = (uint16_t)swiglu_bits(s0, s1, variant, 1.0f); });
    FK_XCD_STAMP(0, 6);
    meta_store<KIND, kBlock, false>(md, tid, meta + 2 * MW);
    xcd_barrier<0>(sync, okw);
    const bool ok = xcd_wait_ok(okw);  // tested in front of the additions into the sum rows
    FK_XCD_STAMP(0, 7);

    // ---- down_proj of the unit over its intermediate row ----
    if (!idle) stage_vector<KIND>(mid, a.inter >> 3, dcs, xs, sx);
    __syncthreads();
    FK_XCD_STAMP(0, 8);
    tile_partials<KIND, NL, kBlock>(D, td, pd, rd, xs, sx, meta + 2 * MW, work);
    __syncthreads();
    FK_XCD_STAMP(0, 9);
    if (!idle && ok) {
        long long* out = routed ? a.out_sums : a.out_sums2;
        XcdControl* ctl = sync.ctl;
        // a route's full dot product is rounded to T before it is weighted and summed (routed_qmv_reduce.rs:236-322);
        // a shared unit contributes its K-slice of the shared expert's dot product as it is
        tile_rows<false, true>(td, work, work, [&](uint32_t r, float s0, float) {
            xcd_sum_add(out, out0 + r, routed ? __fmul_rn(route_w, round_bf16(s0)) : s0, ctl);
        });
    }
    FK_XCD_STAMP(0, 10);
    xcd_mark_placement(sync, a.mark_placement);
}

// ================================================================================================ host
namespace {

struct MoeGeometry {
    uint32_t n_shared, gu_rows, down_rows, gate_cpr, down_cpr;
    LdsPlan lp;
    uint32_t lds;
};
MoeGeometry moe_geometry(const XcdMoeShape& s) {
    MoeGeometry g;
    const uint32_t cv = chunk_values(s.bits);
    g.n_shared = s.inter ? s.shared_inter / s.inter : 0u;
    g.gu_rows = s.inter / kXcdSlots;
    g.down_rows = s.hidden / kXcdSlots;
    g.gate_cpr = s.hidden / cv;
    g.down_cpr = s.inter / cv;
    g.lp.cs_max = g.gate_cpr > g.down_cpr ? g.gate_cpr : g.down_cpr;
    g.lp.work_floats = 2u * kMoeNl * kBlock;
    g.lp.att_elems = 0;
    g.lp.meta_words = kMetaWords;
    g.lds = xcd_lds_bytes<W_Q4>(g.lp);
    return g;
}

}  // namespace

fk_status xcd_moe_supported(const XcdMoeShape& s) {
    if (s.bits != 4) return set_error(FK_ERR_UNSUPPORTED, "xcd moe: 4-bit weights only");
    if (s.group != 32 && s.group != 64 && s.group != 128) return set_error(FK_ERR_UNSUPPORTED, "xcd moe: group size must be 32, 64 or 128");
    if (s.hidden == 0 || s.inter == 0 || s.shared_inter == 0 || s.experts == 0 || s.top_k == 0)
        return set_error(FK_ERR_INVALID, "xcd moe: shape parameters missing");
    if (s.experts > kXcdSlots || s.top_k > s.experts) return set_error(FK_ERR_UNSUPPORTED, "xcd moe: at most 64 experts (one router logit per block of an XCD)");
    if (s.shared_inter % s.inter) return set_error(FK_ERR_UNSUPPORTED, "xcd moe: the shared width must be a multiple of an expert's");
    const MoeGeometry g = moe_geometry(s);
    if (g.n_shared < 1 || s.top_k + g.n_shared > kXcds)
        return set_error(FK_ERR_UNSUPPORTED, "xcd moe: routes + shared units (shared width / expert width) must be at most 8, one per XCD");
    if (s.hidden % 128 || s.inter % 128 || s.hidden > (uint32_t)kInGroups * kBlock * 8)
        return set_error(FK_ERR_UNSUPPORTED, "xcd moe: widths must be multiples of 128, hidden at most 4096");
    if (s.inter % kXcdSlots || s.hidden % kXcdSlots)
        return set_error(FK_ERR_UNSUPPORTED, "xcd moe: expert width and hidden must be multiples of 64 (whole rows per block)");
    if (s.hidden % s.group || s.inter % s.group) return set_error(FK_ERR_UNSUPPORTED, "xcd moe: widths must be whole quantisation groups");
    // a tile is one pass of 6 requests per thread; the groups of a gate / up tile are fetched four per lane as one
    // aligned run
    const uint32_t budget = (uint32_t)kMoeNl * kBlock;
    const uint32_t gg = s.hidden / s.group, dg = s.inter / s.group;
    if (g.gu_rows * g.gate_cpr > budget || g.down_rows * g.down_cpr > budget)
        return set_error(FK_ERR_UNSUPPORTED, "xcd moe: a block's tile holds more than 1536 16-byte chunks");
    if (g.gu_rows * gg > kMetaWords || g.down_rows * dg > kMetaWords)
        return set_error(FK_ERR_UNSUPPORTED, "xcd moe: a block's tile holds more than 768 quantisation groups");
    if ((g.gu_rows * gg) % 4) return set_error(FK_ERR_UNSUPPORTED, "xcd moe: a block's gate / up tile must hold a multiple of four quantisation groups");
    if (g.lp.cs_max > 10u * 16u) return set_error(FK_ERR_UNSUPPORTED, "xcd moe: rows of more than 160 chunks are not served");
    if (2u * ((g.lds + 1023u) & ~1023u) > kCuLdsBytes) return set_error(FK_ERR_UNSUPPORTED, "xcd moe: two workgroups must fit the LDS of one CU");
    const DeviceFacts* dev;
    FK_TRY(device_facts(&dev));
    if (dev->cus != (int)(kXcds * 32)) return set_error(FK_ERR_UNSUPPORTED, "xcd moe: needs 8 XCDs of 32 CUs");
    return require_two_blocks_per_cu(reinterpret_cast<const void*>(&xcd_moe_kernel<W_Q4>), g.lds, "expert");
}

size_t xcd_moe_scratch_bytes(const XcdMoeShape& s) { return (size_t)kXcds * kXcdSlots * 4 + (size_t)kXcds * s.inter * 2; }

fk_status plan_xcd_moe(const XcdMoeRequest& rq, Launch* out) {
    const XcdMoeShape& s = rq.shape;
    FK_TRY(xcd_moe_supported(s));
    if (!rq.router_w || !rq.route_scale || !rq.scratch || !rq.out_sums || !rq.out_sums2 || !rq.workspace)
        return set_error(FK_ERR_INVALID, "xcd moe: null router, scratch, sum row or workspace");
    if (rq.out_sums2 == rq.out_sums || rq.out_sums2 == rq.sums_in || rq.out_sums2 == rq.clear)
        return set_error(FK_ERR_INVALID, "xcd moe: the shared expert's sum row must be a row of its own");
    if (((uintptr_t)rq.router_w | (uintptr_t)rq.scratch) & 15u) return set_error(FK_ERR_INVALID, "xcd moe: router rows and scratch must be 16-byte aligned");
    if (rq.swiglu_variant < 0 || rq.swiglu_variant > 2) return set_error(FK_ERR_INVALID, "xcd moe: swiglu variant must be 0, 1 or 2");
    const MoeGeometry g = moe_geometry(s);
    XcdMoeArgs a;
    memset(&a, 0, sizeof(a));
    XcdLayerShape ls;
    memset(&ls, 0, sizeof(ls));
    ls.hidden = s.hidden;
    ls.bits = s.bits;
    ls.group = s.group;
    FK_TRY(fill_input(ls, rq.sums_in, rq.residual, rq.x_out, rq.clear, rq.out_sums, rq.norm_w, rq.eps, &a.in));
    FK_TRY(bind_mat(rq.gate, s.experts * s.inter, s.hidden, ls, &a.gate, "expert gate_proj"));
    FK_TRY(bind_mat(rq.up, s.experts * s.inter, s.hidden, ls, &a.up, "expert up_proj"));
    FK_TRY(bind_mat(rq.down, s.experts * s.hidden, s.inter, ls, &a.down, "expert down_proj"));
    FK_TRY(bind_mat(rq.sgate, s.shared_inter, s.hidden, ls, &a.sgate, "shared gate_proj"));
    FK_TRY(bind_mat(rq.sup, s.shared_inter, s.hidden, ls, &a.sup, "shared up_proj"));
    FK_TRY(bind_mat(rq.sdown, s.hidden, s.shared_inter, ls, &a.sdown, "shared down_proj"));
    a.router_w = rq.router_w;
    a.route_scale = rq.route_scale;
    a.experts = s.experts;
    a.top_k = s.top_k;
    a.n_shared = g.n_shared;
    a.inter = s.inter;
    a.gu_rows = g.gu_rows;
    a.down_rows = g.down_rows;
    a.swiglu_variant = rq.swiglu_variant;
    a.logits_xcd = reinterpret_cast<uint32_t*>(rq.scratch);
    a.mid = reinterpret_cast<uint16_t*>(reinterpret_cast<unsigned char*>(rq.scratch) + (size_t)kXcds * kXcdSlots * 4);
    a.logits_out = rq.logits_out;
    a.idx_out = rq.idx_out;
    a.weight_out = rq.weight_out;
    a.out_sums = rq.out_sums;
    a.out_sums2 = rq.out_sums2;
    a.ctl = reinterpret_cast<XcdControl*>(rq.workspace);
    a.spin_limit = rq.spin_limit ? rq.spin_limit : (1u << 20);
    a.cs_max = g.lp.cs_max;
    a.work_floats = g.lp.work_floats;
    a.mark_placement = rq.mark_placement ? 1u : 0u;
    out->func = reinterpret_cast<const void*>(&xcd_moe_kernel<W_Q4>);
    FK_TRY(require_two_blocks_per_cu(out->func, g.lds, "expert"));
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
