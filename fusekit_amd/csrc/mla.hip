// The two small kernels a mixture-of-experts decoder with low-rank (MLA-style) keys needs next to
// the streaming kernels: the cache store of a key given in two parts, and the router.
// Both are launch-latency sized; what matters is one launch each and the reference's rounding.
#include "fk_host.hpp"
#include "fk_device.hpp"
#include "rope_device.hpp"
#include "route_device.hpp"

namespace fk {

// ------------------------------------------------ split-key cache store (+ rotation of Q1)
//
// Cache K row = [K0 | K1] (src/codegen/kernels/kv_cache_store_decode.rs:268-352): K0 holds n_kv
// heads, K1 n_kv heads or ONE head shared by all of them; the first rope_dims of K1 are rotated at
// the token's position while written, as traditional (2i, 2i+1) or half-split (i, i + half) pairs.
// K0 and V rows are k0_stride / v_stride elements apart, so both may alias one packed
// [n_kv, k0_dim + v_dim] projection output (:103-140).  The query's second part, Q1 of the packed
// [n_heads, q0_dim + q1_dim] rows, gets the same rotation in place and is rounded to T, which is
// what the rotary op writes when it is not sunk into the attention kernel
// (sdpa_decode.rs:592-660 keeps fp32 there).
// One wave per head: blocks [0, n_heads) the query heads, then n_kv key heads, then n_kv value heads.
__global__ __launch_bounds__(kWave) void split_rope_store_kernel(const SplitStoreArgs a) {
    uint32_t b = blockIdx.x;
    const uint32_t lane = threadIdx.x, tr = blockIdx.y;   // tr: active token row (position offset + tr)
    const uint32_t pos0 = a.offset_ptr ? *a.offset_ptr : a.offset_imm;
    const uint32_t pos = pos0 + tr;
    const uint32_t wpos = (a.write_offset_ptr ? *a.write_offset_ptr : (a.use_write_imm ? a.write_offset_imm : pos0)) + tr;
    const uint32_t row = wpos % a.capacity;
    const uint32_t half = a.rope_dims / 2;

    auto rotate = [&](const uint16_t* src, uint16_t* dst) __attribute__((always_inline)) {
        for (uint32_t i = lane; i < half; i += kWave) {
            const uint32_t lo_i = a.traditional ? 2 * i : i, hi_i = a.traditional ? 2 * i + 1 : i + half;
            float lo, hi;
            rope_rotate(bf16_bits_to_f32(src[lo_i]), bf16_bits_to_f32(src[hi_i]), i, half, pos, a.base_log2, lo, hi);
            dst[lo_i] = (uint16_t)f32_to_bf16_bits(lo);
            dst[hi_i] = (uint16_t)f32_to_bf16_bits(hi);
        }
    };
    if (b < a.n_heads) {
        uint16_t* q1 = a.q + ((size_t)tr * a.n_heads + b) * (a.q0_dim + a.q1_dim) + a.q0_dim;
        rotate(q1, q1);
        return;
    }
    b -= a.n_heads;
    if (b < a.n_kv) {
        uint16_t* dst = a.cache_k + ((size_t)b * a.capacity + row) * (a.k0_dim + a.k1_dim);
        const uint16_t* k0 = a.k0 + (size_t)tr * a.k0_row_stride + (size_t)b * a.k0_stride;
        for (uint32_t d = lane; d < a.k0_dim; d += kWave) dst[d] = k0[d];
        const uint16_t* k1 = a.k1 + (size_t)tr * a.k1_row_stride + (size_t)(a.k1_heads == 1 ? 0 : b) * a.k1_dim;
        rotate(k1, dst + a.k0_dim);
        for (uint32_t d = 2 * half + lane; d < a.k1_dim; d += kWave) dst[a.k0_dim + d] = k1[d];
        return;
    }
    b -= a.n_kv;
    uint16_t* dst = a.cache_v + ((size_t)b * a.capacity + row) * a.v_dim;
    const uint16_t* v = a.v + (size_t)tr * a.v_row_stride + (size_t)b * a.v_stride;
    for (uint32_t d = lane; d < a.v_dim; d += kWave) dst[d] = v[d];
}

fk_status plan_split_rope_store(const SplitStoreArgs& a, Launch* out) {
    const DeviceFacts* dev;
    FK_TRY(device_facts(&dev));
    if (!a.k0 || !a.k1 || !a.v || !a.cache_k || !a.cache_v) return set_error(FK_ERR_INVALID, "split store: null pointer");
    if (a.n_heads && !a.q) return set_error(FK_ERR_INVALID, "split store: query heads without a query");
    if (a.n_kv == 0 || a.k0_dim == 0 || a.k1_dim == 0 || a.v_dim == 0 || a.capacity == 0)
        return set_error(FK_ERR_INVALID, "split store: empty shape");
    if (a.k1_heads != 1 && a.k1_heads != a.n_kv)
        return set_error(FK_ERR_INVALID, "split store: K1 has one head or one per KV head");
    if (a.k0_stride < a.k0_dim || a.v_stride < a.v_dim) return set_error(FK_ERR_INVALID, "split store: stride below the row width");
    if (a.rope_dims % 2 || a.rope_dims > a.k1_dim || (a.n_heads && a.rope_dims > a.q1_dim))
        return set_error(FK_ERR_INVALID, "split store: rope_dims must be even and within K1 (and Q1)");
    if (a.n_heads && a.q0_dim + a.q1_dim != a.k0_dim + a.k1_dim)
        return set_error(FK_ERR_INVALID, "split store: query and key widths differ");
    out->func = reinterpret_cast<const void*>(&split_rope_store_kernel);
    if (a.rows > 65535) return set_error(FK_ERR_UNSUPPORTED, "split store: at most 65535 rows per launch");
    if (a.rows > 1 && a.rows > a.capacity) return set_error(FK_ERR_INVALID, "split store: more rows than cache rows");
    out->grid = dim3(a.n_heads + 2 * a.n_kv, a.rows ? a.rows : 1, 1);
    out->block = dim3(kWave, 1, 1);
    out->shmem = 0;
    out->set_args(a);
    return FK_OK;
}

// ------------------------------------------------------------------ softmax top-k route
//
// Router of a mixture-of-experts block (src/codegen/kernels/single.rs:2615-2760): softmax over
// row_n logits, prob = float(T(exp(score - max) * (1 / sum))) rounded to T BEFORE the ordering,
// the top_k largest in descending order with ties to the lower index, weight = T(prob * scale) with
// one scale per row set or one per route.  row_n is a power of two of at most 256, top_k < row_n
// and at most 32 (the reference's admission, :2636-2641).  One wave per row; a lane holds four
// probabilities and the selection is top_k rounds of a wave-wide arg-max.
struct RouteArgs {
    const uint16_t* logits;
    const uint16_t* scale;
    uint32_t* idx;
    uint16_t* weight;
    uint32_t row_n, top_k, scale_per_route;
};
__global__ __launch_bounds__(kWave) void softmax_topk_route_kernel(const RouteArgs a) {
    const uint32_t r = blockIdx.x, lane = threadIdx.x;
    const uint16_t* l = a.logits + (size_t)r * a.row_n;
    float x[4];
    uint32_t p[4];
#pragma unroll
    for (uint32_t j = 0; j < 4; ++j) {
        const uint32_t i = lane + j * kWave;
        x[j] = i < a.row_n ? bf16_bits_to_f32(l[i]) : -INFINITY;
    }
    route_candidates(x, a.row_n, lane, p);
    for (uint32_t k = 0; k < a.top_k; ++k) {
        float best;
        uint32_t best_i;
        route_take_best(p, best, best_i);
        if (lane == 0) {
            const size_t o = (size_t)r * a.top_k + k;
            const float sc = bf16_bits_to_f32(a.scale[a.scale_per_route ? o : 0]);
            a.idx[o] = best_i;
            a.weight[o] = (uint16_t)f32_to_bf16_bits(best * sc);
        }
    }
}

fk_status plan_softmax_topk_route(const uint16_t* logits, const uint16_t* scale, bool scale_per_route, uint32_t rows,
                                  uint32_t row_n, uint32_t top_k, uint32_t* idx, uint16_t* weight, Launch* out) {
    const DeviceFacts* dev;
    FK_TRY(device_facts(&dev));
    if (!logits || !scale || !idx || !weight) return set_error(FK_ERR_INVALID, "softmax top-k route: null pointer");
    if (rows == 0) return set_error(FK_ERR_INVALID, "softmax top-k route: no rows");
    if (row_n < 2 || row_n > 256 || (row_n & (row_n - 1)) || top_k == 0 || top_k >= row_n || top_k > 32)
        return set_error(FK_ERR_UNSUPPORTED,
                         "softmax top-k route: row_n must be a power of two of at most 256, top_k below row_n and at most 32");
    RouteArgs a{logits, scale, idx, weight, row_n, top_k, scale_per_route ? 1u : 0u};
    out->func = reinterpret_cast<const void*>(&softmax_topk_route_kernel);
    out->grid = dim3(rows, 1, 1);
    out->block = dim3(kWave, 1, 1);
    out->shmem = 0;
    out->set_args(a);
    return FK_OK;
}

// ------------------------------------------------------------------ router in one launch
//
// RMSNorm of the hidden row, the router projection (bf16 [experts, hidden]) and the softmax top-k
// route as ONE launch: three launch-latency sized kernels become one.  The arithmetic is the
// composition of the three (kernels/mod.rs:4424-4516 norm with its two roundings; a linear layer
// with fp32 accumulation and one rounding to T; single.rs:2615-2760), and the normalised row is
// written out for the expert projections that follow.
// One wave per expert (a single CU cannot pull the whole matrix quickly: its requests in flight are
// bounded, 256 KB took 15 us from one block): the wave requests its weight row, the activations and
// the norm weights in the same 16-byte-per-lane layout, normalises in registers, reduces its dot
// product and publishes the logit through an agent-scope store; the wave that arrives last at the
// counter routes.  The counter returns to zero for the next launch.
constexpr int kRouterChunks = 8;   // 16-byte pieces per lane and row: hidden <= 4096
struct RouterArgs {
    const uint16_t* x;
    const uint16_t* norm_w;   // null: x is used as it is
    const uint16_t* w;        // bf16 [experts, hidden]
    const uint16_t* scale;    // one bf16 value
    uint16_t* xn;             // [hidden] normalised row, or null
    uint16_t* logits;         // [experts] or null
    uint32_t* idx;
    uint16_t* weight;
    uint32_t* workspace;      // [experts] logits as fp32 bits, then the arrival counter
    uint32_t hidden, experts, top_k;
    float eps;
};
__global__ __launch_bounds__(kWave) void moe_router_kernel(const RouterArgs a) {
    const uint32_t e = blockIdx.x, lane = threadIdx.x, tr = blockIdx.y;   // tr: token row
    const uint32_t chunks = a.hidden / (8 * kWave);
    const uint16_t* xrow = a.x + (size_t)tr * a.hidden;
    uint32_t* ws = a.workspace + (size_t)tr * (a.experts + 1);
    uint4 wr[kRouterChunks], xr[kRouterChunks], nr[kRouterChunks];
#pragma unroll
    for (int c = 0; c < kRouterChunks; ++c) {
        const uint32_t o = ((uint32_t)c < chunks ? c * kWave + lane : lane) * 8;   // beyond the row: a harmless repeat
        wr[c] = *reinterpret_cast<const uint4*>(a.w + (size_t)e * a.hidden + o);
        xr[c] = *reinterpret_cast<const uint4*>(xrow + o);
        nr[c] = a.norm_w ? *reinterpret_cast<const uint4*>(a.norm_w + o) : make_uint4(0, 0, 0, 0);
    }
    float xf[kRouterChunks][8];
    float ss = 0.f;
#pragma unroll
    for (int c = 0; c < kRouterChunks; ++c) {
        const uint32_t p[4] = {xr[c].x, xr[c].y, xr[c].z, xr[c].w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            xf[c][2 * i] = bf16_lo(p[i]);
            xf[c][2 * i + 1] = bf16_hi(p[i]);
        }
        if ((uint32_t)c < chunks) {
#pragma unroll
            for (int i = 0; i < 8; ++i) ss = fmaf(xf[c][i], xf[c][i], ss);
        }
    }
    if (a.norm_w) {
        ss = wave_sum(ss);
        const float r = 1.0f / sqrtf(ss / (float)a.hidden + a.eps);
#pragma unroll
        for (int c = 0; c < kRouterChunks; ++c) {
            const uint32_t p[4] = {nr[c].x, nr[c].y, nr[c].z, nr[c].w};
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                xf[c][2 * i] = round_bf16(bf16_lo(p[i]) * round_bf16(xf[c][2 * i] * r));
                xf[c][2 * i + 1] = round_bf16(bf16_hi(p[i]) * round_bf16(xf[c][2 * i + 1] * r));
            }
        }
    }
    float acc = 0.f;
#pragma unroll
    for (int c = 0; c < kRouterChunks; ++c) {
        if ((uint32_t)c >= chunks) continue;
        const uint32_t p[4] = {wr[c].x, wr[c].y, wr[c].z, wr[c].w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            acc = fmaf(bf16_lo(p[i]), xf[c][2 * i], acc);
            acc = fmaf(bf16_hi(p[i]), xf[c][2 * i + 1], acc);
        }
        if (e == 0 && a.xn) {
            uint4 o;
            o.x = pack_bf16(xf[c][0], xf[c][1]); o.y = pack_bf16(xf[c][2], xf[c][3]);
            o.z = pack_bf16(xf[c][4], xf[c][5]); o.w = pack_bf16(xf[c][6], xf[c][7]);
            *reinterpret_cast<uint4*>(a.xn + (size_t)tr * a.hidden + (c * kWave + lane) * 8) = o;
        }
    }
    acc = round_bf16(wave_sum(acc));
    if (a.top_k == 0) {   // the consumer routes for itself: publish the logit and leave
        if (lane == 0) a.logits[(size_t)tr * a.experts + e] = (uint16_t)(__float_as_uint(acc) >> 16);
        return;
    }
    uint32_t* counter = ws + a.experts;
    uint32_t last = 0;
    if (lane == 0) {
        __hip_atomic_store(&ws[e], __float_as_uint(acc), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (a.logits) a.logits[(size_t)tr * a.experts + e] = (uint16_t)(__float_as_uint(acc) >> 16);
        wait_memory_ops_done();
        last = atomicAdd(counter, 1u) == a.experts - 1 ? 1u : 0u;
    }
    last = __builtin_amdgcn_readfirstlane(last);
    if (!last) return;
    if (lane == 0) __hip_atomic_store(counter, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);

    // softmax top-k over the published logits: the arithmetic of softmax_topk_route_kernel
    float x[4];
    uint32_t p[4];
#pragma unroll
    for (uint32_t j = 0; j < 4; ++j) {
        const uint32_t i = lane + j * kWave;
        x[j] = i < a.experts ? __uint_as_float(__hip_atomic_load(&ws[i], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)) : -INFINITY;
    }
    route_candidates(x, a.experts, lane, p);
    const float sc = bf16_bits_to_f32(a.scale[0]);
    for (uint32_t k = 0; k < a.top_k; ++k) {
        float best;
        uint32_t best_i;
        route_take_best(p, best, best_i);
        if (lane == 0) {
            a.idx[(size_t)tr * a.top_k + k] = best_i;
            a.weight[(size_t)tr * a.top_k + k] = (uint16_t)f32_to_bf16_bits(best * sc);
        }
    }
}

fk_status plan_moe_router(const uint16_t* x, const uint16_t* norm_w, float eps, const uint16_t* w, const uint16_t* scale,
                          uint32_t hidden, uint32_t experts, uint32_t top_k, uint16_t* xn, uint16_t* logits, uint32_t* idx,
                          uint16_t* weight, uint32_t* workspace, Launch* out, uint32_t rows) {
    const DeviceFacts* dev;
    FK_TRY(device_facts(&dev));
    if (!x || !w) return set_error(FK_ERR_INVALID, "router: null pointer");
    if (top_k == 0 && !logits) return set_error(FK_ERR_INVALID, "router: without a route the logits are the output");
    if (top_k != 0 && (!scale || !idx || !weight || !workspace)) return set_error(FK_ERR_INVALID, "router: null pointer");
    if (hidden == 0 || hidden % (8 * kWave) || hidden > (uint32_t)kRouterChunks * 8 * kWave)
        return set_error(FK_ERR_UNSUPPORTED, "router: hidden must be a multiple of 512 of at most 4096");
    if (experts < 2 || experts > 256 || (experts & (experts - 1)) || top_k >= experts || top_k > 32)
        return set_error(FK_ERR_UNSUPPORTED, "router: experts must be a power of two of at most 256, top_k below it and at most 32");
    if (((uintptr_t)x | (uintptr_t)w | (uintptr_t)norm_w | (uintptr_t)xn) & 15u)
        return set_error(FK_ERR_INVALID, "router: activations and weights must be 16-byte aligned");
    RouterArgs a{x, norm_w, w, scale, xn, logits, idx, weight, workspace, hidden, experts, top_k, eps};
    out->func = reinterpret_cast<const void*>(&moe_router_kernel);
    if (rows == 0 || rows > 65535) return set_error(FK_ERR_INVALID, "router: rows must lie in 1 .. 65535");
    out->grid = dim3(experts, rows, 1);
    out->block = dim3(kWave, 1, 1);
    out->shmem = 0;
    out->set_args(a);
    return FK_OK;
}

}  // namespace fk
