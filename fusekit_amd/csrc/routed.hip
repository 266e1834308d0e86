// Mixture-of-experts routed projections for decode, gfx950.
//
// A route is one (token, slot) pair: it reads one activation row and one expert's
// weight matrix out of an expert-stacked tensor [E, O, K*bits/32].  Every route is
// an ordinary flat-stream GEMV whose weight, scale and bias base pointers are
// offset by the expert index, which lives in device memory (the router wrote it
// earlier in the same graph), so the offset is applied inside the kernel: a block
// serves exactly one route (block / blocks_per_route), stages that route's
// activation row once and walks the route's tiles persistently.
//
//   routed gate/up + SwiGLU : out0[route, o] = T(((sig(g) * g) * u) * route_weight)
//   routed down + reduce    : part[route, o] = T(dot), then
//                             out[tok, o] = T(sum_slots rw * part + shared + residual)
// The weighted sum runs in slot order in fp32 in a second small kernel, so the
// result does not depend on which block finishes first.
#include <map>
#include <mutex>

#include "fk_host.hpp"
#include "gemv_kernel.hpp"

namespace fk {

struct RoutedArgs {
    GemvArgs g;                    // geometry of ONE route; pointers at expert 0 / activation row 0 / route 0
    const uint32_t* expert_idx;    // [n_routes]
    const uint32_t* row_idx;       // [n_routes] activation row per route, or null = the route index
    const uint16_t* route_weight;  // [n_routes] bf16 or null
    uint32_t n_experts, n_x_rows, blocks_per_route;
    uint32_t w_stride;             // 16-byte chunks per expert
    uint32_t s_stride;             // scale (= bias) elements per expert
    uint32_t y_stride;             // output elements per route
};

// GemvArgs as one route sees it.  n_mats is a compile-time 1 so that every index
// into the small arrays is static and the view lives in scalar registers.
struct RouteView {
    const uint4* w[2];
    const uint16_t* sc[2];
    const uint16_t* bi[2];
    const uint16_t* bias[2];
    uint16_t* y[2];
    uint32_t n[2];
    uint32_t tile_start[2];
    static constexpr uint32_t n_mats = 1;
    uint32_t K, cpr, gshift, R, n_tiles, lr;
    float inv_cpr;
    const uint16_t* x;
    const uint16_t* norm_w;
    float eps;
    const uint16_t* res;
    const uint16_t* res2;
    int swiglu_variant;
    float y_scale;
};

template <WKind KIND, int NSEG>
__global__ __launch_bounds__(kGemvBlock) void routed_gemv_kernel(const RoutedArgs a) {
    extern __shared__ uint4 lds_raw[];
    const uint32_t route = blockIdx.x / a.blocks_per_route, sub = blockIdx.x - route * a.blocks_per_route;
    uint32_t e = a.expert_idx[route];
    e = e < a.n_experts ? e : a.n_experts - 1;  // routed_qmv_swiglu.rs:138
    uint32_t row = a.row_idx ? a.row_idx[route] : route;
    row = row < a.n_x_rows ? row : a.n_x_rows - 1;

    RouteView v;
#pragma unroll
    for (int m = 0; m < 2; ++m) {
        v.w[m] = a.g.w[m] + (size_t)e * a.w_stride;
        v.sc[m] = a.g.sc[m] + (size_t)e * a.s_stride;
        v.bi[m] = a.g.bi[m] + (size_t)e * a.s_stride;
        v.bias[m] = nullptr;
        v.y[m] = a.g.y[m] + (size_t)route * a.y_stride;
        v.n[m] = a.g.n[m];
        v.tile_start[m] = 0;
    }
    v.K = a.g.K; v.cpr = a.g.cpr; v.gshift = a.g.gshift; v.R = a.g.R; v.n_tiles = a.g.n_tiles; v.lr = a.g.lr;
    v.inv_cpr = a.g.inv_cpr;
    v.x = a.g.x + (size_t)row * a.g.K;
    v.norm_w = nullptr;
    v.eps = 0.f;
    v.res = nullptr;
    v.res2 = nullptr;
    v.swiglu_variant = 1;
    v.y_scale = a.route_weight ? bf16_bits_to_f32(a.route_weight[route]) : 1.0f;

    uint4 wa[kGemvUnroll];
    uint32_t sa[kGemvUnroll], ba[kGemvUnroll];
    uint4 xr[kStageRegs], wr[kStageRegs];
    stage_fetch(v, xr, wr);
    gemv_prefetch<KIND, NSEG>(v, sub, wa, sa, ba);
    gemv_run<KIND, NSEG, false>(v, sub, a.blocks_per_route, lds_raw, wa, sa, ba, xr, wr);
}

struct RouteReduceArgs {
    const uint16_t* parts;         // [n_routes (+ n_tokens shared rows), O] bf16
    const uint16_t* route_weight;  // [n_routes] or null (input already weighted)
    const uint16_t* residual;      // [n_tokens, O] or null
    uint16_t* out;                 // [n_tokens, O]
    uint32_t n_tokens, top_k, O, has_shared;
};

// routed_qmv_reduce.rs:236-322: partial = float(rw) * float(T(dot)), summed in slot
// order, the shared expert's T(dot) last, then the extra residual; one round.
__global__ __launch_bounds__(256) void route_reduce_kernel(const RouteReduceArgs a) {
    const uint32_t i = blockIdx.x * 256u + threadIdx.x;
    if (i >= a.n_tokens * a.O) return;
    const uint32_t t = i / a.O, o = i - t * a.O;
    float acc = 0.f;
    for (uint32_t sl = 0; sl < a.top_k; ++sl) {
        const uint32_t r = t * a.top_k + sl;
        const float p = bf16_bits_to_f32(a.parts[(size_t)r * a.O + o]);
        const float rw = a.route_weight ? bf16_bits_to_f32(a.route_weight[r]) : 1.0f;
        acc = __fadd_rn(acc, __fmul_rn(rw, p));  // two roundings, as two statements in the reference
    }
    if (a.has_shared) acc = __fadd_rn(acc, bf16_bits_to_f32(a.parts[(size_t)(a.n_tokens * a.top_k + t) * a.O + o]));
    if (a.residual) acc = __fadd_rn(acc, bf16_bits_to_f32(a.residual[i]));
    a.out[i] = (uint16_t)f32_to_bf16_bits(acc);
}

namespace {

template <WKind KIND, int NSEG>
const void* routed_func() {
    return reinterpret_cast<const void*>(&routed_gemv_kernel<KIND, NSEG>);
}

const void* select_routed(uint32_t bits, bool swiglu) {
    switch (bits) {
        case 4: return swiglu ? routed_func<W_Q4, 2>() : routed_func<W_Q4, 1>();
        case 8: return swiglu ? routed_func<W_Q8, 2>() : routed_func<W_Q8, 1>();
        default: return swiglu ? routed_func<W_BF16, 2>() : routed_func<W_BF16, 1>();
    }
}

uint32_t resident_blocks(const void* func, uint32_t lds_bytes, int cus) {
    static std::mutex mu;
    static std::map<std::pair<const void*, uint32_t>, int> cache;
    std::lock_guard<std::mutex> lk(mu);
    auto key = std::make_pair(func, lds_bytes);
    auto it = cache.find(key);
    if (it == cache.end()) {
        if (lds_bytes > 48 * 1024)
            (void)hipFuncSetAttribute(func, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes);
        int per_cu = 0;
        if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, func, kGemvBlock, lds_bytes) != hipSuccess || per_cu < 1)
            per_cu = 1;
        it = cache.emplace(key, per_cu).first;
    }
    return (uint32_t)it->second * (uint32_t)cus;
}

}  // namespace

// One launch serving n_routes routes over expert-stacked weights.  `w_a` (and
// `w_b` for the gate/up pair) describe ONE expert's matrix [n, k]; their pointers
// are the base of the stacked tensors.
fk_status plan_routed_gemv(const uint16_t* x, uint32_t n_x_rows, const fk_weight* w_a, const fk_weight* w_b,
                           uint32_t n_experts, const uint32_t* row_idx, const uint32_t* expert_idx,
                           const uint16_t* route_weight, uint32_t n_routes, uint16_t* y, Launch* out) {
    const DeviceFacts* dev;
    FK_TRY(device_facts(&dev));
    if (!expert_idx) return set_error(FK_ERR_INVALID, "routed: null expert_idx");
    if (n_experts == 0 || n_routes == 0 || n_x_rows == 0)
        return set_error(FK_ERR_INVALID, "routed: experts, routes and activation rows must be positive");
    if (n_routes > 65536) return set_error(FK_ERR_UNSUPPORTED, "routed: at most 65536 routes per launch");
    if (!w_a) return set_error(FK_ERR_INVALID, "routed: null weight");
    const bool swiglu = w_b != nullptr;

    GemvRequest rq;
    rq.mats[0] = w_a;
    rq.mats[1] = w_b;
    rq.n_mats = 1;
    rq.swiglu = swiglu;
    rq.swiglu_variant = 1;
    rq.x = x;
    rq.y[0] = y;
    const void* func = select_routed(w_a->bits, swiglu);

    // Two passes: the first sizes LDS with a nominal grid, the second plans the
    // tiles for the share of the resident blocks one route gets.
    Launch base;
    uint32_t per_route = (uint32_t)dev->cus * 4u / n_routes;
    for (int pass = 0; pass < 2; ++pass) {
        t_gemv_grid_override = per_route ? per_route : 1u;
        const fk_status s = plan_gemv(rq, &base);
        t_gemv_grid_override = 0;
        FK_TRY(s);
        per_route = resident_blocks(func, base.shmem, dev->cus) / n_routes;
    }
    GemvArgs g;
    memcpy(&g, base.args, sizeof(g));

    const uint64_t w_stride = (uint64_t)w_a->n * g.cpr;
    const uint64_t s_stride = w_a->bits == 16 ? 0 : (uint64_t)w_a->n * (w_a->k / w_a->group);
    if (w_stride > 0xffffffffull) return set_error(FK_ERR_UNSUPPORTED, "routed: expert matrix too large");

    RoutedArgs a;
    memset(&a, 0, sizeof(a));
    a.g = g;
    a.expert_idx = expert_idx;
    a.row_idx = row_idx;
    a.route_weight = route_weight;
    a.n_experts = n_experts;
    a.n_x_rows = n_x_rows;
    a.blocks_per_route = base.grid.x;
    a.w_stride = (uint32_t)w_stride;
    a.s_stride = (uint32_t)s_stride;
    a.y_stride = w_a->n;

    out->func = func;
    out->grid = dim3(base.grid.x * n_routes, 1, 1);
    out->block = dim3(kGemvBlock, 1, 1);
    out->shmem = base.shmem;
    out->set_args(a);
    if (base.shmem > 48 * 1024)
        FK_HIP(hipFuncSetAttribute(func, hipFuncAttributeMaxDynamicSharedMemorySize, (int)base.shmem));
    return FK_OK;
}

fk_status plan_route_reduce(const uint16_t* parts, const uint16_t* route_weight, const uint16_t* residual,
                            uint16_t* out_ptr, uint32_t n_tokens, uint32_t top_k, uint32_t O, bool has_shared,
                            Launch* out) {
    if (!parts || !out_ptr) return set_error(FK_ERR_INVALID, "route reduce: null tensor");
    if (n_tokens == 0 || top_k == 0 || O == 0) return set_error(FK_ERR_INVALID, "route reduce: empty shape");
    if ((uint64_t)n_tokens * O > 0x7fffffffull) return set_error(FK_ERR_UNSUPPORTED, "route reduce: output too large");
    RouteReduceArgs a;
    a.parts = parts;
    a.route_weight = route_weight;
    a.residual = residual;
    a.out = out_ptr;
    a.n_tokens = n_tokens;
    a.top_k = top_k;
    a.O = O;
    a.has_shared = has_shared ? 1u : 0u;
    out->func = reinterpret_cast<const void*>(&route_reduce_kernel);
    out->grid = dim3((n_tokens * O + 255u) / 256u, 1, 1);
    out->block = dim3(256, 1, 1);
    out->shmem = 0;
    out->set_args(a);
    return FK_OK;
}

}  // namespace fk
