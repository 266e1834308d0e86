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
#include <atomic>
#include <map>
#include <mutex>

#include "fk_host.hpp"
#include "gemv_kernel.hpp"
#include "route_device.hpp"

namespace fk {

static std::atomic<bool> g_routed_fused_reduce{true};   // off: always the three launches (tests compare the two)

struct RoutedArgs {
    GemvArgs g;                    // geometry of ONE route; pointers at expert 0 / activation row 0 / route 0
    const uint32_t* expert_idx;    // [n_routes]
    const uint32_t* row_idx;       // [n_routes] activation row per route, or null = the route index
    const uint16_t* route_weight;  // [n_routes] bf16 or null
    uint32_t n_experts, n_x_rows, blocks_per_route;
    uint32_t w_stride;             // 16-byte chunks per expert
    uint32_t s_stride;             // scale (= bias) elements per expert
    uint32_t y_stride;             // output elements per route
    // Shared experts as extra routes (one token): routes n_routes .. n_routes + x_routes - 1 read row block
    // (route - n_routes) of these matrices -- [x_routes * O, K], i.e. a stack of their own -- unweighted,
    // into xy [x_routes * O]: the shared gate/up pair rides in the routed launch.
    const uint4* xw[2];
    const uint16_t* xsc[2];
    const uint16_t* xbi[2];
    uint16_t* xy;
    uint32_t n_routes, x_routes;
    // Routing inside this launch (one token): with `logits` (bf16 [n_experts]) every wave ranks them itself --
    // softmax, probabilities rounded to T, the n_routes largest, ties to the lower index -- and takes the
    // route-th winner as its expert; the first block of a route writes idx_out / weight_out [n_routes] for the
    // kernels that follow.  A router kernel then only publishes logits: no cross-block hand-over anywhere.
    const uint16_t* logits;
    const uint16_t* route_scale;   // one bf16 value
    uint32_t* idx_out;
    uint16_t* weight_out;
    // Several tokens: the routes in the order they are SERVED, order[position] = route (plan_route_order sorts them
    // by expert), or null = as listed.  Routes that chose the same expert then sit next to each other in the grid, and
    // with a multiple of eight blocks per route the blocks that walk the same tiles of the same slice land on the same
    // XCD at the same time: the slice comes from HBM once and from that XCD's L2 for the other rows.  Inputs,
    // outputs and arithmetic of a route are untouched.
    const uint32_t* order;
    // The same serving order found by every wave for itself (up to 64 routes): lane i takes expert_idx[i], ranks the
    // key (expert, i) among all routes, and the lane whose rank is the block's position names the route.  No order
    // array, no launch in front to write one, and the expert and the activation row of the route come out of the same
    // trip to memory.
    uint32_t rank_in_kernel;
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
    kernarg_warm<(int)sizeof(RoutedArgs)>();
    const uint32_t pos = blockIdx.x / a.blocks_per_route, sub = blockIdx.x - pos * a.blocks_per_route;
    uint32_t route = pos;
    uint32_t e = 0, row = 0;
    if (a.order && pos < a.n_routes) {
        route = a.order[pos];
        route = route < a.n_routes ? route : pos;   // a device array is not trusted with addresses
    }
    const bool ranked = a.rank_in_kernel && pos < a.n_routes;   // uniform per block
    if (ranked) {
        const uint32_t lane = threadIdx.x & (kWave - 1), li = lane < a.n_routes ? lane : 0u;
        uint32_t ei = a.expert_idx[li];
        uint32_t ri = a.row_idx ? a.row_idx[li] : li;
        ei = ei < a.n_experts ? ei : a.n_experts - 1;  // routed_qmv_swiglu.rs:138
        const uint32_t key = lane < a.n_routes ? ei * kWave + lane : 0xffffffffu;   // distinct per route
        uint32_t rank = 0;
        for (uint32_t j = 0; j < a.n_routes; ++j) rank += (uint32_t)__builtin_amdgcn_readlane((int)key, (int)j) < key ? 1u : 0u;
        const unsigned long long hit = __ballot(rank == pos && lane < a.n_routes);   // exactly one lane
        route = hit ? (uint32_t)__builtin_ctzll(hit) : pos;
        e = (uint32_t)__builtin_amdgcn_readlane((int)ei, (int)route);
        row = (uint32_t)__builtin_amdgcn_readlane((int)ri, (int)route);
        row = row < a.n_x_rows ? row : a.n_x_rows - 1;
    }
    const bool extra = route >= a.n_routes;     // uniform per block
    const uint32_t lookup = extra ? 0u : route;
    float routed_weight = 1.0f;
    if (!a.logits) {
        if (!ranked) {
            e = a.expert_idx[lookup];
            e = e < a.n_experts ? e : a.n_experts - 1;  // routed_qmv_swiglu.rs:138
            row = a.row_idx ? a.row_idx[lookup] : lookup;
            row = row < a.n_x_rows ? row : a.n_x_rows - 1;
        }
        if (a.route_weight && !extra) routed_weight = bf16_bits_to_f32(a.route_weight[lookup]);
    }
    if (extra) row = 0;
    // The activation row is known here in both forms (row 0 when the launch ranks the logits itself): it is
    // requested BEFORE the ranking, whose logits cost a trip to memory and whose result only the weight addresses
    // need.
    uint4 xr[kStageRegs], wr[kStageRegs];
    stage_fetch(StageLead{a.g.x + (size_t)row * a.g.K, nullptr, a.g.K}, xr, wr);
    if (a.logits && !extra) {
        const uint32_t lane = threadIdx.x & (kWave - 1);
        float x[4];
        uint32_t p[4];
        const uint32_t scale_bits = a.route_scale[0];  // requested with the logits, used behind the ranking
#pragma unroll
        for (uint32_t j = 0; j < 4; ++j) {  // clamped index, straight-line: four requests, one wait
            const uint32_t i = lane + j * kWave;
            const float v = bf16_bits_to_f32(a.logits[i < a.n_experts ? i : 0u]);
            x[j] = i < a.n_experts ? v : -INFINITY;
        }
        route_candidates(x, a.n_experts, lane, p);
        float best = 0.f;
        for (uint32_t k = 0; k <= route; ++k) route_take_best(p, best, e);
        const uint32_t wbits = f32_to_bf16_bits(best * bf16_bits_to_f32(scale_bits));
        if (sub == 0 && threadIdx.x == 0) {
            a.idx_out[route] = e;
            a.weight_out[route] = (uint16_t)wbits;
        }
        e = __builtin_amdgcn_readfirstlane(e);
        if (a.route_weight) routed_weight = bf16_bits_to_f32(wbits);   // any non-null pointer: apply the weight here
    }
    if (extra) e = route - a.n_routes;

    RouteView v;
#pragma unroll
    for (int m = 0; m < 2; ++m) {
        v.w[m] = (extra ? a.xw[m] : a.g.w[m]) + (size_t)e * a.w_stride;
        v.sc[m] = (extra ? a.xsc[m] : a.g.sc[m]) + (size_t)e * a.s_stride;
        v.bi[m] = (extra ? a.xbi[m] : a.g.bi[m]) + (size_t)e * a.s_stride;
        v.bias[m] = nullptr;
        v.y[m] = extra ? a.xy + (size_t)e * a.y_stride : a.g.y[m] + (size_t)route * a.y_stride;
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
    v.y_scale = routed_weight;

    uint4 wa[kGemvUnroll];
    uint32_t sa[kGemvUnroll], ba[kGemvUnroll];
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

// ---------------------------------------------------------------- down + reduce in one launch
//
// One token, int4: out[o] = T(sum_slots rw_r * T(W_down[e_r][o, :] . h[r, :]) + T(W_shared[o, :] . shared_x)
// + residual[o]), the sum in slot order with the reference's roundings (routed_qmv_reduce.rs:236-322),
// without the per-route partial rows ever leaving the chip: a wave owns an output row, requests that row's
// 16-byte pieces of every routed expert and of the shared matrix at once (lane c holds codes 32c .. 32c + 31),
// reduces one dot product after the other across its lanes and adds them in slot order.  The activations of
// all routes sit in LDS in the pairing the int4 dot wants, with the sum of every 32 of them for the bias term.
constexpr int kDrBlock = 512, kDrWaves = kDrBlock / kWave, kDrRows = 1, kDrRoutes = 8, kDrSharedPasses = 2, kDrStage = 3;
struct DownReduceArgs {
    const uint16_t* h;             // [n_h_rows, K]
    const uint4* w; const uint16_t* sc; const uint16_t* bi;      // stacked [E, O, ...]
    const uint32_t* expert_idx;    // [top_k]
    const uint32_t* row_idx;       // [top_k] row of h per slot, or null = the slot
    const uint16_t* route_weight;  // [top_k] or null
    const uint16_t* shared_x;      // [SK] or null
    const uint4* sw; const uint16_t* ssc; const uint16_t* sbi;   // shared [O, SK]
    const uint16_t* residual;      // [O] or null
    uint16_t* out;                 // [O]
    uint32_t K, SK, O, top_k, n_experts, n_h_rows, gdiv;         // gdiv: 32-code pieces per quantisation group
};
__global__ __launch_bounds__(kDrBlock) void routed_down_reduce_kernel(const DownReduceArgs a) {
    extern __shared__ uint4 dr_lds[];
    kernarg_warm<(int)sizeof(DownReduceArgs)>();
    const uint32_t tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
    const uint32_t cpr = a.K / 32, scpr = a.SK / 32, gpr = cpr / a.gdiv, sgpr = scpr / a.gdiv;
    const uint32_t routed8 = a.top_k * a.K / 8, total8 = routed8 + a.SK / 8;
    uint4* xs = dr_lds;                                      // per route: [word slot 0..3][piece]
    float* sx = reinterpret_cast<float*>(xs + total8);       // per route: [piece] sum of its 32 activations

    uint32_t ex[kDrRoutes];
#pragma unroll
    for (int r = 0; r < kDrRoutes; ++r) {
        const uint32_t e = a.expert_idx[(uint32_t)r < a.top_k ? r : 0u];
        ex[r] = e < a.n_experts ? e : a.n_experts - 1;      // routed_qmv_swiglu.rs:138 clamps the same way
    }
    // every weight request of this wave's rows, before the activations are staged
    // (scale and bias stay two raw values until they are used: combining them here would wait for each pair)
    uint4 wq[kDrRows][kDrRoutes], wsq[kDrRows][kDrSharedPasses];
    uint16_t sc_r[kDrRows][kDrRoutes], bi_r[kDrRows][kDrRoutes], sc_s[kDrRows][kDrSharedPasses], bi_s[kDrRows][kDrSharedPasses];
#pragma unroll
    for (int i = 0; i < kDrRows; ++i) {
        const uint32_t o = blockIdx.x * (kDrRows * kDrWaves) + wave + i * kDrWaves;
#pragma unroll
        for (int r = 0; r < kDrRoutes; ++r) {
            // a lane beyond the row repeats piece 0 (its result is dropped): no branch around the requests
            const uint32_t c = lane < cpr ? lane : 0u;
            const size_t row = (size_t)ex[r] * a.O + o;
            const size_t g = row * gpr + c / a.gdiv;
            wq[i][r] = a.w[row * cpr + c];
            sc_r[i][r] = a.sc[g];
            bi_r[i][r] = a.bi[g];
        }
#pragma unroll
        for (int p = 0; p < kDrSharedPasses; ++p) {
            const uint32_t c = lane + p * kWave;
            wsq[i][p] = make_uint4(0, 0, 0, 0);
            sc_s[i][p] = bi_s[i][p] = 0;
            if (a.sw) {
                const uint32_t cc = c < scpr ? c : 0u;
                const size_t g = (size_t)o * sgpr + cc / a.gdiv;
                wsq[i][p] = a.sw[(size_t)o * scpr + cc];
                sc_s[i][p] = a.ssc[g];
                bi_s[i][p] = a.sbi[g];
            }
        }
    }
    // activations: eight per thread and step, re-paired for the int4 dot, summed per 32.  The first
    // kDrStage steps request all their rows before any is used (one memory round trip, not one per step).
    auto source = [&](uint32_t j) __attribute__((always_inline)) {
        if (j >= routed8) return a.shared_x + 8 * (j - routed8);
        const uint32_t r = j / (a.K / 8), jl = j - r * (a.K / 8);
        uint32_t row = a.row_idx ? a.row_idx[r] : r;
        row = row < a.n_h_rows ? row : a.n_h_rows - 1;
        return a.h + (size_t)row * a.K + 8 * jl;
    };
    auto place = [&](uint32_t j, const uint4& v) __attribute__((always_inline)) {
        uint32_t base = routed8, jl = j - routed8, pieces = scpr;
        if (j < routed8) {
            const uint32_t r = j / (a.K / 8);
            base = r * (a.K / 8); jl = j - base; pieces = cpr;
        }
        const uint32_t piece = jl >> 2, slot = jl & 3u;
        uint4 pr;
        pr.x = __builtin_amdgcn_perm(v.y, v.x, 0x05040100u);   // (x0, x2)
        pr.y = __builtin_amdgcn_perm(v.w, v.z, 0x05040100u);   // (x4, x6)
        pr.z = __builtin_amdgcn_perm(v.y, v.x, 0x07060302u);   // (x1, x3)
        pr.w = __builtin_amdgcn_perm(v.w, v.z, 0x07060302u);   // (x5, x7)
        xs[base + slot * pieces + piece] = pr;
        float s8 = ((bf16_lo(v.x) + bf16_hi(v.x)) + (bf16_lo(v.y) + bf16_hi(v.y))) +
                   ((bf16_lo(v.z) + bf16_hi(v.z)) + (bf16_lo(v.w) + bf16_hi(v.w)));
        s8 += __shfl_xor(s8, 1, kWave);
        s8 += __shfl_xor(s8, 2, kWave);
        if (slot == 0) sx[(base >> 2) + piece] = s8;
    };
    uint4 sv[kDrStage];
#pragma unroll
    for (int it = 0; it < kDrStage; ++it) {
        const uint32_t j = tid + it * kDrBlock;
        sv[it] = *reinterpret_cast<const uint4*>(source(j < total8 ? j : 0u));
    }
#pragma unroll
    for (int it = 0; it < kDrStage; ++it) {
        const uint32_t j = tid + it * kDrBlock;
        if (j < total8) place(j, sv[it]);
    }
    for (uint32_t j = tid + kDrStage * kDrBlock; j < total8; j += kDrBlock) place(j, *reinterpret_cast<const uint4*>(source(j)));
    __syncthreads();

    auto piece_dot = [&](const uint4& wv, uint32_t scale, uint32_t bias, uint32_t base, uint32_t pieces, uint32_t c) __attribute__((always_inline)) {
        float d0 = 0.f, d1 = 0.f;
        d0 = q4_word_dot(wv.x, xs[base + c], d0);
        d1 = q4_word_dot(wv.y, xs[base + pieces + c], d1);
        d0 = q4_word_dot(wv.z, xs[base + 2 * pieces + c], d0);
        d1 = q4_word_dot(wv.w, xs[base + 3 * pieces + c], d1);
        return fmaf(bf16_bits_to_f32(scale), d0 + d1, bf16_bits_to_f32(bias) * sx[(base >> 2) + c]);
    };
#pragma unroll
    for (int i = 0; i < kDrRows; ++i) {
        const uint32_t o = blockIdx.x * (kDrRows * kDrWaves) + wave + i * kDrWaves;
        float acc = 0.f;
#pragma unroll
        for (int r = 0; r < kDrRoutes; ++r) {
            if ((uint32_t)r >= a.top_k) break;
            float d = lane < cpr ? piece_dot(wq[i][r], sc_r[i][r], bi_r[i][r], r * (a.K / 8), cpr, lane) : 0.f;
            d = round_bf16(wave_sum(d));
            const float rw = a.route_weight ? bf16_bits_to_f32(a.route_weight[r]) : 1.0f;
            acc = __fadd_rn(acc, __fmul_rn(rw, d));
        }
        if (a.sw) {
            float d = 0.f;
#pragma unroll
            for (int p = 0; p < kDrSharedPasses; ++p) {
                const uint32_t c = lane + p * kWave;
                if (c < scpr) d += piece_dot(wsq[i][p], sc_s[i][p], bi_s[i][p], routed8, scpr, c);
            }
            acc = __fadd_rn(acc, round_bf16(wave_sum(d)));
        }
        if (a.residual) acc = __fadd_rn(acc, bf16_bits_to_f32(a.residual[o]));
        if (lane == 0) a.out[o] = (uint16_t)f32_to_bf16_bits(acc);
    }
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
                           const uint16_t* route_weight, uint32_t n_routes, uint16_t* y, Launch* out,
                           const fk_weight* sh_a, const fk_weight* sh_b, uint16_t* sh_y, const RouteInKernel* rk,
                           const uint32_t* order) {
    const DeviceFacts* dev;
    FK_TRY(device_facts(&dev));
    if (order && (rk || sh_a)) return set_error(FK_ERR_UNSUPPORTED, "routed: a serving order goes with listed routes of several tokens only");
    const bool rank_in_kernel = order == kOrderInKernel;
    if (rank_in_kernel && (n_routes > 64 || n_experts > (1u << 24)))
        return set_error(FK_ERR_UNSUPPORTED, "routed: the launch ranks up to 64 routes itself; more take an order array (fk_route_order)");
    if (rk) {
        if (!rk->logits || !rk->scale || !rk->idx_out || !rk->weight_out) return set_error(FK_ERR_INVALID, "routed: null routing tensor");
        if (n_x_rows != 1) return set_error(FK_ERR_UNSUPPORTED, "routed: the launch routes for one token only");
        if (n_experts < 2 || n_experts > 256 || (n_experts & (n_experts - 1)) || n_routes >= n_experts || n_routes > 32)
            return set_error(FK_ERR_UNSUPPORTED, "routed: experts must be a power of two of at most 256, routes below it and at most 32");
    } else if (!expert_idx) {
        return set_error(FK_ERR_INVALID, "routed: null expert_idx");
    }
    uint32_t x_routes = 0;
    if (sh_a) {
        if (!w_b || !sh_b || !sh_y) return set_error(FK_ERR_INVALID, "routed: shared experts come as a gate/up pair with an output");
        if (n_x_rows != 1) return set_error(FK_ERR_UNSUPPORTED, "routed: shared experts ride along for one token only");
        for (const fk_weight* w : {sh_a, sh_b})
            if (!w->w || w->k != w_a->k || w->bits != w_a->bits || w->group != w_a->group || w->n != sh_a->n || w->n == 0 ||
                w->n % w_a->n || (w->bits != 16 && (!w->scales || !w->biases)))
                return set_error(FK_ERR_INVALID, "routed: shared matrices must be whole row blocks of the expert shape");
        x_routes = sh_a->n / w_a->n;
    }
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
    const uint32_t all_routes = n_routes + x_routes;
    uint32_t per_route = (uint32_t)dev->cus * 4u / all_routes;
    for (int pass = 0; pass < 2; ++pass) {
        t_gemv_grid_override = per_route ? per_route : 1u;
        const fk_status s = plan_gemv(rq, &base);
        t_gemv_grid_override = 0;
        FK_TRY(s);
        per_route = resident_blocks(func, base.shmem, dev->cus) / all_routes;
        // served in expert order: a whole number of XCD rounds per route, so that block (position, i) and block
        // (position + 1, i) share an XCD
        if (order && per_route >= 8) per_route &= ~7u;
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
    a.n_routes = n_routes;
    a.x_routes = x_routes;
    a.order = rank_in_kernel ? nullptr : order;
    a.rank_in_kernel = rank_in_kernel ? 1u : 0u;
    if (rk) {
        a.logits = rk->logits; a.route_scale = rk->scale; a.idx_out = rk->idx_out; a.weight_out = rk->weight_out;
        a.route_weight = rk->apply_weight ? rk->scale : nullptr;
    }
    if (sh_a) {
        a.xw[0] = static_cast<const uint4*>(sh_a->w); a.xw[1] = static_cast<const uint4*>(sh_b->w);
        a.xsc[0] = sh_a->scales; a.xsc[1] = sh_b->scales;
        a.xbi[0] = sh_a->biases; a.xbi[1] = sh_b->biases;
        a.xy = sh_y;
    }

    out->func = func;
    out->grid = dim3(base.grid.x * all_routes, 1, 1);
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

size_t routed_parts_bytes(uint32_t n_tokens, uint32_t top_k, uint32_t out_dim) {
    return (((size_t)n_tokens * top_k + n_tokens) * out_dim * sizeof(uint16_t) + 255) & ~(size_t)255;
}

size_t routed_reduce_workspace_bytes(uint32_t n_tokens, uint32_t top_k, uint32_t out_dim, uint32_t shared_k, uint32_t group) {
    size_t b = routed_parts_bytes(n_tokens, top_k, out_dim);
    if (n_tokens > 1 && shared_k) {
        size_t q = 0;
        if (qgemm_workspace_bytes(n_tokens, out_dim, shared_k, group ? group : 64, &q) == FK_OK) b += q;
    }
    return b;
}

// The fused form serves one token of int4 weights whose rows fit the lanes of a wave; anything else takes
// the three launches.
static bool down_reduce_fits(const fk_weight* Wd, const fk_weight* Ws, uint32_t n_tokens, uint32_t top_k) {
    if (n_tokens != 1 || top_k > (uint32_t)kDrRoutes || Wd->bits != 4 || (Wd->group != 32 && Wd->group != 64 && Wd->group != 128))
        return false;
    if (Wd->k % Wd->group || Wd->k > 32u * kWave || Wd->n % (kDrRows * kDrWaves)) return false;
    if (Ws && (Ws->bits != 4 || Ws->group != Wd->group || Ws->k % Ws->group || Ws->k > 32u * kWave * kDrSharedPasses)) return false;
    const size_t lds = ((size_t)top_k * Wd->k + (Ws ? Ws->k : 0)) * (2 + 4.0 / 32);
    return lds <= 60 * 1024;
}

fk_status plan_routed_reduce_chain(const uint16_t* h, uint32_t n_h_rows, const fk_weight* Wd, uint32_t n_experts,
                                   const uint32_t* row_idx, const uint32_t* expert_idx, const uint16_t* route_weight,
                                   const uint16_t* shared_x, const fk_weight* W_shared, const uint16_t* residual,
                                   uint32_t n_tokens, uint32_t top_k, uint16_t* out_ptr, uint16_t* parts, Launch* out,
                                   const uint32_t* order) {
    if (!Wd || !out_ptr || !h) return set_error(FK_ERR_INVALID, "routed reduce: null weight, input or output");
    if (n_tokens == 0 || top_k == 0) return set_error(FK_ERR_INVALID, "routed reduce: empty route set");
    if ((shared_x != nullptr) != (W_shared != nullptr))
        return set_error(FK_ERR_INVALID, "routed reduce: shared_x and W_shared come together");
    if (W_shared && W_shared->n != Wd->n)
        return set_error(FK_ERR_UNSUPPORTED, "routed reduce: the shared expert must have the routed experts' output width");
    if ((uint64_t)n_tokens * top_k > 65536) return set_error(FK_ERR_UNSUPPORTED, "routed reduce: too many routes");
    const uint32_t n_routes = n_tokens * top_k;
    if (g_routed_fused_reduce && down_reduce_fits(Wd, W_shared, n_tokens, top_k)) {
        const DeviceFacts* dev;
        FK_TRY(device_facts(&dev));
        if (!expert_idx) return set_error(FK_ERR_INVALID, "routed: null expert_idx");
        if (n_experts == 0 || n_h_rows == 0) return set_error(FK_ERR_INVALID, "routed: experts and activation rows must be positive");
        if (!Wd->w || !Wd->scales || !Wd->biases || (W_shared && (!W_shared->w || !W_shared->scales || !W_shared->biases)))
            return set_error(FK_ERR_INVALID, "routed reduce: null weight arrays");
        if (((uintptr_t)h | (uintptr_t)shared_x | (uintptr_t)Wd->w | (uintptr_t)(W_shared ? W_shared->w : nullptr)) & 15u)
            return set_error(FK_ERR_INVALID, "routed reduce: activations and weights must be 16-byte aligned");
        DownReduceArgs a;
        memset(&a, 0, sizeof(a));
        a.h = h;
        a.w = static_cast<const uint4*>(Wd->w); a.sc = Wd->scales; a.bi = Wd->biases;
        a.expert_idx = expert_idx; a.row_idx = row_idx; a.route_weight = route_weight;
        a.shared_x = shared_x;
        if (W_shared) { a.sw = static_cast<const uint4*>(W_shared->w); a.ssc = W_shared->scales; a.sbi = W_shared->biases; a.SK = W_shared->k; }
        a.residual = residual; a.out = out_ptr;
        a.K = Wd->k; a.O = Wd->n; a.top_k = top_k; a.n_experts = n_experts; a.n_h_rows = n_h_rows; a.gdiv = Wd->group / 32;
        const size_t lds = ((size_t)top_k * a.K + a.SK) / 8 * 16 + ((size_t)top_k * a.K + a.SK) / 32 * 4;
        out->func = reinterpret_cast<const void*>(&routed_down_reduce_kernel);
        out->grid = dim3(a.O / (kDrRows * kDrWaves), 1, 1);
        out->block = dim3(kDrBlock, 1, 1);
        out->shmem = (uint32_t)lds;
        out->set_args(a);
        if (lds > 48 * 1024)
            FK_HIP(hipFuncSetAttribute(out->func, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
        return FK_OK;
    }
    if (!parts) return set_error(FK_ERR_INVALID, "routed reduce: workspace required");
    FK_TRY(plan_routed_gemv(h, n_h_rows, Wd, nullptr, n_experts, row_idx, expert_idx, nullptr, n_routes, parts, out, nullptr,
                            nullptr, nullptr, nullptr, order));
    if (W_shared && n_tokens == 1) {
        GemvRequest rq;
        rq.mats[0] = W_shared;
        rq.y[0] = parts + (size_t)n_routes * Wd->n;
        rq.x = shared_x;
        Launch shared;
        FK_TRY(plan_gemv(rq, &shared));
        out->then.push_back(shared);
    } else if (W_shared) {
        // several tokens: the shared expert's rows through the multi-row matmul, T(dot) per token into the
        // rows behind the routes'; its own workspace follows the partial rows (routed_reduce_workspace_bytes)
        unsigned char* qws = reinterpret_cast<unsigned char*>(parts) + routed_parts_bytes(n_tokens, top_k, Wd->n);
        Launch main, red;
        FK_TRY(plan_qgemm(W_shared, shared_x, n_tokens, nullptr, nullptr, parts + (size_t)n_routes * Wd->n, qws, &main, &red));
        out->then.push_back(main);
        if (red.func) out->then.push_back(red);
    }
    Launch reduce;
    FK_TRY(plan_route_reduce(parts, route_weight, residual, out_ptr, n_tokens, top_k, Wd->n, W_shared != nullptr, &reduce));
    out->then.push_back(reduce);
    return FK_OK;
}

void set_routed_fused_reduce(bool on) { g_routed_fused_reduce = on; }

// ---------------------------------------------------------------- routes in expert order
// order[position] = route, the routes sorted by expert index (clamped as the routed kernels clamp it), routes of one
// expert in their listed order: a stable counting sort by one block.  Each thread ranks its routes against the
// list in LDS: rank = routes with a smaller expert + earlier routes with the same one.
constexpr uint32_t kOrderMaxRoutes = 2048;
struct RouteOrderArgs {
    const uint32_t* expert_idx;
    uint32_t* order;
    uint32_t n_routes, n_experts;
};
__global__ __launch_bounds__(256) void route_order_kernel(const RouteOrderArgs a) {
    __shared__ uint32_t ex[kOrderMaxRoutes];
    for (uint32_t r = threadIdx.x; r < a.n_routes; r += 256) {
        const uint32_t e = a.expert_idx[r];
        ex[r] = e < a.n_experts ? e : a.n_experts - 1;
    }
    __syncthreads();
    for (uint32_t r = threadIdx.x; r < a.n_routes; r += 256) {
        const uint32_t e = ex[r];
        uint32_t rank = 0;
        for (uint32_t j = 0; j < a.n_routes; ++j) rank += (ex[j] < e || (ex[j] == e && j < r)) ? 1u : 0u;
        a.order[rank] = r;
    }
}

fk_status plan_route_order(const uint32_t* expert_idx, uint32_t n_routes, uint32_t n_experts, uint32_t* order, Launch* out) {
    if (!expert_idx || !order) return set_error(FK_ERR_INVALID, "route order: null array");
    if (n_routes == 0 || n_experts == 0) return set_error(FK_ERR_INVALID, "route order: routes and experts must be positive");
    if (n_routes > kOrderMaxRoutes) return set_error(FK_ERR_UNSUPPORTED, "route order: at most 2048 routes");
    RouteOrderArgs a{expert_idx, order, n_routes, n_experts};
    out->func = reinterpret_cast<const void*>(&route_order_kernel);
    out->grid = dim3(1, 1, 1);
    out->block = dim3(256, 1, 1);
    out->shmem = 0;
    out->set_args(a);
    return FK_OK;
}

}  // namespace fk
