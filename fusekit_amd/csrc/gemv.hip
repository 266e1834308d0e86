// Launch planner and template instances of the flat-stream GEMV.
#include "fk_host.hpp"
#include "gemv_kernel.hpp"

namespace fk {

GemvPolicy g_gemv_policy;

namespace {

template <WKind KIND, int NSEG, bool NORM>
const void* gemv_func() {
    return reinterpret_cast<const void*>(&gemv_stream_kernel<KIND, NSEG, NORM>);
}

const void* select_gemv(WKind kind, bool swiglu, bool norm) {
#define FK_PICK(KIND)                                                                    \
    return swiglu ? (norm ? gemv_func<KIND, 2, true>() : gemv_func<KIND, 2, false>())    \
                  : (norm ? gemv_func<KIND, 1, true>() : gemv_func<KIND, 1, false>())
    switch (kind) {
        case W_Q4: FK_PICK(W_Q4);
        case W_Q8: FK_PICK(W_Q8);
        default: FK_PICK(W_BF16);
    }
#undef FK_PICK
}

uint32_t ilog2(uint32_t v) {
    uint32_t r = 0;
    while ((1u << (r + 1)) <= v) ++r;
    return r;
}

}  // namespace

fk_status plan_gemv(const GemvRequest& rq, Launch* out) {
    const DeviceFacts* dev;
    FK_TRY(device_facts(&dev));
    const int nm = rq.swiglu ? 2 : rq.n_mats;
    if (nm < 1 || nm > kMaxMats) return set_error(FK_ERR_INVALID, "gemv: 1..3 matrices");
    const fk_weight* w0 = rq.mats[0];
    if (!w0 || !rq.x) return set_error(FK_ERR_INVALID, "gemv: null weight or activation pointer");
    const uint32_t K = w0->k, bits = w0->bits;
    if (bits != 4 && bits != 8 && bits != 16) return set_error(FK_ERR_UNSUPPORTED, "gemv: bits must be 4, 8 or 16");
    if (K == 0 || K % 64 != 0) return set_error(FK_ERR_UNSUPPORTED, "gemv: K must be a positive multiple of 64");
    uint32_t group = w0->group;
    if (bits != 16 && group != 32 && group != 64 && group != 128)
        return set_error(FK_ERR_UNSUPPORTED, "gemv: group size must be 32, 64 or 128");
    for (int m = 0; m < nm; ++m) {
        const fk_weight* w = rq.mats[m];
        if (!w || !w->w) return set_error(FK_ERR_INVALID, "gemv: null weight");
        if (w->k != K || w->bits != bits || (bits != 16 && w->group != group))
            return set_error(FK_ERR_INVALID, "gemv: fused matrices must share K, bits and group size");
        if (bits != 16 && (!w->scales || !w->biases)) return set_error(FK_ERR_INVALID, "gemv: null scales/biases");
        if (w->n == 0) return set_error(FK_ERR_INVALID, "gemv: matrix with zero rows");
        if (!rq.swiglu && !rq.y[m]) return set_error(FK_ERR_INVALID, "gemv: null output");
    }
    if (rq.swiglu) {
        if (rq.mats[0]->n != rq.mats[1]->n) return set_error(FK_ERR_INVALID, "gemv: gate and up need equal rows");
        if (!rq.y[0]) return set_error(FK_ERR_INVALID, "gemv: null output");
    }
    const WKind kind = bits == 4 ? W_Q4 : (bits == 8 ? W_Q8 : W_BF16);
    const uint32_t values = bits == 4 ? 32u : (bits == 8 ? 16u : 8u);
    const uint32_t cpr = K / values;
    const uint32_t nseg = rq.swiglu ? 2u : 1u;
    constexpr uint32_t kBatch = kGemvBlock * kGemvUnroll;

    // Rows per tile: keep a tile near one batch of 16-byte loads per lane, then
    // pick the R whose tile count spreads most evenly over the compute units
    // (cost = tiles-per-CU x (tile chunks + a fixed per-tile overhead)).
    uint32_t r_max = kBatch / (nseg * cpr);
    if (r_max < 1) r_max = 1;
    if (r_max > kGemvBlock) r_max = kGemvBlock;
    uint32_t best_r = 1;
    uint64_t best_cost = ~0ull;
    auto tiles_for = [&](uint32_t r) {
        uint64_t t = 0;
        if (rq.swiglu) return (uint64_t)((rq.mats[0]->n + r - 1) / r);
        for (int m = 0; m < nm; ++m) t += (rq.mats[m]->n + r - 1) / r;
        return t;
    };
    for (uint32_t r = 1; r <= r_max; ++r) {
        const uint64_t tiles = tiles_for(r);
        const uint64_t per_cu = (tiles + dev->cus - 1) / dev->cus;
        const uint64_t cost = per_cu * ((uint64_t)r * cpr * nseg + kGemvBlock);
        if (cost <= best_cost) {
            best_cost = cost;
            best_r = r;
        }
    }
    if (g_gemv_policy.rows_per_tile) best_r = g_gemv_policy.rows_per_tile;
    const uint32_t R = best_r;
    const uint64_t tiles = tiles_for(R);
    if (tiles > 0x7fffffffull) return set_error(FK_ERR_UNSUPPORTED, "gemv: too many tiles");

    GemvArgs a;
    memset(&a, 0, sizeof(a));
    uint32_t t0 = 0;
    for (int m = 0; m < nm; ++m) {
        a.w[m] = reinterpret_cast<const uint4*>(rq.mats[m]->w);
        a.sc[m] = rq.mats[m]->scales;
        a.bi[m] = rq.mats[m]->biases;
        a.bias[m] = rq.bias[m];
        a.y[m] = rq.y[m];
        a.n[m] = rq.mats[m]->n;
        a.tile_start[m] = t0;
        t0 += (rq.mats[m]->n + R - 1) / R;
    }
    a.tile_start[nm] = t0;
    a.n_mats = nm;
    a.K = K;
    a.cpr = cpr;
    a.gshift = bits == 16 ? 0 : ilog2(group / values);
    a.R = R;
    a.n_tiles = (uint32_t)tiles;
    uint32_t lr = 1u << ilog2(kGemvBlock / R ? kGemvBlock / R : 1);
    if (lr > 64) lr = 64;
    while (lr > 1 && lr > cpr) lr >>= 1;
    a.lr = lr;
    a.inv_cpr = 1.0f / (float)cpr;
    a.x = rq.x;
    a.norm_w = rq.norm_w;
    a.eps = rq.eps;
    a.res = rq.res;
    a.res2 = rq.res2;
    a.swiglu_variant = rq.swiglu_variant;

    uint32_t lds = 0;
    switch (kind) {
        case W_Q4: lds = gemv_lds_bytes<W_Q4>(cpr, R * cpr, nseg); break;
        case W_Q8: lds = gemv_lds_bytes<W_Q8>(cpr, R * cpr, nseg); break;
        default: lds = gemv_lds_bytes<W_BF16>(cpr, R * cpr, nseg); break;
    }
    if ((int)lds > dev->max_dyn_lds) return set_error(FK_ERR_UNSUPPORTED, "gemv: K too large for LDS staging");

    uint32_t grid_cap = g_gemv_policy.grid_blocks ? g_gemv_policy.grid_blocks : (uint32_t)dev->cus * 8u;
    out->func = select_gemv(kind, rq.swiglu, rq.norm_w != nullptr);
    out->grid = dim3((uint32_t)(tiles < grid_cap ? tiles : grid_cap), 1, 1);
    out->block = dim3(kGemvBlock, 1, 1);
    out->shmem = lds;
    out->set_args(a);
    if (lds > 48 * 1024) {
        FK_HIP(hipFuncSetAttribute(out->func, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    }
    return FK_OK;
}

}  // namespace fk
