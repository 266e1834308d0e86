// Launch planner and template instances of the flat-stream GEMV.
#include <stdlib.h>

#include <map>
#include <mutex>

#include "fk_host.hpp"

#include "fk_probe.hpp"
FK_PROBE_DEFINE(gemv, 2048, 8)
#define FK_GEMV_STAMP(i) FK_PROBE_STAMP(gemv, 2048, 8, blockIdx.x, threadIdx.x == 0, i)
#include "gemv_kernel.hpp"
#include "gemv_rows.hpp"

namespace fk {

GemvPolicy g_gemv_policy = [] {
    GemvPolicy p;
    const char* e = getenv("FUSEKIT_GEMV_FLAT_ONLY");  // "1": never pick the row-group form (measurements, tests)
    p.flat_only = e && e[0] == '1';
    return p;
}();
thread_local uint32_t t_gemv_grid_override = 0;

namespace {

template <WKind KIND, int NSEG>
const void* gemv_func() {
    return reinterpret_cast<const void*>(&gemv_stream_kernel<KIND, NSEG>);
}

const void* select_gemv(WKind kind, bool swiglu) {
    switch (kind) {
        case W_Q4: return swiglu ? gemv_func<W_Q4, 2>() : gemv_func<W_Q4, 1>();
        case W_Q8: return swiglu ? gemv_func<W_Q8, 2>() : gemv_func<W_Q8, 1>();
        default: return swiglu ? gemv_func<W_BF16, 2>() : gemv_func<W_BF16, 1>();
    }
}

template <WKind KIND, bool TAIL, bool ARGMAX>
const void* rows_func(uint32_t nb) {
    switch (nb) {
        case 3: return reinterpret_cast<const void*>(&gemv_rows_kernel<KIND, 3, TAIL, ARGMAX>);
        case 4: return reinterpret_cast<const void*>(&gemv_rows_kernel<KIND, 4, TAIL, ARGMAX>);
        default: return reinterpret_cast<const void*>(&gemv_rows_kernel<KIND, 5, TAIL, ARGMAX>);
    }
}
template <WKind KIND>
const void* rows_func(uint32_t nb, bool tail, bool argmax) {
    if (argmax) return tail ? rows_func<KIND, true, true>(nb) : rows_func<KIND, false, true>(nb);
    return tail ? rows_func<KIND, true, false>(nb) : rows_func<KIND, false, false>(nb);
}
const void* rows_func(WKind kind, uint32_t nb, bool tail, bool argmax) {
    switch (kind) {
        case W_Q4: return rows_func<W_Q4>(nb, tail, argmax);
        case W_Q8: return rows_func<W_Q8>(nb, tail, argmax);
        default: return rows_func<W_BF16>(nb, tail, argmax);
    }
}

// Blocks of `func` one CU holds at once (registers and LDS decide); cached per (kernel, LDS bytes).
uint32_t blocks_per_cu(const void* func, uint32_t lds_bytes) {
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
    return (uint32_t)it->second;
}

uint32_t ilog2(uint32_t v) {
    uint32_t r = 0;
    while ((1u << (r + 1)) <= v) ++r;
    return r;
}

}  // namespace

// Shapes of the row-group form: rows of whole 256-byte blocks that the staging registers cover, group size 64,
// 32-bit byte offsets into the matrix, and enough rows that every CU gets at least two blocks of four-row passes.
// Batches of 5, 4 or 3 column blocks, whichever leaves the fewest unused slots in a row's last batch (at most 7 %).
uint32_t gemv_rows_batch(uint32_t n, uint32_t k, uint32_t bits, uint32_t group) {
    if (g_gemv_policy.flat_only || (bits != 4 && bits != 8 && bits != 16) || (bits != 16 && group != 64)) return 0;
    const uint32_t values = bits == 4 ? 32u : (bits == 8 ? 16u : 8u);
    if (k == 0 || k % values != 0) return 0;
    const uint32_t cpr = k / values;
    if (cpr % kRowLanes != 0 || k > (uint32_t)kStageRegs * kGemvBlock * 8u) return 0;
    const DeviceFacts* dev;
    if (device_facts(&dev) != FK_OK) return 0;
    const uint64_t passes = ((uint64_t)n + kPassRows - 1) / kPassRows;
    if (passes < 2ull * kBlockWaves * dev->cus || (uint64_t)n * cpr * 16ull > 0xffffffffull) return 0;
    const uint32_t cpl = cpr / kRowLanes;
    uint32_t nb = 0, best_slots = ~0u;
    for (uint32_t c : {5u, 4u, 3u}) {
        const uint32_t slots = (cpl + c - 1) / c * c;
        if (slots < best_slots) best_slots = slots, nb = c;
    }
    return best_slots * 100u <= cpl * 107u ? nb : 0u;
}

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
    if (rq.argmax && (!rq.argmax->next_token || !rq.argmax->workspace))
        return set_error(FK_ERR_INVALID, "gemv: head argmax needs a token slot and a workspace");
    const WKind kind = bits == 4 ? W_Q4 : (bits == 8 ? W_Q8 : W_BF16);
    const uint32_t values = bits == 4 ? 32u : (bits == 8 ? 16u : 8u);
    const uint32_t cpr = K / values;
    const uint32_t nseg = rq.swiglu ? 2u : 1u;

    // Row-group form (gemv_rows.hpp): see gemv_rows_batch for the shapes.
    const uint32_t rows_nb = (!rq.swiglu && nm == 1 && !t_gemv_grid_override && !g_gemv_policy.rows_per_tile && !rq.res &&
                              !rq.res2 && !rq.bias[0])
                                 ? gemv_rows_batch(rq.mats[0]->n, K, bits, bits == 16 ? 64 : group)
                                 : 0u;
    if (rows_nb) {
        const uint32_t cpl = cpr / kRowLanes, nb = rows_nb;
        const uint32_t mb = bits == 4 ? 16u : 8u;
        bool ok = true;
        const uint64_t passes = (rq.mats[0]->n + kPassRows - 1) / kPassRows;
        if (bits != 16 && (((uintptr_t)rq.mats[0]->scales | (uintptr_t)rq.mats[0]->biases) & (mb - 1)) != 0) ok = false;
        if (((uintptr_t)rq.mats[0]->w & 15u) != 0) ok = false;
        const uint32_t lds = kind == W_Q4 ? gemv_rows_lds_bytes<W_Q4>(cpr)
                             : (kind == W_Q8 ? gemv_rows_lds_bytes<W_Q8>(cpr) : gemv_rows_lds_bytes<W_BF16>(cpr));
        if (ok && (int)lds <= dev->max_dyn_lds) {
            const void* f = rows_func(kind, nb, cpl % nb != 0, rq.argmax != nullptr);
            // whole rounds: every wave of the grid gets the same number of passes (to within one)
            const uint64_t cap = g_gemv_policy.grid_blocks ? g_gemv_policy.grid_blocks : (uint64_t)blocks_per_cu(f, lds) * dev->cus;
            const uint64_t block_passes = (passes + kBlockWaves - 1) / kBlockWaves;
            const uint64_t rounds = (block_passes + cap - 1) / cap;
            const uint64_t blocks = (block_passes + rounds - 1) / rounds;
            if (rq.argmax && blocks > kHeadArgmaxMaxBlocks)
                return set_error(FK_ERR_UNSUPPORTED, "gemv: head argmax over more blocks than its workspace holds");
            GemvArgmaxArgs a;
            memset(&a, 0, sizeof(a));
            if (rq.argmax) {
                a.tail.next_token = rq.argmax->next_token;
                a.tail.history = rq.argmax->history;
                a.tail.hist_counter = rq.argmax->hist_counter;
                a.tail.hist_capacity = rq.argmax->hist_capacity;
                a.tail.counter = reinterpret_cast<uint32_t*>(rq.argmax->workspace);
                a.tail.partial = reinterpret_cast<uint64_t*>(reinterpret_cast<char*>(rq.argmax->workspace) + 8);
            }
            uint32_t t0 = 0;
            for (int m = 0; m < nm; ++m) {
                a.w[m] = reinterpret_cast<const uint4*>(rq.mats[m]->w);
                a.sc[m] = rq.mats[m]->scales;
                a.bi[m] = rq.mats[m]->biases;
                a.bias[m] = rq.bias[m];
                a.y[m] = rq.y[m];
                a.n[m] = rq.mats[m]->n;
                a.tile_start[m] = t0;
                t0 += (rq.mats[m]->n + kPassRows - 1) / kPassRows;
            }
            a.tile_start[nm] = t0;
            a.n_mats = nm;
            a.K = K;
            a.cpr = cpr;
            a.gshift = bits == 16 ? 0 : ilog2(group / values);
            a.R = kPassRows;
            a.n_tiles = (uint32_t)passes;
            a.lr = kRowLanes;
            a.inv_cpr = 1.0f / (float)cpr;
            a.x = rq.x;
            a.norm_w = rq.norm_w;
            a.eps = rq.eps;
            a.res = rq.res;
            a.res2 = rq.res2;
            a.y_scale = 1.0f;
            out->func = f;
            out->grid = dim3((uint32_t)blocks, 1, 1);
            out->block = dim3(kGemvBlock, 1, 1);
            out->shmem = lds;
            if (rq.argmax)
                out->set_args(a);
            else
                out->set_args(static_cast<const GemvArgs&>(a));
            out->n_lead = 0;
            out->add_lead(a.x);
            out->add_lead(a.norm_w);
            out->add_lead(a.K);
            if (lds > 48 * 1024) FK_HIP(hipFuncSetAttribute(out->func, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
            return FK_OK;
        }
    }
    if (rq.argmax) return set_error(FK_ERR_UNSUPPORTED, "gemv: head argmax needs a shape the row-group form takes");
    const void* func = select_gemv(kind, rq.swiglu);
    auto tiles_for = [&](uint32_t r) {
        uint64_t t = 0;
        if (rq.swiglu) return (uint64_t)((rq.mats[0]->n + r - 1) / r);
        for (int m = 0; m < nm; ++m) t += (rq.mats[m]->n + r - 1) / r;
        return t;
    };
    auto lds_for = [&](uint32_t r) {
        switch (kind) {
            case W_Q4: return gemv_lds_bytes<W_Q4>(cpr, r * cpr, nseg);
            case W_Q8: return gemv_lds_bytes<W_Q8>(cpr, r * cpr, nseg);
            default: return gemv_lds_bytes<W_BF16>(cpr, r * cpr, nseg);
        }
    };
    // Blocks that can be resident at once (registers and LDS decide): the grid never
    // exceeds it, so no block waits for a slot and then pays the whole start-up chain
    // (stage x, first loads) a second time; surplus tiles go to the persistent loop,
    // whose next batch is already in flight while the current one is consumed.
    auto resident_for = [&](uint32_t lds_bytes) -> uint32_t { return blocks_per_cu(func, lds_bytes) * (uint32_t)dev->cus; };

    // Rows per tile.  A batch (4 x 16-byte loads per lane) costs the same whether its
    // lanes are full or not, and the blocks resident on a CU share its issue slots, so
    // the first figure of merit is the number of batches the busiest CU runs,
    // ceil(blocks / CUs) x tiles per block x batches per tile; ties go to the least
    // total work, batches over all tiles plus one unit per block for its start-up
    // (argument fetch, activation staging).  Measured on the 4B-class gate/up pair
    // (2 x 9728 x 2560): 19 rows per tile = 512 blocks of three 97 %-full batches runs
    // 10.4 us where one-batch tiles of 6 rows on 1280 blocks ran 12.2 us.
    const uint32_t pos = kGemvBlock * (kGemvUnroll / nseg);
    uint32_t r_max = 8 * pos / cpr;  // up to eight batches per tile
    if (r_max < 1) r_max = 1;
    if (r_max > kGemvBlock) r_max = kGemvBlock;
    uint32_t best_r = 1, best_blocks = 1;
    uint64_t best_cost = ~0ull, best_waste = ~0ull;
    for (uint32_t r = 1; r <= r_max; ++r) {
        const uint32_t lds_r = lds_for(r);
        if ((int)lds_r > dev->max_dyn_lds) continue;
        const uint64_t tiles = tiles_for(r);
        uint64_t cap = t_gemv_grid_override ? t_gemv_grid_override
                       : (g_gemv_policy.grid_blocks ? g_gemv_policy.grid_blocks : resident_for(lds_r));
        const uint64_t blocks = tiles < cap ? tiles : cap;
        const uint64_t per_block = (tiles + blocks - 1) / blocks;
        const uint64_t batches = ((uint64_t)r * cpr + pos - 1) / pos;
        // fewer than two blocks (eight waves) on a CU cannot hide the load latency:
        // such a choice is priced as if it ran two
        uint64_t per_cu = (blocks + dev->cus - 1) / dev->cus;
        if (per_cu < 512 / kGemvBlock) per_cu = 512 / kGemvBlock;
        const uint64_t cost = per_cu * per_block * batches;
        const uint64_t waste = tiles * batches + blocks;
        if (cost < best_cost || (cost == best_cost && waste < best_waste)) {
            best_cost = cost;
            best_waste = waste;
            best_r = r;
            best_blocks = (uint32_t)blocks;
        }
    }
    if (best_cost == ~0ull) return set_error(FK_ERR_UNSUPPORTED, "gemv: K too large for LDS staging");
    if (g_gemv_policy.rows_per_tile) {
        best_r = g_gemv_policy.rows_per_tile;
        const uint64_t tiles = tiles_for(best_r);
        const uint64_t cap = t_gemv_grid_override ? t_gemv_grid_override
                             : (g_gemv_policy.grid_blocks ? g_gemv_policy.grid_blocks : resident_for(lds_for(best_r)));
        best_blocks = (uint32_t)(tiles < cap ? tiles : cap);
    }
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
    a.y_scale = 1.0f;

    const uint32_t lds = lds_for(R);
    if ((int)lds > dev->max_dyn_lds) return set_error(FK_ERR_UNSUPPORTED, "gemv: K too large for LDS staging");
    out->func = func;
    out->grid = dim3(best_blocks, 1, 1);
    out->block = dim3(kGemvBlock, 1, 1);
    out->shmem = lds;
    out->set_args(a);
    out->n_lead = 0;
    out->add_lead(a.x);
    out->add_lead(a.norm_w);
    out->add_lead(a.K);
    if (lds > 48 * 1024) {
        FK_HIP(hipFuncSetAttribute(out->func, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    }
    return FK_OK;
}

}  // namespace fk
