// GQA scaled-dot-product attention for one new token over a bf16 KV cache
// (split-K "flash decoding"), gfx950.
//
// Grid (splits, kv heads, head tiles).  A block owns one KV head, one range of
// `chunk_len` cache positions and up to GT query heads of that KV head's group,
// so every K and V element is read from HBM once and used for all of them.
//   phase A  scores: a key row is spread over LPK lanes (16 bytes = 8 dims per
//            lane, 1 KiB contiguous per wave load); each lane dots its 8 dims
//            with the matching q slice of each head (registers), a butterfly
//            over the LPK lanes finishes the dot; scores land in LDS.
//   softmax  per head by one wave: max, exp, sum (fp32, probabilities are never
//            rounded to bf16).
//   phase B  o += p * v with the same lane layout over V rows; lanes keep 8
//            output dims per head, reduced over key slots at the end.
// A range that covers the whole context writes the output directly; otherwise
// the block stores (m, l, o) and the last block to finish per (kv head, head
// tile) merges the partials in split order (so the result does not depend on
// arrival order) and resets the counter for the next launch.
#include "fk_host.hpp"

#include "fk_probe.hpp"
FK_PROBE_DEFINE(sdpa, 4096, 10)
#define FK_SDPA_STAMP(i) \
    FK_PROBE_STAMP(sdpa, 4096, 10, blockIdx.x + gridDim.x * (blockIdx.y + gridDim.y * blockIdx.z), threadIdx.x == 0, i)
#include "sdpa_kernel.hpp"

namespace fk {

namespace {
uint32_t pow2_ceil(uint32_t v) {
    uint32_t p = 1;
    while (p < v) p <<= 1;
    return p;
}
}  // namespace

// Positions per range: every lane owns exactly kSteps key rows, i.e.
// kSteps * (block threads / lanes per key row).  128 positions for head_dim 128
// (64 KiB of K+V per block); a 32k context then spreads over 256 ranges x kv heads.
uint32_t sdpa_chunk_len(uint32_t qk_dim, uint32_t v_dim, bool fused) {
    const uint32_t lpk = pow2_ceil(qk_dim / 8), lpv = pow2_ceil(v_dim / 8);
    const uint32_t wide = lpk > lpv ? lpk : lpv;
    return (fused ? kSdpaStepsFused : kSdpaSteps) * (kSdpaBlock / wide);
}

fk_status sdpa_workspace_bytes(uint32_t n_heads, uint32_t n_kv, uint32_t qk_dim, uint32_t v_dim, uint32_t max_len,
                               size_t* partial_bytes, size_t* counter_bytes) {
    const uint32_t chunk = sdpa_chunk_len(qk_dim, v_dim, false);
    const uint32_t n_splits = (max_len + chunk - 1) / chunk;
    *partial_bytes = (size_t)n_heads * n_splits * (v_dim + 2) * sizeof(float);
    *counter_bytes = (size_t)n_heads * sizeof(uint32_t);  // >= n_kv * head tiles
    (void)n_kv;
    return FK_OK;
}

fk_status plan_sdpa_decode(const uint16_t* q, const uint16_t* k, const uint16_t* v, uint16_t* out,
                           const uint32_t* kv_len_ptr, uint32_t kv_len_imm, uint32_t max_len, uint32_t n_heads,
                           uint32_t n_kv, uint32_t qk_dim, uint32_t v_dim, uint32_t capacity, float scale,
                           float* partials, uint32_t* counters, Launch* out_launch, uint32_t rows,
                           const KvQuant* quant, const SdpaFusion* fusion) {
    const DeviceFacts* dev;
    FK_TRY(device_facts(&dev));
    if (!q || !k || !v || !out) return set_error(FK_ERR_INVALID, "sdpa: null tensor");
    if (n_kv == 0 || n_heads == 0 || n_heads % n_kv != 0)
        return set_error(FK_ERR_INVALID, "sdpa: n_heads must be a positive multiple of n_kv");
    if (qk_dim == 0 || v_dim == 0 || qk_dim % 8 || v_dim % 8 || qk_dim > 512 || v_dim > 512)
        return set_error(FK_ERR_UNSUPPORTED, "sdpa: head dims must be multiples of 8, at most 512");
    if (max_len == 0 || max_len > capacity) return set_error(FK_ERR_INVALID, "sdpa: kv length outside (0, capacity]");
    if (rows == 0 || rows > 1024) return set_error(FK_ERR_INVALID, "sdpa: 1..1024 active rows");
    const uint32_t kvq = quant ? quant->bits : 0u;
    if (kvq) {
        if (kvq != 4 && kvq != 8) return set_error(FK_ERR_UNSUPPORTED, "sdpa: quantised cache bits must be 4 or 8");
        if (!quant->k_scales || !quant->k_biases || !quant->v_scales || !quant->v_biases)
            return set_error(FK_ERR_INVALID, "sdpa: null cache scales / biases");
        const uint32_t g = quant->group;
        if ((g != 32 && g != 64 && g != 128) || qk_dim % g || v_dim % g)
            return set_error(FK_ERR_UNSUPPORTED, "sdpa: cache group size must be 32, 64 or 128 and divide the head dims");
    }
    if (fusion) {
        if (kvq || rows != 1) return set_error(FK_ERR_UNSUPPORTED, "sdpa: the fused rope/store form takes one row and a bf16 cache");
        if (!fusion->k_new || !fusion->v_new) return set_error(FK_ERR_INVALID, "sdpa: null new k / v row");
        if (fusion->rope_dims % 2 || fusion->rope_dims > qk_dim)
            return set_error(FK_ERR_INVALID, "sdpa: rope_dims must be even and within the head");
        if ((fusion->q_norm == nullptr) != (fusion->k_norm == nullptr))
            return set_error(FK_ERR_INVALID, "sdpa: q and k head norms come together");
        if (fusion->q0_dim) {
            if (fusion->q0_dim >= qk_dim || fusion->rope_dims > qk_dim - fusion->q0_dim || !fusion->k1_new || fusion->q_norm)
                return set_error(FK_ERR_INVALID, "sdpa: split heads need a second part that holds the rotated dims, a k1 row and no head norm");
            if (fusion->k0_stride < fusion->q0_dim || fusion->v_stride < v_dim || (fusion->k1_heads != 1 && fusion->k1_heads != n_kv))
                return set_error(FK_ERR_INVALID, "sdpa: split heads: strides below the row widths or a k1 head count other than 1 / n_kv");
            if ((fusion->v_stride * 2) % 16 || ((uintptr_t)fusion->v_new & 15u))
                return set_error(FK_ERR_INVALID, "sdpa: new value rows must be 16-byte aligned");
        }
    }
    if (!kv_len_ptr && rows > 1 && kv_len_imm + rows - 1 > max_len)
        return set_error(FK_ERR_INVALID, "sdpa: the last row's kv length exceeds max_len");
    if (!kv_len_ptr && (kv_len_imm == 0 || kv_len_imm > max_len))
        return set_error(FK_ERR_INVALID, "sdpa: kv_len outside (0, max_len]");
    const uint32_t chunk = sdpa_chunk_len(qk_dim, v_dim, false);
    const uint32_t n_chunks = (max_len + chunk - 1) / chunk;
    const uint32_t G = n_heads / n_kv;
    // Tiles of 1, 2 or 4 heads run the wave-local form, which needs a key row and its value row on
    // the same lanes (equal lanes per row); other shapes take the tile of 8, which goes through LDS.
    // Rows of different widths (192 / 128) both take the lane count of the wider one -- the spare
    // lanes of the narrower row idle -- as long as a row fits a wave; bf16 caches only.
    const uint32_t lpk0 = pow2_ceil(qk_dim / 8), lpv0 = pow2_ceil(v_dim / 8), lp_wide = lpk0 > lpv0 ? lpk0 : lpv0;
    const bool same_lanes = lpk0 == lpv0 || (!kvq && lp_wide <= (uint32_t)kWave);
    int gt = !same_lanes ? 8 : (G >= 8 ? 8 : (G >= 4 ? (G == 4 ? 4 : 8) : (G >= 2 ? (G == 2 ? 2 : 4) : 1)));
    // Groups of 2 .. 4 query heads per KV head: smaller tiles mean more blocks with fewer registers each, and the
    // repeated K / V reads of a KV head's tiles hit the L2.  Measured (32 q / 8 kv heads x 128, cold caches), tiles
    // of 1 / 2 / 4 heads: 512 positions 7.9 / 8.5 / 9.1 us, 4096 16.5 / 14.6 / 16.0, 32768 53.8 / 42.0 / 41.7;
    // the 4B decode loop at context 64 .. 576: 568 / 566 / 550 tokens/s.
    // (a quantised cache keeps its larger tile beyond 2048 positions: int4 at 32768 ran 41.4 us with 4 heads, 44.4 with 2)
    if (same_lanes && G >= 2 && G <= 4) gt = max_len <= 2048 ? 1 : (kvq ? gt : 2);
    // Long contexts: a block walks several consecutive ranges (online softmax, the next
    // range's rows in flight), so that the grid stays near one to two blocks per CU and
    // the final merge, which costs one memory round trip per 16 partials, stays short.
    // Measured (32 q / 8 kv heads x 128): 4096 positions are fastest with 32 splits,
    // 32768 with 64.
    // (several active rows multiply the tiles: each row then needs fewer ranges to fill the chip; 8 rows x 16 heads at
    // a capacity of 1024 ran 16 ranges per row and head -- 2048 blocks, most of them past the context -- in 14.4 us)
    const uint32_t tiles = n_kv * ((G + gt - 1) / gt) * rows;
    uint32_t want = (n_chunks > 128 ? 2u : 1u) * (uint32_t)dev->cus / tiles;
    if (want < 1) want = 1;
    if (want > 256) want = 256;
    const uint32_t cpb = (n_chunks + want - 1) / want;
    const uint32_t n_splits = (n_chunks + cpb - 1) / cpb;
    if (n_splits > 1 && (!partials || !counters))
        return set_error(FK_ERR_INVALID, "sdpa: workspace required when the context spans several ranges");

    SdpaArgs a;
    memset(&a, 0, sizeof(a));
    a.q = q; a.k = k; a.v = v; a.out = out;
    a.kv_len_ptr = kv_len_ptr;
    a.kv_len_imm = kv_len_imm;
    a.n_heads = n_heads; a.n_kv = n_kv; a.qk_dim = qk_dim; a.v_dim = v_dim; a.capacity = capacity;
    a.chunk_len = chunk;
    a.n_splits = n_splits;
    a.chunks_per_block = cpb;
    a.rows = rows;
    if (kvq) {
        a.k_scales = quant->k_scales; a.k_biases = quant->k_biases;
        a.v_scales = quant->v_scales; a.v_biases = quant->v_biases;
        a.kv_group = quant->group;
    }
    if (fusion) {
        a.k_new = fusion->k_new; a.v_new = fusion->v_new;
        a.q_norm = fusion->q_norm; a.k_norm = fusion->k_norm;
        a.cache_k_w = const_cast<uint16_t*>(k);
        a.cache_v_w = const_cast<uint16_t*>(v);
        a.rope_dims = fusion->rope_dims;
        a.eps = fusion->eps; a.base_log2 = fusion->base_log2;
        a.rope_tab = fusion->rope_tab;
        a.k1_new = fusion->k1_new;
        a.q0_dim = fusion->q0_dim; a.k0_stride = fusion->k0_stride; a.k1_heads = fusion->k1_heads;
        a.traditional = fusion->traditional;
        a.v_stride = fusion->q0_dim ? fusion->v_stride : v_dim;
    }
    a.lpk = gt <= 4 ? lp_wide : lpk0;
    a.lpv = gt <= 4 ? lp_wide : lpv0;
    a.scale = scale;
    a.partials = partials;
    a.counters = counters;

    const void* func = nullptr;
#define FK_SDPA_PICK(Q)                                                                         \
    switch (gt) {                                                                               \
        case 1: func = reinterpret_cast<const void*>(&sdpa_decode_kernel<1, Q>); break;         \
        case 2: func = reinterpret_cast<const void*>(&sdpa_decode_kernel<2, Q>); break;         \
        case 4: func = reinterpret_cast<const void*>(&sdpa_decode_kernel<4, Q>); break;         \
        default: func = reinterpret_cast<const void*>(&sdpa_decode_kernel<8, Q>); break;        \
    }
    if (fusion) {
        // whole-width rotation of at most 128 dims with a table: the form whose loads run ahead
        const bool fast = fusion->rope_tab && fusion->rope_dims == qk_dim && qk_dim <= 128;
#define FK_SDPA_FUSED(F)                                                                           \
    switch (gt) {                                                                                  \
        case 1: func = reinterpret_cast<const void*>(&sdpa_rope_store_kernel<1, F>); break;        \
        case 2: func = reinterpret_cast<const void*>(&sdpa_rope_store_kernel<2, F>); break;        \
        case 4: func = reinterpret_cast<const void*>(&sdpa_rope_store_kernel<4, F>); break;        \
        default: func = reinterpret_cast<const void*>(&sdpa_rope_store_kernel<8, F>); break;       \
    }
        if (fast) {
            FK_SDPA_FUSED(true)
        } else {
            FK_SDPA_FUSED(false)
        }
#undef FK_SDPA_FUSED
    } else if (kvq == 4) {
        FK_SDPA_PICK(4)
    } else if (kvq == 8) {
        FK_SDPA_PICK(8)
    } else {
        FK_SDPA_PICK(0)
    }
#undef FK_SDPA_PICK
    out_launch->func = func;
    out_launch->grid = dim3(n_splits, n_kv, ((G + gt - 1) / gt) * rows);
    out_launch->block = dim3(kSdpaBlock, 1, 1);
    out_launch->shmem = (uint32_t)(sdpa_lds_floats(gt, chunk, qk_dim, v_dim, fusion != nullptr) * sizeof(float));
    out_launch->set_args(a);
    return FK_OK;
}

}  // namespace fk
