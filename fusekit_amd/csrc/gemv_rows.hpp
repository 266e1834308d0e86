// Row-group GEMV for gfx950: the steady-state form of the weight-streaming GEMV for rows that are a whole number of
// 256-byte blocks (16 chunks of 16 bytes).
//
// Sixteen adjacent lanes share a row, a wave works on four consecutive rows at a time (a "pass"), and a lane walks
// its row in steps of 16 chunks: column block i of the row is chunks 16 i .. 16 i + 15, one per lane, so a wave load
// is four contiguous 256-byte pieces.  Each lane keeps ONE fp32 accumulator for its row across all its chunks; the
// row's sum is a 16-lane DPP butterfly at the end of the pass.  Against the flat-stream form (gemv_kernel.hpp)
// this removes, per chunk, the partial's trip through LDS, the row-sum phase with its two block barriers per
// tile, and every per-chunk address computation: a lane's LDS addresses (staged activations in the BLOCKED layout
// of stage_activations, chunk sums, scales and biases) are one lane constant plus a per-batch scalar plus
// compile-time offsets.  Waves of a block share only the staged activations; after staging they never meet again.
//
// Scales and biases: a column block of a row spans `16 >> gshift` quantisation groups, one short contiguous run of
// each array (16 bytes for int4 g64, 8 for int8 g64).  Lane s of a row's sixteen fetches the scales of the batch's
// column block s and lane 8 + s its biases, ONE vector memory instruction per batch beside the NB weight loads;
// the lane parks its vector in a wave-private LDS slot, and every lane then reads the 16-bit entry
// of its own chunk's group.  LDS operations of one wave execute in order, so no barrier is involved.
//
// Batches (NB column blocks of one pass) are double-buffered in registers: batch k + 1 is requested before batch k
// is consumed.  Work is dealt to waves pass by pass: pass (k * gridDim.x + block) * 4 + wave.
#pragma once
#include <type_traits>

#include "argmax_tail.hpp"
#include "gemv_kernel.hpp"

namespace fk {

constexpr int kRowLanes = 16;                 // lanes per row
constexpr int kPassRows = kWave / kRowLanes;  // rows per wave and pass
constexpr int kBlockWaves = kGemvBlock / kWave;

template <WKind KIND>
struct RowsMeta {  // bf16: no scales
    using vec = uint32_t;
    static constexpr uint32_t kGshift = 0;
};
template <>
struct RowsMeta<W_Q4> {  // group 64 = 2 chunks: 8 groups per column block
    using vec = uint4;
    static constexpr uint32_t kGshift = 1;
};
template <>
struct RowsMeta<W_Q8> {  // group 64 = 4 chunks: 4 groups per column block
    using vec = uint2;
    static constexpr uint32_t kGshift = 2;
};

// LDS: staged activations, chunk sums, block_sum scratch, one metadata slot per lane (a row's sixteen slots are
// followed by 16 bytes of padding, so that the four rows of a wave read their entries from different banks).
template <WKind KIND>
__host__ __device__ inline uint32_t gemv_rows_lds_bytes(uint32_t cpr) {
    const uint32_t meta = KIND == W_BF16 ? 0u : (uint32_t)(kGemvBlock * sizeof(typename RowsMeta<KIND>::vec) + kGemvBlock);
    return ChunkTraits<KIND>::kPieces * cpr * 16u + cpr * 4u + 64u + meta;
}

// One chunk against its staged activations (pieces 16 uint4 apart); returns the raw dot for the quantised kinds
// (the caller applies scale and bias) and acc + dot for bf16.
template <WKind KIND>
__device__ __forceinline__ float rows_chunk_dot(uint4 wv, const uint4* xp, float acc) {
    if constexpr (KIND == W_Q4) {
        float d0 = 0.f, d1 = 0.f;
        d0 = q4_word_dot(wv.x, xp[0], d0);
        d1 = q4_word_dot(wv.y, xp[16], d1);
        d0 = q4_word_dot(wv.z, xp[32], d0);
        d1 = q4_word_dot(wv.w, xp[48], d1);
        return d0 + d1;
    } else if constexpr (KIND == W_Q8) {
        float d0 = 0.f, d1 = 0.f;
        d0 = q8_word_dot(wv.x, xp[0], d0);
        d1 = q8_word_dot(wv.y, xp[16], d1);
        d0 = q8_word_dot(wv.z, xp[32], d0);
        d1 = q8_word_dot(wv.w, xp[48], d1);
        return d0 + d1;
    } else {
        const uint4 x = xp[0];
        acc = dot2_bf16(wv.x, x.x, acc);
        acc = dot2_bf16(wv.y, x.y, acc);
        acc = dot2_bf16(wv.z, x.z, acc);
        acc = dot2_bf16(wv.w, x.w, acc);
        return acc;
    }
}

// GemvArgs as the flat form reads them (one matrix, R = kPassRows, n_tiles = number of passes); no projection bias
// and no residual: their per-row loads at the end of a pass would have to be waited for together with everything
// issued before them, the next batch included.  The matrix, its scales and its y are addressed with 32-bit offsets
// and K is at most kStageRegs * kGemvBlock * 8 (the planner checks both).
// TAIL: a row's column blocks are not a multiple of NB, so a row's last batch has unused slots; they repeat the
// row's last column block with scale and bias zero (bf16: their result is dropped).
//
// The loop body is straight-line as far as memory requests go: a branch around a request makes the compiler wait
// for EVERY outstanding load where the paths join, which would serialise the prefetch.  A wave that has run out of
// passes therefore still issues its NB + 1 requests once more, all lanes at the first bytes of the arrays.
//
// ARGMAX: the rows are logits and the launch also selects the greedy token (argmax_tail.hpp): a lane keeps the best
// (value, row) candidate of the rows it has stored, on the bf16 value it stored, and the block hands its best to
// argmax_block_finish once its waves have run out of passes -- the only block barrier after staging.
struct GemvArgmaxArgs : GemvArgs {
    ArgmaxTail tail;
};

template <WKind KIND, int NB, bool TAIL, bool ARGMAX = false>
__global__ __launch_bounds__(kGemvBlock) void gemv_rows_kernel(const uint16_t* x, const uint16_t* norm_w, uint32_t K,
                                                               const std::conditional_t<ARGMAX, GemvArgmaxArgs, GemvArgs> a) {
    extern __shared__ uint4 lds_raw[];
    constexpr int PIECES = ChunkTraits<KIND>::kPieces;
    constexpr bool QUANT = KIND != W_BF16;
    using MV = typename RowsMeta<KIND>::vec;
    constexpr uint32_t MB = sizeof(MV);
    constexpr uint32_t GSH = RowsMeta<KIND>::kGshift;
    constexpr uint32_t GPB = 16u >> GSH;  // groups per column block

    uint4 xr[kStageRegs], wr[kStageRegs];
    stage_fetch(StageLead{x, norm_w, K}, xr, wr);  // from the leading parameters: before the argument block arrives
    kernarg_warm<24 + (int)sizeof(a)>();

    const uint32_t lane = threadIdx.x & (kWave - 1), l16 = lane & (kRowLanes - 1), rg = lane / kRowLanes;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    const uint32_t cpr = a.cpr, cpl = cpr / kRowLanes, gpr = cpr >> GSH, n = a.n[0];
    const uint32_t n_pass = a.n_tiles, stride = gridDim.x * kBlockWaves;
    const char* wbase = reinterpret_cast<const char*>(a.w[0]);
    uint16_t* ybase = a.y[0];

    uint4* xs = lds_raw;
    float* sx = reinterpret_cast<float*>(xs + PIECES * cpr);
    float* scratch = sx + cpr;
    constexpr uint32_t ROW_SLOTS = kRowLanes * MB + 16;  // bytes of a row's slots, padded
    char* meta = reinterpret_cast<char*>(scratch + 16) + wave * (kPassRows * ROW_SLOTS);
    const uint4* x_lane = xs + l16;
    const float* sx_lane = sx + l16;
    char* meta_wr = meta + rg * ROW_SLOTS + l16 * MB;                        // this lane's slot
    const char* meta_rd = meta + rg * ROW_SLOTS + (l16 >> GSH) * 2u;        // scales; biases 8 * MB further
    const uint32_t ms = (l16 & 7u) < (uint32_t)NB ? (l16 & 7u) : 0u;         // the column block whose run this lane fetches
    const uint16_t* marr = (l16 & 8u) ? a.bi[0] : a.sc[0];

    // A lane's request addresses, as offsets from the arrays' starts: its row (rows past the matrix repeat the last
    // one) times the row pitch, plus its place in column block 0; the batch's column block is added when it is issued.
    uint32_t pass = blockIdx.x * kBlockWaves + wave, cb = 0;  // the batch being consumed
    const bool any = pass < n_pass;
    auto row_of = [&](uint32_t p) {
        const uint32_t r = p * kPassRows + rg;
        return r < n ? r : n - 1;
    };
    uint32_t row = row_of(any ? pass : 0u);  // of the batch being ISSUED
    auto issue = [&](uint32_t row_i, uint32_t cb_i, bool live, uint4(&wv)[NB], MV& mv) {
        const uint32_t w_off = live ? ((row_i * cpr + l16) << 4) + cb_i * (kRowLanes * 16) : 0u;
#pragma unroll
        for (int s = 0; s < NB; ++s) {
            uint32_t i = s;
            if constexpr (TAIL) i = cb_i + s < cpl ? s : cpl - 1 - cb_i;
            if (!live) i = 0;
            wv[s] = *reinterpret_cast<const uint4*>(wbase + w_off + i * (kRowLanes * 16));
        }
        if constexpr (QUANT) {
            uint32_t mi = ms;
            if constexpr (TAIL) mi = cb_i + ms < cpl ? ms : cpl - 1 - cb_i;
            const uint32_t m_off = live ? row_i * gpr + (cb_i + mi) * GPB : 0u;
            mv = *reinterpret_cast<const MV*>(marr + m_off);
        }
    };

    uint4 wa[NB], wb[NB];
    MV ma, mb;
    issue(row, 0, any, wa, ma);  // weights stream while x is staged

    stage_activations<KIND, GemvArgs, true, true>(a, xs, sx, scratch, xr, wr);
    // The staging code consumes its loads under lane conditions; an unconditional use here tells the compiler that
    // every one of them has arrived (otherwise the loop below waits, each time it first reuses one of those
    // registers, as if the load were still outstanding -- and with it for the batch just requested).
#pragma unroll
    for (int i = 0; i < kStageRegs; ++i) asm volatile("" ::"v"(xr[i].x), "v"(wr[i].x));
    if constexpr (!ARGMAX) {
        if (!any) return;
    }

    float acc = 0.f;
    [[maybe_unused]] uint64_t best = 0;
    // Value and offset of the last output stored.  Stores and loads complete in issue order on one counter, so
    // overwriting a store's registers before the loads issued ahead of it have been waited for anyway would make
    // the compiler wait for all of those loads early, before the next batch is requested: the two are kept alive
    // (the empty asm statements below) until the next batch's natural wait has passed.
    uint32_t held_v = 0, held_o = 0;
    // Consumes the batch in (cur, mcur) while the next one streams into (nxt, mnxt); false once the wave is done.
    auto step = [&](uint4(&cur)[NB], MV& mcur, uint4(&nxt)[NB], MV& mnxt) -> bool {
        const bool wrap = cb + NB >= cpl;
        const uint32_t npass = wrap ? pass + stride : pass, ncb = wrap ? 0u : cb + NB;
        const bool live = npass < n_pass;
        const uint32_t row_c = row;  // the consumed batch's row
        row = row_of(live ? npass : 0u);
        issue(row, ncb, live, nxt, mnxt);

        if constexpr (QUANT) {
            MV mw = mcur;
            if constexpr (TAIL) {
                if (cb + ms >= cpl) mw = MV{};  // unused slot: scale and bias zero
            }
            *reinterpret_cast<MV*>(meta_wr) = mw;
            __builtin_amdgcn_wave_barrier();
            asm volatile("" ::"v"(held_v), "v"(held_o));
        }
        const uint4* xb = x_lane + cb * (PIECES * 16);
        const float* sxb = sx_lane + cb * 16;
#pragma unroll
        for (int s = 0; s < NB; ++s) {
            // (an unused slot's scale and bias are zero, but 0 * inf would poison the row: its activation block
            // is clamped like its weights instead of reading whatever lies behind the staged activations)
            uint32_t xo = s;
            if constexpr (TAIL) xo = cb + s < cpl ? s : cpl - 1 - cb;
            if constexpr (QUANT) {
                const float d = rows_chunk_dot<KIND>(cur[s], xb + xo * (PIECES * 16), 0.f);
                const float sc = bf16_bits_to_f32(*reinterpret_cast<const uint16_t*>(meta_rd + s * MB));
                const float bi = bf16_bits_to_f32(*reinterpret_cast<const uint16_t*>(meta_rd + (8 + s) * MB));
                acc = fmaf(sc, d, fmaf(bi, sxb[xo * 16], acc));
            } else {
                const float v = rows_chunk_dot<KIND>(cur[s], xb + xo * (PIECES * 16), acc);
                if constexpr (TAIL)
                    acc = cb + s < cpl ? v : acc;
                else
                    acc = v;
                if (s == 0) asm volatile("" ::"v"(held_v), "v"(held_o));
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        if constexpr (QUANT) __builtin_amdgcn_wave_barrier();  // the next batch's slot writes stay behind these reads

        if (wrap && pass < n_pass) {
            const float total = group_sum(acc, kRowLanes);
            held_v = f32_to_bf16_bits(total);
            held_o = row_c * 2u;
            // Every lane of the row stores the (same) value, and the lanes of a row past the matrix have computed
            // its last row once more, bit for bit: no lane condition, hence no divergent branch inside the loop
            // (one would make the compiler restructure the whole loop around a single exit, and the paths it
            // then has to assume make it wait for the newest batch where it need not).
            *reinterpret_cast<uint16_t*>(reinterpret_cast<char*>(ybase) + held_o) = (uint16_t)held_v;
            if constexpr (ARGMAX) {
                const uint64_t cand = argmax_candidate(held_v, row_c);
                best = cand > best ? cand : best;
            }
            acc = 0.f;
        }
        pass = npass;
        cb = ncb;
        return live;
    };
    // One exit per pair of steps: with an exit between the two, the compiler routes both through one latch block
    // and must then assume, at the loop's top, that the batch requested by the first step may still be in flight
    // in the registers it is about to reuse -- it waits for it, and the prefetch is gone.  A wave with an odd
    // number of batches therefore consumes one dead batch (requested with live = false) whose result is dropped.
    bool more = any;
    while (more) {
        step(wa, ma, wb, mb);
        more = step(wb, mb, wa, ma);
    }
    if constexpr (ARGMAX) {
        __shared__ uint64_t best_of_wave[kBlockWaves];
        __shared__ uint32_t is_last;
        argmax_block_finish<kGemvBlock>(a.tail, best, best_of_wave, &is_last);
    }
}

}  // namespace fk
