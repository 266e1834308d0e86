// Flat-stream weight-streaming GEMV for gfx950 (batch-1 decode).
//
// The weight matrix is read as one flat sequence of 16-byte chunks, so every
// wave load is 1 KiB of contiguous HBM whatever K is.  A chunk holds 32 int4,
// 16 int8 or 8 bf16 weights of one row and always lies inside one quantization
// group.  Activations are staged once per (persistent) block into LDS in a
// chunk-interleaved layout -- piece j of chunk c at uint4 index j*cpr + c -- so
// that lanes walking consecutive chunks read consecutive 16-byte LDS words.
// Each lane turns its chunk into one fp32 partial, partials of a tile of R rows
// go through LDS, and a second phase adds each row's partials in a fixed order
// and applies the epilogue.  No atomics touch the value path.
//
// int4 dequantisation costs 7 VALU ops per packed word (two masks, one shift,
// four fp8->bf16 pair converts, see q4_word_dot) plus four v_dot2c_f32_bf16; the
// affine bias folds into one per-chunk term b * Sx, Sx being the chunk's
// activation sum (computed once per block).
#pragma once
#include "fk_device.hpp"

// Hook for timing probes: a build may define FK_GEMV_STAMP(i) to record a clock at
// phase boundary i; the library build leaves it empty.
#ifndef FK_GEMV_STAMP
#define FK_GEMV_STAMP(i)
#endif

namespace fk {

enum WKind : int { W_Q4 = 0, W_Q8 = 1, W_BF16 = 2 };

constexpr int kGemvBlock = 256;
constexpr int kGemvUnroll = 4;  // 16-byte loads in flight per lane and batch
constexpr int kMaxMats = 3;

struct GemvArgs {
    const uint4* w[kMaxMats];
    const uint16_t* sc[kMaxMats];
    const uint16_t* bi[kMaxMats];
    const uint16_t* bias[kMaxMats];  // optional bf16 projection bias per matrix
    uint16_t* y[kMaxMats];
    uint32_t n[kMaxMats];           // rows per matrix
    uint32_t tile_start[kMaxMats + 1];  // first tile of each matrix (fan-out mode)
    uint32_t n_mats;
    uint32_t K;
    uint32_t cpr;      // 16-byte chunks per row
    uint32_t gshift;   // chunk index >> gshift = quantization group index
    uint32_t R;        // rows per tile (per segment)
    uint32_t n_tiles;
    uint32_t lr;       // lanes per row in the row-sum phase (power of two)
    float inv_cpr;
    const uint16_t* x;       // bf16 activations [K]
    const uint16_t* norm_w;  // fused RMSNorm weight or null
    float eps;
    const uint16_t* res;   // optional residual (matrix 0)
    const uint16_t* res2;  // optional second residual
    int swiglu_variant;
    float y_scale;  // SwiGLU variant 1 only: multiplies the fp32 product before the final round
};

template <WKind KIND>
struct ChunkTraits;
template <>
struct ChunkTraits<W_Q4> {
    static constexpr int kValues = 32, kPieces = 4;
};
template <>
struct ChunkTraits<W_Q8> {
    static constexpr int kValues = 16, kPieces = 4;
};
template <>
struct ChunkTraits<W_BF16> {
    static constexpr int kValues = 8, kPieces = 1;
};

// LDS bytes the kernel needs: staged activations + per-chunk sums + partials + scratch.
template <WKind KIND>
__host__ __device__ inline uint32_t gemv_lds_bytes(uint32_t cpr, uint32_t seg_chunks, uint32_t nseg) {
    const uint32_t pos = kGemvBlock * (kGemvUnroll / nseg);
    const uint32_t seg_pad = (seg_chunks + pos - 1) / pos * pos;
    return ChunkTraits<KIND>::kPieces * cpr * 16u + cpr * 4u + nseg * seg_pad * 4u + 64u;
}

__device__ __forceinline__ float q8_word_dot(uint32_t w, uint4 xf, float d) {
    d = fmaf((float)(w & 0xffu), __uint_as_float(xf.x), d);
    d = fmaf((float)((w >> 8) & 0xffu), __uint_as_float(xf.y), d);
    d = fmaf((float)((w >> 16) & 0xffu), __uint_as_float(xf.z), d);
    d = fmaf((float)(w >> 24), __uint_as_float(xf.w), d);
    return d;
}

// One chunk -> one fp32 partial.
template <WKind KIND>
__device__ __forceinline__ float chunk_partial(uint4 wv, uint32_t s_bits, uint32_t b_bits, const uint4* xs,
                                               const float* sx, uint32_t c, uint32_t cpr) {
    if constexpr (KIND == W_Q4) {
        float d0 = 0.f, d1 = 0.f;  // two chains keep the dot unit busy
        d0 = q4_word_dot(wv.x, xs[c], d0);
        d1 = q4_word_dot(wv.y, xs[cpr + c], d1);
        d0 = q4_word_dot(wv.z, xs[2 * cpr + c], d0);
        d1 = q4_word_dot(wv.w, xs[3 * cpr + c], d1);
        const float s = bf16_bits_to_f32(s_bits), b = bf16_bits_to_f32(b_bits), sum_x = sx[c];
        return fmaf(s, d0 + d1, b * sum_x);
    } else if constexpr (KIND == W_Q8) {
        float d0 = 0.f, d1 = 0.f;
        d0 = q8_word_dot(wv.x, xs[c], d0);
        d1 = q8_word_dot(wv.y, xs[cpr + c], d1);
        d0 = q8_word_dot(wv.z, xs[2 * cpr + c], d0);
        d1 = q8_word_dot(wv.w, xs[3 * cpr + c], d1);
        const float s = bf16_bits_to_f32(s_bits), b = bf16_bits_to_f32(b_bits);
        return fmaf(s, d0 + d1, b * sx[c]);
    } else {
        const uint4 xp = xs[c];
        float d = 0.f;
        d = dot2_bf16(wv.x, xp.x, d);
        d = dot2_bf16(wv.y, xp.y, d);
        d = dot2_bf16(wv.z, xp.z, d);
        d = dot2_bf16(wv.w, xp.w, d);
        return d;
    }
}

// SwiGLU epilogue on the two fp32 accumulators; the three rounding variants the
// reference emits (rmsnorm_gateup_swiglu.rs:236-257, msl.rs:1286-1294, msl.rs:2441-2449).
__device__ __forceinline__ uint32_t swiglu_bits(float acc_g, float acc_u, int variant, float y_scale) {
    const float g = round_bf16(acc_g), u = round_bf16(acc_u);
    if (variant == 0) {
        const float e = round_bf16(expf(fabsf(g)));
        const float den = round_bf16(1.0f + e);
        const float sig_y = round_bf16(1.0f / den);
        const float sig = (g < 0.0f) ? sig_y : round_bf16(1.0f - sig_y);
        const float silu = round_bf16(g * sig);
        return f32_to_bf16_bits(silu * u);
    } else if (variant == 1) {
        const float sig = 1.0f / (1.0f + expf(-g));
        return f32_to_bf16_bits(((sig * g) * u) * y_scale);  // routed_qmv_swiglu.rs:420-446 (1.0 elsewhere)
    } else {
        const float sig = round_bf16(1.0f / (1.0f + expf(-g)));
        const float gated = round_bf16(sig * g);
        return f32_to_bf16_bits(gated * u);
    }
}

// Stage x (optionally RMS-normalised: T(w * T(x * r))) into the chunk-interleaved
// LDS layout and compute the per-chunk sums.  Every thread handles 8 consecutive
// elements per step; the first kStageRegs steps stay in registers between the
// sum-of-squares pass and the write pass, so x and the norm weight are fetched
// once.  The threads that hold the pieces of one chunk are adjacent lanes, so the
// chunk sum is a 2- or 4-lane butterfly.  K must be a multiple of 64.
constexpr int kStageRegs = 5;

// Issues the loads of the register-resident part of x (and the norm weight).  A
// stand-alone kernel calls this BEFORE the weight prefetch: loads return in issue
// order, so x queued behind a batch of weight rows would wait for HBM although it
// sits in cache.
struct StageLead {  // what stage_fetch reads, as a kernel's leading parameters
    const uint16_t* x;
    const uint16_t* norm_w;
    uint32_t K;
};
template <typename ARGS>
__device__ __forceinline__ void stage_fetch(const ARGS& a, uint4 (&xr)[kStageRegs], uint4 (&wr)[kStageRegs]) {
    // Straight-line on purpose (clamped index, the norm weight replaced by x itself
    // when there is none): with branches around the loads the compiler falls back to
    // waiting for every outstanding load, weight prefetch included.
    const uint32_t n8 = a.K >> 3;
    const uint4* x8 = reinterpret_cast<const uint4*>(a.x);
    const uint4* w8 = a.norm_w ? reinterpret_cast<const uint4*>(a.norm_w) : x8;
#pragma unroll
    for (int i = 0; i < kStageRegs; ++i) {
        const uint32_t t = threadIdx.x + i * kGemvBlock;
        const uint32_t tc = t < n8 ? t : 0u;
        xr[i] = x8[tc];
        wr[i] = w8[tc];
    }
}

// BLOCKED: the layout of the row-group kernel (gemv_rows.hpp): piece j of chunk c at uint4 index
// ((c / 16) * PIECES + j) * 16 + c % 16, so that the 16 lanes sharing a row read 256 contiguous bytes and a
// chunk's pieces sit at fixed distances from each other.
// SHORT: the caller guarantees K <= kStageRegs * kGemvBlock * 8, so the loops over the rest of a long row are
// left out (their loads, conditional and issued after the caller's prefetch, blur the compiler's account of which
// registers still have a load outstanding).
template <WKind KIND, typename ARGS, bool BLOCKED = false, bool SHORT = false>
__device__ __forceinline__ void stage_activations(const ARGS& a, uint4* xs, float* sx, float* scratch,
                                                  uint4 (&xr)[kStageRegs], uint4 (&wr)[kStageRegs]) {
    const bool NORM = a.norm_w != nullptr;  // uniform; one code path serves both
    const uint32_t K = a.K, cpr = a.cpr, n8 = K >> 3;
    const uint4* x8 = reinterpret_cast<const uint4*>(a.x);
    const uint4* w8 = reinterpret_cast<const uint4*>(a.norm_w);
    float r = 1.0f;
    if (NORM) {
        float ss = 0.f;
        auto add_sq = [&](uint4 v) {
            const uint32_t p[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float lo = bf16_lo(p[i]), hi = bf16_hi(p[i]);
                ss = fmaf(lo, lo, ss);
                ss = fmaf(hi, hi, ss);
            }
        };
#pragma unroll
        for (int i = 0; i < kStageRegs; ++i)
            if (threadIdx.x + i * kGemvBlock < n8) add_sq(xr[i]);
        if constexpr (!SHORT)
            for (uint32_t t = threadIdx.x + kStageRegs * kGemvBlock; t < n8; t += kGemvBlock) add_sq(x8[t]);
        FK_GEMV_STAMP(5);
        ss = block_sum<kGemvBlock>(ss, scratch);
        r = 1.0f / sqrtf(ss / (float)K + a.eps);
        FK_GEMV_STAMP(6);
    }
    auto emit = [&](uint32_t t, uint4 v, uint4 wv) {
        // nb: the staged values as bf16 pairs in element order (0,1) (2,3) (4,5) (6,7).  With the
        // norm each pair takes two packed conversions: T(x * r), then T(w * that).
        uint32_t nb[4] = {v.x, v.y, v.z, v.w};
        if (NORM) {
            const uint32_t q[4] = {wv.x, wv.y, wv.z, wv.w};
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const uint32_t xr_ = pack_bf16(bf16_lo(nb[i]) * r, bf16_hi(nb[i]) * r);
                nb[i] = pack_bf16(bf16_lo(q[i]) * bf16_lo(xr_), bf16_hi(q[i]) * bf16_hi(xr_));
            }
        }
        float f[8];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            f[2 * i] = bf16_lo(nb[i]);
            f[2 * i + 1] = bf16_hi(nb[i]);
        }
        float s8 = ((f[0] + f[1]) + (f[2] + f[3])) + ((f[4] + f[5]) + (f[6] + f[7]));
        const bool live = t < n8;
        if constexpr (KIND == W_Q4) {
            // word j of chunk c; activation pairs (0,2) (4,6) (1,3) (5,7) as q4_word_dot wants
            const uint32_t c = t >> 2, j = t & 3u;
            if (live)
                xs[BLOCKED ? ((c >> 4) * 4 + j) * 16 + (c & 15u) : j * cpr + c] =
                                  make_uint4(__builtin_amdgcn_perm(nb[1], nb[0], 0x05040100u),
                                             __builtin_amdgcn_perm(nb[3], nb[2], 0x05040100u),
                                             __builtin_amdgcn_perm(nb[1], nb[0], 0x07060302u),
                                             __builtin_amdgcn_perm(nb[3], nb[2], 0x07060302u));
            s8 = group_sum(s8, 4);  // the four lanes that hold the words of one chunk
            if (live && j == 0) sx[c] = s8;
        } else if constexpr (KIND == W_Q8) {
            const uint32_t c = t >> 1, j = (t & 1u) * 2u;
            if (live) {
                const uint32_t at = BLOCKED ? ((c >> 4) * 4 + j) * 16 + (c & 15u) : j * cpr + c;
                xs[at] = make_uint4(__float_as_uint(f[0]), __float_as_uint(f[1]), __float_as_uint(f[2]),
                                    __float_as_uint(f[3]));
                xs[at + (BLOCKED ? 16u : cpr)] = make_uint4(__float_as_uint(f[4]), __float_as_uint(f[5]),
                                                            __float_as_uint(f[6]), __float_as_uint(f[7]));
            }
            s8 = group_sum(s8, 2);
            if (live && j == 0) sx[c] = s8;
        } else {
            if (live) xs[t] = make_uint4(nb[0], nb[1], nb[2], nb[3]);
        }
    };
    // whole waves past the end skip the step (the chunk-sum butterflies need whole waves)
#pragma unroll
    for (int i = 0; i < kStageRegs; ++i)
        if ((threadIdx.x & ~(uint32_t)(kWave - 1)) + i * kGemvBlock < n8) emit(threadIdx.x + i * kGemvBlock, xr[i], wr[i]);
    // long rows: the rest is fetched again (whole waves stay in the loop so the
    // butterflies above see all their lanes)
    if constexpr (!SHORT) {
        const uint32_t n8_up = (n8 + kWave - 1) / kWave * kWave;
        for (uint32_t t = threadIdx.x + kStageRegs * kGemvBlock; t < n8_up; t += kGemvBlock) {
            uint4 v = make_uint4(0, 0, 0, 0), wv = make_uint4(0, 0, 0, 0);
            if (t < n8) {
                v = x8[t];
                if (NORM) wv = w8[t];
            }
            emit(t, v, wv);
        }
    }
    FK_GEMV_STAMP(7);
    __syncthreads();
}

// Per-tile facts, uniform over the block (scalar registers).
template <int NSEG>
struct GemvTile {
    const char* w[NSEG];
    const char* sc[NSEG];
    const char* bi[NSEG];
    uint32_t m, row0, valid;
};

// ARGS is GemvArgs (kernel argument) or a constant-address-space view of one that
// lives in device memory; either way the fields are read through scalar loads.
template <WKind KIND, int NSEG, typename ARGS>
__device__ __forceinline__ GemvTile<NSEG> gemv_tile(const ARGS& a, uint32_t tile) {
    GemvTile<NSEG> t;
    const uint32_t R = a.R, cpr = a.cpr;
    if constexpr (NSEG == 2) {
        t.m = 0;
        t.row0 = tile * R;
    } else {
        t.m = (a.n_mats > 1 && tile >= a.tile_start[1]) ? ((a.n_mats > 2 && tile >= a.tile_start[2]) ? 2u : 1u) : 0u;
        t.row0 = (tile - a.tile_start[t.m]) * R;
    }
    const uint32_t left = a.n[t.m] - t.row0;
    t.valid = left < R ? left : R;
    const size_t base = (size_t)t.row0 * cpr;
#pragma unroll
    for (int sg = 0; sg < NSEG; ++sg) {
        const uint32_t mm = (NSEG == 2) ? (uint32_t)sg : t.m;
        t.w[sg] = reinterpret_cast<const char*>(a.w[mm] + base);
        if constexpr (KIND != W_BF16) {
            t.sc[sg] = reinterpret_cast<const char*>(a.sc[mm] + (base >> a.gshift));
            t.bi[sg] = reinterpret_cast<const char*>(a.bi[mm] + (base >> a.gshift));
        }
    }
    return t;
}

// Issues the 16-byte weight loads (and scale/bias) of one batch into registers.
// Slot j belongs to segment j / SLOTS, so every slot's base pointer is uniform
// and the per-lane part of the address is a 32-bit byte offset.  Straight-line:
// positions outside the tile's valid rows read chunk 0 of the tile instead
// (always in bounds); their partials are never consumed.
template <WKind KIND, int NSEG, typename ARGS>
__device__ __forceinline__ void gemv_load_batch(const ARGS& a, uint4 (&wv)[kGemvUnroll],
                                                uint32_t (&sc)[kGemvUnroll], uint32_t (&bi)[kGemvUnroll],
                                                uint32_t tile, uint32_t b0) {
    constexpr int SLOTS = kGemvUnroll / NSEG;
    const GemvTile<NSEG> t = gemv_tile<KIND, NSEG, ARGS>(a, tile);
    const uint32_t valid_chunks = t.valid * a.cpr;
#pragma unroll
    for (int j = 0; j < kGemvUnroll; ++j) {
        const int sg = j / SLOTS;
        const uint32_t pos = b0 + (j % SLOTS) * kGemvBlock + threadIdx.x;
        const uint32_t idx = pos < valid_chunks ? pos : 0u;
        wv[j] = *reinterpret_cast<const uint4*>(t.w[sg] + (idx << 4));
        if constexpr (KIND != W_BF16) {
            const uint32_t goff = (idx >> a.gshift) << 1;
            sc[j] = *reinterpret_cast<const uint16_t*>(t.sc[sg] + goff);
            bi[j] = *reinterpret_cast<const uint16_t*>(t.bi[sg] + goff);
        }
    }
}

// First batch of this block's first tile: pure weight traffic, independent of the
// activations, so a caller may issue it before x exists (before a grid barrier).
template <WKind KIND, int NSEG, typename ARGS>
__device__ __forceinline__ void gemv_prefetch(const ARGS& a, uint32_t block_id, uint4 (&wv)[kGemvUnroll],
                                              uint32_t (&sc)[kGemvUnroll], uint32_t (&bi)[kGemvUnroll]) {
    if (block_id < a.n_tiles) gemv_load_batch<KIND, NSEG, ARGS>(a, wv, sc, bi, block_id, 0);
}

// The block's share of one GEMV: tiles block_id, block_id + n_blocks, ...
// (wa, sa, ba) must hold the batch gemv_prefetch loaded for the same arguments.
//
// NSEG = 1: fan-out over up to three matrices sharing x (plain GEMV, QKV,
//           residual projections, LM head); each tile lies inside one matrix.
// NSEG = 2: gate/up pair; a tile holds R gate rows and the same R up rows and
//           the epilogue is SwiGLU.
// COH: the outputs will be read by other blocks of the same launch, so they are
// stored write-through (see st_u16).  The inputs need nothing special as long as
// the caller guarantees that no block has read their addresses earlier in this
// launch (the whole-token kernel gives every layer its own activation buffers).
template <WKind KIND, int NSEG, bool COH, typename ARGS>
__device__ __forceinline__ void gemv_run(const ARGS& a, uint32_t block_id, uint32_t n_blocks, uint4* lds_raw,
                                         uint4 (&wa)[kGemvUnroll], uint32_t (&sa)[kGemvUnroll],
                                         uint32_t (&ba)[kGemvUnroll], uint4 (&xr)[kStageRegs],
                                         uint4 (&wr)[kStageRegs]) {
    constexpr int PIECES = ChunkTraits<KIND>::kPieces;
    constexpr int SLOTS = kGemvUnroll / NSEG;                // register slots per segment and batch
    constexpr uint32_t POS = kGemvBlock * SLOTS;             // chunk positions of a segment per batch
    const uint32_t cpr = a.cpr, R = a.R;
    const uint32_t seg_chunks = R * cpr;                     // chunks of one segment of a full tile
    const uint32_t seg_pad = (seg_chunks + POS - 1) / POS * POS;

    uint4* xs = lds_raw;
    float* sx = reinterpret_cast<float*>(xs + PIECES * cpr);
    float* part = sx + cpr;                                  // [NSEG][seg_pad]
    float* scratch = part + NSEG * seg_pad;

    // Column (chunk within its row) of each slot's position; advanced per batch
    // instead of dividing by cpr for every chunk.
    uint32_t col0[SLOTS], col[SLOTS];
#pragma unroll
    for (int jj = 0; jj < SLOTS; ++jj) {
        const uint32_t pos = jj * kGemvBlock + threadIdx.x;
        const uint32_t row = (uint32_t)(((float)pos + 0.5f) * a.inv_cpr);
        col0[jj] = col[jj] = pos - row * cpr;
    }
    const uint32_t col_step = POS % cpr;

    uint32_t tile = block_id, b0 = 0;
    bool first_batch = true;  // probe builds only: marks the first batch for FK_GEMV_STAMP

    // Consumes the batch held in cur* while the following batch streams into nxt*.
    // Returns false once this block has no tile left.  (Two copies of this body,
    // one per register set, cost code size but no register moves and no spills.)
    auto step = [&](uint4(&cur)[kGemvUnroll], uint32_t(&csc)[kGemvUnroll], uint32_t(&cbi)[kGemvUnroll],
                    uint4(&nxt)[kGemvUnroll], uint32_t(&nsc)[kGemvUnroll], uint32_t(&nbi)[kGemvUnroll]) -> bool {
        uint32_t ntile = tile, nb0 = b0 + POS;
        if (nb0 >= seg_chunks) {
            ntile = tile + n_blocks;
            nb0 = 0;
        }
        if (ntile < a.n_tiles) gemv_load_batch<KIND, NSEG, ARGS>(a, nxt, nsc, nbi, ntile, nb0);

        float p[kGemvUnroll];
#pragma unroll
        for (int j = 0; j < kGemvUnroll; ++j) {
            p[j] = chunk_partial<KIND>(cur[j], csc[j], cbi[j], xs, sx, col[j % SLOTS], cpr);
            // Keep the scheduler from hoisting every chunk's LDS reads to the top
            // (that costs ~200 VGPRs); other waves hide the LDS latency instead.
            __builtin_amdgcn_sched_barrier(0);
        }
        if (first_batch) FK_GEMV_STAMP(3);
        first_batch = false;
        // `part` is padded to whole batches, so the store needs no guard (a guard
        // would let the compiler sink all the arithmetic into the branch).
#pragma unroll
        for (int j = 0; j < kGemvUnroll; ++j)
            part[(j / SLOTS) * seg_pad + b0 + (j % SLOTS) * kGemvBlock + threadIdx.x] = p[j];

        if (ntile != tile) {
            // tile complete: add each row's partials in a fixed order, then the epilogue
            __syncthreads();
            const GemvTile<NSEG> t = gemv_tile<KIND, NSEG, ARGS>(a, tile);
            const uint32_t lr = a.lr, lane = threadIdx.x & (lr - 1);
            for (uint32_t rr = threadIdx.x / lr; rr < R; rr += kGemvBlock / lr) {
                float s0 = 0.f, s1 = 0.f;
                uint32_t i_first = lane;
                if constexpr (NSEG == 1) {
                    // the first eight partials of a lane are read in one go (clamped positions, masked additions in the
                    // loop's order, so the sums keep their bits): one trip to the LDS instead of one per partial
                    // (4864 x 896 int4: 4.59 -> 4.50 us; with the gate / up pair's two sums it gained nothing)
                    float v0[8];
#pragma unroll
                    for (int k = 0; k < 8; ++k) {
                        const uint32_t i = lane + (uint32_t)k * lr;
                        v0[k] = part[rr * cpr + (i < cpr ? i : 0u)];
                    }
#pragma unroll
                    for (int k = 0; k < 8; ++k) s0 += lane + (uint32_t)k * lr < cpr ? v0[k] : 0.f;
                    i_first = lane + 8u * lr;
                }
                for (uint32_t i = i_first; i < cpr; i += lr) {
                    s0 += part[rr * cpr + i];
                    if constexpr (NSEG == 2) s1 += part[seg_pad + rr * cpr + i];
                }
                s0 = group_sum(s0, lr);
                if constexpr (NSEG == 2) s1 = group_sum(s1, lr);
                if (lane == 0 && rr < t.valid) {
                    const uint32_t n = t.row0 + rr, m = t.m;
                    if constexpr (NSEG == 2) {
                        st_u16<COH>(a.y[0] + n, swiglu_bits(s0, s1, a.swiglu_variant, a.y_scale));
                    } else {
                        float v = s0;
                        if (a.bias[m]) v += bf16_bits_to_f32(a.bias[m][n]);
                        if (m == 0 && a.res) v += bf16_bits_to_f32(a.res[n]);
                        uint32_t o = f32_to_bf16_bits(v);
                        if (m == 0 && a.res2)
                            o = f32_to_bf16_bits(bf16_bits_to_f32(o) + bf16_bits_to_f32(a.res2[n]));
                        st_u16<COH>(a.y[m] + n, o);
                    }
                }
            }
            __syncthreads();
#pragma unroll
            for (int jj = 0; jj < SLOTS; ++jj) col[jj] = col0[jj];
        } else {
#pragma unroll
            for (int jj = 0; jj < SLOTS; ++jj) {
                const uint32_t c = col[jj] + col_step;
                col[jj] = c >= cpr ? c - cpr : c;
            }
        }
        tile = ntile;
        b0 = nb0;
        return tile < a.n_tiles;
    };

    uint4 wb[kGemvUnroll];
    uint32_t sb[kGemvUnroll], bb[kGemvUnroll];
    FK_GEMV_STAMP(1);
    stage_activations<KIND, ARGS>(a, xs, sx, scratch, xr, wr);
    FK_GEMV_STAMP(2);
    if (block_id >= a.n_tiles) return;
    while (true) {
        if (!step(wa, sa, ba, wb, sb, bb)) break;
        if (!step(wb, sb, bb, wa, sa, ba)) break;
    }
    FK_GEMV_STAMP(4);
}

// Form for callers whose activations do not exist yet when the weights are
// prefetched (the whole-token kernel prefetches across a grid barrier).
template <WKind KIND, int NSEG, bool COH, typename ARGS>
__device__ __forceinline__ void gemv_run(const ARGS& a, uint32_t block_id, uint32_t n_blocks, uint4* lds_raw,
                                         uint4 (&wa)[kGemvUnroll], uint32_t (&sa)[kGemvUnroll],
                                         uint32_t (&ba)[kGemvUnroll]) {
    uint4 xr[kStageRegs], wr[kStageRegs];
    stage_fetch(a, xr, wr);
    gemv_run<KIND, NSEG, COH, ARGS>(a, block_id, n_blocks, lds_raw, wa, sa, ba, xr, wr);
}

// x, norm_w and K also travel as LEADING parameters: those reach a wave in registers at its launch (kernel argument
// preload), so the activations are requested before the argument block -- one trip to memory away -- has arrived.
template <WKind KIND, int NSEG>
__global__ __launch_bounds__(kGemvBlock) void gemv_stream_kernel(const uint16_t* x, const uint16_t* norm_w, uint32_t K,
                                                                 const GemvArgs a) {
    extern __shared__ uint4 lds_raw[];
    uint4 wa[kGemvUnroll];
    uint32_t sa[kGemvUnroll], ba[kGemvUnroll];
    uint4 xr[kStageRegs], wr[kStageRegs];
    FK_GEMV_STAMP(0);
    stage_fetch(StageLead{x, norm_w, K}, xr, wr);          // activations first: they return first
    kernarg_warm<24 + (int)sizeof(GemvArgs)>();
    gemv_prefetch<KIND, NSEG>(a, blockIdx.x, wa, sa, ba);  // weights stream while x is staged
    gemv_run<KIND, NSEG, false>(a, blockIdx.x, gridDim.x, lds_raw, wa, sa, ba, xr, wr);
}

}  // namespace fk
