// Device-side building blocks of the XCD-resident launches (xcd_layer.hip, xcd_moe.hip): the hand-over inside an XCD,
// the input of a launch (sum row + residual, RMSNorm, staging), projection tiles streamed by 256 threads, row sums.
// The planners' shared host helpers follow at the end.  Everything is internal to the including file.  The includer defines FK_XCD_STAMP(k, i) first (a timing probe, empty
// in the library build).
#pragma once
#include "xcd_layer.hpp"

namespace fk {
namespace {

constexpr int kBlock = kGemvBlock;  // 256 threads

__device__ __forceinline__ uint32_t xcc_id() {
    uint32_t v;
    asm volatile("s_getreg_b32 %0, hwreg(HW_REG_XCC_ID)" : "=s"(v));
    return v & 0xfu;
}

// ---- hand-over inside an XCD ------------------------------------------------------------------
struct XcdSync {
    XcdControl* ctl;
    uint32_t xcd, slot, epoch, spin_limit;
    bool aborted;
};

// Ordinary stores of this block that other blocks of the XCD will read must have been acknowledged before
// the flag is published: every wave waits for its own memory counter, the block barrier collects the
// waves, thread 0 publishes.  Wave 0 then polls the XCD's 64 flag words (one per lane, L1-bypassing
// loads that are served by the XCD's L2) until every one has reached the epoch.
// One wave publishes this block's arrival (its stores of the stage must be complete) and polls the XCD's 64
// flag words, one per lane, until every block has reached the epoch; returns false when it gave up.
__device__ __forceinline__ bool xcd_publish_and_wait(const XcdSync& s, uint32_t lane) {
    uint32_t* flags = s.ctl->flags + s.xcd * kXcdSlots;
    if (lane == 0) __hip_atomic_store(flags + s.slot, s.epoch, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    uint32_t spins = 0;
    for (;;) {
        const uint32_t v = __hip_atomic_load(flags + lane, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (__all((int)((int32_t)(v - s.epoch) >= 0))) return true;
        ++spins;
        if ((spins & 255u) == 0u && __hip_atomic_load(&s.ctl->abort_flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0u)
            return false;
        if (spins > s.spin_limit) {
            if (lane == 0) __hip_atomic_store(&s.ctl->abort_flag, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            return false;
        }
        __builtin_amdgcn_s_sleep(1);
    }
}

// Whole block; the wave that starts at thread POLL publishes and polls.  `okw`: one word of LDS through which that
// wave tells the block how the wait ended: 0 when it gave up or another block had raised the abort word.  The caller
// reads the word after the barrier (xcd_wait_ok) and, once it is 0, does nothing that outlives the launch -- no cache
// append, no addition into a sum row -- with values built from rows that were never finished.  Where nothing of that
// kind follows at once, the word is read at the barrier and tested only in front of those effects, so that the LDS
// round trip is not on the path.
template <int POLL>
__device__ __forceinline__ void xcd_barrier(XcdSync& s, uint32_t* okw) {
    s.epoch += 1;
    wait_memory_ops_done();
    __syncthreads();
    if (threadIdx.x >= POLL && threadIdx.x < POLL + kWave) {
        const bool ok = xcd_publish_and_wait(s, threadIdx.x - POLL);
        if (threadIdx.x == POLL) *okw = ok ? 1u : 0u;
    }
    __syncthreads();
}
__device__ __forceinline__ bool xcd_wait_ok(const uint32_t* okw) { return *reinterpret_cast<const volatile uint32_t*>(okw) != 0u; }

// Last thing a block does in a launch that was asked to (parameter mark_placement: one launch per token is enough to
// watch how the device deals workgroups, and the memory-side operation at the very end of EVERY launch cost 0.1-0.3 us
// each): flip its bit of its XCD's placement word (see XcdControl).
__device__ __forceinline__ void xcd_mark_placement(const XcdSync& s, uint32_t wanted) {
    if (wanted && threadIdx.x == 0)
        (void)__hip_atomic_fetch_xor(&s.ctl->placement[s.xcd].bits, 1ull << s.slot, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// ---- activation staging (the chunk-interleaved LDS layout of the streaming GEMV) -------------------
// Group t holds elements 8t .. 8t+7 of the vector: v = their bf16 bits, wv the norm weights' (NORM).
// With NORM the staged value is T(w * T(x * r)) (src/codegen/kernels/mod.rs:4464-4472).  Every lane of a
// wave must call this together (the chunk sums are quad butterflies); `live` masks lanes past the end.
template <WKind KIND>
__device__ __forceinline__ void stage_emit(uint4* xs, float* sx, uint32_t cs, uint32_t t, bool live, uint4 v, uint4 wv,
                                           float r, bool NORM) {
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
    if constexpr (KIND == W_Q4) {
        const uint32_t c = t >> 2, j = t & 3u;
        if (live)
            xs[j * cs + c] = make_uint4(__builtin_amdgcn_perm(nb[1], nb[0], 0x05040100u),
                                        __builtin_amdgcn_perm(nb[3], nb[2], 0x05040100u),
                                        __builtin_amdgcn_perm(nb[1], nb[0], 0x07060302u),
                                        __builtin_amdgcn_perm(nb[3], nb[2], 0x07060302u));
        s8 = group_sum(s8, 4);
        if (live && j == 0) sx[c] = s8;
    } else if constexpr (KIND == W_Q8) {
        const uint32_t c = t >> 1, j = (t & 1u) * 2u;
        if (live) {
            xs[j * cs + c] = make_uint4(__float_as_uint(f[0]), __float_as_uint(f[1]), __float_as_uint(f[2]),
                                        __float_as_uint(f[3]));
            xs[(j + 1) * cs + c] = make_uint4(__float_as_uint(f[4]), __float_as_uint(f[5]), __float_as_uint(f[6]),
                                              __float_as_uint(f[7]));
        }
        s8 = group_sum(s8, 2);
        if (live && j == 0) sx[c] = s8;
    } else {
        if (live) xs[t] = make_uint4(nb[0], nb[1], nb[2], nb[3]);
    }
}

// A vector of n8 groups of 8 bf16 values that other blocks of this XCD wrote: L1-bypassing loads, staged as is.
template <WKind KIND>
__device__ __forceinline__ void stage_vector(const uint16_t* src, uint32_t n8, uint32_t cs, uint4* xs, float* sx) {
    const uint4* s8 = reinterpret_cast<const uint4*>(src);
    const uint32_t n8_up = (n8 + kWave - 1) / kWave * kWave;
    for (uint32_t t = threadIdx.x; t < n8_up; t += kBlock) {
        const bool live = t < n8;
        const uint4 v = ld_u128<true>(s8 + (live ? t : 0u));
        stage_emit<KIND>(xs, sx, cs, t, live, v, v, 1.0f, false);
    }
}

// ---- the input of a launch -------------------------------------------------------------------
//   x = T(f32(sum row) + residual) for the WHOLE vector (every block computes all of it: one round trip, no
//   hand-over), its sum of squares, then T(w * T(x * r)) staged into LDS for the projections.
// Thread t of the block takes the groups of eight elements t and t + 256 (hidden <= 4096).  The requests go out
// first (input_request), the block's first weight requests behind them, then the values are used (input_stage).
constexpr int kInGroups = 2;
constexpr int kGuAhead = 3;  // gate requests of the MLP launch that go out ahead of its input's staging

__device__ __forceinline__ float xcd_sum_to_f32(uint32_t lo, uint32_t hi) {
    return fmaf((float)lo, kXcdSumInv, (float)(int32_t)hi);
}
__device__ __forceinline__ void xcd_sum_add(long long* row, uint32_t e, float v, XcdControl* ctl) {
    // beyond the fixed-point range, or not finite: clamp and tell the host (branch-free but for the rare store)
    const bool bad = !(fabsf(v) < kXcdSumLimit);
    v = v != v ? 0.f : fminf(fmaxf(v, -kXcdSumLimit), kXcdSumLimit);
    if (__any((int)bad)) {
        if (bad) __hip_atomic_store(&ctl->overflow, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    const long long q = __float2ll_rn(v * kXcdSumScale);
    (void)__hip_atomic_fetch_add(reinterpret_cast<unsigned long long*>(row) + xcd_sum_index(e), (unsigned long long)q,
                                 __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

struct InputRegs {
    uint4 sv[kInGroups][4], rv[kInGroups], nw[kInGroups];
};

// What input_request reads of a launch's input, as leading kernel parameters: they reach a wave in registers when it
// starts (kernel argument preload), so the sum row is requested before the argument block -- one trip to memory
// away -- has arrived.
struct XcdInputLead {
    const long long* sums;
    const uint16_t* residual;
    const uint16_t* norm_w;
    uint32_t hidden;
};

// Zeroes the sum row the launch after this one adds into (16-byte units spread over the grid).  Called once the
// input has been consumed: a wave's memory counter completes in order, and in the whole-token launch these are
// write-through stores (a line left dirty in this XCD's L2 would later overwrite the other XCDs' additions) that
// take a trip to memory.
template <bool TOKEN, typename IN>
__device__ __forceinline__ void input_clear(const IN& in) {
    if (!in.clear) return;
    const uint32_t u = blockIdx.x * kBlock + threadIdx.x;
    if (u < in.row_elems / 2) {
        if constexpr (TOKEN) {
            unsigned long long* c = reinterpret_cast<unsigned long long*>(in.clear) + 2 * (size_t)u;
            __hip_atomic_store(c, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __hip_atomic_store(c + 1, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        } else {
            reinterpret_cast<uint4*>(in.clear)[u] = make_uint4(0, 0, 0, 0);
        }
    }
}

// TOKEN: the launch runs every layer of a token (xcd_token_kernel).  The sum row was then written memory-side by
// other XCDs earlier in the SAME launch: it is read with L1-bypassing loads.  `xres`, if given, is the block's own
// copy of the residual row in LDS (every block computes the whole row in every phase).
template <bool TOKEN, typename IN>
__device__ __forceinline__ void input_request(const IN& in, InputRegs& r, const uint4* xres) {
    const uint32_t n8 = in.hidden >> 3, lane = threadIdx.x & (kWave - 1);
    const uint4* s16 = reinterpret_cast<const uint4*>(in.sums);
    const uint4* r8 = reinterpret_cast<const uint4*>(in.residual);
    const uint4* w8 = reinterpret_cast<const uint4*>(in.norm_w);
#pragma unroll
    for (int i = 0; i < kInGroups; ++i) {
        const uint32_t t = threadIdx.x + i * kBlock, sec = t >> 6;  // the wave's section of 64 groups
        if (sec * kWave < n8) {                                      // wave-uniform
            const uint32_t tc = t < n8 ? t : 0u;
            if (in.sums) {
#pragma unroll
                for (int k = 0; k < 4; ++k) r.sv[i][k] = ld_u128<TOKEN>(s16 + (sec * 4 + k) * kWave + lane);  // padded row: in bounds
            }
            r.rv[i] = (TOKEN && xres) ? xres[tc] : r8[tc];
            r.nw[i] = w8[tc];
        }
    }
}

// Placed behind the LAST request of a launch's start-up, before input_stage.  input_request and input_stage test
// the same (wave-uniform) conditions, and without this the compiler merges the two regions: the conversion of the
// sum row ends up directly behind its loads, inside the first condition, and the wave then sits out a whole trip
// to memory -- twice, once per group -- before it requests the residual, the scales and biases and its first pass
// of weights.  The empty statement makes every input register a value that exists only from here on, so the
// arithmetic cannot move ahead of the requests in between.
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
__device__ __forceinline__ void pin128(uint4& v) {  // as ONE 128-bit register operand: the load's tuple stays whole
    u32x4_t t = {v.x, v.y, v.z, v.w};
    asm volatile("" : "+v"(t));
    v = make_uint4(t.x, t.y, t.z, t.w);
}
template <typename IN>
__device__ __forceinline__ void input_pin(const IN& in, InputRegs& r) {
    const uint32_t n8 = in.hidden >> 3;
#pragma unroll
    for (int i = 0; i < kInGroups; ++i) {
        const uint32_t t = threadIdx.x + i * kBlock, sec = t >> 6;
        if (sec * kWave < n8) {  // as in input_request / input_stage: registers of a skipped group hold nothing
            if (in.sums) {
#pragma unroll
                for (int k = 0; k < 4; ++k) pin128(r.sv[i][k]);
            }
            pin128(r.rv[i]);
            pin128(r.nw[i]);
        }
    }
}

// Whole block (two block barriers inside); `red`: 4 floats of LDS; `xres_out` (LDS, or null): where the block keeps
// the row for the next phase of the same launch.
template <WKind KIND, int PROBE, typename IN>
__device__ __forceinline__ void input_stage(const IN& in, const InputRegs& r, uint4* xs, float* sx, uint32_t cs,
                                            float* red, uint4* xres_out = nullptr) {
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
                if (xres_out) xres_out[t] = xv[i];
            }
        }
    }
    FK_XCD_STAMP(PROBE, 2);
    sq = wave_sum(sq);
    if ((threadIdx.x & (kWave - 1)) == 0) red[threadIdx.x / kWave] = sq;
    __syncthreads();
    sq = (red[0] + red[1]) + (red[2] + red[3]);
    const float rr = 1.0f / sqrtf(sq / (float)in.hidden + in.eps);
    FK_XCD_STAMP(PROBE, 3);
#pragma unroll
    for (int i = 0; i < kInGroups; ++i) {
        const uint32_t t = threadIdx.x + i * kBlock, sec = t >> 6;
        if (sec * kWave < n8) stage_emit<KIND>(xs, sx, cs, t, t < n8, xv[i], r.nw[i], rr, true);
    }
    __syncthreads();
}

// ---- projection tiles ----------------------------------------------------------------------------
// A tile: rows [row0, row0 + rows) x chunks [col0, col0 + cs) of a matrix; flat position p = row * cs + col.
// A pass covers NL * 256 positions; positions past the tile read the tile's first chunk (in bounds).
// Weights are requested as 16-byte chunks, one per lane and position (1 KiB contiguous per wave instruction).
// Scales and biases are NOT fetched per chunk (two more memory instructions per chunk, each as expensive to
// issue as the 16-byte one): the block fetches the tile's groups once, kMetaRegs per thread, and parks them
// in LDS as (scale | bias << 16) words.
template <int NL>
struct TileRegs {
    uint4 w[NL];
};
constexpr int kMetaRegs = 3;  // one-pass flavour: a tile holds at most 3 * 256 = 768 quantisation groups per matrix
// The flavour with the pass loop serves larger tiles (an 8B-class int4 gate / up tile is 28 rows x 64 groups): there a
// thread fetches a second run of four groups, 2048 per tile and matrix.
constexpr uint32_t kMetaWords = kMetaRegs * 256u, kMetaWordsBig = 8u * 256u;
template <bool ONE>
constexpr uint32_t meta_words() { return ONE ? kMetaWords : kMetaWordsBig; }
struct MetaRegs {
    uint32_t s[4], b[4];   // [0..1]: groups 4 ti .. 4 ti + 3; [2..3] (BIG): groups 4 (ti + SN) .. + 3
};

struct Tile {
    uint32_t row0, rows, col0, cs;
    float inv_cs;
};

// SN threads stream a tile; `ti` is the calling thread's index among them.  A thread's j-th position in pass p is
// pos = (p * NL + j) * SN + ti = row * cs + col.  The thread keeps, per j, the column (it addresses the staged
// activations) and the chunk's index in the matrix (the request); both are worked out once per tile and advanced
// from pass to pass without a multiplication.  The flat position itself indexes the partials, and pos >> gshift
// the tile's quantisation groups (cs is a whole number of groups).
template <int NL>
struct TilePos {
    uint32_t p0;            // position of j = 0
    uint32_t col[NL], gidx[NL];
};
template <int NL, int SN, typename MAT>
__device__ __forceinline__ void tile_pos_init(const MAT& m, const Tile& t, uint32_t ti, TilePos<NL>& p) {
    p.p0 = ti;
#pragma unroll
    for (int j = 0; j < NL; ++j) {
        const uint32_t pos = j * SN + ti;
        const uint32_t row = (uint32_t)(((float)pos + 0.5f) * t.inv_cs);
        p.col[j] = pos - row * t.cs;
        p.gidx[j] = (t.row0 + row) * m.cpr + t.col0 + p.col[j];
    }
}
template <int NL, int SN, typename MAT>
__device__ __forceinline__ void tile_pos_next(const MAT& m, const Tile& t, uint32_t step_c, uint32_t step_g, TilePos<NL>& p) {
    p.p0 += NL * SN;
    const uint32_t skip = m.cpr - t.cs;
#pragma unroll
    for (int j = 0; j < NL; ++j) {
        const uint32_t c = p.col[j] + step_c;
        const bool wrap = c >= t.cs;
        p.col[j] = wrap ? c - t.cs : c;
        p.gidx[j] += step_g + (wrap ? skip : 0u);
    }
}

template <WKind KIND, int NL, int SN, int J0 = 0, int J1 = NL, typename MAT>
__device__ __forceinline__ void tile_load(const MAT& m, const Tile& t, const TilePos<NL>& p, TileRegs<NL>& r) {
    const uint32_t total = t.rows * t.cs, first = t.row0 * m.cpr + t.col0;
#pragma unroll
    for (int j = J0; j < J1; ++j) r.w[j] = m.w[p.p0 + j * SN < total ? p.gidx[j] : first];
}

// Group gi of the tile = (row gi / gpr, group gi % gpr of the row's slice), gpr groups per row slice.
// A vector memory instruction costs the CU about as much to issue whether it moves 2 or 16 bytes per lane, so
// a tile of whole rows whose row holds a multiple of four groups (its groups are then one contiguous,
// 8-byte-aligned run of the scale and of the bias array) is fetched four groups per lane and instruction.
// RUN: the tile's groups are one contiguous, 8-byte aligned run of a multiple of four entries of the scale and of
// the bias array (the host plans it so): a tile of whole rows, or a K-slice tile of a matrix whose scales and
// biases were re-laid out per XCD (fk_xcd_kslice_meta: [xcd][row][groups of the slice]; `xcd` then selects the copy).
template <WKind KIND, int SN, bool RUN, bool BIG = false, typename MAT>
__device__ __forceinline__ void meta_fetch(const MAT& m, const Tile& t, uint32_t ti, MetaRegs& r, uint32_t xcd = 0) {
    if constexpr (KIND != W_BF16) {
        const uint32_t gpr = t.cs >> m.gshift, total = t.rows * gpr;
        const size_t g0 = t.cs == m.cpr ? (size_t)t.row0 * gpr : ((size_t)xcd * m.rows + t.row0) * gpr;
        if constexpr (RUN) {
            // kMetaRegs * SN groups at most: lane ti takes groups 4 ti .. 4 ti + 3 (s[0..1] / b[0..1] hold them)
            const uint32_t gi = 4u * ti;
            const size_t e = gi < total ? g0 + gi : g0;
            const uint2 sv = *reinterpret_cast<const uint2*>(m.sc + e), bv = *reinterpret_cast<const uint2*>(m.bi + e);
            r.s[0] = sv.x;
            r.s[1] = sv.y;
            r.b[0] = bv.x;
            r.b[1] = bv.y;
            if constexpr (BIG) {  // straight-line: a lane past the tile's groups repeats the first entries
                const uint32_t gi2 = 4u * (ti + (uint32_t)SN);
                const size_t e2 = gi2 < total ? g0 + gi2 : g0;
                const uint2 sv2 = *reinterpret_cast<const uint2*>(m.sc + e2), bv2 = *reinterpret_cast<const uint2*>(m.bi + e2);
                r.s[2] = sv2.x;
                r.s[3] = sv2.y;
                r.b[2] = bv2.x;
                r.b[3] = bv2.y;
            }
        } else {
            const float inv = 1.0f / (float)gpr;
#pragma unroll
            for (int k = 0; k < kMetaRegs; ++k) {
                const uint32_t gi = k * SN + ti;
                const uint32_t row = (uint32_t)(((float)gi + 0.5f) * inv);
                const size_t e = gi < total ? g0 + (size_t)row * (m.cpr >> m.gshift) + (gi - row * gpr) : g0;
                r.s[k] = m.sc[e];
                r.b[k] = m.bi[e];
            }
        }
    }
}
template <WKind KIND, int SN, bool RUN, bool BIG = false>
__device__ __forceinline__ void meta_store(const MetaRegs& r, uint32_t ti, uint32_t* meta) {
    if constexpr (KIND != W_BF16) {
        if constexpr (RUN) {
            if (BIG || 4u * ti < (uint32_t)kMetaRegs * SN)
                *reinterpret_cast<uint4*>(meta + 4u * ti) =
                    make_uint4((r.s[0] & 0xffffu) | (r.b[0] << 16), (r.s[0] >> 16) | (r.b[0] & 0xffff0000u),
                               (r.s[1] & 0xffffu) | (r.b[1] << 16), (r.s[1] >> 16) | (r.b[1] & 0xffff0000u));
            if constexpr (BIG)
                *reinterpret_cast<uint4*>(meta + 4u * (ti + (uint32_t)SN)) =
                    make_uint4((r.s[2] & 0xffffu) | (r.b[2] << 16), (r.s[2] >> 16) | (r.b[2] & 0xffff0000u),
                               (r.s[3] & 0xffffu) | (r.b[3] << 16), (r.s[3] >> 16) | (r.b[3] & 0xffff0000u));
        } else {
#pragma unroll
            for (int k = 0; k < kMetaRegs; ++k) meta[k * SN + ti] = r.s[k] | (r.b[k] << 16);
        }
    }
}

// One fp32 partial per chunk into part[pos]; positions past the tile land in the padding of `part` (it holds whole
// passes) and read group 0's scale and bias.
template <WKind KIND, int NL, int SN, typename MAT>
__device__ __forceinline__ void tile_partials(const MAT& m, const Tile& t, const TilePos<NL>& p, const TileRegs<NL>& r,
                                              const uint4* xs, const float* sx, const uint32_t* meta, float* part) {
    const uint32_t total = t.rows * t.cs;
#pragma unroll
    for (int j = 0; j < NL; ++j) {
        const uint32_t pos = p.p0 + j * SN;
        uint32_t sb = 0, bb = 0;
        if constexpr (KIND != W_BF16) {
            const uint32_t mw = meta[(pos < total ? pos : 0u) >> m.gshift];
            sb = mw & 0xffffu;
            bb = mw >> 16;
        }
        part[pos] = chunk_partial<KIND>(r.w[j], sb, bb, xs, sx, p.col[j], t.cs);
        __builtin_amdgcn_sched_barrier(0);
    }
}

// All passes of a tile whose first pass is already in `r0` (positions `p` at pass 0): pass k + 1 is requested
// before pass k is consumed.  `after_last_request` runs once the tile's last pass has been requested (the caller
// queues what it needs next behind it).
// ONE: the launch was planned with every tile within one pass; the loop (and the second set of registers it keeps)
// is then not compiled at all, and the waits for `r0` are counted with the caller's requests behind them.  (In the
// loop those requests sit under a condition; the compiler then counts without them, and every chunk of a pass also
// waits for as many of the caller's requests as the pass has chunks in flight -- at the end for all of them.  A
// run-time test for one pass inside this general form costs it registers: 26-31 spilled in the MLP kernel.)
template <WKind KIND, int NL, int SN, bool ONE = false, typename MAT, typename F>
__device__ __forceinline__ void tile_run(const MAT& m, const Tile& t, TilePos<NL>& p, TileRegs<NL>& r0, const uint4* xs,
                                         const float* sx, const uint32_t* meta, float* part, F after_last_request) {
    if constexpr (ONE) {
        after_last_request();  // (the o_proj slice: in front of or behind the arithmetic made no difference)
        tile_partials<KIND, NL, SN>(m, t, p, r0, xs, sx, meta, part);
        return;
    }
    const uint32_t n_pass = (t.rows * t.cs + NL * SN - 1) / (NL * SN);
    const uint32_t step_r = (NL * SN) / t.cs, step_c = (NL * SN) - step_r * t.cs, step_g = step_r * m.cpr + step_c;
    TileRegs<NL> r1;
    TilePos<NL> q = p;
    if (n_pass <= 1) after_last_request();
    for (uint32_t k = 0; k < n_pass; k += 2) {
        if (k + 1 < n_pass) {
            tile_pos_next<NL, SN>(m, t, step_c, step_g, q);
            tile_load<KIND, NL, SN>(m, t, q, r1);
            if (k + 2 >= n_pass) after_last_request();
        }
        tile_partials<KIND, NL, SN>(m, t, p, r0, xs, sx, meta, part);
        if (k + 1 < n_pass) {
            p = q;
            if (k + 2 < n_pass) {
                tile_pos_next<NL, SN>(m, t, step_c, step_g, q);
                tile_load<KIND, NL, SN>(m, t, q, r0);
                if (k + 3 >= n_pass) after_last_request();
            }
            tile_partials<KIND, NL, SN>(m, t, p, r1, xs, sx, meta, part);
            p = q;
        }
    }
}

// The gate / up pair: both matrices' passes interleaved, so that one pass of each is in flight while one is consumed.
// (Same shape and tile: one set of positions serves both.)
template <WKind KIND, int NL, int SN, bool ONE = false, typename MAT, typename F>
__device__ __forceinline__ void tile_run_pair(const MAT& ma, const MAT& mb, const Tile& t, TilePos<NL>& p,
                                              TileRegs<NL>& a0, TileRegs<NL>& b0, const uint4* xs, const float* sx,
                                              const uint32_t* meta_a, const uint32_t* meta_b, float* part_a, float* part_b,
                                              F after_last_request) {
    if constexpr (ONE) {
        // The caller's requests (the down_proj slice) go out BEHIND the arithmetic of both matrices: they are not
        // needed before the hand-over that follows, and in front they only lengthen the queue the gate / up chunks
        // stand in (4B int4, same box: in front 798 tok/s, between the two matrices 809, behind 821).
        tile_partials<KIND, NL, SN>(ma, t, p, a0, xs, sx, meta_a, part_a);
        tile_partials<KIND, NL, SN>(mb, t, p, b0, xs, sx, meta_b, part_b);
        after_last_request();
        return;
    }
    const uint32_t n_pass = (t.rows * t.cs + NL * SN - 1) / (NL * SN);
    const uint32_t step_r = (NL * SN) / t.cs, step_c = (NL * SN) - step_r * t.cs, step_g = step_r * ma.cpr + step_c;
    TileRegs<NL> a1, b1;
    TilePos<NL> q = p;
    if (n_pass <= 1) after_last_request();
    for (uint32_t k = 0; k < n_pass; k += 2) {
        if (k + 1 < n_pass) {
            tile_pos_next<NL, SN>(ma, t, step_c, step_g, q);
            tile_load<KIND, NL, SN>(ma, t, q, a1);
            tile_load<KIND, NL, SN>(mb, t, q, b1);
            if (k + 2 >= n_pass) after_last_request();
        }
        tile_partials<KIND, NL, SN>(ma, t, p, a0, xs, sx, meta_a, part_a);
        tile_partials<KIND, NL, SN>(mb, t, p, b0, xs, sx, meta_b, part_b);
        if (k + 1 < n_pass) {
            p = q;
            if (k + 2 < n_pass) {
                tile_pos_next<NL, SN>(ma, t, step_c, step_g, q);
                tile_load<KIND, NL, SN>(ma, t, q, a0);
                tile_load<KIND, NL, SN>(mb, t, q, b0);
                if (k + 3 >= n_pass) after_last_request();
            }
            tile_partials<KIND, NL, SN>(ma, t, p, a1, xs, sx, meta_a, part_a);
            tile_partials<KIND, NL, SN>(mb, t, p, b1, xs, sx, meta_b, part_b);
            p = q;
        }
    }
}

// Lanes that share a row in the row-sum phase: about four to eight partials per lane, at most 16 lanes (so that
// the cross-lane sum stays inside a 16-lane row of the wave).
__device__ __forceinline__ uint32_t lanes_per_row(uint32_t cs) {
    uint32_t lr = 1;
    while (lr < 16 && lr * 8 <= cs) lr <<= 1;
    return lr;
}

// Adds each row's partials in a fixed order; f(row, sum0, sum1) runs in one lane per row.
// ONCE (the one-pass flavour): when a row group of 16, 8, ... lanes covers every row of the tile in ONE round and a lane
// then holds at most ten partials per matrix, all its LDS reads go out first (clamped positions) and a row's epilogue
// runs once -- instead of rounds of a read-wait-add loop (gate / up rows of the 4B-class MLP launch: two rounds of
// sixteen lanes and five dependent LDS trips each took 1.65 us; one round of eight lanes 1.1).
template <bool TWO, bool ONCE = false, typename F>
__device__ __forceinline__ void tile_rows(const Tile& t, const float* part, const float* part1, F f) {
    if constexpr (ONCE) {
        // the widest row group (at most 16 lanes) with which every row of the tile fits one round
        uint32_t lr1 = 16;
        while (lr1 > 1 && t.rows * lr1 > (uint32_t)kBlock) lr1 >>= 1;
        if (t.rows * lr1 <= (uint32_t)kBlock && t.cs <= 10u * lr1) {
            const uint32_t lane1 = threadIdx.x & (lr1 - 1), rr = threadIdx.x / lr1;
            const bool ok = rr < t.rows;
            const uint32_t base = (ok ? rr : 0u) * t.cs;
            float v0[10], v1[10];
#pragma unroll
            for (int k = 0; k < 10; ++k) {
                const uint32_t i = lane1 + lr1 * k;
                const uint32_t at = base + (i < t.cs ? i : 0u);
                v0[k] = part[at];
                if constexpr (TWO) v1[k] = part1[at];
            }
            float s0 = 0.f, s1 = 0.f;
#pragma unroll
            for (int k = 0; k < 10; ++k) {
                const bool in = lane1 + lr1 * k < t.cs;
                s0 += in ? v0[k] : 0.f;
                if constexpr (TWO) s1 += in ? v1[k] : 0.f;
            }
            s0 = group_sum(s0, lr1);
            if constexpr (TWO) s1 = group_sum(s1, lr1);
            if (ok && lane1 == 0) f(rr, s0, s1);
            return;
        }
    }
    const uint32_t lr = lanes_per_row(t.cs), lane = threadIdx.x & (lr - 1);
    const uint32_t step = kBlock / lr, rows_up = (t.rows + step - 1) / step * step;
    auto one = [&](uint32_t rr) {
        const bool ok = rr < t.rows;
        float s0 = 0.f, s1 = 0.f;
        if (ok)
            for (uint32_t i = lane; i < t.cs; i += lr) {
                s0 += part[rr * t.cs + i];
                if constexpr (TWO) s1 += part1[rr * t.cs + i];
            }
        s0 = group_sum(s0, lr);
        if constexpr (TWO) s1 = group_sum(s1, lr);
        if (ok && lane == 0) f(rr, s0, s1);
    };
    // Up to two rounds (the 4B-class tiles) run straight-line: f stores to memory, and in front of a LOOP with
    // stores in it the compiler waits for every request still in flight -- here the next projection's weights,
    // requested just before, whose trip to memory the row sums and the hand-over are meant to cover.
    if (rows_up <= 2 * step) {
        one(threadIdx.x / lr);
        if (rows_up > step) one(threadIdx.x / lr + step);
        return;
    }
    for (uint32_t rr = threadIdx.x / lr; rr < rows_up; rr += step) one(rr);
}

// An empty tile (a block without work in this projection) still issues its loads, clamped to the tile's
// first chunk: it is moved to row 0 so that those loads stay inside the matrix.
__device__ __forceinline__ Tile make_tile(uint32_t row0, uint32_t rows, uint32_t col0, uint32_t cs) {
    Tile t;
    t.row0 = rows ? row0 : 0u;
    t.rows = rows;
    t.col0 = col0;
    t.cs = cs;
    t.inv_cs = 1.0f / (float)cs;
    return t;
}

// LDS layout shared by both kernels (floats unless noted):
//   xs   uint4 [PIECES * cs_max]      staged activations
//   sx   [cs_max]                     per-chunk sums
//   work [work_floats]                chunk partials of a tile (two segments for gate / up), or the attention's LDS
//   meta uint32 [3][kMetaRegs * 256]  (scale | bias << 16) of the groups of up to three tiles
//   att  uint16 [att_elems]           merged attention rows (attention launch)
//   scratch [16]
struct LdsPlan {
    uint32_t cs_max, work_floats, att_elems;
    uint32_t meta_words;   // per matrix: kMetaWords (one-pass flavour) or kMetaWordsBig
};
static_assert(kBlock == 256, "the metadata areas are sized for 256 streaming threads");
template <WKind KIND>
__host__ __device__ inline uint32_t xcd_lds_bytes(const LdsPlan& p) {
    return ChunkTraits<KIND>::kPieces * p.cs_max * 16u + p.cs_max * 4u + p.work_floats * 4u + 3u * p.meta_words * 4u +
           ((p.att_elems * 2u + 15u) & ~15u) + 64u;
}

// One of two matrices, chosen by a block-uniform condition.  Field by field, so that the choice stays in scalar
// registers (a reference chosen between two members of the argument block makes the compiler copy both to private
// memory).
__device__ __forceinline__ XcdMat pick_mat(bool first, const XcdMat& a, const XcdMat& b) {
    XcdMat m;
    m.w = first ? a.w : b.w;
    m.sc = first ? a.sc : b.sc;
    m.bi = first ? a.bi : b.bi;
    m.rows = first ? a.rows : b.rows;
    m.cpr = first ? a.cpr : b.cpr;
    m.gshift = first ? a.gshift : b.gshift;
    return m;
}

// Workgroups are dealt to the XCDs round-robin, starting wherever the previous dispatch stopped: the XCD is read
// from the hardware, and workgroups i and i + 8 land on the same XCD, so i / 8 numbers the 64 blocks of each XCD.
// (Were the dealing ever different, two blocks would share a flag word, a hand-over wait would run into its spin
// limit and the launch would report it.)
__device__ __forceinline__ XcdSync xcd_sync_init(XcdControl* ctl, uint32_t spin_limit) {
    XcdSync sync;
    sync.ctl = ctl;
    sync.xcd = xcc_id() & (kXcds - 1);
    sync.slot = blockIdx.x / kXcds;
    sync.spin_limit = spin_limit;
    sync.aborted = false;
    sync.epoch = __hip_atomic_load(ctl->flags + sync.xcd * kXcdSlots + sync.slot, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    return sync;
}

// ---- host side: what the planners of these launches share ------------------------------------
inline uint32_t ilog2u(uint32_t v) {
    uint32_t r = 0;
    while ((1u << (r + 1)) <= v) ++r;
    return r;
}
inline uint32_t ceil_div(uint32_t a, uint32_t b) { return (a + b - 1) / b; }
inline uint32_t chunk_values(uint32_t bits) { return bits == 4 ? 32u : (bits == 8 ? 16u : 8u); }

inline fk_status bind_mat(const fk_weight* w, uint32_t n, uint32_t k, const XcdLayerShape& s, XcdMat* m, const char* what) {
    if (!w || !w->w) return set_error(FK_ERR_INVALID, std::string("xcd layer: null weight ") + what);
    if (w->n != n || w->k != k || w->bits != s.bits || (s.bits != 16 && w->group != s.group))
        return set_error(FK_ERR_INVALID, std::string("xcd layer: weight ") + what + " does not match the layer shape");
    if (s.bits != 16 && (!w->scales || !w->biases)) return set_error(FK_ERR_INVALID, std::string("xcd layer: null scales / biases of ") + what);
    if (((uintptr_t)w->w & 15u) || (s.bits != 16 && (((uintptr_t)w->scales | (uintptr_t)w->biases) & 7u)))
        return set_error(FK_ERR_INVALID, std::string("xcd layer: ") + what + " needs 16-byte aligned weights and 8-byte aligned scales / biases");
    m->w = reinterpret_cast<const uint4*>(w->w);
    m->sc = w->scales;
    m->bi = w->biases;
    m->rows = n;
    m->cpr = k / chunk_values(s.bits);
    m->gshift = s.bits == 16 ? 0 : ilog2u(s.group / chunk_values(s.bits));
    return FK_OK;
}

inline fk_status fill_input(const XcdLayerShape& s, const long long* sums, const uint16_t* residual, uint16_t* x_out,
                     long long* clear, const long long* out_sums, const uint16_t* norm_w, float eps, XcdInput* in) {
    if (!residual || !x_out || !norm_w) return set_error(FK_ERR_INVALID, "xcd layer: null residual, x_out or norm weight");
    if (residual == x_out) return set_error(FK_ERR_INVALID, "xcd layer: x_out must not be the residual row");
    if (out_sums == sums || out_sums == clear || (clear && clear == sums))
        return set_error(FK_ERR_INVALID, "xcd layer: the sum rows read, added into and cleared must be three different rows");
    in->sums = sums;
    in->residual = residual;
    in->x_out = x_out;
    in->clear = clear;
    in->norm_w = norm_w;
    in->eps = eps;
    in->hidden = s.hidden;
    in->row_elems = xcd_sum_row_elems(s.hidden);
    return FK_OK;
}

inline fk_status set_lds_limit(const void* func, uint32_t lds) {
    const DeviceFacts* dev;
    FK_TRY(device_facts(&dev));
    if ((int)lds > dev->max_dyn_lds) return set_error(FK_ERR_UNSUPPORTED, "xcd layer: LDS need exceeds the CU");
    if (lds > 48 * 1024) FK_HIP(hipFuncSetAttribute(func, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    return FK_OK;
}

// Both launches need their 512 workgroups resident TOGETHER, two per CU: a block that has not started cannot publish
// its arrival, and the blocks that did would poll until their spin limit.  First the plain budget (two blocks' LDS in
// the 160 KiB of a gfx950 CU, whatever device is present -- this part also runs without one), then the device's own
// answer for the kernel as compiled (registers included).
constexpr uint32_t kCuLdsBytes = 160u * 1024u;
inline fk_status require_two_blocks_per_cu(const void* func, uint32_t lds, const char* what) {
    if (2u * ((lds + 1023u) & ~1023u) > kCuLdsBytes)
        return set_error(FK_ERR_UNSUPPORTED, std::string("xcd layer: the ") + what + " launch needs " + std::to_string(lds) +
                                                 " bytes of LDS per workgroup; two workgroups do not fit one CU, so its 512 "
                                                 "workgroups cannot all be resident");
    const DeviceFacts* dev;
    FK_TRY(device_facts(&dev));
    if ((int)lds > dev->max_dyn_lds) return set_error(FK_ERR_UNSUPPORTED, "xcd layer: LDS need exceeds the CU");
    if (lds > 48 * 1024) FK_HIP(hipFuncSetAttribute(func, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    int per_cu = 0;
    FK_HIP(hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, func, kBlock, lds));
    if ((long long)per_cu * dev->cus < (long long)kXcdGrid)
        return set_error(FK_ERR_UNSUPPORTED, std::string("xcd layer: only ") + std::to_string(per_cu) + " workgroup(s) of the " + what +
                                                 " launch fit one CU on this device; its 512 workgroups cannot all be resident");
    return FK_OK;
}

}  // namespace
}  // namespace fk
