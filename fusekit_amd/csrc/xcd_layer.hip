// XCD-resident decoder layer: the attention launch and the MLP launch (see xcd_layer.hpp for the scheme).
#include "xcd_layer.hpp"

// Timing probes (empty in the library build): launch k (0 attention, 1 MLP), boundary i, by the first thread of
// the block's first and last wave-pair.
#include "fk_probe.hpp"
FK_PROBE_DEFINE(xcd, 1024, 16)
#define FK_XCD_STAMP(k, i) FK_PROBE_STAMP(xcd, 1024, 16, (k) * 512 + blockIdx.x, threadIdx.x == 0 || threadIdx.x == 256, i)

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

}  // namespace

// =============================================================================================== MLP launch
constexpr int kMlpBlock = kBlock;

// One MLP phase of one block.  `sync` carries the block's XCD, slot and hand-over epoch; `xres_in` / `xres_out`:
// the residual row in LDS (token kernel only).
// EARLY: the caller has already issued input_request into `inr` (the stand-alone launch does so before anything
// else, from its leading parameters).
template <WKind KIND, int NLA, int NLB, bool TOKEN, bool EARLY, bool ONE = false, typename ARGS, typename LEAD>
__device__ __forceinline__ void xcd_mlp_phase(const ARGS& a, const LEAD& lead, InputRegs& inr, XcdSync& sync, uint4* lds_raw,
                                              const uint4* xres_in, uint4* xres_out) {
    const uint32_t cs_max = a.cs_max, work_floats = a.work_floats;
    constexpr int PIECES = ChunkTraits<KIND>::kPieces;
    uint4* xs = lds_raw;
    float* sx = reinterpret_cast<float*>(xs + PIECES * cs_max);
    float* work = sx + cs_max;
    constexpr uint32_t MW = meta_words<ONE>();
    uint32_t* meta = reinterpret_cast<uint32_t*>(work + work_floats);  // [3][MW]
    float* red = reinterpret_cast<float*>(meta + 3 * MW);              // [16]
    const uint32_t tid = threadIdx.x;
    constexpr bool streams = true;

    FK_XCD_STAMP(1, 0);
    const uint32_t per_xcd = a.inter / kXcds;
    const uint32_t gu0 = sync.slot * a.gu_rows;
    const uint32_t gu_n = gu0 < per_xcd ? ((per_xcd - gu0) < a.gu_rows ? (per_xcd - gu0) : a.gu_rows) : 0u;
    const Tile tg = make_tile(sync.xcd * per_xcd + gu0, gu_n, 0, a.gate.cpr);
    const uint32_t d0 = sync.slot * a.down_rows;
    const uint32_t d_n = d0 < a.in.hidden ? ((a.in.hidden - d0) < a.down_rows ? (a.in.hidden - d0) : a.down_rows) : 0u;
    const Tile td = make_tile(d0, d_n, sync.xcd * a.down_cs, a.down_cs);

    MetaRegs mg, mu, md;
    TileRegs<NLA> rg, ru;
    TileRegs<NLB> rd;
    TilePos<NLA> pg;
    TilePos<NLB> pd;
    // Requested now, behind the input: the groups' scales and biases and the first pass of gate / up -- a few
    // KiB per CU.  The later passes stream while the earlier ones are consumed; the down_proj slice is queued
    // behind the last of them.
    if constexpr (!EARLY) input_request<TOKEN>(lead, inr, xres_in);
    tile_pos_init<NLA, kBlock>(a.gate, tg, tid, pg);
    tile_pos_init<NLB, kBlock>(a.down, td, tid, pd);
    meta_fetch<KIND, kBlock, true, !ONE>(a.gate, tg, tid, mg);
    meta_fetch<KIND, kBlock, true, !ONE>(a.up, tg, tid, mu);
    // Only kGuAhead requests of the gate matrix go out ahead of the input's staging, the rest of the pass and the up
    // matrix's behind it: a wave cannot stage before it has ISSUED what stands in front, issue stalls once the CU's
    // request queue is full, and the block's staging waits for its slowest wave.  With all twelve in front the
    // median block had its activations staged 1.3 us later than the attention launch has; with none the stream
    // starts too late (4B int4, tok/s by requests in front: 12: 780, 6: 791, 4: 796, 3: 796, 2: 790, 1: 781, 0: 774; with the
    // down_proj slice requested behind the arithmetic: 6: 802, 4: 819, 3: 828, 2: 820).
    constexpr int GP = kGuAhead < NLA ? kGuAhead : NLA;
    tile_load<KIND, NLA, kBlock, 0, GP>(a.gate, tg, pg, rg);
    FK_XCD_STAMP(1, 1);
    input_pin(lead, inr);
    input_stage<KIND, 1>(a.in, inr, xs, sx, a.gate.cpr, red, xres_out);
    tile_load<KIND, NLA, kBlock, GP, NLA>(a.gate, tg, pg, rg);
    tile_load<KIND, NLA, kBlock>(a.up, tg, pg, ru);
    FK_XCD_STAMP(1, 5);
    input_clear<TOKEN>(a.in);
    meta_store<KIND, kBlock, true, !ONE>(mg, tid, meta);
    meta_store<KIND, kBlock, true, !ONE>(mu, tid, meta + MW);
    meta_fetch<KIND, kBlock, true, !ONE>(a.down, td, tid, md, sync.xcd);  // not needed before the hand-over: kept off the start-up path
    __syncthreads();

    // ---- gate / up rows of this XCD's slice, SwiGLU ----
    const uint32_t seg = (gu_n * a.gate.cpr + NLA * kBlock - 1) / (NLA * kBlock) * (NLA * kBlock);
    if (streams) {
        auto request_down = [&]() { tile_load<KIND, NLB, kBlock>(a.down, td, pd, rd); };
        if (gu_n)
            tile_run_pair<KIND, NLA, kBlock, ONE>(a.gate, a.up, tg, pg, rg, ru, xs, sx, meta, meta + MW, work, work + seg,
                                             request_down);
        else
            request_down();
    }
    FK_XCD_STAMP(1, 6);
    meta_store<KIND, kBlock, true, !ONE>(md, tid, meta + 2 * MW);
    __syncthreads();
    FK_XCD_STAMP(1, 12);
    if (streams && gu_n) {
        uint16_t* mid = a.mid + (size_t)sync.xcd * per_xcd + gu0;
        const int variant = a.swiglu_variant;
        tile_rows<true, ONE>(tg, work, work + seg,
                        [&](uint32_t r, float s0, float s1) { mid[r] = (uint16_t)swiglu_bits(s0, s1, variant, 1.0f); });

    }
    FK_XCD_STAMP(1, 7);
    uint32_t* okw = reinterpret_cast<uint32_t*>(red) + 8;
    xcd_barrier<0>(sync, okw);
    const bool ok = xcd_wait_ok(okw);  // tested in front of the additions into the sum row
    FK_XCD_STAMP(1, 8);

    // ---- down_proj over this XCD's K-slice: fp32 partial row ----
    if (streams) stage_vector<KIND>(a.mid + (size_t)sync.xcd * per_xcd, per_xcd >> 3, a.down_cs, xs, sx);
    __syncthreads();
    FK_XCD_STAMP(1, 9);
    if (streams && d_n) tile_run<KIND, NLB, kBlock, ONE>(a.down, td, pd, rd, xs, sx, meta + 2 * MW, work, []() {});
    __syncthreads();
    FK_XCD_STAMP(1, 10);
    if (streams && d_n && ok) {
        long long* out = a.out_sums;
        XcdControl* ctl = sync.ctl;
        tile_rows<false, ONE>(td, work, work, [&](uint32_t r, float s0, float) { xcd_sum_add(out, d0 + r, s0, ctl); });
    }
    FK_XCD_STAMP(1, 11);
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

template <WKind KIND, int NLA, int NLB, bool ONE>
__global__ __launch_bounds__(kMlpBlock, 2) void xcd_mlp_kernel(const long long* sums, const uint16_t* residual,
                                                               const uint16_t* norm_w, uint32_t hidden, const XcdMlpArgs a) {
    extern __shared__ uint4 lds_raw[];
    // The input is requested from the leading parameters before the argument block is touched.
    const XcdInputLead lead{sums, residual, norm_w, hidden};
    InputRegs inr;
    input_request<false>(lead, inr, nullptr);
    kernarg_warm<32 + (int)sizeof(XcdMlpArgs)>();
    XcdSync sync = xcd_sync_init(a.ctl, a.spin_limit);
    xcd_mlp_phase<KIND, NLA, NLB, false, true, ONE>(a, lead, inr, sync, lds_raw, nullptr, nullptr);
    xcd_mark_placement(sync, a.mark_placement);
}

// =============================================================================================== attention launch
constexpr int kAttnStream = kBlock;

template <WKind KIND, int NLA, int NLB, bool TOKEN, bool EARLY, bool ONE = false, typename ARGS, typename LEAD>
__device__ __forceinline__ void xcd_attn_phase(const ARGS& a, const LEAD& lead, InputRegs& inr, XcdSync& sync, uint4* lds_raw,
                                               const uint4* xres_in, uint4* xres_out) {
    const uint32_t cs_max = a.cs_max, work_floats = a.work_floats, att_elems = a.att_elems;
    (void)att_elems;
    constexpr int PIECES = ChunkTraits<KIND>::kPieces;
    uint4* xs = lds_raw;
    float* sx = reinterpret_cast<float*>(xs + PIECES * cs_max);
    float* work = sx + cs_max;
    constexpr uint32_t MW = meta_words<ONE>();
    uint32_t* meta = reinterpret_cast<uint32_t*>(work + work_floats);  // [3][MW]; two used
    uint16_t* att = reinterpret_cast<uint16_t*>(meta + 3 * MW);

    // Requested now, looked at only behind the start-up requests (the pin below): used at once, the wave would sit
    // out this load's trip to memory before it has asked for anything else.
    uint32_t kv_len_raw = *a.sdpa.kv_len_ptr;
    const uint32_t tid = threadIdx.x, ti = tid;
    constexpr bool streams = true;
    float* red = reinterpret_cast<float*>(att + ((att_elems + 7u) & ~7u));  // [16]

    FK_XCD_STAMP(0, 0);
    // tile of the q / k / v projections: the XCD's q rows first, then its k rows, then its v rows
    const uint32_t R = a.qkv_tile_rows, tix = sync.slot;
    const bool has_tile = tix < a.q_tiles + 2 * a.kv_tiles;
    const uint32_t part_id = tix < a.q_tiles ? 0u : (tix < a.q_tiles + a.kv_tiles ? 1u : 2u);
    const uint32_t tl = part_id == 0 ? tix : (part_id == 1 ? tix - a.q_tiles : tix - a.q_tiles - a.kv_tiles);
    const uint32_t part_rows = part_id == 0 ? a.q_rows : a.kv_rows;
    const uint32_t pr0 = tl * R;
    const uint32_t pr_n = has_tile ? ((part_rows - pr0) < R ? (part_rows - pr0) : R) : 0u;
    const auto& mq = part_id == 0 ? a.wq : (part_id == 1 ? a.wk : a.wv);
    const Tile tq = make_tile(sync.xcd * part_rows + pr0, pr_n, 0, a.wq.cpr);
    const uint32_t o0 = sync.slot * a.o_rows;
    const uint32_t o_n = o0 < a.in.hidden ? ((a.in.hidden - o0) < a.o_rows ? (a.in.hidden - o0) : a.o_rows) : 0u;
    const Tile to = make_tile(o0, o_n, sync.xcd * a.o_cs, a.o_cs);

    MetaRegs mmq, mmo;
    TileRegs<NLA> rq;
    TileRegs<NLB> ro;
    TilePos<NLA> pq;
    TilePos<NLB> po;
    if constexpr (!EARLY) input_request<TOKEN>(lead, inr, xres_in);
    tile_pos_init<NLA, kAttnStream>(mq, tq, ti, pq);
    tile_pos_init<NLB, kAttnStream>(a.wo, to, ti, po);
    meta_fetch<KIND, kAttnStream, true, !ONE>(mq, tq, ti, mmq);
    tile_load<KIND, NLA, kAttnStream>(mq, tq, pq, rq);  // all of it ahead of the staging: 2 or 3 of 5 were no faster here
    FK_XCD_STAMP(0, 1);
    asm volatile("" : "+v"(kv_len_raw));
    const uint32_t kv_len0 = __builtin_amdgcn_readfirstlane(kv_len_raw);
    input_pin(lead, inr);
    input_stage<KIND, 0>(a.in, inr, xs, sx, a.wq.cpr, red, xres_out);
    FK_XCD_STAMP(0, 5);
    input_clear<TOKEN>(a.in);
    meta_store<KIND, kAttnStream, true, !ONE>(mmq, ti, meta);
    meta_fetch<KIND, kAttnStream, true, !ONE>(a.wo, to, ti, mmo, sync.xcd);  // not needed before the attention is done
    __syncthreads();
    FK_XCD_STAMP(0, 13);

    // ---- q / k / v rows of this XCD's KV head; the o_proj slice is requested behind their last pass ----
    if (streams) {
        auto request_o = [&]() { tile_load<KIND, NLB, kAttnStream>(a.wo, to, po, ro); };
        if (pr_n)
            tile_run<KIND, NLA, kAttnStream, ONE>(mq, tq, pq, rq, xs, sx, meta, work, request_o);
        else
            request_o();
    }
    FK_XCD_STAMP(0, 14);
    __syncthreads();
    FK_XCD_STAMP(0, 15);
    if (pr_n) {
        uint16_t* dst = (part_id == 0 ? a.q : (part_id == 1 ? a.k : a.v)) + (size_t)sync.xcd * part_rows + pr0;
        tile_rows<false, ONE>(tq, work, work, [&](uint32_t r, float s0, float) { dst[r] = (uint16_t)f32_to_bf16_bits(s0); });
    }
    FK_XCD_STAMP(0, 6);
    uint32_t* okw = reinterpret_cast<uint32_t*>(red) + 8;
    xcd_barrier<0>(sync, okw);
    if (!xcd_wait_ok(okw)) return;  // the attention phase appends to the cache
    FK_XCD_STAMP(0, 7);

    // ---- head norm + RoPE + cache append + attention: block = (query head of the group, key range) ----
    const uint32_t G = a.sdpa.n_heads / a.sdpa.n_kv;
    {
        const uint32_t gz = sync.slot % G, split = sync.slot / G;
        if (split < a.sdpa.n_splits)
            sdpa_block<1, 2, std::remove_cv_t<std::remove_reference_t<decltype((a.sdpa))>>, 0, true, true>(a.sdpa, kv_len0, split, sync.xcd, gz, G, work);
    }
    FK_XCD_STAMP(0, 8);
    xcd_barrier<0>(sync, okw);
    const bool ok2 = xcd_wait_ok(okw);  // tested in front of the additions into the sum row
    FK_XCD_STAMP(0, 9);

    // ---- merge the ranges of each of the group's heads (range order), rows to LDS ----
    {
        const uint32_t span = a.sdpa.chunk_len * a.sdpa.chunks_per_block;
        const uint32_t covered = a.sdpa.n_splits * span < a.sdpa.capacity ? a.sdpa.n_splits * span : a.sdpa.capacity;
        const uint32_t kv_len = kv_len0 < 1u ? 1u : (kv_len0 > covered ? covered : kv_len0);
        const uint32_t n_active = (kv_len + span - 1) / span;
        const uint32_t row = a.sdpa.v_dim + 2;
        const uint32_t lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
        for (uint32_t h = wave; h < G; h += kBlock / kWave) {
            const float* ph = a.sdpa.partials + (size_t)(sync.xcd * G + h) * a.sdpa.n_splits * row;
            for (uint32_t d2 = lane; d2 < ((a.sdpa.v_dim >> 1) + kWave - 1) / kWave * kWave; d2 += kWave) {
                const bool live = d2 < (a.sdpa.v_dim >> 1);
                const float* pd = ph + 2 + 2 * (live ? d2 : 0u);
                float M = -INFINITY, L = 0.f, o0_ = 0.f, o1_ = 0.f;
                // all requests first (clamped indices: straight-line), then the fold in range order; up to 8 ranges
                // (a context of 8 x the range length) take half the requests.  The (maximum, sum) pair of range i is
                // fetched by lane i alone and handed to the wave through scalar registers: one request, not N.
                auto merge = [&](auto n_const) {
                    constexpr uint32_t N = decltype(n_const)::value;
                    float2 po[N];
                    const float2 mine = ld_f32x2<true>(ph + (size_t)(lane < n_active ? lane : 0u) * row);
#pragma unroll
                    for (uint32_t i = 0; i < N; ++i) po[i] = ld_f32x2<true>(pd + (size_t)(i < n_active ? i : 0u) * row);
                    float2 ml[N];
#pragma unroll
                    for (uint32_t i = 0; i < N; ++i) {
                        ml[i].x = __uint_as_float(__builtin_amdgcn_readlane(__float_as_uint(mine.x), i));
                        ml[i].y = __uint_as_float(__builtin_amdgcn_readlane(__float_as_uint(mine.y), i));
                    }
                    M = ml[0].x;
#pragma unroll
                    for (uint32_t i = 1; i < N; ++i) M = i < n_active ? fmaxf(M, ml[i].x) : M;
#pragma unroll
                    for (uint32_t i = 0; i < N; ++i) {
                        const float w = i < n_active ? expf(ml[i].x - M) : 0.f;
                        L = fmaf(ml[i].y, w, L);
                        o0_ = fmaf(po[i].x, w, o0_);
                        o1_ = fmaf(po[i].y, w, o1_);
                    }
                };
                if (n_active <= kXcdMaxRanges / 4)
                    merge(std::integral_constant<uint32_t, kXcdMaxRanges / 4>{});
                else if (n_active <= kXcdMaxRanges / 2)
                    merge(std::integral_constant<uint32_t, kXcdMaxRanges / 2>{});
                else
                    merge(std::integral_constant<uint32_t, kXcdMaxRanges>{});
                const float inv_l = 1.0f / L;
                if (live) {
                    att[h * a.sdpa.v_dim + 2 * d2] = (uint16_t)f32_to_bf16_bits(o0_ * inv_l);
                    att[h * a.sdpa.v_dim + 2 * d2 + 1] = (uint16_t)f32_to_bf16_bits(o1_ * inv_l);
                }
            }
        }
    }
    __syncthreads();
    FK_XCD_STAMP(0, 10);
    // ---- o_proj over this XCD's K-slice (its heads' columns): fp32 partial row ----
    {
        const uint32_t n8 = (G * a.sdpa.v_dim) >> 3, n8_up = (n8 + kWave - 1) / kWave * kWave;
        const uint4* a8 = reinterpret_cast<const uint4*>(att);
        for (uint32_t t = threadIdx.x; t < n8_up; t += kBlock) {
            const bool live = t < n8;
            const uint4 v = a8[live ? t : 0u];
            stage_emit<KIND>(xs, sx, a.o_cs, t, live, v, v, 1.0f, false);
        }
    }
    meta_store<KIND, kAttnStream, true, !ONE>(mmo, ti, meta + MW);
    __syncthreads();
    if (streams && o_n) tile_run<KIND, NLB, kAttnStream, ONE>(a.wo, to, po, ro, xs, sx, meta + MW, work, []() {});
    __syncthreads();
    FK_XCD_STAMP(0, 11);
    if (o_n && ok2) {
        long long* out = a.out_sums;
        XcdControl* ctl = sync.ctl;
        // (the one-round form was slower here: 835 against 837 tok/s; the o_proj slice has 16 chunks per row)
        tile_rows<false>(to, work, work, [&](uint32_t r, float s0, float) { xcd_sum_add(out, o0 + r, s0, ctl); });
    }
    FK_XCD_STAMP(0, 12);
}

template <WKind KIND, int NLA, int NLB, bool ONE>
__global__ __launch_bounds__(kBlock, 2) void xcd_attn_kernel(const long long* sums, const uint16_t* residual,
                                                             const uint16_t* norm_w, uint32_t hidden, const XcdAttnArgs a) {
    extern __shared__ uint4 lds_raw[];
    const XcdInputLead lead{sums, residual, norm_w, hidden};
    InputRegs inr;
    input_request<false>(lead, inr, nullptr);
    kernarg_warm<32 + (int)sizeof(XcdAttnArgs)>();
    XcdSync sync = xcd_sync_init(a.ctl, a.spin_limit);
    xcd_attn_phase<KIND, NLA, NLB, false, true, ONE>(a, lead, inr, sync, lds_raw, nullptr, nullptr);
    xcd_mark_placement(sync, a.mark_placement);
}

// ---- the whole token in one launch --------------------------------------------------------------------------
// Device-wide barrier in two levels: every block publishes its arrival word as in a hand-over; the leader block of
// each XCD (slot 0) waits for its 64 blocks, adds one to `arrivals` (a memory-side add) and waits until all eight
// leaders have (L1-bypassing loads see memory-side additions), then releases its XCD through `release[xcd]`, which
// the other 63 blocks poll.  Counters only grow; every wait is bounded.  Returns false after an abort.
struct XcdGlobalSync {
    uint32_t arrivals_base, release_base, k;
};
__device__ __forceinline__ XcdGlobalSync xcd_global_init(const XcdSync& s) {
    XcdGlobalSync g;
    // a fast leader may already have arrived at the first barrier: it completes only with all eight, so the count
    // read here lies within 7 of the last completed multiple of 8
    g.arrivals_base = __hip_atomic_load(&s.ctl->arrivals, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) & ~7u;
    g.release_base = __hip_atomic_load(&s.ctl->release[s.xcd], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    g.k = 0;
    return g;
}
__device__ __forceinline__ bool xcd_global_barrier(XcdSync& s, XcdGlobalSync& g) {
    s.epoch += 1;
    g.k += 1;
    wait_memory_ops_done();
    __syncthreads();
    if (threadIdx.x < (uint32_t)kWave) {
        const uint32_t lane = threadIdx.x;
        bool ok = true;
        if (s.slot == 0) {
            ok = xcd_publish_and_wait(s, lane);
            if (ok) {
                if (lane == 0) (void)__hip_atomic_fetch_add(&s.ctl->arrivals, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                const uint32_t target = g.arrivals_base + kXcds * g.k;
                uint32_t spins = 0;
                for (;;) {
                    const uint32_t v = __hip_atomic_load(&s.ctl->arrivals, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    if ((int32_t)(v - target) >= 0) break;
                    if (++spins > s.spin_limit || ((spins & 255u) == 0u &&
                                                   __hip_atomic_load(&s.ctl->abort_flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0u)) {
                        if (lane == 0) __hip_atomic_store(&s.ctl->abort_flag, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                        ok = false;
                        break;
                    }
                    __builtin_amdgcn_s_sleep(1);
                }
            }
            // released also after a failure, so that the XCD's blocks leave their wait at once and see the abort word
            if (lane == 0) __hip_atomic_store(&s.ctl->release[s.xcd], g.release_base + g.k, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
        } else {
            if (lane == 0) __hip_atomic_store(s.ctl->flags + s.xcd * kXcdSlots + s.slot, s.epoch, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
            const uint32_t target = g.release_base + g.k;
            uint32_t spins = 0;
            for (;;) {
                const uint32_t v = __hip_atomic_load(&s.ctl->release[s.xcd], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                if ((int32_t)(v - target) >= 0) break;
                if (++spins > s.spin_limit) {
                    if (lane == 0) __hip_atomic_store(&s.ctl->abort_flag, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    break;
                }
                __builtin_amdgcn_s_sleep(1);
            }
        }
    }
    __syncthreads();
    return __hip_atomic_load(&s.ctl->abort_flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == 0u;
}

template <WKind KIND, int NLQ, int NLO, int NLG, int NLD>
__global__ __launch_bounds__(kBlock, 2) void xcd_token_kernel(const XcdTokenArgs t) {
    extern __shared__ uint4 lds_raw[];
    uint4* xres = lds_raw + t.xres_off;
    XcdSync sync = xcd_sync_init(t.ctl, t.spin_limit);
    XcdGlobalSync gs = xcd_global_init(sync);
    // The argument blocks never change while the kernel runs: read through the constant address space, every field
    // is a scalar load, as for kernel arguments.
#if defined(__HIP_DEVICE_COMPILE__)
    typedef __attribute__((address_space(4))) XcdAttnArgs ConstAttn;
    typedef __attribute__((address_space(4))) XcdMlpArgs ConstMlp;
#else
    typedef XcdAttnArgs ConstAttn;
    typedef XcdMlpArgs ConstMlp;
#endif
    // The next phase's argument block is pulled into this XCD's L2 while the current phase runs (one request per
    // 64 bytes by a few lanes), so that its scalar loads do not start the phase with a trip to memory.
    auto touch = [&](const void* p, uint32_t bytes) {
        if (threadIdx.x * 64u < bytes) (void)*reinterpret_cast<const volatile uint32_t*>(reinterpret_cast<const char*>(p) + threadIdx.x * 64u);
    };
    for (uint32_t l = 0; l < t.n_layers; ++l) {
        touch(t.mlp + l, sizeof(XcdMlpArgs));
        {
            InputRegs inr;
            xcd_attn_phase<KIND, NLQ, NLO, true, false>(*(const ConstAttn*)(t.attn + l), ((const ConstAttn*)(t.attn + l))->in, inr, sync, lds_raw, l ? xres : nullptr, xres);
        }
        if (!xcd_global_barrier(sync, gs)) return;
        if (l + 1 < t.n_layers) touch(t.attn + l + 1, sizeof(XcdAttnArgs));
        {
            InputRegs inr;
            xcd_mlp_phase<KIND, NLG, NLD, true, false>(*(const ConstMlp*)(t.mlp + l), ((const ConstMlp*)(t.mlp + l))->in, inr, sync, lds_raw, xres, xres);
        }
        if (l + 1 < t.n_layers && !xcd_global_barrier(sync, gs)) return;
    }
    xcd_mark_placement(sync, t.mark_placement);
}

// ---- a whole layer in one launch ------------------------------------------------------------------------------
// Attention phase (the stand-alone launch's, input requested from the leading parameters), a device-wide barrier,
// MLP phase.  What crosses the barrier: the sum row the attention phase added into (memory-side additions, read with
// L1-bypassing loads), the residual row (every block holds its own copy in LDS) and the row the attention phase
// cleared for the MLP phase to add into (write-through stores).  Everything else is private to an XCD as in the
// separate launches.
template <WKind KIND, int NLQ, int NLO, int NLG, int NLD>
__global__ __launch_bounds__(kBlock, 2) void xcd_layer_kernel(const long long* sums, const uint16_t* residual,
                                                              const uint16_t* norm_w, uint32_t hidden, const XcdLayerArgs t) {
    extern __shared__ uint4 lds_raw[];
    const XcdInputLead lead{sums, residual, norm_w, hidden};
    InputRegs inr;
    input_request<false>(lead, inr, nullptr);
    kernarg_warm<768>();
    kernarg_warm<32 + (int)sizeof(XcdLayerArgs), 12>();
    uint4* xres = lds_raw + t.xres_off;
    XcdSync sync = xcd_sync_init(t.attn.ctl, t.attn.spin_limit);
    XcdGlobalSync gs = xcd_global_init(sync);
    xcd_attn_phase<KIND, NLQ, NLO, true, true, true>(t.attn, lead, inr, sync, lds_raw, nullptr, xres);
    if (!xcd_global_barrier(sync, gs)) return;
    {
        InputRegs inm;
        xcd_mlp_phase<KIND, NLG, NLD, true, false, true>(t.mlp, t.mlp.in, inm, sync, lds_raw, xres, nullptr);
    }
    xcd_mark_placement(sync, t.mark_placement);
}

__global__ __launch_bounds__(kBlock) void xcd_reduce_kernel(const XcdReduceArgs a) {
    const uint32_t i = blockIdx.x * kBlock + threadIdx.x;
    if (i >= a.hidden) return;
    const uint32_t at = xcd_sum_index(i);
    const unsigned long long s = (unsigned long long)a.sums[at];
    a.x[i] = (uint16_t)f32_to_bf16_bits(xcd_sum_to_f32((uint32_t)s, (uint32_t)(s >> 32)) + bf16_bits_to_f32(a.residual[i]));
    if (a.clear) a.clear[at] = 0;
}

// dst[(h * n + r) * gl + g] = src[r * groups + h * gl + g]: the scales (or biases) of a [n, groups] matrix, the
// K dimension cut into 8 slices of gl = groups / 8 groups, one contiguous copy per slice.
__global__ __launch_bounds__(kBlock) void xcd_kslice_meta_kernel(const uint16_t* src, uint16_t* dst, uint32_t n, uint32_t groups) {
    const uint32_t gl = groups / kXcds;
    const size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x;
    if (i >= (size_t)n * groups) return;
    const uint32_t g = (uint32_t)(i % gl), r = (uint32_t)((i / gl) % n), h = (uint32_t)(i / ((size_t)gl * n));
    dst[i] = src[(size_t)r * groups + h * gl + g];
}

// =============================================================================================== host side
fk_status xcd_kslice_meta(const uint16_t* src, uint32_t n, uint32_t groups, uint16_t* dst, hipStream_t stream) {
    const DeviceFacts* dev;
    FK_TRY(device_facts(&dev));
    if (!src || !dst || n == 0 || groups == 0 || groups % kXcds) return set_error(FK_ERR_INVALID, "xcd k-slice scales: null buffer, or groups per row not a multiple of 8");
    const size_t total = (size_t)n * groups;
    hipLaunchKernelGGL(xcd_kslice_meta_kernel, dim3((unsigned)((total + kBlock - 1) / kBlock)), dim3(kBlock), 0, stream, src, dst, n, groups);
    FK_HIP(hipGetLastError());
    return FK_OK;
}

namespace {

constexpr int kNlQkv = 5, kNlO = 3, kNlGu = 6, kNlDown = 6;  // 16-byte requests per streaming thread and pass
constexpr int kNlGuToken = 4;  // the whole-token launch holds both phases' registers: shallower gate / up passes
// Stand-alone attention launch with 8-bit weights: twice the chunks per tile, and passes deep enough that the
// 4B-class tiles are one pass there as well (18.5 -> 17.8 us).  The MLP launch keeps its depth: with 12 requests per
// matrix and thread in one go it was slower (24.0 -> 24.8 us) than two passes of 6.
struct PassDepth {
    int qkv, o, gu, down;
};
constexpr PassDepth depth_of(WKind k) {
    return k == W_Q8 ? PassDepth{9, 5, kNlGu, kNlDown} : PassDepth{kNlQkv, kNlO, kNlGu, kNlDown};
}
inline PassDepth depth_of_bits(uint32_t bits) { return depth_of(bits == 4 ? W_Q4 : (bits == 8 ? W_Q8 : W_BF16)); }

uint32_t ilog2u(uint32_t v) {
    uint32_t r = 0;
    while ((1u << (r + 1)) <= v) ++r;
    return r;
}
uint32_t ceil_div(uint32_t a, uint32_t b) { return (a + b - 1) / b; }
uint32_t chunk_values(uint32_t bits) { return bits == 4 ? 32u : (bits == 8 ? 16u : 8u); }

fk_status bind_mat(const fk_weight* w, uint32_t n, uint32_t k, const XcdLayerShape& s, XcdMat* m, const char* what) {
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

template <WKind KIND>
const void* mlp_func(bool one) {
    constexpr PassDepth d = depth_of(KIND);  // the deeper passes only where they make the launch one pass
    return one ? reinterpret_cast<const void*>(&xcd_mlp_kernel<KIND, d.gu, d.down, true>)
               : reinterpret_cast<const void*>(&xcd_mlp_kernel<KIND, kNlGu, kNlDown, false>);
}
template <WKind KIND>
const void* attn_func(bool one) {
    constexpr PassDepth d = depth_of(KIND);
    return one ? reinterpret_cast<const void*>(&xcd_attn_kernel<KIND, d.qkv, d.o, true>)
               : reinterpret_cast<const void*>(&xcd_attn_kernel<KIND, kNlQkv, kNlO, false>);
}

template <WKind KIND>
const void* layer_func() {
    constexpr PassDepth d = depth_of(KIND);
    return reinterpret_cast<const void*>(&xcd_layer_kernel<KIND, d.qkv, d.o, d.gu, d.down>);
}

uint32_t lds_for(uint32_t bits, const LdsPlan& p) {
    return bits == 4 ? xcd_lds_bytes<W_Q4>(p) : (bits == 8 ? xcd_lds_bytes<W_Q8>(p) : xcd_lds_bytes<W_BF16>(p));
}

fk_status fill_input(const XcdLayerShape& s, const long long* sums, const uint16_t* residual, uint16_t* x_out,
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

fk_status set_lds_limit(const void* func, uint32_t lds) {
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
fk_status require_two_blocks_per_cu(const void* func, uint32_t lds, const char* what) {
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

// What a launch's shape decides: tiles, kernel flavour, LDS.
struct MlpGeometry {
    uint32_t gate_cpr, down_cpr, gu_rows, down_rows, down_cs;
    bool one;
    LdsPlan lp;
    uint32_t lds;
    const void* func;
};
MlpGeometry mlp_geometry(const XcdLayerShape& s, bool for_token) {
    MlpGeometry g;
    const uint32_t cv = chunk_values(s.bits);
    g.gate_cpr = s.hidden / cv;
    g.down_cpr = s.inter / cv;
    g.gu_rows = ceil_div(s.inter / kXcds, kXcdSlots);
    g.down_rows = ceil_div(s.hidden, kXcdSlots);
    g.down_cs = g.down_cpr / kXcds;
    auto padded = [](uint32_t chunks, int nl) { return ceil_div(chunks, nl * kBlock) * nl * kBlock; };
    g.lp.cs_max = g.gate_cpr > g.down_cs ? g.gate_cpr : g.down_cs;
    const PassDepth deep = depth_of_bits(s.bits);
    // every tile within one pass (the 4B-class shapes): the flavour compiled without the pass loop
    g.one = !for_token && g.gu_rows * g.gate_cpr <= (uint32_t)deep.gu * kBlock && g.down_rows * g.down_cs <= (uint32_t)deep.down * kBlock;
    const PassDepth depth = for_token ? PassDepth{kNlQkv, kNlO, kNlGuToken, kNlDown} : (g.one ? deep : PassDepth{kNlQkv, kNlO, kNlGu, kNlDown});
    const uint32_t gu = 2 * padded(g.gu_rows * g.gate_cpr, depth.gu), dn = padded(g.down_rows * g.down_cs, depth.down);
    g.lp.work_floats = gu > dn ? gu : dn;
    g.lp.att_elems = 0;
    g.lp.meta_words = g.one ? kMetaWords : kMetaWordsBig;
    g.lds = lds_for(s.bits, g.lp);
    g.func = s.bits == 4 ? mlp_func<W_Q4>(g.one) : (s.bits == 8 ? mlp_func<W_Q8>(g.one) : mlp_func<W_BF16>(g.one));
    return g;
}

struct AttnGeometry {
    uint32_t wq_cpr, wo_cpr, q_rows, kv_rows, R, q_tiles, kv_tiles, o_rows, o_cs;
    uint32_t chunk_len, chunks_per_block, n_splits;
    bool one;
    LdsPlan lp;
    uint32_t lds;
    const void* func;
};
AttnGeometry attn_geometry(const XcdLayerShape& s, bool for_token = false) {
    AttnGeometry g;
    const uint32_t cv = chunk_values(s.bits), G = s.n_heads / s.n_kv;
    g.wq_cpr = s.hidden / cv;
    g.wo_cpr = s.n_heads * s.head_dim / cv;
    g.q_rows = G * s.head_dim;
    g.kv_rows = s.head_dim;
    uint32_t R = 1;
    while (ceil_div(g.q_rows, R) + 2 * ceil_div(g.kv_rows, R) > kXcdSlots) ++R;
    g.R = R;
    g.q_tiles = ceil_div(g.q_rows, R);
    g.kv_tiles = ceil_div(g.kv_rows, R);
    g.o_rows = ceil_div(s.hidden, kXcdSlots);
    g.o_cs = g.wo_cpr / kXcds;
    // attention of one KV head per XCD: blocks = (query head of the group) x (key range)
    g.chunk_len = sdpa_chunk_len(s.head_dim, s.head_dim, false);
    uint32_t splits = kXcdSlots / G;
    if (splits > kXcdMaxRanges) splits = kXcdMaxRanges;
    const uint32_t n_chunks = ceil_div(s.capacity, g.chunk_len);
    g.chunks_per_block = ceil_div(n_chunks, splits);
    g.n_splits = ceil_div(n_chunks, g.chunks_per_block);
    auto padded = [](uint32_t chunks, int nl) { return ceil_div(chunks, nl * kAttnStream) * nl * kAttnStream; };
    g.lp.cs_max = g.wq_cpr > g.o_cs ? g.wq_cpr : g.o_cs;
    // partial rows padded to whole passes: of this launch's depths and of the whole-token launch's (it shares this plan)
    const PassDepth deep = depth_of_bits(s.bits);
    g.one = !for_token && R * g.wq_cpr <= (uint32_t)deep.qkv * kAttnStream && g.o_rows * g.o_cs <= (uint32_t)deep.o * kAttnStream;
    const PassDepth depth = g.one ? deep : PassDepth{kNlQkv, kNlO, kNlGu, kNlDown};
    auto larger = [](uint32_t x, uint32_t y) { return x > y ? x : y; };
    uint32_t wf = larger(padded(R * g.wq_cpr, depth.qkv), padded(R * g.wq_cpr, kNlQkv));
    const uint32_t wo_ = larger(padded(g.o_rows * g.o_cs, depth.o), padded(g.o_rows * g.o_cs, kNlO));
    wf = wf > wo_ ? wf : wo_;
    const uint32_t sf = sdpa_lds_floats(1, g.chunk_len, s.head_dim, s.head_dim, true);
    g.lp.work_floats = wf > sf ? wf : sf;
    g.lp.att_elems = G * s.head_dim;
    g.lp.meta_words = g.one ? kMetaWords : kMetaWordsBig;   // the whole-token launch runs the flavour with the pass loop
    g.lds = lds_for(s.bits, g.lp);
    g.func = s.bits == 4 ? attn_func<W_Q4>(g.one) : (s.bits == 8 ? attn_func<W_Q8>(g.one) : attn_func<W_BF16>(g.one));
    return g;
}

}  // namespace

// The shape rules and the LDS budget come first and need no device; the device's CU count and its occupancy answer for
// the two kernels come last.
fk_status xcd_layer_supported(const XcdLayerShape& s) {
    if (s.bits != 4 && s.bits != 8 && s.bits != 16) return set_error(FK_ERR_UNSUPPORTED, "xcd layer: bits must be 4, 8 or 16");
    const uint32_t cv = chunk_values(s.bits), unit = s.bits == 16 ? cv : (s.group > cv ? s.group : cv);
    if (s.bits != 16 && s.group != 32 && s.group != 64 && s.group != 128)
        return set_error(FK_ERR_UNSUPPORTED, "xcd layer: group size must be 32, 64 or 128");
    if (s.n_kv != kXcds) return set_error(FK_ERR_UNSUPPORTED, "xcd layer: needs exactly 8 KV heads (one per XCD)");
    if (s.n_heads % s.n_kv) return set_error(FK_ERR_INVALID, "xcd layer: n_heads must be a multiple of n_kv");
    const uint32_t G = s.n_heads / s.n_kv;
    if (G != 1 && G != 2 && G != 4 && G != 8) return set_error(FK_ERR_UNSUPPORTED, "xcd layer: 1, 2, 4 or 8 query heads per KV head");
    if (s.head_dim != 64 && s.head_dim != 128) return set_error(FK_ERR_UNSUPPORTED, "xcd layer: head_dim must be 64 or 128");
    if (s.hidden % 64 || s.hidden > (uint32_t)kInGroups * kBlock * 8) return set_error(FK_ERR_UNSUPPORTED, "xcd layer: hidden must be a multiple of 64, at most 4096");
    if (s.bits != 16 && (s.hidden / s.group) % 4) return set_error(FK_ERR_UNSUPPORTED, "xcd layer: hidden must hold a multiple of four quantisation groups");
    if ((G * s.head_dim) % unit) return set_error(FK_ERR_UNSUPPORTED, "xcd layer: a KV head's query columns must be whole quantisation groups");
    if (s.inter % (kXcds * unit) || s.inter % (kXcds * 8)) return set_error(FK_ERR_UNSUPPORTED, "xcd layer: intermediate / 8 must be whole quantisation groups");
    if (s.capacity == 0) return set_error(FK_ERR_INVALID, "xcd layer: zero cache capacity");
    const MlpGeometry mg = mlp_geometry(s, false);
    const AttnGeometry ag = attn_geometry(s);
    if (s.bits != 16) {
        // a tile's quantisation groups are fetched once per block: 768 per matrix in the one-pass flavour, 2048 in the
        // flavour with the pass loop
        const uint32_t n_q = s.n_heads * s.head_dim;
        const uint32_t budget_a = ag.lp.meta_words, budget_m = mg.lp.meta_words;
        uint32_t R = 1;
        while (ceil_div(G * s.head_dim, R) + 2 * ceil_div(s.head_dim, R) > kXcdSlots) ++R;
        if (R * (s.hidden / s.group) > budget_a || ceil_div(s.hidden, kXcdSlots) * (n_q / kXcds / s.group) > budget_a ||
            ceil_div(s.inter / kXcds, kXcdSlots) * (s.hidden / s.group) > budget_m ||
            ceil_div(s.hidden, kXcdSlots) * (s.inter / kXcds / s.group) > budget_m)
            return set_error(FK_ERR_UNSUPPORTED, "xcd layer: a block's tile holds more quantisation groups than the kernel fetches");
        // the groups of a block's o_proj / down_proj tile are fetched four per lane from the per-XCD copies
        const uint32_t rpb = ceil_div(s.hidden, kXcdSlots);
        if (s.hidden % kXcdSlots || (rpb * (n_q / kXcds / s.group)) % 4 || (rpb * (s.inter / kXcds / s.group)) % 4)
            return set_error(FK_ERR_UNSUPPORTED, "xcd layer: a block's o_proj / down_proj tile must hold a multiple of four quantisation groups");
    }
    if (2u * ((mg.lds + 1023u) & ~1023u) > kCuLdsBytes || 2u * ((ag.lds + 1023u) & ~1023u) > kCuLdsBytes)
        return set_error(FK_ERR_UNSUPPORTED, "xcd layer: two workgroups of a launch must fit the LDS of one CU (MLP launch " +
                                                 std::to_string(mg.lds) + " bytes, attention launch " + std::to_string(ag.lds) +
                                                 " bytes per workgroup): its 512 workgroups could not all be resident");
    const DeviceFacts* dev;
    FK_TRY(device_facts(&dev));
    if (dev->cus != (int)(kXcds * 32)) return set_error(FK_ERR_UNSUPPORTED, "xcd layer: needs 8 XCDs of 32 CUs");
    FK_TRY(require_two_blocks_per_cu(mg.func, mg.lds, "MLP"));
    FK_TRY(require_two_blocks_per_cu(ag.func, ag.lds, "attention"));
    return FK_OK;
}

size_t xcd_workspace_bytes() { return sizeof(XcdControl); }

fk_status xcd_check_control(void* workspace) {
    if (!workspace) return set_error(FK_ERR_INVALID, "xcd layer: null control block");
    static_assert(offsetof(XcdControl, abort_flag) == sizeof(uint32_t) * kXcds * kXcdSlots, "control block layout");
    // everything behind the arrival words in one copy
    constexpr size_t off = offsetof(XcdControl, abort_flag);
    alignas(8) unsigned char tail[sizeof(XcdControl) - off];
    FK_HIP(hipMemcpy(tail, reinterpret_cast<const char*>(workspace) + off, sizeof(tail), hipMemcpyDeviceToHost));
    auto word = [&](size_t o) {
        uint32_t v;
        memcpy(&v, tail + (o - off), 4);
        return v;
    };
    const char* what = nullptr;
    if (word(offsetof(XcdControl, abort_flag)))
        what = "a hand-over wait exceeded its spin limit";
    else if (word(offsetof(XcdControl, overflow)))
        what = "a contribution to a sum row was not finite or reached 2^27 in magnitude (the fixed-point range)";
    else
        for (uint32_t x = 0; x < kXcds; ++x) {
            unsigned long long bits;
            memcpy(&bits, tail + (offsetof(XcdControl, placement) + x * sizeof(XcdPlacement) - off), 8);
            if (bits != 0ull && bits != ~0ull) what = "two workgroups of a launch ran in the same (XCD, slot): the dispatch order is not the round-robin dealing the layer cut relies on";
        }
    if (!what) return FK_OK;
    // the arrival words of a failed launch are inconsistent: start over from zero
    FK_HIP(hipMemset(workspace, 0, sizeof(XcdControl)));
    return set_error(FK_ERR_HIP, std::string("xcd layer: ") + what +
                                     "; results are invalid (the control block was reset; zero the sum rows and decode the token again)");
}
size_t xcd_sum_row_bytes(uint32_t hidden) { return (size_t)xcd_sum_row_elems(hidden) * sizeof(long long); }

size_t xcd_attn_partials_bytes(const XcdLayerShape& s) {
    return (size_t)s.n_heads * kXcdMaxRanges * (s.head_dim + 2) * sizeof(float);
}

fk_status plan_xcd_mlp(const XcdMlpRequest& rq, Launch* out) {
    const XcdLayerShape& s = rq.shape;
    FK_TRY(xcd_layer_supported(s));
    if (!rq.mid || !rq.out_sums || !rq.workspace) return set_error(FK_ERR_INVALID, "xcd mlp: null mid, sum row or workspace");
    if (rq.swiglu_variant < 0 || rq.swiglu_variant > 2) return set_error(FK_ERR_INVALID, "xcd mlp: swiglu variant must be 0, 1 or 2");
    XcdMlpArgs a;
    memset(&a, 0, sizeof(a));
    FK_TRY(fill_input(s, rq.sums_in, rq.residual, rq.x_out, rq.clear, rq.out_sums, rq.norm_w, rq.eps, &a.in));
    FK_TRY(bind_mat(rq.wgate, s.inter, s.hidden, s, &a.gate, "gate_proj"));
    FK_TRY(bind_mat(rq.wup, s.inter, s.hidden, s, &a.up, "up_proj"));
    FK_TRY(bind_mat(rq.wdown, s.hidden, s.inter, s, &a.down, "down_proj"));
    const MlpGeometry g = mlp_geometry(s, rq.for_token);
    a.inter = s.inter;
    a.gu_rows = g.gu_rows;
    a.down_rows = g.down_rows;
    a.down_cs = g.down_cs;
    a.swiglu_variant = rq.swiglu_variant;
    a.mid = rq.mid;
    a.out_sums = rq.out_sums;
    a.ctl = reinterpret_cast<XcdControl*>(rq.workspace);
    a.spin_limit = rq.spin_limit ? rq.spin_limit : (1u << 20);
    a.mark_placement = rq.mark_placement ? 1u : 0u;
    const LdsPlan lp = g.lp;
    const uint32_t lds = g.lds;
    out->func = g.func;
    if (rq.for_token)
        FK_TRY(set_lds_limit(out->func, lds));  // an argument block for the whole-token launch, which is planned (and checked) as a whole
    else
        FK_TRY(require_two_blocks_per_cu(out->func, lds, "MLP"));
    out->grid = dim3(kXcdGrid, 1, 1);
    out->block = dim3(kMlpBlock, 1, 1);
    out->shmem = lds;
    a.cs_max = lp.cs_max;
    a.work_floats = lp.work_floats;
    out->set_args(a);
    out->n_lead = 0;
    out->add_lead(a.in.sums);
    out->add_lead(a.in.residual);
    out->add_lead(a.in.norm_w);
    out->add_lead(a.in.hidden);
    return FK_OK;
}

fk_status plan_xcd_attn(const XcdAttnRequest& rq, Launch* out) {
    const XcdLayerShape& s = rq.shape;
    FK_TRY(xcd_layer_supported(s));
    if (!rq.q || !rq.k || !rq.v || !rq.cache_k || !rq.cache_v || !rq.kv_len || !rq.rope_tab || !rq.att_partials ||
        !rq.out_sums || !rq.workspace)
        return set_error(FK_ERR_INVALID, "xcd attention: null buffer");
    if ((rq.q_norm == nullptr) != (rq.k_norm == nullptr)) return set_error(FK_ERR_INVALID, "xcd attention: q and k head norms come together");
    const uint32_t n_q = s.n_heads * s.head_dim, n_kvd = s.n_kv * s.head_dim;
    XcdAttnArgs a;
    memset(&a, 0, sizeof(a));
    FK_TRY(fill_input(s, rq.sums_in, rq.residual, rq.x_out, rq.clear, rq.out_sums, rq.norm_w, rq.eps, &a.in));
    FK_TRY(bind_mat(rq.wq, n_q, s.hidden, s, &a.wq, "q_proj"));
    FK_TRY(bind_mat(rq.wk, n_kvd, s.hidden, s, &a.wk, "k_proj"));
    FK_TRY(bind_mat(rq.wv, n_kvd, s.hidden, s, &a.wv, "v_proj"));
    FK_TRY(bind_mat(rq.wo, s.hidden, n_q, s, &a.wo, "o_proj"));
    const AttnGeometry g = attn_geometry(s, rq.for_token);
    a.q_rows = g.q_rows;
    a.kv_rows = g.kv_rows;
    a.qkv_tile_rows = g.R;
    a.q_tiles = g.q_tiles;
    a.kv_tiles = g.kv_tiles;
    a.o_rows = g.o_rows;
    a.o_cs = g.o_cs;
    a.q = rq.q;
    a.k = rq.k;
    a.v = rq.v;
    // attention of one KV head per XCD: blocks = (query head of the group) x (key range)
    SdpaArgs& sd = a.sdpa;
    sd.q = rq.q;
    sd.k = rq.cache_k;
    sd.v = rq.cache_v;
    sd.out = nullptr;
    sd.kv_len_ptr = rq.kv_len;
    sd.n_heads = s.n_heads;
    sd.n_kv = s.n_kv;
    sd.qk_dim = sd.v_dim = s.head_dim;
    sd.capacity = s.capacity;
    sd.chunk_len = g.chunk_len;
    sd.chunks_per_block = g.chunks_per_block;
    sd.n_splits = g.n_splits;
    sd.rows = 1;
    uint32_t lp_ = 1;
    while (lp_ < s.head_dim / 8) lp_ <<= 1;
    sd.lpk = sd.lpv = lp_;
    sd.scale = 1.0f / sqrtf((float)s.head_dim);
    sd.partials = rq.att_partials;
    sd.counters = nullptr;
    sd.k_new = rq.k;
    sd.v_new = rq.v;
    sd.q_norm = rq.q_norm;
    sd.k_norm = rq.k_norm;
    sd.cache_k_w = rq.cache_k;
    sd.cache_v_w = rq.cache_v;
    sd.rope_dims = s.head_dim;
    sd.eps = rq.eps;
    sd.base_log2 = (float)log2((double)rq.theta);
    sd.rope_tab = rq.rope_tab;
    sd.v_stride = s.head_dim;
    sd.k1_heads = 1;
    a.out_sums = rq.out_sums;
    a.ctl = reinterpret_cast<XcdControl*>(rq.workspace);
    a.spin_limit = rq.spin_limit ? rq.spin_limit : (1u << 20);
    a.mark_placement = rq.mark_placement ? 1u : 0u;
    const LdsPlan lp = g.lp;
    const uint32_t lds = g.lds;
    out->func = g.func;
    if (rq.for_token)
        FK_TRY(set_lds_limit(out->func, lds));  // an argument block for the whole-token launch, which is checked as a whole
    else
        FK_TRY(require_two_blocks_per_cu(out->func, lds, "attention"));
    out->grid = dim3(kXcdGrid, 1, 1);
    out->block = dim3(kBlock, 1, 1);
    out->shmem = lds;
    a.cs_max = lp.cs_max;
    a.work_floats = lp.work_floats;
    a.att_elems = lp.att_elems;
    out->set_args(a);
    out->n_lead = 0;
    out->add_lead(a.in.sums);
    out->add_lead(a.in.residual);
    out->add_lead(a.in.norm_w);
    out->add_lead(a.in.hidden);
    return FK_OK;
}

fk_status plan_xcd_layer(const Launch& la, const Launch& lm, Launch* out) {
    if (la.args_size != sizeof(XcdAttnArgs) || lm.args_size != sizeof(XcdMlpArgs))
        return set_error(FK_ERR_INVALID, "xcd layer launch: not an attention launch followed by an MLP launch");
    XcdLayerArgs t;
    memset(&t, 0, sizeof(t));
    memcpy(&t.attn, la.args, sizeof(XcdAttnArgs));
    memcpy(&t.mlp, lm.args, sizeof(XcdMlpArgs));
    const void* func = nullptr;
    if (la.func == attn_func<W_Q4>(true) && lm.func == mlp_func<W_Q4>(true)) func = layer_func<W_Q4>();
    if (la.func == attn_func<W_Q8>(true) && lm.func == mlp_func<W_Q8>(true)) func = layer_func<W_Q8>();
    if (la.func == attn_func<W_BF16>(true) && lm.func == mlp_func<W_BF16>(true)) func = layer_func<W_BF16>();
    if (!func) return set_error(FK_ERR_UNSUPPORTED, "xcd layer launch: both launches must take their one-pass flavour, same weight kind");
    if (t.attn.ctl != t.mlp.ctl) return set_error(FK_ERR_INVALID, "xcd layer launch: the two launches use different control blocks");
    if (!t.mlp.in.sums || t.mlp.in.sums != t.attn.out_sums || t.mlp.in.residual != t.attn.in.x_out ||
        t.mlp.in.hidden != t.attn.in.hidden)
        return set_error(FK_ERR_INVALID, "xcd layer launch: the MLP launch must read the sum row the attention launch adds into and the row it writes");
    if (t.attn.in.clear != t.mlp.out_sums)
        return set_error(FK_ERR_INVALID, "xcd layer launch: the attention launch must clear the row the MLP launch adds into");
    const uint32_t phase_lds = ((la.shmem > lm.shmem ? la.shmem : lm.shmem) + 15u) & ~15u;
    t.xres_off = phase_lds / 16u;
    t.mark_placement = (t.attn.mark_placement | t.mlp.mark_placement) ? 1u : 0u;
    const uint32_t lds = phase_lds + t.attn.in.hidden * 2u;
    out->func = func;
    FK_TRY(require_two_blocks_per_cu(out->func, lds, "whole-layer"));
    out->grid = dim3(kXcdGrid, 1, 1);
    out->block = dim3(kBlock, 1, 1);
    out->shmem = lds;
    out->set_args(t);
    out->n_lead = 0;
    out->add_lead(t.attn.in.sums);
    out->add_lead(t.attn.in.residual);
    out->add_lead(t.attn.in.norm_w);
    out->add_lead(t.attn.in.hidden);
    return FK_OK;
}

fk_status plan_xcd_token(const XcdAttnArgs* h_attn, const XcdMlpArgs* h_mlp, uint32_t n_layers, uint32_t bits,
                         const XcdAttnArgs* d_attn, const XcdMlpArgs* d_mlp, uint32_t attn_lds, uint32_t mlp_lds, Launch* out) {
    if (!h_attn || !h_mlp || !d_attn || !d_mlp || n_layers == 0) return set_error(FK_ERR_INVALID, "xcd token: empty layer list");
    for (uint32_t l = 0; l < n_layers; ++l) {
        if (h_attn[l].ctl != h_attn[0].ctl || h_mlp[l].ctl != h_attn[0].ctl)
            return set_error(FK_ERR_INVALID, "xcd token: every launch of the run must use the same control block");
        if (h_attn[l].in.hidden != h_attn[0].in.hidden || h_mlp[l].in.hidden != h_attn[0].in.hidden)
            return set_error(FK_ERR_INVALID, "xcd token: layers of different width");
        for (uint32_t m = 0; m < l; ++m)
            if (h_attn[l].q == h_attn[m].q || h_attn[l].k == h_attn[m].k || h_attn[l].v == h_attn[m].v)
                return set_error(FK_ERR_UNSUPPORTED, "xcd token: every layer needs its own q / k / v rows inside one launch");
    }
    XcdTokenArgs t;
    memset(&t, 0, sizeof(t));
    t.attn = d_attn;
    t.mlp = d_mlp;
    t.n_layers = n_layers;
    t.ctl = h_attn[0].ctl;
    t.spin_limit = h_attn[0].spin_limit;
    t.mark_placement = h_attn[0].mark_placement;
    const uint32_t phase_lds = ((attn_lds > mlp_lds ? attn_lds : mlp_lds) + 15u) & ~15u;
    t.xres_off = phase_lds / 16u;
    const uint32_t lds = phase_lds + h_attn[0].in.hidden * 2u;
    auto func = [&]() -> const void* {
        if (bits == 4) return reinterpret_cast<const void*>(&xcd_token_kernel<W_Q4, kNlQkv, kNlO, kNlGuToken, kNlDown>);
        if (bits == 8) return reinterpret_cast<const void*>(&xcd_token_kernel<W_Q8, kNlQkv, kNlO, kNlGuToken, kNlDown>);
        return reinterpret_cast<const void*>(&xcd_token_kernel<W_BF16, kNlQkv, kNlO, kNlGuToken, kNlDown>);
    };
    out->func = func();
    FK_TRY(require_two_blocks_per_cu(out->func, lds, "whole-token"));
    out->grid = dim3(kXcdGrid, 1, 1);
    out->block = dim3(kBlock, 1, 1);
    out->shmem = lds;
    out->set_args(t);
    return FK_OK;
}

fk_status plan_xcd_reduce(const long long* sums, const uint16_t* residual, uint16_t* x, long long* clear, uint32_t hidden,
                          Launch* out) {
    const DeviceFacts* dev;
    FK_TRY(device_facts(&dev));
    if (!sums || !residual || !x || hidden == 0) return set_error(FK_ERR_INVALID, "xcd reduce: null buffer or zero width");
    XcdReduceArgs a{sums, residual, x, clear, hidden};
    out->func = reinterpret_cast<const void*>(&xcd_reduce_kernel);
    out->grid = dim3(ceil_div(hidden, kBlock), 1, 1);
    out->block = dim3(kBlock, 1, 1);
    out->shmem = 0;
    out->set_args(a);
    return FK_OK;
}

}  // namespace fk
