// Device side of the split-K attention decode: SdpaArgs, the per-work-item
// function sdpa_block and the stand-alone kernel.  See sdpa.hip for the scheme.
#pragma once
#include <stddef.h>

#include <type_traits>

#include "fk_device.hpp"
#include "rope_device.hpp"

// Hook for timing probes: a build may define FK_SDPA_STAMP(i) to record a clock at
// phase boundary i; the library build leaves it empty.
#ifndef FK_SDPA_STAMP
#define FK_SDPA_STAMP(i)
#endif

namespace fk {

constexpr int kSdpaBlock = 256;
constexpr int kSdpaWaves = kSdpaBlock / kWave;
constexpr int kSdpaSteps = 4;       // K rows (and at most as many V rows) each lane owns per range
constexpr int kSdpaStepsFused = 4;  // inside the whole-token kernel: half the registers, twice the ranges

struct SdpaArgs {
    const uint16_t* q;
    const uint16_t* k;
    const uint16_t* v;
    uint16_t* out;
    const uint32_t* kv_len_ptr;  // device scalar, or null -> kv_len_imm
    uint32_t kv_len_imm;
    uint32_t n_heads, n_kv, qk_dim, v_dim, capacity;
    uint32_t chunk_len, n_splits;
    uint32_t chunks_per_block;  // consecutive ranges one block walks (online softmax across them)
    uint32_t rows;              // active token rows (stand-alone kernel): row r attends to kv_len + r positions
    // Quantised cache (stand-alone kernel, KVQ = 4 or 8): k / v point at packed uint32
    // [n_kv, capacity, dim * bits / 32]; scales / biases are bf16 [n_kv, capacity, dim / kv_group].
    const uint16_t* k_scales;
    const uint16_t* k_biases;
    const uint16_t* v_scales;
    const uint16_t* v_biases;
    uint32_t kv_group;
    uint32_t lpk, lpv;  // lanes per key row / value row (powers of two)
    float scale;
    float* partials;     // [n_heads][n_splits][v_dim + 2]
    uint32_t* counters;  // [n_kv * head tiles], zero before the first launch
    // Fused mode (the whole-token kernel): q, k_new, v_new are the raw projection
    // outputs of this token at position kv_len - 1.  Every block transforms its q
    // heads itself (head norm + RoPE); the block whose range holds the new position
    // transforms k_new, uses it and v_new in place of the cache row and writes both
    // into the cache.
    const uint16_t* k_new;
    const uint16_t* v_new;
    const uint16_t* q_norm;
    const uint16_t* k_norm;
    uint16_t* cache_k_w;
    uint16_t* cache_v_w;
    uint32_t rope_dims;
    float eps, base_log2;
    const float* rope_tab;  // (cos, sin) per pair at this token's position, or null
    // Heads given as two parts (low-rank keys): q0_dim != 0 means q = [Q0 | Q1] with the first rope_dims of
    // Q1 rotated, the new key row = [k_new row (k0_stride apart) | k1_new (one shared head or one per KV
    // head)] with the same rotation on its second part, v_new rows v_stride apart (both may point into one
    // packed projection output); no head norm in this form.
    const uint16_t* k1_new;
    uint32_t q0_dim, k0_stride, v_stride, k1_heads, traditional;
};

// m[GT] at 0, l[GT] at 8 (GT <= 8), the last-block flag at 16, the per-range rescale factors at 24;
// wave-local form: per-wave maxima [wave][8] at 32 and per-wave sums [wave][8] at 64.
constexpr uint32_t kSdpaStatFloats = 96;

// LDS floats one block needs.
__host__ __device__ inline uint32_t sdpa_lds_floats(uint32_t gt, uint32_t chunk, uint32_t qk_dim, uint32_t v_dim,
                                                     bool fused) {
    uint32_t lpv = 1;
    while (lpv < v_dim / 8) lpv <<= 1;
    const uint32_t slots = kSdpaBlock / lpv;  // key rows handled side by side in the value phase
    return gt * chunk + slots * gt * v_dim + kSdpaStatFloats + (fused ? (gt + 1) * qk_dim / 2 + 8 : 0);
}

// One (range, kv head, head tile) work item.  Uniform per block; `kv_len` already read.
// MODE 0: q is already rotated and the new K/V rows are in the cache.  MODE 1: a phase of the
// whole-token kernel (kv_len known on entry, coherent stores); MODE 2: a kernel of its own.  In
// modes 1 and 2 the block applies head norm + RoPE to its q heads itself, and the block whose
// range holds the new position does the same for the new k row, uses it and v_new in place of
// the cache row and appends both to the cache.
// FASTHEAD (mode 2): heads rotated over their whole width of at most 128 dims with a rotary table;
// the transforms' loads are issued ahead of the cache rows and used after them.
// NOMERGE: the caller merges the ranges' results itself: every active block writes its (m, l, o) partial with
// ordinary stores -- also when one range covers the context -- and returns; no arrival counter is touched.
template <int GT, int MODE, typename ARGS, int KVQ = 0, bool FASTHEAD = false, bool NOMERGE = false>
__device__ __forceinline__ void sdpa_block(const ARGS& a, uint32_t kv_raw, uint32_t split, uint32_t kvh,
                                           uint32_t gz, uint32_t gz_count, float* lds, uint32_t kv_add = 0) {
    // kv_raw + kv_add positions are visible (kv_add: the row's index among several active rows).  The sum is formed
    // inside settle(), behind the points where the length is first allowed to be looked at: formed by the caller, it
    // is a use of the loaded length at the very top of the kernel.
    uint32_t kv_len = 0;
    constexpr bool FUSED = MODE == 1;   // inside the whole-token kernel
    constexpr bool XFORM = MODE != 0;   // q / new-row transforms happen here
    // Tiles of up to 4 heads outside the whole-token kernel: every wave runs the online softmax
    // over its own 16 keys of a range in registers (scores never leave the lanes that computed
    // them, a key row and its value row share their lanes: the planner guarantees lpk == lpv), so
    // the ranges of a block need no barrier; the waves meet once, after the last range.
    constexpr bool WAVES = MODE != 1 && GT <= 4;
    constexpr int kSteps = FUSED ? kSdpaStepsFused : kSdpaSteps;
    static_assert(!(XFORM && KVQ != 0), "the fused forms read a bf16 cache");
    const uint32_t span = a.chunk_len * a.chunks_per_block;  // cache positions per block
    const uint32_t blk0 = split * span;
    const uint32_t G = a.n_heads / a.n_kv;
    const uint32_t h0 = kvh * G + gz * GT;
    const uint32_t gcount = (G - gz * GT) < (uint32_t)GT ? (G - gz * GT) : (uint32_t)GT;
    // Stand-alone kernel: kv_len is still on its way from memory (a scalar load the
    // caller issued); nothing below touches it until the first K/V rows have been
    // requested, so that round trip overlaps the cache reads.
    uint32_t n_active = 0, blk_keys = 0, n_chunks = 0;
    uint32_t pos = 0;  // fused: position of the new token
    auto settle = [&]() {
        // a device scalar is not trusted: a length beyond what the launch was sized for would leave ranges
        // without a block (the last-arrival count would never complete), zero would divide by an empty sum
        const uint32_t covered = a.n_splits * span < a.capacity ? a.n_splits * span : a.capacity;
        const uint32_t given = kv_raw + kv_add;
        kv_len = given < 1u ? 1u : (given > covered ? covered : given);
        pos = XFORM ? kv_len - 1 : 0u;
        n_active = (kv_len + span - 1) / span;
        if (split < n_active) {
            blk_keys = (kv_len - blk0) < span ? (kv_len - blk0) : span;
            n_chunks = (blk_keys + a.chunk_len - 1) / a.chunk_len;
        }
    };
    if constexpr (FUSED) {
        settle();
        if (split >= n_active) return;  // uniform: whole block leaves before any barrier
    }
    const uint32_t tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
    FK_SDPA_STAMP(0);

    float* s = lds;                               // [GT][chunk_len]
    float* red = s + GT * a.chunk_len;            // [value slots][GT][v_dim]
    float* stat = red + (kSdpaBlock / a.lpv) * GT * a.v_dim;  // m[GT], l[GT], misc
    uint16_t* qn = reinterpret_cast<uint16_t*>(stat + kSdpaStatFloats);  // fused: [GT][qk_dim] + k row
    uint16_t* kn = qn + GT * a.qk_dim;
    bool blk_owner = false;

    // Head norm + RoPE of this block's q heads (one wave per head), and of the new k row
    // in the block that owns its position; results in LDS as bf16.  Then one block per kv
    // head appends the new rows to the cache.
    auto head_dst = [&](uint32_t h) { return h < gcount ? qn + h * a.qk_dim : kn; };
    auto transform_heads = [&](uint32_t h_first) {
        blk_owner = pos >= blk0 && pos < blk0 + blk_keys;
        for (uint32_t h = h_first + wave; h < gcount + (blk_owner ? 1u : 0u); h += kSdpaWaves) {
            if (a.q0_dim) {
                const uint32_t d1 = a.qk_dim - a.q0_dim;
                if (h < gcount) {
                    const uint16_t* qh = a.q + (size_t)(h0 + h) * a.qk_dim;
                    split_head_transform(qh, qh + a.q0_dim, head_dst(h), a.q0_dim, d1, a.rope_dims, a.traditional != 0, pos,
                                         a.base_log2, lane, a.rope_tab);
                } else {
                    split_head_transform(a.k_new + (size_t)kvh * a.k0_stride, a.k1_new + (size_t)(a.k1_heads == 1 ? 0 : kvh) * d1,
                                         kn, a.q0_dim, d1, a.rope_dims, a.traditional != 0, pos, a.base_log2, lane, a.rope_tab);
                }
            } else if (h < gcount) {
                head_transform(a.q + (size_t)(h0 + h) * a.qk_dim, head_dst(h), a.q_norm, a.qk_dim, a.rope_dims,
                               pos, a.base_log2, a.eps, true, lane, a.rope_tab);
            } else {
                head_transform(a.k_new + (size_t)kvh * a.qk_dim, kn, a.k_norm, a.qk_dim, a.rope_dims, pos, a.base_log2,
                               a.eps, true, lane, a.rope_tab);
            }
        }
        __syncthreads();
        if (blk_owner && gz == 0) {
            const size_t row = (size_t)kvh * a.capacity + (pos % a.capacity);
            for (uint32_t d = tid; d < a.qk_dim; d += kSdpaBlock) a.cache_k_w[row * a.qk_dim + d] = kn[d];
            for (uint32_t d = tid; d < a.v_dim; d += kSdpaBlock)
                a.cache_v_w[row * a.v_dim + d] = a.v_new[(size_t)kvh * (MODE == 2 ? a.v_stride : a.v_dim) + d];
        }
    };
    // Whole-token kernel: done before the K/V loads are issued: the trigonometry needs
    // ~60 registers that the 64 registers of in-flight rows would otherwise have to share.
    if constexpr (MODE == 1) transform_heads(0);

    const uint32_t lpk = a.lpk, cpk = a.qk_dim >> 3;
    const uint32_t lpv = a.lpv, cpv = a.v_dim >> 3;
    const uint32_t ck = tid & (lpk - 1), kslot = tid / lpk, kslots = kSdpaBlock / lpk;
    const uint32_t cv = tid & (lpv - 1), vslot = tid / lpv, vslots = kSdpaBlock / lpv;
    const bool kcol_ok = ck < cpk, vcol_ok = cv < cpv;

    // Running softmax state per head (m, l) in LDS; the value accumulators stay in
    // registers across ranges: a lane owns the same 8 output dims in every range.
    if (tid < (uint32_t)GT) {
        stat[tid] = -INFINITY;
        stat[8 + tid] = 0.f;
    }
    float m_run[GT], l_run[GT];  // wave-local form: running maximum (uniform) and this lane row's share of the sum
#pragma unroll
    for (int h = 0; h < GT; ++h) {
        m_run[h] = -INFINITY;
        l_run[h] = 0.f;
    }
    float acc[GT][8];
    float accb[GT];  // quantised V: sum_j p_j * bias_j of this lane's group, added to its 8 dims at the end
#pragma unroll
    for (int h = 0; h < GT; ++h) {
        accb[h] = 0.f;
#pragma unroll
        for (int i = 0; i < 8; ++i) acc[h][i] = 0.f;
    }

    // This lane's 8 dims of each query head; fetched before the K/V rows so that the
    // scores can start as soon as the first keys arrive (loads return in order).
    // The request is straight-line (a lane past the head width or a head past the tile reads a valid address and
    // is zeroed afterwards): with the load under a condition the compiler waits for it where the paths join, i.e.
    // before the K/V rows are requested -- a whole trip to memory at the start of every block.  settle_q zeroes the
    // unused lanes and derives what the quantised forms need; it runs behind the first K/V request.
    uint4 qf[GT];
    float sq[GT];  // quantised K: sum of this lane's 8 query dims (the affine bias term b * sum q)
    auto load_q = [&]() {
#pragma unroll
        for (int h = 0; h < GT; ++h) {
            const uint32_t hc = (uint32_t)h < gcount ? (uint32_t)h : 0u, cc = kcol_ok ? ck : 0u;
            if constexpr (XFORM)
                qf[h] = *reinterpret_cast<const uint4*>(qn + hc * a.qk_dim + 8 * cc);
            else
                qf[h] = *reinterpret_cast<const uint4*>(a.q + (size_t)(h0 + hc) * a.qk_dim + 8 * cc);
        }
    };
    auto settle_q = [&]() {
#pragma unroll
        for (int h = 0; h < GT; ++h) {
            pin_u128(qf[h]);  // looked at only from here on
            if (!(kcol_ok && (uint32_t)h < gcount)) qf[h] = make_uint4(0, 0, 0, 0);
            if constexpr (KVQ != 0) {
                const uint4 v = qf[h];
                sq[h] = ((bf16_lo(v.x) + bf16_hi(v.x)) + (bf16_lo(v.y) + bf16_hi(v.y))) +
                        ((bf16_lo(v.z) + bf16_hi(v.z)) + (bf16_lo(v.w) + bf16_hi(v.w)));
                if constexpr (KVQ == 4)  // nibble pairing of q4_word_dot: (x0,x2) (x4,x6) (x1,x3) (x5,x7)
                    qf[h] = make_uint4((v.x & 0xffffu) | (v.y << 16), (v.z & 0xffffu) | (v.w << 16),
                                       (v.x >> 16) | (v.y & 0xffff0000u), (v.z >> 16) | (v.w & 0xffff0000u));
            }
        }
    };
    if constexpr (MODE != 2) load_q();
    if constexpr (MODE == 1) settle_q();  // whole-token kernel: q comes from LDS, its rows are requested per range

    // All K and V loads of a range are issued up front (the range is sized so that
    // each lane owns kSteps rows of each), so one HBM round trip covers both phases.
    // Stand-alone: every row that exists in the cache allocation is requested, whether
    // or not it is below kv_len (rows past kv_len are masked where they are used).
    uint4 kc[kSteps], vc[kSteps];
    uint4 kn_[kSteps], vn_[kSteps];  // stand-alone: the next range, in flight while this one is consumed
    auto request_rows = [&](uint4(&kd)[kSteps], uint4(&vd)[kSteps], uint32_t key0, uint32_t nkeys, bool owner,
                            uint32_t jpos) {
        const uint16_t* kbase = a.k + ((size_t)kvh * a.capacity + key0) * a.qk_dim + 8 * ck;
        const uint16_t* vbase = a.v + ((size_t)kvh * a.capacity + key0) * a.v_dim + 8 * cv;
        if constexpr (KVQ != 0) {
            // 8 dims per lane as in the bf16 layout: one packed word (int4) or two (int8) in
            // .x / .y, the group's scale and bias bits in .z; rows clamped as below.
            constexpr uint32_t WPL = KVQ == 4 ? 1u : 2u;
            const uint32_t kw = a.qk_dim * KVQ / 32u, vw = a.v_dim * KVQ / 32u;
            const uint32_t kg = a.qk_dim / a.kv_group, vg = a.v_dim / a.kv_group;
            const uint32_t kcol = kcol_ok ? ck : 0u, vcol = vcol_ok ? cv : 0u;
            const uint32_t* kp = reinterpret_cast<const uint32_t*>(a.k) + (size_t)kvh * a.capacity * kw + kcol * WPL;
            const uint32_t* vp = reinterpret_cast<const uint32_t*>(a.v) + (size_t)kvh * a.capacity * vw + vcol * WPL;
            const size_t kmeta = (size_t)kvh * a.capacity * kg + (8u * kcol) / a.kv_group;
            const size_t vmeta = (size_t)kvh * a.capacity * vg + (8u * vcol) / a.kv_group;
            const uint32_t last = a.capacity - 1;
#pragma unroll
            for (int u = 0; u < kSteps; ++u) {
                const uint32_t r0 = key0 + kslot + u * kslots, r = r0 < last ? r0 : last;
                kd[u].x = kp[(size_t)r * kw];
                kd[u].y = WPL == 2 ? kp[(size_t)r * kw + 1] : 0u;
                kd[u].z = (uint32_t)a.k_scales[kmeta + (size_t)r * kg] | ((uint32_t)a.k_biases[kmeta + (size_t)r * kg] << 16);
                kd[u].w = 0u;
            }
#pragma unroll
            for (int u = 0; u < kSteps; ++u) {
                const uint32_t r0 = key0 + vslot + u * vslots, r = r0 < last ? r0 : last;
                vd[u].x = vp[(size_t)r * vw];
                vd[u].y = WPL == 2 ? vp[(size_t)r * vw + 1] : 0u;
                vd[u].z = (uint32_t)a.v_scales[vmeta + (size_t)r * vg] | ((uint32_t)a.v_biases[vmeta + (size_t)r * vg] << 16);
                vd[u].w = 0u;
            }
            return;
        }
        if constexpr (MODE != 1) {
            // Straight-line, clamped (row to the last row of the allocation, a lane beyond
            // the head width to column 0): no branch separates the loads, so the compiler
            // can wait for exactly the rows it needs while later requests stay in flight.
            const uint16_t* khead = a.k + (size_t)kvh * a.capacity * a.qk_dim + (kcol_ok ? 8 * ck : 0u);
            const uint16_t* vhead = a.v + (size_t)kvh * a.capacity * a.v_dim + (vcol_ok ? 8 * cv : 0u);
            const uint32_t last = a.capacity - 1;
#pragma unroll
            for (int u = 0; u < kSteps; ++u) {
                const uint32_t r = key0 + kslot + u * kslots;
                kd[u] = *reinterpret_cast<const uint4*>(khead + (size_t)(r < last ? r : last) * a.qk_dim);
            }
#pragma unroll
            for (int u = 0; u < kSteps; ++u) {
                const uint32_t r = key0 + vslot + u * vslots;
                vd[u] = *reinterpret_cast<const uint4*>(vhead + (size_t)(r < last ? r : last) * a.v_dim);
            }
            return;
        }
#pragma unroll
        for (int u = 0; u < kSteps; ++u) {
            const uint32_t j = kslot + u * kslots;
            kd[u] = make_uint4(0, 0, 0, 0);
            if (kcol_ok && j < nkeys && !(owner && j == jpos))
                kd[u] = *reinterpret_cast<const uint4*>(kbase + (size_t)j * a.qk_dim);
        }
#pragma unroll
        for (int u = 0; u < kSteps; ++u) {
            const uint32_t j = vslot + u * vslots;
            vd[u] = make_uint4(0, 0, 0, 0);
            if (vcol_ok && j < nkeys) {
                const uint16_t* src = vbase + (size_t)j * a.v_dim;
                if (owner && j == jpos) {  // the new row, not yet cached
                    vd[u] = *reinterpret_cast<const uint4*>(a.v_new + (size_t)kvh * a.v_dim + 8 * cv);
                } else {
                    vd[u] = *reinterpret_cast<const uint4*>(src);
                }
            }
        }
    };
    uint4 vnew = make_uint4(0, 0, 0, 0);  // mode 2: this lane's 8 dims of the new V row
    if constexpr (MODE != 1) {
        // Mode 2, fast heads: every wave requests the inputs of two heads (its own index and
        // that plus the wave count; index gcount is the new k row) before the cache rows, so
        // they arrive first and the transforms run while the rows are still in flight.
        HeadPair ha, hb;
        const uint32_t half = a.qk_dim >> 1, hi_a = wave, hi_b = wave + kSdpaWaves;
        if constexpr (MODE == 2 && FASTHEAD) {
            auto src = [&](uint32_t h) {
                return h < gcount ? a.q + (size_t)(h0 + h) * a.qk_dim : a.k_new + (size_t)kvh * a.qk_dim;
            };
            ha = head_pair_fetch(src(hi_a), hi_a < gcount ? a.q_norm : a.k_norm, a.rope_tab, half, lane);
            hb = head_pair_fetch(src(hi_b), hi_b < gcount ? a.q_norm : a.k_norm, a.rope_tab, half, lane);
        }
        // The first range always exists and is requested before kv_len has arrived.  Later
        // ranges wait for it (it was the kernel's first request and is long back by now):
        // a fixed grid sized for the whole cache would otherwise read every range's rows
        // each launch, megabytes of traffic for a context of a few hundred tokens.
        // (kv_len is made opaque at both places where it is first looked at: settle() runs on both paths, and
        // the compiler otherwise computes its common part once, AHEAD of the branch -- the first range's request
        // then waits for the length after all)
        if (split != 0) {
            asm volatile("" : "+v"(kv_raw));
            settle();
            if (split >= n_active) return;
        }
        request_rows(kc, vc, blk0, 0, false, 0);
        if constexpr (MODE == 0) settle_q();
        if constexpr (MODE == 2)
            vnew = *reinterpret_cast<const uint4*>(a.v_new + (size_t)kvh * a.v_stride + (vcol_ok ? 8 * cv : 0u));
        asm volatile("" : "+v"(kv_raw));
        settle();
        if (split >= n_active) return;  // uniform: whole block leaves before any barrier
        if constexpr (MODE == 2) {
            if constexpr (FASTHEAD) {
                const bool own = pos >= blk0 && pos < blk0 + blk_keys;
                head_pair_apply(ha, head_dst(hi_a), a.q_norm != nullptr, half, a.eps, lane,
                                hi_a < gcount || (hi_a == gcount && own));
                head_pair_apply(hb, head_dst(hi_b), a.q_norm != nullptr, half, a.eps, lane,
                                hi_b < gcount || (hi_b == gcount && own));
                transform_heads(2 * kSdpaWaves);  // a ninth head (tile of 8 plus the k row), barrier, cache append
            } else {
                // the transforms' own loads queue behind the cache rows requested above; q comes
                // back from LDS rotated
                transform_heads(0);
            }
            load_q();
            settle_q();
        }
    }

    for (uint32_t c = 0; c < n_chunks; ++c) {
    const uint32_t key0 = blk0 + c * a.chunk_len;
    const uint32_t nkeys = (kv_len - key0) < a.chunk_len ? (kv_len - key0) : a.chunk_len;
    const bool owner = XFORM && pos >= key0 && pos < key0 + nkeys;
    const uint32_t jpos = pos - key0;
    if constexpr (FUSED) {
        request_rows(kc, vc, key0, nkeys, owner, jpos);
    } else {
        if (c + 1 < n_chunks) request_rows(kn_, vn_, key0 + a.chunk_len, 0, false, 0);
    }

    FK_SDPA_STAMP(1);
    if constexpr (XFORM) {
        if (owner && kcol_ok) {
#pragma unroll
            for (int u = 0; u < kSteps; ++u)
                if (kslot + u * kslots == jpos) kc[u] = *reinterpret_cast<const uint4*>(kn + 8 * ck);
        }
    }
    // q . k of key row u and head h, complete in every lane of the row
    auto score = [&](int u, int h) {
        float d = 0.f;
        if constexpr (KVQ == 4) {
            d = q4_word_dot(kc[u].x, qf[h], 0.f);
            d = fmaf(bf16_lo(kc[u].z), d, bf16_hi(kc[u].z) * sq[h]);  // s * sum(q * code) + b * sum(q)
        } else if constexpr (KVQ == 8) {
            const uint32_t w0 = kc[u].x, w1 = kc[u].y;
            d = dot2_bf16(pack_bf16((float)(w0 & 0xffu), (float)((w0 >> 8) & 0xffu)), qf[h].x, d);
            d = dot2_bf16(pack_bf16((float)((w0 >> 16) & 0xffu), (float)(w0 >> 24)), qf[h].y, d);
            d = dot2_bf16(pack_bf16((float)(w1 & 0xffu), (float)((w1 >> 8) & 0xffu)), qf[h].z, d);
            d = dot2_bf16(pack_bf16((float)((w1 >> 16) & 0xffu), (float)(w1 >> 24)), qf[h].w, d);
            d = fmaf(bf16_lo(kc[u].z), d, bf16_hi(kc[u].z) * sq[h]);
        } else {
            d = dot2_bf16(kc[u].x, qf[h].x, d);
            d = dot2_bf16(kc[u].y, qf[h].y, d);
            d = dot2_bf16(kc[u].z, qf[h].z, d);
            d = dot2_bf16(kc[u].w, qf[h].w, d);
        }
        return d;  // this lane's 8 dims only: scores_of() finishes the dot over the row's lanes
    };
    // All scores of the range: the per-lane dots first, then ONE uniform choice of the row width
    // around the cross-lane sums (a width test inside every sum costs six scalar branches each).
    auto scores_of = [&](float(&d)[kSteps][GT]) {
#pragma unroll
        for (int u = 0; u < kSteps; ++u)
#pragma unroll
            for (int h = 0; h < GT; ++h) d[u][h] = score(u, h);
        auto reduce = [&](auto width) {
#pragma unroll
            for (int u = 0; u < kSteps; ++u)
#pragma unroll
                for (int h = 0; h < GT; ++h) d[u][h] = group_sum(d[u][h], decltype(width)::value);
        };
        if (lpk == 16) reduce(std::integral_constant<int, 16>{});
        else if (lpk == 8) reduce(std::integral_constant<int, 8>{});
        else if (lpk == 32) reduce(std::integral_constant<int, 32>{});
        else if (lpk == 64) reduce(std::integral_constant<int, 64>{});
        else if (lpk == 4) reduce(std::integral_constant<int, 4>{});
        else if (lpk == 2) reduce(std::integral_constant<int, 2>{});
    };
    // This lane's 8 dims of value row u as floats (quantised: the codes; `vs`, `vb` the group's
    // scale and bias).  Rows past kv_len were requested speculatively: their bits may be
    // anything, so they are zeroed.
    auto value = [&](int u, uint32_t j, float(&f)[8], float& vs, float& vb) {
        const bool ok = j < nkeys && vcol_ok;
        if constexpr (KVQ != 0) {
            vs = ok ? bf16_lo(vc[u].z) : 0.f;
            vb = ok ? bf16_hi(vc[u].z) : 0.f;
            if constexpr (KVQ == 4) {
                const uint32_t even = vc[u].x & 0x0F0F0F0Fu, odd = (vc[u].x >> 4) & 0x0F0F0F0Fu;
                f[0] = (float)(even & 0xffu); f[2] = (float)((even >> 8) & 0xffu);
                f[4] = (float)((even >> 16) & 0xffu); f[6] = (float)(even >> 24);
                f[1] = (float)(odd & 0xffu); f[3] = (float)((odd >> 8) & 0xffu);
                f[5] = (float)((odd >> 16) & 0xffu); f[7] = (float)(odd >> 24);
            } else {
                const uint32_t w0 = vc[u].x, w1 = vc[u].y;
                f[0] = (float)(w0 & 0xffu); f[1] = (float)((w0 >> 8) & 0xffu);
                f[2] = (float)((w0 >> 16) & 0xffu); f[3] = (float)(w0 >> 24);
                f[4] = (float)(w1 & 0xffu); f[5] = (float)((w1 >> 8) & 0xffu);
                f[6] = (float)((w1 >> 16) & 0xffu); f[7] = (float)(w1 >> 24);
            }
        } else {
            vs = 1.f;
            vb = 0.f;
            uint4 vv = (FUSED || ok) ? vc[u] : make_uint4(0, 0, 0, 0);
            if constexpr (MODE == 2) {
                if (owner && j == jpos && vcol_ok) vv = vnew;  // the new row, not yet cached
            }
            f[0] = bf16_lo(vv.x); f[1] = bf16_hi(vv.x); f[2] = bf16_lo(vv.y); f[3] = bf16_hi(vv.y);
            f[4] = bf16_lo(vv.z); f[5] = bf16_hi(vv.z); f[6] = bf16_lo(vv.w); f[7] = bf16_hi(vv.w);
        }
    };

    if constexpr (WAVES) {
        // ---------------- wave-local: scores, online softmax and value sums in registers ----------------
        // Scores and running maxima are kept in base-2 units (scale * log2(e) folded into one
        // multiply), so a probability is one v_exp_f32.
        float pr[kSteps][GT];
        scores_of(pr);
        const float scale2 = a.scale * 1.44269504088896341f;
#pragma unroll
        for (int u = 0; u < kSteps; ++u) {
            const bool live = kslot + u * kslots < nkeys;
#pragma unroll
            for (int h = 0; h < GT; ++h) pr[u][h] = live ? pr[u][h] * scale2 : -INFINITY;
        }
        float mx[GT];
#pragma unroll
        for (int h = 0; h < GT; ++h) {
            mx[h] = pr[0][h];
#pragma unroll
            for (int u = 1; u < kSteps; ++u) mx[h] = fmaxf(mx[h], pr[u][h]);
        }
        if (lpk < 16) {  // two or more key rows share a 16-lane row: finish the maximum inside it
#pragma unroll
            for (int h = 0; h < GT; ++h) {
                mx[h] = dpp_max<0xB1>(mx[h]);
                mx[h] = dpp_max<0x4E>(mx[h]);
                mx[h] = dpp_max<0x141>(mx[h]);
                mx[h] = dpp_max<0x140>(mx[h]);
            }
        }
#pragma unroll
        for (int h = 0; h < GT; ++h) {
            // every 16-lane row is uniform now: the wave's maximum is that of lanes 0, 16, 32, 48
            const float r0 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(mx[h]), 0));
            const float r1 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(mx[h]), 16));
            const float r2 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(mx[h]), 32));
            const float r3 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(mx[h]), 48));
            const float m_new = fmaxf(fmaxf(m_run[h], fmaxf(r0, r1)), fmaxf(r2, r3));
            const float m_ref = m_new == -INFINITY ? 0.f : m_new;  // no live key yet: every term below is 2^-inf = 0
            const float alpha = __builtin_amdgcn_exp2f(m_run[h] - m_ref);
            float psum = 0.f;
#pragma unroll
            for (int u = 0; u < kSteps; ++u) {
                pr[u][h] = __builtin_amdgcn_exp2f(pr[u][h] - m_ref);
                psum += pr[u][h];
            }
            l_run[h] = fmaf(l_run[h], alpha, psum);
            m_run[h] = m_new;
            if (alpha != 1.f) {  // the maximum rose (rare after the first ranges)
                accb[h] *= alpha;
#pragma unroll
                for (int i = 0; i < 8; ++i) acc[h][i] *= alpha;
            }
        }
#pragma unroll
        for (int u = 0; u < kSteps; ++u) {
            float f[8], vs, vb;
            value(u, vslot + u * vslots, f, vs, vb);
#pragma unroll
            for (int h = 0; h < GT; ++h) {
                const float p = pr[u][h];
                const float ps = KVQ != 0 ? p * vs : p;
                if constexpr (KVQ != 0) accb[h] = fmaf(p, vb, accb[h]);
#pragma unroll
                for (int i = 0; i < 8; ++i) acc[h][i] = fmaf(ps, f[i], acc[h][i]);
            }
        }
    } else {
    // ---------------- phase A: scores ----------------
    {
        float d[kSteps][GT];
        scores_of(d);
#pragma unroll
        for (int u = 0; u < kSteps; ++u) {
            const uint32_t j = kslot + u * kslots;
#pragma unroll
            for (int h = 0; h < GT; ++h)
                if (ck == 0 && j < nkeys) s[h * a.chunk_len + j] = d[u][h] * a.scale;
        }
    }
    FK_SDPA_STAMP(2);
    __syncthreads();
    FK_SDPA_STAMP(3);

    // ---------------- softmax over this range, one wave per head ----------------
    // Online form: the running maximum may rise, in which case what was summed so
    // far is rescaled by alpha = exp(m_old - m_new) (0 for the first range).
    for (uint32_t h = wave; h < gcount; h += kSdpaWaves) {
        float* sh = s + h * a.chunk_len;
        const float m_old = stat[h], l_old = stat[8 + h];
        float m = m_old;
        for (uint32_t j = lane; j < nkeys; j += kWave) m = fmaxf(m, sh[j]);
        m = wave_max(m);
        float l = 0.f;
        for (uint32_t j = lane; j < nkeys; j += kWave) {
            const float p = expf(sh[j] - m);
            sh[j] = p;
            l += p;
        }
        l = wave_sum(l);
        if (lane == 0) {
            const float alpha = c ? expf(m_old - m) : 0.f;
            stat[h] = m;
            stat[8 + h] = c ? fmaf(l_old, alpha, l) : l;
            stat[24 + h] = alpha;
        }
    }
    __syncthreads();

    FK_SDPA_STAMP(4);
    // ---------------- phase B: o = sum_j p_j v_j ----------------
    if (c) {
#pragma unroll
        for (int h = 0; h < GT; ++h) {
            const float alpha = stat[24 + h];
#pragma unroll
            for (int i = 0; i < 8; ++i) acc[h][i] *= alpha;
            accb[h] *= alpha;
        }
    }
#pragma unroll
    for (int u = 0; u < kSteps; ++u) {
        const uint32_t j = vslot + u * vslots;
        const uint32_t jj = j < nkeys ? j : 0u;
        const float live = j < nkeys ? 1.f : 0.f;
        float f[8], vs, vb;
        value(u, j, f, vs, vb);
#pragma unroll
        for (int h = 0; h < GT; ++h) {
            const float p = s[h * a.chunk_len + jj] * live;
            const float ps = KVQ != 0 ? p * vs : p;
            if constexpr (KVQ != 0) accb[h] = fmaf(p, vb, accb[h]);
#pragma unroll
            for (int i = 0; i < 8; ++i) acc[h][i] = fmaf(ps, f[i], acc[h][i]);
        }
    }
    }
    if (c + 1 < n_chunks) {
        if constexpr (!WAVES) __syncthreads();  // the scores are overwritten by the next range
        if constexpr (MODE != 1) {
#pragma unroll
            for (int u = 0; u < kSteps; ++u) {
                kc[u] = kn_[u];
                vc[u] = vn_[u];
            }
        }
    }
    }  // ranges of this block
    FK_SDPA_STAMP(5);

    if constexpr (WAVES) {
        // The waves meet: maxima through LDS, every wave rescales its sums to the block's
        // maximum (exp(-inf) = 0 for a wave that saw no live key) and publishes its share of l.
        float* wm = stat + 32;
        float* wl = stat + 64;
        if (lane == 0) {
#pragma unroll
            for (int h = 0; h < GT; ++h) wm[wave * 8 + h] = m_run[h];
        }
        __syncthreads();
        const float inv_lanes = 1.0f / (float)lpk;  // a row's sum is held by each of its lpk lanes (power of two: exact)
#pragma unroll
        for (int h = 0; h < GT; ++h) {
            float M = wm[h];
#pragma unroll
            for (int w = 1; w < kSdpaWaves; ++w) M = fmaxf(M, wm[w * 8 + h]);
            const float f = __builtin_amdgcn_exp2f(m_run[h] - M);
            accb[h] *= f;
#pragma unroll
            for (int i = 0; i < 8; ++i) acc[h][i] *= f;
            const float lw = wave_sum(l_run[h]) * inv_lanes * f;
            if (lane == 0) wl[wave * 8 + h] = lw;
            if (tid == 0) stat[h] = M * 0.693147180559945309f;  // back to natural units for the (m, l, o) partials
        }
    }
    // Every lane parks its sums in LDS, [value slot][head][dim]; the output loop below
    // adds the slots in index order (no cross-lane shuffles, fixed order).
    if constexpr (KVQ != 0) {
#pragma unroll
        for (int h = 0; h < GT; ++h)
#pragma unroll
            for (int i = 0; i < 8; ++i) acc[h][i] += accb[h];
    }
    if (vcol_ok) {
#pragma unroll
        for (int h = 0; h < GT; ++h) {
            float4* dst = reinterpret_cast<float4*>(red + ((size_t)vslot * GT + h) * a.v_dim + 8 * cv);
            dst[0] = make_float4(acc[h][0], acc[h][1], acc[h][2], acc[h][3]);
            dst[1] = make_float4(acc[h][4], acc[h][5], acc[h][6], acc[h][7]);
        }
    }
    __syncthreads();
    if constexpr (WAVES) {
        if (tid < (uint32_t)GT) {
            const float* wl = stat + 64;
            float l = wl[tid];
#pragma unroll
            for (int w = 1; w < kSdpaWaves; ++w) l += wl[w * 8 + tid];
            stat[8 + tid] = l;
        }
        __syncthreads();
    }

    FK_SDPA_STAMP(6);
    const uint32_t n_out = gcount * a.v_dim;
    const bool direct = !NOMERGE && (n_active == 1);
    for (uint32_t e = tid; e < n_out; e += kSdpaBlock) {
        const uint32_t h = e / a.v_dim, d = e - h * a.v_dim;
        float o = 0.f;
        for (uint32_t sl = 0; sl < vslots; ++sl) o += red[(sl * GT + h) * a.v_dim + d];
        if (direct) {
            st_u16<FUSED>(a.out + (size_t)(h0 + h) * a.v_dim + d, f32_to_bf16_bits(o / stat[8 + h]));
        } else {
            float* p = a.partials + ((size_t)(h0 + h) * a.n_splits + split) * (a.v_dim + 2);
            st_f32<!NOMERGE>(p + 2 + d, o);
            if (d == 0) {
                st_f32<!NOMERGE>(p, stat[h]);
                st_f32<!NOMERGE>(p + 1, stat[8 + h]);
            }
        }
    }
    FK_SDPA_STAMP(7);
    if (direct || NOMERGE) return;

    // ---------------- last block merges the partials ----------------
    // Partials and the arrival counter move through agent-scope (write-through /
    // cache-bypassing) accesses, so no device-wide fence is needed: every wave waits
    // until its own stores have landed, the block barrier collects the waves, then one
    // thread counts the block in.
    wait_memory_ops_done();
    __syncthreads();
    uint32_t* flag = reinterpret_cast<uint32_t*>(stat + 16);
    if (tid == 0) {
        const uint32_t prev = atomicAdd(&a.counters[kvh * gz_count + gz], 1u);
        *flag = (prev == n_active - 1) ? 1u : 0u;
    }
    __syncthreads();
    FK_SDPA_STAMP(8);
    if (*flag == 0u) return;
    if (tid == 0)  // ready for the next launch (or the next layer of this one)
        __hip_atomic_store(&a.counters[kvh * gz_count + gz], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);

    // One wave per head, no block barriers.  The ranges are taken 16 at a time and folded
    // into a running (M, L, o) with the usual rescaling, in range order, so the result does
    // not depend on arrival order.  Per batch a lane issues 17 eight-byte loads: (m, l) of
    // range base + (lane % 16), handed to the other lanes through scalar registers, and its
    // own two output dims of each of the 16 ranges; the next batch's loads are in flight
    // while the current one is folded in.
    constexpr uint32_t kBatch = 16;
    const uint32_t row = a.v_dim + 2;
    for (uint32_t h = wave; h < gcount; h += kSdpaWaves) {
        const float* ph = a.partials + (size_t)(h0 + h) * a.n_splits * row;
        for (uint32_t d2 = lane; d2 < ((a.v_dim >> 1) + kWave - 1) / kWave * kWave; d2 += kWave) {
            const bool live = d2 < (a.v_dim >> 1);
            const float* pd = ph + 2 + 2 * (live ? d2 : 0u);
            float M = -INFINITY, L = 0.f, o0 = 0.f, o1 = 0.f;
            auto fetch = [&](uint32_t base, float2& ml, float2(&po)[kBatch]) {
                const uint32_t mine = base + (lane & (kBatch - 1));
                ml = ld_f32x2<true>(ph + (size_t)(mine < n_active ? mine : base) * row);
#pragma unroll
                for (uint32_t i = 0; i < kBatch; ++i)
                    po[i] = ld_f32x2<true>(pd + (size_t)(base + i < n_active ? base + i : base) * row);
            };
            auto fold = [&](uint32_t base, const float2& ml, const float2(&po)[kBatch]) {
                float pm[kBatch], pl[kBatch];
#pragma unroll
                for (uint32_t i = 0; i < kBatch; ++i) {
                    pm[i] = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(ml.x), i));
                    pl[i] = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(ml.y), i));
                }
                float mn = fmaxf(M, pm[0]);
#pragma unroll
                for (uint32_t i = 1; i < kBatch; ++i) mn = base + i < n_active ? fmaxf(mn, pm[i]) : mn;
                const float alpha = base ? expf(M - mn) : 0.f;
                L *= alpha;
                o0 *= alpha;
                o1 *= alpha;
#pragma unroll
                for (uint32_t i = 0; i < kBatch; ++i) {
                    const float w = base + i < n_active ? expf(pm[i] - mn) : 0.f;
                    L = fmaf(pl[i], w, L);
                    o0 = fmaf(po[i].x, w, o0);
                    o1 = fmaf(po[i].y, w, o1);
                }
                M = mn;
            };
            float2 ml_a, ml_b, po_a[kBatch], po_b[kBatch];
            uint32_t base = 0;
            fetch(0, ml_a, po_a);
            while (base + kBatch < n_active) {  // straight-line body: request the next batch, fold this one
                fetch(base + kBatch, ml_b, po_b);
                fold(base, ml_a, po_a);
                ml_a = ml_b;
#pragma unroll
                for (uint32_t i = 0; i < kBatch; ++i) po_a[i] = po_b[i];
                base += kBatch;
            }
            fold(base, ml_a, po_a);
            const float inv_l = 1.0f / L;
            if (live) {
                uint16_t* dst = a.out + (size_t)(h0 + h) * a.v_dim + 2 * d2;
                st_u16<FUSED>(dst, f32_to_bf16_bits(o0 * inv_l));
                st_u16<FUSED>(dst + 1, f32_to_bf16_bits(o1 * inv_l));
            }
        }
    }
    FK_SDPA_STAMP(9);
}

// The context length of a stand-alone launch: ONE unconditional load (a load under a branch would be waited for at
// the join, ahead of the cache reads it is meant to overlap) through a GLOBAL pointer -- the device scalar, or the
// immediate's own place in the kernel-argument segment.  (Selected as generic pointers the two make a flat load,
// and a flat load's completion can only be awaited with vmcnt(0): every cache row requested behind it would be
// waited for with it.)
__device__ __forceinline__ uint32_t sdpa_load_kv_len(const SdpaArgs& a) {
#if defined(__HIP_DEVICE_COMPILE__)
    typedef const __attribute__((address_space(1))) uint32_t* global_u32;
    const global_u32 imm = (global_u32)((uintptr_t)__builtin_amdgcn_kernarg_segment_ptr() + offsetof(SdpaArgs, kv_len_imm));
    const global_u32 dev = (global_u32)(uintptr_t)a.kv_len_ptr;
    return *(a.kv_len_ptr ? dev : imm);
#else
    return a.kv_len_ptr ? *a.kv_len_ptr : a.kv_len_imm;
#endif
}

template <int GT, int KVQ = 0>
__global__ __launch_bounds__(kSdpaBlock) void sdpa_decode_kernel(const SdpaArgs a) {
    extern __shared__ __align__(16) float lds[];
    // One unconditional load (the immediate is read from the kernel-argument segment
    // when there is no device scalar): a load under a branch would be waited for at
    // the join, ahead of the cache reads it is meant to overlap.
    kernarg_warm<(int)sizeof(SdpaArgs)>();
    const uint32_t kv_len0 = sdpa_load_kv_len(a);
    if (a.rows <= 1) {
        sdpa_block<GT, false, SdpaArgs, KVQ>(a, kv_len0, blockIdx.x, blockIdx.y, blockIdx.z, gridDim.z, lds);
        return;
    }
    // Several active rows (multi-token verification, chunked prefill): grid.z carries
    // (row, head tile).  Row r is the token at position kv_len0 - 1 + r: it attends to
    // kv_len0 + r cache rows (causal inside the group), with its own q, out and workspace.
    const uint32_t gz_count = gridDim.z / a.rows;
    const uint32_t tr = blockIdx.z / gz_count, gz = blockIdx.z - tr * gz_count;
    SdpaArgs r = a;
    r.q = a.q + (size_t)tr * a.n_heads * a.qk_dim;
    r.out = a.out + (size_t)tr * a.n_heads * a.v_dim;
    r.partials = a.partials + (size_t)tr * a.n_heads * a.n_splits * (a.v_dim + 2);
    r.counters = a.counters + (size_t)tr * a.n_kv * gz_count;
    sdpa_block<GT, false, SdpaArgs, KVQ>(r, kv_len0, blockIdx.x, blockIdx.y, gz, gz_count, lds, tr);
}

// RoPE (+ head norm) of q and of the new k row, the cache append and the attention in one
// launch: a.q / a.k_new / a.v_new are the raw projection outputs of the token at position
// kv_len - 1, a.k / a.v the cache it is appended to.
template <int GT, bool FASTHEAD>
__global__ __launch_bounds__(kSdpaBlock) void sdpa_rope_store_kernel(const SdpaArgs a) {
    extern __shared__ __align__(16) float lds[];
    kernarg_warm<(int)sizeof(SdpaArgs)>();
    const uint32_t kv_len0 = sdpa_load_kv_len(a);
    sdpa_block<GT, 2, SdpaArgs, 0, FASTHEAD>(a, kv_len0, blockIdx.x, blockIdx.y, blockIdx.z, gridDim.z, lds);
}

}  // namespace fk
