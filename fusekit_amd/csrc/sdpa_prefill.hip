// Causal attention for a group of token rows (chunked prompt prefill, multi-token
// verification) on the gfx950 matrix cores.  Semantics of the reference's prefill kernel
// (src/codegen/kernels/sdpa_prefill.rs:1-205): row l_q of the group sits at position
// q_kv = (kv_len - L) + l_q and sees cache positions 0 .. q_kv; scores and softmax in
// fp32, one rounding of the output.  The reference runs one threadgroup per (row, head)
// with all scores in threadgroup memory (kv_len <= 4096); here the scores never leave
// registers and kv_len is bounded by the cache only.
//
// Two forms share the arithmetic.  Up to 64 rows (few rows, possibly a long cache):
// one block = one query head x 32 consecutive rows; its four waves take the 64-position
// steps of the visible range round-robin (wave w: steps w, w + 4, ...), each with its own
// running (reference, sum, output), and the four are merged once at the end in wave order.
// More rows: one block = one head x 128 rows, a 32-row tile per wave, K and V shared through
// LDS (described at sdpa_prefill_tile_kernel below).
//
// Per step a wave computes, with v_mfma_f32_32x32x16_bf16,
//     S^T[kv, q] = K[kv, :] . Q[q, :]        A = K rows (read from the cache as they lie),
//                                            B = Q rows (in registers for the whole kernel)
// so that a lane owns ONE query (column q = lane % 32) and 32 of the 64 scores of it: the
// softmax statistics are lane-local plus one exchange between the two half-waves, and the
// rescale of the output accumulators is lane-local too, because the second product is
//     O^T[d, q] += V^T[d, kv] . P^T[kv, q]   A = V^T, B = P^T = the score registers as they lie.
// Only V needs a transposition: the step's V rows are written through LDS as [d][kv] (two
// bytes at a time), in the order of kv that makes a lane's eight values of one matrix
// instruction contiguous.  Both products run over an index (d for the first, kv for the
// second) whose order inside the instruction is free as long as A and B agree, which is what
// lets every global read be a contiguous run per lane.
#include <type_traits>
#include <utility>

#include "fk_device.hpp"
#include "fk_host.hpp"

namespace fk {

typedef __bf16 pf_bf16x8_t __attribute__((ext_vector_type(8)));
typedef float pf_f32x16_t __attribute__((ext_vector_type(16)));
typedef unsigned int pf_u32x2_t __attribute__((ext_vector_type(2)));
typedef unsigned int pf_u32x4_t __attribute__((ext_vector_type(4)));

constexpr int kPrefillBlock = 256;
constexpr uint32_t kPrefillWaves = 4;
constexpr uint32_t kPrefillRows = 32;    // query rows per block
constexpr uint32_t kPrefillStep = 64;    // cache positions per wave step
constexpr uint32_t kPrefillVtStride = kPrefillStep + 8;  // bf16 per row of the transposed V tile (rows stay 16-byte aligned)

constexpr uint32_t prefill_lds_bytes(uint32_t d) {
    const uint32_t vt = kPrefillWaves * d * kPrefillVtStride * 2u;
    const uint32_t merge = 1024u + kPrefillWaves * kPrefillRows * (d + 4u) * 4u;
    return vt > merge ? vt : merge;
}

struct SdpaPrefillArgs {
    const uint16_t* q;    // [rows, n_heads, D]
    const uint16_t* k;    // [n_kv, capacity, D]
    const uint16_t* v;
    uint16_t* out;        // [rows, n_heads, D]
    uint32_t rows, kv_len, n_heads, heads_per_kv, capacity, row_tiles;
    float scale2;         // softmax scale times log2(e)
    const uint32_t* kv_len_ptr;  // optional: the count on the device (a replayed graph), instead of kv_len
};

// Positions in the cache including the group's rows.  A device value is clamped to what the
// host validated for an immediate one (rows <= kv_len <= capacity), so no address leaves the cache.
__device__ __forceinline__ uint32_t prefill_kv_len(const SdpaPrefillArgs& a) {
    uint32_t n = a.kv_len_ptr ? *a.kv_len_ptr : a.kv_len;
    n = n < a.rows ? a.rows : n;
    return n > a.capacity ? a.capacity : n;
}

__device__ __forceinline__ float other_half_max(float v) {
    const pf_u32x2_t r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float both_halves_sum(float v) {
    const pf_u32x2_t r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

// LDS traffic of ONE wave with itself: the hardware runs a wave's LDS instructions in order,
// the fence keeps the compiler from reordering them.
__device__ __forceinline__ void wave_lds_fence() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// The rescale of the output accumulators, in place in the accumulation registers of the matrix unit.
// Written as plain C++ this multiply makes the compiler copy all of them to vector registers at the
// head of EVERY pass, taken or not; spelled out, the copies stay inside the rare branch that calls
// this (128 rows x 4096 positions: 112 -> 105 us).  The trailing s_nop covers the wait states a
// matrix instruction needs after the write.
template <int DT>
__device__ __forceinline__ void rescale_accumulators(pf_f32x16_t (&oacc)[DT], float alpha) {
#pragma unroll
    for (int i = 0; i < DT; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            float x = oacc[i][r], t;
            asm volatile("v_accvgpr_read_b32 %1, %0\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 %0, %1\n\ts_nop 3"
                         : "+a"(x), "=&v"(t)
                         : "v"(alpha));
            oacc[i][r] = x;
        }
}

// One 64-position step of the running softmax of a lane's query.  Register r of score tile t is
// cache position kv0 + 32 t + r % 4 + 8 (r / 4) + 4 kb; scores become base-2 exponents; positions
// at or past q_limit are in the query's future (only steps with `mask` set can hold any).  Leaves
// the 32 probabilities as 16 bf16 pairs in register order, rescales the output accumulators when
// some lane's running maximum moved.
template <int DT>
__device__ __forceinline__ void softmax_step(const pf_f32x16_t (&s)[2], float scale2, bool mask, uint32_t kv0, uint32_t kb,
                                             uint32_t q_limit, float& m_run, float& l_run, pf_f32x16_t (&oacc)[DT],
                                             uint32_t (&pk)[16]) {
    float sv[32];
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int r = 0; r < 16; ++r) sv[t * 16 + r] = s[t][r] * scale2;
    if (mask) {
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const uint32_t kv = kv0 + (uint32_t)(t * 32 + r % 4 + 8 * (r / 4)) + 4u * kb;
                if (kv >= q_limit) sv[t * 16 + r] = -INFINITY;
            }
    }
    float mt = sv[0];
#pragma unroll
    for (int i = 1; i < 32; ++i) mt = fmaxf(mt, sv[i]);
    mt = other_half_max(mt);
    // m_run is the REFERENCE the probabilities are taken against, not the exact running maximum:
    // it moves only when a step's maximum has outgrown it by more than 2^8, so probabilities lie
    // in (0, 256] (bf16 keeps their relative precision, the sum is fp32) and the accumulators are
    // rescaled on the first step and then almost never.  With the exact maximum some lane of a
    // wave moves in about every second step, also late in a long context.
    const bool grow = mt > m_run + 8.0f;
    const float m_new = grow ? mt : m_run;
    const float m_ref = m_new == -INFINITY ? 0.f : m_new;  // a row that has seen nothing yet
    const float alpha = grow ? __builtin_amdgcn_exp2f(m_run - m_ref) : 1.0f;
    float psum = 0.f;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        const float p0 = __builtin_amdgcn_exp2f(sv[2 * i] - m_ref), p1 = __builtin_amdgcn_exp2f(sv[2 * i + 1] - m_ref);
        psum += p0 + p1;
        pk[i] = pack_bf16(p0, p1);
    }
    l_run = l_run * alpha + psum;
    m_run = m_new;
    if (__builtin_amdgcn_ballot_w64(alpha != 1.f) != 0) rescale_accumulators<DT>(oacc, alpha);
}

template <int D>
__global__ __launch_bounds__(kPrefillBlock) void sdpa_prefill_kernel(const SdpaPrefillArgs a) {
    constexpr int KB = D / 16;  // matrix steps over the head dimension (first product)
    constexpr int DT = D / 32;  // 32-wide tiles of the output dimension (second product)
    constexpr int VP = D / 8;   // 16-byte pieces of one V row
    constexpr uint32_t VS = kPrefillVtStride;
    extern __shared__ uint4 lds_raw[];

    const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6, kb = lane >> 5, nl = lane & 31u;
    const uint32_t head = blockIdx.x % a.n_heads;
    const uint32_t tile = a.row_tiles - 1u - blockIdx.x / a.n_heads;  // the longest rows start first
    const uint32_t kvh = head / a.heads_per_kv;
    const uint32_t r0 = tile * kPrefillRows;
    const uint32_t live = a.rows - r0 < kPrefillRows ? a.rows - r0 : kPrefillRows;
    const uint32_t prior = prefill_kv_len(a) - a.rows;      // positions in the cache before this group
    const uint32_t kv_end = prior + r0 + live;     // positions the last live row sees
    const uint32_t first_limit = prior + r0 + 1u;  // positions the first row sees
    const uint32_t n_steps = (kv_end + kPrefillStep - 1u) / kPrefillStep;

    uint16_t* vt = reinterpret_cast<uint16_t*>(lds_raw) + wave * ((uint32_t)D * VS);

    // B operand of the first product: lane (q = nl, kb) holds d = kb * D/2 + 8 j + (0..7) for step j
    const uint32_t rq = r0 + (nl < live ? nl : live - 1u);  // rows past the group repeat the last one; never stored
    const uint32_t q_limit = prior + rq + 1u;               // positions this lane's query sees
    uint4 qreg[KB];
    {
        const uint4* qp = reinterpret_cast<const uint4*>(a.q + ((size_t)rq * a.n_heads + head) * D + kb * (D / 2));
#pragma unroll
        for (int j = 0; j < KB; ++j) qreg[j] = qp[j];
    }

    const uint16_t* kbase = a.k + (size_t)kvh * a.capacity * D;
    const uint16_t* vbase = a.v + (size_t)kvh * a.capacity * D;
    uint4 kreg[2][KB], vreg[VP];
    // Requests only (nothing here uses a loaded value).  Positions past the visible range read
    // the last visible row instead: their scores are masked, and their V rows meet a zero
    // probability, so they only need to be finite.
    auto fetch_k = [&](uint32_t kv0) __attribute__((always_inline)) {
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            uint32_t kv = kv0 + (uint32_t)t * 32u + nl;
            kv = kv < kv_end ? kv : kv_end - 1u;
            const uint4* p = reinterpret_cast<const uint4*>(kbase + (size_t)kv * D + kb * (D / 2));
#pragma unroll
            for (int j = 0; j < KB; ++j) kreg[t][j] = p[j];
        }
    };
    auto fetch_v = [&](uint32_t kv0) __attribute__((always_inline)) {
        uint32_t kv = kv0 + lane;
        kv = kv < kv_end ? kv : kv_end - 1u;
        const uint4* p = reinterpret_cast<const uint4*>(vbase + (size_t)kv * D);
#pragma unroll
        for (int i = 0; i < VP; ++i) vreg[i] = p[i];
    };

    float m_run = -INFINITY, l_run = 0.f;  // l_run: this lane's share (its half-wave's scores)
    pf_f32x16_t oacc[DT];
#pragma unroll
    for (int i = 0; i < DT; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) oacc[i][r] = 0.f;

    // Position of cache row `lane` inside a row of the transposed tile: bits 2 and 3 swapped, so
    // that the rows a lane's score registers 8t .. 8t+7 stand for (8 u + 4 kb + e, u = 0..1,
    // e = 0..3, inside a block of 16) are the eight contiguous entries 8 kb + 4 u + e.
    const uint32_t vpos = (lane & ~12u) | ((lane & 4u) << 1) | ((lane & 8u) >> 1);

    uint32_t step = wave;
    if (step < n_steps) {
        fetch_k(step * kPrefillStep);
        fetch_v(step * kPrefillStep);
    }
    for (; step < n_steps; step += kPrefillWaves) {
        const uint32_t kv0 = step * kPrefillStep;
        const uint32_t kv_next = kv0 + kPrefillWaves * kPrefillStep;  // past the range on the last pass: clamped

        pf_f32x16_t s[2];
#pragma unroll
        for (int t = 0; t < 2; ++t) {
#pragma unroll
            for (int r = 0; r < 16; ++r) s[t][r] = 0.f;
#pragma unroll
            for (int j = 0; j < KB; ++j)
                s[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(pf_bf16x8_t, kreg[t][j]),
                                                               __builtin_bit_cast(pf_bf16x8_t, qreg[j]), s[t], 0, 0, 0);
        }
        fetch_k(kv_next);

        // V rows of this step -> LDS, transposed
#pragma unroll
        for (int i = 0; i < VP; ++i) {
            const uint32_t w4[4] = {vreg[i].x, vreg[i].y, vreg[i].z, vreg[i].w};
#pragma unroll
            for (int e = 0; e < 8; ++e)
                vt[(uint32_t)(i * 8 + e) * VS + vpos] = (uint16_t)(e & 1 ? w4[e >> 1] >> 16 : w4[e >> 1] & 0xffffu);
        }
        fetch_v(kv_next);

        uint32_t pk[16];
        softmax_step<DT>(s, a.scale2, kv0 + kPrefillStep > first_limit, kv0, kb, q_limit, m_run, l_run, oacc, pk);

        wave_lds_fence();  // the transposed tile is complete
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            const uint4 pb = make_uint4(pk[c * 4 + 0], pk[c * 4 + 1], pk[c * 4 + 2], pk[c * 4 + 3]);
#pragma unroll
            for (int i = 0; i < DT; ++i) {
                const uint4 va = *reinterpret_cast<const uint4*>(vt + (uint32_t)(i * 32 + (int)nl) * VS + c * 16 + kb * 8);
                oacc[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(pf_bf16x8_t, va),
                                                                  __builtin_bit_cast(pf_bf16x8_t, pb), oacc[i], 0, 0, 0);
            }
        }
        wave_lds_fence();  // the tile has been read before the next pass overwrites it
    }

    // ---- merge of the four waves, in wave order --------------------------------------------
    l_run = both_halves_sum(l_run);
    __syncthreads();  // every wave has left its loop: the tiles' LDS is free
    float* ml = reinterpret_cast<float*>(lds_raw);  // [wave][m x 32 | l x 32]
    float* ob = ml + 256;                           // [wave][row][D + 4]
    constexpr uint32_t OS = D + 4;
    if (kb == 0) {
        ml[wave * 64u + nl] = m_run;
        ml[wave * 64u + 32u + nl] = l_run;
    }
    __syncthreads();
    float mx = ml[nl];  // wave 0 always holds position 0, which every row sees: finite
#pragma unroll
    for (uint32_t w = 1; w < kPrefillWaves; ++w) mx = fmaxf(mx, ml[w * 64u + nl]);
    float lsum = 0.f;
#pragma unroll
    for (uint32_t w = 0; w < kPrefillWaves; ++w) lsum += __builtin_amdgcn_exp2f(ml[w * 64u + nl] - mx) * ml[w * 64u + 32u + nl];
    const float f = __builtin_amdgcn_exp2f(m_run - mx) / lsum;
    // register r of tile i is output dimension 32 i + r % 4 + 8 (r / 4) + 4 kb of query nl
#pragma unroll
    for (int i = 0; i < DT; ++i)
#pragma unroll
        for (int g = 0; g < 4; ++g)
            *reinterpret_cast<float4*>(ob + (wave * kPrefillRows + nl) * OS + (uint32_t)(i * 32 + 8 * g) + 4u * kb) =
                make_float4(oacc[i][4 * g + 0] * f, oacc[i][4 * g + 1] * f, oacc[i][4 * g + 2] * f, oacc[i][4 * g + 3] * f);
    __syncthreads();
    for (uint32_t idx = threadIdx.x; idx < kPrefillRows * (uint32_t)VP; idx += kPrefillBlock) {
        const uint32_t row = idx / (uint32_t)VP, piece = idx % (uint32_t)VP;
        if (row >= live) continue;
        float o[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (uint32_t w = 0; w < kPrefillWaves; ++w) {
            const float4 lo = *reinterpret_cast<const float4*>(ob + (w * kPrefillRows + row) * OS + piece * 8u);
            const float4 hi = *reinterpret_cast<const float4*>(ob + (w * kPrefillRows + row) * OS + piece * 8u + 4u);
            o[0] += lo.x; o[1] += lo.y; o[2] += lo.z; o[3] += lo.w;
            o[4] += hi.x; o[5] += hi.y; o[6] += hi.z; o[7] += hi.w;
        }
        *reinterpret_cast<uint4*>(a.out + ((size_t)(r0 + row) * a.n_heads + head) * D + piece * 8u) =
            make_uint4(pack_bf16(o[0], o[1]), pack_bf16(o[2], o[3]), pack_bf16(o[4], o[5]), pack_bf16(o[6], o[7]));
    }
}

// ---- the form for more than 64 rows ------------------------------------------------------------
// One block = one query head x 128 consecutive rows, one 32-row tile per wave.  The four waves
// walk the SAME 64-position steps, so a step's K and V rows are fetched once per block, with
// coalesced 16-byte loads, and shared through LDS (two buffers: the next step is written while
// this one is multiplied, one barrier per step):
//   K  as it lies, rows padded by 16 bytes: a lane's fragment of the first product is one
//      16-byte read, conflict free;
//   V  transposed to [d][position]: two threads that hold the same 8 dimensions of two
//      neighbouring rows exchange their words (one cross-lane move per register) so that each
//      writes whole 32-bit words (position pair x one dimension); the 8-position groups of a
//      row are XOR-swizzled with the dimension's piece index to spread the banks.
// A wave's arithmetic is that of the kernel above (same softmax_step, same register layouts)
// except that the head dimension is taken in natural order here (d = 16 j + 8 kb + e).
constexpr int kPrefillTileDepth = 2;  // steps of K / V rows in flight per thread (1, 2 and 3 measured alike)
constexpr uint32_t prefill_tile_ks(uint32_t d) { return d + 8u; }                       // bf16 per staged K row
constexpr uint32_t prefill_tile_buf(uint32_t d) { return kPrefillStep * prefill_tile_ks(d) + d * kPrefillVtStride; }  // bf16 per buffer
constexpr uint32_t prefill_tile_lds_bytes(uint32_t d) {
    const uint32_t stage = 2u * prefill_tile_buf(d) * 2u;
    const uint32_t outb = kPrefillWaves * kPrefillRows * (d + 4u) * 4u;
    return stage > outb ? stage : outb;
}

template <typename F, int... I>
__device__ __forceinline__ void static_for_impl(F&& f, std::integer_sequence<int, I...>) {
    (f(std::integral_constant<int, I>{}), ...);
}
template <int N, typename F>
__device__ __forceinline__ void static_for(F&& f) {
    static_for_impl(f, std::make_integer_sequence<int, N>{});
}

// value of the thread that holds the neighbouring cache row (lane ^ PIECES) -> (even row's, odd row's)
template <int PIECES>
__device__ __forceinline__ void pair_rows(uint32_t w, bool odd, uint32_t& even_row, uint32_t& odd_row) {
    if constexpr (PIECES == 16) {
        const pf_u32x2_t r = __builtin_amdgcn_permlane16_swap(w, w, false, false);  // (rows 0,0,2,2 | rows 1,1,3,3) of 16 lanes
        even_row = r[0];
        odd_row = r[1];
    } else {
        static_assert(PIECES == 8, "8 or 16 pieces per row");
        const uint32_t other = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)w, 0x128, 0xF, 0xF, false);  // row_ror:8 = lane ^ 8
        even_row = odd ? other : w;
        odd_row = odd ? w : other;
    }
}

template <int D, int PF>
__global__ __launch_bounds__(kPrefillBlock) void sdpa_prefill_tile_kernel(const SdpaPrefillArgs a) {
    constexpr int KB = D / 16, DT = D / 32, VP = D / 8;
    constexpr int PPT = (int)kPrefillStep * VP / kPrefillBlock;  // 16-byte pieces per thread, tile and matrix
    constexpr uint32_t KS = prefill_tile_ks(D), VS = kPrefillVtStride, BUF = prefill_tile_buf(D);
    extern __shared__ uint4 lds_raw[];
    uint16_t* lds = reinterpret_cast<uint16_t*>(lds_raw);

    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6, kb = lane >> 5, nl = lane & 31u;
    const uint32_t head = blockIdx.x % a.n_heads;
    const uint32_t grp = a.row_tiles - 1u - blockIdx.x / a.n_heads;  // row_tiles counts 128-row groups here; longest first
    const uint32_t kvh = head / a.heads_per_kv;
    const uint32_t r0 = (grp * kPrefillWaves + wave) * kPrefillRows;
    const uint32_t live = r0 < a.rows ? (a.rows - r0 < kPrefillRows ? a.rows - r0 : kPrefillRows) : 0u;
    const uint32_t prior = prefill_kv_len(a) - a.rows;
    const uint32_t grp_end = (grp + 1u) * kPrefillWaves * kPrefillRows;
    const uint32_t kv_end_blk = prior + (grp_end < a.rows ? grp_end : a.rows);  // positions the block's last row sees
    const uint32_t first_limit = prior + r0 + 1u;
    const uint32_t n_steps = (kv_end_blk + kPrefillStep - 1u) / kPrefillStep;

    uint32_t rq = r0 + (nl < live ? nl : (live ? live - 1u : 0u));
    rq = rq < a.rows ? rq : a.rows - 1u;  // a wave without rows loads something valid and computes nothing
    const uint32_t q_limit = prior + rq + 1u;
    uint4 qreg[KB];
    {
        const uint4* qp = reinterpret_cast<const uint4*>(a.q + ((size_t)rq * a.n_heads + head) * D + kb * 8u);
#pragma unroll
        for (int j = 0; j < KB; ++j) qreg[j] = qp[2 * j];
    }

    // this thread's pieces of a step: cache row srow + (256 / VP) i, dimensions 8 piece .. 8 piece + 7
    const uint32_t srow = tid / (uint32_t)VP, piece = tid % (uint32_t)VP;
    const bool odd = (srow & 1u) != 0;
    const uint16_t* kbase = a.k + (size_t)kvh * a.capacity * D + piece * 8u;
    const uint16_t* vbase = a.v + (size_t)kvh * a.capacity * D + piece * 8u;
    // PF steps of K and V rows are in flight per thread (slot = step % PF): with one block of one
    // wave per SIMD on a CU, the depth of this ring is what hides the memory latency.
    uint4 kst[PF][PPT], vst[PF][PPT];
    auto fetch = [&](auto slot, uint32_t kv0) __attribute__((always_inline)) {  // requests only; rows past the block's range repeat its last row
        constexpr int S = decltype(slot)::value;
#pragma unroll
        for (int i = 0; i < PPT; ++i) {
            uint32_t kv = kv0 + srow + (uint32_t)i * (kPrefillBlock / VP);
            kv = kv < kv_end_blk ? kv : kv_end_blk - 1u;
            kst[S][i] = *reinterpret_cast<const uint4*>(kbase + (size_t)kv * D);
            vst[S][i] = *reinterpret_cast<const uint4*>(vbase + (size_t)kv * D);
        }
    };
    const uint32_t perm_sel = odd ? 0x07060302u : 0x05040100u;  // (even row's, odd row's) halves of this thread's dimension
    auto stage = [&](auto slot, uint16_t* buf) __attribute__((always_inline)) {
        constexpr int S = decltype(slot)::value;
        uint16_t* ks = buf;
        uint16_t* vt = buf + kPrefillStep * KS;
#pragma unroll
        for (int i = 0; i < PPT; ++i) {
            const uint32_t row = srow + (uint32_t)i * (kPrefillBlock / VP);
            *reinterpret_cast<pf_u32x4_t*>(ks + row * KS + piece * 8u) = __builtin_bit_cast(pf_u32x4_t, kst[S][i]);
            // position of the row pair inside a transposed row: bits 2 and 3 of the row swapped (the
            // order the score registers hold), groups of 8 swizzled with the piece index
            const uint32_t re = row & ~1u;
            const uint32_t pos = (re & ~12u) | ((re & 4u) << 1) | ((re & 8u) >> 1);
            uint16_t* dst = vt + (piece * 8u + (odd ? 1u : 0u)) * VS + ((((pos >> 3) ^ (piece & 7u)) << 3) | (pos & 7u));
            const pf_u32x4_t w4 = __builtin_bit_cast(pf_u32x4_t, vst[S][i]);
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                uint32_t ev, od;
                pair_rows<VP>(w4[c], odd, ev, od);
                *reinterpret_cast<uint32_t*>(dst + (uint32_t)(2 * c) * VS) = __builtin_amdgcn_perm(od, ev, perm_sel);
            }
        }
    };

    float m_run = -INFINITY, l_run = 0.f;
    pf_f32x16_t oacc[DT];
#pragma unroll
    for (int i = 0; i < DT; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) oacc[i][r] = 0.f;

    auto pass = [&](auto uc, uint32_t step) __attribute__((always_inline)) {
        constexpr int NEXT = (decltype(uc)::value + 1) % PF;  // slot of step + 1
        const uint32_t kv0 = step * kPrefillStep;
        const uint16_t* ks = lds + (step & 1u) * BUF;
        const uint16_t* vt = ks + kPrefillStep * KS;
        // Fragments are read from LDS in one batch ahead of the matrix instructions that use them (a
        // read followed at once by its instruction would pay the LDS latency 32 times per step); the
        // V fragments are requested before the softmax, which needs none of them.
        // Every wave computes every step of its block, also one whose positions all lie in its rows'
        // future (at most the last two steps) and a wave without rows (it repeats the group's last
        // row): such scores are masked and add exact zeros, and a pass without branches keeps the
        // accumulators where the matrix unit wants them.
        pf_f32x16_t s[2];
        {
            uint4 ka[2][KB];
#pragma unroll
            for (int t = 0; t < 2; ++t)
#pragma unroll
                for (int j = 0; j < KB; ++j)
                    ka[t][j] = *reinterpret_cast<const uint4*>(ks + (uint32_t)(t * 32 + (int)nl) * KS + j * 16 + kb * 8);
            __builtin_amdgcn_sched_barrier(0);  // all reads are issued before the first matrix instruction
#pragma unroll
            for (int t = 0; t < 2; ++t) {
#pragma unroll
                for (int r = 0; r < 16; ++r) s[t][r] = 0.f;
#pragma unroll
                for (int j = 0; j < KB; ++j)
                    s[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(pf_bf16x8_t, ka[t][j]),
                                                                   __builtin_bit_cast(pf_bf16x8_t, qreg[j]), s[t], 0, 0, 0);
            }
        }
        // the next step's rows go to the other buffer (every wave finished reading it before the
        // barrier that ended the previous pass), then their slot is requested again, PF steps on
        stage(std::integral_constant<int, NEXT>{}, lds + ((step + 1u) & 1u) * BUF);
        fetch(std::integral_constant<int, NEXT>{}, kv0 + (uint32_t)(PF + 1) * kPrefillStep);
        {
            uint4 va[4][DT];
#pragma unroll
            for (int c = 0; c < 4; ++c)
#pragma unroll
                for (int i = 0; i < DT; ++i) {
                    const uint32_t d = (uint32_t)(i * 32) + nl;
                    va[c][i] = *reinterpret_cast<const uint4*>(vt + d * VS + ((((uint32_t)(2 * c) + kb) ^ ((d >> 3) & 7u)) << 3));
                }
            uint32_t pk[16];
            softmax_step<DT>(s, a.scale2, kv0 + kPrefillStep > first_limit, kv0, kb, q_limit, m_run, l_run, oacc, pk);
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                const uint4 pb = make_uint4(pk[c * 4 + 0], pk[c * 4 + 1], pk[c * 4 + 2], pk[c * 4 + 3]);
#pragma unroll
                for (int i = 0; i < DT; ++i)
                    oacc[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(pf_bf16x8_t, va[c][i]),
                                                                      __builtin_bit_cast(pf_bf16x8_t, pb), oacc[i], 0, 0, 0);
            }
        }
        __syncthreads();
    };

    static_for<PF>([&](auto u) __attribute__((always_inline)) { fetch(u, (uint32_t)decltype(u)::value * kPrefillStep); });
    stage(std::integral_constant<int, 0>{}, lds);
    fetch(std::integral_constant<int, 0>{}, (uint32_t)PF * kPrefillStep);
    __syncthreads();
    for (uint32_t base = 0; base < n_steps; base += PF)  // n_steps is the same for the whole block
        static_for<PF>([&](auto u) __attribute__((always_inline)) {
            if (base + (uint32_t)decltype(u)::value < n_steps) pass(u, base + (uint32_t)decltype(u)::value);
        });

    // ---- output: through this wave's own LDS rows, so that the stores are whole 16-byte pieces ----
    // (the last barrier of the loop has freed both buffers)
    if (live == 0) return;
    l_run = both_halves_sum(l_run);
    const float f = 1.0f / l_run;
    constexpr uint32_t OS = D + 4;
    float* ob = reinterpret_cast<float*>(lds_raw) + wave * kPrefillRows * OS;
#pragma unroll
    for (int i = 0; i < DT; ++i)
#pragma unroll
        for (int g = 0; g < 4; ++g)
            *reinterpret_cast<float4*>(ob + nl * OS + (uint32_t)(i * 32 + 8 * g) + 4u * kb) =
                make_float4(oacc[i][4 * g + 0] * f, oacc[i][4 * g + 1] * f, oacc[i][4 * g + 2] * f, oacc[i][4 * g + 3] * f);
    wave_lds_fence();
    for (uint32_t idx = lane; idx < kPrefillRows * (uint32_t)VP; idx += 64u) {
        const uint32_t row = idx / (uint32_t)VP, pc = idx % (uint32_t)VP;
        if (row >= live) continue;
        const float4 lo = *reinterpret_cast<const float4*>(ob + row * OS + pc * 8u);
        const float4 hi = *reinterpret_cast<const float4*>(ob + row * OS + pc * 8u + 4u);
        *reinterpret_cast<uint4*>(a.out + ((size_t)(r0 + row) * a.n_heads + head) * D + pc * 8u) =
            make_uint4(pack_bf16(lo.x, lo.y), pack_bf16(lo.z, lo.w), pack_bf16(hi.x, hi.y), pack_bf16(hi.z, hi.w));
    }
}

fk_status plan_sdpa_prefill(const uint16_t* q, const uint16_t* cache_k, const uint16_t* cache_v, uint16_t* out,
                            uint32_t rows, uint32_t kv_len, uint32_t n_heads, uint32_t n_kv, uint32_t head_dim,
                            uint32_t capacity, float scale, Launch* l, const uint32_t* kv_len_ptr) {
    const DeviceFacts* dev;
    FK_TRY(device_facts(&dev));
    if (!q || !cache_k || !cache_v || !out) return set_error(FK_ERR_INVALID, "sdpa_prefill: null pointer");
    if (rows == 0 || kv_len < rows) return set_error(FK_ERR_INVALID, "sdpa_prefill: kv_len counts the rows of the group, so 1 <= rows <= kv_len");
    if (kv_len > capacity) return set_error(FK_ERR_INVALID, "sdpa_prefill: kv_len exceeds the cache capacity");
    if (n_heads == 0 || n_kv == 0 || n_heads % n_kv) return set_error(FK_ERR_INVALID, "sdpa_prefill: n_heads must be a multiple of n_kv");
    if (head_dim != 64 && head_dim != 128)
        return set_error(FK_ERR_UNSUPPORTED, "sdpa_prefill: head dimension 64 or 128 (use fk_sdpa_decode_rows for other shapes)");
    if (((uintptr_t)q | (uintptr_t)cache_k | (uintptr_t)cache_v | (uintptr_t)out) & 15u)
        return set_error(FK_ERR_INVALID, "sdpa_prefill: pointers must be 16-byte aligned");
    SdpaPrefillArgs a;
    memset(&a, 0, sizeof(a));
    a.q = q; a.k = cache_k; a.v = cache_v; a.out = out;
    a.kv_len_ptr = kv_len_ptr;
    if (rows > capacity) return set_error(FK_ERR_INVALID, "sdpa_prefill: more rows than the cache holds");
    a.rows = rows; a.kv_len = kv_len; a.n_heads = n_heads; a.heads_per_kv = n_heads / n_kv; a.capacity = capacity;
    a.scale2 = scale * 1.4426950408889634f;
    // Two forms: a block per 32 rows whose waves split the positions, or a block per 128 rows whose
    // waves share every step's K and V through LDS.  The second does a 64-position step of its 128
    // rows in 1.65 us against 4 x 0.93 us, but has a quarter of the blocks: it is taken when the first
    // form would need more rounds over the CUs than that advantage is worth (measured at head
    // dimension 128: 128 rows x 32 heads 65 against 105 us, 512 rows 118 against 106 us at 4096 positions).
    const uint64_t blocks_split = (uint64_t)n_heads * ((rows + kPrefillRows - 1u) / kPrefillRows);
    const uint64_t blocks_tile = (uint64_t)n_heads * ((rows + kPrefillWaves * kPrefillRows - 1u) / (kPrefillWaves * kPrefillRows));
    const uint64_t cus = (uint64_t)(dev->cus > 0 ? dev->cus : 1);
    const bool shared_tiles = ((blocks_tile + cus - 1) / cus) * 165u < ((blocks_split + cus - 1) / cus) * 93u;
    const uint32_t rows_per_block = shared_tiles ? kPrefillWaves * kPrefillRows : kPrefillRows;
    a.row_tiles = (rows + rows_per_block - 1u) / rows_per_block;
    if ((uint64_t)a.row_tiles * n_heads > 0x7fffffffull) return set_error(FK_ERR_UNSUPPORTED, "sdpa_prefill: too many rows");
    if (shared_tiles)
        l->func = head_dim == 64 ? reinterpret_cast<const void*>(&sdpa_prefill_tile_kernel<64, kPrefillTileDepth>)
                                 : reinterpret_cast<const void*>(&sdpa_prefill_tile_kernel<128, kPrefillTileDepth>);
    else
        l->func = head_dim == 64 ? reinterpret_cast<const void*>(&sdpa_prefill_kernel<64>)
                                 : reinterpret_cast<const void*>(&sdpa_prefill_kernel<128>);
    l->grid = dim3(a.row_tiles * n_heads, 1, 1);
    l->block = dim3(kPrefillBlock, 1, 1);
    l->shmem = shared_tiles ? prefill_tile_lds_bytes(head_dim) : prefill_lds_bytes(head_dim);
    if ((int)l->shmem > dev->max_dyn_lds) return set_error(FK_ERR_UNSUPPORTED, "sdpa_prefill: LDS tile does not fit");
    if (l->shmem > 48 * 1024) FK_HIP(hipFuncSetAttribute(l->func, hipFuncAttributeMaxDynamicSharedMemorySize, (int)l->shmem));
    l->set_args(a);
    return FK_OK;
}

}  // namespace fk
