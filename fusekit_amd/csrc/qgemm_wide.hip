// Shared-stream matmul for 2 .. 10 activation rows: y[M, N] = epilogue(x[M, K] @ dequant(W)^T) in ONE launch,
// the weight matrix read once for all rows.  Replaces the reference's small-M kernels (fusekit_qmv_wide_impl,
// src/codegen/msl.rs:462-546; fusekit_qmv_fast_m_impl, :1307-1485; policy kernels/mod.rs:164-186: 2..10 rows,
// group 64, 4 or 8 bits) -- there up to five activation vectors share a dequantised weight fragment in
// registers and the stream is read ceil(M / 5) times; here the ten rows share it through the matrix cores and
// the stream is read once.
//
// Same arithmetic as the exact form of qgemm_kernel (qgemm.hip): the integer codes go into
// v_mfma_f32_32x32x16_bf16 as exact bf16 values with the WEIGHTS as the B operand, the integer dot of a
// quantisation group is accumulated in a zeroed C tile and folded into the fp32 accumulators as
// s * dot + b * Sx(row, group).  What differs is the cut: a block owns 32 weight rows over ALL of K and its
// waves (4 or 8) split K between them in slabs of 256, so there is no split-k workspace and no second kernel --
// the waves' accumulators meet in LDS, are added in wave order, and the epilogue (bias, residual, or SwiGLU of a
// gate / up pair streamed side by side) runs in the same launch.  Every wave stages the activation slab it is
// about to use in its OWN piece of LDS (M <= 10 rows x 256 k = 5 KB; LDS operations of one wave execute in order),
// so the main loop has no block barrier at all; rows 10 .. 31 of the matrix operand read one zero row.
// Matrices with few rows run eight waves per block instead of four (N / 32 blocks of four waves would leave most
// of the chip without a wave).
#include "fk_host.hpp"
#include "gemv_kernel.hpp"

#include "fk_probe.hpp"
FK_PROBE_DEFINE(wide, 2048, 8)
#define FK_WIDE_STAMP(i) FK_PROBE_STAMP(wide, 2048, 8, blockIdx.x, threadIdx.x == 0, i)

namespace fk {

namespace {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x16_t __attribute__((ext_vector_type(16)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));

constexpr uint32_t kWideMaxRows = 10;             // activation rows (the reference's upper bound for this path)
constexpr uint32_t kWideSlab = 256;               // k per wave and step
constexpr uint32_t kWideXS = kWideSlab / 8 + 1;   // uint4 per staged activation row (+1: bank spread)
constexpr uint32_t kWideXRows = kWideMaxRows + 1; // staged rows + the zero row
constexpr int kWideXPT = kWideMaxRows * (kWideSlab / 8) / kWave;  // 16-byte pieces of x per lane and slab

struct QgemmWideArgs {
    const uint4* w[3];     // the matrix, the gate / up pair, or up to three matrices served side by side (segments)
    const uint16_t* sc[3];
    const uint16_t* bi[3];
    const uint16_t* x;     // [M, x_stride] bf16
    const uint16_t* bias;  // [N] or null (single matrix)
    const uint16_t* res;   // [M, N] or null (single matrix)
    uint16_t* y;           // [M, N]
    uint32_t M, N, K;
    uint32_t cpr, gpr;
    int variant;           // SwiGLU rounding variant (pair)
    // 16-row form with one matrix per block: segment s owns blocks [blk0[s], blk0[s + 1]) and writes ys[s] with its own
    // row stride; norm_w: the activations are RMS-normalised as they are staged, T(w * T(x * r)) per element
    uint32_t n_seg, x_stride;
    uint32_t ns[3], blk0[3], y_stride[3];
    uint16_t* ys[3];
    const uint16_t* norm_w;
    float eps;
};

// LDS per wave: staged activations [kWideXRows][kWideXS] uint4, group sums [4][32] floats; per block
// additionally the waves' results [waves][mats][kWideMaxRows][32] floats.
__host__ __device__ constexpr uint32_t wide_wave_lds() { return kWideXRows * kWideXS * 16u + 4u * 32u * 4u; }
__host__ __device__ constexpr uint32_t wide_meet_bytes(uint32_t waves, uint32_t mats) { return waves * mats * kWideMaxRows * 32u * 4u; }
__host__ __device__ constexpr uint32_t wide_lds_bytes(uint32_t waves, uint32_t mats) {
    return waves * wide_wave_lds() + wide_meet_bytes(waves, mats) + 64u;   // + one 1/rms per activation row
}

template <WKind KIND, int MATS, int WAVES>
__global__ __launch_bounds__(WAVES* kWave) void qgemm_wide_kernel(const QgemmWideArgs a) {
    constexpr uint32_t VPL = KIND == W_Q4 ? 32u : 16u;  // codes per 16-byte lane load
    constexpr int MF = VPL / 8;                         // MFMA steps per load
    constexpr int LOADS = kWideSlab / (2u * VPL);       // 16-byte weight loads per lane, matrix and slab
    constexpr int UNITS = kWideSlab / 64u;              // groups per slab
    constexpr uint32_t LPG = 64u / (2u * VPL);          // loads per group
    extern __shared__ uint4 lds_raw[];
    const uint32_t lane = threadIdx.x & 63u, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), kb = lane >> 5, nl = lane & 31u;
    uint4* xs = reinterpret_cast<uint4*>(reinterpret_cast<char*>(lds_raw) + wave * wide_wave_lds());  // [kWideXRows][kWideXS]
    float* sxs = reinterpret_cast<float*>(xs + kWideXRows * kWideXS);                                  // [UNITS][32]
    float* meet = reinterpret_cast<float*>(reinterpret_cast<char*>(lds_raw) + WAVES * wide_wave_lds()); // [WAVES][MATS][rows][32]

    const uint32_t M = a.M, n = blockIdx.x * 32u + nl, nc = n < a.N ? n : a.N - 1;  // rows past the end repeat the last
    const uint32_t n_slabs = (a.K + kWideSlab - 1) / kWideSlab;

    // the zero row and the group sums of rows that do not exist (read by the fold, never stored)
    for (uint32_t i = lane; i < kWideXS; i += kWave) xs[kWideMaxRows * kWideXS + i] = make_uint4(0, 0, 0, 0);
    for (uint32_t i = lane; i < UNITS * 32u; i += kWave) sxs[i] = 0.f;
    const uint32_t arow = nl < M ? nl : kWideMaxRows;  // this lane's row of the A operand

    const uint4* wrow[MATS];
    const uint16_t *srow[MATS], *brow[MATS];
#pragma unroll
    for (int q = 0; q < MATS; ++q) {
        wrow[q] = a.w[q] + (size_t)nc * a.cpr;
        srow[q] = a.sc[q] + (size_t)nc * a.gpr;
        brow[q] = a.bi[q] + (size_t)nc * a.gpr;
    }

    f32x16_t acc[MATS];
#pragma unroll
    for (int q = 0; q < MATS; ++q)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[q][r] = 0.f;

    // A slab's requests: weights, scale / bias pairs and this lane's pieces of the activations.  Straight-line (a
    // branch around requests makes the compiler wait for everything outstanding where the paths join): a slab past
    // the end (`live` false) reads the first bytes of the arrays.
    struct Slab {
        uint4 w[MATS][LOADS], x[kWideXPT];
        uint32_t sb[MATS][UNITS];
    };
    auto fetch = [&](uint32_t slab, Slab& B) {
        const bool live = slab < n_slabs;
        const uint32_t ks0 = live ? slab * kWideSlab : 0u;
        const uint32_t slab_k = a.K - ks0 < kWideSlab ? a.K - ks0 : kWideSlab;
        const uint32_t loads = live ? slab_k / (2u * VPL) : 0u, units = live ? slab_k >> 6 : 0u, s8 = live ? slab_k >> 3 : 0u;
#pragma unroll
        for (int q = 0; q < MATS; ++q) {
            const uint4* wp = (live ? wrow[q] : a.w[q]) + ks0 / VPL + (live ? kb : 0u);
#pragma unroll
            for (int t = 0; t < LOADS; ++t) B.w[q][t] = wp[2u * ((uint32_t)t < loads ? (uint32_t)t : 0u)];
#pragma unroll
            for (int u = 0; u < UNITS; ++u) {
                const uint32_t g = (ks0 >> 6) + ((uint32_t)u < units ? (uint32_t)u : 0u);
                B.sb[q][u] = (uint32_t)(live ? srow[q] : a.sc[q])[g] | ((uint32_t)(live ? brow[q] : a.bi[q])[g] << 16);
            }
        }
#pragma unroll
        for (int i = 0; i < kWideXPT; ++i) {
            const uint32_t idx = lane + (uint32_t)i * kWave, m = idx / (kWideSlab / 8), k8 = idx % (kWideSlab / 8);
            const bool have = m < M && k8 < s8;
            B.x[i] = *reinterpret_cast<const uint4*>(a.x + (size_t)(have ? m : 0u) * a.x_stride + ks0 + (have ? k8 : 0u) * 8u);
        }
    };
    auto consume = [&](uint32_t slab, const Slab& B) {
        const uint32_t ks0 = slab * kWideSlab;
        const uint32_t slab_k = a.K - ks0 < kWideSlab ? a.K - ks0 : kWideSlab;
        // park the slab's activations (the previous slab's fragments have been read: LDS operations of a wave are
        // executed in order)
#pragma unroll
        for (int i = 0; i < kWideXPT; ++i) {
            const uint32_t idx = lane + (uint32_t)i * kWave, m = idx / (kWideSlab / 8), k8 = idx % (kWideSlab / 8);
            uint4 v = (m < M && k8 < (slab_k >> 3)) ? B.x[i] : make_uint4(0, 0, 0, 0);
            if constexpr (KIND == W_Q4) {
                // nibble pairing of the int4 unpack: (x0,x2) (x4,x6) (x1,x3) (x5,x7)
                v = make_uint4((v.x & 0xffffu) | (v.y << 16), (v.z & 0xffffu) | (v.w << 16),
                               (v.x >> 16) | (v.y & 0xffff0000u), (v.z >> 16) | (v.w & 0xffff0000u));
            }
            xs[m * kWideXS + k8] = v;
        }
        __builtin_amdgcn_wave_barrier();
        // group sums of the staged rows: lane (g, m) = (lane / 16, lane % 16) adds the 64 values of its group
        {
            const uint32_t g = lane >> 4, m = lane & 15u;
            if (m < M) {
                // (pairs of bf16 against a pair of ones: v_dot2_f32_bf16, no unpacking; two chains)
                float s0 = 0.f, s1 = 0.f;
                if (g < (slab_k >> 6)) {
#pragma unroll
                    for (uint32_t i = 0; i < 8; ++i) {
                        const uint4 v = xs[m * kWideXS + g * 8u + i];
                        s0 = dot2_bf16(v.x, 0x3F803F80u, s0);
                        s1 = dot2_bf16(v.y, 0x3F803F80u, s1);
                        s0 = dot2_bf16(v.z, 0x3F803F80u, s0);
                        s1 = dot2_bf16(v.w, 0x3F803F80u, s1);
                    }
                }
                sxs[g * 32u + m] = s0 + s1;
            }
        }
        __builtin_amdgcn_wave_barrier();

        const uint32_t loads = slab_k / (2u * VPL);
        // two C tiles per matrix, used alternately: consecutive matrix instructions do not wait for each other
        // (a group's first instruction on a tile starts from a constant zero operand instead of a cleared tile)
        f32x16_t c[MATS][2];
        const f32x16_t zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int t = 0; t < LOADS; ++t) {
            if ((uint32_t)t < loads) {  // wave-uniform
                const uint4* xa = xs + arow * kWideXS + (((uint32_t)t * 2u + kb) * VPL >> 3);
#pragma unroll
                for (int j = 0; j < MF; ++j) {
                    const uint4 av = xa[j];
#pragma unroll
                    for (int q = 0; q < MATS; ++q) {
                        const uint32_t wd[4] = {B.w[q][t].x, B.w[q][t].y, B.w[q][t].z, B.w[q][t].w};
                        uint4 bw;
                        if constexpr (KIND == W_Q4) {
                            const uint32_t even = wd[j] & 0x0F0F0F0Fu, odd = (wd[j] >> 4) & 0x0F0F0F0Fu;
                            bw.x = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(even, 512.0f, false));
                            bw.y = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(even, 512.0f, true));
                            bw.z = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(odd, 512.0f, false));
                            bw.w = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(odd, 512.0f, true));
                        } else {
                            const uint32_t w0 = wd[(2 * j) & 3], w1 = wd[(2 * j + 1) & 3];
                            auto pair = [](float lo, float hi) {
                                const bf16x2_t p = {(__bf16)lo, (__bf16)hi};  // integers <= 255 are exact in bf16
                                return __builtin_bit_cast(uint32_t, p);
                            };
                            bw.x = pair((float)(w0 & 0xffu), (float)((w0 >> 8) & 0xffu));
                            bw.y = pair((float)((w0 >> 16) & 0xffu), (float)(w0 >> 24));
                            bw.z = pair((float)(w1 & 0xffu), (float)((w1 >> 8) & 0xffu));
                            bw.w = pair((float)((w1 >> 16) & 0xffu), (float)(w1 >> 24));
                        }
                        // step (t % LPG) * MF + j of its group: the first two start their tiles
                        const bool first = ((uint32_t)t & (LPG - 1u)) * MF + j < 2;
                        c[q][j & 1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, av),
                                                                              __builtin_bit_cast(bf16x8_t, bw),
                                                                              first ? zero : c[q][j & 1], 0, 0, 0);
                    }
                }
                if (((uint32_t)t & (LPG - 1u)) == LPG - 1u) {
                    // group complete: fold the integer dot into the accumulators.  Register r of this lane is
                    // activation row (r % 4) + 8 * (r / 4) + 4 * kb; rows 16 .. 31 do not exist here (r >= 8).
                    const uint32_t gl = ((uint32_t)t * 2u * VPL) >> 6;
                    const float* sxg = sxs + gl * 32u + 4u * kb;
                    const float4 sx0 = *reinterpret_cast<const float4*>(sxg), sx1 = *reinterpret_cast<const float4*>(sxg + 8);
#pragma unroll
                    for (int q = 0; q < MATS; ++q) {
                        const uint32_t sb = B.sb[q][gl];
                        const float sf = bf16_bits_to_f32(sb & 0xffffu), bf = bf16_bits_to_f32(sb >> 16);
                        acc[q][0] += fmaf(sf, c[q][0][0] + c[q][1][0], bf * sx0.x);
                        acc[q][1] += fmaf(sf, c[q][0][1] + c[q][1][1], bf * sx0.y);
                        acc[q][2] += fmaf(sf, c[q][0][2] + c[q][1][2], bf * sx0.z);
                        acc[q][3] += fmaf(sf, c[q][0][3] + c[q][1][3], bf * sx0.w);
                        acc[q][4] += fmaf(sf, c[q][0][4] + c[q][1][4], bf * sx1.x);
                        acc[q][5] += fmaf(sf, c[q][0][5] + c[q][1][5], bf * sx1.y);
                        acc[q][6] += fmaf(sf, c[q][0][6] + c[q][1][6], bf * sx1.z);
                        acc[q][7] += fmaf(sf, c[q][0][7] + c[q][1][7], bf * sx1.w);
                    }
                }
            }
        }
        __builtin_amdgcn_wave_barrier();  // the next slab's pieces are written behind these reads
    };

    // Two sets of registers: slab i + 1 is requested before slab i is touched.  (One loop exit per pair of steps,
    // so that the compiler does not have to assume, at the loop's top, that the set it is about to refill is
    // still being loaded.)
    Slab A, B;
    FK_WIDE_STAMP(0);
    fetch(wave, A);
    FK_WIDE_STAMP(1);
    for (uint32_t slab = wave; slab < n_slabs; slab += 2 * WAVES) {
        fetch(slab + WAVES, B);
        consume(slab, A);
        if (slab == wave) FK_WIDE_STAMP(2);
        fetch(slab + 2 * WAVES, A);
        if (slab + WAVES < n_slabs) consume(slab + WAVES, B);
        if (slab == wave) FK_WIDE_STAMP(3);
    }
    FK_WIDE_STAMP(4);

    // The waves meet: every wave parks its sums of the rows that exist, [wave][matrix][row][weight row of the block].
#pragma unroll
    for (int q = 0; q < MATS; ++q)
#pragma unroll
        for (int r = 0; r < 8; ++r) {
            const uint32_t m = (uint32_t)(r % 4 + 8 * (r / 4)) + 4u * kb;
            if (m < M) meet[((wave * MATS + q) * kWideMaxRows + m) * 32u + nl] = acc[q][r];
        }
    __syncthreads();
    FK_WIDE_STAMP(5);
    for (uint32_t e = threadIdx.x; e < M * 32u; e += WAVES * kWave) {
        const uint32_t m = e >> 5, col = e & 31u, nn = blockIdx.x * 32u + col;
        if (nn >= a.N) continue;
        float s[MATS];
#pragma unroll
        for (int q = 0; q < MATS; ++q) {
            s[q] = 0.f;
            for (int w = 0; w < WAVES; ++w) s[q] += meet[((w * MATS + q) * kWideMaxRows + m) * 32u + col];
        }
        uint32_t o;
        if constexpr (MATS == 2) {
            o = swiglu_bits(s[0], s[1], a.variant, 1.0f);
        } else {
            float v = s[0];
            if (a.bias) v += bf16_bits_to_f32(a.bias[nn]);
            if (a.res) v += bf16_bits_to_f32(a.res[(size_t)m * a.N + nn]);
            o = f32_to_bf16_bits(v);
        }
        a.y[(size_t)m * a.N + nn] = (uint16_t)o;
    }
    FK_WIDE_STAMP(6);
}


// ---- up to 8 rows: 16 x 16 x 32 tiles ---------------------------------------------------------------------------
// v_mfma_f32_16x16x32_bf16: lane (c = lane % 16, kq = lane / 16) supplies 8 values of k block kq for row / column c
// and holds C[4 * kq + r][c].  A quantisation group is 64 codes = two k blocks of 32, so one instruction would mix
// two groups; instead the A operand carries every activation row TWICE -- row m with only the k blocks 0, 1, row
// m + 8 with only the k blocks 2, 3 -- and one instruction yields the integer dots of two groups side by side:
// lanes kq 0, 1 hold the even group's dots of rows 0..7, lanes kq 2, 3 the odd group's.  A lane therefore folds
// exactly the group whose codes it loaded (one scale / bias pair per lane and double group), and the two halves
// meet once at the end.  Against the 32 x 32 x 16 form: no padding rows beyond 8 of 16 (there 22 of 32), four
// accumulator registers per tile instead of sixteen, a fold of 4 values instead of 8 x 2.
// A block still owns 32 weight rows (two tiles of 16) over all of K, its waves split K in slabs of 256.
template <WKind KIND, int MATS, int WAVES, int TILES>
__global__ __launch_bounds__(WAVES* kWave) void qgemm_wide16_kernel(const QgemmWideArgs a) {
    constexpr uint32_t VPL = KIND == W_Q4 ? 32u : 16u;  // codes per 16-byte lane load
    constexpr int MF = VPL / 8;                         // matrix instructions per load
    constexpr int LU = 32 / VPL;                        // loads per lane, tile and double group
    constexpr int DGS = kWideSlab / 128u;               // double groups per slab
    constexpr int UNITS = kWideSlab / 64u;
    extern __shared__ uint4 lds_raw[];
    const uint32_t lane = threadIdx.x & 63u, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t c16 = lane & 15u, kq = lane >> 4, gsel = kq >> 1, hf = kq & 1u;
    uint4* xs = reinterpret_cast<uint4*>(reinterpret_cast<char*>(lds_raw) + wave * wide_wave_lds());
    float* sxs = reinterpret_cast<float*>(xs + kWideXRows * kWideXS);
    float* meet = reinterpret_cast<float*>(reinterpret_cast<char*>(lds_raw) + WAVES * wide_wave_lds());

    float* rrs = reinterpret_cast<float*>(reinterpret_cast<char*>(meet) + wide_meet_bytes(WAVES, MATS));  // [rows] 1 / rms

    const uint32_t M = a.M;
    const uint32_t n_slabs = (a.K + kWideSlab - 1) / kWideSlab;
    // one matrix per block: which of the (up to three) matrices this block serves
    uint32_t seg = 0, blk = blockIdx.x;
    if constexpr (MATS == 1) {
        if (a.n_seg > 1 && blockIdx.x >= a.blk0[1]) seg = 1;
        if (a.n_seg > 2 && blockIdx.x >= a.blk0[2]) seg = 2;
        blk = blockIdx.x - a.blk0[seg];
    }
    const uint32_t N = MATS == 1 ? a.ns[seg] : a.N;
    const uint4* wb[MATS];
    const uint16_t *scb[MATS], *bib[MATS];
#pragma unroll
    for (int q = 0; q < MATS; ++q) {
        wb[q] = a.w[MATS == 1 ? seg : (uint32_t)q];
        scb[q] = a.sc[MATS == 1 ? seg : (uint32_t)q];
        bib[q] = a.bi[MATS == 1 ? seg : (uint32_t)q];
    }
    const bool normed = a.norm_w != nullptr;
    if (normed) {
        // 1 / rms of every activation row: wave w takes rows w, w + WAVES, ...
        for (uint32_t m = wave; m < M; m += WAVES) {
            const uint4* xr = reinterpret_cast<const uint4*>(a.x + (size_t)m * a.x_stride);
            float ss = 0.f;
            for (uint32_t i = lane; i < (a.K >> 3); i += kWave) {
                const uint4 v = xr[i];
                const uint32_t wd[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
                for (int t = 0; t < 4; ++t) {
                    const float lo = bf16_lo(wd[t]), hi = bf16_hi(wd[t]);
                    ss = fmaf(lo, lo, ss);
                    ss = fmaf(hi, hi, ss);
                }
            }
            ss = wave_sum(ss);
            if (lane == 0) rrs[m] = 1.0f / sqrtf(ss / (float)a.K + a.eps);
        }
        __syncthreads();
    }
    for (uint32_t i = lane; i < kWideXS; i += kWave) xs[kWideMaxRows * kWideXS + i] = make_uint4(0, 0, 0, 0);
    for (uint32_t i = lane; i < UNITS * 32u; i += kWave) sxs[i] = 0.f;
    // A operand row c16: activation row c16 % 8, live only in the k blocks of group half c16 / 8
    const uint32_t am = c16 & 7u;
    const uint32_t arow = (am < M && (c16 >> 3) == gsel) ? am : kWideMaxRows;

    const uint4* wrow[MATS][TILES];
    const uint16_t *srow[MATS][TILES], *brow[MATS][TILES];
#pragma unroll
    for (int q = 0; q < MATS; ++q)
#pragma unroll
        for (int h = 0; h < TILES; ++h) {
            const uint32_t n = blk * (16u * TILES) + (uint32_t)h * 16u + c16, nc = n < N ? n : N - 1;
            wrow[q][h] = wb[q] + (size_t)nc * a.cpr;
            srow[q][h] = scb[q] + (size_t)nc * a.gpr;
            brow[q][h] = bib[q] + (size_t)nc * a.gpr;
        }

    f32x4_t acc[MATS][TILES];
#pragma unroll
    for (int q = 0; q < MATS; ++q)
#pragma unroll
        for (int h = 0; h < TILES; ++h) acc[q][h] = f32x4_t{0.f, 0.f, 0.f, 0.f};

    struct Slab {
        uint4 w[MATS][TILES][DGS * LU], x[kWideXPT], nw;
        uint32_t sb[MATS][TILES][DGS];
    };
    // code offset inside a slab of this lane's load u of double group d
    auto k_of = [&](int d, int u) { return (uint32_t)d * 128u + gsel * 64u + (hf + 2u * (uint32_t)u) * VPL; };
    auto fetch = [&](uint32_t slab, Slab& B) {
        const bool live = slab < n_slabs;
        const uint32_t ks0 = live ? slab * kWideSlab : 0u;
        const uint32_t slab_k = a.K - ks0 < kWideSlab ? a.K - ks0 : kWideSlab;
        const uint32_t s8 = live ? slab_k >> 3 : 0u;
#pragma unroll
        for (int q = 0; q < MATS; ++q)
#pragma unroll
            for (int h = 0; h < TILES; ++h) {
#pragma unroll
                for (int d = 0; d < DGS; ++d) {
#pragma unroll
                    for (int u = 0; u < LU; ++u) {
                        const bool have = live && k_of(d, u) < slab_k;   // K is whole groups: a group is inside or outside
                        B.w[q][h][d * LU + u] = (have ? wrow[q][h] : wb[q])[have ? (ks0 + k_of(d, u)) / VPL : 0u];
                    }
                    const uint32_t gl = 2u * (uint32_t)d + gsel;
                    const bool have = live && gl * 64u < slab_k;
                    const uint32_t g = have ? (ks0 >> 6) + gl : 0u;
                    B.sb[q][h][d] = (uint32_t)(have ? srow[q][h] : scb[q])[g] | ((uint32_t)(have ? brow[q][h] : bib[q])[g] << 16);
                }
            }
#pragma unroll
        for (int i = 0; i < kWideXPT; ++i) {
            const uint32_t idx = lane + (uint32_t)i * kWave, m = idx / (kWideSlab / 8), k8 = idx % (kWideSlab / 8);
            const bool have = m < M && k8 < s8;
            B.x[i] = *reinterpret_cast<const uint4*>(a.x + (size_t)(have ? m : 0u) * a.x_stride + ks0 + (have ? k8 : 0u) * 8u);
        }
        // the norm weights of this lane's pieces: k8 = lane % 32 for every one of them (straight-line: without a norm
        // the request reads the activations' first bytes)
        {
            const uint32_t k8 = lane & (kWideSlab / 8 - 1);
            B.nw = *reinterpret_cast<const uint4*>((normed ? a.norm_w : a.x) + (normed ? ks0 + (k8 < s8 ? k8 : 0u) * 8u : 0u));
        }
    };
    auto consume = [&](uint32_t slab, const Slab& B) {
        const uint32_t ks0 = slab * kWideSlab;
        const uint32_t slab_k = a.K - ks0 < kWideSlab ? a.K - ks0 : kWideSlab;
#pragma unroll
        for (int i = 0; i < kWideXPT; ++i) {
            const uint32_t idx = lane + (uint32_t)i * kWave, m = idx / (kWideSlab / 8), k8 = idx % (kWideSlab / 8);
            uint4 v = (m < M && k8 < (slab_k >> 3)) ? B.x[i] : make_uint4(0, 0, 0, 0);
            if (normed) {  // block-uniform
                const float r = rrs[m < M ? m : 0u];
                const uint32_t xv[4] = {v.x, v.y, v.z, v.w}, wv[4] = {B.nw.x, B.nw.y, B.nw.z, B.nw.w};
                uint32_t o[4];
#pragma unroll
                for (int t = 0; t < 4; ++t) {
                    const uint32_t xr2 = pack_bf16(bf16_lo(xv[t]) * r, bf16_hi(xv[t]) * r);   // T(x * r)
                    o[t] = pack_bf16(bf16_lo(wv[t]) * bf16_lo(xr2), bf16_hi(wv[t]) * bf16_hi(xr2));  // T(w * .)
                }
                v = make_uint4(o[0], o[1], o[2], o[3]);
            }
            if constexpr (KIND == W_Q4) {
                v = make_uint4((v.x & 0xffffu) | (v.y << 16), (v.z & 0xffffu) | (v.w << 16),
                               (v.x >> 16) | (v.y & 0xffff0000u), (v.z >> 16) | (v.w & 0xffff0000u));
            }
            if (m < kWideMaxRows) xs[m * kWideXS + k8] = v;
        }
        __builtin_amdgcn_wave_barrier();
        {
            const uint32_t g = lane >> 4, m = lane & 15u;
            if (m < M) {
                float s0 = 0.f, s1 = 0.f;
                if (g < (slab_k >> 6)) {
#pragma unroll
                    for (uint32_t i = 0; i < 8; ++i) {
                        const uint4 v = xs[m * kWideXS + g * 8u + i];
                        s0 = dot2_bf16(v.x, 0x3F803F80u, s0);
                        s1 = dot2_bf16(v.y, 0x3F803F80u, s1);
                        s0 = dot2_bf16(v.z, 0x3F803F80u, s0);
                        s1 = dot2_bf16(v.w, 0x3F803F80u, s1);
                    }
                }
                sxs[g * 32u + m] = s0 + s1;
            }
        }
        __builtin_amdgcn_wave_barrier();

        const f32x4_t zero = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int d = 0; d < DGS; ++d) {
            if ((uint32_t)d * 128u < slab_k) {  // wave-uniform; a lane whose group lies past the slab multiplies zeros
                f32x4_t c[MATS][TILES];
#pragma unroll
                for (int u = 0; u < LU; ++u) {
                    const uint4* xa = xs + arow * kWideXS + (k_of(d, u) >> 3);
#pragma unroll
                    for (int j = 0; j < MF; ++j) {
                        const uint4 av = xa[j];
#pragma unroll
                        for (int q = 0; q < MATS; ++q)
#pragma unroll
                            for (int h = 0; h < TILES; ++h) {
                                const uint4 wv = B.w[q][h][d * LU + u];
                                const uint32_t wd[4] = {wv.x, wv.y, wv.z, wv.w};
                                uint4 bw;
                                if constexpr (KIND == W_Q4) {
                                    const uint32_t even = wd[j] & 0x0F0F0F0Fu, odd = (wd[j] >> 4) & 0x0F0F0F0Fu;
                                    bw.x = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(even, 512.0f, false));
                                    bw.y = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(even, 512.0f, true));
                                    bw.z = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(odd, 512.0f, false));
                                    bw.w = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(odd, 512.0f, true));
                                } else {
                                    const uint32_t w0 = wd[(2 * j) & 3], w1 = wd[(2 * j + 1) & 3];
                                    auto pair = [](float lo, float hi) {
                                        const bf16x2_t p = {(__bf16)lo, (__bf16)hi};  // integers <= 255 are exact in bf16
                                        return __builtin_bit_cast(uint32_t, p);
                                    };
                                    bw.x = pair((float)(w0 & 0xffu), (float)((w0 >> 8) & 0xffu));
                                    bw.y = pair((float)((w0 >> 16) & 0xffu), (float)(w0 >> 24));
                                    bw.z = pair((float)(w1 & 0xffu), (float)((w1 >> 8) & 0xffu));
                                    bw.w = pair((float)((w1 >> 16) & 0xffu), (float)(w1 >> 24));
                                }
                                const bool first = u * MF + j == 0;
                                c[q][h] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, av),
                                                                                 __builtin_bit_cast(bf16x8_t, bw),
                                                                                 first ? zero : c[q][h], 0, 0, 0);
                            }
                    }
                }
                // fold this lane's group (2 d + gsel): C register r is activation row 4 * hf + r
                const float4 sx = *reinterpret_cast<const float4*>(sxs + (2u * (uint32_t)d + gsel) * 32u + 4u * hf);
#pragma unroll
                for (int q = 0; q < MATS; ++q)
#pragma unroll
                    for (int h = 0; h < TILES; ++h) {
                        const uint32_t sb = B.sb[q][h][d];
                        const float sf = bf16_bits_to_f32(sb & 0xffffu), bf = bf16_bits_to_f32(sb >> 16);
                        acc[q][h][0] += fmaf(sf, c[q][h][0], bf * sx.x);
                        acc[q][h][1] += fmaf(sf, c[q][h][1], bf * sx.y);
                        acc[q][h][2] += fmaf(sf, c[q][h][2], bf * sx.z);
                        acc[q][h][3] += fmaf(sf, c[q][h][3], bf * sx.w);
                    }
            }
        }
        __builtin_amdgcn_wave_barrier();
    };

    Slab A, B;
    fetch(wave, A);
    for (uint32_t slab = wave; slab < n_slabs; slab += 2 * WAVES) {
        fetch(slab + WAVES, B);
        consume(slab, A);
        fetch(slab + 2 * WAVES, A);
        if (slab + WAVES < n_slabs) consume(slab + WAVES, B);
    }

    // the two group halves of a row meet (lane ^ 32), then the waves as in the 32 x 32 form
#pragma unroll
    for (int q = 0; q < MATS; ++q)
#pragma unroll
        for (int h = 0; h < TILES; ++h)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const float v = acc[q][h][r] + __shfl_xor(acc[q][h][r], 32);
                const uint32_t m = 4u * hf + (uint32_t)r;
                if (gsel == 0 && m < M) meet[((wave * MATS + q) * kWideMaxRows + m) * 32u + (uint32_t)h * 16u + c16] = v;
            }
    __syncthreads();
    constexpr uint32_t COLS = 16u * TILES;
    uint16_t* yo = MATS == 1 ? a.ys[seg] : a.y;
    const uint32_t yst = MATS == 1 ? a.y_stride[seg] : a.N;
    for (uint32_t e = threadIdx.x; e < M * COLS; e += WAVES * kWave) {
        const uint32_t m = e / COLS, col = e % COLS, nn = blk * COLS + col;
        if (nn >= N) continue;
        float s[MATS];
#pragma unroll
        for (int q = 0; q < MATS; ++q) {
            s[q] = 0.f;
            for (int w = 0; w < WAVES; ++w) s[q] += meet[((w * MATS + q) * kWideMaxRows + m) * 32u + col];
        }
        uint32_t o;
        if constexpr (MATS == 2) {
            o = swiglu_bits(s[0], s[1], a.variant, 1.0f);
        } else {
            float v = s[0];
            if (a.bias) v += bf16_bits_to_f32(a.bias[nn]);
            if (a.res) v += bf16_bits_to_f32(a.res[(size_t)m * N + nn]);
            o = f32_to_bf16_bits(v);
        }
        yo[(size_t)m * yst + nn] = (uint16_t)o;
    }
}

template <WKind KIND, int MATS>
const void* wide_func(uint32_t waves, bool tiles16, bool one_tile) {
    if (tiles16 && one_tile)
        return waves == 8 ? reinterpret_cast<const void*>(&qgemm_wide16_kernel<KIND, MATS, 8, 1>)
                          : reinterpret_cast<const void*>(&qgemm_wide16_kernel<KIND, MATS, 4, 1>);
    if (tiles16)
        return waves == 8 ? reinterpret_cast<const void*>(&qgemm_wide16_kernel<KIND, MATS, 8, 2>)
                          : reinterpret_cast<const void*>(&qgemm_wide16_kernel<KIND, MATS, 4, 2>);
    return waves == 8 ? reinterpret_cast<const void*>(&qgemm_wide_kernel<KIND, MATS, 8>)
                      : reinterpret_cast<const void*>(&qgemm_wide_kernel<KIND, MATS, 4>);
}

}  // namespace

static bool g_wide_on = true;
static const bool g_wide_tiles16 = true;   // 9728 x 2560 int4, 8 rows: 13.86 us with 32 x 32 x 16 tiles, 12.51 with 16 x 16 x 32
void set_qgemm_wide(bool on) { g_wide_on = on; }
bool qgemm_takes_wide(uint32_t M, uint32_t group) { return g_wide_on && M >= 2 && M <= kWideMaxRows && group == 64; }

// W1 (and SwiGLU of the pair) or bias / res (single matrix).
fk_status plan_qgemm_wide(const fk_weight* W0, const fk_weight* W1, const uint16_t* x, uint32_t M, const uint16_t* bias,
                          const uint16_t* res, int variant, uint16_t* y, Launch* out, const uint16_t* norm_w, float eps) {
    const DeviceFacts* dev;
    FK_TRY(device_facts(&dev));
    if (!qgemm_takes_wide(M, W0->group)) return set_error(FK_ERR_UNSUPPORTED, "qgemm (shared stream): 2..10 rows, group size 64");
    if (W0->k % 64u) return set_error(FK_ERR_UNSUPPORTED, "qgemm (shared stream): K must be a multiple of 64");
    QgemmWideArgs a;
    memset(&a, 0, sizeof(a));
    const fk_weight* Ws[2] = {W0, W1};
    for (int q = 0; q < (W1 ? 2 : 1); ++q) {
        a.w[q] = reinterpret_cast<const uint4*>(Ws[q]->w);
        a.sc[q] = Ws[q]->scales;
        a.bi[q] = Ws[q]->biases;
    }
    a.x = x; a.bias = bias; a.res = res; a.y = y;
    a.M = M; a.N = W0->n; a.K = W0->k;
    a.n_seg = 1; a.x_stride = W0->k;
    a.ns[0] = W0->n; a.blk0[0] = 0; a.y_stride[0] = W0->n; a.ys[0] = y;
    if (norm_w) {  // the activations are RMS-normalised while they are staged: the 16-row form only
        if (M > 8 || !g_wide_tiles16) return set_error(FK_ERR_UNSUPPORTED, "qgemm (shared stream): a fused norm takes 2..8 rows");
        if (((uintptr_t)norm_w | (uintptr_t)x) & 15u) return set_error(FK_ERR_INVALID, "qgemm (shared stream): rows and norm weights must be 16-byte aligned");
        a.norm_w = norm_w;
        a.eps = eps;
    }
    a.cpr = W0->k / (W0->bits == 4 ? 32u : 16u);
    a.gpr = W0->k / 64u;
    a.variant = variant;
    // Eight waves per block (K split eight ways) while every block still finds a CU of its own; four beyond
    // (registers allow one eight-wave block per CU).  Measured with the 32 x 32 x 16 form, 8 rows of int4, serialised
    // graph, against the split-k kernel + reduction: 6144 x 2560 8.5 us (15.6), 2560 x 4096 11.2 (18.4),
    // 2048 x 1408 5.8 (10.2), 1408 x 2048 6.9 (11.4), 9728 x 2560 14.0 (16.3), 2560 x 9728 21.0 (21.7).
    const bool t16 = g_wide_tiles16 && M <= 8;   // up to 8 rows: the 16 x 16 x 32 tiling
    // The 16-row form may give a block ONE tile: twice the blocks, each wave half the arithmetic per slab.  What these
    // launches lack is waves to hide their LDS round trips behind, not bandwidth, so the smaller block wins wherever
    // the grid is short (8 rows of int4, one / two tiles: 2048 x 2048 5.8 / 7.7 us, 3072 x 2048 6.0 / 7.7,
    // 2560 x 9728 13.3 / 18.8, 9728 x 2560 11.8 / 12.6) and loses where the two-tile grid already fills the chip or
    // the eight-wave form would be lost (6144 x 2560 9.6 / 8.1, 19456 x 2560 17.3 / 16.3, 77824 x 2560 54 / 46).
    const uint32_t n_slabs = (W0->k + kWideSlab - 1) / kWideSlab, b16 = (W0->n + 15u) / 16u, b32 = (W0->n + 31u) / 32u;
    const uint32_t cus = (uint32_t)dev->cus;
    const bool deep = n_slabs >= 5u;
    const bool one_tile = t16 && ((deep && b16 <= cus) || (!(deep && b32 <= cus) && b16 <= 3u * cus));
    const uint32_t blocks = one_tile ? b16 : b32;
    const uint32_t waves = (blocks <= cus && deep) ? 8u : 4u;
    const bool q4 = W0->bits == 4;
    out->func = W1 ? (q4 ? wide_func<W_Q4, 2>(waves, t16, one_tile) : wide_func<W_Q8, 2>(waves, t16, one_tile))
                   : (q4 ? wide_func<W_Q4, 1>(waves, t16, one_tile) : wide_func<W_Q8, 1>(waves, t16, one_tile));
    out->grid = dim3(blocks, 1, 1);
    out->block = dim3(waves * kWave, 1, 1);
    out->shmem = wide_lds_bytes(waves, W1 ? 2u : 1u);
    out->set_args(a);
    if (out->shmem > 48 * 1024)
        FK_HIP(hipFuncSetAttribute(out->func, hipFuncAttributeMaxDynamicSharedMemorySize, (int)out->shmem));
    return FK_OK;
}

// Up to three matrices over the same activations in ONE launch of the 16-row form (2 .. 8 rows), each with its own
// output and row stride; with norm_w the rows are RMS-normalised while they are staged.  The row form of the
// RMSNorm -> Q, K, V fan-out (src/codegen/kernels/rmsnorm_qkv.rs:53-736 with active_m > 1).
fk_status plan_qgemm_wide_fan(const uint16_t* x, uint32_t x_stride, uint32_t M, const uint16_t* norm_w, float eps,
                              const WideSeg* segs, uint32_t n_seg, Launch* out) {
    const DeviceFacts* dev;
    FK_TRY(device_facts(&dev));
    if (!x || !segs || n_seg == 0 || n_seg > 3) return set_error(FK_ERR_INVALID, "qgemm fan-out: one to three matrices");
    const fk_weight* W0 = segs[0].W;
    if (!W0) return set_error(FK_ERR_INVALID, "qgemm fan-out: null weight");
    if (!g_wide_on || M < 2 || M > 8 || W0->group != 64 || (W0->bits != 4 && W0->bits != 8))
        return set_error(FK_ERR_UNSUPPORTED, "qgemm fan-out: 2..8 rows, 4- or 8-bit weights, group size 64");
    if (W0->k % 64u || x_stride < W0->k || x_stride % 8u || ((uintptr_t)x & 15u) || (norm_w && ((uintptr_t)norm_w & 15u)))
        return set_error(FK_ERR_INVALID, "qgemm fan-out: K must be whole groups, rows and norm weights 16-byte aligned");
    QgemmWideArgs a;
    memset(&a, 0, sizeof(a));
    uint32_t b16 = 0, b32 = 0;
    for (uint32_t i = 0; i < n_seg; ++i) {
        const fk_weight* W = segs[i].W;
        if (!W || !W->w || !W->scales || !W->biases || !segs[i].y) return set_error(FK_ERR_INVALID, "qgemm fan-out: null matrix or output");
        if (W->k != W0->k || W->bits != W0->bits || W->group != W0->group || W->n == 0)
            return set_error(FK_ERR_INVALID, "qgemm fan-out: the matrices must share K, bits and group size");
        if (segs[i].y_stride < W->n) return set_error(FK_ERR_INVALID, "qgemm fan-out: output row stride below the matrix's rows");
        a.w[i] = reinterpret_cast<const uint4*>(W->w);
        a.sc[i] = W->scales;
        a.bi[i] = W->biases;
        a.ns[i] = W->n;
        a.ys[i] = segs[i].y;
        a.y_stride[i] = segs[i].y_stride;
        b16 += (W->n + 15u) / 16u;
        b32 += (W->n + 31u) / 32u;
    }
    a.x = x; a.M = M; a.N = W0->n; a.K = W0->k;
    a.cpr = W0->k / (W0->bits == 4 ? 32u : 16u);
    a.gpr = W0->k / 64u;
    a.n_seg = n_seg; a.x_stride = x_stride;
    a.norm_w = norm_w; a.eps = eps;
    const uint32_t n_slabs = (W0->k + kWideSlab - 1) / kWideSlab, cus = (uint32_t)dev->cus;
    const bool deep = n_slabs >= 5u;
    const bool one_tile = (deep && b16 <= cus) || (!(deep && b32 <= cus) && b16 <= 3u * cus);   // as plan_qgemm_wide
    uint32_t blocks = 0;
    for (uint32_t i = 0; i < n_seg; ++i) {
        a.blk0[i] = blocks;
        blocks += one_tile ? (a.ns[i] + 15u) / 16u : (a.ns[i] + 31u) / 32u;
    }
    const uint32_t waves = (blocks <= cus && deep) ? 8u : 4u;
    out->func = W0->bits == 4 ? wide_func<W_Q4, 1>(waves, true, one_tile) : wide_func<W_Q8, 1>(waves, true, one_tile);
    out->grid = dim3(blocks, 1, 1);
    out->block = dim3(waves * kWave, 1, 1);
    out->shmem = wide_lds_bytes(waves, 1u);
    out->set_args(a);
    if (out->shmem > 48 * 1024)
        FK_HIP(hipFuncSetAttribute(out->func, hipFuncAttributeMaxDynamicSharedMemorySize, (int)out->shmem));
    return FK_OK;
}

}  // namespace fk
