// Multi-row quantised matmul y[M, N] = T(x[M, K] @ dequant(W)^T) on the gfx950
// matrix cores: the path for 2 .. a few hundred activation rows (multi-token
// prediction, batched decode, prefill), where the weight stream is still the
// dominant traffic and must be read once for all rows.
//
// v_mfma_f32_32x32x16_bf16 with the WEIGHTS as the B operand: a lane then owns one
// weight row n (output column) for all 16 accumulator registers, so the affine
// scale and bias of (n, group) are one value per lane and group:
//     acc[m, n] += s[n, g] * (sum_k q[n, k] x[m, k])  +  b[n, g] * Sx[m, g]
// The integer codes go into the MFMA as exact bf16 values (int4 through the fp8
// convert used by the GEMV, int8 through v_cvt_f32_ubyte + v_cvt_pk_bf16_f32), the
// inner sum is accumulated per group in a zeroed C tile and folded into the fp32
// accumulators with the scale when the group ends.
//
// Lane (n = lane % 32, kb = lane / 32) loads 16 bytes = 32 int4 (16 int8) codes of
// row n: the two kb halves read adjacent 16-byte pieces, so one wave load covers
// 64 (32) consecutive k of 32 rows, all inside one quantisation group (group size
// 64 or 128).  MFMA step j takes word j (words 2j, 2j+1) of every lane: its 16 k
// values are 8 from each half, matched by the activation fragment read from LDS.
//
// From 65 activation rows up (MT = 4) the affine map is applied BEFORE the matrix
// instruction instead: w = T(s * q + b), one bf16 rounding per weight element, as the
// reference's multi-row path does (it dequantises into bf16 tiles, msl.rs:2318-2440), and the
// products accumulate straight into the fp32 result.  The fold per group (32 VALU
// instructions per tile of 32 rows and group of 64) is what bounds the exact form; the
// dequantised form spends 22 VALU instructions per fragment, shared by four tiles, and is
// bound by the matrix cores.
//
// A block is 4 waves = 128 weight rows over one k range and MT tiles of 32
// activation rows (MT = 1, 2 or 4 by the row count): a fragment of unpacked weights
// feeds MT matrix instructions, so the unpack work, which bounds this kernel, is
// shared by up to 128 rows.  x is staged per k slab (512, or 256 for MT = 4) into LDS
// in the lane order the MFMA wants (and, for int4, in the nibble pairing of the unpack).  The k dimension is
// split over blocks until the grid fills the chip; partial sums go to an fp32
// workspace and a second kernel adds them in split order and applies the epilogue,
// so the result does not depend on block scheduling.
#include <mutex>

#include <stdlib.h>

#include "fk_host.hpp"
#include "gemv_kernel.hpp"

namespace fk {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x16_t __attribute__((ext_vector_type(16)));

constexpr int kQgemmBlock = 256;
constexpr uint32_t kQgemmRows = 128;   // weight rows per block
constexpr uint32_t kQgemmMTile = 32;   // activation rows per block
constexpr uint32_t qgemm_slab_k(int mt) { return mt == 4 ? 256u : 512u; }                // k staged per LDS slab
constexpr uint32_t qgemm_x_stride(int mt) { return qgemm_slab_k(mt) / 8 + 1; }            // uint4 per staged row (+1: bank spread)
constexpr uint32_t qgemm_lds_bytes(int mt) {
    return (uint32_t)mt * kQgemmMTile * qgemm_x_stride(mt) * 16u + (qgemm_slab_k(mt) / 64u) * (uint32_t)mt * kQgemmMTile * 4u;
}

struct QgemmArgs {
    const uint4* w;
    const uint16_t* sc;
    const uint16_t* bi;
    const uint16_t* x;  // [M, K] bf16
    float* partial;     // [ksplit, M, N]
    uint32_t M, N, K;
    uint32_t cpr;          // 16-byte chunks per weight row
    uint32_t gpr;          // groups per row
    uint32_t group;        // 64 or 128
    uint32_t k_per_split;  // multiple of group
    uint32_t n_blocks;     // blocks along N
    // the tile form with one k split writes finished outputs (null: partial sums as above)
    uint16_t* y;
    const uint16_t* bias;
    const uint16_t* res;
    // the tile form over up to three matrices that share x and K (a q / k / v fan-out): n_seg > 1, the blocks along N
    // run through the matrices in turn (seg[i].nb_end: first block behind matrix i); partial sums of all matrices lie
    // side by side in rows of n_total columns (matrix i from column seg[i].col0)
    uint32_t n_seg, n_total;
    struct Seg {
        const uint4* w;
        const uint16_t* sc;
        const uint16_t* bi;
        uint16_t* y;
        const uint16_t* bias;
        uint32_t N, nb_end, col0, pad;
    } seg[3];
    // the tile form for a gate / up pair: the second matrix (same shape), its partial sums, the SwiGLU variant
    const uint4* w2;
    const uint16_t* sc2;
    const uint16_t* bi2;
    float* partial2;
    int variant;
};

template <WKind KIND, int MT>
__global__ __launch_bounds__(kQgemmBlock) void qgemm_kernel(const QgemmArgs a) {
    constexpr uint32_t VPL = KIND == W_Q4 ? 32u : 16u;  // codes per 16-byte lane load
    constexpr int MF = VPL / 8;                         // MFMA steps per load
    constexpr uint32_t SLAB = qgemm_slab_k(MT), XS = qgemm_x_stride(MT), ROWS = MT * kQgemmMTile;
    constexpr bool DEQ = MT == 4;  // weights dequantised to bf16 before the multiply (see the head of this file)
    constexpr int LOADS = SLAB / (2u * VPL);            // 16-byte weight loads per lane and slab
    constexpr int UNITS = SLAB / 64u;                   // 64-k units per slab (one scale / bias pair each)
    constexpr uint32_t S8 = SLAB / 8u;                  // 16-byte pieces of x per row and slab
    constexpr int XPT = ROWS * S8 / kQgemmBlock;        // pieces of x per thread and slab
    extern __shared__ uint4 lds_raw[];
    uint4* xs = lds_raw;                                       // [ROWS][XS]
    float* sxs = reinterpret_cast<float*>(xs + ROWS * XS);     // [groups in slab][ROWS]

    const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6, kb = lane >> 5, nl = lane & 31u;
    const uint32_t nb = blockIdx.x % a.n_blocks, ks = blockIdx.x / a.n_blocks;
    const uint32_t m0 = blockIdx.y * ROWS;
    const uint32_t mt = a.M - m0 < ROWS ? a.M - m0 : ROWS;  // live activation rows of this block
    const uint32_t n = nb * kQgemmRows + wave * 32u + nl;
    const uint32_t nc = n < a.N ? n : a.N - 1;  // rows past the end read the last row; never stored
    const uint32_t k0 = ks * a.k_per_split;
    const uint32_t k1 = k0 + a.k_per_split < a.K ? k0 + a.k_per_split : a.K;

    const uint4* wrow = a.w + (size_t)nc * a.cpr;
    const uint16_t* srow = a.sc + (size_t)nc * a.gpr;
    const uint16_t* brow = a.bi + (size_t)nc * a.gpr;
    const uint32_t lpg_mask = a.group / (2u * VPL) - 1u;  // loads per group - 1 (power of two)
    const uint32_t g8 = a.group >> 3;
    const uint32_t gshift = a.group == 128 ? 7u : 6u;

    f32x16_t acc[MT];
#pragma unroll
    for (int i = 0; i < MT; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[i][r] = 0.f;

    // Everything a slab needs from memory is requested one slab ahead, while the previous one
    // is multiplied: the weight pieces and scale / bias pairs of this lane's row, and this
    // thread's share of the activations (parked in registers until the LDS tile is free).
    // With one request in flight per lane the kernel ran at the latency of its loads.
    uint4 wq[LOADS], xq[XPT];
    uint32_t sbq[UNITS];
    auto fetch = [&](uint32_t ks0) {
        const uint32_t slab_k = k1 - ks0 < SLAB ? k1 - ks0 : SLAB;
        const uint32_t loads = slab_k / (2u * VPL), units = slab_k >> 6, s8 = slab_k >> 3;
        const uint4* wp = wrow + ks0 / VPL + kb;
#pragma unroll
        for (int t = 0; t < LOADS; ++t) wq[t] = wp[2u * ((uint32_t)t < loads ? (uint32_t)t : 0u)];
#pragma unroll
        for (int u = 0; u < UNITS; ++u) {
            const uint32_t g = (ks0 + ((uint32_t)u < units ? (uint32_t)u : 0u) * 64u) >> gshift;
            sbq[u] = (uint32_t)srow[g] | ((uint32_t)brow[g] << 16);
        }
        // requests only: nothing here may use a loaded value (that would wait for it before the
        // remaining requests are made); rows and slab tails that do not exist are zeroed when
        // the piece is written to LDS
#pragma unroll
        for (int i = 0; i < XPT; ++i) {
            const uint32_t idx = threadIdx.x + (uint32_t)i * kQgemmBlock, m = idx / S8, k8 = idx % S8;
            const bool live = m < mt && k8 < s8;
            xq[i] = *reinterpret_cast<const uint4*>(a.x + (size_t)(m0 + (live ? m : 0u)) * a.K + ks0 + (live ? k8 : 0u) * 8u);
        }
    };
    fetch(k0);

    for (uint32_t ks0 = k0; ks0 < k1; ks0 += SLAB) {
        const uint32_t slab_k = k1 - ks0 < SLAB ? k1 - ks0 : SLAB;
        __syncthreads();  // the previous slab has been consumed
#pragma unroll
        for (int i = 0; i < XPT; ++i) {
            const uint32_t idx = threadIdx.x + (uint32_t)i * kQgemmBlock, m = idx / S8, k8 = idx % S8;
            uint4 v = (m < mt && k8 < (slab_k >> 3)) ? xq[i] : make_uint4(0, 0, 0, 0);
            if constexpr (KIND == W_Q4 && !DEQ) {
                // nibble pairing of q4_word_dot: (x0,x2) (x4,x6) (x1,x3) (x5,x7); the dequantising
                // form pairs its codes in element order instead and takes x as it lies
                v = make_uint4((v.x & 0xffffu) | (v.y << 16), (v.z & 0xffffu) | (v.w << 16),
                               (v.x >> 16) | (v.y & 0xffff0000u), (v.z >> 16) | (v.w & 0xffff0000u));
            }
            xs[m * XS + k8] = v;
        }
        uint4 wcur[LOADS];
        uint32_t sbcur[UNITS];
#pragma unroll
        for (int t = 0; t < LOADS; ++t) wcur[t] = wq[t];
#pragma unroll
        for (int u = 0; u < UNITS; ++u) sbcur[u] = sbq[u];
        if (ks0 + SLAB < k1) fetch(ks0 + SLAB);
        __syncthreads();
        if constexpr (!DEQ) {
            const uint32_t ng = slab_k / a.group;
            for (uint32_t idx = threadIdx.x; idx < ng * ROWS; idx += kQgemmBlock) {
                const uint32_t g = idx / ROWS, m = idx - g * ROWS;
                float s = 0.f;
                for (uint32_t i = 0; i < g8; ++i) {
                    const uint4 v = xs[m * XS + g * g8 + i];
                    s += ((bf16_lo(v.x) + bf16_hi(v.x)) + (bf16_lo(v.y) + bf16_hi(v.y))) +
                         ((bf16_lo(v.z) + bf16_hi(v.z)) + (bf16_lo(v.w) + bf16_hi(v.w)));
                }
                sxs[idx] = s;
            }
            __syncthreads();
        }

        const uint32_t loads = slab_k / (2u * VPL);
        f32x16_t c[MT];
#pragma unroll
        for (int i = 0; i < MT; ++i)
#pragma unroll
            for (int r = 0; r < 16; ++r) c[i][r] = 0.f;
#pragma unroll
        for (int t = 0; t < LOADS; ++t) {
            if ((uint32_t)t < loads) {
                const uint32_t sb = sbcur[(t * 2 * (int)VPL) / 64];
                const float sf = bf16_bits_to_f32(sb & 0xffffu), bf = bf16_bits_to_f32(sb >> 16);
                const uint32_t wd[4] = {wcur[t].x, wcur[t].y, wcur[t].z, wcur[t].w};
                const uint4* xa = xs + nl * XS + (((uint32_t)t * 2u + kb) * VPL >> 3);
#pragma unroll
                for (int j = 0; j < MF; ++j) {
                    uint4 bw;
                    if constexpr (DEQ) {
                        // eight codes of this lane in element order: int4 word j holds them as nibbles
                        // (even ones in the bytes of `lo`, odd ones in those of `hi`), int8 as bytes
                        const uint32_t lo = KIND == W_Q4 ? (wd[j] & 0x0F0F0F0Fu) : wd[(2 * j) & 3];
                        const uint32_t hi = KIND == W_Q4 ? ((wd[j] >> 4) & 0x0F0F0F0Fu) : wd[(2 * j + 1) & 3];
                        auto dq = [&](uint32_t byte) { return fmaf((float)byte, sf, bf); };
                        if constexpr (KIND == W_Q4) {
                            bw.x = pack_bf16(dq(lo & 0xffu), dq(hi & 0xffu));
                            bw.y = pack_bf16(dq((lo >> 8) & 0xffu), dq((hi >> 8) & 0xffu));
                            bw.z = pack_bf16(dq((lo >> 16) & 0xffu), dq((hi >> 16) & 0xffu));
                            bw.w = pack_bf16(dq(lo >> 24), dq(hi >> 24));
                        } else {
                            bw.x = pack_bf16(dq(lo & 0xffu), dq((lo >> 8) & 0xffu));
                            bw.y = pack_bf16(dq((lo >> 16) & 0xffu), dq(lo >> 24));
                            bw.z = pack_bf16(dq(hi & 0xffu), dq((hi >> 8) & 0xffu));
                            bw.w = pack_bf16(dq((hi >> 16) & 0xffu), dq(hi >> 24));
                        }
                    } else if constexpr (KIND == W_Q4) {
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
                    // the unpacked fragment serves every tile of activation rows
#pragma unroll
                    for (int i = 0; i < MT; ++i) {
                        const uint4 av = xa[i * kQgemmMTile * XS + j];
                        if constexpr (DEQ)
                            acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, av),
                                                                             __builtin_bit_cast(bf16x8_t, bw), acc[i], 0, 0, 0);
                        else
                            c[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, av),
                                                                           __builtin_bit_cast(bf16x8_t, bw), c[i], 0, 0, 0);
                    }
                }
                if constexpr (!DEQ) {
                    if (((uint32_t)t & lpg_mask) == lpg_mask) {
                        // group complete: fold the integer dot into the accumulators.  Register r
                        // of this lane is activation row (r % 4) + 8 * (r / 4) + 4 * kb of its tile.
                        const uint32_t gl = ((uint32_t)t * 2u * VPL) >> gshift;  // group inside the slab
#pragma unroll
                        for (int i = 0; i < MT; ++i) {
                            const float* sxg = sxs + gl * ROWS + i * kQgemmMTile + 4u * kb;
#pragma unroll
                            for (int q = 0; q < 4; ++q) {
                                const float4 sx4 = *reinterpret_cast<const float4*>(sxg + 8 * q);
                                acc[i][4 * q + 0] += fmaf(sf, c[i][4 * q + 0], bf * sx4.x);
                                acc[i][4 * q + 1] += fmaf(sf, c[i][4 * q + 1], bf * sx4.y);
                                acc[i][4 * q + 2] += fmaf(sf, c[i][4 * q + 2], bf * sx4.z);
                                acc[i][4 * q + 3] += fmaf(sf, c[i][4 * q + 3], bf * sx4.w);
                            }
#pragma unroll
                            for (int r = 0; r < 16; ++r) c[i][r] = 0.f;
                        }
                    }
                }
            }
        }
    }

    if (n < a.N) {
        float* dst = a.partial + ((size_t)ks * a.M + m0) * a.N + n;
#pragma unroll
        for (int i = 0; i < MT; ++i)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const uint32_t m = (uint32_t)(i * (int)kQgemmMTile + r % 4 + 8 * (r / 4)) + 4u * kb;
                if (m < mt) dst[(size_t)m * a.N] = acc[i][r];
            }
    }
}

// ---- the tile form: from 65 activation rows ---------------------------------------------------------------------
// A block of EIGHT waves owns 256 activation rows x 128 weight rows and walks k in slabs of 64.  Both operands of a slab
// are staged in LDS once per block -- the activations as they lie, the weights dequantised to bf16 (w = T(s q + b), the
// arithmetic of the form above) by the one thread that loaded their 16 codes -- and every wave multiplies a 64 x 64
// part of the tile from there (four accumulators, 4 fragment reads per 4 matrix instructions).  Two waves share a SIMD:
// while one unpacks, stages or waits, the other one's matrix instructions keep the pipe busy (one wave per SIMD with
// everything interleaved by hand ran its phases one after the other: 65 us for 512 x 9728 x 2560, of which the matrix
// instructions alone are 21).  Two LDS buffers; a slab is requested two passes before it is staged (parked in named
// registers, one set for even and one for odd slabs), one barrier per slab.  Staged rows are 9 pieces of 16 bytes
// apart (8 used), which spreads the fragment reads of 8 neighbouring lanes over all banks.
// With one k split the block finishes its outputs itself (bias, residual, one rounding: the arithmetic of the second
// kernel below for one split); otherwise partial sums go out in the layout of the form above.
constexpr int kTileBlock = 512;
constexpr uint32_t kTileM = 256, kTileN = 128, kTileK = 64;   // (up to 128 activation rows: tiles of 128 rows, TM below)
// activation rows from which the form is planned: every row count of the bf16-weight arithmetic (a tile of 256 rows that
// is three quarters empty still beats the older form below, which unpacks per wave: 80-row prompt passes 14.7 k against
// 12.8 k tok/s on the 4B-class model, 128-row passes 22.2 k against 19.5 k; with tiles of 128 rows for up to 128 rows
// 18.1 k and 27.0 k)
constexpr uint32_t kTileMinRows = 65;
constexpr uint32_t kTileStride = kTileK / 8 + 1;                            // uint4 per staged row
// one buffer: x rows, then weight rows (a gate / up pair: the up rows behind the gate rows)
constexpr uint32_t tile_buf_pieces(bool pair, uint32_t tm) { return (tm + (pair ? 2u : 1u) * kTileN) * kTileStride; }
constexpr uint32_t tile_lds_bytes(bool pair, uint32_t tm) { return 2u * tile_buf_pieces(pair, tm) * 16u; }

// Piece p (codes 8 p .. 8 p + 7, element order) of the 16 codes one thread loaded (int4: w.x, w.y; int8: all of w) as
// eight bf16 weights T(s q + b).
template <WKind KIND>
__device__ __forceinline__ uint4 tile_unpack_piece(int p, const uint4 w, float sf, float bf) {
    uint4 bw;
    if constexpr (KIND == W_Q4) {
        const uint32_t word = p ? w.y : w.x;
        const uint32_t lo = word & 0x0F0F0F0Fu, hi = (word >> 4) & 0x0F0F0F0Fu;
        bw.x = pack_bf16(fmaf((float)(lo & 0xffu), sf, bf), fmaf((float)(hi & 0xffu), sf, bf));
        bw.y = pack_bf16(fmaf((float)((lo >> 8) & 0xffu), sf, bf), fmaf((float)((hi >> 8) & 0xffu), sf, bf));
        bw.z = pack_bf16(fmaf((float)((lo >> 16) & 0xffu), sf, bf), fmaf((float)((hi >> 16) & 0xffu), sf, bf));
        bw.w = pack_bf16(fmaf((float)(lo >> 24), sf, bf), fmaf((float)(hi >> 24), sf, bf));
    } else {
        const uint32_t lo = p ? w.z : w.x, hi = p ? w.w : w.y;
        bw.x = pack_bf16(fmaf((float)(lo & 0xffu), sf, bf), fmaf((float)((lo >> 8) & 0xffu), sf, bf));
        bw.y = pack_bf16(fmaf((float)((lo >> 16) & 0xffu), sf, bf), fmaf((float)(lo >> 24), sf, bf));
        bw.z = pack_bf16(fmaf((float)(hi & 0xffu), sf, bf), fmaf((float)((hi >> 8) & 0xffu), sf, bf));
        bw.w = pack_bf16(fmaf((float)((hi >> 16) & 0xffu), sf, bf), fmaf((float)(hi >> 24), sf, bf));
    }
    return bw;
}

// PAIR: a gate / up pair of the same shape in one launch -- the activations are requested and staged once for both,
// every wave keeps a second set of accumulators, and with one k split SwiGLU is applied to the finished sums here
// (swiglu_bits, as the second kernel applies it to the sums of one split).
// TM: activation rows of a tile, 256 or 128 (row counts up to 128: four waves along the weight rows instead of two, a
// wave's part 64 x 32).
template <WKind KIND, bool PAIR, uint32_t TM>
__global__ __launch_bounds__(kTileBlock) void qgemm_tile_kernel(const QgemmArgs a) {
    extern __shared__ uint4 lds_raw[];
    constexpr uint32_t kTileBufPieces = tile_buf_pieces(PAIR, TM);
    constexpr uint32_t WM = TM / 64u, WN = 8u / WM;   // waves along the activation rows / along the weight rows
    constexpr uint32_t WCOLS = kTileN / WN;           // weight rows of a wave's part: 64 or 32
    constexpr int NJ = (int)(WCOLS / 32u);            // 32-wide accumulator tiles along them
    constexpr int XP = (int)(TM / 64u);               // x pieces per thread and slab

    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6, kb = lane >> 5, nl = lane & 31u;
    const uint32_t wm = wave / WN, wn = wave % WN;   // the wave's part: rows 64 wm, weight rows WCOLS wn
    uint32_t nb = blockIdx.x % a.n_blocks;
    const uint32_t ks = blockIdx.x / a.n_blocks;
    // the matrix this block works on (one, or the fan-out's matrix whose range of blocks holds nb)
    const uint4* w_mat = a.w;
    const uint16_t *sc_mat = a.sc, *bi_mat = a.bi, *bias_mat = a.bias;
    uint16_t* y_mat = a.y;
    uint32_t N = a.N, col0 = 0, row_cols = a.N;   // row_cols: columns of a row of partial sums
    if (!PAIR && a.n_seg > 1u) {
        const uint32_t si = nb >= a.seg[0].nb_end ? (nb >= a.seg[1].nb_end ? 2u : 1u) : 0u;
        nb -= si ? a.seg[si - 1u].nb_end : 0u;
        w_mat = a.seg[si].w;
        sc_mat = a.seg[si].sc;
        bi_mat = a.seg[si].bi;
        bias_mat = a.seg[si].bias;
        y_mat = a.seg[si].y;
        N = a.seg[si].N;
        col0 = a.seg[si].col0;
        row_cols = a.n_total;
    }
    const uint32_t m0 = blockIdx.y * TM, n0 = nb * kTileN;
    const uint32_t k0 = ks * a.k_per_split;
    const uint32_t k1 = k0 + a.k_per_split < a.K ? k0 + a.k_per_split : a.K;
    const uint32_t gshift = a.group == 128 ? 7u : 6u;
    const uint32_t slabs = (k1 - k0) / kTileK;

    // staging roles: x pieces (row tid / 8 + 64 i, piece tid % 8), i < 4; 16 codes of weight row tid / 4, quarter
    // tid % 4 of the slab (8 bytes of int4, 16 of int8)
    const uint32_t xr = tid >> 3, xp = tid & 7u;
    const uint32_t wr = tid >> 2, wq = tid & 3u;
    const uint32_t wrow = n0 + wr < N ? n0 + wr : N - 1;   // rows past the end read the last row; never stored
    // Every request is a block-uniform base (scalar registers, advanced by the slab) plus a per-lane 32-bit byte offset
    // that never changes: no vector address arithmetic per slab (the planner admits the form only while the operands
    // stay under 4 GB).
    const unsigned char* wbase = reinterpret_cast<const unsigned char*>(w_mat);
    const unsigned char* xbase = reinterpret_cast<const unsigned char*>(a.x);
    const unsigned char* sbase = reinterpret_cast<const unsigned char*>(sc_mat);
    const unsigned char* bbase = reinterpret_cast<const unsigned char*>(bi_mat);
    const unsigned char* w2base = reinterpret_cast<const unsigned char*>(a.w2);
    const unsigned char* s2base = reinterpret_cast<const unsigned char*>(a.sc2);
    const unsigned char* b2base = reinterpret_cast<const unsigned char*>(a.bi2);
    const uint32_t woff = wrow * a.cpr * 16u + wq * (KIND == W_Q4 ? 8u : 16u);
    const uint32_t soff = wrow * a.gpr * 2u;
    uint32_t xoff[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const uint32_t m = m0 + xr + 64u * (uint32_t)(i < XP ? i : 0);   // (TM = 128: two pieces per thread; 2, 3 unused)
        xoff[i] = (m < a.M ? m : a.M - 1) * a.K * 2u + xp * 16u;
    }

    f32x16_t acc[2][NJ], acc2[PAIR ? 2 : 1][PAIR ? NJ : 1];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < NJ; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                acc[i][j][r] = 0.f;
                if constexpr (PAIR) acc2[i][j][r] = 0.f;
            }

    // (Macros over named registers, not lambdas over a struct or arrays: an object whose address a closure holds, or an
    // array, stays in scratch once a fence stands between its writes and its reads.)
#define FK_TILE_DECLARE(S) uint4 S##x0, S##x1, S##x2, S##x3, S##w, S##v; uint16_t S##sc, S##bi, S##sc2, S##bi2
#define FK_TILE_REQUEST(S, slab)                                                                                      \
    {                                                                                                                 \
        const uint32_t kf = k0 + ((slab) < slabs ? (slab) : 0u) * kTileK; /* past the end: the first slab (unused) */ \
        const unsigned char* xk = xbase + (size_t)kf * 2u;                                                           \
        S##x0 = *reinterpret_cast<const uint4*>(xk + xoff[0]);                                                        \
        S##x1 = *reinterpret_cast<const uint4*>(xk + xoff[1]);                                                        \
        if constexpr (XP == 4) {                                                                                      \
            S##x2 = *reinterpret_cast<const uint4*>(xk + xoff[2]);                                                    \
            S##x3 = *reinterpret_cast<const uint4*>(xk + xoff[3]);                                                    \
        }                                                                                                             \
        if constexpr (KIND == W_Q4) {                                                                                 \
            const uint2 v = *reinterpret_cast<const uint2*>(wbase + (kf >> 1) + woff);                                \
            S##w = make_uint4(v.x, v.y, 0u, 0u);                                                                      \
        } else {                                                                                                      \
            S##w = *reinterpret_cast<const uint4*>(wbase + kf + woff);                                                \
        }                                                                                                             \
        const uint32_t g = kf >> gshift;                                                                              \
        S##sc = *reinterpret_cast<const uint16_t*>(sbase + g * 2u + soff); /* kept apart: combining the two here */   \
        S##bi = *reinterpret_cast<const uint16_t*>(bbase + g * 2u + soff); /* would wait for both loads on the spot */ \
        if constexpr (PAIR) {                                                                                         \
            if constexpr (KIND == W_Q4) {                                                                             \
                const uint2 v = *reinterpret_cast<const uint2*>(w2base + (kf >> 1) + woff);                           \
                S##v = make_uint4(v.x, v.y, 0u, 0u);                                                                  \
            } else {                                                                                                  \
                S##v = *reinterpret_cast<const uint4*>(w2base + kf + woff);                                           \
            }                                                                                                         \
            S##sc2 = *reinterpret_cast<const uint16_t*>(s2base + g * 2u + soff);                                      \
            S##bi2 = *reinterpret_cast<const uint16_t*>(b2base + g * 2u + soff);                                      \
        }                                                                                                             \
        /* keeps the requests where they are written: left alone, the compiler moves them down to their first use */  \
        asm volatile("" ::: "memory");                                                                                \
    }
#define FK_TILE_STAGE(S, to)                                                                                          \
    {                                                                                                                 \
        uint4* xs_w = lds_raw + (to) * kTileBufPieces;                                                                \
        uint4* xd = xs_w + xr * kTileStride + xp;                                                                     \
        xd[0 * 64 * kTileStride] = S##x0; xd[1 * 64 * kTileStride] = S##x1;                                           \
        if constexpr (XP == 4) { xd[2 * 64 * kTileStride] = S##x2; xd[3 * 64 * kTileStride] = S##x3; }                \
        /* pinned here: left alone, the compiler widens the two values where they are loaded, a pass earlier, and   \
           waits there for every request in flight */                                                                 \
        uint32_t sc_bits = S##sc, bi_bits = S##bi;                                                                    \
        asm volatile("" : "+v"(sc_bits), "+v"(bi_bits));                                                              \
        const float sf = bf16_bits_to_f32(sc_bits), bf = bf16_bits_to_f32(bi_bits);                                   \
        uint4* wd = xs_w + TM * kTileStride + wr * kTileStride + wq * 2u;                                             \
        wd[0] = tile_unpack_piece<KIND>(0, S##w, sf, bf);                                                             \
        wd[1] = tile_unpack_piece<KIND>(1, S##w, sf, bf);                                                             \
        if constexpr (PAIR) {                                                                                         \
            uint32_t sc2_bits = S##sc2, bi2_bits = S##bi2;                                                            \
            asm volatile("" : "+v"(sc2_bits), "+v"(bi2_bits));                                                        \
            const float sf2 = bf16_bits_to_f32(sc2_bits), bf2 = bf16_bits_to_f32(bi2_bits);                           \
            wd[kTileN * kTileStride] = tile_unpack_piece<KIND>(0, S##v, sf2, bf2);                                    \
            wd[kTileN * kTileStride + 1] = tile_unpack_piece<KIND>(1, S##v, sf2, bf2);                                \
        }                                                                                                             \
    }
    auto multiply = [&](uint32_t from) {
        const uint4* xs = lds_raw + from * kTileBufPieces;
        const uint4* xa = xs + (wm * 64u + nl) * kTileStride + kb;
        const uint4* wb = xs + (TM + wn * WCOLS + nl) * kTileStride + kb;
#pragma unroll
        for (int st = 0; st < (int)kTileK / 16; ++st) {
            uint4 af[2], bfr[NJ];
#pragma unroll
            for (int i = 0; i < 2; ++i) af[i] = xa[(uint32_t)i * 32u * kTileStride + 2u * (uint32_t)st];
#pragma unroll
            for (int j = 0; j < NJ; ++j) bfr[j] = wb[(uint32_t)j * 32u * kTileStride + 2u * (uint32_t)st];
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int j = 0; j < NJ; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, af[i]),
                                                                        __builtin_bit_cast(bf16x8_t, bfr[j]), acc[i][j], 0, 0, 0);
            if constexpr (PAIR) {
                uint4 bf2[NJ];
#pragma unroll
                for (int j = 0; j < NJ; ++j) bf2[j] = wb[((uint32_t)j * 32u + kTileN) * kTileStride + 2u * (uint32_t)st];
#pragma unroll
                for (int i = 0; i < 2; ++i)
#pragma unroll
                    for (int j = 0; j < NJ; ++j)
                        acc2[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, af[i]),
                                                                             __builtin_bit_cast(bf16x8_t, bf2[j]), acc2[i][j], 0, 0, 0);
                // (a step's fragment reads stay behind the step before: requested all at once, the four steps' 24
                // fragments push the pair form's 128 accumulator registers into scratch)
                asm volatile("" ::: "memory");
            }
        }
    };
    FK_TILE_DECLARE(e_);
    FK_TILE_DECLARE(o_);
    // slab s parks in the set of its parity; pass q stages slab q, requests slab q + 2 into the set it has just emptied
    // and multiplies slab q - 1
    FK_TILE_REQUEST(e_, 0u);
    FK_TILE_REQUEST(o_, 1u);
    FK_TILE_STAGE(e_, 0u);
    FK_TILE_REQUEST(e_, 2u);
    __syncthreads();
    uint32_t buf = 0;   // a pass multiplies from `buf` and stages into the other one
    uint32_t q = 1;
    for (; q + 1 <= slabs; q += 2) {
        FK_TILE_STAGE(o_, buf ^ 1u);
        FK_TILE_REQUEST(o_, q + 2u);
        multiply(buf);
        __syncthreads();
        buf ^= 1u;
        FK_TILE_STAGE(e_, buf ^ 1u);
        FK_TILE_REQUEST(e_, q + 3u);
        multiply(buf);
        __syncthreads();
        buf ^= 1u;
    }
    // the last slab of an odd count (the pair form is only planned for even counts: a conditional multiply behind the
    // loop sends its 128 accumulator registers through scratch)
    if constexpr (!PAIR)
        if (q <= slabs) multiply(buf);
#undef FK_TILE_DECLARE
#undef FK_TILE_REQUEST
#undef FK_TILE_STAGE

    // register r of a lane is activation row (r % 4) + 8 (r / 4) + 4 kb of its 32 x 32 tile, column nl
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
        const uint32_t n = n0 + wn * WCOLS + (uint32_t)j * 32u + nl;
        if (n >= N) continue;
        const float bias = (y_mat && bias_mat) ? bf16_bits_to_f32(bias_mat[n]) : 0.f;
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const uint32_t m = m0 + wm * 64u + (uint32_t)(i * 32 + r % 4 + 8 * (r / 4)) + 4u * kb;
                if (m >= a.M) continue;
                if constexpr (PAIR) {
                    if (a.y) {   // one k split: SwiGLU of the two finished sums, as the second kernel forms it
                        a.y[(size_t)m * a.N + n] = (uint16_t)swiglu_bits(acc[i][j][r], acc2[i][j][r], a.variant, 1.0f);
                    } else {
                        a.partial[((size_t)ks * a.M + m) * a.N + n] = acc[i][j][r];
                        a.partial2[((size_t)ks * a.M + m) * a.N + n] = acc2[i][j][r];
                    }
                } else if (y_mat) {   // one k split: finished here, in the order of additions of the second kernel
                    float v = acc[i][j][r];
                    if (bias_mat) v += bias;
                    if (a.res) v += bf16_bits_to_f32(a.res[(size_t)m * N + n]);
                    y_mat[(size_t)m * N + n] = (uint16_t)f32_to_bf16_bits(v);
                } else {
                    a.partial[((size_t)ks * a.M + m) * row_cols + col0 + n] = acc[i][j][r];
                }
            }
    }
}

struct QgemmReduceArgs {
    const float* p0;  // [ksplit, M, N]
    const float* p1;  // second matrix (up projection) for the SwiGLU pair, or null
    const uint16_t* bias;
    const uint16_t* res;
    uint16_t* y;
    uint32_t M, N, ksplit;
    int variant;
};

// Four consecutive outputs per thread (N a multiple of 4: 16-byte loads of the sums, one 8-byte
// store); same order of additions per element as the scalar form below.
__global__ __launch_bounds__(256) void qgemm_reduce4_kernel(const QgemmReduceArgs a) {
    const uint32_t total = a.M * a.N, i = (blockIdx.x * 256u + threadIdx.x) * 4u;
    if (i >= total) return;
    float s0[4] = {0.f, 0.f, 0.f, 0.f}, s1[4] = {0.f, 0.f, 0.f, 0.f};
    for (uint32_t ks = 0; ks < a.ksplit; ++ks) {
        const float4 v = *reinterpret_cast<const float4*>(a.p0 + (size_t)ks * total + i);
        s0[0] += v.x; s0[1] += v.y; s0[2] += v.z; s0[3] += v.w;
        if (a.p1) {
            const float4 u = *reinterpret_cast<const float4*>(a.p1 + (size_t)ks * total + i);
            s1[0] += u.x; s1[1] += u.y; s1[2] += u.z; s1[3] += u.w;
        }
    }
    uint32_t o[4];
    if (a.p1) {
#pragma unroll
        for (int e = 0; e < 4; ++e) o[e] = swiglu_bits(s0[e], s1[e], a.variant, 1.0f);
    } else {
        const uint32_t n = i % a.N;  // i and N are multiples of 4: the four share a row
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            float v = s0[e];
            if (a.bias) v += bf16_bits_to_f32(a.bias[n + e]);
            if (a.res) v += bf16_bits_to_f32(a.res[i + e]);
            o[e] = f32_to_bf16_bits(v);
        }
    }
    *reinterpret_cast<uint2*>(a.y + i) = make_uint2(o[0] | (o[1] << 16), o[2] | (o[3] << 16));
}

__global__ __launch_bounds__(256) void qgemm_reduce_kernel(const QgemmReduceArgs a) {
    const uint32_t i = blockIdx.x * 256u + threadIdx.x, total = a.M * a.N;
    if (i >= total) return;
    float s0 = 0.f, s1 = 0.f;
    for (uint32_t ks = 0; ks < a.ksplit; ++ks) {
        s0 += a.p0[(size_t)ks * total + i];
        if (a.p1) s1 += a.p1[(size_t)ks * total + i];
    }
    if (a.p1) {
        a.y[i] = (uint16_t)swiglu_bits(s0, s1, a.variant, 1.0f);
        return;
    }
    if (a.bias) s0 += bf16_bits_to_f32(a.bias[i % a.N]);
    if (a.res) s0 += bf16_bits_to_f32(a.res[i]);
    a.y[i] = (uint16_t)f32_to_bf16_bits(s0);
}

// Split-k sums of a fan-out (rows of n_total columns, the matrices side by side) to the matrices' own outputs; four
// consecutive columns per thread (every matrix's N is a multiple of 4), additions in split order, then the bias.
struct QgemmFanReduceArgs {
    const float* p;
    uint32_t M, n_total, ksplit, n_seg;
    uint16_t* y[3];
    const uint16_t* bias[3];
    uint32_t col0[3], N[3];
};
__global__ __launch_bounds__(256) void qgemm_fan_reduce_kernel(const QgemmFanReduceArgs a) {
    const uint32_t total = a.M * a.n_total, i = (blockIdx.x * 256u + threadIdx.x) * 4u;
    if (i >= total) return;
    float s[4] = {0.f, 0.f, 0.f, 0.f};
    for (uint32_t ks = 0; ks < a.ksplit; ++ks) {
        const float4 v = *reinterpret_cast<const float4*>(a.p + (size_t)ks * total + i);
        s[0] += v.x; s[1] += v.y; s[2] += v.z; s[3] += v.w;
    }
    const uint32_t m = i / a.n_total, c = i - m * a.n_total;
    const uint32_t si = (a.n_seg > 2u && c >= a.col0[2]) ? 2u : ((a.n_seg > 1u && c >= a.col0[1]) ? 1u : 0u);
    const uint32_t n = c - a.col0[si];
    uint32_t o[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        float v = s[e];
        if (a.bias[si]) v += bf16_bits_to_f32(a.bias[si][n + e]);
        o[e] = f32_to_bf16_bits(v);
    }
    *reinterpret_cast<uint2*>(a.y[si] + (size_t)m * a.N[si] + n) = make_uint2(o[0] | (o[1] << 16), o[2] | (o[3] << 16));
}

namespace {

// forms 8 .. 11: the tile form (9, 11: a gate / up pair; 10, 11: tiles of 128 activation rows)
uint32_t qgemm_form_lds_bytes(int mt) { return mt >= 8 ? tile_lds_bytes(mt & 1, mt >= 10 ? 128u : 256u) : qgemm_lds_bytes(mt); }

struct QgemmShape {
    uint32_t n_blocks, m_tiles, ksplit, k_per_split;
    int mt;           // tiles of 32 activation rows per block; 8: the tile form
    uint32_t tile_m;  // the tile form's activation rows per tile: 256 or 128
    int form(bool pair) const { return mt == 8 ? 8 + (pair ? 1 : 0) + (tile_m == 128u ? 2 : 0) : mt; }
};

const void* qgemm_func(uint32_t bits, int mt) {
    const bool q4 = bits == 4;
    switch (mt) {
        case 8: return q4 ? reinterpret_cast<const void*>(&qgemm_tile_kernel<W_Q4, false, 256>) : reinterpret_cast<const void*>(&qgemm_tile_kernel<W_Q8, false, 256>);
        case 9: return q4 ? reinterpret_cast<const void*>(&qgemm_tile_kernel<W_Q4, true, 256>) : reinterpret_cast<const void*>(&qgemm_tile_kernel<W_Q8, true, 256>);   // a gate / up pair
        case 10: return q4 ? reinterpret_cast<const void*>(&qgemm_tile_kernel<W_Q4, false, 128>) : reinterpret_cast<const void*>(&qgemm_tile_kernel<W_Q8, false, 128>);   // tiles of 128 rows
        case 11: return q4 ? reinterpret_cast<const void*>(&qgemm_tile_kernel<W_Q4, true, 128>) : reinterpret_cast<const void*>(&qgemm_tile_kernel<W_Q8, true, 128>);
        case 1: return q4 ? reinterpret_cast<const void*>(&qgemm_kernel<W_Q4, 1>) : reinterpret_cast<const void*>(&qgemm_kernel<W_Q8, 1>);
        case 2: return q4 ? reinterpret_cast<const void*>(&qgemm_kernel<W_Q4, 2>) : reinterpret_cast<const void*>(&qgemm_kernel<W_Q8, 2>);
        default: return q4 ? reinterpret_cast<const void*>(&qgemm_kernel<W_Q4, 4>) : reinterpret_cast<const void*>(&qgemm_kernel<W_Q8, 4>);
    }
}

// Blocks of this kernel form that are resident at once (registers and LDS decide).
uint32_t qgemm_resident(const DeviceFacts* dev, uint32_t bits, int mt) {
    static std::mutex mu;
    static int cache[2][12] = {};
    std::lock_guard<std::mutex> lk(mu);
    int& slot = cache[bits == 4 ? 0 : 1][mt];
    if (slot == 0) {
        const void* f = qgemm_func(bits, mt);
        const uint32_t lds = qgemm_form_lds_bytes(mt);
        if (lds > 48 * 1024) (void)hipFuncSetAttribute(f, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        int per_cu = 0;
        if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, f, mt == 8 ? kTileBlock : kQgemmBlock, lds) != hipSuccess || per_cu < 1) per_cu = 1;
        if (mt == 8) per_cu = 1;         // the tile form: one block (two LDS buffers, 128 accumulator registers per lane) per CU
        slot = per_cu > 2 ? 2 : per_cu;  // more than two blocks per CU gain nothing here (512 rows: 66.4 us with 2, 65.9 with 4)
    }
    return (uint32_t)slot * (uint32_t)dev->cus;
}

fk_status qgemm_shape(const DeviceFacts* dev, uint32_t M, uint32_t N, uint32_t K, uint32_t group, uint32_t bits,
                      QgemmShape* out) {
    if (M == 0 || N == 0 || K == 0) return set_error(FK_ERR_INVALID, "qgemm: empty shape");
    if (group != 64 && group != 128) return set_error(FK_ERR_UNSUPPORTED, "qgemm: group size must be 64 or 128");
    if (K % group) return set_error(FK_ERR_UNSUPPORTED, "qgemm: K must be a multiple of the group size");
    if ((uint64_t)M * N > 0x7fffffffull) return set_error(FK_ERR_UNSUPPORTED, "qgemm: output too large");
    QgemmShape s;
    s.n_blocks = (N + kQgemmRows - 1) / kQgemmRows;
    // 8: the tile form (its requests are 32-bit byte offsets from a uniform base: operands under 4 GB)
    const bool tile_ok = M >= kTileMinRows && (uint64_t)M * K * 2 < (1ull << 32) && (uint64_t)N * K < (1ull << 32);
    s.mt = tile_ok ? 8 : (M > 64 ? 4 : (M > 32 ? 2 : 1));
    s.tile_m = M <= 128u ? 128u : kTileM;   // up to 128 rows: tiles of 128 rows (a 256-row tile would be half empty)
    s.m_tiles = s.mt == 8 ? (M + s.tile_m - 1) / s.tile_m : (M + kQgemmMTile * s.mt - 1) / (kQgemmMTile * s.mt);
    if (s.mt == 8) s.n_blocks = (N + kTileN - 1) / kTileN;
    // Split k until the grid fills what is resident at once, never beyond (a block that waits
    // for a slot doubles the run time), and keep at least 256 k per block.  Every split writes
    // and re-reads an fp32 copy of the output.
    const uint32_t blocks = s.n_blocks * s.m_tiles;
    const uint32_t target = qgemm_resident(dev, bits, s.mt);
    const uint32_t want = target / blocks;
    uint32_t max_split = K / 256u;
    if (max_split < 1) max_split = 1;
    uint32_t split = want < 1 ? 1 : (want > max_split ? max_split : want);
    const uint32_t groups = K / group;
    s.k_per_split = (groups + split - 1) / split * group;
    s.ksplit = (K + s.k_per_split - 1) / s.k_per_split;
    if (s.m_tiles > 65535) return set_error(FK_ERR_UNSUPPORTED, "qgemm: too many activation rows");
    *out = s;
    return FK_OK;
}

fk_status check_weight(const fk_weight* W, const char* who) {
    if (!W || !W->w || !W->scales || !W->biases) return set_error(FK_ERR_INVALID, std::string(who) + ": null weight");
    if (W->bits != 4 && W->bits != 8)
        return set_error(FK_ERR_UNSUPPORTED, std::string(who) + ": quantised weights (4 or 8 bits) only");
    return FK_OK;
}

// `direct` (optional): where a launch that needs no second kernel -- the tile form with one k split -- writes its
// finished outputs; *finished then says whether it does.
struct QgemmDirect {
    uint16_t* y;
    const uint16_t* bias;
    const uint16_t* res;
};
fk_status plan_qgemm_main(const DeviceFacts* dev, const fk_weight* W, const uint16_t* x, uint32_t M, float* partial,
                          QgemmShape* shape, Launch* out, const QgemmDirect* direct = nullptr, bool* finished = nullptr) {
    FK_TRY(qgemm_shape(dev, M, W->n, W->k, W->group, W->bits, shape));
    if (finished) *finished = false;
    QgemmArgs a;
    memset(&a, 0, sizeof(a));
    a.w = reinterpret_cast<const uint4*>(W->w);
    a.sc = W->scales;
    a.bi = W->biases;
    a.x = x;
    a.partial = partial;
    a.M = M;
    a.N = W->n;
    a.K = W->k;
    a.cpr = W->k / (W->bits == 4 ? 32u : 16u);
    a.gpr = W->k / W->group;
    a.group = W->group;
    a.k_per_split = shape->k_per_split;
    a.n_blocks = shape->n_blocks;
    if (direct && shape->mt == 8 && shape->ksplit == 1) {
        a.y = direct->y;
        a.bias = direct->bias;
        a.res = direct->res;
        if (finished) *finished = true;
    }
    out->func = qgemm_func(W->bits, shape->form(false));
    out->grid = dim3(shape->n_blocks * shape->ksplit, shape->m_tiles, 1);
    out->block = dim3(shape->mt == 8 ? kTileBlock : kQgemmBlock, 1, 1);
    out->shmem = qgemm_form_lds_bytes(shape->form(false));
    out->set_args(a);
    if (out->shmem > 48 * 1024)
        FK_HIP(hipFuncSetAttribute(out->func, hipFuncAttributeMaxDynamicSharedMemorySize, (int)out->shmem));
    return FK_OK;
}

void plan_reduce(const float* p0, const float* p1, const uint16_t* bias, const uint16_t* res, uint16_t* y, uint32_t M,
                 uint32_t N, uint32_t ksplit, int variant, Launch* out) {
    QgemmReduceArgs r;
    r.p0 = p0; r.p1 = p1; r.bias = bias; r.res = res; r.y = y;
    r.M = M; r.N = N; r.ksplit = ksplit; r.variant = variant;
    const bool by4 = N % 4u == 0 && ((reinterpret_cast<uintptr_t>(p0) | reinterpret_cast<uintptr_t>(p1)) & 15u) == 0 &&
                     (reinterpret_cast<uintptr_t>(y) & 7u) == 0;
    out->func = by4 ? reinterpret_cast<const void*>(&qgemm_reduce4_kernel) : reinterpret_cast<const void*>(&qgemm_reduce_kernel);
    out->grid = dim3(by4 ? (M * N / 4u + 255u) / 256u : (M * N + 255u) / 256u, 1, 1);
    out->block = dim3(256, 1, 1);
    out->shmem = 0;
    out->set_args(r);
}

}  // namespace

// the epilogue of a product whose fp32 sums are complete (the library route)
void plan_qgemm_epilogue(const float* p0, const float* p1, const uint16_t* bias, const uint16_t* res, uint16_t* y,
                         uint32_t M, uint32_t N, uint32_t ksplit, int variant, Launch* out) {
    plan_reduce(p0, p1, bias, res, y, M, N, ksplit, variant, out);
}

fk_status qgemm_workspace_bytes(uint32_t M, uint32_t N, uint32_t K, uint32_t group, size_t* bytes) {
    const DeviceFacts* dev;
    FK_TRY(device_facts(&dev));
    if (group == 0) {  // dense bf16 weights: the library route's fp32 sums only
        if (M == 0 || N == 0 || K == 0) return set_error(FK_ERR_INVALID, "qgemm: empty shape");
        *bytes = qgemm_library_sums_bytes(M, N, K);
        return FK_OK;
    }
    // the split depends on the kernel form (4- or 8-bit codes): size for the larger of the two
    QgemmShape s4, s8;
    FK_TRY(qgemm_shape(dev, M, N, K, group, 4, &s4));
    FK_TRY(qgemm_shape(dev, M, N, K, group, 8, &s8));
    *bytes = (size_t)(s4.ksplit > s8.ksplit ? s4.ksplit : s8.ksplit) * M * N * sizeof(float);
    // direct calls with many rows may take the library route, which also parks the dequantised matrix
    // here; dense bf16 weights always take it and need the fp32 sums only
    const size_t lib = qgemm_takes_library(M) ? qgemm_library_workspace_bytes(M, N, K) : qgemm_library_sums_bytes(M, N, K);
    if (lib > *bytes) *bytes = lib;
    return FK_OK;
}

fk_status plan_qgemm(const fk_weight* W, const uint16_t* x, uint32_t M, const uint16_t* bias, const uint16_t* res,
                     uint16_t* y, void* workspace, Launch* main, Launch* reduce) {
    const DeviceFacts* dev;
    FK_TRY(device_facts(&dev));
    FK_TRY(check_weight(W, "qgemm"));
    if (!x || !y || !workspace) return set_error(FK_ERR_INVALID, "qgemm: null activation, output or workspace");
    if (qgemm_takes_wide(M, W->group)) {  // 2..10 rows: one launch, no split-k sums (reduce stays empty)
        *reduce = Launch();
        return plan_qgemm_wide(W, nullptr, x, M, bias, res, 0, y, main);
    }
    QgemmShape s;
    const QgemmDirect direct{y, bias, res};
    bool finished = false;
    FK_TRY(plan_qgemm_main(dev, W, x, M, static_cast<float*>(workspace), &s, main, &direct, &finished));
    if (finished)
        *reduce = Launch();   // the tile form with one k split rounds its outputs itself
    else
        plan_reduce(static_cast<float*>(workspace), nullptr, bias, res, y, M, W->n, s.ksplit, 0, reduce);
    return FK_OK;
}

// Up to three matrices over the same activation rows (same K, bits and group size; every N a multiple of 4) as ONE
// launch of the tile form whose blocks along N run through the matrices in turn, finished by one second kernel when k
// is split.  *fused = false (and nothing planned) when the tile form does not apply: the caller runs the matrices one
// by one.
fk_status plan_qgemm_fanout(const fk_weight* const* W, uint32_t n_mats, const uint16_t* x, uint32_t M,
                            const uint16_t* const* bias, uint16_t* const* y, void* workspace, Launch* main, Launch* reduce,
                            bool* fused) {
    const DeviceFacts* dev;
    FK_TRY(device_facts(&dev));
    *fused = false;
    if (n_mats < 2 || n_mats > 3 || !W || !y) return set_error(FK_ERR_INVALID, "qgemm fan-out: two or three matrices");
    if (!x || !workspace) return set_error(FK_ERR_INVALID, "qgemm fan-out: null activation or workspace");
    uint32_t n_total = 0, blocks_n = 0;
    for (uint32_t i = 0; i < n_mats; ++i) {
        FK_TRY(check_weight(W[i], "qgemm fan-out"));
        if (!y[i]) return set_error(FK_ERR_INVALID, "qgemm fan-out: null output");
        if (W[i]->k != W[0]->k || W[i]->bits != W[0]->bits || W[i]->group != W[0]->group)
            return set_error(FK_ERR_INVALID, "qgemm fan-out: the matrices need the same K, bits and group size");
        if (W[i]->n % 4u) return FK_OK;
        n_total += W[i]->n;
        blocks_n += (W[i]->n + kTileN - 1) / kTileN;
    }
    QgemmShape s;
    FK_TRY(qgemm_shape(dev, M, blocks_n * kTileN, W[0]->k, W[0]->group, W[0]->bits, &s));
    if (s.mt != 8 || (uint64_t)M * n_total > 0x7fffffffull) return FK_OK;
    for (uint32_t i = 0; i < n_mats; ++i)
        if ((uint64_t)W[i]->n * W[i]->k >= (1ull << 32)) return FK_OK;
    QgemmArgs a;
    memset(&a, 0, sizeof(a));
    a.x = x;
    a.partial = static_cast<float*>(workspace);
    a.M = M;
    a.N = W[0]->n;
    a.K = W[0]->k;
    a.cpr = W[0]->k / (W[0]->bits == 4 ? 32u : 16u);
    a.gpr = W[0]->k / W[0]->group;
    a.group = W[0]->group;
    a.k_per_split = s.k_per_split;
    a.n_blocks = blocks_n;
    a.n_seg = n_mats;
    a.n_total = n_total;
    QgemmFanReduceArgs r;
    memset(&r, 0, sizeof(r));
    uint32_t nb = 0, col = 0;
    for (uint32_t i = 0; i < 3; ++i) {
        const uint32_t j = i < n_mats ? i : n_mats - 1;   // unused entries repeat the last matrix (never selected)
        if (i < n_mats) nb += (W[i]->n + kTileN - 1) / kTileN;
        a.seg[i].w = reinterpret_cast<const uint4*>(W[j]->w);
        a.seg[i].sc = W[j]->scales;
        a.seg[i].bi = W[j]->biases;
        a.seg[i].y = s.ksplit == 1 ? y[j] : nullptr;
        a.seg[i].bias = bias ? bias[j] : nullptr;
        a.seg[i].N = W[j]->n;
        a.seg[i].nb_end = i < n_mats ? nb : 0xffffffffu;
        a.seg[i].col0 = i < n_mats ? col : 0u;
        r.y[i] = y[j];
        r.bias[i] = bias ? bias[j] : nullptr;
        r.col0[i] = i < n_mats ? col : 0xffffffffu;
        r.N[i] = W[j]->n;
        if (i < n_mats) col += W[i]->n;
    }
    a.w = a.seg[0].w;
    a.sc = a.seg[0].sc;
    a.bi = a.seg[0].bi;
    main->func = qgemm_func(W[0]->bits, s.form(false));
    main->grid = dim3(blocks_n * s.ksplit, s.m_tiles, 1);
    main->block = dim3(kTileBlock, 1, 1);
    main->shmem = qgemm_form_lds_bytes(s.form(false));
    main->set_args(a);
    FK_HIP(hipFuncSetAttribute(main->func, hipFuncAttributeMaxDynamicSharedMemorySize, (int)main->shmem));
    *reduce = Launch();
    if (s.ksplit > 1) {
        r.p = a.partial;
        r.M = M;
        r.n_total = n_total;
        r.ksplit = s.ksplit;
        r.n_seg = n_mats;
        reduce->func = reinterpret_cast<const void*>(&qgemm_fan_reduce_kernel);
        reduce->grid = dim3((M * n_total / 4u + 255u) / 256u, 1, 1);
        reduce->block = dim3(256, 1, 1);
        reduce->shmem = 0;
        reduce->set_args(r);
    }
    *fused = true;
    return FK_OK;
}

fk_status plan_qgemm_swiglu(const fk_weight* Wg, const fk_weight* Wu, const uint16_t* x, uint32_t M, int variant,
                            uint16_t* out, void* workspace, Launch* gate, Launch* up, Launch* reduce) {
    const DeviceFacts* dev;
    FK_TRY(device_facts(&dev));
    FK_TRY(check_weight(Wg, "qgemm_swiglu"));
    FK_TRY(check_weight(Wu, "qgemm_swiglu"));
    if (Wg->n != Wu->n || Wg->k != Wu->k || Wg->group != Wu->group)
        return set_error(FK_ERR_INVALID, "qgemm_swiglu: gate and up need the same shape and group size");
    if (variant < 0 || variant > 2) return set_error(FK_ERR_INVALID, "qgemm_swiglu: variant must be 0, 1 or 2");
    if (!x || !out || !workspace) return set_error(FK_ERR_INVALID, "qgemm_swiglu: null activation, output or workspace");
    if (qgemm_takes_wide(M, Wg->group)) {  // 2..10 rows: gate, up and SwiGLU in one launch (up, reduce stay empty)
        *up = Launch();
        *reduce = Launch();
        return plan_qgemm_wide(Wg, Wu, x, M, nullptr, nullptr, variant, out, gate);
    }
    QgemmShape s;
    float* p0 = static_cast<float*>(workspace);
    FK_TRY(plan_qgemm_main(dev, Wg, x, M, p0, &s, gate));
    float* p1 = p0 + (size_t)s.ksplit * M * Wg->n;
    if (s.mt == 8 && Wg->bits == Wu->bits && Wg->k % 128u == 0 && s.k_per_split % 128u == 0) {   // (even slab counts)
        // the tile form takes the pair in ONE launch (activations staged once, two sets of accumulators); with one k
        // split it applies SwiGLU itself
        QgemmArgs a;
        memcpy(&a, gate->args, sizeof(a));
        a.w2 = reinterpret_cast<const uint4*>(Wu->w);
        a.sc2 = Wu->scales;
        a.bi2 = Wu->biases;
        a.partial2 = p1;
        a.variant = variant;
        a.y = s.ksplit == 1 ? out : nullptr;
        a.bias = a.res = nullptr;
        gate->func = qgemm_func(Wg->bits, s.form(true));
        gate->shmem = qgemm_form_lds_bytes(s.form(true));
        gate->set_args(a);
        FK_HIP(hipFuncSetAttribute(gate->func, hipFuncAttributeMaxDynamicSharedMemorySize, (int)gate->shmem));
        *up = Launch();
        if (s.ksplit == 1)
            *reduce = Launch();
        else
            plan_reduce(p0, p1, nullptr, nullptr, out, M, Wg->n, s.ksplit, variant, reduce);
        return FK_OK;
    }
    FK_TRY(plan_qgemm_main(dev, Wu, x, M, p1, &s, up));
    plan_reduce(p0, p1, nullptr, nullptr, out, M, Wg->n, s.ksplit, variant, reduce);
    return FK_OK;
}

}  // namespace fk
