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
// A block is 4 waves = 128 weight rows over one k range and one tile of 32
// activation rows; x is staged per 512-k slab into LDS in the lane order the MFMA
// wants (and, for int4, in the nibble pairing of the unpack).  The k dimension is
// split over blocks until the grid fills the chip; partial sums go to an fp32
// workspace and a second kernel adds them in split order and applies the epilogue,
// so the result does not depend on block scheduling.
#include "fk_host.hpp"
#include "gemv_kernel.hpp"

namespace fk {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x16_t __attribute__((ext_vector_type(16)));

constexpr int kQgemmBlock = 256;
constexpr uint32_t kQgemmRows = 128;   // weight rows per block
constexpr uint32_t kQgemmMTile = 32;   // activation rows per block
constexpr uint32_t kQgemmSlabK = 512;  // k staged per LDS slab
constexpr uint32_t kQgemmXStride = kQgemmSlabK / 8 + 1;  // uint4 per staged row (+1: bank spread)

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
};

constexpr uint32_t kQgemmLdsBytes = kQgemmMTile * kQgemmXStride * 16u + (kQgemmSlabK / 64u) * kQgemmMTile * 4u;

template <WKind KIND>
__global__ __launch_bounds__(kQgemmBlock) void qgemm_kernel(const QgemmArgs a) {
    constexpr uint32_t VPL = KIND == W_Q4 ? 32u : 16u;  // codes per 16-byte lane load
    constexpr int MF = VPL / 8;                         // MFMA steps per load
    extern __shared__ uint4 lds_raw[];
    uint4* xs = lds_raw;                                                      // [32][kQgemmXStride]
    float* sxs = reinterpret_cast<float*>(xs + kQgemmMTile * kQgemmXStride);  // [groups in slab][32]

    const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6, kb = lane >> 5, nl = lane & 31u;
    const uint32_t nb = blockIdx.x % a.n_blocks, ks = blockIdx.x / a.n_blocks;
    const uint32_t m0 = blockIdx.y * kQgemmMTile;
    const uint32_t mt = a.M - m0 < kQgemmMTile ? a.M - m0 : kQgemmMTile;
    const uint32_t n = nb * kQgemmRows + wave * 32u + nl;
    const uint32_t nc = n < a.N ? n : a.N - 1;  // rows past the end read the last row; never stored
    const uint32_t k0 = ks * a.k_per_split;
    const uint32_t k1 = k0 + a.k_per_split < a.K ? k0 + a.k_per_split : a.K;

    const uint4* wrow = a.w + (size_t)nc * a.cpr;
    const uint16_t* srow = a.sc + (size_t)nc * a.gpr;
    const uint16_t* brow = a.bi + (size_t)nc * a.gpr;
    const uint32_t lpg_mask = a.group / (2u * VPL) - 1u;  // loads per group - 1 (power of two)
    const uint32_t g8 = a.group >> 3;

    f32x16_t acc;
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[r] = 0.f;

    for (uint32_t ks0 = k0; ks0 < k1; ks0 += kQgemmSlabK) {
        const uint32_t slab_k = k1 - ks0 < kQgemmSlabK ? k1 - ks0 : kQgemmSlabK;
        const uint32_t s8 = slab_k >> 3;
        __syncthreads();  // the previous slab has been consumed
        for (uint32_t idx = threadIdx.x; idx < mt * s8; idx += kQgemmBlock) {
            const uint32_t m = idx / s8, k8 = idx - m * s8;
            uint4 v = *reinterpret_cast<const uint4*>(a.x + (size_t)(m0 + m) * a.K + ks0 + k8 * 8u);
            if constexpr (KIND == W_Q4) {
                // nibble pairing of q4_word_dot: (x0,x2) (x4,x6) (x1,x3) (x5,x7)
                v = make_uint4((v.x & 0xffffu) | (v.y << 16), (v.z & 0xffffu) | (v.w << 16),
                               (v.x >> 16) | (v.y & 0xffff0000u), (v.z >> 16) | (v.w & 0xffff0000u));
            }
            xs[m * kQgemmXStride + k8] = v;
        }
        __syncthreads();
        const uint32_t ng = slab_k / a.group;
        for (uint32_t idx = threadIdx.x; idx < ng * kQgemmMTile; idx += kQgemmBlock) {
            const uint32_t g = idx >> 5, m = idx & 31u;
            float s = 0.f;
            if (m < mt) {
                for (uint32_t i = 0; i < g8; ++i) {
                    const uint4 v = xs[m * kQgemmXStride + g * g8 + i];
                    s += ((bf16_lo(v.x) + bf16_hi(v.x)) + (bf16_lo(v.y) + bf16_hi(v.y))) +
                         ((bf16_lo(v.z) + bf16_hi(v.z)) + (bf16_lo(v.w) + bf16_hi(v.w)));
                }
            }
            sxs[idx] = s;
        }
        __syncthreads();

        const uint32_t loads = slab_k / (2u * VPL);
        const uint4* wp = wrow + ks0 / VPL + kb;
        const uint32_t gbase = ks0 / a.group;
        uint4 cur = wp[0];
        f32x16_t c;
#pragma unroll
        for (int r = 0; r < 16; ++r) c[r] = 0.f;
        for (uint32_t t = 0; t < loads; ++t) {
            const uint32_t tn = t + 1 < loads ? t + 1 : t;
            const uint4 nxt = wp[2u * tn];
            const uint32_t gl = (t * 2u * VPL) / a.group;  // group of this load inside the slab
            const uint32_t s_bits = srow[gbase + gl], b_bits = brow[gbase + gl];
            const uint32_t wd[4] = {cur.x, cur.y, cur.z, cur.w};
            const uint4* xa = xs + nl * kQgemmXStride + ((t * 2u + kb) * VPL >> 3);
#pragma unroll
            for (int j = 0; j < MF; ++j) {
                uint4 bw;
                if constexpr (KIND == W_Q4) {
                    const uint32_t even = wd[j] & 0x0F0F0F0Fu, odd = (wd[j] >> 4) & 0x0F0F0F0Fu;
                    bw.x = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(even, 512.0f, false));
                    bw.y = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(even, 512.0f, true));
                    bw.z = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(odd, 512.0f, false));
                    bw.w = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(odd, 512.0f, true));
                } else {
                    const uint32_t w0 = wd[2 * j], w1 = wd[2 * j + 1];
                    auto pair = [](float lo, float hi) {
                        const bf16x2_t p = {(__bf16)lo, (__bf16)hi};  // integers <= 255 are exact in bf16
                        return __builtin_bit_cast(uint32_t, p);
                    };
                    bw.x = pair((float)(w0 & 0xffu), (float)((w0 >> 8) & 0xffu));
                    bw.y = pair((float)((w0 >> 16) & 0xffu), (float)(w0 >> 24));
                    bw.z = pair((float)(w1 & 0xffu), (float)((w1 >> 8) & 0xffu));
                    bw.w = pair((float)((w1 >> 16) & 0xffu), (float)(w1 >> 24));
                }
                const uint4 av = xa[j];
                c = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, av),
                                                            __builtin_bit_cast(bf16x8_t, bw), c, 0, 0, 0);
            }
            if ((t & lpg_mask) == lpg_mask) {
                // group complete: fold the integer dot into the accumulators.  Register r
                // of this lane is activation row (r % 4) + 8 * (r / 4) + 4 * kb.
                const float s = bf16_bits_to_f32(s_bits), b = bf16_bits_to_f32(b_bits);
                const float* sxg = sxs + gl * kQgemmMTile + 4u * kb;
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const float4 sx4 = *reinterpret_cast<const float4*>(sxg + 8 * q);
                    acc[4 * q + 0] += fmaf(s, c[4 * q + 0], b * sx4.x);
                    acc[4 * q + 1] += fmaf(s, c[4 * q + 1], b * sx4.y);
                    acc[4 * q + 2] += fmaf(s, c[4 * q + 2], b * sx4.z);
                    acc[4 * q + 3] += fmaf(s, c[4 * q + 3], b * sx4.w);
                }
#pragma unroll
                for (int r = 0; r < 16; ++r) c[r] = 0.f;
            }
            cur = nxt;
        }
    }

    if (n < a.N) {
        float* dst = a.partial + ((size_t)ks * a.M + m0) * a.N + n;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const uint32_t m = (uint32_t)(r % 4 + 8 * (r / 4)) + 4u * kb;
            if (m < mt) dst[(size_t)m * a.N] = acc[r];
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

namespace {

struct QgemmShape {
    uint32_t n_blocks, m_tiles, ksplit, k_per_split;
};

fk_status qgemm_shape(const DeviceFacts* dev, uint32_t M, uint32_t N, uint32_t K, uint32_t group, QgemmShape* out) {
    if (M == 0 || N == 0 || K == 0) return set_error(FK_ERR_INVALID, "qgemm: empty shape");
    if (group != 64 && group != 128) return set_error(FK_ERR_UNSUPPORTED, "qgemm: group size must be 64 or 128");
    if (K % group) return set_error(FK_ERR_UNSUPPORTED, "qgemm: K must be a multiple of the group size");
    if ((uint64_t)M * N > 0x7fffffffull) return set_error(FK_ERR_UNSUPPORTED, "qgemm: output too large");
    QgemmShape s;
    s.n_blocks = (N + kQgemmRows - 1) / kQgemmRows;
    s.m_tiles = (M + kQgemmMTile - 1) / kQgemmMTile;
    // Split k until about two blocks per CU exist, but keep at least 256 k per block.
    const uint32_t want = (2u * (uint32_t)dev->cus + s.n_blocks * s.m_tiles - 1) / (s.n_blocks * s.m_tiles);
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

fk_status plan_qgemm_main(const DeviceFacts* dev, const fk_weight* W, const uint16_t* x, uint32_t M, float* partial,
                          QgemmShape* shape, Launch* out) {
    FK_TRY(qgemm_shape(dev, M, W->n, W->k, W->group, shape));
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
    out->func = W->bits == 4 ? reinterpret_cast<const void*>(&qgemm_kernel<W_Q4>)
                             : reinterpret_cast<const void*>(&qgemm_kernel<W_Q8>);
    out->grid = dim3(shape->n_blocks * shape->ksplit, shape->m_tiles, 1);
    out->block = dim3(kQgemmBlock, 1, 1);
    out->shmem = kQgemmLdsBytes;
    out->set_args(a);
    return FK_OK;
}

void plan_reduce(const float* p0, const float* p1, const uint16_t* bias, const uint16_t* res, uint16_t* y, uint32_t M,
                 uint32_t N, uint32_t ksplit, int variant, Launch* out) {
    QgemmReduceArgs r;
    r.p0 = p0; r.p1 = p1; r.bias = bias; r.res = res; r.y = y;
    r.M = M; r.N = N; r.ksplit = ksplit; r.variant = variant;
    out->func = reinterpret_cast<const void*>(&qgemm_reduce_kernel);
    out->grid = dim3((M * N + 255u) / 256u, 1, 1);
    out->block = dim3(256, 1, 1);
    out->shmem = 0;
    out->set_args(r);
}

}  // namespace

fk_status qgemm_workspace_bytes(uint32_t M, uint32_t N, uint32_t K, uint32_t group, size_t* bytes) {
    const DeviceFacts* dev;
    FK_TRY(device_facts(&dev));
    QgemmShape s;
    FK_TRY(qgemm_shape(dev, M, N, K, group, &s));
    *bytes = (size_t)s.ksplit * M * N * sizeof(float);
    return FK_OK;
}

fk_status plan_qgemm(const fk_weight* W, const uint16_t* x, uint32_t M, const uint16_t* bias, const uint16_t* res,
                     uint16_t* y, void* workspace, Launch* main, Launch* reduce) {
    const DeviceFacts* dev;
    FK_TRY(device_facts(&dev));
    FK_TRY(check_weight(W, "qgemm"));
    if (!x || !y || !workspace) return set_error(FK_ERR_INVALID, "qgemm: null activation, output or workspace");
    QgemmShape s;
    FK_TRY(plan_qgemm_main(dev, W, x, M, static_cast<float*>(workspace), &s, main));
    plan_reduce(static_cast<float*>(workspace), nullptr, bias, res, y, M, W->n, s.ksplit, 0, reduce);
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
    QgemmShape s;
    float* p0 = static_cast<float*>(workspace);
    FK_TRY(plan_qgemm_main(dev, Wg, x, M, p0, &s, gate));
    float* p1 = p0 + (size_t)s.ksplit * M * Wg->n;
    FK_TRY(plan_qgemm_main(dev, Wu, x, M, p1, &s, up));
    plan_reduce(p0, p1, nullptr, nullptr, out, M, Wg->n, s.ksplit, variant, reduce);
    return FK_OK;
}

}  // namespace fk
