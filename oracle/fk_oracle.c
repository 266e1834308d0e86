/*
 * fk_oracle.c -- CPU restatement of the decode hot path of Pribess/FuseKit.
 *
 * THIS IS TEST INFRASTRUCTURE, NOT PRODUCT CODE.  Only tests/, the smoke check
 * and the benchmark's cpu_baseline leg may load it, and only as the checker or
 * the reported CPU baseline.  The shipped library never links or calls it.
 *
 * The arithmetic that FuseKit's emitted Metal kernels perform ultimately
 * mirrors MLX (Apple, v0.31.2 per reference BENCHMARKS.md:16): mx.quantize,
 * mx.quantized_matmul, mx.fast.rms_norm, mx.fast.rope and
 * mx.fast.scaled_dot_product_attention.  MLX is not vendored in the reference
 * and is not installed here; the reference holds no golden vectors for this
 * path.  Each function below therefore follows the reference's own statement
 * of the arithmetic (file:line cited per function, paths relative to the
 * reference root) and is pinned by tests/test_oracle_*.py through closed
 * forms, invariants, brute force and an independent numpy formulation.
 *
 * Pin status per function (see tests/test_oracle_pins.py):
 *   quantize/pack/unpack ........ pinned (exhaustive nibble/lane, invariants)
 *   qgemv / linear .............. pinned (numpy float64 matmul on dequant W)
 *   rms_norm .................... pinned (closed forms + numpy restatement)
 *   rope ........................ pinned (norm preservation, pos 0, composition)
 *   swiglu A/B/C ................ pinned (numpy restatement per variant; A vs B
 *                                 vs C agree within bf16 noise)
 *   sdpa_decode ................. pinned (float64 softmax attention; kv_len=1;
 *                                 chunk-merge invariance)
 *   argmax ...................... pinned (brute force, tie rule)
 *   routed gate/up, routed reduce pinned (reduce to the pinned dense pair / qGEMV on the
 *                                 selected expert's slice; slot-order fp32 sum restated
 *                                 in numpy; clamp, row_idx, shared expert, residual)
 *   qgemm ....................... pinned as the row-wise repetition of qGEMV; the
 *                                 reference's multi-row path rounds every dequantised
 *                                 weight to bf16 first (MLX QuantizedBlockLoader, not
 *                                 vendored): that rounding is parity unpinned
 *   qgemm, weights rounded to bf16 pinned as arithmetic (numpy: dequantise, round to bf16,
 *                                 float64 matmul; one-hot rows return T(s*q+b) exactly); that
 *                                 MLX rounds exactly there is read from the reference's
 *                                 emitter, MLX itself is not vendored: parity unpinned
 *   quantised KV store / attention pinned (V rows and unrotated K rows = the pinned quantiser
 *                                 bit for bit; rotated K rows dequantise to within the
 *                                 quantiser's step of the pinned bf16 RoPE; only the
 *                                 addressed row written; attention = float64 softmax
 *                                 attention over the dequantised cache)
 *   sdpa_prefill ................ pinned (every row = the pinned sdpa_decode over the positions
 *                                 it sees, to one bf16 step: the reference normalises the
 *                                 scores before the product with V here and after it there;
 *                                 float64 causal softmax attention in numpy; row 0 of a fresh
 *                                 group returns V[0]; later cache rows never influence a row)
 *   split-key cache store ....... pinned (equals the pinned rope + plain store on the assembled
 *                                 [K0 | K1] row for half-split pairs; traditional pairs against
 *                                 a numpy complex rotation; shared K1 head, packed source)
 *   split-query attention ....... pinned (equals the pinned sdpa_decode on [Q0 | rope(Q1)] to one
 *                                 bf16 step of the rotated query; position kv_len - 1)
 *   softmax top-k route ......... pinned (equal logits -> 1/N exactly, indices 0..k-1; numpy
 *                                 float64 softmax + stable sort; probabilities tie after the
 *                                 rounding to T and the lower index wins)
 *   hand-derived known answers .. tests/golden/known_answers.json
 *   MLX-internal accumulation order, Metal fast::cos/sin/exp bit patterns:
 *                                 parity unpinned (cannot be observed here;
 *                                 irrelevant under the rel-L2 <= 1e-2 bar).
 *
 * Conventions: activations "T" are bfloat16 held as uint16_t bit patterns;
 * every T(...) in the reference is a round-to-nearest-even fp32->bf16 here.
 * Dot products accumulate in double and are narrowed to float once, so the
 * oracle is the closest fp32 value any summation order may aim for; two fp32
 * summation orders of the projections can be switched on (fko_set_accum_mode)
 * to measure the envelope fp32 arithmetic leaves around those values.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

#define FKO_API __attribute__((visibility("default")))

/* ------------------------------------------------------------------ bf16 */

static inline float bf16_to_f32(uint16_t h) {
    uint32_t u = (uint32_t)h << 16;
    float f;
    memcpy(&f, &u, 4);
    return f;
}

static inline uint16_t f32_to_bf16(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u); /* quiet NaN */
    uint32_t lsb = (u >> 16) & 1u;
    u += 0x7fffu + lsb;
    return (uint16_t)(u >> 16);
}

static inline float rbf(float f) { return bf16_to_f32(f32_to_bf16(f)); }

FKO_API void fko_f32_to_bf16(const float *in, uint16_t *out, int64_t n) {
    for (int64_t i = 0; i < n; ++i) out[i] = f32_to_bf16(in[i]);
}
FKO_API void fko_bf16_to_f32(const uint16_t *in, float *out, int64_t n) {
    for (int64_t i = 0; i < n; ++i) out[i] = bf16_to_f32(in[i]);
}

FKO_API int fko_num_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}
FKO_API void fko_set_num_threads(int n) {
#ifdef _OPENMP
    omp_set_num_threads(n);
#else
    (void)n;
#endif
}

/* ------------------------------------------------------- Q0: quantizer */
/*
 * MLX-affine quantizer, restated from the reference's own restatement at
 * src/codegen/kernels/rope_kv_cache_store_decode_quant.rs:208-221 (same block
 * in src/codegen/kernels/rmsnorm_qkv.rs:565-580); layout per
 * src/fusion/ir.rs:236-242 and scripts/poc_int4_gemv.py:19-24:
 *   packed u32 [N, K*bits/32], value j of a word at bits (j*bits), LSB first;
 *   scales/biases T [N, K/group].
 * The scale/bias are rounded to T *after* the integer codes are chosen from
 * the fp32 scale/bias, as in the reference (codes from fp32, meta stored T).
 */
FKO_API void fko_quantize_affine(const float *w, int64_t n, int64_t k, int bits, int group,
                                 uint32_t *packed, uint16_t *scales, uint16_t *biases) {
    const int per_word = 32 / bits;
    const int mask = (1 << bits) - 1;
    const int64_t words = k / per_word, groups = k / group;
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < n; ++r) {
        const float *row = w + r * k;
        uint32_t *prow = packed + r * words;
        memset(prow, 0, (size_t)words * 4);
        for (int64_t g = 0; g < groups; ++g) {
            const float *x = row + g * group;
            float vmin = x[0], vmax = x[0];
            for (int i = 1; i < group; ++i) {
                vmin = x[i] < vmin ? x[i] : vmin;
                vmax = x[i] > vmax ? x[i] : vmax;
            }
            float scale_abs = fmaxf((vmax - vmin) / (float)mask, 1.0e-7f);
            int lo_anchor = fabsf(vmin) > fabsf(vmax);
            float scale = lo_anchor ? scale_abs : -scale_abs;
            float edge = lo_anchor ? vmin : vmax;
            float q0 = roundf(edge / scale);
            int at_zero = (q0 == 0.0f);
            scale = at_zero ? scale : (edge / q0);
            float bias = at_zero ? 0.0f : edge;
            float inv_scale = (scale != 0.0f) ? (1.0f / scale) : 0.0f;
            for (int i = 0; i < group; ++i) {
                int qi = (int)roundf((x[i] - bias) * inv_scale);
                qi = qi < 0 ? 0 : (qi > mask ? mask : qi);
                int64_t col = g * group + i;
                prow[col / per_word] |= ((uint32_t)qi & (uint32_t)mask) << ((col % per_word) * bits);
            }
            scales[r * groups + g] = f32_to_bf16(scale);
            biases[r * groups + g] = f32_to_bf16(bias);
        }
    }
}

/* w[i,j] = q(packed[i, j/per_word], j%per_word) * scales[i, j/g] + biases[i, j/g]
 * (src/fusion/ir.rs:236-242).  Integer codes out for the bit-exact tests. */
FKO_API void fko_unpack_codes(const uint32_t *packed, int64_t n, int64_t k, int bits, uint8_t *codes) {
    const int per_word = 32 / bits;
    const uint32_t mask = (1u << bits) - 1u;
    for (int64_t r = 0; r < n; ++r)
        for (int64_t j = 0; j < k; ++j)
            codes[r * k + j] =
                (uint8_t)((packed[r * (k / per_word) + j / per_word] >> ((j % per_word) * bits)) & mask);
}

FKO_API void fko_dequantize(const uint32_t *packed, const uint16_t *scales, const uint16_t *biases,
                            int64_t n, int64_t k, int bits, int group, float *out) {
    const int per_word = 32 / bits;
    const uint32_t mask = (1u << bits) - 1u;
    const int64_t words = k / per_word, groups = k / group;
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < n; ++r)
        for (int64_t j = 0; j < k; ++j) {
            uint32_t q = (packed[r * words + j / per_word] >> ((j % per_word) * bits)) & mask;
            float s = bf16_to_f32(scales[r * groups + j / group]);
            float b = bf16_to_f32(biases[r * groups + j / group]);
            out[r * k + j] = (float)q * s + b;
        }
}

/* ------------------------------------------------ seeded synthetic data */
/*
 * Test-data generator that the GPU library's synthetic fill (kinds 3 / 4) reproduces bit for bit:
 * only integer arithmetic, exact int -> float conversions and single IEEE operations (one fused
 * multiply-add, written as such on both sides), so a model instantiated in HBM and one built on
 * the host from the same seeds hold the same bytes.  Not part of the reference: it replaces
 * "weights drawn N(0, 0.02^2) from a seed" (MLX's generator cannot run here).
 *   z(seed, i) = (2 * S - 524280) * (1 / 107019.84),  S = sum of eight 16-bit fields of two
 *                splitmix64 words keyed by (seed, i): mean 0, variance 1, |z| < 4.9
 *   value      = fma(std, z, mean) * rowscale(i / row_len)
 *   rowscale(j) (row_len != 0 and tau != 0): u = floor(tau * z(seed ^ K, j) * 8),
 *                rowscale = (1 + (u & 7) / 8) * 2^(u >> 3): a log-normal-like spread of row norms
 *   rows j < loud_rows are multiplied by loud_gain * 2^-j instead (a few dominant rows, each half as loud
 *                as the one before, so that two of them rarely compete at equal strength)
 */
static inline uint64_t splitmix64(uint64_t z) {
    z += 0x9E3779B97F4A7C15ull;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}
static inline float ih_normal(uint64_t seed, uint64_t i) {
    const uint64_t r0 = splitmix64(seed * 0xD1342543DE82EF95ull + i), r1 = splitmix64(r0);
    int32_t sum = 0;
    for (int f = 0; f < 4; ++f) sum += (int32_t)((r0 >> (16 * f)) & 0xFFFF) + (int32_t)((r1 >> (16 * f)) & 0xFFFF);
    return (float)(2 * sum - 524280) * 9.3440616e-06f;
}
static inline float row_scale(uint64_t seed, uint64_t row, float tau) {
    const float t = floorf((tau * ih_normal(seed ^ 0x5DEECE66Dull, row)) * 8.0f);
    const int u = (int)t;
    return ldexpf(1.0f + (float)(u & 7) * 0.125f, u >> 3);
}
/* kind 3: fp32 out, kind 4: bf16 out */
FKO_API void fko_synth_fill(void *out, int64_t count, uint64_t seed, float mean, float std, int kind,
                            int64_t row_len, float tau, int64_t loud_rows, float loud_gain) {
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < count; ++i) {
        float v = fmaf(std, ih_normal(seed, (uint64_t)i), mean);
        if (row_len && i / row_len < loud_rows) v = v * ldexpf(loud_gain, -(int)(i / row_len));
        else if (row_len && tau != 0.0f) v = v * row_scale(seed, (uint64_t)(i / row_len), tau);
        if (kind == 3) ((float *)out)[i] = v;
        else ((uint16_t *)out)[i] = f32_to_bf16(v);
    }
}

/* --------------------------------------------------------- K1: linear */
/*
 * One weight matrix [n, k] in one of three storage kinds:
 *   bits 4 / 8 : MLX-affine (packed, scales, biases, group)
 *   bits 16    : dense bf16 (packed points at uint16 data, scales/biases NULL)
 */
typedef struct {
    const void *w;
    const uint16_t *scales;
    const uint16_t *biases;
    int64_t n, k;
    int bits, group;
} fko_weight;

/* Accumulation mode of every projection (linear_acc), process-wide; tests switch it to measure how far fp32
 * summation orders -- which the reference's own kernels use -- sit from the double sums:
 *   0  double accumulation, narrowed to float once (default: the value any fp32 order aims for)
 *   1  fp32, the per-element form in element order: acc += x[k] * (q*s + b)
 *      (src/codegen/kernels/mod.rs:2850-2908 read literally, one accumulator)
 *   2  fp32, the qdot form per quantisation group, acc += s * sum(x*q) + b * sum(x), groups in order
 *      (src/codegen/kernels/mod.rs:2634-2713); dense rows: 32 interleaved partial sums added as a
 *      simdgroup sum does (pairwise tree), src/codegen/msl.rs:310-440 */
static int g_accum_mode = 0;
FKO_API void fko_set_accum_mode(int mode) { g_accum_mode = mode; }
FKO_API int fko_get_accum_mode(void) { return g_accum_mode; }

static inline uint32_t code_at(const uint32_t *prow, int64_t j, int bits, int per_word, uint32_t mask) {
    return (prow[j / per_word] >> ((j % per_word) * bits)) & mask;
}

/* acc[i] = sum_k x[k] * (q*s + b), the per-element form of
 * src/codegen/kernels/mod.rs:2850-2908 (q4) and :3053-3104 (q8); dense rows
 * as src/codegen/kernels/linear_residual.rs:342-346.  x is fp32 holding values
 * the caller already rounded to T where the reference does.  Mode 0 keeps four
 * double accumulators (elements j = 0..3 mod 4), added (a0 + a1) + (a2 + a3). */
static void linear_acc(const fko_weight *W, const float *x, float *acc) {
    const int64_t n = W->n, k = W->k;
    const int mode = g_accum_mode;
    if (W->bits == 16) {
        const uint16_t *d = (const uint16_t *)W->w;
#pragma omp parallel for schedule(static)
        for (int64_t r = 0; r < n; ++r) {
            const uint16_t *row = d + r * k;
            if (mode == 0) {
                double a[4] = {0.0, 0.0, 0.0, 0.0};
                int64_t j = 0;
                for (; j + 4 <= k; j += 4)
                    for (int e = 0; e < 4; ++e) a[e] += (double)x[j + e] * (double)bf16_to_f32(row[j + e]);
                for (; j < k; ++j) a[0] += (double)x[j] * (double)bf16_to_f32(row[j]);
                acc[r] = (float)((a[0] + a[1]) + (a[2] + a[3]));
            } else if (mode == 1) {
                float a = 0.0f;
                for (int64_t j = 0; j < k; ++j) a += x[j] * bf16_to_f32(row[j]);
                acc[r] = a;
            } else {
                float lane[32];
                for (int i = 0; i < 32; ++i) lane[i] = 0.0f;
                for (int64_t j = 0; j < k; ++j) lane[j & 31] += x[j] * bf16_to_f32(row[j]);
                for (int w = 16; w >= 1; w >>= 1)
                    for (int i = 0; i < w; ++i) lane[i] += lane[i + w];
                acc[r] = lane[0];
            }
        }
        return;
    }
    const int bits = W->bits, per_word = 32 / bits, group = W->group;
    const uint32_t mask = (1u << bits) - 1u;
    const int64_t words = k / per_word, groups = k / group;
    const uint32_t *p = (const uint32_t *)W->w;
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < n; ++r) {
        const uint32_t *prow = p + r * words;
        if (mode == 0) {
            double a[4] = {0.0, 0.0, 0.0, 0.0};
            float wv[128];
            for (int64_t g = 0; g < groups; ++g) {
                const float s = bf16_to_f32(W->scales[r * groups + g]);
                const float b = bf16_to_f32(W->biases[r * groups + g]);
                const float *xg = x + g * group;
                const uint32_t *pw = prow + g * (group / per_word);
                /* fp32 dequant as in the reference: float(q) * s + b, two roundings */
                if (bits == 4) {
                    for (int w = 0; w < group / 8; ++w)
                        for (int e = 0; e < 8; ++e) wv[w * 8 + e] = (float)((pw[w] >> (4 * e)) & 15u) * s + b;
                } else {
                    for (int w = 0; w < group / 4; ++w)
                        for (int e = 0; e < 4; ++e) wv[w * 4 + e] = (float)((pw[w] >> (8 * e)) & 255u) * s + b;
                }
                for (int i = 0; i < group; i += 4)
                    for (int e = 0; e < 4; ++e) a[e] += (double)xg[i + e] * (double)wv[i + e];
            }
            acc[r] = (float)((a[0] + a[1]) + (a[2] + a[3]));
        } else if (mode == 1) {
            float a = 0.0f;
            for (int64_t g = 0; g < groups; ++g) {
                const float s = bf16_to_f32(W->scales[r * groups + g]);
                const float b = bf16_to_f32(W->biases[r * groups + g]);
                for (int i = 0; i < group; ++i) {
                    const int64_t j = g * group + i;
                    const float wvj = (float)code_at(prow, j, bits, per_word, mask) * s + b;
                    a += x[j] * wvj;
                }
            }
            acc[r] = a;
        } else {
            float a = 0.0f;
            for (int64_t g = 0; g < groups; ++g) {
                const float s = bf16_to_f32(W->scales[r * groups + g]);
                const float b = bf16_to_f32(W->biases[r * groups + g]);
                float dq = 0.0f, sx = 0.0f;
                for (int i = 0; i < group; ++i) {
                    const int64_t j = g * group + i;
                    dq += x[j] * (float)code_at(prow, j, bits, per_word, mask);
                    sx += x[j];
                }
                a += s * dq + b * sx;
            }
            acc[r] = a;
        }
    }
}

FKO_API void fko_linear_acc(const fko_weight *W, const uint16_t *x_bf16, float *acc) {
    float *x = (float *)malloc(sizeof(float) * (size_t)W->k);
    for (int64_t j = 0; j < W->k; ++j) x[j] = bf16_to_f32(x_bf16[j]);
    linear_acc(W, x, acc);
    free(x);
}

/* y = T(acc (+bias)) : quantized GEMV with one final round
 * (src/codegen/msl.rs:434-438); bias added in fp32 before the round
 * (src/codegen/kernels/rmsnorm_qkv.rs:417-422). */
FKO_API void fko_qgemv(const fko_weight *W, const uint16_t *x, const uint16_t *bias, uint16_t *y) {
    float *acc = (float *)malloc(sizeof(float) * (size_t)W->n);
    fko_linear_acc(W, x, acc);
    for (int64_t i = 0; i < W->n; ++i) {
        float a = acc[i];
        if (bias) a += bf16_to_f32(bias[i]);
        y[i] = f32_to_bf16(a);
    }
    free(acc);
}

/* K1r: y = T(acc + float(res)); optional second residual rounds twice
 * (src/codegen/kernels/linear_residual.rs:374-381). */
FKO_API void fko_linear_residual(const fko_weight *W, const uint16_t *x, const uint16_t *res,
                                 const uint16_t *res2, uint16_t *y) {
    float *acc = (float *)malloc(sizeof(float) * (size_t)W->n);
    fko_linear_acc(W, x, acc);
    for (int64_t i = 0; i < W->n; ++i) {
        uint16_t y0 = f32_to_bf16(acc[i] + (res ? bf16_to_f32(res[i]) : 0.0f));
        if (res2) y0 = f32_to_bf16(bf16_to_f32(y0) + bf16_to_f32(res2[i]));
        y[i] = y0;
    }
    free(acc);
}

/* ------------------------------------------------------------ N: norm */
/* r = rsqrt(sum(x^2)/H + eps) (precise rsqrt, src/codegen/kernels/rmsnorm_qkv.rs:325);
 * norm_y[i] = float(T(w[i] * T(x[i] * r))) (src/codegen/kernels/mod.rs:4464-4472). */
static void rmsnorm_f(const uint16_t *x, const uint16_t *w, int64_t h, float eps, float *out) {
    double ss = 0.0;
    for (int64_t i = 0; i < h; ++i) {
        double v = bf16_to_f32(x[i]);
        ss += v * v;
    }
    float r = 1.0f / sqrtf((float)ss / (float)h + eps);
    for (int64_t i = 0; i < h; ++i) {
        float t = rbf(bf16_to_f32(x[i]) * r);
        out[i] = rbf(bf16_to_f32(w[i]) * t);
    }
}

FKO_API void fko_rmsnorm(const uint16_t *x, const uint16_t *w, int64_t h, float eps, uint16_t *y) {
    float *o = (float *)malloc(sizeof(float) * (size_t)h);
    rmsnorm_f(x, w, h, eps, o);
    for (int64_t i = 0; i < h; ++i) y[i] = f32_to_bf16(o[i]);
    free(o);
}

/* ------------------------------------------------------------ K2: QKV */
/* Non-sink variant of src/codegen/kernels/rmsnorm_qkv.rs:53-736: norm into
 * fp32 scratch, three projections, bf16 bias added before the round. */
FKO_API void fko_rmsnorm_qkv(const uint16_t *x, const uint16_t *norm_w, float eps, const fko_weight *Wq,
                             const fko_weight *Wk, const fko_weight *Wv, const uint16_t *bq,
                             const uint16_t *bk, const uint16_t *bv, uint16_t *q, uint16_t *k,
                             uint16_t *v) {
    const int64_t h = Wq->k;
    float *ny = (float *)malloc(sizeof(float) * (size_t)h);
    rmsnorm_f(x, norm_w, h, eps, ny);
    const fko_weight *Ws[3] = {Wq, Wk, Wv};
    const uint16_t *bs[3] = {bq, bk, bv};
    uint16_t *outs[3] = {q, k, v};
    for (int m = 0; m < 3; ++m) {
        float *acc = (float *)malloc(sizeof(float) * (size_t)Ws[m]->n);
        linear_acc(Ws[m], ny, acc);
        for (int64_t i = 0; i < Ws[m]->n; ++i) {
            float a = acc[i];
            if (bs[m]) a += bf16_to_f32(bs[m][i]);
            outs[m][i] = f32_to_bf16(a);
        }
        free(acc);
    }
    free(ny);
}

/* ---------------------------------------------------------- K3a: SwiGLU */
/* variant 0 ("A"): every op in T -- src/codegen/kernels/rmsnorm_gateup_swiglu.rs:236-257
 * variant 1 ("B"): fp32 sigmoid, one round -- src/codegen/msl.rs:1286-1294
 * variant 2 ("C"): rounds sig and gated -- src/codegen/msl.rs:2441-2449      */
static uint16_t swiglu_apply(float acc_g, float acc_u, int variant) {
    float g = rbf(acc_g), u = rbf(acc_u);
    if (variant == 0) {
        float e = rbf(expf(fabsf(g)));
        float den = rbf(1.0f + e);
        float sig_y = rbf(1.0f / den);
        float sig = (g < 0.0f) ? sig_y : rbf(1.0f - sig_y);
        float silu = rbf(g * sig);
        return f32_to_bf16(silu * u);
    } else if (variant == 1) {
        float sig = 1.0f / (1.0f + expf(-g));
        return f32_to_bf16((sig * g) * u);
    } else {
        float sig = rbf(1.0f / (1.0f + expf(-g)));
        float gated = rbf(sig * g);
        return f32_to_bf16(gated * u);
    }
}

FKO_API uint16_t fko_swiglu_scalar(float acc_g, float acc_u, int variant) {
    return swiglu_apply(acc_g, acc_u, variant);
}

/* norm_w == NULL: x is consumed as is (QmvSwiglu, src/codegen/kernels/qmv_swiglu.rs:20-246);
 * otherwise RmsNormGateUpSwiglu (src/codegen/kernels/rmsnorm_gateup_swiglu.rs:27-267). */
FKO_API void fko_gateup_swiglu(const uint16_t *x, const uint16_t *norm_w, float eps, const fko_weight *Wg,
                               const fko_weight *Wu, int variant, uint16_t *out) {
    const int64_t h = Wg->k, n = Wg->n;
    float *ny = (float *)malloc(sizeof(float) * (size_t)h);
    if (norm_w)
        rmsnorm_f(x, norm_w, h, eps, ny);
    else
        for (int64_t i = 0; i < h; ++i) ny[i] = bf16_to_f32(x[i]);
    float *ag = (float *)malloc(sizeof(float) * (size_t)n);
    float *au = (float *)malloc(sizeof(float) * (size_t)n);
    linear_acc(Wg, ny, ag);
    linear_acc(Wu, ny, au);
    for (int64_t i = 0; i < n; ++i) out[i] = swiglu_apply(ag[i], au[i], variant);
    free(ny);
    free(ag);
    free(au);
}

/* ------------------------------------------------------------- R: RoPE */
/* Half-split RoPE, pair (d, d+half): inv = exp2(-(d/half) * log2(theta)) with
 * log2(theta) computed in double then narrowed to float; angle = pos * inv in
 * fp32 (src/codegen/kernels/rope_q_decode.rs:93-114).  The reference uses
 * Metal fast::cos/sin; libm cosf/sinf stand in (bit patterns unpinned). */
static inline void rope_pair(float lo, float hi, int64_t d, int64_t half, uint32_t pos, float base_log2,
                             float *olo, float *ohi) {
    float d_norm = (float)d / (float)half;
    float inv_freq = exp2f(-d_norm * base_log2);
    float angle = (float)pos * inv_freq;
    float c = cosf(angle), s = sinf(angle);
    *olo = lo * c - hi * s;
    *ohi = hi * c + lo * s;
}

/* In-place on q [n_heads, head_dim]; rotates the first rope_dims of each head. */
FKO_API void fko_rope_q(uint16_t *q, int64_t n_heads, int64_t head_dim, int64_t rope_dims, float theta,
                        uint32_t pos) {
    const float base_log2 = (float)log2((double)theta);
    const int64_t half = rope_dims / 2;
    for (int64_t h = 0; h < n_heads; ++h)
        for (int64_t d = 0; d < half; ++d) {
            uint16_t *p = q + h * head_dim;
            float lo, hi;
            rope_pair(bf16_to_f32(p[d]), bf16_to_f32(p[d + half]), d, half, pos, base_log2, &lo, &hi);
            p[d] = f32_to_bf16(lo);
            p[d + half] = f32_to_bf16(hi);
        }
}

/* RoPE(K) then store K,V at cache row (write_offset % capacity); cache layout
 * [n_kv, capacity, head_dim] (src/codegen/kernels/rope_kv_cache_store_decode.rs:87-137). */
FKO_API void fko_rope_kv_store(const uint16_t *k, const uint16_t *v, int64_t n_kv, int64_t head_dim,
                               int64_t rope_dims, float theta, uint32_t pos, uint32_t write_offset,
                               uint32_t capacity, uint16_t *cache_k, uint16_t *cache_v) {
    const float base_log2 = (float)log2((double)theta);
    const int64_t half = rope_dims / 2;
    const int64_t row = write_offset % capacity;
    for (int64_t h = 0; h < n_kv; ++h) {
        uint16_t *ck = cache_k + (h * (int64_t)capacity + row) * head_dim;
        uint16_t *cv = cache_v + (h * (int64_t)capacity + row) * head_dim;
        const uint16_t *kh = k + h * head_dim;
        for (int64_t d = 0; d < head_dim; ++d) ck[d] = kh[d];
        for (int64_t d = 0; d < half; ++d) {
            float lo, hi;
            rope_pair(bf16_to_f32(kh[d]), bf16_to_f32(kh[d + half]), d, half, pos, base_log2, &lo, &hi);
            ck[d] = f32_to_bf16(lo);
            ck[d + half] = f32_to_bf16(hi);
        }
        for (int64_t d = 0; d < head_dim; ++d) cv[d] = v[h * head_dim + d];
    }
}

/* Per-head RMSNorm T(w*T(x*r)) followed by RoPE on the normed T values
 * (src/codegen/kernels/rmsnorm_rope_kv_cache_store_decode.rs:101-152; the q
 * side follows src/codegen/kernels/rmsnorm_rope_qgate_decode.rs:84-136 without
 * the gate half).  In place on [n_heads, head_dim]. */
FKO_API void fko_headnorm_rope(uint16_t *x, const uint16_t *w, int64_t n_heads, int64_t head_dim,
                               int64_t rope_dims, float eps, float theta, uint32_t pos) {
    const float base_log2 = (float)log2((double)theta);
    const int64_t half = rope_dims / 2;
    float *ny = (float *)malloc(sizeof(float) * (size_t)head_dim);
    for (int64_t h = 0; h < n_heads; ++h) {
        uint16_t *p = x + h * head_dim;
        rmsnorm_f(p, w, head_dim, eps, ny);
        for (int64_t d = 0; d < head_dim; ++d) p[d] = f32_to_bf16(ny[d]);
        for (int64_t d = 0; d < half; ++d) {
            float lo, hi;
            rope_pair(ny[d], ny[d + half], d, half, pos, base_log2, &lo, &hi);
            p[d] = f32_to_bf16(lo);
            p[d + half] = f32_to_bf16(hi);
        }
    }
    free(ny);
}

/* Plain store of prepared K/V rows (no rope, no norm). */
FKO_API void fko_kv_store(const uint16_t *k, const uint16_t *v, int64_t n_kv, int64_t k_dim, int64_t v_dim,
                          uint32_t write_offset, uint32_t capacity, uint16_t *cache_k, uint16_t *cache_v) {
    const int64_t row = write_offset % capacity;
    for (int64_t h = 0; h < n_kv; ++h) {
        memcpy(cache_k + (h * (int64_t)capacity + row) * k_dim, k + h * k_dim, (size_t)k_dim * 2);
        memcpy(cache_v + (h * (int64_t)capacity + row) * v_dim, v + h * v_dim, (size_t)v_dim * 2);
    }
}

/* ------------------------------------------------- quantised KV cache */
/*
 * Store (src/codegen/kernels/rope_kv_cache_store_decode_quant.rs:100-260): the K row after
 * half-split RoPE stays in fp32 (it is NOT rounded to T before quantisation), the V row is
 * taken as is; every group of `group` dims along the head is quantised with the Q0 formula.
 * Layout (src/codegen/kernels/sdpa_decode_quant.rs:10-17): packed u32 [n_kv, capacity,
 * D*bits/32], scales / biases T [n_kv, capacity, D/group].  With a norm weight the head is
 * first normalised as in fko_headnorm_rope (T(w*T(x*r))) and rotated from those T values.
 */
FKO_API void fko_rope_kv_store_quant(const uint16_t *k, const uint16_t *v, const uint16_t *k_norm, int64_t n_kv,
                                     int64_t head_dim, int64_t rope_dims, float theta, float eps, uint32_t pos,
                                     uint32_t write_offset, uint32_t capacity, int bits, int group,
                                     uint32_t *ck_packed, uint16_t *ck_scales, uint16_t *ck_biases,
                                     uint32_t *cv_packed, uint16_t *cv_scales, uint16_t *cv_biases) {
    const float base_log2 = (float)log2((double)theta);
    const int64_t half = rope_dims / 2, words = head_dim * bits / 32, groups = head_dim / group;
    const int64_t row = write_offset % capacity;
    float *kr = (float *)malloc(sizeof(float) * (size_t)head_dim), *vr = (float *)malloc(sizeof(float) * (size_t)head_dim);
    for (int64_t h = 0; h < n_kv; ++h) {
        const uint16_t *kh = k + h * head_dim;
        float r = 1.0f;
        if (k_norm) {
            double ss = 0.0;
            for (int64_t d = 0; d < head_dim; ++d) ss += (double)bf16_to_f32(kh[d]) * (double)bf16_to_f32(kh[d]);
            r = 1.0f / sqrtf((float)(ss / (double)head_dim) + eps);
        }
        for (int64_t d = 0; d < head_dim; ++d) {
            const float x = bf16_to_f32(kh[d]);
            kr[d] = k_norm ? rbf(bf16_to_f32(k_norm[d]) * rbf(x * r)) : x;
            vr[d] = bf16_to_f32(v[h * head_dim + d]);
        }
        for (int64_t d = 0; d < half; ++d) {
            float lo, hi;
            rope_pair(kr[d], kr[d + half], d, half, pos, base_log2, &lo, &hi);
            kr[d] = lo;
            kr[d + half] = hi;
        }
        const int64_t o = h * (int64_t)capacity + row;
        fko_quantize_affine(kr, 1, head_dim, bits, group, ck_packed + o * words, ck_scales + o * groups, ck_biases + o * groups);
        fko_quantize_affine(vr, 1, head_dim, bits, group, cv_packed + o * words, cv_scales + o * groups, cv_biases + o * groups);
    }
    free(kr); free(vr);
}

/* Attention over the quantised cache (sdpa_decode_quant.rs): k_jd = code * scale + bias in fp32,
 * everything else as fko_sdpa_decode. */
FKO_API void fko_sdpa_decode_quant(const uint16_t *q, const uint32_t *ck_packed, const uint16_t *ck_scales,
                                   const uint16_t *ck_biases, const uint32_t *cv_packed, const uint16_t *cv_scales,
                                   const uint16_t *cv_biases, int64_t n_heads, int64_t n_kv, int64_t qk_dim,
                                   int64_t v_dim, uint32_t kv_len, uint32_t capacity, int bits, int group, float scale,
                                   uint16_t *out) {
    const int64_t per_kv = n_heads / n_kv;
    const int per_word = 32 / bits;
    const uint32_t mask = (1u << bits) - 1u;
#pragma omp parallel for schedule(static)
    for (int64_t h = 0; h < n_heads; ++h) {
        const int64_t kvh = h / per_kv;
        float *s = (float *)malloc(sizeof(float) * (size_t)kv_len);
        double *acc = (double *)calloc((size_t)v_dim, sizeof(double));
        float m = -INFINITY;
        for (uint32_t j = 0; j < kv_len; ++j) {
            const int64_t o = kvh * (int64_t)capacity + j;
            double dot = 0.0;
            for (int64_t d = 0; d < qk_dim; ++d) {
                const uint32_t code = (ck_packed[o * (qk_dim / per_word) + d / per_word] >> ((d % per_word) * bits)) & mask;
                const float kd = (float)code * bf16_to_f32(ck_scales[o * (qk_dim / group) + d / group]) +
                                 bf16_to_f32(ck_biases[o * (qk_dim / group) + d / group]);
                dot += (double)bf16_to_f32(q[h * qk_dim + d]) * (double)kd;
            }
            s[j] = (float)dot * scale;
            m = s[j] > m ? s[j] : m;
        }
        double l = 0.0;
        for (uint32_t j = 0; j < kv_len; ++j) {
            const float p = expf(s[j] - m);
            l += (double)p;
            const int64_t o = kvh * (int64_t)capacity + j;
            for (int64_t d = 0; d < v_dim; ++d) {
                const uint32_t code = (cv_packed[o * (v_dim / per_word) + d / per_word] >> ((d % per_word) * bits)) & mask;
                const float vd = (float)code * bf16_to_f32(cv_scales[o * (v_dim / group) + d / group]) +
                                 bf16_to_f32(cv_biases[o * (v_dim / group) + d / group]);
                acc[d] += (double)p * (double)vd;
            }
        }
        for (int64_t d = 0; d < v_dim; ++d) out[h * v_dim + d] = f32_to_bf16((float)(acc[d] / l));
        free(s); free(acc);
    }
}

/* ------------------------------------------------------------ K4: SDPA */
/* s_j = (q . k_j) * scale in fp32; softmax in fp32 (probabilities never
 * rounded to T); o = sum p_j v_j / l; one final round
 * (src/codegen/kernels/sdpa_decode.rs:1064-1211); GQA kv_head = head /
 * (n_heads / n_kv) (:393); caches [n_kv, capacity, dim] (:799,868). */
static void sdpa_decode_core(const float *qf, const uint16_t *cache_k, const uint16_t *cache_v, int64_t n_heads,
                             int64_t n_kv, int64_t qk_dim, int64_t v_dim, uint32_t kv_len, uint32_t capacity,
                             float scale, uint16_t *out) {
    const int64_t per_kv = n_heads / n_kv;
#pragma omp parallel for schedule(static)
    for (int64_t h = 0; h < n_heads; ++h) {
        const int64_t kvh = h / per_kv;
        float *s = (float *)malloc(sizeof(float) * (size_t)kv_len);
        float m = -INFINITY;
        for (uint32_t j = 0; j < kv_len; ++j) {
            const uint16_t *kr = cache_k + (kvh * (int64_t)capacity + j) * qk_dim;
            double dot = 0.0;
            for (int64_t d = 0; d < qk_dim; ++d) dot += (double)qf[h * qk_dim + d] * (double)bf16_to_f32(kr[d]);
            s[j] = (float)dot * scale;
            m = s[j] > m ? s[j] : m;
        }
        double l = 0.0;
        for (uint32_t j = 0; j < kv_len; ++j) {
            s[j] = expf(s[j] - m);
            l += s[j];
        }
        for (int64_t d = 0; d < v_dim; ++d) {
            double o = 0.0;
            for (uint32_t j = 0; j < kv_len; ++j)
                o += (double)s[j] * (double)bf16_to_f32(cache_v[(kvh * (int64_t)capacity + j) * v_dim + d]);
            out[h * v_dim + d] = f32_to_bf16((float)(o / l));
        }
        free(s);
    }
}

FKO_API void fko_sdpa_decode(const uint16_t *q, const uint16_t *cache_k, const uint16_t *cache_v,
                             int64_t n_heads, int64_t n_kv, int64_t qk_dim, int64_t v_dim,
                             uint32_t kv_len, uint32_t capacity, float scale, uint16_t *out) {
    float *qf = (float *)malloc(sizeof(float) * (size_t)(n_heads * qk_dim));
    for (int64_t i = 0; i < n_heads * qk_dim; ++i) qf[i] = bf16_to_f32(q[i]);
    sdpa_decode_core(qf, cache_k, cache_v, n_heads, n_kv, qk_dim, v_dim, kv_len, capacity, scale, out);
    free(qf);
}

/* One element of a rotated slice, written per element as the reference's emitters do
 * (src/codegen/kernels/kv_cache_store_decode.rs:293-331, sdpa_decode.rs:622-652): traditional
 * pairs are (2i, 2i+1), half-split pairs (i, i + half); inv_freq = exp2(-(i/half) * log2 base). */
static float rope_slice_elem(const uint16_t *src, int64_t d1, int64_t rope_dims, int traditional, float base_log2,
                             uint32_t pos) {
    const int64_t half = rope_dims / 2;
    const int64_t pair = traditional ? d1 / 2 : (d1 < half ? d1 : d1 - half);
    const float d_norm = (float)pair / (float)half;
    const float inv_freq = exp2f(-d_norm * base_log2);
    const float angle = (float)pos * inv_freq;
    const float c = cosf(angle), sn = sinf(angle);
    const int64_t lo_idx = traditional ? pair * 2 : pair, hi_idx = traditional ? lo_idx + 1 : pair + half;
    const float lo = bf16_to_f32(src[lo_idx]), hi = bf16_to_f32(src[hi_idx]);
    const int lo_lane = traditional ? (d1 & 1) == 0 : d1 < half;
    return lo_lane ? lo * c - hi * sn : hi * c + lo * sn;
}

/* Attention with the query given as two parts, Q = [Q0 | Q1] per head, Q1 rotated inside the
 * kernel at position kv_len - 1 and kept in fp32 -- never rounded to T -- before the dot products
 * (src/codegen/kernels/sdpa_decode.rs:283-294 buffers, :592-660 staging); the rest as
 * fko_sdpa_decode.  q0 / q1 rows are q0_stride / q1_stride elements apart (one packed
 * [n_heads, q0_dim + q1_dim] tensor: q1 = q0 + q0_dim, both strides q0_dim + q1_dim). */
FKO_API void fko_sdpa_decode_split_q(const uint16_t *q0, int64_t q0_stride, const uint16_t *q1, int64_t q1_stride,
                                     int64_t q0_dim, int64_t q1_dim, int64_t rope_dims, int traditional, float theta,
                                     const uint16_t *cache_k, const uint16_t *cache_v, int64_t n_heads, int64_t n_kv,
                                     int64_t v_dim, uint32_t kv_len, uint32_t capacity, float scale, uint16_t *out) {
    const int64_t qk_dim = q0_dim + q1_dim;
    const float base_log2 = (float)log2((double)theta);
    const uint32_t pos = kv_len > 0 ? kv_len - 1 : 0;
    float *qf = (float *)malloc(sizeof(float) * (size_t)(n_heads * qk_dim));
    for (int64_t h = 0; h < n_heads; ++h)
        for (int64_t d = 0; d < qk_dim; ++d) {
            float v;
            if (d < q0_dim)
                v = bf16_to_f32(q0[h * q0_stride + d]);
            else if (d - q0_dim >= rope_dims)
                v = bf16_to_f32(q1[h * q1_stride + d - q0_dim]);
            else
                v = rope_slice_elem(q1 + h * q1_stride, d - q0_dim, rope_dims, traditional, base_log2, pos);
            qf[h * qk_dim + d] = v;
        }
    sdpa_decode_core(qf, cache_k, cache_v, n_heads, n_kv, qk_dim, v_dim, kv_len, capacity, scale, out);
    free(qf);
}

/* Cache store of a key given as two parts: cache K row = [K0 | K1]; K1 has n_kv heads or ONE
 * head shared by all (MLA's rotary key) and its first rope_dims are rotated at `pos` while it is
 * written; K0 and V rows are k0_stride / v_stride elements apart, so both may alias one packed
 * [n_kv, k0_dim + v_dim] tensor (src/codegen/kernels/kv_cache_store_decode.rs:268-352; packed
 * source :103-140). */
FKO_API void fko_kv_store_split(const uint16_t *k0, int64_t k0_stride, const uint16_t *k1, int64_t k1_heads,
                                const uint16_t *v, int64_t v_stride, int64_t n_kv, int64_t k0_dim, int64_t k1_dim,
                                int64_t v_dim, int64_t rope_dims, int traditional, float theta, uint32_t pos,
                                uint32_t write_offset, uint32_t capacity, uint16_t *cache_k, uint16_t *cache_v) {
    const float base_log2 = (float)log2((double)theta);
    const int64_t row = write_offset % capacity, k_dim = k0_dim + k1_dim;
    for (int64_t h = 0; h < n_kv; ++h) {
        uint16_t *ck = cache_k + (h * (int64_t)capacity + row) * k_dim;
        uint16_t *cv = cache_v + (h * (int64_t)capacity + row) * v_dim;
        const uint16_t *k1h = k1 + (k1_heads == 1 ? 0 : h) * k1_dim;
        for (int64_t d = 0; d < k0_dim; ++d) ck[d] = k0[h * k0_stride + d];
        for (int64_t d1 = 0; d1 < k1_dim; ++d1)
            ck[k0_dim + d1] = d1 >= rope_dims ? k1h[d1]
                                              : f32_to_bf16(rope_slice_elem(k1h, d1, rope_dims, traditional, base_log2, pos));
        for (int64_t d = 0; d < v_dim; ++d) cv[d] = v[h * v_stride + d];
    }
}

/* Router of a mixture-of-experts block: softmax over ROW_N logits, the top_k largest in
 * descending order, ties to the lower index (src/codegen/kernels/single.rs:2615-2760):
 * row_max and sum in fp32, prob = float(T(exp(score - row_max) * (1 / sum))) -- rounded to T
 * BEFORE the sort (:2707-2709) -- sort key (-prob, index) (:2726-2728), weight = T(prob * scale)
 * with one scale for the row or one per route (:2748-2750). */
FKO_API void fko_softmax_topk_route(const uint16_t *logits, int64_t rows, int64_t row_n, int64_t top_k,
                                    const uint16_t *scale, int scale_per_route, uint32_t *idx, uint16_t *weight) {
    float *prob = (float *)malloc(sizeof(float) * (size_t)row_n);
    char *taken = (char *)malloc((size_t)row_n);
    for (int64_t r = 0; r < rows; ++r) {
        const uint16_t *l = logits + r * row_n;
        float m = -INFINITY;
        for (int64_t i = 0; i < row_n; ++i) m = bf16_to_f32(l[i]) > m ? bf16_to_f32(l[i]) : m;
        double sum = 0.0;
        for (int64_t i = 0; i < row_n; ++i) sum += (double)expf(bf16_to_f32(l[i]) - m);
        const float inv = 1.0f / (float)sum;
        for (int64_t i = 0; i < row_n; ++i) {
            prob[i] = bf16_to_f32(f32_to_bf16(expf(bf16_to_f32(l[i]) - m) * inv));
            taken[i] = 0;
        }
        for (int64_t k = 0; k < top_k; ++k) {   /* selection = the first top_k of the (-prob, index) order */
            int64_t best = -1;
            for (int64_t i = 0; i < row_n; ++i)
                if (!taken[i] && (best < 0 || prob[i] > prob[best])) best = i;
            taken[best] = 1;
            const float sc = bf16_to_f32(scale[scale_per_route ? r * top_k + k : 0]);
            idx[r * top_k + k] = (uint32_t)best;
            weight[r * top_k + k] = f32_to_bf16(prob[best] * sc);
        }
    }
    free(prob);
    free(taken);
}

/* Causal attention of a group of L rows (src/codegen/kernels/sdpa_prefill.rs): row l_q sits at
 * q_kv = (kv_len - L) + l_q and positions kv > q_kv are masked (:95, :109); scores dot * SCALE
 * (:104-124); max, exp, sum, then the scores are normalised BEFORE the product with V
 * (:128-181); out = T(sum_kv score * v) (:183-199).  q, out [L, n_heads, dim]. */
FKO_API void fko_sdpa_prefill(const uint16_t *q, const uint16_t *cache_k, const uint16_t *cache_v, int64_t rows,
                              int64_t n_heads, int64_t n_kv, int64_t dim, uint32_t kv_len, uint32_t capacity,
                              float scale, uint16_t *out) {
    const int64_t per_kv = n_heads / n_kv;
#pragma omp parallel for schedule(dynamic)
    for (int64_t it = 0; it < rows * n_heads; ++it) {
        const int64_t l_q = it / n_heads, h = it % n_heads, kvh = h / per_kv;
        const uint32_t q_kv = (kv_len - (uint32_t)rows) + (uint32_t)l_q;
        const uint16_t *qr = q + (l_q * n_heads + h) * dim;
        float *s = (float *)malloc(sizeof(float) * (size_t)(q_kv + 1));
        float m = -INFINITY;
        for (uint32_t j = 0; j <= q_kv; ++j) { /* kv > q_kv: exp(-inf) = 0, contributes nothing */
            const uint16_t *kr = cache_k + (kvh * (int64_t)capacity + j) * dim;
            double dot = 0.0;
            for (int64_t d = 0; d < dim; ++d) dot += (double)bf16_to_f32(qr[d]) * (double)bf16_to_f32(kr[d]);
            s[j] = (float)dot * scale;
            m = s[j] > m ? s[j] : m;
        }
        double l = 0.0;
        for (uint32_t j = 0; j <= q_kv; ++j) {
            s[j] = expf(s[j] - m);
            l += s[j];
        }
        const float inv = 1.0f / (float)l;
        for (uint32_t j = 0; j <= q_kv; ++j) s[j] *= inv;
        for (int64_t d = 0; d < dim; ++d) {
            double o = 0.0;
            for (uint32_t j = 0; j <= q_kv; ++j)
                o += (double)s[j] * (double)bf16_to_f32(cache_v[(kvh * (int64_t)capacity + j) * dim + d]);
            out[(l_q * n_heads + h) * dim + d] = f32_to_bf16((float)o);
        }
        free(s);
    }
}

/* -------------------------------------------------------- E / H / A / U */
/* x = T(embed[token] * scale) (src/codegen/kernels/embed_lookup_decode.rs:74-99). */
FKO_API void fko_embed_lookup(const fko_weight *E, uint32_t token, float out_scale, uint16_t *x) {
    const int64_t k = E->k;
    if (E->bits == 16) {
        const uint16_t *row = (const uint16_t *)E->w + (int64_t)token * k;
        for (int64_t d = 0; d < k; ++d) x[d] = f32_to_bf16(bf16_to_f32(row[d]) * out_scale);
        return;
    }
    const int bits = E->bits, per_word = 32 / bits;
    const uint32_t mask = (1u << bits) - 1u;
    const int64_t words = k / per_word, groups = k / E->group;
    const uint32_t *p = (const uint32_t *)E->w + (int64_t)token * words;
    for (int64_t d = 0; d < k; ++d) {
        uint32_t qv = (p[d / per_word] >> ((d % per_word) * bits)) & mask;
        float s = bf16_to_f32(E->scales[(int64_t)token * groups + d / E->group]);
        float b = bf16_to_f32(E->biases[(int64_t)token * groups + d / E->group]);
        x[d] = f32_to_bf16(((float)qv * s + b) * out_scale);
    }
}

/* Final RMSNorm + vocabulary GEMV, logits rounded to T
 * (src/codegen/kernels/final_rmsnorm_lm_head.rs:225-330). */
FKO_API void fko_final_rmsnorm_lm_head(const uint16_t *x, const uint16_t *norm_w, float eps,
                                       const fko_weight *W, uint16_t *logits) {
    float *ny = (float *)malloc(sizeof(float) * (size_t)W->k);
    float *acc = (float *)malloc(sizeof(float) * (size_t)W->n);
    rmsnorm_f(x, norm_w, W->k, eps, ny);
    linear_acc(W, ny, acc);
    for (int64_t i = 0; i < W->n; ++i) logits[i] = f32_to_bf16(acc[i]);
    free(ny);
    free(acc);
}

/* Greedy argmax, lowest index wins ties; a NaN never wins (v > max is false)
 * (src/codegen/kernels/argmax_logits_decode.rs:63-95). */
FKO_API uint32_t fko_argmax(const uint16_t *logits, int64_t n) {
    float best = -INFINITY;
    uint32_t idx = 0;
    for (int64_t i = 0; i < n; ++i) {
        float v = bf16_to_f32(logits[i]);
        if (v > best) {
            best = v;
            idx = (uint32_t)i;
        }
    }
    return idx;
}

/* top-1 minus top-2 logit (0 on an exact tie): the margin the token-identity
 * test logs per step. */
FKO_API float fko_top2_margin(const uint16_t *logits, int64_t n) {
    float a = -INFINITY, b = -INFINITY;
    for (int64_t i = 0; i < n; ++i) {
        float v = bf16_to_f32(logits[i]);
        if (v > a) {
            b = a;
            a = v;
        } else if (v > b) {
            b = v;
        }
    }
    return a - b;
}

/* ------------------------------------------------------- M1 / M2: MoE */
/*
 * Stacked expert weights: packed u32 [E, O, K*bits/32], scales / biases T [E, O, K/group]
 * (src/codegen/kernels/routed_qmv_swiglu.rs:44-61).  Route r = tok * top_k + slot reads
 * activation row row_idx[r] and expert expert_idx[r] (clamped to E-1, :128-139).
 *
 * M1 (routed_qmv_swiglu.rs:420-446): g = T(acc_gate), u = T(acc_up),
 *    sig = 1 / (1 + exp(-g)) in fp32, out0[r, o] = T(((sig * g) * u) * rw_r)
 *    with rw_r = route_weight[r] when pre-scaling, else 1.
 */
static fko_weight expert_slice(const fko_weight *W, int64_t e) {
    fko_weight s = *W;
    const int64_t per_word = 32 / W->bits;
    s.w = (const uint32_t *)W->w + e * W->n * (W->k / per_word);
    if (W->scales) {
        s.scales = W->scales + e * W->n * (W->k / W->group);
        s.biases = W->biases + e * W->n * (W->k / W->group);
    }
    return s;
}

FKO_API void fko_routed_qmv_swiglu(const uint16_t *x, const fko_weight *Wg, const fko_weight *Wu,
                                   int64_t n_experts, const uint32_t *row_idx, const uint32_t *expert_idx,
                                   const uint16_t *route_weight /* or NULL */, int64_t n_routes, uint16_t *out0) {
    const int64_t K = Wg->k, O = Wg->n;
    float *xf = (float *)malloc(sizeof(float) * (size_t)K);
    float *ag = (float *)malloc(sizeof(float) * (size_t)O), *au = (float *)malloc(sizeof(float) * (size_t)O);
    for (int64_t r = 0; r < n_routes; ++r) {
        int64_t e = expert_idx[r];
        if (e > n_experts - 1) e = n_experts - 1;
        const fko_weight g = expert_slice(Wg, e), u = expert_slice(Wu, e);
        for (int64_t j = 0; j < K; ++j) xf[j] = bf16_to_f32(x[(int64_t)row_idx[r] * K + j]);
        linear_acc(&g, xf, ag);
        linear_acc(&u, xf, au);
        const float rw = route_weight ? bf16_to_f32(route_weight[r]) : 1.0f;
        for (int64_t o = 0; o < O; ++o) {
            const float gv = rbf(ag[o]), uv = rbf(au[o]);
            const float sig = 1.0f / (1.0f + expf(-gv));
            out0[r * O + o] = f32_to_bf16(((sig * gv) * uv) * rw);
        }
    }
    free(xf); free(ag); free(au);
}

/* M2 (routed_qmv_reduce.rs:240, 315-322, 422-434): per token, slots in order,
 *    acc += rw_r * float(T(dot_r))   (rw_r = 1 when the input was pre-weighted),
 *    acc += residual_extra[tok, o] when present; out[tok, o] = T(acc).
 *    dot_r = W_down[expert_r] . h[r, :]  with h = M1's out0. */
FKO_API void fko_routed_qmv_reduce(const uint16_t *h, const fko_weight *Wd, int64_t n_experts,
                                   const uint32_t *row_idx /* or NULL */, const uint32_t *expert_idx,
                                   const uint16_t *route_weight /* or NULL */, const uint16_t *shared_x /* or NULL */,
                                   const fko_weight *Wshared /* or NULL */,
                                   const uint16_t *residual_extra /* or NULL */, int64_t n_tokens, int64_t top_k,
                                   uint16_t *out) {
    const int64_t K = Wd->k, O = Wd->n;
    const int64_t xk = (Wshared && Wshared->k > K) ? Wshared->k : K;
    float *xf = (float *)malloc(sizeof(float) * (size_t)xk);
    float *dot = (float *)malloc(sizeof(float) * (size_t)O);
    float *acc = (float *)malloc(sizeof(float) * (size_t)O);
    for (int64_t t = 0; t < n_tokens; ++t) {
        for (int64_t o = 0; o < O; ++o) acc[o] = 0.0f;
        for (int64_t sl = 0; sl < top_k; ++sl) {
            const int64_t r = t * top_k + sl;
            int64_t e = expert_idx[r];
            if (e > n_experts - 1) e = n_experts - 1;
            const fko_weight d = expert_slice(Wd, e);
            const int64_t row = row_idx ? (int64_t)row_idx[r] : r;
            for (int64_t j = 0; j < K; ++j) xf[j] = bf16_to_f32(h[row * K + j]);
            linear_acc(&d, xf, dot);
            const float rw = route_weight ? bf16_to_f32(route_weight[r]) : 1.0f;
            for (int64_t o = 0; o < O; ++o) {
                const float partial = rw * rbf(dot[o]);
                acc[o] += partial;
            }
        }
        if (Wshared) { /* routed_qmv_reduce.rs:250-307: one more partial, T(dot) of the shared expert */
            for (int64_t j = 0; j < Wshared->k; ++j) xf[j] = bf16_to_f32(shared_x[t * Wshared->k + j]);
            linear_acc(Wshared, xf, dot);
            for (int64_t o = 0; o < O; ++o) acc[o] += rbf(dot[o]);
        }
        for (int64_t o = 0; o < O; ++o) {
            float a = acc[o];
            if (residual_extra) a += bf16_to_f32(residual_extra[t * O + o]);
            out[t * O + o] = f32_to_bf16(a);
        }
    }
    free(xf); free(dot); free(acc);
}

/* G: multi-row quantised matmul y[M, N] = T(x[M, K] @ dequant(W)^T (+ bias)), the row-wise
 *    repetition of K1 (qMM-T semantics, src/codegen/msl.rs:2318-2440: fp32 accumulate, one round). */
FKO_API void fko_qgemm(const fko_weight *W, const uint16_t *x, int64_t m, const uint16_t *bias, uint16_t *y) {
    for (int64_t r = 0; r < m; ++r) fko_qgemv(W, x + r * W->k, bias, y + r * W->n);
}

/* G, large-M form: the reference's multi-row kernels dequantise a tile of weights into the
 *    activation type before the multiply (msl.rs:2318-2440: QuantizedBlockLoader of MLX fills a
 *    threadgroup tile of T), i.e. w = T(s * q + b), one bf16 rounding per weight element, then
 *    y[M, N] = T(x @ w^T (+ bias)) with fp32 accumulation.  `acc_out` (optional) receives the
 *    unrounded sums. */
FKO_API void fko_qgemm_bf16w(const fko_weight *W, const uint16_t *x, int64_t m, const uint16_t *bias, uint16_t *y,
                             float *acc_out) {
    const int64_t N = W->n, K = W->k;
    const int per_word = 32 / W->bits;
    const uint32_t mask = (1u << W->bits) - 1u;
#pragma omp parallel for schedule(static)
    for (int64_t n = 0; n < N; ++n) {
        float *w = (float *)malloc(sizeof(float) * (size_t)K);
        for (int64_t k = 0; k < K; ++k) {
            const uint32_t q = (((const uint32_t *)W->w)[n * (K / per_word) + k / per_word] >> ((k % per_word) * W->bits)) & mask;
            const float s = bf16_to_f32(W->scales[n * (K / W->group) + k / W->group]);
            const float b = bf16_to_f32(W->biases[n * (K / W->group) + k / W->group]);
            w[k] = rbf(fmaf((float)q, s, b));
        }
        for (int64_t r = 0; r < m; ++r) {
            double acc = 0.0;
            for (int64_t k = 0; k < K; ++k) acc += (double)bf16_to_f32(x[r * K + k]) * (double)w[k];
            float a = (float)acc;
            if (acc_out) acc_out[r * N + n] = a;
            if (bias) a += bf16_to_f32(bias[n]);
            y[r * N + n] = f32_to_bf16(a);
        }
        free(w);
    }
}

/* --------------------------------------------------- dense decoder step */
/*
 * One decode step of the dense decoder in the reference's decode_pipeline
 * order (src/codegen/task_graph_json.rs:54-65; per-token protocol
 * python_runtime/src/lib.rs:1181-1226):
 *   embed -> L x [ rmsnorm_qkv | (head-norm +) rope_q | (head-norm +) rope_k +
 *   kv store | sdpa | o_proj + residual | rmsnorm gate/up swiglu | down +
 *   residual ] -> final norm + lm head -> argmax.
 */
typedef struct {
    const uint16_t *input_norm, *post_norm; /* [hidden] */
    fko_weight wq, wk, wv, wo, wgate, wup, wdown;
    const uint16_t *bq, *bk, *bv;       /* optional projection biases */
    const uint16_t *q_norm, *k_norm;    /* optional per-head norms [head_dim] */
    uint16_t *cache_k, *cache_v;        /* [n_kv, capacity, head_dim] */
    /* quantised cache (model kv_bits != 0): packed [n_kv, capacity, head_dim*bits/32], scales / biases
     * [n_kv, capacity, head_dim/group] */
    uint32_t *ck_packed; uint16_t *ck_scales, *ck_biases;
    uint32_t *cv_packed; uint16_t *cv_scales, *cv_biases;
} fko_layer;

typedef struct {
    int64_t n_layers, hidden, n_heads, n_kv, head_dim, inter, vocab;
    float eps, theta, attn_scale, embed_scale;
    int swiglu_variant;
    uint32_t capacity;
    fko_weight embed;   /* [vocab, hidden] */
    fko_weight lm_head; /* [vocab, hidden]; may alias embed (tied) */
    const uint16_t *final_norm;
    const fko_layer *layers;
    int kv_bits, kv_group; /* 0: bf16 cache */
} fko_model;

FKO_API uint32_t fko_decoder_step(const fko_model *M, uint32_t token, uint32_t offset,
                                  uint16_t *logits_out /* [vocab] or NULL */, float *margin_out) {
    const int64_t H = M->hidden, NQ = M->n_heads * M->head_dim, NKV = M->n_kv * M->head_dim;
    uint16_t *x = (uint16_t *)malloc(2 * (size_t)H), *x2 = (uint16_t *)malloc(2 * (size_t)H);
    uint16_t *q = (uint16_t *)malloc(2 * (size_t)NQ), *k = (uint16_t *)malloc(2 * (size_t)NKV);
    uint16_t *v = (uint16_t *)malloc(2 * (size_t)NKV), *att = (uint16_t *)malloc(2 * (size_t)NQ);
    uint16_t *mid = (uint16_t *)malloc(2 * (size_t)M->inter);
    fko_embed_lookup(&M->embed, token, M->embed_scale, x);
    for (int64_t l = 0; l < M->n_layers; ++l) {
        const fko_layer *L = &M->layers[l];
        fko_rmsnorm_qkv(x, L->input_norm, M->eps, &L->wq, &L->wk, &L->wv, L->bq, L->bk, L->bv, q, k, v);
        if (M->kv_bits) {
            if (L->q_norm) fko_headnorm_rope(q, L->q_norm, M->n_heads, M->head_dim, M->head_dim, M->eps, M->theta, offset);
            else fko_rope_q(q, M->n_heads, M->head_dim, M->head_dim, M->theta, offset);
            fko_rope_kv_store_quant(k, v, L->k_norm, M->n_kv, M->head_dim, M->head_dim, M->theta, M->eps, offset, offset,
                                    M->capacity, M->kv_bits, M->kv_group, L->ck_packed, L->ck_scales, L->ck_biases,
                                    L->cv_packed, L->cv_scales, L->cv_biases);
        } else if (L->q_norm) {
            fko_headnorm_rope(q, L->q_norm, M->n_heads, M->head_dim, M->head_dim, M->eps, M->theta, offset);
            fko_headnorm_rope(k, L->k_norm, M->n_kv, M->head_dim, M->head_dim, M->eps, M->theta, offset);
            fko_kv_store(k, v, M->n_kv, M->head_dim, M->head_dim, offset, M->capacity, L->cache_k, L->cache_v);
        } else {
            fko_rope_q(q, M->n_heads, M->head_dim, M->head_dim, M->theta, offset);
            fko_rope_kv_store(k, v, M->n_kv, M->head_dim, M->head_dim, M->theta, offset, offset, M->capacity,
                              L->cache_k, L->cache_v);
        }
        if (M->kv_bits)
            fko_sdpa_decode_quant(q, L->ck_packed, L->ck_scales, L->ck_biases, L->cv_packed, L->cv_scales, L->cv_biases,
                                  M->n_heads, M->n_kv, M->head_dim, M->head_dim, offset + 1, M->capacity, M->kv_bits,
                                  M->kv_group, M->attn_scale, att);
        else
            fko_sdpa_decode(q, L->cache_k, L->cache_v, M->n_heads, M->n_kv, M->head_dim, M->head_dim, offset + 1,
                            M->capacity, M->attn_scale, att);
        fko_linear_residual(&L->wo, att, x, NULL, x2);
        fko_gateup_swiglu(x2, L->post_norm, M->eps, &L->wgate, &L->wup, M->swiglu_variant, mid);
        fko_linear_residual(&L->wdown, mid, x2, NULL, x);
    }
    uint16_t *logits = logits_out ? logits_out : (uint16_t *)malloc(2 * (size_t)M->vocab);
    fko_final_rmsnorm_lm_head(x, M->final_norm, M->eps, &M->lm_head, logits);
    uint32_t next = fko_argmax(logits, M->vocab);
    if (margin_out) *margin_out = fko_top2_margin(logits, M->vocab);
    if (!logits_out) free(logits);
    free(x); free(x2); free(q); free(k); free(v); free(att); free(mid);
    return next;
}
