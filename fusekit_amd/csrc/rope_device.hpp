// Per-head transform shared by the rope/store kernel and the fused attention
// phase: optional RMSNorm with the reference's two roundings, T(w * T(x * r)),
// then half-split RoPE on the first rope_dims of the head.  One wave per head.
#pragma once
#include "fk_device.hpp"

namespace fk {

__device__ __forceinline__ void rope_rotate(float lo, float hi, uint32_t d, uint32_t half, uint32_t pos,
                                            float base_log2, float& olo, float& ohi) {
    // inv = exp2(-(d/half) * log2(theta)); angle = pos * inv (reference rope_q_decode.rs:93-114)
    const float d_norm = (float)d / (float)half;
    // The fp32 exponent is rounded like the reference's; 2^t itself goes through
    // double so that the fp32 frequency is the correctly rounded one on every
    // platform (an ulp of inv_freq is 2.5e-3 rad at position 32767).
    const float inv_freq = (float)exp2((double)(-d_norm * base_log2));
    const float angle = (float)pos * inv_freq;
    float sn, cs;
    sincosf(angle, &sn, &cs);
    olo = lo * cs - hi * sn;
    ohi = hi * cs + lo * sn;
}

// src -> dst (may alias: every pair is read and written by one lane).  `copy_tail`
// writes the dims outside the rotation too (needed when dst != src or when the
// norm changed them).
// (cos, sin) of pair d at this position: the value rope_rotate would compute, so a
// table filled once per token gives bit-identical rotations in every layer.
__device__ __forceinline__ void rope_cos_sin(uint32_t d, uint32_t half, uint32_t pos, float base_log2, float& cs,
                                             float& sn) {
    const float d_norm = (float)d / (float)half;
    const float inv_freq = (float)exp2((double)(-d_norm * base_log2));
    sincosf((float)pos * inv_freq, &sn, &cs);
}

// `tab` (optional): interleaved (cos, sin) per pair, as rope_cos_sin fills it.
__device__ __forceinline__ void head_transform(const uint16_t* src, uint16_t* dst, const uint16_t* nw, uint32_t dim,
                                               uint32_t rope_dims, uint32_t pos, float base_log2, float eps,
                                               bool copy_tail, uint32_t lane, const float* tab = nullptr) {
    float r = 1.f;
    if (nw) {
        float ss = 0.f;
        for (uint32_t d = lane; d < dim; d += kWave) {
            const float x = bf16_bits_to_f32(src[d]);
            ss = fmaf(x, x, ss);
        }
        ss = wave_sum(ss);
        r = 1.0f / sqrtf(ss / (float)dim + eps);
    }
    auto value = [&](uint32_t d) {
        const float x = bf16_bits_to_f32(src[d]);
        return nw ? round_bf16(bf16_bits_to_f32(nw[d]) * round_bf16(x * r)) : x;
    };
    const uint32_t half = rope_dims / 2;
    for (uint32_t d = lane; d < half; d += kWave) {
        float lo, hi;
        if (tab) {
            const float vlo = value(d), vhi = value(d + half), cs = tab[2 * d], sn = tab[2 * d + 1];
            lo = vlo * cs - vhi * sn;
            hi = vhi * cs + vlo * sn;
        } else {
            rope_rotate(value(d), value(d + half), d, half, pos, base_log2, lo, hi);
        }
        dst[d] = (uint16_t)f32_to_bf16_bits(lo);
        dst[d + half] = (uint16_t)f32_to_bf16_bits(hi);
    }
    if (copy_tail)
        for (uint32_t d = 2 * half + lane; d < dim; d += kWave) dst[d] = (uint16_t)f32_to_bf16_bits(value(d));
}

// A head given as two parts: dst = [p0 (d0 dims) | p1 (d1 dims)], the first rope_dims of p1 rotated as
// traditional (2i, 2i+1) or half-split (i, i + rope_dims / 2) pairs at `pos`; `tab` as in head_transform.
// The arithmetic of the split-key cache store (mla.hip), for the attention kernel that appends the new
// row itself.
__device__ __forceinline__ void split_head_transform(const uint16_t* p0, const uint16_t* p1, uint16_t* dst, uint32_t d0,
                                                     uint32_t d1, uint32_t rope_dims, bool traditional, uint32_t pos,
                                                     float base_log2, uint32_t lane, const float* tab) {
    for (uint32_t d = lane; d < d0; d += kWave) dst[d] = p0[d];
    const uint32_t half = rope_dims / 2;
    uint16_t* o = dst + d0;
    for (uint32_t i = lane; i < half; i += kWave) {
        const uint32_t lo_i = traditional ? 2 * i : i, hi_i = traditional ? 2 * i + 1 : i + half;
        const float xl = bf16_bits_to_f32(p1[lo_i]), xh = bf16_bits_to_f32(p1[hi_i]);
        float lo, hi;
        if (tab) {
            const float cs = tab[2 * i], sn = tab[2 * i + 1];
            lo = xl * cs - xh * sn;
            hi = xh * cs + xl * sn;
        } else {
            rope_rotate(xl, xh, i, half, pos, base_log2, lo, hi);
        }
        o[lo_i] = (uint16_t)f32_to_bf16_bits(lo);
        o[hi_i] = (uint16_t)f32_to_bf16_bits(hi);
    }
    for (uint32_t d = 2 * half + lane; d < d1; d += kWave) o[d] = p1[d];
}

// The same transform for a head that is rotated over its whole width of at most 128 dims, split
// in two so that a caller can put other memory requests between the loads and their use: lane
// d < half owns the pair (d, d + half); head_pair_fetch issues every load (raw values, norm weights,
// table entry), head_pair_apply does the arithmetic of head_transform on them.
struct HeadPair {
    float xlo, xhi, wlo, whi, cs, sn;
};

__device__ __forceinline__ HeadPair head_pair_fetch(const uint16_t* src, const uint16_t* nw, const float* tab,
                                                    uint32_t half, uint32_t lane) {
    const uint32_t d = lane < half ? lane : 0u;
    const uint16_t* w = nw ? nw : src;  // no norm: a harmless load instead of a branch around one
    HeadPair p;
    p.xlo = bf16_bits_to_f32(src[d]);
    p.xhi = bf16_bits_to_f32(src[d + half]);
    p.wlo = bf16_bits_to_f32(w[d]);
    p.whi = bf16_bits_to_f32(w[d + half]);
    p.cs = tab[2 * d];
    p.sn = tab[2 * d + 1];
    return p;
}

__device__ __forceinline__ void head_pair_apply(const HeadPair& p, uint16_t* dst, bool has_norm, uint32_t half,
                                                float eps, uint32_t lane, bool write) {
    float vlo = p.xlo, vhi = p.xhi;
    if (has_norm) {
        float ss = lane < half ? fmaf(p.xhi, p.xhi, fmaf(p.xlo, p.xlo, 0.f)) : 0.f;
        ss = wave_sum(ss);
        const float r = 1.0f / sqrtf(ss / (float)(2 * half) + eps);
        vlo = round_bf16(p.wlo * round_bf16(p.xlo * r));
        vhi = round_bf16(p.whi * round_bf16(p.xhi * r));
    }
    const float lo = vlo * p.cs - vhi * p.sn;
    const float hi = vhi * p.cs + vlo * p.sn;
    if (write && lane < half) {
        dst[lane] = (uint16_t)f32_to_bf16_bits(lo);
        dst[lane + half] = (uint16_t)f32_to_bf16_bits(hi);
    }
}

}  // namespace fk
