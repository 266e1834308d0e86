// Softmax top-k route of one row of router logits inside a wave: the arithmetic of the reference's
// SoftmaxTopKRoute (src/codegen/kernels/single.rs:2615-2760), shared by the stand-alone router kernels and
// by the expert kernel that routes for itself.  Lane l holds logits l, l + 64, l + 128, l + 192.
//
// A candidate is one 32-bit key: the probability, already rounded to bf16 (its low 16 bits are zero, and a
// non-negative float orders like its bit pattern), with 256 - index in the low bits.  The largest key is the
// largest probability and, among equal ones, the lowest index -- the reference's sort key (-prob, index) --
// so one round of the selection is a local maximum and one integer wave maximum over DPP row operations
// (no LDS-crossbar shuffles: six rounds of those cost 3 us).  0 marks "no candidate".
#pragma once
#include "fk_device.hpp"

namespace fk {

template <int CTRL>
__device__ __forceinline__ uint32_t dpp_umax(uint32_t v) {
    const uint32_t moved = (uint32_t)__builtin_amdgcn_update_dpp((int)v, (int)v, CTRL, 0xF, 0xF, false);
    return v > moved ? v : moved;
}
// All 64 lanes active; every lane returns the maximum.
__device__ __forceinline__ uint32_t wave_umax(uint32_t v) {
    v = dpp_umax<0xB1>(v);
    v = dpp_umax<0x4E>(v);
    v = dpp_umax<0x141>(v);
    v = dpp_umax<0x140>(v);
    const uint32_t r0 = (uint32_t)__builtin_amdgcn_readlane((int)v, 0), r1 = (uint32_t)__builtin_amdgcn_readlane((int)v, 16);
    const uint32_t r2 = (uint32_t)__builtin_amdgcn_readlane((int)v, 32), r3 = (uint32_t)__builtin_amdgcn_readlane((int)v, 48);
    const uint32_t a = r0 > r1 ? r0 : r1, b = r2 > r3 ? r2 : r3;
    return a > b ? a : b;
}

// x[j] = logit of expert lane + 64 j (any value beyond n) -> key[j] of float(T(exp(x - max) / sum)), 0 beyond n.
__device__ __forceinline__ void route_candidates(const float (&x)[4], uint32_t n, uint32_t lane, uint32_t (&key)[4]) {
    float m = -INFINITY;
#pragma unroll
    for (uint32_t j = 0; j < 4; ++j) m = lane + j * kWave < n ? fmaxf(m, x[j]) : m;
    m = wave_max(m);
    float p[4];
    float sum = 0.f;
#pragma unroll
    for (uint32_t j = 0; j < 4; ++j) {
        p[j] = lane + j * kWave < n ? expf(x[j] - m) : 0.f;
        sum += p[j];
    }
    sum = wave_sum(sum);
    const float inv = 1.0f / sum;
#pragma unroll
    for (uint32_t j = 0; j < 4; ++j) {
        const uint32_t i = lane + j * kWave;
        key[j] = i < n ? (__float_as_uint(round_bf16(p[j] * inv)) | (256u - i)) : 0u;
    }
}

// The best remaining candidate, removed from the set; uniform result (probability as float, expert index).
__device__ __forceinline__ void route_take_best(uint32_t (&key)[4], float& best, uint32_t& best_i) {
    uint32_t k = key[0] > key[1] ? key[0] : key[1];
    const uint32_t k2 = key[2] > key[3] ? key[2] : key[3];
    k = wave_umax(k > k2 ? k : k2);
#pragma unroll
    for (uint32_t j = 0; j < 4; ++j) key[j] = key[j] == k ? 0u : key[j];
    best = __uint_as_float(k & 0xffff0000u);
    best_i = 256u - (k & 0x1ffu);
}

}  // namespace fk
