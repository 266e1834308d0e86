// Softmax top-k route of one row of router logits inside a wave: the arithmetic of the reference's
// SoftmaxTopKRoute (src/codegen/kernels/single.rs:2615-2760), shared by the stand-alone router kernels and
// by the expert kernel that routes for itself.  Lane l holds logits l, l + 64, l + 128, l + 192.
#pragma once
#include "fk_device.hpp"

namespace fk {

// x[j] = logit of expert lane + 64 j (any value beyond n) -> p[j] = float(T(exp(x - max) / sum)), -1 beyond n.
__device__ __forceinline__ void route_probabilities(const float (&x)[4], uint32_t n, uint32_t lane, float (&p)[4]) {
    float m = -INFINITY;
#pragma unroll
    for (uint32_t j = 0; j < 4; ++j) m = lane + j * kWave < n ? fmaxf(m, x[j]) : m;
    m = wave_max(m);
    float sum = 0.f;
#pragma unroll
    for (uint32_t j = 0; j < 4; ++j) {
        p[j] = lane + j * kWave < n ? expf(x[j] - m) : 0.f;
        sum += p[j];
    }
    sum = wave_sum(sum);
    const float inv = 1.0f / sum;
#pragma unroll
    for (uint32_t j = 0; j < 4; ++j) p[j] = lane + j * kWave < n ? round_bf16(p[j] * inv) : -1.f;  // -1: not a candidate
}

// The largest remaining probability (ties to the lower index), removed from the candidates; uniform result.
__device__ __forceinline__ void route_take_best(float (&p)[4], uint32_t lane, float& best, uint32_t& best_i) {
    best = -1.f;
    best_i = 0xffffffffu;
#pragma unroll
    for (uint32_t j = 0; j < 4; ++j)   // ascending index within the lane: '>' keeps the lower one on ties
        if (p[j] > best) {
            best = p[j];
            best_i = lane + j * kWave;
        }
#pragma unroll
    for (uint32_t off = 1; off < kWave; off <<= 1) {
        const float ob = __shfl_xor(best, off, kWave);
        const uint32_t oi = __shfl_xor(best_i, off, kWave);
        if (ob > best || (ob == best && oi < best_i)) {
            best = ob;
            best_i = oi;
        }
    }
#pragma unroll
    for (uint32_t j = 0; j < 4; ++j)
        if (best_i == lane + j * kWave) p[j] = -1.f;
}

}  // namespace fk
