// Device-side helpers shared by the gfx950 kernels: bf16 bit handling, wave64
// reductions and block reductions with a fixed (deterministic) order.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace fk {

constexpr int kWave = 64;

typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));

__device__ __forceinline__ float bf16_bits_to_f32(uint32_t h) { return __uint_as_float(h << 16); }
__device__ __forceinline__ float bf16_lo(uint32_t pair) { return __uint_as_float(pair << 16); }
__device__ __forceinline__ float bf16_hi(uint32_t pair) { return __uint_as_float(pair & 0xffff0000u); }

// fp32 -> bf16, round to nearest even, NaN kept quiet: one v_cvt_pk_bf16_f32.  The
// instruction agrees bit for bit, on all 2^32 inputs (NaN payloads included), with
// the integer formulation  u += 0x7fff + ((u >> 16) & 1); u >>= 16  (NaN: (u >> 16) | 0x40).
__device__ __forceinline__ uint32_t pack_bf16(float lo, float hi) {
    const bf16x2_t p = {(__bf16)lo, (__bf16)hi};
    return __builtin_bit_cast(uint32_t, p);
}
__device__ __forceinline__ uint32_t f32_to_bf16_bits(float f) { return pack_bf16(f, 0.0f) & 0xffffu; }
// T(v) as a float again: the rounding boundary the reference places on every
// value it casts to the activation type.
__device__ __forceinline__ float round_bf16(float f) { return __uint_as_float(pack_bf16(0.0f, f) & 0xffff0000u); }

// acc + a.lo*b.lo + a.hi*b.hi with bf16 inputs, fp32 accumulate (v_dot2c_f32_bf16).
__device__ __forceinline__ float dot2_bf16(uint32_t a, uint32_t b, float acc) {
    return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, a), __builtin_bit_cast(bf16x2_t, b), acc,
                                           false);
}

// Activation traffic between blocks of ONE running kernel (the persistent
// whole-token kernel).  Each XCD has its own L2 and the per-CU caches are not
// coherent, so data another block wrote during the same launch must be stored
// write-through (agent scope) and may be read with ordinary loads only from
// addresses nobody has read earlier in the launch; buffers that ARE reused inside
// a launch (attention partials, counters) are read with agent-scope loads, which
// bypass the caches.  COH = false compiles to ordinary loads and stores.
template <bool COH>
__device__ __forceinline__ uint32_t ld_u16(const uint16_t* p) {
    if constexpr (COH) return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    return *p;
}
template <bool COH>
__device__ __forceinline__ void st_u16(uint16_t* p, uint32_t v) {
    if constexpr (COH)
        __hip_atomic_store(p, (uint16_t)v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    else
        *p = (uint16_t)v;
}
template <bool COH>
__device__ __forceinline__ uint4 ld_u128(const uint4* p) {
    if constexpr (COH) {
        const unsigned long long* q = reinterpret_cast<const unsigned long long*>(p);
        const unsigned long long lo = __hip_atomic_load(q, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        const unsigned long long hi = __hip_atomic_load(q + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        return make_uint4((uint32_t)lo, (uint32_t)(lo >> 32), (uint32_t)hi, (uint32_t)(hi >> 32));
    }
    return *p;
}
template <bool COH>
__device__ __forceinline__ float ld_f32(const float* p) {
    if constexpr (COH) return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    return *p;
}
// Two adjacent floats (8-byte aligned) in one load.
template <bool COH>
__device__ __forceinline__ float2 ld_f32x2(const float* p) {
    if constexpr (COH) {
        const unsigned long long v = __hip_atomic_load(reinterpret_cast<const unsigned long long*>(p), __ATOMIC_RELAXED,
                                                       __HIP_MEMORY_SCOPE_AGENT);
        return make_float2(__uint_as_float((uint32_t)v), __uint_as_float((uint32_t)(v >> 32)));
    }
    return *reinterpret_cast<const float2*>(p);
}
template <bool COH>
__device__ __forceinline__ void st_f32(float* p, float v) {
    if constexpr (COH)
        __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    else
        *p = v;
}

// Eight int4 codes of one packed word against eight activations.  A byte
// 0000nnnn read as fp8 e4m3 is exactly n * 2^-9 (subnormal for n < 8, (8+m)*2^-9
// above), so v_cvt_scalef32_pk_bf16_fp8 with scale 512 turns two such bytes into
// the bf16 pair (n_a, n_b) in one instruction.  w & 0x0F0F0F0F holds nibbles
// 0,2,4,6 in its bytes and (w >> 4) & 0x0F0F0F0F nibbles 1,3,5,7, which fixes the
// activation pairing: xp = {(x0,x2), (x4,x6), (x1,x3), (x5,x7)}.
__device__ __forceinline__ float q4_word_dot(uint32_t w, uint4 xp, float d) {
    const uint32_t even = w & 0x0F0F0F0Fu, odd = (w >> 4) & 0x0F0F0F0Fu;
    const bf16x2_t e0 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(even, 512.0f, false);
    const bf16x2_t e1 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(even, 512.0f, true);
    const bf16x2_t o0 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(odd, 512.0f, false);
    const bf16x2_t o1 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(odd, 512.0f, true);
    d = __builtin_amdgcn_fdot2_f32_bf16(e0, __builtin_bit_cast(bf16x2_t, xp.x), d, false);
    d = __builtin_amdgcn_fdot2_f32_bf16(e1, __builtin_bit_cast(bf16x2_t, xp.y), d, false);
    d = __builtin_amdgcn_fdot2_f32_bf16(o0, __builtin_bit_cast(bf16x2_t, xp.z), d, false);
    d = __builtin_amdgcn_fdot2_f32_bf16(o1, __builtin_bit_cast(bf16x2_t, xp.w), d, false);
    return d;
}

// An empty statement that takes a 128-bit value as ONE register operand: whatever computes with the value afterwards
// cannot be scheduled ahead of this point, and the four registers of a load stay one tuple (separate operands per
// component make the compiler copy the tuple apart, and wait for the load to do so).
typedef uint32_t fk_u32x4_t __attribute__((ext_vector_type(4)));
__device__ __forceinline__ void pin_u128(uint4& v) {
    fk_u32x4_t t = {v.x, v.y, v.z, v.w};
    asm volatile("" : "+v"(t));
    v = make_uint4(t.x, t.y, t.z, t.w);
}

// Blocks until every global store and load this wave has issued is complete
// (s_waitcnt vmcnt(0) lgkmcnt(0)).  With write-through (agent-scope) stores this is
// the whole "release" a block needs before it signals other blocks through an
// atomic counter: a workgroup-scope fence compiles to no wait at all on this part,
// and an agent-scope fence adds a write-back of the whole L2.
__device__ __forceinline__ void wait_memory_ops_done() { __builtin_amdgcn_s_waitcnt(0x0070); }

// Reads one word of every 64-byte line of the kernel's argument block (BYTES from its start) and makes the wave wait
// for them once.  A long kernel otherwise fetches its arguments where it first uses them, phase by phase, and each
// first touch of a line is a scalar-cache miss -- a trip to the L2 -- in the middle of that phase; after this the
// later fetches hit.  Call it where the wave waits for its first arguments anyway.
// (FROM: the first line covered; a block of more than twelve lines takes a second call with FROM = 12.)
template <int BYTES, int FROM = 0>
__device__ __forceinline__ void kernarg_warm() {
    typedef const uint32_t __attribute__((address_space(4))) * karg_t;
    karg_t ka = (karg_t)__builtin_amdgcn_kernarg_segment_ptr();
    constexpr int LINES = (BYTES + 63) / 64 - FROM;
    static_assert(LINES >= 1 && LINES <= 12, "argument block larger than this helper covers");
    uint32_t v[12];
#pragma unroll
    for (int i = 0; i < 12; ++i) v[i] = ka[(FROM + (i < LINES ? i : 0)) * 16];
    // one statement that takes them all: every request goes out before the one wait
    asm volatile("" ::"s"(v[0]), "s"(v[1]), "s"(v[2]), "s"(v[3]), "s"(v[4]), "s"(v[5]), "s"(v[6]), "s"(v[7]), "s"(v[8]),
                 "s"(v[9]), "s"(v[10]), "s"(v[11]));
}

// v + (v of the lane selected by a DPP control): cross-lane adds inside a row of
// 16 lanes without going through the LDS crossbar.
template <int CTRL>
__device__ __forceinline__ float dpp_add(float v) {
    const int moved = __builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xF, 0xF, true);
    return v + __int_as_float(moved);
}

// Sum over `width` adjacent lanes (a power of two <= 64, groups aligned to width);
// every lane of the group ends with the total.  Widths up to 16 use DPP only:
// quad_perm [1,0,3,2], quad_perm [2,3,0,1], row_half_mirror, row_mirror.
__device__ __forceinline__ float group_sum(float v, int width) {
    if (width >= 2) v = dpp_add<0xB1>(v);
    if (width >= 4) v = dpp_add<0x4E>(v);
    if (width >= 8) v = dpp_add<0x141>(v);
    if (width >= 16) v = dpp_add<0x140>(v);
    if (width == 32) v += __shfl_xor(v, 16, kWave);
    if (width >= 64) {
        // every lane of row i holds that row's total: (r0 + r1) + (r2 + r3) through scalar
        // registers, the value the two butterfly steps over 16 and 32 lanes give
        const float r0 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 0));
        const float r1 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 16));
        const float r2 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 32));
        const float r3 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 48));
        v = (r0 + r1) + (r2 + r3);
    }
    return v;
}
// All 64 lanes must be active (the cross-row step reads lanes 0, 16, 32, 48 directly).
__device__ __forceinline__ float wave_sum(float v) { return group_sum(v, 64); }
template <int CTRL>
__device__ __forceinline__ float dpp_max(float v) {
    const int moved = __builtin_amdgcn_update_dpp(__float_as_int(v), __float_as_int(v), CTRL, 0xF, 0xF, false);
    return fmaxf(v, __int_as_float(moved));
}
__device__ __forceinline__ float wave_max(float v) {
    v = dpp_max<0xB1>(v);
    v = dpp_max<0x4E>(v);
    v = dpp_max<0x141>(v);
    v = dpp_max<0x140>(v);
    const float r0 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 0));
    const float r1 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 16));
    const float r2 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 32));
    const float r3 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 48));
    return fmaxf(fmaxf(r0, r1), fmaxf(r2, r3));
}

// Block-wide sum; every thread returns the same value.  `scratch` holds one
// float per wave plus one.  Waves are added in index order, so the result does
// not depend on scheduling.
template <int BLOCK>
__device__ __forceinline__ float block_sum(float v, float* scratch) {
    constexpr int NW = BLOCK / kWave;
    v = wave_sum(v);
    if ((threadIdx.x & (kWave - 1)) == 0) scratch[threadIdx.x / kWave] = v;
    __syncthreads();
    // every thread adds the wave totals itself (LDS broadcast reads): one barrier.  The
    // caller must not rewrite `scratch` before its next barrier.
    float t = 0.f;
#pragma unroll
    for (int i = 0; i < NW; ++i) t += scratch[i];
    return t;
}

template <int BLOCK>
__device__ __forceinline__ float block_max(float v, float* scratch) {
    constexpr int NW = BLOCK / kWave;
    v = wave_max(v);
    if ((threadIdx.x & (kWave - 1)) == 0) scratch[threadIdx.x / kWave] = v;
    __syncthreads();
    if (threadIdx.x == 0) {
        float t = scratch[0];
#pragma unroll
        for (int i = 1; i < NW; ++i) t = fmaxf(t, scratch[i]);
        scratch[NW] = t;
    }
    __syncthreads();
    float r = scratch[NW];
    __syncthreads();
    return r;
}

}  // namespace fk
