// MLX-affine weight quantiser on the GPU (Q0) and the seeded synthetic-data
// generator used to instantiate random-init models directly in HBM.
#include "fk_host.hpp"
#include "fk_device.hpp"

namespace fk {

struct QuantArgs {
    const float* w;
    uint32_t* packed;
    uint16_t* scales;
    uint16_t* biases;
    size_t n_groups;  // rows * K / group
    uint32_t bits, group;
};

// One thread per quantisation group.  Arithmetic, statement for statement, of
// the reference's restatement of mx.quantize
// (src/codegen/kernels/rope_kv_cache_store_decode_quant.rs:208-221):
//   scale = max((max - min) / mask, 1e-7); anchor = larger-magnitude edge;
//   q0 = round(edge / scale); scale = edge / q0, bias = edge unless q0 == 0;
//   q = clamp(round((x - bias) / scale), 0, mask), packed LSB first.
__global__ __launch_bounds__(256) void quantize_affine_kernel(const QuantArgs a) {
    const size_t g = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (g >= a.n_groups) return;
    const uint32_t group = a.group, bits = a.bits, per_word = 32 / bits;
    const int mask = (1 << bits) - 1;
    const float* x = a.w + g * group;
    float vmin = x[0], vmax = x[0];
    for (uint32_t i = 1; i < group; ++i) {
        const float v = x[i];
        vmin = v < vmin ? v : vmin;
        vmax = v > vmax ? v : vmax;
    }
    const float scale_abs = fmaxf((vmax - vmin) / (float)mask, 1.0e-7f);
    const bool lo_anchor = fabsf(vmin) > fabsf(vmax);
    float scale = lo_anchor ? scale_abs : -scale_abs;
    const float edge = lo_anchor ? vmin : vmax;
    const float q0 = roundf(edge / scale);
    const bool at_zero = (q0 == 0.0f);
    scale = at_zero ? scale : (edge / q0);
    const float bias = at_zero ? 0.0f : edge;
    const float inv_scale = (scale != 0.0f) ? (1.0f / scale) : 0.0f;
    uint32_t* out = a.packed + g * (group / per_word);
    for (uint32_t wi = 0; wi < group / per_word; ++wi) {
        uint32_t word = 0;
        for (uint32_t el = 0; el < per_word; ++el) {
            const float d = x[wi * per_word + el] - bias;
            int qi = (int)roundf(d * inv_scale);
            qi = qi < 0 ? 0 : (qi > mask ? mask : qi);
            word |= ((uint32_t)qi & (uint32_t)mask) << (el * bits);
        }
        out[wi] = word;
    }
    a.scales[g] = (uint16_t)f32_to_bf16_bits(scale);
    a.biases[g] = (uint16_t)f32_to_bf16_bits(bias);
}

fk_status plan_quantize(const float* w, size_t n, size_t k, uint32_t bits, uint32_t group, uint32_t* packed,
                        uint16_t* scales, uint16_t* biases, Launch* out) {
    const DeviceFacts* dev;
    FK_TRY(device_facts(&dev));
    if (!w || !packed || !scales || !biases) return set_error(FK_ERR_INVALID, "quantize: null pointer");
    if (bits != 4 && bits != 8) return set_error(FK_ERR_UNSUPPORTED, "quantize: bits must be 4 or 8");
    if (group != 32 && group != 64 && group != 128) return set_error(FK_ERR_UNSUPPORTED, "quantize: group 32, 64 or 128");
    if (n == 0 || k == 0 || k % group) return set_error(FK_ERR_INVALID, "quantize: K must be a positive multiple of the group size");
    QuantArgs a{w, packed, scales, biases, n * (k / group), bits, group};
    const size_t blocks = (a.n_groups + 255) / 256;
    if (blocks > 0x7fffffffull) return set_error(FK_ERR_UNSUPPORTED, "quantize: matrix too large for one launch");
    out->func = reinterpret_cast<const void*>(&quantize_affine_kernel);
    out->grid = dim3((uint32_t)blocks, 1, 1);
    out->block = dim3(256, 1, 1);
    out->shmem = 0;
    out->set_args(a);
    return FK_OK;
}

// ---------------------------------------------------------------- synthetic data
struct SynthArgs {
    void* out;
    size_t count;
    uint64_t seed;
    float mean, std;
    uint32_t kind;  // 0: fp32 normal, 1: bf16 normal, 2: uint32 uniform in [0, bound); 3 / 4: see synth_exact
    uint32_t bound;
    uint64_t row_len;  // kinds 3 / 4: elements per row for the row-norm spread (0: none)
    float tau;
    uint64_t loud_rows;  // kinds 3 / 4: row j < loud_rows is multiplied by loud_gain * 2^-j instead
    float loud_gain;
};

__device__ __forceinline__ uint64_t splitmix64(uint64_t z) {
    z += 0x9E3779B97F4A7C15ull;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}

// Kinds 3 (fp32) and 4 (bf16): values a host can reproduce bit for bit, because only integer
// arithmetic, exact int -> float conversions and single IEEE operations are involved (no
// transcendental function, the one multiply-add written as a fused one):
//   z(seed, i) = (2 * S - 524280) * (1 / 107019.84), S = the sum of the eight 16-bit fields of two
//                splitmix64 words keyed by (seed, i): mean 0, variance 1, |z| < 4.9
//   value      = fma(std, z, mean) * rowscale(i / row_len)
//   rowscale(j), when row_len and tau are non-zero: u = floor(tau * z(seed ^ K, j) * 8),
//                (1 + (u & 7) / 8) * 2^(u >> 3): row norms spread like a log-normal;
//                rows j < loud_rows are multiplied by loud_gain * 2^-j instead (a few dominant rows,
//                each half as loud as the one before).
__device__ __forceinline__ float ih_normal(uint64_t seed, uint64_t i) {
    const uint64_t r0 = splitmix64(seed * 0xD1342543DE82EF95ull + i), r1 = splitmix64(r0);
    int32_t sum = 0;
#pragma unroll
    for (int f = 0; f < 4; ++f) sum += (int32_t)((r0 >> (16 * f)) & 0xFFFF) + (int32_t)((r1 >> (16 * f)) & 0xFFFF);
    return __fmul_rn((float)(2 * sum - 524280), 9.3440616e-06f);
}
__device__ __forceinline__ float synth_exact(const SynthArgs& a, size_t i) {
    float v = __fmaf_rn(a.std, ih_normal(a.seed, i), a.mean);
    if (a.row_len && i / a.row_len < a.loud_rows) {
        v = __fmul_rn(v, ldexpf(a.loud_gain, -(int)(i / a.row_len)));
    } else if (a.row_len && a.tau != 0.0f) {
        const float t = floorf(__fmul_rn(__fmul_rn(a.tau, ih_normal(a.seed ^ 0x5DEECE66Dull, i / a.row_len)), 8.0f));
        const int u = (int)t;
        v = __fmul_rn(v, ldexpf(__fmaf_rn((float)(u & 7), 0.125f, 1.0f), u >> 3));
    }
    return v;
}

// Counter-based: element i depends only on (seed, i), so any launch shape gives
// the same bytes.  Normals by Box-Muller on two 24-bit uniforms (kinds 0 / 1).
__global__ __launch_bounds__(256) void synth_kernel(const SynthArgs a) {
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < a.count; i += (size_t)gridDim.x * 256) {
        const uint64_t r = splitmix64(a.seed * 0xD1342543DE82EF95ull + i);
        if (a.kind == 2) {
            reinterpret_cast<uint32_t*>(a.out)[i] = (uint32_t)(((r >> 32) * (uint64_t)a.bound) >> 32);
            continue;
        }
        if (a.kind >= 3) {
            const float e = synth_exact(a, i);
            if (a.kind == 3)
                reinterpret_cast<float*>(a.out)[i] = e;
            else
                reinterpret_cast<uint16_t*>(a.out)[i] = (uint16_t)f32_to_bf16_bits(e);
            continue;
        }
        const float u1 = ((float)((r >> 40) & 0xFFFFFF) + 1.0f) * (1.0f / 16777216.0f);  // (0, 1]
        const float u2 = (float)((r >> 8) & 0xFFFFFF) * (1.0f / 16777216.0f);            // [0, 1)
        const float z = sqrtf(-2.0f * logf(u1)) * cosf(6.28318530717958647692f * u2);
        const float v = a.mean + a.std * z;
        if (a.kind == 0)
            reinterpret_cast<float*>(a.out)[i] = v;
        else
            reinterpret_cast<uint16_t*>(a.out)[i] = (uint16_t)f32_to_bf16_bits(v);
    }
}

fk_status plan_synth(void* out_ptr, size_t count, uint64_t seed, float mean, float std, uint32_t kind, uint32_t bound,
                     Launch* out, uint64_t row_len, float tau, uint64_t loud_rows, float loud_gain) {
    const DeviceFacts* dev;
    FK_TRY(device_facts(&dev));
    if (!out_ptr || count == 0) return set_error(FK_ERR_INVALID, "synth: null pointer or zero count");
    if (kind > 4 || (kind == 2 && bound == 0)) return set_error(FK_ERR_INVALID, "synth: bad kind or bound");
    SynthArgs a{out_ptr, count, seed, mean, std, kind, bound, row_len, tau, loud_rows, loud_gain};
    size_t blocks = (count + 255) / 256;
    if (blocks > (size_t)dev->cus * 16) blocks = (size_t)dev->cus * 16;
    out->func = reinterpret_cast<const void*>(&synth_kernel);
    out->grid = dim3((uint32_t)blocks, 1, 1);
    out->block = dim3(256, 1, 1);
    out->shmem = 0;
    out->set_args(a);
    return FK_OK;
}

}  // namespace fk
