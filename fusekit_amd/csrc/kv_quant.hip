// Quantised KV-cache store: RoPE (+ optional per-head RMSNorm) of the new K rows in fp32, the
// V rows as they are, every group of `group` dims quantised with the MLX-affine formula and
// written in the mlx-lm QuantizedKVCache layout (packed uint32 [n_kv, capacity, dim*bits/32],
// scales / biases bf16 [n_kv, capacity, dim/group]).  Replaces
// src/codegen/kernels/rope_kv_cache_store_decode_quant.rs:100-260: as there, the rotated K value
// is NOT rounded to bf16 before it is quantised.  One wave per (K or V head, token row).
#include "fk_host.hpp"
#include "fk_device.hpp"
#include "rope_device.hpp"

namespace fk {

constexpr uint32_t kKvQuantMaxDim = 512;

__global__ __launch_bounds__(kWave) void kv_store_quant_kernel(const KvQuantStore a) {
    __shared__ float row[kKvQuantMaxDim];
    __shared__ uint8_t codes[kKvQuantMaxDim];
    const uint32_t lane = threadIdx.x, b = blockIdx.x, tr = blockIdx.y;
    const bool is_v = b >= a.n_kv;
    const uint32_t h = is_v ? b - a.n_kv : b;
    const uint32_t pos = (a.offset_ptr ? *a.offset_ptr : a.offset_imm) + tr;
    const uint32_t crow = (a.write_offset_ptr ? *a.write_offset_ptr + tr : pos) % a.capacity;
    const uint16_t* src = (is_v ? a.v : a.k) + ((size_t)tr * a.n_kv + h) * a.dim;

    if (is_v) {
        for (uint32_t d = lane; d < a.dim; d += kWave) row[d] = bf16_bits_to_f32(src[d]);
    } else {
        float r = 1.f;
        if (a.k_norm) {
            float ss = 0.f;
            for (uint32_t d = lane; d < a.dim; d += kWave) {
                const float x = bf16_bits_to_f32(src[d]);
                ss = fmaf(x, x, ss);
            }
            ss = wave_sum(ss);
            r = 1.0f / sqrtf(ss / (float)a.dim + a.eps);
        }
        auto value = [&](uint32_t d) {
            const float x = bf16_bits_to_f32(src[d]);
            return a.k_norm ? round_bf16(bf16_bits_to_f32(a.k_norm[d]) * round_bf16(x * r)) : x;
        };
        const uint32_t half = a.rope_dims / 2;
        for (uint32_t d = lane; d < half; d += kWave) {
            float lo, hi;
            rope_rotate(value(d), value(d + half), d, half, pos, a.base_log2, lo, hi);
            row[d] = lo;
            row[d + half] = hi;
        }
        for (uint32_t d = 2 * half + lane; d < a.dim; d += kWave) row[d] = value(d);
    }
    __syncthreads();

    // Per group: min / max over the wave, then the quantiser's arithmetic statement for statement
    // (see quantize_affine_kernel); every lane derives the same scale and bias.
    const uint32_t groups = a.dim / a.group, per_word = 32u / a.bits;
    const int mask = (1 << a.bits) - 1;
    uint32_t* packed = (is_v ? a.cv_packed : a.ck_packed) + ((size_t)h * a.capacity + crow) * (a.dim / per_word);
    uint16_t* scales = (is_v ? a.cv_scales : a.ck_scales) + ((size_t)h * a.capacity + crow) * groups;
    uint16_t* biases = (is_v ? a.cv_biases : a.ck_biases) + ((size_t)h * a.capacity + crow) * groups;
    for (uint32_t g = 0; g < groups; ++g) {
        const float* x = row + g * a.group;
        float vmin = INFINITY, vmax = -INFINITY;
        for (uint32_t i = lane; i < a.group; i += kWave) {
            vmin = fminf(vmin, x[i]);
            vmax = fmaxf(vmax, x[i]);
        }
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) {
            vmin = fminf(vmin, __shfl_xor(vmin, o, kWave));
            vmax = fmaxf(vmax, __shfl_xor(vmax, o, kWave));
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
        for (uint32_t i = lane; i < a.group; i += kWave) {
            int qi = (int)roundf((x[i] - bias) * inv_scale);
            qi = qi < 0 ? 0 : (qi > mask ? mask : qi);
            codes[g * a.group + i] = (uint8_t)qi;
        }
        if (lane == 0) {
            scales[g] = (uint16_t)f32_to_bf16_bits(scale);
            biases[g] = (uint16_t)f32_to_bf16_bits(bias);
        }
    }
    __syncthreads();
    for (uint32_t wi = lane; wi < a.dim / per_word; wi += kWave) {
        uint32_t word = 0;
        for (uint32_t el = 0; el < per_word; ++el) word |= (uint32_t)codes[wi * per_word + el] << (el * a.bits);
        packed[wi] = word;
    }
}

fk_status plan_kv_store_quant(const KvQuantStore& in, Launch* out) {
    const DeviceFacts* dev;
    FK_TRY(device_facts(&dev));
    KvQuantStore a = in;
    if (!a.k || !a.v || !a.ck_packed || !a.ck_scales || !a.ck_biases || !a.cv_packed || !a.cv_scales || !a.cv_biases)
        return set_error(FK_ERR_INVALID, "kv store (quantised): null pointer");
    if (a.bits != 4 && a.bits != 8) return set_error(FK_ERR_UNSUPPORTED, "kv store (quantised): bits must be 4 or 8");
    if (a.group != 32 && a.group != 64 && a.group != 128)
        return set_error(FK_ERR_UNSUPPORTED, "kv store (quantised): group size must be 32, 64 or 128");
    if (a.n_kv == 0 || a.dim == 0 || a.dim % a.group || a.dim > kKvQuantMaxDim)
        return set_error(FK_ERR_INVALID, "kv store (quantised): head dim must be a multiple of the group size, at most 512");
    if (a.rope_dims % 2 || a.rope_dims > a.dim) return set_error(FK_ERR_INVALID, "kv store (quantised): bad rope_dims");
    if (a.capacity == 0) return set_error(FK_ERR_INVALID, "kv store (quantised): zero capacity");
    if (!a.rows) a.rows = 1;
    if (a.rows > 65535 || a.rows > a.capacity) return set_error(FK_ERR_INVALID, "kv store (quantised): too many rows");
    out->func = reinterpret_cast<const void*>(&kv_store_quant_kernel);
    out->grid = dim3(2 * a.n_kv, a.rows, 1);
    out->block = dim3(kWave, 1, 1);
    out->shmem = 0;
    out->set_args(a);
    return FK_OK;
}

// Rows [0, rows) of every head of a quantised cache as bf16, T(code * scale + bias): the operand
// form the matrix-core prefill attention takes (a prompt pass dequantises the visible prefix once per
// layer, a few MB, instead of running the single-row kernel once per row).  One thread per packed word.
struct KvDequantArgs {
    const uint32_t* packed;
    const uint16_t* scales;
    const uint16_t* biases;
    uint16_t* out;  // [n_kv, out_capacity, dim]
    uint32_t n_kv, dim, capacity, out_capacity, rows, bits, group;
};

__global__ __launch_bounds__(256) void kv_dequant_kernel(const KvDequantArgs a) {
    const uint32_t per_word = 32u / a.bits, wpr = a.dim / per_word;
    const size_t total = (size_t)a.n_kv * a.rows * wpr;
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (size_t)gridDim.x * 256) {
        const uint32_t w = (uint32_t)(i % wpr);
        const size_t hr = i / wpr;
        const uint32_t row = (uint32_t)(hr % a.rows), h = (uint32_t)(hr / a.rows);
        const size_t src_row = (size_t)h * a.capacity + row;
        const uint32_t g = (w * per_word) / a.group;
        const float s = bf16_bits_to_f32(a.scales[src_row * (a.dim / a.group) + g]);
        const float b = bf16_bits_to_f32(a.biases[src_row * (a.dim / a.group) + g]);
        const uint32_t word = a.packed[src_row * wpr + w];
        uint16_t* dst = a.out + ((size_t)h * a.out_capacity + row) * a.dim + w * per_word;
        auto dq = [&](uint32_t code) { return fmaf((float)code, s, b); };
        if (a.bits == 4) {
            *reinterpret_cast<uint4*>(dst) =
                make_uint4(pack_bf16(dq(word & 15u), dq((word >> 4) & 15u)), pack_bf16(dq((word >> 8) & 15u), dq((word >> 12) & 15u)),
                           pack_bf16(dq((word >> 16) & 15u), dq((word >> 20) & 15u)), pack_bf16(dq((word >> 24) & 15u), dq(word >> 28)));
        } else {
            *reinterpret_cast<uint2*>(dst) =
                make_uint2(pack_bf16(dq(word & 255u), dq((word >> 8) & 255u)), pack_bf16(dq((word >> 16) & 255u), dq(word >> 24)));
        }
    }
}

fk_status plan_kv_dequant(const uint32_t* packed, const uint16_t* scales, const uint16_t* biases, uint32_t n_kv, uint32_t dim,
                          uint32_t capacity, uint32_t bits, uint32_t group, uint32_t rows, uint16_t* out, uint32_t out_capacity,
                          Launch* l) {
    const DeviceFacts* dev;
    FK_TRY(device_facts(&dev));
    if (!packed || !scales || !biases || !out) return set_error(FK_ERR_INVALID, "kv dequant: null pointer");
    if (bits != 4 && bits != 8) return set_error(FK_ERR_UNSUPPORTED, "kv dequant: bits must be 4 or 8");
    if (group != 32 && group != 64 && group != 128) return set_error(FK_ERR_UNSUPPORTED, "kv dequant: group size must be 32, 64 or 128");
    if (n_kv == 0 || dim == 0 || dim % group || dim % 8u) return set_error(FK_ERR_INVALID, "kv dequant: head dim must be a multiple of the group size");
    if (rows == 0 || rows > capacity || rows > out_capacity) return set_error(FK_ERR_INVALID, "kv dequant: rows must fit both caches");
    if (reinterpret_cast<uintptr_t>(out) & 15u) return set_error(FK_ERR_INVALID, "kv dequant: output must be 16-byte aligned");
    KvDequantArgs a{packed, scales, biases, out, n_kv, dim, capacity, out_capacity, rows, bits, group};
    const size_t total = (size_t)n_kv * rows * (dim * bits / 32u);
    size_t blocks = (total + 255) / 256;
    if (blocks > (size_t)dev->cus * 16) blocks = (size_t)dev->cus * 16;
    l->func = reinterpret_cast<const void*>(&kv_dequant_kernel);
    l->grid = dim3((uint32_t)blocks, 1, 1);
    l->block = dim3(256, 1, 1);
    l->shmem = 0;
    l->set_args(a);
    return FK_OK;
}

}  // namespace fk
