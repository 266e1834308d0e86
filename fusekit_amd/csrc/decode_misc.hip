// Small decode kernels around the four streaming kernels: RoPE / per-head
// RMSNorm / KV-cache store, embedding lookup, greedy argmax, the per-token step
// counter and a fill kernel.  All are launch-latency sized (a few KB of data);
// what matters is that each is one launch and keeps the reference's rounding
// boundaries.
#include "fk_host.hpp"
#include "fk_device.hpp"
#include "rope_device.hpp"
#include "argmax_tail.hpp"

namespace fk {

// ---------------------------------------------------------------- RoPE + store
//
// One wave per head.  Blocks [0, n_q) rotate a q head in place, blocks
// [n_q, n_q + n_kv) rotate a k head into the cache row, blocks beyond copy a v
// head into the cache row.  With a norm weight the head is first RMS-normalised
// with the reference's two roundings, T(w * T(x * r)), and the rotation acts on
// those T values.
__global__ __launch_bounds__(kWave) void rope_store_kernel(const RopeArgs a) {
    const uint32_t b = blockIdx.x, lane = threadIdx.x, tr = blockIdx.y;  // tr: active token row
    const uint32_t pos0 = a.offset_ptr ? *a.offset_ptr : a.offset_imm;
    const uint32_t pos = pos0 + tr;
    const uint32_t wpos = (a.write_offset_ptr ? *a.write_offset_ptr : (a.use_write_imm ? a.write_offset_imm : pos0)) + tr;
    const uint32_t row = wpos % a.capacity;

    if (b >= a.n_q + a.n_kv) {  // V head: straight copy into the cache row
        const uint32_t h = b - a.n_q - a.n_kv;
        const uint16_t* src = a.v + ((size_t)tr * a.n_kv + h) * a.v_dim;
        uint16_t* dst = a.cache_v + ((size_t)h * a.capacity + row) * a.v_dim;
        if ((a.v_dim & 1u) == 0) {  // rows are then 4-byte aligned
            const uint32_t* s2 = reinterpret_cast<const uint32_t*>(src);
            uint32_t* d2 = reinterpret_cast<uint32_t*>(dst);
            for (uint32_t d = lane; d < a.v_dim / 2u; d += kWave) d2[d] = s2[d];
        } else {
            for (uint32_t d = lane; d < a.v_dim; d += kWave) dst[d] = src[d];
        }
        return;
    }
    const bool is_q = b < a.n_q;
    const uint32_t h = is_q ? b : b - a.n_q;
    const uint32_t dim = is_q ? a.head_dim : a.k_dim;
    const uint16_t* src = is_q ? a.q + ((size_t)tr * a.n_q + h) * dim : a.k + ((size_t)tr * a.n_kv + h) * dim;
    uint16_t* dst = is_q ? a.q + ((size_t)tr * a.n_q + h) * dim : a.cache_k + ((size_t)h * a.capacity + row) * dim;
    const uint16_t* nw = is_q ? a.q_norm : a.k_norm;

    const float* tab = a.rope_tab ? a.rope_tab + (size_t)tr * a.rope_dims : nullptr;
    head_transform(src, dst, nw, dim, a.rope_on ? a.rope_dims : 0u, pos, a.base_log2, a.eps, nw != nullptr || !is_q,
                   lane, tab);
}

// The rotary table of a prompt pass: without it every (head, row) wave evaluates exp2 in double and
// sincosf per pair; the table is filled once per pass and serves every layer.
struct RopeTabArgs {
    float* tab;
    uint32_t half, offset, rows;
    float base_log2;
};
__global__ __launch_bounds__(256) void rope_table_kernel(const RopeTabArgs a) {
    const uint32_t i = blockIdx.x * 256u + threadIdx.x;
    if (i >= a.rows * a.half) return;
    const uint32_t r = i / a.half, d = i - r * a.half;
    float cs, sn;
    rope_cos_sin(d, a.half, a.offset + r, a.base_log2, cs, sn);
    a.tab[2 * (size_t)i] = cs;
    a.tab[2 * (size_t)i + 1] = sn;
}

fk_status plan_rope_table(float* tab, uint32_t rope_dims, float base_log2, uint32_t offset, uint32_t rows, Launch* out) {
    const DeviceFacts* dev;
    FK_TRY(device_facts(&dev));
    if (!tab || rows == 0) return set_error(FK_ERR_INVALID, "rope table: null table or zero rows");
    if (rope_dims == 0 || rope_dims % 2) return set_error(FK_ERR_INVALID, "rope table: rope_dims must be even and non-zero");
    if ((uint64_t)rows * (rope_dims / 2) > 0x7fffffffull) return set_error(FK_ERR_UNSUPPORTED, "rope table: too large");
    RopeTabArgs a{tab, rope_dims / 2, offset, rows, base_log2};
    out->func = reinterpret_cast<const void*>(&rope_table_kernel);
    out->grid = dim3((rows * (rope_dims / 2) + 255u) / 256u, 1, 1);
    out->block = dim3(256, 1, 1);
    out->shmem = 0;
    out->set_args(a);
    return FK_OK;
}

// Row form for prompt passes (rotation over the whole head of 64 or 128 dims, rotary table given):
// a head row is spread over HL = dim / 8 adjacent lanes with 16 bytes each, so a wave moves 8 (4)
// head rows with one 16-byte load and one store per lane and ONE dependent round trip to memory; the
// pair (d, d + dim/2) sits HL/2 lanes apart and is exchanged as packed bf16, the norm's sum of squares
// is a butterfly over the HL lanes.  One wave per (head, row) with 2-byte accesses took 92 us for
// 4096 rows of the 4B-class model; the kernel is bound by its short chains, not by bytes.
template <int HL>
__global__ __launch_bounds__(256) void rope_rows_fast_kernel(const RopeArgs a) {
    constexpr uint32_t DIM = HL * 8u, HPW = kWave / HL;
    const uint32_t lane = threadIdx.x & (kWave - 1u);
    const uint32_t heads = a.n_q + 2u * a.n_kv, groups = (heads + HPW - 1u) / HPW;
    const uint32_t wg = blockIdx.x * 4u + (threadIdx.x >> 6);
    const uint32_t tr = wg / groups, g = wg - tr * groups;
    if (tr >= a.rows) return;  // whole waves
    const uint32_t b_raw = g * HPW + lane / HL, p = lane % HL;
    const bool live = b_raw < heads;
    const uint32_t b = live ? b_raw : heads - 1u;  // lanes past the last head repeat it and store nothing
    const uint32_t pos0 = a.offset_ptr ? *a.offset_ptr : a.offset_imm;
    const uint32_t wpos = (a.write_offset_ptr ? *a.write_offset_ptr : (a.use_write_imm ? a.write_offset_imm : pos0)) + tr;
    const uint32_t row = wpos % a.capacity;
    const uint16_t* src;
    uint16_t* dst;
    const uint16_t* nw = nullptr;
    bool rotate = true;
    if (b < a.n_q) {
        src = dst = a.q + ((size_t)tr * a.n_q + b) * DIM;
        nw = a.q_norm;
    } else if (b < a.n_q + a.n_kv) {
        const uint32_t h = b - a.n_q;
        src = a.k + ((size_t)tr * a.n_kv + h) * DIM;
        dst = a.cache_k + ((size_t)h * a.capacity + row) * DIM;
        nw = a.k_norm;
    } else {
        const uint32_t h = b - a.n_q - a.n_kv;
        src = a.v + ((size_t)tr * a.n_kv + h) * DIM;
        dst = a.cache_v + ((size_t)h * a.capacity + row) * DIM;
        rotate = false;
    }
    // every load is issued before anything is used; lanes without a norm weight read their own row instead
    const uint4 xv = *reinterpret_cast<const uint4*>(src + p * 8u);
    const uint4 wv = *reinterpret_cast<const uint4*>((nw ? nw : src) + p * 8u);
    const float4* tp = reinterpret_cast<const float4*>(a.rope_tab + (size_t)tr * DIM + 2u * ((p % (HL / 2u)) * 8u));
    const float4 t0 = tp[0], t1 = tp[1], t2 = tp[2], t3 = tp[3];  // (cos, sin) of this lane's eight pairs
    const float cs[8] = {t0.x, t0.z, t1.x, t1.z, t2.x, t2.z, t3.x, t3.z};
    const float sn[8] = {t0.y, t0.w, t1.y, t1.w, t2.y, t2.w, t3.y, t3.w};

    uint32_t pv[4] = {xv.x, xv.y, xv.z, xv.w};
    const uint32_t wq[4] = {wv.x, wv.y, wv.z, wv.w};
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const float lo = bf16_lo(pv[i]), hi = bf16_hi(pv[i]);
        ss = fmaf(lo, lo, ss);
        ss = fmaf(hi, hi, ss);
    }
    ss = group_sum(ss, HL);  // all lanes take part; used only where there is a norm weight
    if (nw) {
        const float r = 1.0f / sqrtf(ss / (float)DIM + a.eps);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const uint32_t xr = pack_bf16(bf16_lo(pv[i]) * r, bf16_hi(pv[i]) * r);   // T(x * r)
            pv[i] = pack_bf16(bf16_lo(wq[i]) * bf16_lo(xr), bf16_hi(wq[i]) * bf16_hi(xr));  // T(w * that)
        }
    }
    uint32_t ov[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) ov[i] = (uint32_t)__shfl_xor((int)pv[i], (int)(HL / 2u), kWave);
    uint4 res = make_uint4(pv[0], pv[1], pv[2], pv[3]);
    if (rotate) {
        const bool second = p >= HL / 2u;  // this lane holds the d + dim/2 side of its pairs
        uint32_t o[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const float a0 = bf16_lo(pv[i]), a1 = bf16_hi(pv[i]), b0 = bf16_lo(ov[i]), b1 = bf16_hi(ov[i]);
            const float r0 = second ? a0 * cs[2 * i] + b0 * sn[2 * i] : a0 * cs[2 * i] - b0 * sn[2 * i];
            const float r1 = second ? a1 * cs[2 * i + 1] + b1 * sn[2 * i + 1] : a1 * cs[2 * i + 1] - b1 * sn[2 * i + 1];
            o[i] = pack_bf16(r0, r1);
        }
        res = make_uint4(o[0], o[1], o[2], o[3]);
    } else {
        res = xv;  // V rows are copied as they are
    }
    if (live) *reinterpret_cast<uint4*>(dst + p * 8u) = res;
}

fk_status plan_rope_store(const RopeArgs& in, Launch* out) {
    const DeviceFacts* dev;
    FK_TRY(device_facts(&dev));
    RopeArgs a = in;
    if (a.n_q && !a.q) return set_error(FK_ERR_INVALID, "rope: null q");
    if (a.n_kv && (!a.cache_k || !a.cache_v || !a.k || !a.v)) return set_error(FK_ERR_INVALID, "rope: null k/v/cache");
    if (a.n_q + a.n_kv == 0) return set_error(FK_ERR_INVALID, "rope: nothing to do");
    if (a.n_kv && a.capacity == 0) return set_error(FK_ERR_INVALID, "rope: zero cache capacity");
    if (a.rope_on && (a.rope_dims == 0 || a.rope_dims % 2 || (a.n_q && a.rope_dims > a.head_dim) ||
                      (a.n_kv && a.rope_dims > a.k_dim)))
        return set_error(FK_ERR_INVALID, "rope: rope_dims must be even and within the head");
    if (!a.capacity) a.capacity = 1;
    if (!a.rows) a.rows = 1;
    if (a.rows > 65535) return set_error(FK_ERR_UNSUPPORTED, "rope: too many rows");
    if (a.n_kv && a.rows > a.capacity) return set_error(FK_ERR_INVALID, "rope: more rows than the cache holds");
    const bool aligned = ((reinterpret_cast<uintptr_t>(a.q) | reinterpret_cast<uintptr_t>(a.k) | reinterpret_cast<uintptr_t>(a.v) |
                           reinterpret_cast<uintptr_t>(a.cache_k) | reinterpret_cast<uintptr_t>(a.cache_v) |
                           reinterpret_cast<uintptr_t>(a.q_norm) | reinterpret_cast<uintptr_t>(a.k_norm) |
                           reinterpret_cast<uintptr_t>(a.rope_tab)) & 15u) == 0;
    const uint32_t dim = a.n_q ? a.head_dim : a.k_dim;
    if (a.rows >= 8 && a.rope_tab && a.rope_on && a.n_q && a.n_kv && (dim == 64 || dim == 128) && a.rope_dims == dim &&
        a.k_dim == dim && a.v_dim == dim && aligned) {
        const uint32_t hpw = dim == 128 ? 4u : 8u, heads = a.n_q + 2 * a.n_kv;
        const uint64_t waves = (uint64_t)a.rows * ((heads + hpw - 1u) / hpw);
        out->func = dim == 128 ? reinterpret_cast<const void*>(&rope_rows_fast_kernel<16>) : reinterpret_cast<const void*>(&rope_rows_fast_kernel<8>);
        out->grid = dim3((uint32_t)((waves + 3u) / 4u), 1, 1);
        out->block = dim3(256, 1, 1);
        out->shmem = 0;
        out->set_args(a);
        return FK_OK;
    }
    out->func = reinterpret_cast<const void*>(&rope_store_kernel);
    out->grid = dim3(a.n_q + 2 * a.n_kv, a.rows, 1);
    out->block = dim3(kWave, 1, 1);
    out->shmem = 0;
    out->set_args(a);
    return FK_OK;
}

// ---------------------------------------------------------------- embedding
struct EmbedArgs {
    const void* w;
    const uint16_t* scales;
    const uint16_t* biases;
    const uint32_t* token_ptr;
    uint32_t token_imm;
    uint32_t vocab, hidden, bits, group;
    float out_scale;
    uint16_t* x;
};

// x = T(embed[token] * scale); quantised rows unpack (word >> ((d % lanes) * bits)) & mask
// (reference embed_lookup_decode.rs:74-99).
__global__ __launch_bounds__(256) void embed_lookup_kernel(const EmbedArgs a) {
    const uint32_t d = blockIdx.x * 256 + threadIdx.x, tr = blockIdx.y;
    if (d >= a.hidden) return;
    uint32_t token = a.token_ptr ? a.token_ptr[tr] : a.token_imm;
    if (token >= a.vocab) token = a.vocab - 1;  // never read outside the table
    float val;
    if (a.bits == 16) {
        val = bf16_bits_to_f32(reinterpret_cast<const uint16_t*>(a.w)[(size_t)token * a.hidden + d]);
    } else {
        const uint32_t per = 32 / a.bits, mask = (1u << a.bits) - 1u;
        const uint32_t word = reinterpret_cast<const uint32_t*>(a.w)[(size_t)token * (a.hidden / per) + d / per];
        const uint32_t qv = (word >> ((d % per) * a.bits)) & mask;
        const size_t g = (size_t)token * (a.hidden / a.group) + d / a.group;
        val = (float)qv * bf16_bits_to_f32(a.scales[g]) + bf16_bits_to_f32(a.biases[g]);
    }
    a.x[(size_t)tr * a.hidden + d] = (uint16_t)f32_to_bf16_bits(val * a.out_scale);
}

fk_status plan_embed(const fk_weight* E, const uint32_t* token_ptr, uint32_t token_imm, float out_scale,
                     uint16_t* x, Launch* out, uint32_t rows) {
    const DeviceFacts* dev;
    FK_TRY(device_facts(&dev));
    if (!E || !E->w || !x) return set_error(FK_ERR_INVALID, "embed: null pointer");
    if (E->bits != 4 && E->bits != 8 && E->bits != 16) return set_error(FK_ERR_UNSUPPORTED, "embed: bits 4, 8 or 16");
    if (E->bits != 16 && (!E->scales || !E->biases || E->group == 0 || E->k % E->group))
        return set_error(FK_ERR_INVALID, "embed: bad quantisation metadata");
    if (!token_ptr && token_imm >= E->n) return set_error(FK_ERR_INVALID, "embed: token id outside the vocabulary");
    EmbedArgs a;
    memset(&a, 0, sizeof(a));
    a.w = E->w; a.scales = E->scales; a.biases = E->biases;
    a.token_ptr = token_ptr; a.token_imm = token_imm;
    a.vocab = E->n; a.hidden = E->k; a.bits = E->bits; a.group = E->group;
    a.out_scale = out_scale;
    a.x = x;
    if (rows == 0 || rows > 65535 || (rows > 1 && !token_ptr))
        return set_error(FK_ERR_INVALID, "embed: rows need a device token array");
    out->func = reinterpret_cast<const void*>(&embed_lookup_kernel);
    out->grid = dim3((E->k + 255) / 256, rows, 1);
    out->block = dim3(256, 1, 1);
    out->shmem = 0;
    out->set_args(a);
    return FK_OK;
}

// ---------------------------------------------------------------- argmax
struct ArgmaxArgs {
    const uint16_t* logits;
    uint32_t n;
    ArgmaxTail tail;
};

// Two stages in one launch (argmax_tail.hpp): every block reduces a slice to one packed candidate, the last block
// to finish reduces the candidates.
__global__ __launch_bounds__(256) void argmax_kernel(const ArgmaxArgs a) {
    __shared__ uint64_t sm[256 / kWave];
    __shared__ uint32_t is_last;
    uint64_t best = 0;
    for (uint32_t i = blockIdx.x * 256 + threadIdx.x; i < a.n; i += gridDim.x * 256) {
        const uint64_t cand = argmax_candidate(a.logits[i], i);
        best = cand > best ? cand : best;
    }
    argmax_block_finish<256>(a.tail, best, sm, &is_last);
}

fk_status plan_argmax(const uint16_t* logits, uint32_t n, uint32_t* next_token, uint32_t* history,
                      uint32_t* hist_counter, uint32_t hist_capacity, void* workspace, Launch* out) {
    const DeviceFacts* dev;
    FK_TRY(device_facts(&dev));
    if (!logits || !next_token || !workspace) return set_error(FK_ERR_INVALID, "argmax: null pointer");
    if (n == 0) return set_error(FK_ERR_INVALID, "argmax: empty logits");
    uint32_t grid = (n + 2047) / 2048;
    if (grid > 160) grid = 160;
    ArgmaxArgs a;
    memset(&a, 0, sizeof(a));
    a.logits = logits; a.n = n; a.tail.next_token = next_token;
    a.tail.history = history; a.tail.hist_counter = hist_counter; a.tail.hist_capacity = hist_capacity;
    a.tail.counter = reinterpret_cast<uint32_t*>(workspace);
    a.tail.partial = reinterpret_cast<uint64_t*>(reinterpret_cast<char*>(workspace) + 8);
    out->func = reinterpret_cast<const void*>(&argmax_kernel);
    out->grid = dim3(grid, 1, 1);
    out->block = dim3(256, 1, 1);
    out->shmem = 0;
    out->set_args(a);
    return FK_OK;
}

// ---------------------------------------------------------------- step counter
// offset = step_counter++ ; kv_len = offset + 1 (reference kernels/mod.rs:544-563).
struct StepArgs {
    uint32_t* step_counter;
    uint32_t* offset;
    uint32_t* kv_len;
    float* rope_tab;  // optional: (cos, sin) of every rotary pair at this position, for all layers
    uint32_t half;
    float base_log2;
};
__global__ void step_init_kernel(const StepArgs a) {
    const uint32_t o = *a.step_counter;
    __syncthreads();  // every thread has read the counter before thread 0 advances it
    if (threadIdx.x == 0) {
        *a.step_counter = o + 1;
        *a.offset = o;
        *a.kv_len = o + 1;
    }
    if (a.rope_tab && threadIdx.x < a.half) {
        float cs, sn;
        rope_cos_sin(threadIdx.x, a.half, o, a.base_log2, cs, sn);
        a.rope_tab[2 * threadIdx.x] = cs;
        a.rope_tab[2 * threadIdx.x + 1] = sn;
    }
}

fk_status plan_step_init(uint32_t* step_counter, uint32_t* offset, uint32_t* kv_len, Launch* out, float* rope_tab,
                         uint32_t rope_dims, float base_log2) {
    const DeviceFacts* dev;
    FK_TRY(device_facts(&dev));
    if (!step_counter || !offset || !kv_len) return set_error(FK_ERR_INVALID, "step_init: null pointer");
    if (rope_tab && (rope_dims == 0 || rope_dims % 2 || rope_dims > 512))
        return set_error(FK_ERR_INVALID, "step_init: rope_dims must be even, at most 512");
    StepArgs a{step_counter, offset, kv_len, rope_tab, rope_tab ? rope_dims / 2 : 0u, base_log2};
    out->func = reinterpret_cast<const void*>(&step_init_kernel);
    out->grid = dim3(1, 1, 1);
    out->block = dim3(rope_tab && rope_dims / 2 > kWave ? ((rope_dims / 2 + kWave - 1) / kWave) * kWave : kWave, 1, 1);
    out->shmem = 0;
    out->set_args(a);
    return FK_OK;
}

// ---------------------------------------------------------------- fill
struct FillArgs {
    uint32_t* p;
    uint32_t value;
    size_t count;
};
__global__ __launch_bounds__(256) void fill_u32_kernel(const FillArgs a) {
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < a.count; i += (size_t)gridDim.x * 256) a.p[i] = a.value;
}

fk_status plan_fill_u32(void* p, uint32_t value, size_t count, Launch* out) {
    const DeviceFacts* dev;
    FK_TRY(device_facts(&dev));
    if (!p || count == 0) return set_error(FK_ERR_INVALID, "fill: null pointer or zero count");
    FillArgs a{reinterpret_cast<uint32_t*>(p), value, count};
    size_t blocks = (count + 255) / 256;
    if (blocks > (size_t)dev->cus * 8) blocks = (size_t)dev->cus * 8;
    out->func = reinterpret_cast<const void*>(&fill_u32_kernel);
    out->grid = dim3((uint32_t)blocks, 1, 1);
    out->block = dim3(256, 1, 1);
    out->shmem = 0;
    out->set_args(a);
    return FK_OK;
}


// RMSNorm of `rows` activation rows, y = T(w * T(x * r)) with r = 1/sqrt(mean(x^2) + eps)
// per row (the arithmetic the GEMV fuses for one row, kernels/mod.rs:4424-4516), for the
// multi-row path whose matrix-core matmul takes already normalised rows.  One block per row.
struct NormRowsArgs {
    const uint16_t* x;
    const uint16_t* w;
    uint16_t* y;
    uint32_t hidden;
    float eps;
};
__global__ __launch_bounds__(256) void rmsnorm_rows_kernel(const NormRowsArgs a) {
    __shared__ float scratch[8];
    const uint16_t* x = a.x + (size_t)blockIdx.x * a.hidden;
    uint16_t* y = a.y + (size_t)blockIdx.x * a.hidden;
    float ss = 0.f;
    for (uint32_t i = threadIdx.x; i < a.hidden; i += 256) {
        const float v = bf16_bits_to_f32(x[i]);
        ss = fmaf(v, v, ss);
    }
    ss = block_sum<256>(ss, scratch);
    const float r = 1.0f / sqrtf(ss / (float)a.hidden + a.eps);
    for (uint32_t i = threadIdx.x; i < a.hidden; i += 256)
        y[i] = (uint16_t)f32_to_bf16_bits(bf16_bits_to_f32(a.w[i]) * round_bf16(bf16_bits_to_f32(x[i]) * r));
}

fk_status plan_rmsnorm_rows(const uint16_t* x, const uint16_t* w, float eps, uint32_t rows, uint32_t hidden, uint16_t* y,
                            Launch* out) {
    const DeviceFacts* dev;
    FK_TRY(device_facts(&dev));
    if (!x || !w || !y) return set_error(FK_ERR_INVALID, "rmsnorm rows: null pointer");
    if (rows == 0 || hidden == 0) return set_error(FK_ERR_INVALID, "rmsnorm rows: empty shape");
    NormRowsArgs a{x, w, y, hidden, eps};
    out->func = reinterpret_cast<const void*>(&rmsnorm_rows_kernel);
    out->grid = dim3(rows, 1, 1);
    out->block = dim3(256, 1, 1);
    out->shmem = 0;
    out->set_args(a);
    return FK_OK;
}

// Plain device-to-device copy in 16-byte pieces.  Besides moving buffers it is the
// known-traffic kernel hardware byte counters are calibrated against.
struct CopyArgs {
    uint4* dst;
    const uint4* src;
    size_t count;  // 16-byte pieces
};
__global__ __launch_bounds__(256) void copy_u128_kernel(const CopyArgs a) {
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < a.count; i += (size_t)gridDim.x * 256) a.dst[i] = a.src[i];
}

fk_status plan_copy(void* dst, const void* src, size_t nbytes, Launch* out) {
    const DeviceFacts* dev;
    FK_TRY(device_facts(&dev));
    if (!dst || !src || nbytes == 0) return set_error(FK_ERR_INVALID, "copy: null pointer or zero size");
    if (nbytes % 16 || (reinterpret_cast<uintptr_t>(dst) | reinterpret_cast<uintptr_t>(src)) % 16)
        return set_error(FK_ERR_INVALID, "copy: pointers and size must be multiples of 16 bytes");
    CopyArgs a{reinterpret_cast<uint4*>(dst), reinterpret_cast<const uint4*>(src), nbytes / 16};
    size_t blocks = (a.count + 255) / 256;
    if (blocks > (size_t)dev->cus * 8) blocks = (size_t)dev->cus * 8;
    out->func = reinterpret_cast<const void*>(&copy_u128_kernel);
    out->grid = dim3((uint32_t)blocks, 1, 1);
    out->block = dim3(256, 1, 1);
    out->shmem = 0;
    out->set_args(a);
    return FK_OK;
}

// ---------------------------------------------------------------- plain read (measurement aid)
// Streams `count` 16-byte pieces through the chip and keeps only their XOR: the upper bound of what ANY read-only
// kernel of this access pattern (1 KiB contiguous per wave instruction, several requests in flight per lane) gets
// from HBM on the device at hand.  The streaming GEMVs are priced against the published peak AND against this.
struct ReadArgs {
    const uint4* src;
    size_t count;
    unsigned long long* out;  // [grid] one word per block
    size_t span;              // pieces per block (a multiple of 8 * 256), blocks walk contiguous spans
};
__global__ __launch_bounds__(256) void read_reduce_kernel(const ReadArgs a) {
    uint4 acc = make_uint4(0, 0, 0, 0);
    auto fold = [&](const uint4& v) {
        acc.x ^= v.x;
        acc.y ^= v.y;
        acc.z ^= v.z;
        acc.w ^= v.w;
    };
    // a block reads its own contiguous span, 32 KiB (8 requests per lane) per round
    const size_t begin = (size_t)blockIdx.x * a.span;
    const size_t end = begin + a.span < a.count ? begin + a.span : a.count;
    size_t i = begin + threadIdx.x;
    for (; i + 7 * 256 < end; i += 8 * 256) {
        uint4 v[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) v[j] = a.src[i + j * 256];
#pragma unroll
        for (int j = 0; j < 8; ++j) fold(v[j]);
    }
    for (; i < end; i += 256) fold(a.src[i]);
    unsigned long long w = ((unsigned long long)(acc.x ^ acc.z) << 32) | (acc.y ^ acc.w);
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) w ^= __shfl_xor(w, off);
    __shared__ unsigned long long part[4];
    if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = w;
    __syncthreads();
    if (threadIdx.x == 0) a.out[blockIdx.x] = part[0] ^ part[1] ^ part[2] ^ part[3];
}

fk_status plan_read_reduce(const void* src, size_t nbytes, void* out, size_t out_bytes, uint32_t blocks_per_cu, Launch* l) {
    const DeviceFacts* dev;
    FK_TRY(device_facts(&dev));
    if (!src || !out || nbytes == 0) return set_error(FK_ERR_INVALID, "read: null pointer or zero size");
    if (nbytes % 16 || reinterpret_cast<uintptr_t>(src) % 16 || reinterpret_cast<uintptr_t>(out) % 8)
        return set_error(FK_ERR_INVALID, "read: source and size must be multiples of 16 bytes, the output 8-byte aligned");
    if (blocks_per_cu == 0) blocks_per_cu = 4;  // 2, 4 and 8 read 1 GiB at 5.99, 6.04 and 6.04 TB/s; 1: 5.55
    if (blocks_per_cu > 8) return set_error(FK_ERR_INVALID, "read: at most 8 workgroups per CU");
    ReadArgs a{reinterpret_cast<const uint4*>(src), nbytes / 16, reinterpret_cast<unsigned long long*>(out), 0};
    size_t blocks = (a.count + 8 * 256 - 1) / (8 * 256);
    if (blocks > (size_t)dev->cus * blocks_per_cu) blocks = (size_t)dev->cus * blocks_per_cu;
    a.span = ((a.count + blocks - 1) / blocks + 8 * 256 - 1) / (8 * 256) * (8 * 256);
    if (out_bytes < blocks * 8) return set_error(FK_ERR_INVALID, "read: the output needs 8 bytes per workgroup (fk_read_reduce_out_bytes)");
    l->func = reinterpret_cast<const void*>(&read_reduce_kernel);
    l->grid = dim3((uint32_t)blocks, 1, 1);
    l->block = dim3(256, 1, 1);
    l->shmem = 0;
    l->set_args(a);
    return FK_OK;
}

}  // namespace fk
