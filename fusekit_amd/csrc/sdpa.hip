// GQA scaled-dot-product attention for one new token over a bf16 KV cache
// (split-K "flash decoding"), gfx950.
//
// Grid (splits, kv heads, head tiles).  A block owns one KV head, one range of
// `chunk_len` cache positions and up to GT query heads of that KV head's group,
// so every K and V element is read from HBM once and used for all of them.
//   phase A  scores: a key row is spread over LPK lanes (16 bytes = 8 dims per
//            lane, 1 KiB contiguous per wave load); each lane dots its 8 dims
//            with the matching q slice of each head (registers), a butterfly
//            over the LPK lanes finishes the dot; scores land in LDS.
//   softmax  per head by one wave: max, exp, sum (fp32, probabilities are never
//            rounded to bf16).
//   phase B  o += p * v with the same lane layout over V rows; lanes keep 8
//            output dims per head, reduced over key slots at the end.
// A range that covers the whole context writes the output directly; otherwise
// the block stores (m, l, o) and the last block to finish per (kv head, head
// tile) merges the partials in split order (so the result does not depend on
// arrival order) and resets the counter for the next launch.
#include "fk_host.hpp"
#include "fk_device.hpp"

namespace fk {

constexpr int kSdpaBlock = 256;
constexpr int kSdpaWaves = kSdpaBlock / kWave;
constexpr int kSteps = 8;  // K rows (and at most as many V rows) each lane owns per range

namespace {
uint32_t pow2_ceil(uint32_t v) {
    uint32_t p = 1;
    while (p < v) p <<= 1;
    return p;
}
}  // namespace

struct SdpaArgs {
    const uint16_t* q;
    const uint16_t* k;
    const uint16_t* v;
    uint16_t* out;
    const uint32_t* kv_len_ptr;  // device scalar, or null -> kv_len_imm
    uint32_t kv_len_imm;
    uint32_t n_heads, n_kv, qk_dim, v_dim, capacity;
    uint32_t chunk_len, n_splits;
    uint32_t lpk, lpv;  // lanes per key row / value row (powers of two)
    float scale;
    float* partials;     // [n_heads][n_splits][v_dim + 2]
    uint32_t* counters;  // [n_kv * head tiles], zero before the first launch
};

template <int GT>
__global__ __launch_bounds__(kSdpaBlock) void sdpa_decode_kernel(const SdpaArgs a) {
    extern __shared__ float lds[];
    const uint32_t kv_len = a.kv_len_ptr ? *a.kv_len_ptr : a.kv_len_imm;
    const uint32_t n_active = (kv_len + a.chunk_len - 1) / a.chunk_len;
    const uint32_t split = blockIdx.x, kvh = blockIdx.y, gz = blockIdx.z;
    if (split >= n_active) return;  // uniform: whole block leaves before any barrier

    const uint32_t G = a.n_heads / a.n_kv;
    const uint32_t h0 = kvh * G + gz * GT;
    const uint32_t gcount = (G - gz * GT) < (uint32_t)GT ? (G - gz * GT) : (uint32_t)GT;
    const uint32_t key0 = split * a.chunk_len;
    const uint32_t nkeys = (kv_len - key0) < a.chunk_len ? (kv_len - key0) : a.chunk_len;
    const uint32_t tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;

    float* s = lds;                               // [GT][chunk_len]
    float* red = s + GT * a.chunk_len;            // [waves][GT][v_dim]
    float* stat = red + kSdpaWaves * GT * a.v_dim;  // m[GT], l[GT], misc

    // All K and V loads of the range are issued up front (the range is sized so that
    // each lane owns kSteps rows of each), so one HBM round trip covers both phases.
    const uint32_t lpk = a.lpk, cpk = a.qk_dim >> 3;
    const uint32_t lpv = a.lpv, cpv = a.v_dim >> 3;
    const uint32_t ck = tid & (lpk - 1), kslot = tid / lpk, kslots = kSdpaBlock / lpk;
    const uint32_t cv = tid & (lpv - 1), vslot = tid / lpv, vslots = kSdpaBlock / lpv;
    const bool kcol_ok = ck < cpk, vcol_ok = cv < cpv;
    uint4 kc[kSteps], vc[kSteps];
    {
        const uint16_t* kbase = a.k + ((size_t)kvh * a.capacity + key0) * a.qk_dim + 8 * ck;
        const uint16_t* vbase = a.v + ((size_t)kvh * a.capacity + key0) * a.v_dim + 8 * cv;
#pragma unroll
        for (int u = 0; u < kSteps; ++u) {
            const uint32_t j = kslot + u * kslots;
            kc[u] = make_uint4(0, 0, 0, 0);
            if (kcol_ok && j < nkeys) kc[u] = *reinterpret_cast<const uint4*>(kbase + (size_t)j * a.qk_dim);
        }
#pragma unroll
        for (int u = 0; u < kSteps; ++u) {
            const uint32_t j = vslot + u * vslots;
            vc[u] = make_uint4(0, 0, 0, 0);
            if (vcol_ok && j < nkeys) vc[u] = *reinterpret_cast<const uint4*>(vbase + (size_t)j * a.v_dim);
        }
    }

    // ---------------- phase A: scores ----------------
    {
        uint4 qf[GT];
#pragma unroll
        for (int h = 0; h < GT; ++h) {
            qf[h] = make_uint4(0, 0, 0, 0);
            if (kcol_ok && (uint32_t)h < gcount)
                qf[h] = *reinterpret_cast<const uint4*>(a.q + (size_t)(h0 + h) * a.qk_dim + 8 * ck);
        }
#pragma unroll
        for (int u = 0; u < kSteps; ++u) {
            const uint32_t j = kslot + u * kslots;
#pragma unroll
            for (int h = 0; h < GT; ++h) {
                float d = 0.f;
                d = dot2_bf16(kc[u].x, qf[h].x, d);
                d = dot2_bf16(kc[u].y, qf[h].y, d);
                d = dot2_bf16(kc[u].z, qf[h].z, d);
                d = dot2_bf16(kc[u].w, qf[h].w, d);
                d = group_sum(d, (int)lpk);
                if (ck == 0 && j < nkeys) s[h * a.chunk_len + j] = d * a.scale;
            }
        }
    }
    __syncthreads();

    // ---------------- softmax over this range, one wave per head ----------------
    for (uint32_t h = wave; h < gcount; h += kSdpaWaves) {
        float* sh = s + h * a.chunk_len;
        float m = -INFINITY;
        for (uint32_t j = lane; j < nkeys; j += kWave) m = fmaxf(m, sh[j]);
        m = wave_max(m);
        float l = 0.f;
        for (uint32_t j = lane; j < nkeys; j += kWave) {
            const float p = expf(sh[j] - m);
            sh[j] = p;
            l += p;
        }
        l = wave_sum(l);
        if (lane == 0) {
            stat[h] = m;
            stat[GT + h] = l;
        }
    }
    __syncthreads();

    // ---------------- phase B: o = sum_j p_j v_j ----------------
    {
        float acc[GT][8];
#pragma unroll
        for (int h = 0; h < GT; ++h)
#pragma unroll
            for (int i = 0; i < 8; ++i) acc[h][i] = 0.f;
#pragma unroll
        for (int u = 0; u < kSteps; ++u) {
            const uint32_t j = vslot + u * vslots;
            const uint32_t jj = j < nkeys ? j : 0u;
            const float live = j < nkeys ? 1.f : 0.f;
            const float f[8] = {bf16_lo(vc[u].x), bf16_hi(vc[u].x), bf16_lo(vc[u].y), bf16_hi(vc[u].y),
                                bf16_lo(vc[u].z), bf16_hi(vc[u].z), bf16_lo(vc[u].w), bf16_hi(vc[u].w)};
#pragma unroll
            for (int h = 0; h < GT; ++h) {
                const float p = s[h * a.chunk_len + jj] * live;
#pragma unroll
                for (int i = 0; i < 8; ++i) acc[h][i] = fmaf(p, f[i], acc[h][i]);
            }
        }
        // add the key slots that share this lane's column: first inside the wave ...
#pragma unroll
        for (int h = 0; h < GT; ++h)
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                float v = acc[h][i];
                for (uint32_t o = lpv; o < (uint32_t)kWave; o <<= 1) v += __shfl_xor(v, (int)o, kWave);
                acc[h][i] = v;
            }
        // ... then across waves through LDS
        if (lane < lpv && vcol_ok) {
#pragma unroll
            for (int h = 0; h < GT; ++h)
#pragma unroll
                for (int i = 0; i < 8; ++i) red[(wave * GT + h) * a.v_dim + 8 * cv + i] = acc[h][i];
        }
    }
    __syncthreads();

    const uint32_t n_out = gcount * a.v_dim;
    const bool direct = (n_active == 1);
    for (uint32_t e = tid; e < n_out; e += kSdpaBlock) {
        const uint32_t h = e / a.v_dim, d = e - h * a.v_dim;
        float o = 0.f;
#pragma unroll
        for (int w = 0; w < kSdpaWaves; ++w) o += red[(w * GT + h) * a.v_dim + d];
        if (direct) {
            a.out[(size_t)(h0 + h) * a.v_dim + d] = (uint16_t)f32_to_bf16_bits(o / stat[GT + h]);
        } else {
            float* p = a.partials + ((size_t)(h0 + h) * a.n_splits + split) * (a.v_dim + 2);
            p[2 + d] = o;
            if (d == 0) {
                p[0] = stat[h];
                p[1] = stat[GT + h];
            }
        }
    }
    if (direct) return;

    // ---------------- last block merges the partials ----------------
    __threadfence();
    __syncthreads();
    uint32_t* flag = reinterpret_cast<uint32_t*>(stat + 2 * GT);
    if (tid == 0) {
        const uint32_t prev = atomicAdd(&a.counters[kvh * gridDim.z + gz], 1u);
        *flag = (prev == n_active - 1) ? 1u : 0u;
    }
    __syncthreads();
    if (*flag == 0u) return;
    __threadfence();
    if (tid == 0) a.counters[kvh * gridDim.z + gz] = 0u;  // ready for the next launch

    // weights w_s = exp(m_s - M) / L per head, held in LDS (reuses the score area
    // when the range count fits, else loops in pieces of chunk_len)
    for (uint32_t h = 0; h < gcount; ++h) {
        const float* ph = a.partials + (size_t)(h0 + h) * a.n_splits * (a.v_dim + 2);
        float m = -INFINITY;
        for (uint32_t sp = tid; sp < n_active; sp += kSdpaBlock) m = fmaxf(m, ph[(size_t)sp * (a.v_dim + 2)]);
        m = block_max<kSdpaBlock>(m, stat + 2 * GT + 4);
        float l = 0.f;
        for (uint32_t sp = tid; sp < n_active; sp += kSdpaBlock) {
            const float* p = ph + (size_t)sp * (a.v_dim + 2);
            l += p[1] * expf(p[0] - m);
        }
        l = block_sum<kSdpaBlock>(l, stat + 2 * GT + 4);
        const float inv_l = 1.0f / l;
        // each thread owns output dims; ranges are added in index order
        for (uint32_t d = tid; d < a.v_dim; d += kSdpaBlock) {
            float o = 0.f;
            for (uint32_t sp = 0; sp < n_active; ++sp) {
                const float* p = ph + (size_t)sp * (a.v_dim + 2);
                o = fmaf(p[2 + d], expf(p[0] - m), o);
            }
            a.out[(size_t)(h0 + h) * a.v_dim + d] = (uint16_t)f32_to_bf16_bits(o * inv_l);
        }
    }
}

// Positions per range: every lane owns exactly kSteps key rows, i.e.
// kSteps * (block threads / lanes per key row).  128 positions for head_dim 128
// (64 KiB of K+V per block); a 32k context then spreads over 256 ranges x kv heads.
uint32_t sdpa_chunk_len(uint32_t qk_dim, uint32_t v_dim) {
    const uint32_t lpk = pow2_ceil(qk_dim / 8), lpv = pow2_ceil(v_dim / 8);
    const uint32_t wide = lpk > lpv ? lpk : lpv;
    return kSteps * (kSdpaBlock / wide);
}

fk_status sdpa_workspace_bytes(uint32_t n_heads, uint32_t n_kv, uint32_t qk_dim, uint32_t v_dim, uint32_t max_len,
                               size_t* partial_bytes, size_t* counter_bytes) {
    const uint32_t chunk = sdpa_chunk_len(qk_dim, v_dim);
    const uint32_t n_splits = (max_len + chunk - 1) / chunk;
    *partial_bytes = (size_t)n_heads * n_splits * (v_dim + 2) * sizeof(float);
    *counter_bytes = (size_t)n_heads * sizeof(uint32_t);  // >= n_kv * head tiles
    (void)n_kv;
    return FK_OK;
}

fk_status plan_sdpa_decode(const uint16_t* q, const uint16_t* k, const uint16_t* v, uint16_t* out,
                           const uint32_t* kv_len_ptr, uint32_t kv_len_imm, uint32_t max_len, uint32_t n_heads,
                           uint32_t n_kv, uint32_t qk_dim, uint32_t v_dim, uint32_t capacity, float scale,
                           float* partials, uint32_t* counters, Launch* out_launch) {
    const DeviceFacts* dev;
    FK_TRY(device_facts(&dev));
    if (!q || !k || !v || !out) return set_error(FK_ERR_INVALID, "sdpa: null tensor");
    if (n_kv == 0 || n_heads == 0 || n_heads % n_kv != 0)
        return set_error(FK_ERR_INVALID, "sdpa: n_heads must be a positive multiple of n_kv");
    if (qk_dim == 0 || v_dim == 0 || qk_dim % 8 || v_dim % 8 || qk_dim > 512 || v_dim > 512)
        return set_error(FK_ERR_UNSUPPORTED, "sdpa: head dims must be multiples of 8, at most 512");
    if (max_len == 0 || max_len > capacity) return set_error(FK_ERR_INVALID, "sdpa: kv length outside (0, capacity]");
    if (!kv_len_ptr && (kv_len_imm == 0 || kv_len_imm > max_len))
        return set_error(FK_ERR_INVALID, "sdpa: kv_len outside (0, max_len]");
    const uint32_t chunk = sdpa_chunk_len(qk_dim, v_dim);
    const uint32_t n_splits = (max_len + chunk - 1) / chunk;
    if (n_splits > 1 && (!partials || !counters))
        return set_error(FK_ERR_INVALID, "sdpa: workspace required when the context spans several ranges");
    const uint32_t G = n_heads / n_kv;
    const int gt = G >= 8 ? 8 : (G >= 4 ? (G == 4 ? 4 : 8) : (G >= 2 ? (G == 2 ? 2 : 4) : 1));

    SdpaArgs a;
    memset(&a, 0, sizeof(a));
    a.q = q; a.k = k; a.v = v; a.out = out;
    a.kv_len_ptr = kv_len_ptr;
    a.kv_len_imm = kv_len_imm;
    a.n_heads = n_heads; a.n_kv = n_kv; a.qk_dim = qk_dim; a.v_dim = v_dim; a.capacity = capacity;
    a.chunk_len = chunk;
    a.n_splits = n_splits;
    a.lpk = pow2_ceil(qk_dim / 8);
    a.lpv = pow2_ceil(v_dim / 8);
    a.scale = scale;
    a.partials = partials;
    a.counters = counters;

    const void* func = nullptr;
    switch (gt) {
        case 1: func = reinterpret_cast<const void*>(&sdpa_decode_kernel<1>); break;
        case 2: func = reinterpret_cast<const void*>(&sdpa_decode_kernel<2>); break;
        case 4: func = reinterpret_cast<const void*>(&sdpa_decode_kernel<4>); break;
        default: func = reinterpret_cast<const void*>(&sdpa_decode_kernel<8>); break;
    }
    out_launch->func = func;
    out_launch->grid = dim3(n_splits, n_kv, (G + gt - 1) / gt);
    out_launch->block = dim3(kSdpaBlock, 1, 1);
    out_launch->shmem = (uint32_t)((gt * chunk + kSdpaWaves * gt * v_dim + 2 * gt + 4 + kSdpaWaves + 8) * sizeof(float));
    out_launch->set_args(a);
    return FK_OK;
}

}  // namespace fk
