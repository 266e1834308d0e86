// Dispatcher: named dispatch, hipGraph build / update / replay and the native
// per-token decode loop.  It replaces the Metal indirect-command-buffer runtime
// of the reference (python_runtime/src/lib.rs): build_icb -> fk_build_graph,
// update_icb_bindings -> fk_update_graph_bindings, execute_icb ->
// fk_execute_graph, decode_chunk_gpu_chain -> fk_decode_chunk.
//
// A dispatch names a kernel family by prefix ("fusekit_rmsnorm_qkv_f12" selects
// "fusekit_rmsnorm_qkv"), lists its buffers as (pointer, bytes) in the
// reference emitters' slot order and carries a small key/value parameter block
// (dims, eps, theta, bits ...) in place of the constants the reference bakes
// into kernel text.  Each family has a planner that validates the shapes and
// produces a Launch, and a read/write slot table from which hipGraph edges are
// derived (RAW, WAW and WAR on overlapping byte ranges), the equivalent of the
// reference's host-side barrier mask (python/fusekit_runtime/dispatch.py:36-100).
#include <math.h>

#include <algorithm>
#include <fstream>
#include <functional>
#include <memory>
#include <mutex>
#include <sstream>
#include <string>
#include <vector>

#include "decode_token.hpp"
#include "fk_host.hpp"
#include "fk_json.hpp"
#include "xcd_layer.hpp"

namespace fk {
namespace {

struct Dispatch {
    std::string kernel;
    std::vector<fk_arg> args;
    std::vector<std::pair<std::string, double>> params;

    double param(const char* key, double dflt) const {
        for (const auto& kv : params)
            if (kv.first == key) return kv.second;
        return dflt;
    }
    bool has(const char* key) const {
        for (const auto& kv : params)
            if (kv.first == key) return true;
        return false;
    }
    uint32_t u(const char* key, uint32_t dflt = 0) const { return (uint32_t)param(key, (double)dflt); }
};

struct SlotRW {
    std::vector<uint32_t> reads, writes;
};

template <typename T>
T* arg_ptr(const Dispatch& d, size_t slot) {
    return reinterpret_cast<T*>(d.args[slot].ptr);
}

fk_status need_args(const Dispatch& d, size_t n) {
    if (d.args.size() != n)
        return set_error(FK_ERR_INVALID, d.kernel + ": expected " + std::to_string(n) + " buffers, got " +
                                             std::to_string(d.args.size()));
    for (size_t i = 0; i < n; ++i)
        if (!d.args[i].ptr || d.args[i].nbytes == 0)
            return set_error(FK_ERR_INVALID, d.kernel + ": buffer slot " + std::to_string(i) + " is null or empty");
    return FK_OK;
}

fk_status need_bytes(const Dispatch& d, size_t slot, size_t bytes) {
    if (d.args[slot].nbytes < bytes)
        return set_error(FK_ERR_INVALID, d.kernel + ": buffer slot " + std::to_string(slot) + " holds " +
                                             std::to_string(d.args[slot].nbytes) + " bytes, kernel needs " +
                                             std::to_string(bytes));
    return FK_OK;
}

size_t weight_bytes(uint32_t n, uint32_t k, uint32_t bits) { return (size_t)n * k * bits / 8; }
size_t meta_bytes(uint32_t n, uint32_t k, uint32_t group) { return (size_t)n * (k / group) * 2; }

void all_but_last(size_t n, size_t last, SlotRW* rw) {
    for (uint32_t i = 0; i < n; ++i) (i + last < n ? rw->reads : rw->writes).push_back(i);
}

// Fills an fk_weight from consecutive slots: dense -> [W]; quantised -> W at
// `w_slot`, scales at `s_slot`, biases at `b_slot`.
fk_status bind_weight(const Dispatch& d, uint32_t bits, uint32_t group, uint32_t n, uint32_t k, size_t w_slot,
                      size_t s_slot, size_t b_slot, fk_weight* w) {
    if (bits != 4 && bits != 8 && bits != 16) return set_error(FK_ERR_UNSUPPORTED, d.kernel + ": bits must be 4, 8 or 16");
    w->w = d.args[w_slot].ptr;
    w->n = n;
    w->k = k;
    w->bits = bits;
    w->group = group;
    w->scales = w->biases = nullptr;
    FK_TRY(need_bytes(d, w_slot, weight_bytes(n, k, bits)));
    if (bits != 16) {
        if (group == 0 || k % group) return set_error(FK_ERR_INVALID, d.kernel + ": bad group size");
        w->scales = arg_ptr<const uint16_t>(d, s_slot);
        w->biases = arg_ptr<const uint16_t>(d, b_slot);
        FK_TRY(need_bytes(d, s_slot, meta_bytes(n, k, group)));
        FK_TRY(need_bytes(d, b_slot, meta_bytes(n, k, group)));
    }
    return FK_OK;
}

// ------------------------------------------------------------------ families

// step_counter, offset, kv_len, [rope_tab]  (the table: parameters rope_dims, theta)
fk_status plan_step(const Dispatch& d, Launch* l, SlotRW* rw) {
    FK_TRY(need_args(d, d.args.size() == 4 ? 4 : 3));
    for (int i = 0; i < 3; ++i) FK_TRY(need_bytes(d, i, 4));
    rw->reads = {0};
    rw->writes = {0, 1, 2};
    if (d.args.size() == 4) {
        const uint32_t rope_dims = d.u("rope_dims");
        if (rope_dims == 0) return set_error(FK_ERR_INVALID, d.kernel + ": rope_dims parameter missing");
        FK_TRY(need_bytes(d, 3, (size_t)rope_dims * 4));
        rw->writes.push_back(3);
        return plan_step_init(arg_ptr<uint32_t>(d, 0), arg_ptr<uint32_t>(d, 1), arg_ptr<uint32_t>(d, 2), l,
                              arg_ptr<float>(d, 3), rope_dims, (float)log2(d.param("theta", 10000.0)));
    }
    return plan_step_init(arg_ptr<uint32_t>(d, 0), arg_ptr<uint32_t>(d, 1), arg_ptr<uint32_t>(d, 2), l);
}

// dense: token, table, x ; quantised: token, packed, scales, biases, x
fk_status plan_embed_d(const Dispatch& d, Launch* l, SlotRW* rw) {
    const uint32_t bits = d.u("bits", 16), hidden = d.u("hidden"), vocab = d.u("vocab"), group = d.u("group", 64);
    const size_t n = bits == 16 ? 3 : 5;
    FK_TRY(need_args(d, n));
    fk_weight E;
    FK_TRY(bind_weight(d, bits, group, vocab, hidden, 1, 2, 3, &E));
    const uint32_t rows = d.u("rows", 1);  // active_m > 1: one token id and one output row per active row
    if (rows == 0) return set_error(FK_ERR_INVALID, d.kernel + ": rows must be at least 1");
    FK_TRY(need_bytes(d, 0, (size_t)rows * 4));
    FK_TRY(need_bytes(d, n - 1, (size_t)rows * hidden * 2));
    all_but_last(n, 1, rw);
    return plan_embed(&E, arg_ptr<const uint32_t>(d, 0), 0, (float)d.param("output_scale", 1.0),
                      arg_ptr<uint16_t>(d, n - 1), l, rows);
}

// x, [norm_w], W_q, W_k, W_v, [s_q, s_k, s_v, b_q, b_k, b_v], [bias_q, bias_k, bias_v], q, k, v
// (slot order of the reference emitter, src/codegen/kernels/rmsnorm_qkv.rs:159-204)
fk_status plan_qkv(const Dispatch& d, Launch* l, SlotRW* rw) {
    const uint32_t bits = d.u("bits", 4), group = d.u("group", 64), hidden = d.u("hidden");
    const uint32_t n_q = d.u("n_q"), n_kv = d.u("n_kv");
    const bool has_norm = d.u("has_norm", 1) != 0, has_bias = d.u("has_bias", 0) != 0;
    size_t s = 1;
    const size_t norm_slot = has_norm ? s++ : 0;
    const size_t w_slot = s;
    s += 3;
    const size_t meta_slot = s;
    if (bits != 16) s += 6;
    const size_t bias_slot = s;
    if (has_bias) s += 3;
    const size_t out_slot = s;
    s += 3;
    FK_TRY(need_args(d, s));
    GemvRequest rq;
    fk_weight W[3];
    const uint32_t ns[3] = {n_q, n_kv, n_kv};
    for (int m = 0; m < 3; ++m) {
        FK_TRY(bind_weight(d, bits, group, ns[m], hidden, w_slot + m, meta_slot + m, meta_slot + 3 + m, &W[m]));
        rq.mats[m] = &W[m];
        if (has_bias) {
            FK_TRY(need_bytes(d, bias_slot + m, (size_t)ns[m] * 2));
            rq.bias[m] = arg_ptr<const uint16_t>(d, bias_slot + m);
        }
        FK_TRY(need_bytes(d, out_slot + m, (size_t)ns[m] * 2));
        rq.y[m] = arg_ptr<uint16_t>(d, out_slot + m);
    }
    rq.n_mats = 3;
    const uint32_t rows = d.u("rows", 1);
    if (rows > 1) {
        // Row form (2 .. 8 token rows, the prefill_mN variants' and the multi-row passes' shape): x [rows, x_row_stride],
        // outputs [rows, q / k / v_row_stride] (defaults: dense rows), one shared-stream launch for the three matrices
        // with the norm applied while the rows are staged.
        if (has_bias) return set_error(FK_ERR_UNSUPPORTED, d.kernel + ": the row form takes no bias");
        const uint32_t xs = d.u("x_row_stride", hidden);
        const uint32_t ys[3] = {d.u("q_row_stride", n_q), d.u("k_row_stride", n_kv), d.u("v_row_stride", n_kv)};
        if (xs < hidden) return set_error(FK_ERR_INVALID, d.kernel + ": x_row_stride below hidden");
        FK_TRY(need_bytes(d, 0, ((size_t)(rows - 1) * xs + hidden) * 2));
        WideSeg segs[3];
        for (int m = 0; m < 3; ++m) {
            if (ys[m] < ns[m]) return set_error(FK_ERR_INVALID, d.kernel + ": output row stride below the matrix's rows");
            FK_TRY(need_bytes(d, out_slot + m, ((size_t)(rows - 1) * ys[m] + ns[m]) * 2));
            segs[m] = WideSeg{&W[m], arg_ptr<uint16_t>(d, out_slot + m), ys[m]};
        }
        const uint16_t* nw = nullptr;
        if (has_norm) {
            FK_TRY(need_bytes(d, norm_slot, (size_t)hidden * 2));
            nw = arg_ptr<const uint16_t>(d, norm_slot);
        }
        all_but_last(s, 3, rw);
        return plan_qgemm_wide_fan(arg_ptr<const uint16_t>(d, 0), xs, rows, nw, (float)d.param("eps", 1e-6), segs, 3, l);
    }
    FK_TRY(need_bytes(d, 0, (size_t)hidden * 2));
    rq.x = arg_ptr<const uint16_t>(d, 0);
    if (has_norm) {
        FK_TRY(need_bytes(d, norm_slot, (size_t)hidden * 2));
        rq.norm_w = arg_ptr<const uint16_t>(d, norm_slot);
    }
    rq.eps = (float)d.param("eps", 1e-6);
    all_but_last(s, 3, rw);
    return plan_gemv(rq, l);
}

// x, [norm_w], W_gate, W_up, [s_g, s_u, b_g, b_u], out
fk_status plan_gateup(const Dispatch& d, Launch* l, SlotRW* rw) {
    const uint32_t bits = d.u("bits", 4), group = d.u("group", 64), hidden = d.u("hidden"), inter = d.u("inter");
    const bool has_norm = d.u("has_norm", 1) != 0;
    size_t s = 1;
    const size_t norm_slot = has_norm ? s++ : 0;
    const size_t w_slot = s;
    s += 2;
    const size_t meta_slot = s;
    if (bits != 16) s += 4;
    const size_t out_slot = s++;
    FK_TRY(need_args(d, s));
    GemvRequest rq;
    fk_weight W[2];
    for (int m = 0; m < 2; ++m) {
        FK_TRY(bind_weight(d, bits, group, inter, hidden, w_slot + m, meta_slot + m, meta_slot + 2 + m, &W[m]));
        rq.mats[m] = &W[m];
    }
    rq.swiglu = true;
    const int variant = (int)d.param("variant", 0);
    if (variant < 0 || variant > 2) return set_error(FK_ERR_INVALID, d.kernel + ": swiglu variant must be 0, 1 or 2");
    rq.swiglu_variant = variant;
    const uint32_t rows = d.u("rows", 1);
    if (rows > 1) {
        // Row form (2 .. 8 token rows): x [rows, hidden], out [rows, inter]; the pair streamed once for all rows by the
        // shared-stream matmul, the norm applied while the rows are staged.
        if (bits == 16) return set_error(FK_ERR_UNSUPPORTED, d.kernel + ": the row form takes 4- or 8-bit weights");
        FK_TRY(need_bytes(d, 0, (size_t)rows * hidden * 2));
        FK_TRY(need_bytes(d, out_slot, (size_t)rows * inter * 2));
        const uint16_t* nw = nullptr;
        if (has_norm) {
            FK_TRY(need_bytes(d, norm_slot, (size_t)hidden * 2));
            nw = arg_ptr<const uint16_t>(d, norm_slot);
        }
        all_but_last(s, 1, rw);
        if (rows > 8 || group != 64) return set_error(FK_ERR_UNSUPPORTED, d.kernel + ": the row form takes 2..8 rows and group size 64");
        return plan_qgemm_wide(&W[0], &W[1], arg_ptr<const uint16_t>(d, 0), rows, nullptr, nullptr, variant,
                               arg_ptr<uint16_t>(d, out_slot), l, nw, (float)d.param("eps", 1e-6));
    }
    FK_TRY(need_bytes(d, 0, (size_t)hidden * 2));
    FK_TRY(need_bytes(d, out_slot, (size_t)inter * 2));
    rq.x = arg_ptr<const uint16_t>(d, 0);
    rq.y[0] = arg_ptr<uint16_t>(d, out_slot);
    if (has_norm) {
        FK_TRY(need_bytes(d, norm_slot, (size_t)hidden * 2));
        rq.norm_w = arg_ptr<const uint16_t>(d, norm_slot);
    }
    rq.eps = (float)d.param("eps", 1e-6);
    all_but_last(s, 1, rw);
    return plan_gemv(rq, l);
}

// x, W, [scales, biases], residual, [residual_extra], y   (K = "m", N = "n")
fk_status plan_linres(const Dispatch& d, Launch* l, SlotRW* rw) {
    const uint32_t bits = d.u("bits", 4), group = d.u("group", 64), K = d.u("m"), N = d.u("n");
    const bool extra = d.u("has_extra", 0) != 0;
    size_t s = 2;
    if (bits != 16) s += 2;
    const size_t res_slot = s++;
    const size_t extra_slot = extra ? s++ : 0;
    const size_t out_slot = s++;
    FK_TRY(need_args(d, s));
    GemvRequest rq;
    fk_weight W;
    FK_TRY(bind_weight(d, bits, group, N, K, 1, 2, 3, &W));
    rq.mats[0] = &W;
    FK_TRY(need_bytes(d, 0, (size_t)K * 2));
    FK_TRY(need_bytes(d, res_slot, (size_t)N * 2));
    FK_TRY(need_bytes(d, out_slot, (size_t)N * 2));
    rq.x = arg_ptr<const uint16_t>(d, 0);
    rq.res = arg_ptr<const uint16_t>(d, res_slot);
    if (extra) {
        FK_TRY(need_bytes(d, extra_slot, (size_t)N * 2));
        rq.res2 = arg_ptr<const uint16_t>(d, extra_slot);
    }
    rq.y[0] = arg_ptr<uint16_t>(d, out_slot);
    all_but_last(s, 1, rw);
    return plan_gemv(rq, l);
}

// x, W, [scales, biases], [bias], y
fk_status plan_qgemv_d(const Dispatch& d, Launch* l, SlotRW* rw) {
    const uint32_t bits = d.u("bits", 4), group = d.u("group", 64), K = d.u("m"), N = d.u("n");
    const bool has_bias = d.u("has_bias", 0) != 0;
    size_t s = 2;
    if (bits != 16) s += 2;
    const size_t bias_slot = has_bias ? s++ : 0;
    const size_t out_slot = s++;
    FK_TRY(need_args(d, s));
    GemvRequest rq;
    fk_weight W;
    FK_TRY(bind_weight(d, bits, group, N, K, 1, 2, 3, &W));
    rq.mats[0] = &W;
    FK_TRY(need_bytes(d, 0, (size_t)K * 2));
    FK_TRY(need_bytes(d, out_slot, (size_t)N * 2));
    rq.x = arg_ptr<const uint16_t>(d, 0);
    if (has_bias) {
        FK_TRY(need_bytes(d, bias_slot, (size_t)N * 2));
        rq.bias[0] = arg_ptr<const uint16_t>(d, bias_slot);
    }
    rq.y[0] = arg_ptr<uint16_t>(d, out_slot);
    all_but_last(s, 1, rw);
    return plan_gemv(rq, l);
}

// x, norm_w, W, [scales, biases], logits
// argmax: the direct head; slots behind the logits are next_tok, workspace [, history, hist_counter].
fk_status plan_lm_head(const Dispatch& d, Launch* l, SlotRW* rw, bool argmax) {
    const uint32_t bits = d.u("bits", 16), group = d.u("group", 64), hidden = d.u("hidden"), vocab = d.u("vocab");
    size_t s = 3;
    if (bits != 16) s += 2;
    const size_t out_slot = s++;
    HeadArgmax am;
    if (argmax) {
        const bool hist = d.args.size() == s + 4;
        FK_TRY(need_args(d, s + (hist ? 4 : 2)));
        FK_TRY(need_bytes(d, s, 4));
        FK_TRY(need_bytes(d, s + 1, kHeadArgmaxWorkspaceBytes));
        am.next_token = arg_ptr<uint32_t>(d, s);
        am.workspace = d.args[s + 1].ptr;
        if (hist) {
            FK_TRY(need_bytes(d, s + 3, 4));
            am.history = arg_ptr<uint32_t>(d, s + 2);
            am.hist_counter = arg_ptr<uint32_t>(d, s + 3);
            am.hist_capacity = (uint32_t)(d.args[s + 2].nbytes / 4);
        }
        for (size_t i = 0; i < out_slot; ++i) rw->reads.push_back((uint32_t)i);
        rw->reads.push_back((uint32_t)(s + 1));
        for (size_t i = out_slot; i < d.args.size(); ++i) rw->writes.push_back((uint32_t)i);
        if (hist) rw->reads.push_back((uint32_t)(s + 3));
    } else {
        FK_TRY(need_args(d, s));
    }
    GemvRequest rq;
    fk_weight W;
    FK_TRY(bind_weight(d, bits, group, vocab, hidden, 2, 3, 4, &W));
    rq.mats[0] = &W;
    FK_TRY(need_bytes(d, 0, (size_t)hidden * 2));
    FK_TRY(need_bytes(d, 1, (size_t)hidden * 2));
    FK_TRY(need_bytes(d, out_slot, (size_t)vocab * 2));
    rq.x = arg_ptr<const uint16_t>(d, 0);
    rq.norm_w = arg_ptr<const uint16_t>(d, 1);
    rq.eps = (float)d.param("eps", 1e-6);
    rq.y[0] = arg_ptr<uint16_t>(d, out_slot);
    if (argmax)
        rq.argmax = &am;
    else
        all_but_last(s, 1, rw);
    return plan_gemv(rq, l);
}

float base_log2_of(const Dispatch& d) { return (float)log2(d.param("theta", 10000.0)); }

// Q, [q_weight], offset
fk_status plan_rope_q(const Dispatch& d, Launch* l, SlotRW* rw, bool norm) {
    const size_t n = norm ? 3 : 2;
    FK_TRY(need_args(d, n));
    RopeArgs a;
    memset(&a, 0, sizeof(a));
    a.n_q = d.u("n_heads");
    a.head_dim = d.u("head_dim");
    a.rope_dims = d.u("rope_dims", a.head_dim);
    a.rope_on = a.rope_dims ? 1u : 0u;
    FK_TRY(need_bytes(d, 0, (size_t)a.n_q * a.head_dim * 2));
    a.q = arg_ptr<uint16_t>(d, 0);
    if (norm) {
        FK_TRY(need_bytes(d, 1, (size_t)a.head_dim * 2));
        a.q_norm = arg_ptr<const uint16_t>(d, 1);
    }
    FK_TRY(need_bytes(d, n - 1, 4));
    a.offset_ptr = arg_ptr<const uint32_t>(d, n - 1);
    a.eps = (float)d.param("eps", 1e-6);
    a.base_log2 = base_log2_of(d);
    a.capacity = 1;
    for (uint32_t i = 0; i < n; ++i) rw->reads.push_back(i);
    rw->writes = {0};
    return plan_rope_store(a, l);
}

// [Q], K0, K1, V, cache_k, cache_v, offset, write_offset: the split-key form of kv_cache_store_decode
// (kv_cache_store_decode.rs:206-214), with has_q = 1 also the in-place rotation of the query's second part.
// Parameters: n_kv, k0_dim, k1_dim, v_dim, k1_n_kv, k0_stride, v_stride, rope_dims, traditional, theta,
// capacity; with a query n_heads, q0_dim, q1_dim.
fk_status plan_kv_store_split(const Dispatch& d, Launch* l, SlotRW* rw) {
    const bool has_q = d.u("has_q", 0) != 0;
    const size_t b = has_q ? 1 : 0;
    FK_TRY(need_args(d, b + 7));
    SplitStoreArgs a;
    memset(&a, 0, sizeof(a));
    a.n_kv = d.u("n_kv");
    a.k0_dim = d.u("k0_dim");
    a.k1_dim = d.u("k1_dim");
    a.v_dim = d.u("v_dim");
    a.k1_heads = d.u("k1_n_kv", a.n_kv);
    a.k0_stride = d.u("k0_stride", a.k0_dim);
    a.v_stride = d.u("v_stride", a.v_dim);
    a.rope_dims = d.u("rope_dims", 0);
    a.traditional = d.u("traditional", 0);
    a.capacity = d.u("capacity");
    if (a.n_kv == 0 || a.k0_dim == 0 || a.k1_dim == 0 || a.v_dim == 0 || a.capacity == 0 || a.k1_heads == 0)
        return set_error(FK_ERR_INVALID, d.kernel + ": n_kv / k0_dim / k1_dim / v_dim / capacity parameters missing");
    if (a.k0_stride < a.k0_dim || a.v_stride < a.v_dim) return set_error(FK_ERR_INVALID, d.kernel + ": stride below the row width");
    // rows > 1 (row r at position offset + r): token rows k0_row_stride / k1_row_stride / v_row_stride elements apart
    a.rows = d.u("rows", 1);
    a.k0_row_stride = d.u("k0_row_stride", a.n_kv * a.k0_stride);
    a.k1_row_stride = d.u("k1_row_stride", a.k1_heads * a.k1_dim);
    a.v_row_stride = d.u("v_row_stride", a.n_kv * a.v_stride);
    if (a.rows == 0) return set_error(FK_ERR_INVALID, d.kernel + ": rows must be positive");
    const size_t more = a.rows - 1;
    if (has_q) {
        a.n_heads = d.u("n_heads");
        a.q0_dim = d.u("q0_dim");
        a.q1_dim = d.u("q1_dim");
        if (a.n_heads == 0) return set_error(FK_ERR_INVALID, d.kernel + ": n_heads parameter missing");
        FK_TRY(need_bytes(d, 0, (size_t)a.rows * a.n_heads * (a.q0_dim + a.q1_dim) * 2));
        a.q = arg_ptr<uint16_t>(d, 0);
    }
    FK_TRY(need_bytes(d, b, (more * a.k0_row_stride + (size_t)(a.n_kv - 1) * a.k0_stride + a.k0_dim) * 2));
    FK_TRY(need_bytes(d, b + 1, (more * a.k1_row_stride + (size_t)a.k1_heads * a.k1_dim) * 2));
    FK_TRY(need_bytes(d, b + 2, (more * a.v_row_stride + (size_t)(a.n_kv - 1) * a.v_stride + a.v_dim) * 2));
    FK_TRY(need_bytes(d, b + 3, (size_t)a.n_kv * a.capacity * (a.k0_dim + a.k1_dim) * 2));
    FK_TRY(need_bytes(d, b + 4, (size_t)a.n_kv * a.capacity * a.v_dim * 2));
    FK_TRY(need_bytes(d, b + 5, 4));
    FK_TRY(need_bytes(d, b + 6, 4));
    a.k0 = arg_ptr<const uint16_t>(d, b);
    a.k1 = arg_ptr<const uint16_t>(d, b + 1);
    a.v = arg_ptr<const uint16_t>(d, b + 2);
    a.cache_k = arg_ptr<uint16_t>(d, b + 3);
    a.cache_v = arg_ptr<uint16_t>(d, b + 4);
    a.offset_ptr = arg_ptr<const uint32_t>(d, b + 5);
    a.write_offset_ptr = arg_ptr<const uint32_t>(d, b + 6);
    a.base_log2 = a.rope_dims ? base_log2_of(d) : 0.f;
    for (uint32_t i = 0; i < b + 7; ++i)
        if (i != b + 3 && i != b + 4) rw->reads.push_back(i);
    rw->writes = {(uint32_t)(b + 3), (uint32_t)(b + 4)};
    if (has_q) rw->writes.push_back(0);
    return plan_split_rope_store(a, l);
}

// logits, scale, idx, weight (SoftmaxTopKRoute, single.rs:2615-2760).  Parameters: row_n, top_k, rows,
// scale_per_route.
fk_status plan_softmax_topk_route_d(const Dispatch& d, Launch* l, SlotRW* rw) {
    FK_TRY(need_args(d, 4));
    const uint32_t row_n = d.u("row_n"), top_k = d.u("top_k"), rows = d.u("rows", 1);
    const bool per_route = d.u("scale_per_route", 0) != 0;
    if (row_n == 0 || top_k == 0 || rows == 0) return set_error(FK_ERR_INVALID, d.kernel + ": row_n / top_k parameters missing");
    FK_TRY(need_bytes(d, 0, (size_t)rows * row_n * 2));
    FK_TRY(need_bytes(d, 1, per_route ? (size_t)rows * top_k * 2 : 2));
    FK_TRY(need_bytes(d, 2, (size_t)rows * top_k * 4));
    FK_TRY(need_bytes(d, 3, (size_t)rows * top_k * 2));
    rw->reads = {0, 1};
    rw->writes = {2, 3};
    return plan_softmax_topk_route(arg_ptr<const uint16_t>(d, 0), arg_ptr<const uint16_t>(d, 1), per_route, rows, row_n, top_k,
                                   arg_ptr<uint32_t>(d, 2), arg_ptr<uint16_t>(d, 3), l);
}

// x, [norm_w], router_w, scale, xn, logits, idx, weight, workspace: norm + router projection + softmax top-k
// route in one launch.  Parameters: hidden, experts, top_k, eps, has_norm.
fk_status plan_moe_router_d(const Dispatch& d, Launch* l, SlotRW* rw) {
    const bool has_norm = d.u("has_norm", 1) != 0;
    const size_t b = has_norm ? 2 : 1;
    FK_TRY(need_args(d, b + 7));
    const uint32_t hidden = d.u("hidden"), experts = d.u("experts"), top_k = d.u("top_k"), rows = d.u("rows", 1);
    if (hidden == 0 || experts == 0 || rows == 0) return set_error(FK_ERR_INVALID, d.kernel + ": hidden / experts parameters missing");
    FK_TRY(need_bytes(d, 0, (size_t)rows * hidden * 2));
    if (has_norm) FK_TRY(need_bytes(d, 1, (size_t)hidden * 2));
    FK_TRY(need_bytes(d, b, (size_t)experts * hidden * 2));
    FK_TRY(need_bytes(d, b + 1, 2));
    FK_TRY(need_bytes(d, b + 2, (size_t)rows * hidden * 2));
    FK_TRY(need_bytes(d, b + 3, (size_t)rows * experts * 2));
    if (top_k) {   // top_k = 0: the logits are the output and the last three slots are not touched
        FK_TRY(need_bytes(d, b + 4, (size_t)rows * top_k * 4));
        FK_TRY(need_bytes(d, b + 5, (size_t)rows * top_k * 2));
        FK_TRY(need_bytes(d, b + 6, (size_t)rows * (experts + 1) * 4));
    }
    for (uint32_t i = 0; i < b + 2; ++i) rw->reads.push_back(i);
    rw->reads.push_back((uint32_t)(b + 6));
    for (uint32_t i = b + 2; i < b + 7; ++i) rw->writes.push_back(i);
    return plan_moe_router(arg_ptr<const uint16_t>(d, 0), has_norm ? arg_ptr<const uint16_t>(d, 1) : nullptr,
                           (float)d.param("eps", 1e-6), arg_ptr<const uint16_t>(d, b), arg_ptr<const uint16_t>(d, b + 1), hidden,
                           experts, top_k, arg_ptr<uint16_t>(d, b + 2), arg_ptr<uint16_t>(d, b + 3), arg_ptr<uint32_t>(d, b + 4),
                           arg_ptr<uint16_t>(d, b + 5), arg_ptr<uint32_t>(d, b + 6), l, rows);
}

// K, V, [k_weight], cache_k, cache_v, offset, write_offset
fk_status plan_rope_kv(const Dispatch& d, Launch* l, SlotRW* rw, bool norm, bool rope) {
    const size_t n = norm ? 7 : 6;
    FK_TRY(need_args(d, n));
    const size_t ck = norm ? 3 : 2;
    RopeArgs a;
    memset(&a, 0, sizeof(a));
    a.n_kv = d.u("n_kv");
    a.k_dim = d.u("head_dim");
    a.v_dim = d.u("v_dim", a.k_dim);
    a.rope_dims = rope ? d.u("rope_dims", a.k_dim) : 0;
    a.rope_on = a.rope_dims ? 1u : 0u;
    a.capacity = d.u("capacity");
    if (a.capacity == 0) return set_error(FK_ERR_INVALID, d.kernel + ": capacity parameter missing");
    FK_TRY(need_bytes(d, 0, (size_t)a.n_kv * a.k_dim * 2));
    FK_TRY(need_bytes(d, 1, (size_t)a.n_kv * a.v_dim * 2));
    FK_TRY(need_bytes(d, ck, (size_t)a.n_kv * a.capacity * a.k_dim * 2));
    FK_TRY(need_bytes(d, ck + 1, (size_t)a.n_kv * a.capacity * a.v_dim * 2));
    FK_TRY(need_bytes(d, ck + 2, 4));
    FK_TRY(need_bytes(d, ck + 3, 4));
    a.k = arg_ptr<const uint16_t>(d, 0);
    a.v = arg_ptr<const uint16_t>(d, 1);
    if (norm) {
        FK_TRY(need_bytes(d, 2, (size_t)a.k_dim * 2));
        a.k_norm = arg_ptr<const uint16_t>(d, 2);
    }
    a.cache_k = arg_ptr<uint16_t>(d, ck);
    a.cache_v = arg_ptr<uint16_t>(d, ck + 1);
    a.offset_ptr = arg_ptr<const uint32_t>(d, ck + 2);
    a.write_offset_ptr = arg_ptr<const uint32_t>(d, ck + 3);
    a.eps = (float)d.param("eps", 1e-6);
    a.base_log2 = base_log2_of(d);
    for (uint32_t i = 0; i < n; ++i)
        if (i != ck && i != ck + 1) rw->reads.push_back(i);
    rw->writes = {(uint32_t)ck, (uint32_t)ck + 1};
    return plan_rope_store(a, l);
}

// Q, K, V, [q_weight, k_weight], cache_k, cache_v, offset   (one launch for the whole rope/store stage)
fk_status plan_qkv_rope_store(const Dispatch& d, Launch* l, SlotRW* rw) {
    const bool norm = d.u("has_norm", 0) != 0;
    const size_t n = norm ? 8 : 6;
    FK_TRY(need_args(d, n));
    const size_t ck = norm ? 5 : 3;
    RopeArgs a;
    memset(&a, 0, sizeof(a));
    a.n_q = d.u("n_heads");
    a.n_kv = d.u("n_kv");
    a.head_dim = a.k_dim = a.v_dim = d.u("head_dim");
    a.rope_dims = d.u("rope_dims", a.head_dim);
    a.rope_on = a.rope_dims ? 1u : 0u;
    a.capacity = d.u("capacity");
    if (a.capacity == 0) return set_error(FK_ERR_INVALID, d.kernel + ": capacity parameter missing");
    a.rows = d.u("rows", 1);  // active_m > 1: row r is the token at position offset + r
    if (a.rows == 0) return set_error(FK_ERR_INVALID, d.kernel + ": rows must be at least 1");
    FK_TRY(need_bytes(d, 0, (size_t)a.rows * a.n_q * a.head_dim * 2));
    FK_TRY(need_bytes(d, 1, (size_t)a.rows * a.n_kv * a.head_dim * 2));
    FK_TRY(need_bytes(d, 2, (size_t)a.rows * a.n_kv * a.head_dim * 2));
    FK_TRY(need_bytes(d, ck, (size_t)a.n_kv * a.capacity * a.head_dim * 2));
    FK_TRY(need_bytes(d, ck + 1, (size_t)a.n_kv * a.capacity * a.head_dim * 2));
    FK_TRY(need_bytes(d, ck + 2, 4));
    a.q = arg_ptr<uint16_t>(d, 0);
    a.k = arg_ptr<const uint16_t>(d, 1);
    a.v = arg_ptr<const uint16_t>(d, 2);
    if (norm) {
        FK_TRY(need_bytes(d, 3, (size_t)a.head_dim * 2));
        FK_TRY(need_bytes(d, 4, (size_t)a.head_dim * 2));
        a.q_norm = arg_ptr<const uint16_t>(d, 3);
        a.k_norm = arg_ptr<const uint16_t>(d, 4);
    }
    a.cache_k = arg_ptr<uint16_t>(d, ck);
    a.cache_v = arg_ptr<uint16_t>(d, ck + 1);
    a.offset_ptr = arg_ptr<const uint32_t>(d, ck + 2);
    a.eps = (float)d.param("eps", 1e-6);
    a.base_log2 = base_log2_of(d);
    for (uint32_t i = 0; i < n; ++i)
        if (i != ck && i != ck + 1) rw->reads.push_back(i);
    rw->writes = {0, (uint32_t)ck, (uint32_t)ck + 1};
    return plan_rope_store(a, l);
}

// Q, K, V, kv_len, out, partials, counters
fk_status plan_sdpa_d(const Dispatch& d, Launch* l, SlotRW* rw) {
    FK_TRY(need_args(d, 7));
    const uint32_t n_heads = d.u("n_heads"), n_kv = d.u("n_kv"), qk = d.u("qk_dim", d.u("head_dim"));
    const uint32_t vd = d.u("v_dim", qk), capacity = d.u("capacity"), max_len = d.u("max_len", capacity);
    if (n_heads == 0 || n_kv == 0 || qk == 0 || capacity == 0)
        return set_error(FK_ERR_INVALID, d.kernel + ": n_heads / n_kv / head_dim / capacity parameters missing");
    const float scale = d.has("scale") ? (float)d.param("scale", 0) : 1.0f / sqrtf((float)qk);  // sdpa_decode.rs:248-252
    // rows > 1: row r of q / out attends to kv_len + r positions (kv_len is row 0's); workspace per row
    const uint32_t rows = d.u("rows", 1);
    if (rows == 0) return set_error(FK_ERR_INVALID, d.kernel + ": rows must be positive");
    FK_TRY(need_bytes(d, 0, (size_t)rows * n_heads * qk * 2));
    FK_TRY(need_bytes(d, 1, (size_t)n_kv * capacity * qk * 2));
    FK_TRY(need_bytes(d, 2, (size_t)n_kv * capacity * vd * 2));
    FK_TRY(need_bytes(d, 3, 4));
    FK_TRY(need_bytes(d, 4, (size_t)rows * n_heads * vd * 2));
    size_t pb = 0, cb = 0;
    FK_TRY(sdpa_workspace_bytes(n_heads, n_kv, qk, vd, max_len, &pb, &cb));
    FK_TRY(need_bytes(d, 5, pb * rows));
    FK_TRY(need_bytes(d, 6, cb * rows));
    rw->reads = {0, 1, 2, 3, 5, 6};
    rw->writes = {4, 5, 6};
    return plan_sdpa_decode(arg_ptr<const uint16_t>(d, 0), arg_ptr<const uint16_t>(d, 1), arg_ptr<const uint16_t>(d, 2),
                            arg_ptr<uint16_t>(d, 4), arg_ptr<const uint32_t>(d, 3), 0, max_len, n_heads, n_kv, qk, vd,
                            capacity, scale, arg_ptr<float>(d, 5), arg_ptr<uint32_t>(d, 6), l, rows);
}

// Q, K, V, out: causal attention of `rows` token rows (sdpa_prefill.rs:11-21).  The reference binds
// kv_len, L and capacity as uniforms; here they are the parameters kv_len, rows and capacity,
// because the grid depends on them.
fk_status plan_sdpa_prefill_d(const Dispatch& d, Launch* l, SlotRW* rw) {
    // five slots: Q, K, V, kv_len (device uint32, read at run time: the graph is replayed for any offset), out
    const bool dev_len = d.args.size() == 5;
    FK_TRY(need_args(d, dev_len ? 5 : 4));
    const size_t out_slot = dev_len ? 4 : 3;
    const uint32_t n_heads = d.u("n_heads"), n_kv = d.u("n_kv"), dim = d.u("head_dim"), capacity = d.u("capacity");
    const uint32_t rows = d.u("rows"), kv_len = dev_len ? rows : d.u("kv_len");
    if (dev_len) FK_TRY(need_bytes(d, 3, 4));
    if (n_heads == 0 || n_kv == 0 || dim == 0 || capacity == 0 || rows == 0)
        return set_error(FK_ERR_INVALID, d.kernel + ": n_heads / n_kv / head_dim / capacity / rows parameters missing");
    const float scale = d.has("scale") ? (float)d.param("scale", 0) : 1.0f / sqrtf((float)dim);  // sdpa_prefill.rs:52
    FK_TRY(need_bytes(d, 0, (size_t)rows * n_heads * dim * 2));
    FK_TRY(need_bytes(d, 1, (size_t)n_kv * capacity * dim * 2));
    FK_TRY(need_bytes(d, 2, (size_t)n_kv * capacity * dim * 2));
    FK_TRY(need_bytes(d, out_slot, (size_t)rows * n_heads * dim * 2));
    rw->reads = {0, 1, 2};
    if (dev_len) rw->reads.push_back(3);
    rw->writes = {(uint32_t)out_slot};
    return plan_sdpa_prefill(arg_ptr<const uint16_t>(d, 0), arg_ptr<const uint16_t>(d, 1), arg_ptr<const uint16_t>(d, 2),
                             arg_ptr<uint16_t>(d, out_slot), rows, kv_len, n_heads, n_kv, dim, capacity, scale, l,
                             dev_len ? arg_ptr<const uint32_t>(d, 3) : nullptr);
}

// x, weight, out: RMSNorm of `rows` rows, T(w * T(x * r)) (the norm stage of the reference's multi-row
// variants, which fuse it into their matmul prologue)
fk_status plan_rmsnorm_rows_d(const Dispatch& d, Launch* l, SlotRW* rw) {
    FK_TRY(need_args(d, 3));
    const uint32_t rows = d.u("rows"), hidden = d.u("hidden");
    if (rows == 0 || hidden == 0) return set_error(FK_ERR_INVALID, d.kernel + ": rows / hidden parameters missing");
    FK_TRY(need_bytes(d, 0, (size_t)rows * hidden * 2));
    FK_TRY(need_bytes(d, 1, (size_t)hidden * 2));
    FK_TRY(need_bytes(d, 2, (size_t)rows * hidden * 2));
    rw->reads = {0, 1};
    rw->writes = {2};
    return plan_rmsnorm_rows(arg_ptr<const uint16_t>(d, 0), arg_ptr<const uint16_t>(d, 1), (float)d.param("eps", 1e-6), rows, hidden,
                             arg_ptr<uint16_t>(d, 2), l);
}

// Q, K, V, [q_weight, k_weight], cache_k, cache_v, kv_len, out, partials, counters, [rope_tab]
// (one launch for the rope/store stage and the attention of a layer)
fk_status plan_rope_store_sdpa(const Dispatch& d, Launch* l, SlotRW* rw) {
    const bool norm = d.u("has_norm", 0) != 0, table = d.u("has_table", 0) != 0;
    const size_t c0 = norm ? 5 : 3, n = c0 + 6 + (table ? 1 : 0);
    FK_TRY(need_args(d, n));
    const uint32_t n_heads = d.u("n_heads"), n_kv = d.u("n_kv"), dim = d.u("head_dim");
    const uint32_t capacity = d.u("capacity"), max_len = d.u("max_len", capacity);
    if (n_heads == 0 || n_kv == 0 || dim == 0 || capacity == 0)
        return set_error(FK_ERR_INVALID, d.kernel + ": n_heads / n_kv / head_dim / capacity parameters missing");
    const float scale = d.has("scale") ? (float)d.param("scale", 0) : 1.0f / sqrtf((float)dim);
    SdpaFusion f;
    f.rope_dims = d.u("rope_dims", dim);
    f.eps = (float)d.param("eps", 1e-6);
    f.base_log2 = base_log2_of(d);
    FK_TRY(need_bytes(d, 0, (size_t)n_heads * dim * 2));
    FK_TRY(need_bytes(d, 1, (size_t)n_kv * dim * 2));
    FK_TRY(need_bytes(d, 2, (size_t)n_kv * dim * 2));
    f.k_new = arg_ptr<const uint16_t>(d, 1);
    f.v_new = arg_ptr<const uint16_t>(d, 2);
    if (norm) {
        FK_TRY(need_bytes(d, 3, (size_t)dim * 2));
        FK_TRY(need_bytes(d, 4, (size_t)dim * 2));
        f.q_norm = arg_ptr<const uint16_t>(d, 3);
        f.k_norm = arg_ptr<const uint16_t>(d, 4);
    }
    FK_TRY(need_bytes(d, c0, (size_t)n_kv * capacity * dim * 2));
    FK_TRY(need_bytes(d, c0 + 1, (size_t)n_kv * capacity * dim * 2));
    FK_TRY(need_bytes(d, c0 + 2, 4));
    FK_TRY(need_bytes(d, c0 + 3, (size_t)n_heads * dim * 2));
    size_t pb = 0, cb = 0;
    FK_TRY(sdpa_workspace_bytes(n_heads, n_kv, dim, dim, max_len, &pb, &cb));
    FK_TRY(need_bytes(d, c0 + 4, pb));
    FK_TRY(need_bytes(d, c0 + 5, cb));
    if (table) {
        FK_TRY(need_bytes(d, c0 + 6, (size_t)f.rope_dims * 4));
        f.rope_tab = arg_ptr<const float>(d, c0 + 6);
    }
    for (uint32_t i = 0; i < n; ++i)
        if (i != c0 + 3) rw->reads.push_back(i);
    rw->writes = {(uint32_t)c0, (uint32_t)c0 + 1, (uint32_t)c0 + 3, (uint32_t)c0 + 4, (uint32_t)c0 + 5};
    return plan_sdpa_decode(arg_ptr<const uint16_t>(d, 0), arg_ptr<const uint16_t>(d, c0),
                            arg_ptr<const uint16_t>(d, c0 + 1), arg_ptr<uint16_t>(d, c0 + 3),
                            arg_ptr<const uint32_t>(d, c0 + 2), 0, max_len, n_heads, n_kv, dim, dim, capacity, scale,
                            arg_ptr<float>(d, c0 + 4), arg_ptr<uint32_t>(d, c0 + 5), l, 1, nullptr, &f);
}

// ---- XCD-resident layer (xcd_layer.hpp): two launches per layer -------------------------------------
XcdLayerShape xcd_shape(const Dispatch& d) {
    XcdLayerShape s;
    s.hidden = d.u("hidden");
    s.inter = d.u("inter");
    s.n_heads = d.u("n_heads");
    s.n_kv = d.u("n_kv");
    s.head_dim = d.u("head_dim");
    s.capacity = d.u("capacity");
    s.bits = d.u("bits", 4);
    s.group = d.u("group", 64);
    return s;
}

// [sums_in], residual, x_out, norm_w, W_q, W_k, W_v, [s_q, s_k, s_v, b_q, b_k, b_v], W_o, [s_o, b_o],
// [q_norm, k_norm], q, k, v, cache_k, cache_v, kv_len, rope_tab, att_partials, out_sums, clear_sums, workspace
// (sums_in: the sum row the previous launch added into; out_sums: the row this launch adds into, zero on entry;
// clear_sums: the row this launch zeroes; residual and x_out: one bf16 row each.)
// Parameters: the layer shape (hidden, inter, n_heads, n_kv, head_dim, capacity, bits, group), eps, theta,
// has_sums, has_norm, spin_limit, mark_placement (every block flips its bit of its XCD's placement word as it ends;
// set on one launch per token).
fk_status plan_xcd_attn_d(const Dispatch& d, Launch* l, SlotRW* rw) {
    const XcdLayerShape s = xcd_shape(d);
    const bool has_p = d.u("has_sums", 1) != 0, norm = d.u("has_norm", 0) != 0, q = s.bits != 16;
    size_t i = 0;
    const size_t p_slot = has_p ? i++ : 0, res_slot = i++, x_slot = i++, nw_slot = i++, w_slot = i;
    i += 3;
    const size_t meta_slot = i;
    if (q) i += 6;
    const size_t wo_slot = i++;
    const size_t wo_meta = i;
    if (q) i += 2;
    const size_t hn_slot = i;
    if (norm) i += 2;
    const size_t q_slot = i;
    i += 3;
    const size_t ck_slot = i++, cv_slot = i++, len_slot = i++, tab_slot = i++, ap_slot = i++, op_slot = i++, clr_slot = i++,
                 ws_slot = i++;
    FK_TRY(need_args(d, i));
    if (s.hidden == 0 || s.n_heads == 0 || s.n_kv == 0 || s.head_dim == 0 || s.capacity == 0)
        return set_error(FK_ERR_INVALID, d.kernel + ": layer shape parameters missing");
    const uint32_t n_q = s.n_heads * s.head_dim, n_kvd = s.n_kv * s.head_dim;
    XcdAttnRequest rq;
    memset(&rq, 0, sizeof(rq));
    rq.shape = s;
    if (has_p) {
        FK_TRY(need_bytes(d, p_slot, xcd_sum_row_bytes(s.hidden)));
        rq.sums_in = arg_ptr<const long long>(d, p_slot);
    }
    FK_TRY(need_bytes(d, res_slot, (size_t)s.hidden * 2));
    FK_TRY(need_bytes(d, x_slot, (size_t)s.hidden * 2));
    FK_TRY(need_bytes(d, nw_slot, (size_t)s.hidden * 2));
    rq.residual = arg_ptr<const uint16_t>(d, res_slot);
    rq.x_out = arg_ptr<uint16_t>(d, x_slot);
    rq.norm_w = arg_ptr<const uint16_t>(d, nw_slot);
    rq.eps = (float)d.param("eps", 1e-6);
    fk_weight W[4];
    const uint32_t ns[3] = {n_q, n_kvd, n_kvd};
    for (int m = 0; m < 3; ++m)
        FK_TRY(bind_weight(d, s.bits, s.group, ns[m], s.hidden, w_slot + m, meta_slot + m, meta_slot + 3 + m, &W[m]));
    FK_TRY(bind_weight(d, s.bits, s.group, s.hidden, n_q, wo_slot, wo_meta, wo_meta + 1, &W[3]));
    rq.wq = &W[0];
    rq.wk = &W[1];
    rq.wv = &W[2];
    rq.wo = &W[3];
    if (norm) {
        FK_TRY(need_bytes(d, hn_slot, (size_t)s.head_dim * 2));
        FK_TRY(need_bytes(d, hn_slot + 1, (size_t)s.head_dim * 2));
        rq.q_norm = arg_ptr<const uint16_t>(d, hn_slot);
        rq.k_norm = arg_ptr<const uint16_t>(d, hn_slot + 1);
    }
    FK_TRY(need_bytes(d, q_slot, (size_t)n_q * 2));
    FK_TRY(need_bytes(d, q_slot + 1, (size_t)n_kvd * 2));
    FK_TRY(need_bytes(d, q_slot + 2, (size_t)n_kvd * 2));
    rq.q = arg_ptr<uint16_t>(d, q_slot);
    rq.k = arg_ptr<uint16_t>(d, q_slot + 1);
    rq.v = arg_ptr<uint16_t>(d, q_slot + 2);
    FK_TRY(need_bytes(d, ck_slot, (size_t)s.n_kv * s.capacity * s.head_dim * 2));
    FK_TRY(need_bytes(d, cv_slot, (size_t)s.n_kv * s.capacity * s.head_dim * 2));
    rq.cache_k = arg_ptr<uint16_t>(d, ck_slot);
    rq.cache_v = arg_ptr<uint16_t>(d, cv_slot);
    FK_TRY(need_bytes(d, len_slot, 4));
    rq.kv_len = arg_ptr<const uint32_t>(d, len_slot);
    FK_TRY(need_bytes(d, tab_slot, (size_t)s.head_dim * 4));
    rq.rope_tab = arg_ptr<const float>(d, tab_slot);
    rq.theta = (float)d.param("theta", 10000.0);
    FK_TRY(need_bytes(d, ap_slot, xcd_attn_partials_bytes(s)));
    rq.att_partials = arg_ptr<float>(d, ap_slot);
    FK_TRY(need_bytes(d, op_slot, xcd_sum_row_bytes(s.hidden)));
    rq.out_sums = arg_ptr<long long>(d, op_slot);
    FK_TRY(need_bytes(d, clr_slot, xcd_sum_row_bytes(s.hidden)));
    rq.clear = arg_ptr<long long>(d, clr_slot);
    FK_TRY(need_bytes(d, ws_slot, xcd_workspace_bytes()));
    rq.workspace = d.args[ws_slot].ptr;
    rq.spin_limit = d.u("spin_limit", 0);
    rq.mark_placement = d.u("mark_placement", 0) != 0;
    for (uint32_t j = 0; j < i; ++j) rw->reads.push_back(j);
    rw->writes = {(uint32_t)x_slot, (uint32_t)q_slot, (uint32_t)q_slot + 1, (uint32_t)q_slot + 2, (uint32_t)ck_slot,
                  (uint32_t)cv_slot, (uint32_t)ap_slot, (uint32_t)op_slot, (uint32_t)clr_slot, (uint32_t)ws_slot};
    rq.for_token = d.u("token", 0) != 0;
    return plan_xcd_attn(rq, l);
}

// [sums_in], residual, x_out, norm_w, W_gate, W_up, [s_g, s_u, b_g, b_u], W_down, [s_d, b_d], mid, out_sums, clear_sums,
// workspace
fk_status plan_xcd_mlp_d(const Dispatch& d, Launch* l, SlotRW* rw) {
    const XcdLayerShape s = xcd_shape(d);
    const bool has_p = d.u("has_sums", 1) != 0, q = s.bits != 16;
    size_t i = 0;
    const size_t p_slot = has_p ? i++ : 0, res_slot = i++, x_slot = i++, nw_slot = i++, w_slot = i;
    i += 2;
    const size_t meta_slot = i;
    if (q) i += 4;
    const size_t wd_slot = i++;
    const size_t wd_meta = i;
    if (q) i += 2;
    const size_t mid_slot = i++, op_slot = i++, clr_slot = i++, ws_slot = i++;
    FK_TRY(need_args(d, i));
    if (s.hidden == 0 || s.inter == 0) return set_error(FK_ERR_INVALID, d.kernel + ": layer shape parameters missing");
    XcdMlpRequest rq;
    memset(&rq, 0, sizeof(rq));
    rq.shape = s;
    if (has_p) {
        FK_TRY(need_bytes(d, p_slot, xcd_sum_row_bytes(s.hidden)));
        rq.sums_in = arg_ptr<const long long>(d, p_slot);
    }
    FK_TRY(need_bytes(d, res_slot, (size_t)s.hidden * 2));
    FK_TRY(need_bytes(d, x_slot, (size_t)s.hidden * 2));
    FK_TRY(need_bytes(d, nw_slot, (size_t)s.hidden * 2));
    rq.residual = arg_ptr<const uint16_t>(d, res_slot);
    rq.x_out = arg_ptr<uint16_t>(d, x_slot);
    rq.norm_w = arg_ptr<const uint16_t>(d, nw_slot);
    rq.eps = (float)d.param("eps", 1e-6);
    fk_weight W[3];
    for (int m = 0; m < 2; ++m)
        FK_TRY(bind_weight(d, s.bits, s.group, s.inter, s.hidden, w_slot + m, meta_slot + m, meta_slot + 2 + m, &W[m]));
    FK_TRY(bind_weight(d, s.bits, s.group, s.hidden, s.inter, wd_slot, wd_meta, wd_meta + 1, &W[2]));
    rq.wgate = &W[0];
    rq.wup = &W[1];
    rq.wdown = &W[2];
    rq.swiglu_variant = (int)d.param("variant", 0);
    FK_TRY(need_bytes(d, mid_slot, (size_t)s.inter * 2));
    rq.mid = arg_ptr<uint16_t>(d, mid_slot);
    FK_TRY(need_bytes(d, op_slot, xcd_sum_row_bytes(s.hidden)));
    rq.out_sums = arg_ptr<long long>(d, op_slot);
    FK_TRY(need_bytes(d, clr_slot, xcd_sum_row_bytes(s.hidden)));
    rq.clear = arg_ptr<long long>(d, clr_slot);
    FK_TRY(need_bytes(d, ws_slot, xcd_workspace_bytes()));
    rq.workspace = d.args[ws_slot].ptr;
    rq.spin_limit = d.u("spin_limit", 0);
    rq.mark_placement = d.u("mark_placement", 0) != 0;
    rq.for_token = d.u("token", 0) != 0;
    for (uint32_t j = 0; j < i; ++j) rw->reads.push_back(j);
    rw->writes = {(uint32_t)x_slot, (uint32_t)mid_slot, (uint32_t)op_slot, (uint32_t)clr_slot, (uint32_t)ws_slot};
    return plan_xcd_mlp(rq, l);
}

// The expert block of a mixture-of-experts layer as one XCD-resident launch (xcd_moe_kernel):
// [sums_in], residual, x_out, norm_w, W_router (bf16 [experts, hidden]), route_scale, then (w, scales, biases) of the
// expert gate, up, down stacks and of the shared gate, up, down matrices, logits_out [experts] bf16, idx_out [top_k]
// uint32, weight_out [top_k] bf16, scratch (fk_xcd_moe_scratch_bytes), shared_sums (the sum row of the shared expert's
// dot products, zero on entry), out_sums, clear_sums, workspace.
// Parameters: hidden, inter, shared_inter, experts, top_k, bits, group, eps, variant, has_sums, spin_limit,
// mark_placement.
fk_status plan_xcd_moe_d(const Dispatch& d, Launch* l, SlotRW* rw) {
    XcdMoeShape s;
    s.hidden = d.u("hidden");
    s.inter = d.u("inter");
    s.shared_inter = d.u("shared_inter");
    s.experts = d.u("experts");
    s.top_k = d.u("top_k");
    s.bits = d.u("bits", 4);
    s.group = d.u("group", 64);
    const bool has_p = d.u("has_sums", 1) != 0;
    size_t i = 0;
    const size_t p_slot = has_p ? i++ : 0, res_slot = i++, x_slot = i++, nw_slot = i++, rw_slot = i++, rs_slot = i++, w_slot = i;
    i += 18;
    const size_t lo_slot = i++, io_slot = i++, wo_slot = i++, sc_slot = i++, op2_slot = i++, op_slot = i++, clr_slot = i++, ws_slot = i++;
    FK_TRY(need_args(d, i));
    if (s.hidden == 0 || s.inter == 0 || s.shared_inter == 0 || s.experts == 0 || s.top_k == 0)
        return set_error(FK_ERR_INVALID, d.kernel + ": shape parameters missing");
    if (s.bits != 4) return set_error(FK_ERR_UNSUPPORTED, d.kernel + ": 4-bit weights only");
    XcdMoeRequest rq;
    memset(&rq, 0, sizeof(rq));
    rq.shape = s;
    if (has_p) {
        FK_TRY(need_bytes(d, p_slot, xcd_sum_row_bytes(s.hidden)));
        rq.sums_in = arg_ptr<const long long>(d, p_slot);
    }
    FK_TRY(need_bytes(d, res_slot, (size_t)s.hidden * 2));
    FK_TRY(need_bytes(d, x_slot, (size_t)s.hidden * 2));
    FK_TRY(need_bytes(d, nw_slot, (size_t)s.hidden * 2));
    FK_TRY(need_bytes(d, rw_slot, (size_t)s.experts * s.hidden * 2));
    FK_TRY(need_bytes(d, rs_slot, 2));
    rq.residual = arg_ptr<const uint16_t>(d, res_slot);
    rq.x_out = arg_ptr<uint16_t>(d, x_slot);
    rq.norm_w = arg_ptr<const uint16_t>(d, nw_slot);
    rq.eps = (float)d.param("eps", 1e-6);
    rq.router_w = arg_ptr<const uint16_t>(d, rw_slot);
    rq.route_scale = arg_ptr<const uint16_t>(d, rs_slot);
    fk_weight W[6];
    const uint32_t ns[6] = {s.experts * s.inter, s.experts * s.inter, s.experts * s.hidden, s.shared_inter, s.shared_inter, s.hidden};
    const uint32_t ks[6] = {s.hidden, s.hidden, s.inter, s.hidden, s.hidden, s.shared_inter};
    for (int m = 0; m < 6; ++m)
        FK_TRY(bind_weight(d, s.bits, s.group, ns[m], ks[m], w_slot + 3 * m, w_slot + 3 * m + 1, w_slot + 3 * m + 2, &W[m]));
    rq.gate = &W[0];
    rq.up = &W[1];
    rq.down = &W[2];
    rq.sgate = &W[3];
    rq.sup = &W[4];
    rq.sdown = &W[5];
    rq.swiglu_variant = (int)d.param("variant", 1);
    FK_TRY(need_bytes(d, lo_slot, (size_t)s.experts * 2));
    FK_TRY(need_bytes(d, io_slot, (size_t)s.top_k * 4));
    FK_TRY(need_bytes(d, wo_slot, (size_t)s.top_k * 2));
    rq.logits_out = arg_ptr<uint16_t>(d, lo_slot);
    rq.idx_out = arg_ptr<uint32_t>(d, io_slot);
    rq.weight_out = arg_ptr<uint16_t>(d, wo_slot);
    FK_TRY(need_bytes(d, sc_slot, xcd_moe_scratch_bytes(s)));
    rq.scratch = d.args[sc_slot].ptr;
    FK_TRY(need_bytes(d, op2_slot, xcd_sum_row_bytes(s.hidden)));
    rq.out_sums2 = arg_ptr<long long>(d, op2_slot);
    FK_TRY(need_bytes(d, op_slot, xcd_sum_row_bytes(s.hidden)));
    rq.out_sums = arg_ptr<long long>(d, op_slot);
    FK_TRY(need_bytes(d, clr_slot, xcd_sum_row_bytes(s.hidden)));
    rq.clear = arg_ptr<long long>(d, clr_slot);
    FK_TRY(need_bytes(d, ws_slot, xcd_workspace_bytes()));
    rq.workspace = d.args[ws_slot].ptr;
    rq.spin_limit = d.u("spin_limit", 0);
    rq.mark_placement = d.u("mark_placement", 0) != 0;
    for (uint32_t j = 0; j < i; ++j) rw->reads.push_back(j);
    rw->writes = {(uint32_t)x_slot, (uint32_t)lo_slot, (uint32_t)io_slot, (uint32_t)wo_slot, (uint32_t)sc_slot, (uint32_t)op2_slot,
                  (uint32_t)op_slot, (uint32_t)clr_slot, (uint32_t)ws_slot};
    return plan_xcd_moe(rq, l);
}

// The attention half of a layer with low-rank keys as one XCD-resident launch (xcd_mla_kernel):
// [sums_in, shared_sums_in], residual, x_out, norm_w, W_q, s_q, b_q, W_kv_a, s_a, b_a, latent_norm_w, W_kv_b, s_b, b_b,
// W_o, s_o, b_o (o_proj's scales and biases re-laid out per K-slice: fk_xcd_kslice_meta), q (twice n_heads * (nope + rope)
// elements: the raw rows, then the rows with q_pe rotated), kva (fk_xcd_mla_latent_bytes),
// kvb, cache_k, cache_v, kv_len, rope_tab, att_partials, [clear2_sums], out_sums, clear_sums, workspace.
// Parameters: hidden, n_heads, rank, rope_dim, nope_dim, v_dim, capacity, bits, group, eps, theta, traditional, scale,
// has_sums (0: the input is the residual row alone; 2: the two rows of an expert launch), has_clear2, spin_limit,
// mark_placement.
fk_status plan_xcd_mla_d(const Dispatch& d, Launch* l, SlotRW* rw) {
    XcdMlaShape s;
    s.hidden = d.u("hidden");
    s.n_heads = d.u("n_heads");
    s.rank = d.u("rank");
    s.rope_dim = d.u("rope_dim");
    s.nope_dim = d.u("nope_dim");
    s.v_dim = d.u("v_dim");
    s.capacity = d.u("capacity");
    s.bits = d.u("bits", 4);
    s.group = d.u("group", 64);
    const uint32_t has_p = d.u("has_sums", 0);
    const bool has_c2 = d.u("has_clear2", 0) != 0;
    if (has_p != 0 && has_p != 2) return set_error(FK_ERR_INVALID, d.kernel + ": has_sums must be 0 or 2");
    size_t i = has_p;
    const size_t res_slot = i++, x_slot = i++, nw_slot = i++, wq_slot = i, wa_slot = i + 3, an_slot = i + 6, wb_slot = i + 7, wo_slot = i + 10;
    i += 13;
    const size_t q_slot = i++, kva_slot = i++, kvb_slot = i++, ck_slot = i++, cv_slot = i++, len_slot = i++, tab_slot = i++, ap_slot = i++;
    const size_t c2_slot = has_c2 ? i++ : 0;
    const size_t op_slot = i++, clr_slot = i++, ws_slot = i++;
    FK_TRY(need_args(d, i));
    if (s.hidden == 0 || s.n_heads == 0 || s.rank == 0 || s.rope_dim == 0 || s.nope_dim == 0 || s.v_dim == 0 || s.capacity == 0)
        return set_error(FK_ERR_INVALID, d.kernel + ": shape parameters missing");
    if (s.bits != 4) return set_error(FK_ERR_UNSUPPORTED, d.kernel + ": 4-bit weights only");
    const uint32_t qk = s.nope_dim + s.rope_dim, n_a = s.rank + s.rope_dim, n_b = s.n_heads * (s.nope_dim + s.v_dim);
    XcdMlaRequest rq;
    memset(&rq, 0, sizeof(rq));
    rq.shape = s;
    if (has_p) {
        FK_TRY(need_bytes(d, 0, xcd_sum_row_bytes(s.hidden)));
        FK_TRY(need_bytes(d, 1, xcd_sum_row_bytes(s.hidden)));
        rq.sums_in = arg_ptr<const long long>(d, 0);
        rq.sums2_in = arg_ptr<const long long>(d, 1);
    }
    FK_TRY(need_bytes(d, res_slot, (size_t)s.hidden * 2));
    FK_TRY(need_bytes(d, x_slot, (size_t)s.hidden * 2));
    FK_TRY(need_bytes(d, nw_slot, (size_t)s.hidden * 2));
    rq.residual = arg_ptr<const uint16_t>(d, res_slot);
    rq.x_out = arg_ptr<uint16_t>(d, x_slot);
    rq.norm_w = arg_ptr<const uint16_t>(d, nw_slot);
    rq.eps = (float)d.param("eps", 1e-6);
    fk_weight W[4];
    FK_TRY(bind_weight(d, s.bits, s.group, s.n_heads * qk, s.hidden, wq_slot, wq_slot + 1, wq_slot + 2, &W[0]));
    FK_TRY(bind_weight(d, s.bits, s.group, n_a, s.hidden, wa_slot, wa_slot + 1, wa_slot + 2, &W[1]));
    FK_TRY(bind_weight(d, s.bits, s.group, n_b, s.rank, wb_slot, wb_slot + 1, wb_slot + 2, &W[2]));
    FK_TRY(bind_weight(d, s.bits, s.group, s.hidden, s.n_heads * s.v_dim, wo_slot, wo_slot + 1, wo_slot + 2, &W[3]));
    rq.wq = &W[0];
    rq.wa = &W[1];
    rq.wb = &W[2];
    rq.wo = &W[3];
    FK_TRY(need_bytes(d, an_slot, (size_t)s.rank * 2));
    rq.a_norm = arg_ptr<const uint16_t>(d, an_slot);
    FK_TRY(need_bytes(d, q_slot, (size_t)2 * s.n_heads * qk * 2));   // raw rows, then the rows with q_pe rotated
    FK_TRY(need_bytes(d, kva_slot, xcd_mla_latent_bytes(s)));
    FK_TRY(need_bytes(d, kvb_slot, (size_t)n_b * 2));
    rq.q = arg_ptr<uint16_t>(d, q_slot);
    rq.kva = arg_ptr<uint16_t>(d, kva_slot);
    rq.kvb = arg_ptr<uint16_t>(d, kvb_slot);
    FK_TRY(need_bytes(d, ck_slot, (size_t)s.n_heads * s.capacity * qk * 2));
    FK_TRY(need_bytes(d, cv_slot, (size_t)s.n_heads * s.capacity * s.v_dim * 2));
    rq.cache_k = arg_ptr<uint16_t>(d, ck_slot);
    rq.cache_v = arg_ptr<uint16_t>(d, cv_slot);
    FK_TRY(need_bytes(d, len_slot, 4));
    rq.kv_len = arg_ptr<const uint32_t>(d, len_slot);
    FK_TRY(need_bytes(d, tab_slot, (size_t)s.rope_dim * 4));
    rq.rope_tab = arg_ptr<const float>(d, tab_slot);
    rq.theta = (float)d.param("theta", 10000.0);
    rq.scale = (float)d.param("scale", 0.0);
    rq.traditional = d.u("traditional", 0) != 0;
    FK_TRY(need_bytes(d, ap_slot, xcd_mla_partials_bytes(s)));
    rq.att_partials = arg_ptr<float>(d, ap_slot);
    if (has_c2) {
        FK_TRY(need_bytes(d, c2_slot, xcd_sum_row_bytes(s.hidden)));
        rq.clear2 = arg_ptr<long long>(d, c2_slot);
    }
    FK_TRY(need_bytes(d, op_slot, xcd_sum_row_bytes(s.hidden)));
    rq.out_sums = arg_ptr<long long>(d, op_slot);
    FK_TRY(need_bytes(d, clr_slot, xcd_sum_row_bytes(s.hidden)));
    rq.clear = arg_ptr<long long>(d, clr_slot);
    FK_TRY(need_bytes(d, ws_slot, xcd_workspace_bytes()));
    rq.workspace = d.args[ws_slot].ptr;
    rq.spin_limit = d.u("spin_limit", 0);
    rq.mark_placement = d.u("mark_placement", 0) != 0;
    for (uint32_t j = 0; j < i; ++j) rw->reads.push_back(j);
    rw->writes = {(uint32_t)x_slot, (uint32_t)q_slot, (uint32_t)kva_slot, (uint32_t)kvb_slot, (uint32_t)ck_slot, (uint32_t)cv_slot,
                  (uint32_t)ap_slot, (uint32_t)op_slot, (uint32_t)clr_slot, (uint32_t)ws_slot};
    if (has_c2) rw->writes.push_back((uint32_t)c2_slot);
    return plan_xcd_mla(rq, l);
}

// src, out (8 bytes per workgroup): the plain read kernel (parameter blocks_per_cu)
fk_status plan_read_reduce_d(const Dispatch& d, Launch* l, SlotRW* rw) {
    FK_TRY(need_args(d, 2));
    rw->reads = {0};
    rw->writes = {1};
    return plan_read_reduce(d.args[0].ptr, d.args[0].nbytes, d.args[1].ptr, d.args[1].nbytes, d.u("blocks_per_cu", 0), l);
}

// sum row, residual [hidden] bf16, x [hidden] bf16, sum row to clear (may be the one read) [, second sum row, second row
// to clear [, a third row to clear]]: x = T(f32(row) + residual), with a second row x = T((f32(row) + T(f32(second row))) + residual)
// (parameter hidden)
fk_status plan_xcd_reduce_d(const Dispatch& d, Launch* l, SlotRW* rw) {
    const bool two = d.args.size() >= 6, three = d.args.size() >= 7;
    FK_TRY(need_args(d, three ? 7 : (two ? 6 : 4)));
    const uint32_t hidden = d.u("hidden");
    if (hidden == 0) return set_error(FK_ERR_INVALID, d.kernel + ": hidden parameter missing");
    FK_TRY(need_bytes(d, 0, xcd_sum_row_bytes(hidden)));
    FK_TRY(need_bytes(d, 1, (size_t)hidden * 2));
    FK_TRY(need_bytes(d, 2, (size_t)hidden * 2));
    FK_TRY(need_bytes(d, 3, xcd_sum_row_bytes(hidden)));
    rw->reads = {0, 1};
    rw->writes = {2, 3};
    if (two) {
        FK_TRY(need_bytes(d, 4, xcd_sum_row_bytes(hidden)));
        FK_TRY(need_bytes(d, 5, xcd_sum_row_bytes(hidden)));
        rw->reads.push_back(4);
        rw->writes.push_back(5);
    }
    if (three) {
        FK_TRY(need_bytes(d, 6, xcd_sum_row_bytes(hidden)));
        rw->writes.push_back(6);
    }
    return plan_xcd_reduce(arg_ptr<const long long>(d, 0), arg_ptr<const uint16_t>(d, 1), arg_ptr<uint16_t>(d, 2),
                           arg_ptr<long long>(d, 3), hidden, l, two ? arg_ptr<const long long>(d, 4) : nullptr,
                           two ? arg_ptr<long long>(d, 5) : nullptr, three ? arg_ptr<long long>(d, 6) : nullptr);
}

// Q, K0, K1, V, cache_k, cache_v, kv_len, out, partials, counters, [rope_tab]: split-key store + attention of a
// layer in one launch.  Parameters as the split form of kv_cache_store_decode (n_heads, q0_dim, q1_dim, n_kv,
// v_dim, k1_n_kv, k0_stride, v_stride, rope_dims, traditional, theta, capacity) plus max_len, scale, has_table.
fk_status plan_split_store_sdpa(const Dispatch& d, Launch* l, SlotRW* rw) {
    const bool table = d.u("has_table", 0) != 0;
    const size_t n = 10 + (table ? 1 : 0);
    FK_TRY(need_args(d, n));
    const uint32_t n_heads = d.u("n_heads"), n_kv = d.u("n_kv"), q0 = d.u("q0_dim"), q1 = d.u("q1_dim"), vd = d.u("v_dim");
    const uint32_t capacity = d.u("capacity"), max_len = d.u("max_len", capacity), qk = q0 + q1;
    if (n_heads == 0 || n_kv == 0 || q0 == 0 || q1 == 0 || vd == 0 || capacity == 0)
        return set_error(FK_ERR_INVALID, d.kernel + ": n_heads / n_kv / q0_dim / q1_dim / v_dim / capacity parameters missing");
    const float scale = d.has("scale") ? (float)d.param("scale", 0) : 1.0f / sqrtf((float)qk);
    SdpaFusion f;
    f.q0_dim = q0;
    f.k0_stride = d.u("k0_stride", q0);
    f.v_stride = d.u("v_stride", vd);
    f.k1_heads = d.u("k1_n_kv", n_kv);
    f.traditional = d.u("traditional", 0);
    f.rope_dims = d.u("rope_dims", 0);
    f.base_log2 = f.rope_dims ? base_log2_of(d) : 0.f;
    if (f.k0_stride < q0 || f.v_stride < vd || f.k1_heads == 0) return set_error(FK_ERR_INVALID, d.kernel + ": stride below the row width");
    FK_TRY(need_bytes(d, 0, (size_t)n_heads * qk * 2));
    FK_TRY(need_bytes(d, 1, ((size_t)(n_kv - 1) * f.k0_stride + q0) * 2));
    FK_TRY(need_bytes(d, 2, (size_t)f.k1_heads * q1 * 2));
    FK_TRY(need_bytes(d, 3, ((size_t)(n_kv - 1) * f.v_stride + vd) * 2));
    FK_TRY(need_bytes(d, 4, (size_t)n_kv * capacity * qk * 2));
    FK_TRY(need_bytes(d, 5, (size_t)n_kv * capacity * vd * 2));
    FK_TRY(need_bytes(d, 6, 4));
    FK_TRY(need_bytes(d, 7, (size_t)n_heads * vd * 2));
    size_t pb = 0, cb = 0;
    FK_TRY(sdpa_workspace_bytes(n_heads, n_kv, qk, vd, max_len, &pb, &cb));
    FK_TRY(need_bytes(d, 8, pb));
    FK_TRY(need_bytes(d, 9, cb));
    f.k_new = arg_ptr<const uint16_t>(d, 1);
    f.k1_new = arg_ptr<const uint16_t>(d, 2);
    f.v_new = arg_ptr<const uint16_t>(d, 3);
    if (table) {
        FK_TRY(need_bytes(d, 10, (size_t)f.rope_dims * 4));
        f.rope_tab = arg_ptr<const float>(d, 10);
    }
    for (uint32_t i = 0; i < n; ++i)
        if (i != 7) rw->reads.push_back(i);
    rw->writes = {4, 5, 7, 8, 9};
    return plan_sdpa_decode(arg_ptr<const uint16_t>(d, 0), arg_ptr<const uint16_t>(d, 4), arg_ptr<const uint16_t>(d, 5),
                            arg_ptr<uint16_t>(d, 7), arg_ptr<const uint32_t>(d, 6), 0, max_len, n_heads, n_kv, qk, vd, capacity,
                            scale, arg_ptr<float>(d, 8), arg_ptr<uint32_t>(d, 9), l, 1, nullptr, &f);
}

// K, V, [k_weight], keys_packed, keys_scales, keys_biases, values_packed, values_scales, values_biases, offset,
// write_offset (rope_kv_cache_store_decode_quant.rs:77-98; the capacity is a parameter here)
fk_status plan_rope_kv_quant(const Dispatch& d, Launch* l, SlotRW* rw, uint32_t bits) {
    const bool norm = d.u("has_norm", 0) != 0;
    const size_t n = norm ? 11 : 10, c0 = norm ? 3 : 2;
    FK_TRY(need_args(d, n));
    KvQuantStore a;
    memset(&a, 0, sizeof(a));
    a.n_kv = d.u("n_kv");
    a.dim = d.u("head_dim");
    a.rope_dims = d.u("rope_dims", a.dim);
    a.capacity = d.u("capacity");
    a.bits = bits;
    a.group = d.u("group", 64);
    a.rows = 1;
    if (a.capacity == 0 || a.n_kv == 0 || a.dim == 0 || a.group == 0 || a.dim % a.group)
        return set_error(FK_ERR_INVALID, d.kernel + ": n_kv / head_dim / capacity / group parameters missing or inconsistent");
    const size_t rows = (size_t)a.n_kv * a.capacity;
    FK_TRY(need_bytes(d, 0, (size_t)a.n_kv * a.dim * 2));
    FK_TRY(need_bytes(d, 1, (size_t)a.n_kv * a.dim * 2));
    for (size_t c = 0; c < 2; ++c) {
        FK_TRY(need_bytes(d, c0 + 3 * c, rows * a.dim * bits / 8));
        FK_TRY(need_bytes(d, c0 + 3 * c + 1, rows * (a.dim / a.group) * 2));
        FK_TRY(need_bytes(d, c0 + 3 * c + 2, rows * (a.dim / a.group) * 2));
    }
    FK_TRY(need_bytes(d, c0 + 6, 4));
    FK_TRY(need_bytes(d, c0 + 7, 4));
    a.k = arg_ptr<const uint16_t>(d, 0);
    a.v = arg_ptr<const uint16_t>(d, 1);
    if (norm) {
        FK_TRY(need_bytes(d, 2, (size_t)a.dim * 2));
        a.k_norm = arg_ptr<const uint16_t>(d, 2);
    }
    a.ck_packed = arg_ptr<uint32_t>(d, c0);
    a.ck_scales = arg_ptr<uint16_t>(d, c0 + 1);
    a.ck_biases = arg_ptr<uint16_t>(d, c0 + 2);
    a.cv_packed = arg_ptr<uint32_t>(d, c0 + 3);
    a.cv_scales = arg_ptr<uint16_t>(d, c0 + 4);
    a.cv_biases = arg_ptr<uint16_t>(d, c0 + 5);
    a.offset_ptr = arg_ptr<const uint32_t>(d, c0 + 6);
    a.write_offset_ptr = arg_ptr<const uint32_t>(d, c0 + 7);
    a.eps = (float)d.param("eps", 1e-6);
    a.base_log2 = base_log2_of(d);
    for (uint32_t i = 0; i < n; ++i) {
        if (i >= c0 && i < c0 + 6) rw->writes.push_back(i);
        else rw->reads.push_back(i);
    }
    return plan_kv_store_quant(a, l);
}

// Q, K_packed, K_scales, K_biases, V_packed, V_scales, V_biases, kv_len, out, partials, counters
// (sdpa_decode_quant.rs:184-196; the capacity is a parameter here)
fk_status plan_sdpa_quant_d(const Dispatch& d, Launch* l, SlotRW* rw, uint32_t bits) {
    FK_TRY(need_args(d, 11));
    const uint32_t n_heads = d.u("n_heads"), n_kv = d.u("n_kv"), qk = d.u("qk_dim", d.u("head_dim"));
    const uint32_t vd = d.u("v_dim", qk), capacity = d.u("capacity"), max_len = d.u("max_len", capacity);
    const uint32_t group = d.u("group", 64);
    if (n_heads == 0 || n_kv == 0 || qk == 0 || capacity == 0 || group == 0 || qk % group || vd % group)
        return set_error(FK_ERR_INVALID, d.kernel + ": n_heads / n_kv / head_dim / capacity / group parameters missing or inconsistent");
    const float scale = d.has("scale") ? (float)d.param("scale", 0) : 1.0f / sqrtf((float)qk);
    const size_t rows = (size_t)n_kv * capacity;
    FK_TRY(need_bytes(d, 0, (size_t)n_heads * qk * 2));
    FK_TRY(need_bytes(d, 1, rows * qk * bits / 8));
    FK_TRY(need_bytes(d, 2, rows * (qk / group) * 2));
    FK_TRY(need_bytes(d, 3, rows * (qk / group) * 2));
    FK_TRY(need_bytes(d, 4, rows * vd * bits / 8));
    FK_TRY(need_bytes(d, 5, rows * (vd / group) * 2));
    FK_TRY(need_bytes(d, 6, rows * (vd / group) * 2));
    FK_TRY(need_bytes(d, 7, 4));
    FK_TRY(need_bytes(d, 8, (size_t)n_heads * vd * 2));
    size_t pb = 0, cb = 0;
    FK_TRY(sdpa_workspace_bytes(n_heads, n_kv, qk, vd, max_len, &pb, &cb));
    FK_TRY(need_bytes(d, 9, pb));
    FK_TRY(need_bytes(d, 10, cb));
    rw->reads = {0, 1, 2, 3, 4, 5, 6, 7, 9, 10};
    rw->writes = {8, 9, 10};
    KvQuant qz;
    qz.k_scales = arg_ptr<const uint16_t>(d, 2);
    qz.k_biases = arg_ptr<const uint16_t>(d, 3);
    qz.v_scales = arg_ptr<const uint16_t>(d, 5);
    qz.v_biases = arg_ptr<const uint16_t>(d, 6);
    qz.bits = bits;
    qz.group = group;
    return plan_sdpa_decode(arg_ptr<const uint16_t>(d, 0), arg_ptr<const uint16_t>(d, 1), arg_ptr<const uint16_t>(d, 4),
                            arg_ptr<uint16_t>(d, 8), arg_ptr<const uint32_t>(d, 7), 0, max_len, n_heads, n_kv, qk, vd,
                            capacity, scale, arg_ptr<float>(d, 9), arg_ptr<uint32_t>(d, 10), l, 1, &qz);
}

// x, gate_w, gate_s, gate_b, up_w, up_s, up_b, row_idx, expert_idx, [route_weight], out0
// (routed_qmv_swiglu.rs:99-112).  Parameters: k, o, experts, routes, x_rows, pre_scale.
// route_in_kernel = 1: x, gate w / s / b, up w / s / b, logits, route_scale, idx_out, weight_out, out0,
// [shared gate w / s / b, shared up w / s / b, shared_out]; parameters k, o, experts, routes (= top_k), pre_scale,
// has_shared, shared_o.
fk_status plan_routed_swiglu_routing(const Dispatch& d, Launch* l, SlotRW* rw) {
    const uint32_t bits = d.u("bits", 4), group = d.u("group", 64), K = d.u("k"), O = d.u("o");
    const uint32_t experts = d.u("experts"), routes = d.u("routes");
    const bool has_shared = d.u("has_shared", 0) != 0;
    const size_t n_slots = 12;
    FK_TRY(need_args(d, n_slots + (has_shared ? 7 : 0)));
    if (bits != 4 && bits != 8) return set_error(FK_ERR_UNSUPPORTED, d.kernel + ": bits must be 4 or 8");
    if (experts == 0 || routes == 0 || K == 0 || O == 0)
        return set_error(FK_ERR_INVALID, d.kernel + ": k / o / experts / routes parameters missing");
    fk_weight Wg, Wu, Sg, Su;
    FK_TRY(bind_weight(d, bits, group, O * experts, K, 1, 2, 3, &Wg));
    FK_TRY(bind_weight(d, bits, group, O * experts, K, 4, 5, 6, &Wu));
    Wg.n = Wu.n = O;
    FK_TRY(need_bytes(d, 0, (size_t)K * 2));
    FK_TRY(need_bytes(d, 7, (size_t)experts * 2));
    FK_TRY(need_bytes(d, 8, 2));
    FK_TRY(need_bytes(d, 9, (size_t)routes * 4));
    FK_TRY(need_bytes(d, 10, (size_t)routes * 2));
    FK_TRY(need_bytes(d, 11, (size_t)routes * O * 2));
    for (uint32_t i = 0; i < 9; ++i) rw->reads.push_back(i);
    rw->writes = {9, 10, 11};
    uint16_t* shared_out = nullptr;
    if (has_shared) {
        const uint32_t so = d.u("shared_o");
        if (so == 0) return set_error(FK_ERR_INVALID, d.kernel + ": shared_o parameter missing");
        FK_TRY(bind_weight(d, bits, group, so, K, n_slots, n_slots + 1, n_slots + 2, &Sg));
        FK_TRY(bind_weight(d, bits, group, so, K, n_slots + 3, n_slots + 4, n_slots + 5, &Su));
        FK_TRY(need_bytes(d, n_slots + 6, (size_t)so * 2));
        shared_out = arg_ptr<uint16_t>(d, n_slots + 6);
        for (uint32_t i = 0; i < 6; ++i) rw->reads.push_back((uint32_t)n_slots + i);
        rw->writes.push_back((uint32_t)n_slots + 6);
    }
    RouteInKernel rk;
    rk.logits = arg_ptr<const uint16_t>(d, 7);
    rk.scale = arg_ptr<const uint16_t>(d, 8);
    rk.idx_out = arg_ptr<uint32_t>(d, 9);
    rk.weight_out = arg_ptr<uint16_t>(d, 10);
    rk.apply_weight = d.u("pre_scale", 0) != 0;
    return plan_routed_gemv(arg_ptr<const uint16_t>(d, 0), 1, &Wg, &Wu, experts, nullptr, nullptr, nullptr, routes,
                            arg_ptr<uint16_t>(d, 11), l, has_shared ? &Sg : nullptr, has_shared ? &Su : nullptr, shared_out, &rk);
}

fk_status plan_routed_swiglu(const Dispatch& d, Launch* l, SlotRW* rw) {
    if (d.u("route_in_kernel", 0)) return plan_routed_swiglu_routing(d, l, rw);
    const uint32_t bits = d.u("bits", 4), group = d.u("group", 64), K = d.u("k"), O = d.u("o");
    const uint32_t experts = d.u("experts"), routes = d.u("routes"), x_rows = d.u("x_rows", 1);
    const bool pre_scale = d.u("pre_scale", 0) != 0, has_shared = d.u("has_shared", 0) != 0;
    const size_t n_slots = pre_scale ? 11 : 10;
    // with has_shared = 1: + shared gate w / s / b, shared up w / s / b, shared_out (parameter shared_o rows);
    // with has_order = 1 (several tokens, no shared pair): + order (uint32 [routes], from fusekit_route_order);
    // with expert_order = 1 instead (no slot, up to 64 routes): the launch finds the same order itself
    const bool has_order = d.u("has_order", 0) != 0, expert_order = d.u("expert_order", 0) != 0;
    if (has_order && expert_order) return set_error(FK_ERR_INVALID, d.kernel + ": has_order and expert_order exclude each other");
    FK_TRY(need_args(d, n_slots + (has_shared ? 7 : 0) + (has_order ? 1 : 0)));
    if (bits != 4 && bits != 8) return set_error(FK_ERR_UNSUPPORTED, d.kernel + ": bits must be 4 or 8");
    if (experts == 0 || routes == 0 || K == 0 || O == 0)
        return set_error(FK_ERR_INVALID, d.kernel + ": k / o / experts / routes parameters missing");
    fk_weight Wg, Wu;
    FK_TRY(bind_weight(d, bits, group, O * experts, K, 1, 2, 3, &Wg));
    FK_TRY(bind_weight(d, bits, group, O * experts, K, 4, 5, 6, &Wu));
    Wg.n = Wu.n = O;
    FK_TRY(need_bytes(d, 0, (size_t)x_rows * K * 2));
    FK_TRY(need_bytes(d, 7, (size_t)routes * 4));
    FK_TRY(need_bytes(d, 8, (size_t)routes * 4));
    if (pre_scale) FK_TRY(need_bytes(d, 9, (size_t)routes * 2));
    FK_TRY(need_bytes(d, n_slots - 1, (size_t)routes * O * 2));
    all_but_last(n_slots, 1, rw);
    fk_weight Sg, Su;
    uint16_t* shared_out = nullptr;
    if (has_shared) {
        const uint32_t so = d.u("shared_o");
        if (so == 0) return set_error(FK_ERR_INVALID, d.kernel + ": shared_o parameter missing");
        FK_TRY(bind_weight(d, bits, group, so, K, n_slots, n_slots + 1, n_slots + 2, &Sg));
        FK_TRY(bind_weight(d, bits, group, so, K, n_slots + 3, n_slots + 4, n_slots + 5, &Su));
        FK_TRY(need_bytes(d, n_slots + 6, (size_t)so * 2));
        shared_out = arg_ptr<uint16_t>(d, n_slots + 6);
        for (uint32_t i = 0; i < 6; ++i) rw->reads.push_back((uint32_t)n_slots + i);
        rw->writes.push_back((uint32_t)n_slots + 6);
    }
    const uint32_t* order = expert_order ? kOrderInKernel : nullptr;
    if (has_order) {
        const size_t os = n_slots + (has_shared ? 7 : 0);
        FK_TRY(need_bytes(d, os, (size_t)routes * 4));
        order = arg_ptr<const uint32_t>(d, os);
        rw->reads.push_back((uint32_t)os);
    }
    return plan_routed_gemv(arg_ptr<const uint16_t>(d, 0), x_rows, &Wg, &Wu, experts, arg_ptr<const uint32_t>(d, 7),
                            arg_ptr<const uint32_t>(d, 8), pre_scale ? arg_ptr<const uint16_t>(d, 9) : nullptr, routes,
                            arg_ptr<uint16_t>(d, n_slots - 1), l, has_shared ? &Sg : nullptr, has_shared ? &Su : nullptr,
                            shared_out, nullptr, order);
}

// x, wq, scales, biases, row_idx, expert_idx, [route_weight], [shared_x, shared_w, shared_s, shared_b],
// [residual_extra], out0, workspace   (routed_qmv_reduce.rs:110-145; the workspace slot is this
// library's: per-route results before the ordered sum).  Parameters: k, o, experts, tokens, top_k,
// x_rows, input_preweighted, has_shared, shared_k, has_extra.
fk_status plan_routed_reduce(const Dispatch& d, Launch* l, SlotRW* rw) {
    const uint32_t bits = d.u("bits", 4), group = d.u("group", 64), K = d.u("k"), O = d.u("o");
    const uint32_t experts = d.u("experts"), tokens = d.u("tokens", 1), top_k = d.u("top_k");
    const bool preweighted = d.u("input_preweighted", 0) != 0, has_shared = d.u("has_shared", 0) != 0;
    const bool has_extra = d.u("has_extra", 0) != 0;
    const uint32_t shared_k = d.u("shared_k", K), routes = tokens * top_k, x_rows = d.u("x_rows", routes);
    size_t s = 6;
    const size_t rw_slot = preweighted ? 0 : s++;
    const size_t shared_slot = s;
    if (has_shared) s += 4;
    const size_t extra_slot = has_extra ? s++ : 0;
    const size_t out_slot = s++, ws_slot = s++;
    const bool has_order = d.u("has_order", 0) != 0;   // + order (uint32 [routes], from fusekit_route_order) as the last slot
    const bool expert_order = d.u("expert_order", 0) != 0;   // no slot, up to 64 routes: the launch finds that order itself
    if (has_order && expert_order) return set_error(FK_ERR_INVALID, d.kernel + ": has_order and expert_order exclude each other");
    const size_t order_slot = has_order ? s++ : 0;
    FK_TRY(need_args(d, s));
    if (bits != 4 && bits != 8) return set_error(FK_ERR_UNSUPPORTED, d.kernel + ": bits must be 4 or 8");
    if (experts == 0 || routes == 0 || K == 0 || O == 0)
        return set_error(FK_ERR_INVALID, d.kernel + ": k / o / experts / top_k parameters missing");
    fk_weight Wd, Ws;
    FK_TRY(bind_weight(d, bits, group, O * experts, K, 1, 2, 3, &Wd));
    Wd.n = O;
    FK_TRY(need_bytes(d, 0, (size_t)x_rows * K * 2));
    FK_TRY(need_bytes(d, 4, (size_t)routes * 4));
    FK_TRY(need_bytes(d, 5, (size_t)routes * 4));
    if (!preweighted) FK_TRY(need_bytes(d, rw_slot, (size_t)routes * 2));
    if (has_shared) {
        FK_TRY(bind_weight(d, bits, group, O, shared_k, shared_slot + 1, shared_slot + 2, shared_slot + 3, &Ws));
        FK_TRY(need_bytes(d, shared_slot, (size_t)shared_k * 2));
    }
    if (has_extra) FK_TRY(need_bytes(d, extra_slot, (size_t)tokens * O * 2));
    FK_TRY(need_bytes(d, out_slot, (size_t)tokens * O * 2));
    FK_TRY(need_bytes(d, ws_slot, routed_reduce_workspace_bytes(tokens, top_k, O, has_shared ? shared_k : 0, group)));
    for (uint32_t i = 0; i < out_slot; ++i) rw->reads.push_back(i);
    rw->reads.push_back((uint32_t)ws_slot);
    rw->writes = {(uint32_t)out_slot, (uint32_t)ws_slot};
    const uint32_t* order = expert_order ? kOrderInKernel : nullptr;
    if (has_order) {
        FK_TRY(need_bytes(d, order_slot, (size_t)routes * 4));
        order = arg_ptr<const uint32_t>(d, order_slot);
        rw->reads.push_back((uint32_t)order_slot);
    }

    return plan_routed_reduce_chain(arg_ptr<const uint16_t>(d, 0), x_rows, &Wd, experts, arg_ptr<const uint32_t>(d, 4),
                                    arg_ptr<const uint32_t>(d, 5), preweighted ? nullptr : arg_ptr<const uint16_t>(d, rw_slot),
                                    has_shared ? arg_ptr<const uint16_t>(d, shared_slot) : nullptr, has_shared ? &Ws : nullptr,
                                    has_extra ? arg_ptr<const uint16_t>(d, extra_slot) : nullptr, tokens, top_k,
                                    arg_ptr<uint16_t>(d, out_slot), arg_ptr<uint16_t>(d, ws_slot), l, order);
}

// expert_idx (uint32 [routes]), order (uint32 [routes], written): the routes sorted by expert, stable (parameters
// routes, experts).  No counterpart among the reference's kernels: its routed kernels serve routes as listed.
fk_status plan_route_order_d(const Dispatch& d, Launch* l, SlotRW* rw) {
    FK_TRY(need_args(d, 2));
    const uint32_t routes = d.u("routes"), experts = d.u("experts");
    if (routes == 0 || experts == 0) return set_error(FK_ERR_INVALID, d.kernel + ": routes / experts parameters missing");
    FK_TRY(need_bytes(d, 0, (size_t)routes * 4));
    FK_TRY(need_bytes(d, 1, (size_t)routes * 4));
    rw->reads = {0};
    rw->writes = {1};
    return plan_route_order(arg_ptr<const uint32_t>(d, 0), routes, experts, arg_ptr<uint32_t>(d, 1), l);
}

// x, W, scales, biases, [bias], [residual], y, workspace.  Parameters: m (= K), n, rows, has_bias, has_residual.
fk_status plan_qgemm_d(const Dispatch& d, Launch* l, SlotRW* rw) {
    const uint32_t bits = d.u("bits", 4), group = d.u("group", 64), K = d.u("m"), N = d.u("n"), rows = d.u("rows");
    const bool has_bias = d.u("has_bias", 0) != 0, has_res = d.u("has_residual", 0) != 0;
    size_t s = 4;
    const size_t bias_slot = has_bias ? s++ : 0, res_slot = has_res ? s++ : 0;
    const size_t out_slot = s++, ws_slot = s++;
    FK_TRY(need_args(d, s));
    if (bits != 4 && bits != 8) return set_error(FK_ERR_UNSUPPORTED, d.kernel + ": bits must be 4 or 8");
    if (rows == 0) return set_error(FK_ERR_INVALID, d.kernel + ": rows parameter missing");
    fk_weight W;
    FK_TRY(bind_weight(d, bits, group, N, K, 1, 2, 3, &W));
    FK_TRY(need_bytes(d, 0, (size_t)rows * K * 2));
    if (has_bias) FK_TRY(need_bytes(d, bias_slot, (size_t)N * 2));
    if (has_res) FK_TRY(need_bytes(d, res_slot, (size_t)rows * N * 2));
    FK_TRY(need_bytes(d, out_slot, (size_t)rows * N * 2));
    size_t ws = 0;
    FK_TRY(qgemm_workspace_bytes(rows, N, K, group, &ws));
    FK_TRY(need_bytes(d, ws_slot, ws));
    for (uint32_t i = 0; i < out_slot; ++i) rw->reads.push_back(i);
    rw->reads.push_back((uint32_t)ws_slot);
    rw->writes = {(uint32_t)out_slot, (uint32_t)ws_slot};
    Launch reduce;
    FK_TRY(plan_qgemm(&W, arg_ptr<const uint16_t>(d, 0), rows, has_bias ? arg_ptr<const uint16_t>(d, bias_slot) : nullptr,
                      has_res ? arg_ptr<const uint16_t>(d, res_slot) : nullptr, arg_ptr<uint16_t>(d, out_slot),
                      d.args[ws_slot].ptr, l, &reduce));
    if (reduce.func) l->then.push_back(reduce);
    return FK_OK;
}

// The q / k / v projections of several token rows (fk_qgemm_fanout): x, W_q, W_k, W_v, s_q, s_k, s_v, b_q, b_k, b_v,
// [bias_q, bias_k, bias_v], q, k, v, workspace (fk_qgemm_workspace_bytes(rows, n_q + 2 n_kv, hidden, group)).
// Parameters: hidden (= K), n_q, n_kv, rows, bits, group, has_bias.  One launch of the fused kernel's tile form (plus the
// fan-out's second kernel when k is split); FK_ERR_UNSUPPORTED where that form does not apply (fewer than 65 rows, an n
// that is no multiple of 4): the caller dispatches fusekit_qgemm per matrix then.
fk_status plan_qgemm_fanout_d(const Dispatch& d, Launch* l, SlotRW* rw) {
    const uint32_t bits = d.u("bits", 4), group = d.u("group", 64), K = d.u("hidden"), rows = d.u("rows");
    const uint32_t ns[3] = {d.u("n_q"), d.u("n_kv"), d.u("n_kv")};
    const bool has_bias = d.u("has_bias", 0) != 0;
    size_t s = 10;
    const size_t bias_slot = s;
    if (has_bias) s += 3;
    const size_t out_slot = s;
    s += 3;
    const size_t ws_slot = s++;
    FK_TRY(need_args(d, s));
    if (bits != 4 && bits != 8) return set_error(FK_ERR_UNSUPPORTED, d.kernel + ": bits must be 4 or 8");
    if (rows == 0 || K == 0 || ns[0] == 0 || ns[1] == 0) return set_error(FK_ERR_INVALID, d.kernel + ": hidden / n_q / n_kv / rows parameters missing");
    fk_weight W[3];
    const fk_weight* Wp[3];
    const uint16_t* bias[3] = {nullptr, nullptr, nullptr};
    uint16_t* y[3];
    FK_TRY(need_bytes(d, 0, (size_t)rows * K * 2));
    for (int m = 0; m < 3; ++m) {
        FK_TRY(bind_weight(d, bits, group, ns[m], K, 1 + m, 4 + m, 7 + m, &W[m]));
        Wp[m] = &W[m];
        if (has_bias) {
            FK_TRY(need_bytes(d, bias_slot + m, (size_t)ns[m] * 2));
            bias[m] = arg_ptr<const uint16_t>(d, bias_slot + m);
        }
        FK_TRY(need_bytes(d, out_slot + m, (size_t)rows * ns[m] * 2));
        y[m] = arg_ptr<uint16_t>(d, out_slot + m);
    }
    size_t ws = 0;
    FK_TRY(qgemm_workspace_bytes(rows, ns[0] + 2 * ns[1], K, group, &ws));
    FK_TRY(need_bytes(d, ws_slot, ws));
    for (uint32_t i = 0; i < out_slot; ++i) rw->reads.push_back(i);
    rw->reads.push_back((uint32_t)ws_slot);
    rw->writes = {(uint32_t)out_slot, (uint32_t)out_slot + 1, (uint32_t)out_slot + 2, (uint32_t)ws_slot};
    Launch reduce;
    bool fused = false;
    FK_TRY(plan_qgemm_fanout(Wp, 3, arg_ptr<const uint16_t>(d, 0), rows, has_bias ? bias : nullptr, y, d.args[ws_slot].ptr, l, &reduce,
                             &fused));
    if (fused) {
        if (reduce.func) l->then.push_back(reduce);
        return FK_OK;
    }
    return set_error(FK_ERR_UNSUPPORTED, d.kernel + ": the fan-out needs the fused kernel's tile form (65 rows or more, every n a "
                                         "multiple of 4); dispatch fusekit_qgemm per matrix instead");
}

// x, W_gate, W_up, s_g, s_u, b_g, b_u, out, workspace.  Parameters: hidden, inter, rows, variant.
fk_status plan_qgemm_swiglu_d(const Dispatch& d, Launch* l, SlotRW* rw) {
    const uint32_t bits = d.u("bits", 4), group = d.u("group", 64), hidden = d.u("hidden"), inter = d.u("inter");
    const uint32_t rows = d.u("rows");
    FK_TRY(need_args(d, 9));
    if (bits != 4 && bits != 8) return set_error(FK_ERR_UNSUPPORTED, d.kernel + ": bits must be 4 or 8");
    if (rows == 0) return set_error(FK_ERR_INVALID, d.kernel + ": rows parameter missing");
    fk_weight Wg, Wu;
    FK_TRY(bind_weight(d, bits, group, inter, hidden, 1, 3, 5, &Wg));
    FK_TRY(bind_weight(d, bits, group, inter, hidden, 2, 4, 6, &Wu));
    FK_TRY(need_bytes(d, 0, (size_t)rows * hidden * 2));
    FK_TRY(need_bytes(d, 7, (size_t)rows * inter * 2));
    size_t ws = 0;
    FK_TRY(qgemm_workspace_bytes(rows, inter, hidden, group, &ws));
    FK_TRY(need_bytes(d, 8, 2 * ws));
    rw->reads = {0, 1, 2, 3, 4, 5, 6, 8};
    rw->writes = {7, 8};
    Launch up, reduce;
    FK_TRY(plan_qgemm_swiglu(&Wg, &Wu, arg_ptr<const uint16_t>(d, 0), rows, (int)d.param("variant", 2),
                             arg_ptr<uint16_t>(d, 7), d.args[8].ptr, l, &up, &reduce));
    if (up.func) l->then.push_back(up);
    if (reduce.func) l->then.push_back(reduce);
    return FK_OK;
}

// logits, next_tok, workspace, [history, hist_counter]
fk_status plan_argmax_d(const Dispatch& d, Launch* l, SlotRW* rw) {
    const bool hist = d.args.size() == 5;
    FK_TRY(need_args(d, hist ? 5 : 3));
    const uint32_t vocab = d.u("vocab");
    FK_TRY(need_bytes(d, 0, (size_t)vocab * 2));
    FK_TRY(need_bytes(d, 1, 4));
    FK_TRY(need_bytes(d, 2, kArgmaxWorkspaceBytes));
    uint32_t cap = 0;
    if (hist) {
        cap = (uint32_t)(d.args[3].nbytes / 4);
        FK_TRY(need_bytes(d, 4, 4));
        rw->reads = {0, 2, 4};
        rw->writes = {1, 2, 3, 4};
    } else {
        rw->reads = {0, 2};
        rw->writes = {1, 2};
    }
    return plan_argmax(arg_ptr<const uint16_t>(d, 0), vocab, arg_ptr<uint32_t>(d, 1),
                       hist ? arg_ptr<uint32_t>(d, 3) : nullptr, hist ? arg_ptr<uint32_t>(d, 4) : nullptr, cap,
                       d.args[2].ptr, l);
}

struct Family {
    const char* prefix;
    fk_status (*plan)(const Dispatch&, Launch*, SlotRW*);
};

// Longest prefix first where one family name begins another.
const Family kFamilies[] = {
    {"fusekit_step_init", plan_step},
    {"fusekit_embed_lookup_decode", plan_embed_d},
    {"fusekit_rmsnorm_qkv", plan_qkv},
    {"fusekit_qmv_fanout", plan_qkv},
    {"fusekit_rmsnorm_gateup_swiglu", plan_gateup},
    {"fusekit_qmv_swiglu", plan_gateup},
    {"fusekit_linear_residual", plan_linres},
    {"fusekit_final_rmsnorm_lm_head_argmax",
     [](const Dispatch& d, Launch* l, SlotRW* rw) { return plan_lm_head(d, l, rw, true); }},
    {"fusekit_final_rmsnorm_lm_head",
     [](const Dispatch& d, Launch* l, SlotRW* rw) { return plan_lm_head(d, l, rw, false); }},
    {"fusekit_qgemv", plan_qgemv_d},
    {"fusekit_qgemm", plan_qgemm_d},
    {"fusekit_qgemm_swiglu", plan_qgemm_swiglu_d},
    {"fusekit_qgemm_fanout", plan_qgemm_fanout_d},
    {"fusekit_routed_qmv_swiglu", plan_routed_swiglu},
    {"fusekit_routed_qmv_reduce", plan_routed_reduce},
    {"fusekit_rmsnorm_rope_q_decode",
     [](const Dispatch& d, Launch* l, SlotRW* rw) { return plan_rope_q(d, l, rw, true); }},
    {"fusekit_rmsnorm_rope_kv_cache_store_decode",
     [](const Dispatch& d, Launch* l, SlotRW* rw) { return plan_rope_kv(d, l, rw, true, true); }},
    {"fusekit_rope_q_decode", [](const Dispatch& d, Launch* l, SlotRW* rw) { return plan_rope_q(d, l, rw, false); }},
    {"fusekit_rope_kv_cache_store_decode",
     [](const Dispatch& d, Launch* l, SlotRW* rw) { return plan_rope_kv(d, l, rw, false, true); }},
    {"fusekit_kv_cache_store_decode",
     [](const Dispatch& d, Launch* l, SlotRW* rw) {
         return d.u("split_k", 0) ? plan_kv_store_split(d, l, rw) : plan_rope_kv(d, l, rw, false, false);
     }},
    {"fusekit_softmax_topk_route", plan_softmax_topk_route_d},
    {"fusekit_moe_router", plan_moe_router_d},
    {"fusekit_qkv_rope_store_decode", plan_qkv_rope_store},
    {"fusekit_sdpa_decode", plan_sdpa_d},
    {"fusekit_sdpa_prefill", plan_sdpa_prefill_d},
    {"fusekit_rmsnorm_rows", plan_rmsnorm_rows_d},
    {"fusekit_rope_store_sdpa_decode", plan_rope_store_sdpa},
    {"fusekit_split_store_sdpa_decode", plan_split_store_sdpa},
    {"fusekit_rope_kv_cache_store_decode_q4",
     [](const Dispatch& d, Launch* l, SlotRW* rw) { return plan_rope_kv_quant(d, l, rw, 4); }},
    {"fusekit_rope_kv_cache_store_decode_q8",
     [](const Dispatch& d, Launch* l, SlotRW* rw) { return plan_rope_kv_quant(d, l, rw, 8); }},
    {"fusekit_sdpa_decode_q4", [](const Dispatch& d, Launch* l, SlotRW* rw) { return plan_sdpa_quant_d(d, l, rw, 4); }},
    {"fusekit_sdpa_decode_q8", [](const Dispatch& d, Launch* l, SlotRW* rw) { return plan_sdpa_quant_d(d, l, rw, 8); }},
    {"fusekit_argmax_logits_decode", plan_argmax_d},
    {"fusekit_xcd_attn_block", plan_xcd_attn_d},
    {"fusekit_xcd_mlp_block", plan_xcd_mlp_d},
    {"fusekit_xcd_reduce", plan_xcd_reduce_d},
    {"fusekit_xcd_moe_block", plan_xcd_moe_d},
    {"fusekit_xcd_mla_block", plan_xcd_mla_d},
    {"fusekit_read_reduce", plan_read_reduce_d},
    {"fusekit_route_order", plan_route_order_d},
};

const Family* find_family(const std::string& kernel) {
    const Family* best = nullptr;
    size_t best_len = 0;
    for (const Family& f : kFamilies) {
        const size_t n = strlen(f.prefix);
        if (kernel.compare(0, n, f.prefix) == 0 && (kernel.size() == n || kernel[n] == '_') && n > best_len) {
            best = &f;
            best_len = n;
        }
    }
    return best;
}

fk_status plan_dispatch(const Dispatch& d, Launch* l, SlotRW* rw) {
    const Family* f = find_family(d.kernel);
    if (!f) return set_error(FK_ERR_INVALID, "kernel '" + d.kernel + "' is not in this library");  // lib.rs:412-415
    rw->reads.clear();
    rw->writes.clear();
    l->then.clear();
    return f->plan(d, l, rw);
}

fk_status copy_dispatch(const fk_dispatch& in, Dispatch* out) {
    if (!in.kernel) return set_error(FK_ERR_INVALID, "dispatch without a kernel name");
    if ((in.n_args && !in.args) || (in.n_params && !in.params)) return set_error(FK_ERR_INVALID, "null args / params");
    out->kernel = in.kernel;
    out->args.assign(in.args, in.args + in.n_args);
    out->params.clear();
    for (uint32_t i = 0; i < in.n_params; ++i) {
        if (!in.params[i].key) return set_error(FK_ERR_INVALID, "parameter without a key");
        out->params.emplace_back(in.params[i].key, in.params[i].value);
    }
    return FK_OK;
}

bool overlap(const fk_arg& a, const fk_arg& b) {
    const char* a0 = (const char*)a.ptr;
    const char* b0 = (const char*)b.ptr;
    return a0 < b0 + b.nbytes && b0 < a0 + a.nbytes;
}

struct Node {
    Dispatch d;
    Launch launch;
    SlotRW rw;
    hipGraphNode_t node = nullptr;
    std::vector<hipGraphNode_t> tail;  // nodes of launch.then, chained behind `node`
    std::vector<uint32_t> deps;
    hipGraphNode_t last() const { return tail.empty() ? node : tail.back(); }
};

struct Graph {
    std::vector<Node> nodes;
    hipGraph_t graph = nullptr;
    hipGraphExec_t exec = nullptr;
    std::vector<uint8_t> barriers;  // as given to fk_build_graph (empty: none forced)
    std::vector<void*> xcd_controls;  // control blocks of XCD-resident launches in this graph (abort words)
    std::vector<std::pair<void*, size_t>> xcd_sum_rows;  // the sum rows those launches read, add into and clear
    // Runs of alternating xcd_attn / xcd_mlp dispatches (parameter token_launch = 1) executed as ONE launch each:
    // the nodes keep their own launches (eager execution, profiling), the executable graph holds one kernel node
    // per run, whose per-layer argument blocks sit in device tables.
    struct FusedRun {
        size_t first = 0, count = 0;
        Launch launch;
        void* d_attn = nullptr;
        void* d_mlp = nullptr;
        hipGraphNode_t node = nullptr;
    };
    std::vector<FusedRun> fused;
    std::vector<int> fused_of;  // per node: index into `fused`, or -1
    // persistent whole-token mode: one kernel node; device-side tables it reads
    bool persistent = false;
    Launch token_launch;
    void* d_tables = nullptr;
    uint32_t* d_abort = nullptr;
    unsigned long long* d_trace = nullptr;
    uint32_t trace_len = 0;
    Graph() = default;
    Graph(const Graph&) = delete;
    Graph& operator=(const Graph&) = delete;
    // a graph that fails half-way through its construction is dropped by its builder: release what it holds
    ~Graph() {
        if (exec) (void)hipGraphExecDestroy(exec);
        if (graph) (void)hipGraphDestroy(graph);
        if (d_tables) (void)hipFree(d_tables);
        for (FusedRun& r : fused) {
            if (r.d_attn) (void)hipFree(r.d_attn);
            if (r.d_mlp) (void)hipFree(r.d_mlp);
        }
    }
};

struct DispatcherState {
    std::mutex mu;
    hipStream_t stream = nullptr;
    hipEvent_t ev0 = nullptr, ev1 = nullptr;
    std::vector<std::unique_ptr<Graph>> graphs;
    std::vector<std::string> kernel_names;
    std::vector<const char*> kernel_name_ptrs;
    std::string task_graph_path;
    bool pending = false;
    Graph* pending_graph = nullptr;  // the graph of the launch in flight (graphs live as long as their dispatcher)
};

std::mutex g_mu;
std::vector<std::unique_ptr<DispatcherState>> g_dispatchers;  // append-only, like lib.rs:112

fk_status get_dispatcher(fk_handle h, DispatcherState** out) {
    std::lock_guard<std::mutex> lk(g_mu);
    if (h == 0 || h > g_dispatchers.size()) return set_error(FK_ERR_INVALID, "invalid dispatcher handle");  // lib.rs:198
    *out = g_dispatchers[h - 1].get();
    return FK_OK;
}

fk_status get_graph(DispatcherState* ds, uint32_t id, Graph** out) {
    if (id >= ds->graphs.size()) return set_error(FK_ERR_INVALID, "invalid graph id");  // lib.rs:592
    *out = ds->graphs[id].get();
    return FK_OK;
}

hipKernelNodeParams launch_params(Launch& l, void** slot) {
    hipKernelNodeParams p;
    memset(&p, 0, sizeof(p));
    p.func = const_cast<void*>(l.func);
    p.gridDim = l.grid;
    p.blockDim = l.block;
    p.sharedMemBytes = l.shmem;
    l.params(slot);  // `slot` holds kMaxKernelParams entries
    p.kernelParams = slot;
    p.extra = nullptr;
    return p;
}
hipKernelNodeParams node_params(Node& n, void** slot) { return launch_params(n.launch, slot); }

// Does the later dispatch `b` have to wait for the earlier `a` (RAW / WAW / WAR on overlapping byte ranges)?
bool direct_dep(const std::vector<fk_arg>& aa, const SlotRW& arw, const std::vector<fk_arg>& ba, const SlotRW& brw) {
    for (uint32_t ws : arw.writes) {
        for (uint32_t s : brw.reads)
            if (overlap(aa[ws], ba[s])) return true;
        for (uint32_t s : brw.writes)
            if (overlap(aa[ws], ba[s])) return true;
    }
    for (uint32_t rs : arw.reads)
        for (uint32_t s : brw.writes)
            if (overlap(aa[rs], ba[s])) return true;
    return false;
}

// RAW / WAW / WAR edges on overlapping byte ranges, transitively reduced.
// Returns the ancestor sets (bit j of anc[i]: node j runs before node i).
std::vector<std::vector<uint64_t>> derive_edges(std::vector<Node>& nodes, const uint8_t* barriers) {
    const size_t n = nodes.size();
    const size_t words = (n + 63) / 64;
    std::vector<std::vector<uint64_t>> anc(n, std::vector<uint64_t>(words, 0));
    for (size_t i = 0; i < n; ++i) {
        std::vector<uint32_t> cand;
        for (size_t j = 0; j < i; ++j) {
            const Node &a = nodes[j], &b = nodes[i];
            const bool dep = (barriers && barriers[i]) || direct_dep(a.d.args, a.rw, b.d.args, b.rw);
            if (dep) cand.push_back((uint32_t)j);
        }
        // keep a candidate only if no later candidate already descends from it
        nodes[i].deps.clear();
        for (size_t c = cand.size(); c-- > 0;) {
            const uint32_t j = cand[c];
            if (anc[i][j / 64] >> (j % 64) & 1) continue;  // implied through a kept dependency
            nodes[i].deps.push_back(j);
            anc[i][j / 64] |= 1ull << (j % 64);
            for (size_t w = 0; w < words; ++w) anc[i][w] |= anc[j][w];
        }
        std::sort(nodes[i].deps.begin(), nodes[i].deps.end());
    }
    return anc;
}

// The families whose launches are 512 workgroups that wait for one another (slots end: out_sums, clear_sums, workspace).
bool is_xcd_launch(const std::string& kernel) {
    return kernel.compare(0, 22, "fusekit_xcd_attn_block") == 0 || kernel.compare(0, 21, "fusekit_xcd_mlp_block") == 0 ||
           kernel.compare(0, 21, "fusekit_xcd_moe_block") == 0 || kernel.compare(0, 21, "fusekit_xcd_mla_block") == 0;
}

// An XCD-resident launch needs the whole device to itself: its 512 workgroups must all be resident at once, two per
// CU, and a kernel running beside it would hold CUs and leave some of them waiting (the hand-over waits would then
// run into their spin limit).  Inside a graph that means every other node must be ordered before or after it.
fk_status require_xcd_nodes_ordered(const std::vector<Node>& nodes, const std::vector<std::vector<uint64_t>>& anc) {
    auto is_xcd = [](const Node& nd) { return is_xcd_launch(nd.d.kernel); };
    for (size_t i = 0; i < nodes.size(); ++i) {
        if (!is_xcd(nodes[i])) continue;
        for (size_t j = 0; j < nodes.size(); ++j) {
            if (j == i) continue;
            const bool ordered = j < i ? (anc[i][j / 64] >> (j % 64) & 1) != 0 : (anc[j][i / 64] >> (i % 64) & 1) != 0;
            if (!ordered)
                return set_error(FK_ERR_UNSUPPORTED, "graph: dispatch " + std::to_string(i) + " (" + nodes[i].d.kernel +
                                                         ") needs the device to itself, but dispatch " + std::to_string(j) + " (" +
                                                         nodes[j].d.kernel + ") is not ordered against it; pass barriers that "
                                                         "order them (a decode graph built as a chain does)");
        }
    }
    return FK_OK;
}

fk_status timed(DispatcherState* ds, double* gpu_seconds, const std::function<fk_status()>& body) {
    FK_HIP(hipEventRecord(ds->ev0, ds->stream));
    FK_TRY(body());
    FK_HIP(hipEventRecord(ds->ev1, ds->stream));
    FK_HIP(hipEventSynchronize(ds->ev1));
    float ms = 0.f;
    FK_HIP(hipEventElapsedTime(&ms, ds->ev0, ds->ev1));
    if (gpu_seconds) *gpu_seconds = ms * 1e-3;
    return FK_OK;
}

// ---- persistent whole-token kernel: match the canonical decode pipeline ----
//   step_init, embed_lookup_decode, L x [rmsnorm_qkv, rope/store (one fused task or the
//   q + kv pair, plain or head-norm), sdpa_decode, linear_residual, rmsnorm_gateup_swiglu,
//   linear_residual], final_rmsnorm_lm_head, argmax_logits_decode (with history)
// and turn it into the argument tables of decode_token_kernel.
bool is_family(const Node& n, const char* prefix) {
    const Family* f = find_family(n.d.kernel);
    return f && strcmp(f->prefix, prefix) == 0;
}

template <typename T>
const T& blob(const Node& n) {
    return *reinterpret_cast<const T*>(n.launch.args);
}

fk_status build_token_kernel(std::vector<Node>& nodes, uint32_t spin_limit, Graph* g) {
    const DeviceFacts* dev;
    FK_TRY(device_facts(&dev));
    auto bad = [](const std::string& why) {
        return set_error(FK_ERR_UNSUPPORTED, "persistent decode: task list is not the canonical dense pipeline (" + why + ")");
    };
    const size_t n = nodes.size();
    if (n < 10) return bad("too few tasks");
    if (!is_family(nodes[0], "fusekit_step_init")) return bad("task 0 is not step_init");
    if (!is_family(nodes[1], "fusekit_embed_lookup_decode")) return bad("task 1 is not embed_lookup_decode");
    if (nodes[1].d.u("bits", 16) != 16) return bad("quantised embedding table");
    if (!is_family(nodes[n - 2], "fusekit_final_rmsnorm_lm_head") || nodes[n - 2].d.u("bits", 16) != 16)
        return bad("no dense bf16 final_rmsnorm_lm_head before the argmax");
    if (!is_family(nodes[n - 1], "fusekit_argmax_logits_decode") || nodes[n - 1].d.args.size() != 5)
        return bad("last task is not argmax_logits_decode with history");

    TokenArgs t;
    memset(&t, 0, sizeof(t));
    t.step_counter = arg_ptr<uint32_t>(nodes[0].d, 0);
    t.offset = arg_ptr<uint32_t>(nodes[0].d, 1);
    t.kv_len = arg_ptr<uint32_t>(nodes[0].d, 2);
    t.token = arg_ptr<uint32_t>(nodes[1].d, 0);
    t.embed = arg_ptr<const uint16_t>(nodes[1].d, 1);
    t.x0 = arg_ptr<uint16_t>(nodes[1].d, 2);
    t.hidden = nodes[1].d.u("hidden");
    t.vocab = nodes[1].d.u("vocab");
    t.embed_scale = (float)nodes[1].d.param("output_scale", 1.0);
    const Node& am = nodes[n - 1];
    t.logits = arg_ptr<const uint16_t>(am.d, 0);
    if (arg_ptr<uint32_t>(am.d, 1) != t.token) return bad("argmax does not feed the embedding's token buffer");
    t.history = arg_ptr<uint32_t>(am.d, 3);
    t.hist_counter = arg_ptr<uint32_t>(am.d, 4);
    t.hist_capacity = (uint32_t)(am.d.args[3].nbytes / 4);
    if (am.d.u("vocab") != t.vocab) return bad("argmax and embedding disagree on the vocabulary");

    // walk the layers
    struct LayerIdx { size_t qkv, rope0, rope1, sdpa, o, gateup, down; };
    std::vector<LayerIdx> layers;
    size_t i = 2;
    while (i < n - 2) {
        LayerIdx L{};
        if (!is_family(nodes[i], "fusekit_rmsnorm_qkv")) return bad("expected rmsnorm_qkv at task " + std::to_string(i));
        L.qkv = i++;
        if (is_family(nodes[i], "fusekit_qkv_rope_store_decode")) {
            L.rope0 = L.rope1 = i++;
        } else if ((is_family(nodes[i], "fusekit_rope_q_decode") && is_family(nodes[i + 1], "fusekit_rope_kv_cache_store_decode")) ||
                   (is_family(nodes[i], "fusekit_rmsnorm_rope_q_decode") &&
                    is_family(nodes[i + 1], "fusekit_rmsnorm_rope_kv_cache_store_decode"))) {
            L.rope0 = i;
            L.rope1 = i + 1;
            i += 2;
        } else {
            return bad("expected a rope / KV-store task at " + std::to_string(i));
        }
        if (i + 4 > n - 2) return bad("truncated layer");
        if (!is_family(nodes[i], "fusekit_sdpa_decode")) return bad("expected sdpa_decode at task " + std::to_string(i));
        L.sdpa = i++;
        if (!is_family(nodes[i], "fusekit_linear_residual")) return bad("expected linear_residual at task " + std::to_string(i));
        L.o = i++;
        if (!is_family(nodes[i], "fusekit_rmsnorm_gateup_swiglu")) return bad("expected rmsnorm_gateup_swiglu at task " + std::to_string(i));
        L.gateup = i++;
        if (!is_family(nodes[i], "fusekit_linear_residual")) return bad("expected linear_residual at task " + std::to_string(i));
        L.down = i++;
        layers.push_back(L);
    }
    if (layers.empty()) return bad("no layers");
    const uint32_t bits = nodes[layers[0].qkv].d.u("bits", 4);
    const int kind = bits == 4 ? W_Q4 : (bits == 8 ? W_Q8 : W_BF16);
    const SdpaArgs& s0 = blob<SdpaArgs>(nodes[layers[0].sdpa]);
    const uint32_t G = s0.n_heads / s0.n_kv;
    const int gt = G >= 8 ? 8 : (G >= 4 ? (G == 4 ? 4 : 8) : (G >= 2 ? (G == 2 ? 2 : 4) : 1));
    if (gt == 1) return bad("one query head per kv head");

    std::vector<GemvArgs> gemv(4 * layers.size() + 1);
    std::vector<SdpaArgs> sdpa(layers.size());
    uint32_t grid = (uint32_t)dev->cus * 4, lds_max = 0;
    for (int pass = 0; pass < 3; ++pass) {
        t_gemv_grid_override = grid;
        lds_max = 0;
        fk_status st = FK_OK;
        auto replan = [&](size_t node, GemvArgs* out) -> fk_status {
            Launch l;
            SlotRW rw;
            fk_status r = plan_dispatch(nodes[node].d, &l, &rw);
            if (r != FK_OK) return r;
            *out = *reinterpret_cast<const GemvArgs*>(l.args);
            lds_max = std::max(lds_max, l.shmem);
            return FK_OK;
        };
        for (size_t li = 0; li < layers.size() && st == FK_OK; ++li) {
            const LayerIdx& L = layers[li];
            for (size_t node : {L.qkv, L.o, L.gateup, L.down})
                if (nodes[node].d.u("bits", 4) != bits) st = bad("layers mix weight formats");
            if (st != FK_OK) break;
            if ((st = replan(L.qkv, &gemv[4 * li])) != FK_OK) break;
            if ((st = replan(L.o, &gemv[4 * li + 1])) != FK_OK) break;
            if ((st = replan(L.gateup, &gemv[4 * li + 2])) != FK_OK) break;
            if ((st = replan(L.down, &gemv[4 * li + 3])) != FK_OK) break;
        }
        if (st == FK_OK) st = replan(n - 2, &gemv[4 * layers.size()]);
        t_gemv_grid_override = 0;
        FK_TRY(st);
        lds_max = std::max(lds_max, (uint32_t)(sdpa_lds_floats(gt, sdpa_chunk_len(s0.qk_dim, s0.v_dim, true), s0.qk_dim,
                                                                 s0.v_dim, true) * sizeof(float)));
        lds_max = std::max(lds_max, (uint32_t)(kGemvBlock / kWave * sizeof(unsigned long long)));
        uint32_t max_grid = 0;
        FK_TRY(token_kernel_max_grid(kind, gt, lds_max, &max_grid));
        if (max_grid == grid) break;
        grid = max_grid;
    }
    {   // the final grid is what fits with the final LDS need
        uint32_t max_grid = 0;
        FK_TRY(token_kernel_max_grid(kind, gt, lds_max, &max_grid));
        if (grid > max_grid) grid = max_grid;
    }
    if ((uint64_t)grid * kGemvBlock < t.hidden) return bad("hidden size exceeds one thread per element");

    for (size_t li = 0; li < layers.size(); ++li) {
        const LayerIdx& L = layers[li];
        SdpaArgs s = blob<SdpaArgs>(nodes[L.sdpa]);
        if (s.kv_len_ptr != t.kv_len) return bad("sdpa does not read the step counter's kv_len");
        if (s.n_heads / s.n_kv != G || s.qk_dim != s0.qk_dim || s.v_dim != s0.v_dim) return bad("layers differ in head layout");
        if (s.qk_dim != s.v_dim) return bad("qk_dim != v_dim");
        const RopeArgs& r0 = blob<RopeArgs>(nodes[L.rope0]);
        const RopeArgs& r1 = blob<RopeArgs>(nodes[L.rope1]);
        if (r0.offset_ptr != t.offset || r1.offset_ptr != t.offset) return bad("rope does not read the step counter's offset");
        if (r1.write_offset_ptr && r1.write_offset_ptr != t.offset) return bad("cache row is not the rope position");
        if (r0.q != s.q) return bad("sdpa does not read the rope task's q");
        if (r1.cache_k != s.k || r1.cache_v != s.v) return bad("sdpa does not read the caches the store task writes");
        if (r1.capacity != s.capacity || r1.k_dim != s.qk_dim || r1.v_dim != s.v_dim || r0.head_dim != s.qk_dim)
            return bad("rope and sdpa disagree on dims or capacity");
        if (!r0.rope_on || !r1.rope_on || r0.rope_dims != r1.rope_dims) return bad("rotation must be on for q and k alike");
        if ((r0.q_norm == nullptr) != (r1.k_norm == nullptr)) return bad("q and k head norms must come together");
        // ranges of the in-kernel attention are shorter than the stand-alone kernel's; its
        // partials and counters live in the private arena, sized for that
        s.chunk_len = sdpa_chunk_len(s.qk_dim, s.v_dim, true);
        s.n_splits = (s.capacity + s.chunk_len - 1) / s.chunk_len;
        s.chunks_per_block = 1;
        s.rows = 1;
        s.k_new = r1.k;
        s.v_new = r1.v;
        s.q_norm = r0.q_norm;
        s.k_norm = r1.k_norm;
        s.cache_k_w = r1.cache_k;
        s.cache_v_w = r1.cache_v;
        s.rope_dims = r0.rope_dims;
        s.eps = r0.eps;
        s.base_log2 = r0.base_log2;
        sdpa[li] = s;
    }

    // Private activation arena: every layer gets its own x / q / k / v / att / mid
    // buffers (128-byte aligned), so inside one launch no address is read before the
    // barrier that follows its only write -- plain cached loads can never be stale.
    const uint32_t hidden = t.hidden, n_q = s0.n_heads * s0.qk_dim, n_kvd = s0.n_kv * s0.qk_dim;
    const uint32_t inter = gemv[2].n[0];
    auto al = [](size_t v) { return (v + 127) / 128 * 128; };
    const size_t sz_x = al((size_t)hidden * 2), sz_q = al((size_t)n_q * 2), sz_kv = al((size_t)n_kvd * 2),
                 sz_mid = al((size_t)inter * 2);
    const size_t per_layer = 2 * sz_x + 2 * sz_q + 2 * sz_kv + sz_mid;
    const size_t sz_part = al((size_t)s0.n_heads * sdpa[0].n_splits * (s0.v_dim + 2) * sizeof(float));
    const size_t sz_cnt = al((size_t)s0.n_heads * sizeof(uint32_t));
    if (s0.qk_dim > 2 * kGemvBlock) return bad("head too wide for the rotary table");
    const size_t sz_tab = al((size_t)s0.qk_dim * sizeof(float));
    const size_t arena_bytes = per_layer * layers.size() + sz_x + sz_part + sz_cnt + sz_tab;
    // device tables: [gemv][sdpa][argmax partials][barrier counters][flags][arena]
    const size_t gemv_bytes = gemv.size() * sizeof(GemvArgs), sdpa_bytes = sdpa.size() * sizeof(SdpaArgs);
    const size_t part_off = (gemv_bytes + sdpa_bytes + 255) / 256 * 256, part_bytes = (size_t)grid * 8;
    const size_t bar_off = (part_off + part_bytes + 255) / 256 * 256;
    const size_t n_groups = ((size_t)grid + 31) / 32;
    const size_t top_off = bar_off + n_groups * 128;
    const size_t trace_cap = 5 * layers.size() + 8;
    const size_t trace_off = top_off + 4 * 128;
    const size_t arena_off = (trace_off + trace_cap * 8 + 127) / 128 * 128;
    const size_t total = arena_off + arena_bytes;
    FK_HIP(hipMalloc(&g->d_tables, total));
    char* base = reinterpret_cast<char*>(g->d_tables);
    {
        // layer l: X0_l (input) | X1_l | q | att | k | v | mid ; X0_L after the last layer
        auto buf = [&](size_t l, size_t off) { return reinterpret_cast<uint16_t*>(base + arena_off + l * per_layer + off); };
        const size_t o_x0 = 0, o_x1 = sz_x, o_q = 2 * sz_x, o_att = o_q + sz_q, o_k = o_att + sz_q, o_v = o_k + sz_kv,
                     o_mid = o_v + sz_kv;
        t.x0 = buf(0, o_x0);
        for (size_t l = 0; l < layers.size(); ++l) {
            GemvArgs& qkv = gemv[4 * l];
            GemvArgs& op = gemv[4 * l + 1];
            GemvArgs& gu = gemv[4 * l + 2];
            GemvArgs& dn = gemv[4 * l + 3];
            if (qkv.n_mats != 3 || qkv.n[0] != n_q || qkv.n[1] != n_kvd || qkv.n[2] != n_kvd || qkv.K != hidden ||
                op.K != n_q || op.n[0] != hidden || gu.K != hidden || gu.n[0] != inter || dn.K != inter ||
                dn.n[0] != hidden || !op.res || !dn.res || op.res2 || dn.res2)
                return bad("layer shapes do not chain");
            qkv.x = buf(l, o_x0);
            qkv.y[0] = buf(l, o_q);
            qkv.y[1] = buf(l, o_k);
            qkv.y[2] = buf(l, o_v);
            sdpa[l].q = buf(l, o_q);
            sdpa[l].k_new = buf(l, o_k);
            sdpa[l].v_new = buf(l, o_v);
            sdpa[l].out = buf(l, o_att);
            op.x = buf(l, o_att);
            op.res = buf(l, o_x0);
            op.y[0] = buf(l, o_x1);
            gu.x = buf(l, o_x1);
            gu.y[0] = buf(l, o_mid);
            dn.x = buf(l, o_mid);
            dn.res = buf(l, o_x1);
            dn.y[0] = buf(l + 1, o_x0);  // the next layer's input (or the LM head's)
        }
        GemvArgs& head = gemv[4 * layers.size()];
        if (head.K != hidden) return bad("LM head width");
        head.x = buf(layers.size(), o_x0);
        char* tail = base + arena_off + per_layer * layers.size() + sz_x;
        for (size_t l = 0; l < layers.size(); ++l) {
            sdpa[l].partials = reinterpret_cast<float*>(tail);
            sdpa[l].counters = reinterpret_cast<uint32_t*>(tail + sz_part);
        }
        FK_HIP(hipMemset(tail + sz_part, 0, sz_cnt));
        t.rope_tab = reinterpret_cast<float*>(tail + sz_part + sz_cnt);
        t.rope_dims = sdpa[0].rope_dims;
        t.rope_base_log2 = sdpa[0].base_log2;
        for (size_t l = 0; l < layers.size(); ++l) {
            if (sdpa[l].rope_dims != t.rope_dims || sdpa[l].base_log2 != t.rope_base_log2)
                return bad("layers differ in rotary parameters");
            sdpa[l].rope_tab = t.rope_tab;
        }
    }
    std::vector<unsigned char> host(arena_off, 0);
    memcpy(host.data(), gemv.data(), gemv_bytes);
    memcpy(host.data() + gemv_bytes, sdpa.data(), sdpa_bytes);
    FK_HIP(hipMemcpy(g->d_tables, host.data(), arena_off, hipMemcpyHostToDevice));
    t.gemv = reinterpret_cast<const GemvArgs*>(base);
    t.sdpa = reinterpret_cast<const SdpaArgs*>(base + gemv_bytes);
    t.n_layers = (uint32_t)layers.size();
    t.argmax_partial = reinterpret_cast<unsigned long long*>(base + part_off);
    t.bar_groups = reinterpret_cast<unsigned long long*>(base + bar_off);
    t.bar_counter = reinterpret_cast<unsigned long long*>(base + top_off);
    t.bar_flag = reinterpret_cast<unsigned long long*>(base + top_off + 128);
    t.bar_base = reinterpret_cast<unsigned long long*>(base + top_off + 256);
    t.abort_flag = reinterpret_cast<uint32_t*>(base + top_off + 384);
    t.spin_limit = spin_limit;
    t.trace = reinterpret_cast<unsigned long long*>(base + trace_off);
    t.trace_capacity = (uint32_t)trace_cap;
    g->d_abort = t.abort_flag;
    g->d_trace = t.trace;
    g->trace_len = (uint32_t)(5 * layers.size() + 4);

    TokenKernelSpec spec;
    spec.kind = kind;
    spec.gt = gt;
    spec.lds_bytes = lds_max;
    spec.args = t;
    FK_TRY(plan_token_kernel(spec, grid, &g->token_launch));
    g->persistent = true;
    return FK_OK;
}

// Called with the stream idle.  A failed XCD-resident launch leaves partial sums behind: the control block is reset
// by the check, the graph's sum rows are zeroed here (every token starts from zero rows), and the error text tells the
// caller to decode the token again, which rewrites the cache rows of its position.
fk_status check_abort(Graph* g) {
    for (void* ws : g->xcd_controls) {
        const fk_status st = xcd_check_control(ws);
        if (st != FK_OK) {
            const std::string msg = fk_last_error();
            for (const auto& row : g->xcd_sum_rows) FK_HIP(hipMemset(row.first, 0, row.second));
            return set_error(st, msg + " [the graph's sum rows were zeroed]");
        }
    }
    if (!g->persistent) return FK_OK;
    uint32_t flag = 0;
    FK_HIP(hipMemcpy(&flag, g->d_abort, 4, hipMemcpyDeviceToHost));
    // The flag and the barrier counters stay as the aborted launch left them: the graph is unusable from here
    // on and every later call reports the same error until the caller builds a new one.
    if (flag)
        return set_error(FK_ERR_HIP, "persistent decode kernel: a grid barrier wait exceeded its spin limit; results are "
                                     "invalid and this graph stays unusable: rebuild it with fk_build_decode_graph");
    return FK_OK;
}

}  // namespace
}  // namespace fk

using namespace fk;

extern "C" {

fk_status fk_load_dispatcher(const char* code_object_path, const char* task_graph_path, fk_handle* out) {
    if (!out) return set_error(FK_ERR_INVALID, "null out");
    auto ds = std::make_unique<DispatcherState>();
    // The kernels are compiled into this library; a code-object path is accepted
    // for artifact compatibility and only checked for existence.
    if (code_object_path && *code_object_path && strcmp(code_object_path, "builtin") != 0) {
        std::ifstream f(code_object_path, std::ios::binary);
        if (!f) return set_error(FK_ERR_NOT_FOUND, std::string("code object not found: ") + code_object_path);
    }
    if (task_graph_path && *task_graph_path) {
        std::ifstream f(task_graph_path, std::ios::binary);
        if (!f) return set_error(FK_ERR_NOT_FOUND, std::string("task graph not found: ") + task_graph_path);
        std::stringstream ss;
        ss << f.rdbuf();
        json::Value root;
        std::string err;
        const std::string text = ss.str();
        if (!json::Parser(text).parse(&root, &err)) return set_error(FK_ERR_IO, "task_graph.json: " + err);
        const json::Value* ver = root.get("version");
        if (!ver || !ver->is_number() || (int)ver->num != 2)
            return set_error(FK_ERR_INVALID, "task_graph.json: unsupported version (need 2)");  // plan.rs:175-180
        const json::Value* tasks = root.get("tasks");
        if (!tasks || !tasks->is_array()) return set_error(FK_ERR_INVALID, "task_graph.json: missing tasks[]");
        for (const json::Value& t : tasks->arr) {
            const json::Value* k = t.get("kernel");
            if (!k || !k->is_string()) return set_error(FK_ERR_INVALID, "task_graph.json: task without kernel name");
            if (!find_family(k->str))
                return set_error(FK_ERR_INVALID, "kernel '" + k->str + "' is not in this library");
            if (std::find(ds->kernel_names.begin(), ds->kernel_names.end(), k->str) == ds->kernel_names.end())
                ds->kernel_names.push_back(k->str);
        }
        ds->task_graph_path = task_graph_path;
    } else {
        for (const Family& f : kFamilies) ds->kernel_names.push_back(f.prefix);
    }
    for (const std::string& s : ds->kernel_names) ds->kernel_name_ptrs.push_back(s.c_str());
    // the artifact is validated before the device is touched, so a bad artifact is
    // reported as such even on a machine without a GPU
    const DeviceFacts* dev;
    FK_TRY(device_facts(&dev));
    FK_HIP(hipStreamCreateWithFlags(&ds->stream, hipStreamNonBlocking));
    FK_HIP(hipEventCreate(&ds->ev0));
    FK_HIP(hipEventCreate(&ds->ev1));
    std::lock_guard<std::mutex> lk(g_mu);
    g_dispatchers.push_back(std::move(ds));
    *out = (fk_handle)g_dispatchers.size();
    return FK_OK;
}

fk_status fk_kernel_names(fk_handle h, const char* const** names, size_t* n) {
    DispatcherState* ds;
    FK_TRY(get_dispatcher(h, &ds));
    if (!names || !n) return set_error(FK_ERR_INVALID, "null out");
    *names = ds->kernel_name_ptrs.data();
    *n = ds->kernel_name_ptrs.size();
    return FK_OK;
}

fk_status fk_dispatcher_stream(fk_handle h, fk_stream* out) {
    DispatcherState* ds;
    FK_TRY(get_dispatcher(h, &ds));
    if (!out) return set_error(FK_ERR_INVALID, "null out");
    *out = ds->stream;
    return FK_OK;
}

fk_status fk_dispatch_batch(fk_handle h, const fk_dispatch* list, size_t n, double* gpu_seconds) {
    DispatcherState* ds;
    FK_TRY(get_dispatcher(h, &ds));
    if (!list && n) return set_error(FK_ERR_INVALID, "null dispatch list");
    std::lock_guard<std::mutex> lk(ds->mu);
    std::vector<Launch> launches(n);
    for (size_t i = 0; i < n; ++i) {  // validate everything before launching anything
        Dispatch d;
        SlotRW rw;
        FK_TRY(copy_dispatch(list[i], &d));
        FK_TRY(plan_dispatch(d, &launches[i], &rw));
    }
    return timed(ds, gpu_seconds, [&]() -> fk_status {
        for (size_t i = 0; i < n; ++i) FK_TRY(run_launch(launches[i], ds->stream));  // stream order = barrier between each
        return FK_OK;
    });
}

fk_status fk_dispatch_kernel(fk_handle h, const fk_dispatch* d, double* gpu_seconds) {
    if (!d) return set_error(FK_ERR_INVALID, "null dispatch");
    return fk_dispatch_batch(h, d, 1, gpu_seconds);
}

fk_status fk_plan_geometry(fk_handle h, const fk_dispatch* d, fk_launch_geometry* out) {
    DispatcherState* ds;
    FK_TRY(get_dispatcher(h, &ds));
    if (!d || !out) return set_error(FK_ERR_INVALID, "null dispatch or out");
    Dispatch disp;
    Launch l;
    SlotRW rw;
    FK_TRY(copy_dispatch(*d, &disp));
    FK_TRY(plan_dispatch(disp, &l, &rw));
    memset(out, 0, sizeof(*out));
    if (1 + l.then.size() > FK_MAX_TASK_KERNELS || disp.args.size() > FK_MAX_TASK_SLOTS)
        return set_error(FK_ERR_UNSUPPORTED, "dispatch exceeds the geometry record");
    auto put = [&](const Launch& k) {
        const uint32_t i = out->n_kernels++;
        out->grid[i][0] = k.grid.x; out->grid[i][1] = k.grid.y; out->grid[i][2] = k.grid.z;
        out->threadgroup[i][0] = k.block.x; out->threadgroup[i][1] = k.block.y; out->threadgroup[i][2] = k.block.z;
        out->lds_bytes[i] = k.shmem;
    };
    put(l);
    for (const Launch& k : l.then) put(k);
    out->n_slots = (uint32_t)disp.args.size();
    for (uint32_t s : rw.reads) out->slot_access[s] |= 1;
    for (uint32_t s : rw.writes) out->slot_access[s] |= 2;
    return FK_OK;
}

// The argument block a member of a fused run contributes to the run's device tables: the dispatch planned once
// more with the parameter `token` (the one launch sizes some tiles differently).
fk_status plan_for_token(const Dispatch& d, Launch* l) {
    Dispatch t = d;
    t.params.emplace_back("token", 1.0);
    SlotRW rw;
    return plan_dispatch(t, l, &rw);
}

bool is_family(const Dispatch& d, const char* fam) {
    const size_t n = strlen(fam);
    return d.kernel.compare(0, n, fam) == 0 && (d.kernel.size() == n || d.kernel[n] == '_');
}

fk_status find_fused_runs(Graph* g) {
    const size_t n = g->nodes.size();
    g->fused_of.assign(n, -1);
    size_t i = 0;
    while (i < n) {
        const Dispatch& d = g->nodes[i].d;
        if (!(is_family(d, "fusekit_xcd_attn_block") && d.u("token_launch", 0) != 0)) {
            ++i;
            continue;
        }
        if (d.u("token_launch", 0) == 2) {
            // one launch per LAYER: this attention launch and the MLP launch behind it, as they were planned
            if (i + 1 < n && is_family(g->nodes[i + 1].d, "fusekit_xcd_mlp_block") && g->nodes[i + 1].d.u("token_launch", 0) == 2) {
                Graph::FusedRun run;
                run.first = i;
                run.count = 2;
                const fk_status st = plan_xcd_layer(g->nodes[i].launch, g->nodes[i + 1].launch, &run.launch);
                if (st == FK_ERR_UNSUPPORTED) {  // e.g. a shape whose tiles need the pass loop: the two launches stay
                    i += 2;
                    continue;
                }
                FK_TRY(st);
                g->fused.push_back(run);
                g->fused_of[i] = g->fused_of[i + 1] = (int)g->fused.size() - 1;
                i += 2;
            } else {
                ++i;
            }
            continue;
        }
        size_t j = i;
        while (j + 1 < n && is_family(g->nodes[j].d, "fusekit_xcd_attn_block") && g->nodes[j].d.u("token_launch", 0) == 1 &&
               is_family(g->nodes[j + 1].d, "fusekit_xcd_mlp_block") && g->nodes[j + 1].d.u("token_launch", 0) == 1 &&
               g->nodes[j].d.u("bits", 4) == d.u("bits", 4))
            j += 2;
        const size_t count = j - i;
        if (count < 2) {
            ++i;
            continue;
        }
        const uint32_t layers = (uint32_t)(count / 2);
        std::vector<XcdAttnArgs> ha(layers);
        std::vector<XcdMlpArgs> hm(layers);
        uint32_t attn_lds = 0, mlp_lds = 0;
        for (uint32_t l = 0; l < layers; ++l) {
            Launch la, lm;
            FK_TRY(plan_for_token(g->nodes[i + 2 * l].d, &la));
            FK_TRY(plan_for_token(g->nodes[i + 2 * l + 1].d, &lm));
            if (la.args_size != sizeof(XcdAttnArgs) || lm.args_size != sizeof(XcdMlpArgs))
                return set_error(FK_ERR_INVALID, "fused layer run: unexpected argument block");
            memcpy(&ha[l], la.args, sizeof(XcdAttnArgs));
            memcpy(&hm[l], lm.args, sizeof(XcdMlpArgs));
            attn_lds = std::max(attn_lds, la.shmem);
            mlp_lds = std::max(mlp_lds, lm.shmem);
        }
        Graph::FusedRun run;
        run.first = i;
        run.count = count;
        g->fused.push_back(run);
        Graph::FusedRun& r = g->fused.back();
        FK_HIP(hipMalloc(&r.d_attn, layers * sizeof(XcdAttnArgs)));
        FK_HIP(hipMalloc(&r.d_mlp, layers * sizeof(XcdMlpArgs)));
        FK_HIP(hipMemcpy(r.d_attn, ha.data(), layers * sizeof(XcdAttnArgs), hipMemcpyHostToDevice));
        FK_HIP(hipMemcpy(r.d_mlp, hm.data(), layers * sizeof(XcdMlpArgs), hipMemcpyHostToDevice));
        FK_TRY(plan_xcd_token(ha.data(), hm.data(), layers, d.u("bits", 4), reinterpret_cast<const XcdAttnArgs*>(r.d_attn),
                              reinterpret_cast<const XcdMlpArgs*>(r.d_mlp), attn_lds, mlp_lds, &r.launch));
        for (size_t m = i; m < j; ++m) g->fused_of[m] = (int)g->fused.size() - 1;
        i = j;
    }
    return FK_OK;
}

fk_status fk_build_graph(fk_handle h, const fk_dispatch* list, size_t n, const uint8_t* barriers, uint32_t* graph_id) {
    DispatcherState* ds;
    FK_TRY(get_dispatcher(h, &ds));
    if (!list || n == 0 || !graph_id) return set_error(FK_ERR_INVALID, "empty dispatch list or null out");
    std::lock_guard<std::mutex> lk(ds->mu);
    auto g = std::make_unique<Graph>();
    g->nodes.resize(n);
    for (size_t i = 0; i < n; ++i) {
        FK_TRY(copy_dispatch(list[i], &g->nodes[i].d));
        FK_TRY(plan_dispatch(g->nodes[i].d, &g->nodes[i].launch, &g->nodes[i].rw));
    }
    const auto anc = derive_edges(g->nodes, barriers);
    FK_TRY(require_xcd_nodes_ordered(g->nodes, anc));
    if (barriers) g->barriers.assign(barriers, barriers + n);
    for (size_t i = 0; i < n; ++i) {
        const Node& nd = g->nodes[i];
        if (is_xcd_launch(nd.d.kernel)) {
            void* ws = nd.d.args.back().ptr;
            if (std::find(g->xcd_controls.begin(), g->xcd_controls.end(), ws) == g->xcd_controls.end()) g->xcd_controls.push_back(ws);
            // slots: [sums_in], ..., out_sums, clear_sums, workspace (the planners have checked count and sizes)
            const size_t na = nd.d.args.size(), row_bytes = xcd_sum_row_bytes(nd.d.u("hidden"));
            auto add_row = [&](void* p) {
                for (const auto& r : g->xcd_sum_rows)
                    if (r.first == p) return;
                g->xcd_sum_rows.emplace_back(p, row_bytes);
            };
            add_row(nd.d.args[na - 3].ptr);
            add_row(nd.d.args[na - 2].ptr);
            if (nd.d.kernel.compare(0, 21, "fusekit_xcd_moe_block") == 0) add_row(nd.d.args[na - 4].ptr);  // the shared expert's row
            if (nd.d.kernel.compare(0, 21, "fusekit_xcd_mla_block") == 0) {
                if (nd.d.u("has_sums", 0) != 0) add_row(nd.d.args[1].ptr);
                if (nd.d.u("has_clear2", 0) != 0) add_row(nd.d.args[na - 4].ptr);
            }
            if (nd.d.u("has_sums", 1) != 0) add_row(nd.d.args[0].ptr);
        }
    }
    FK_TRY(find_fused_runs(g.get()));
    FK_HIP(hipGraphCreate(&g->graph, 0));
    for (size_t i = 0; i < n; ++i) {
        Node& nd = g->nodes[i];
        const int fr = g->fused_of[i];
        if (fr >= 0) {
            Graph::FusedRun& run = g->fused[fr];
            if (i != run.first) {
                nd.node = run.node;  // later dispatches that depend on any member wait for the run's launch
                continue;
            }
            std::vector<hipGraphNode_t> deps;
            for (size_t m = run.first; m < run.first + run.count; ++m)
                for (uint32_t j : g->nodes[m].deps)
                    if (j < run.first) {
                        hipGraphNode_t dn = g->nodes[j].last();
                        if (std::find(deps.begin(), deps.end(), dn) == deps.end()) deps.push_back(dn);
                    }
            void* slot[kMaxKernelParams];
            hipKernelNodeParams p = launch_params(run.launch, slot);
            FK_HIP(hipGraphAddKernelNode(&run.node, g->graph, deps.data(), deps.size(), &p));
            nd.node = run.node;
            continue;
        }
        std::vector<hipGraphNode_t> deps;
        for (uint32_t j : nd.deps) {
            hipGraphNode_t dn = g->nodes[j].last();
            if (std::find(deps.begin(), deps.end(), dn) == deps.end()) deps.push_back(dn);
        }
        void* slot[kMaxKernelParams];
        hipKernelNodeParams p = node_params(nd, slot);
        FK_HIP(hipGraphAddKernelNode(&nd.node, g->graph, deps.data(), deps.size(), &p));
        nd.tail.resize(nd.launch.then.size());
        for (size_t f = 0; f < nd.launch.then.size(); ++f) {
            hipGraphNode_t prev = f ? nd.tail[f - 1] : nd.node;
            hipKernelNodeParams fp = launch_params(nd.launch.then[f], slot);
            FK_HIP(hipGraphAddKernelNode(&nd.tail[f], g->graph, &prev, 1, &fp));
        }
    }
    FK_HIP(hipGraphInstantiate(&g->exec, g->graph, nullptr, nullptr, 0));
    ds->graphs.push_back(std::move(g));
    *graph_id = (uint32_t)ds->graphs.size() - 1;
    return FK_OK;
}

fk_status fk_build_decode_graph(fk_handle h, const fk_dispatch* list, size_t n, int persistent, uint32_t spin_limit,
                                uint32_t* graph_id) {
    if (!persistent) {
        // List order, one node behind the other.  Every launch of a decode pipeline fills the chip, so independent
        // tasks gain nothing from running side by side, while a graph that forks anywhere (step_init beside the
        // embedding lookup is enough) is replayed through several queues and costs about 70 us more per replay.
        if (!list || n == 0) return set_error(FK_ERR_INVALID, "empty dispatch list or null out");
        const std::vector<uint8_t> chain(n, 1);
        return fk_build_graph(h, list, n, chain.data(), graph_id);
    }
    DispatcherState* ds;
    FK_TRY(get_dispatcher(h, &ds));
    if (!list || n == 0 || !graph_id) return set_error(FK_ERR_INVALID, "empty dispatch list or null out");
    std::lock_guard<std::mutex> lk(ds->mu);
    auto g = std::make_unique<Graph>();
    g->nodes.resize(n);
    for (size_t i = 0; i < n; ++i) {
        FK_TRY(copy_dispatch(list[i], &g->nodes[i].d));
        FK_TRY(plan_dispatch(g->nodes[i].d, &g->nodes[i].launch, &g->nodes[i].rw));
    }
    FK_TRY(build_token_kernel(g->nodes, spin_limit ? spin_limit : 4000000u, g.get()));
    FK_HIP(hipGraphCreate(&g->graph, 0));
    {
        hipKernelNodeParams p;
        memset(&p, 0, sizeof(p));
        void* slot = g->token_launch.args;
        p.func = const_cast<void*>(g->token_launch.func);
        p.gridDim = g->token_launch.grid;
        p.blockDim = g->token_launch.block;
        p.sharedMemBytes = g->token_launch.shmem;
        p.kernelParams = &slot;
        hipGraphNode_t node;
        FK_HIP(hipGraphAddKernelNode(&node, g->graph, nullptr, 0, &p));
    }
    FK_HIP(hipGraphInstantiate(&g->exec, g->graph, nullptr, nullptr, 0));
    ds->graphs.push_back(std::move(g));
    *graph_id = (uint32_t)ds->graphs.size() - 1;
    return FK_OK;
}

fk_status fk_graph_launch_shape(fk_handle h, uint32_t graph_id, uint32_t* persistent, uint32_t* grid, uint32_t* lds_bytes) {
    DispatcherState* ds;
    FK_TRY(get_dispatcher(h, &ds));
    std::lock_guard<std::mutex> lk(ds->mu);
    Graph* g;
    FK_TRY(get_graph(ds, graph_id, &g));
    if (persistent) *persistent = g->persistent ? 1u : 0u;
    if (grid) *grid = g->persistent ? g->token_launch.grid.x : 0u;
    if (lds_bytes) *lds_bytes = g->persistent ? g->token_launch.shmem : 0u;
    return FK_OK;
}

fk_status fk_graph_phase_trace(fk_handle h, uint32_t graph_id, double* seconds, uint32_t cap, uint32_t* n) {
    DispatcherState* ds;
    FK_TRY(get_dispatcher(h, &ds));
    std::lock_guard<std::mutex> lk(ds->mu);
    Graph* g;
    FK_TRY(get_graph(ds, graph_id, &g));
    if (!g->persistent || !n) return set_error(FK_ERR_INVALID, "phase trace: not a persistent decode graph");
    std::vector<unsigned long long> ticks(g->trace_len);
    FK_HIP(hipMemcpy(ticks.data(), g->d_trace, ticks.size() * 8, hipMemcpyDeviceToHost));
    *n = g->trace_len - 1;
    for (uint32_t i = 0; i + 1 < g->trace_len && i < cap && seconds; ++i)
        seconds[i] = (double)(ticks[i + 1] - ticks[i]) * 1e-8;  // constant-rate clock, 100 MHz
    return FK_OK;
}

fk_status fk_graph_info(fk_handle h, uint32_t graph_id, uint32_t* n_nodes, uint32_t* n_edges) {
    DispatcherState* ds;
    FK_TRY(get_dispatcher(h, &ds));
    std::lock_guard<std::mutex> lk(ds->mu);
    Graph* g;
    FK_TRY(get_graph(ds, graph_id, &g));
    uint32_t e = 0;
    for (const Node& nd : g->nodes) e += (uint32_t)nd.deps.size();
    if (n_nodes) *n_nodes = (uint32_t)g->nodes.size();
    if (n_edges) *n_edges = e;
    return FK_OK;
}

fk_status fk_graph_node_deps(fk_handle h, uint32_t graph_id, uint32_t node, uint32_t* deps, uint32_t cap, uint32_t* n) {
    DispatcherState* ds;
    FK_TRY(get_dispatcher(h, &ds));
    std::lock_guard<std::mutex> lk(ds->mu);
    Graph* g;
    FK_TRY(get_graph(ds, graph_id, &g));
    if (node >= g->nodes.size() || !n) return set_error(FK_ERR_INVALID, "node index out of range");
    const auto& d = g->nodes[node].deps;
    *n = (uint32_t)d.size();
    for (uint32_t i = 0; i < d.size() && i < cap && deps; ++i) deps[i] = d[i];
    return FK_OK;
}

fk_status fk_update_graph_bindings(fk_handle h, uint32_t graph_id, const fk_binding_update* ups, size_t n) {
    DispatcherState* ds;
    FK_TRY(get_dispatcher(h, &ds));
    if (!ups && n) return set_error(FK_ERR_INVALID, "null updates");
    std::lock_guard<std::mutex> lk(ds->mu);
    Graph* g;
    FK_TRY(get_graph(ds, graph_id, &g));
    if (g->persistent) return set_error(FK_ERR_UNSUPPORTED, "a persistent decode graph holds its bindings in device tables; rebuild it instead");
    // validate everything first: a refused update leaves the graph untouched
    std::vector<Dispatch> patched;
    std::vector<uint32_t> touched;
    for (size_t i = 0; i < n; ++i) {
        const fk_binding_update& u = ups[i];
        if (u.cmd_idx >= g->nodes.size()) return set_error(FK_ERR_INVALID, "binding update: command index out of range");
        if (u.slot >= g->nodes[u.cmd_idx].d.args.size())
            return set_error(FK_ERR_INVALID, "binding update: slot out of range");
        if (!u.ptr || u.nbytes == 0) return set_error(FK_ERR_INVALID, "binding update: null or empty buffer");  // lib.rs:602-606
        auto it = std::find(touched.begin(), touched.end(), u.cmd_idx);
        size_t k;
        if (it == touched.end()) {
            touched.push_back(u.cmd_idx);
            patched.push_back(g->nodes[u.cmd_idx].d);
            k = patched.size() - 1;
        } else {
            k = (size_t)(it - touched.begin());
        }
        patched[k].args[u.slot] = fk_arg{u.ptr, u.nbytes};
    }
    std::vector<Launch> launches(touched.size());
    std::vector<SlotRW> rws(touched.size());
    for (size_t k = 0; k < touched.size(); ++k) {
        FK_TRY(plan_dispatch(patched[k], &launches[k], &rws[k]));
        if (launches[k].then.size() != g->nodes[touched[k]].tail.size())
            return set_error(FK_ERR_UNSUPPORTED, "binding update changes the number of kernels of a task");
    }
    // The graph's edges were derived from the byte ranges of the ORIGINAL bindings.  A rebinding that makes two
    // dispatches overlap where they did not (or stop overlapping) would need other edges: refuse it, the caller
    // rebuilds the graph.  Compared pair by pair on the direct dependency predicate, before anything is applied.
    {
        auto view = [&](size_t idx, const std::vector<fk_arg>** args, const SlotRW** rw, bool patched_view) {
            auto it = std::find(touched.begin(), touched.end(), (uint32_t)idx);
            if (patched_view && it != touched.end()) {
                const size_t k = (size_t)(it - touched.begin());
                *args = &patched[k].args;
                *rw = &rws[k];
            } else {
                *args = &g->nodes[idx].d.args;
                *rw = &g->nodes[idx].rw;
            }
        };
        for (uint32_t t : touched)
            for (size_t o = 0; o < g->nodes.size(); ++o) {
                if (o == t) continue;
                const size_t first = o < t ? o : t, second = o < t ? t : o;
                if (!g->barriers.empty() && g->barriers[second]) continue;  // forced edge either way
                const std::vector<fk_arg>*a0, *b0, *a1, *b1;
                const SlotRW *ar0, *br0, *ar1, *br1;
                view(first, &a0, &ar0, false);
                view(second, &b0, &br0, false);
                view(first, &a1, &ar1, true);
                view(second, &b1, &br1, true);
                if (direct_dep(*a0, *ar0, *b0, *br0) != direct_dep(*a1, *ar1, *b1, *br1))
                    return set_error(FK_ERR_UNSUPPORTED,
                                     "binding update changes which dispatches overlap (the graph's dependency edges "
                                     "would change); rebuild the graph with fk_build_graph");
            }
    }
    // all checks passed: apply.  A HIP failure below can still leave the executable graph partly updated;
    // the error is reported and the caller must rebuild.
    std::vector<int> replan;
    for (size_t k = 0; k < touched.size(); ++k) {
        Node& nd = g->nodes[touched[k]];
        nd.d = patched[k];
        nd.launch = launches[k];
        nd.rw = rws[k];
        const int fr = g->fused_of.empty() ? -1 : g->fused_of[touched[k]];
        if (fr >= 0 && !g->fused[fr].d_attn) {
            replan.push_back(fr);  // a layer launch carries both argument blocks by value: planned again below
            continue;
        }
        if (fr >= 0) {
            // member of a run that executes as one launch: its argument block in the run's device table is replaced
            Graph::FusedRun& run = g->fused[fr];
            Launch lt;
            FK_TRY(plan_for_token(nd.d, &lt));
            const size_t pos = touched[k] - run.first;
            char* dst = (pos & 1) ? (char*)run.d_mlp + (pos / 2) * sizeof(XcdMlpArgs) : (char*)run.d_attn + (pos / 2) * sizeof(XcdAttnArgs);
            FK_HIP(hipMemcpy(dst, lt.args, lt.args_size, hipMemcpyHostToDevice));
            continue;
        }
        void* slot[kMaxKernelParams];
        hipKernelNodeParams p = node_params(nd, slot);
        FK_HIP(hipGraphExecKernelNodeSetParams(g->exec, nd.node, &p));
        for (size_t f = 0; f < nd.tail.size(); ++f) {
            hipKernelNodeParams fp = launch_params(nd.launch.then[f], slot);
            FK_HIP(hipGraphExecKernelNodeSetParams(g->exec, nd.tail[f], &fp));
        }
    }
    std::sort(replan.begin(), replan.end());
    replan.erase(std::unique(replan.begin(), replan.end()), replan.end());
    for (int fr : replan) {
        Graph::FusedRun& run = g->fused[fr];
        FK_TRY(plan_xcd_layer(g->nodes[run.first].launch, g->nodes[run.first + 1].launch, &run.launch));
        void* slot[kMaxKernelParams];
        hipKernelNodeParams p = launch_params(run.launch, slot);
        FK_HIP(hipGraphExecKernelNodeSetParams(g->exec, run.node, &p));
    }
    return FK_OK;
}

fk_status fk_execute_graph(fk_handle h, uint32_t graph_id, double* gpu_seconds) {
    DispatcherState* ds;
    FK_TRY(get_dispatcher(h, &ds));
    std::lock_guard<std::mutex> lk(ds->mu);
    Graph* g;
    FK_TRY(get_graph(ds, graph_id, &g));
    if (ds->pending) return set_error(FK_ERR_INVALID, "an async graph launch is pending; call fk_wait_pending first");
    FK_TRY(timed(ds, gpu_seconds, [&]() -> fk_status {
        FK_HIP(hipGraphLaunch(g->exec, ds->stream));
        return FK_OK;
    }));
    return check_abort(g);
}

fk_status fk_execute_graph_repeat(fk_handle h, uint32_t graph_id, uint32_t count, double* gpu_seconds) {
    DispatcherState* ds;
    FK_TRY(get_dispatcher(h, &ds));
    std::lock_guard<std::mutex> lk(ds->mu);
    Graph* g;
    FK_TRY(get_graph(ds, graph_id, &g));
    if (ds->pending) return set_error(FK_ERR_INVALID, "an async graph launch is pending; call fk_wait_pending first");
    FK_TRY(timed(ds, gpu_seconds, [&]() -> fk_status {
        for (uint32_t i = 0; i < count; ++i) FK_HIP(hipGraphLaunch(g->exec, ds->stream));
        return FK_OK;
    }));
    return check_abort(g);
}

fk_status fk_execute_graph_range(fk_handle h, uint32_t graph_id, uint32_t start, uint32_t end, double* gpu_seconds) {
    DispatcherState* ds;
    FK_TRY(get_dispatcher(h, &ds));
    std::lock_guard<std::mutex> lk(ds->mu);
    Graph* g;
    FK_TRY(get_graph(ds, graph_id, &g));
    if (start > end || end > g->nodes.size()) return set_error(FK_ERR_INVALID, "graph range out of bounds");  // lib.rs:781-786
    FK_TRY(timed(ds, gpu_seconds, [&]() -> fk_status {
        for (uint32_t i = start; i < end; ++i) FK_TRY(run_launch(g->nodes[i].launch, ds->stream));
        return FK_OK;
    }));
    return check_abort(g);
}

fk_status fk_profile_graph_nodes(fk_handle h, uint32_t graph_id, double* per_node_seconds, size_t n) {
    DispatcherState* ds;
    FK_TRY(get_dispatcher(h, &ds));
    std::lock_guard<std::mutex> lk(ds->mu);
    Graph* g;
    FK_TRY(get_graph(ds, graph_id, &g));
    if (!per_node_seconds || n < g->nodes.size()) return set_error(FK_ERR_INVALID, "profile buffer too small");
    for (size_t i = 0; i < g->nodes.size(); ++i) {
        FK_TRY(timed(ds, &per_node_seconds[i], [&]() -> fk_status { return run_launch(g->nodes[i].launch, ds->stream); }));
    }
    return check_abort(g);
}

fk_status fk_submit_graph_async(fk_handle h, uint32_t graph_id) {
    DispatcherState* ds;
    FK_TRY(get_dispatcher(h, &ds));
    std::lock_guard<std::mutex> lk(ds->mu);
    Graph* g;
    FK_TRY(get_graph(ds, graph_id, &g));
    if (ds->pending) return set_error(FK_ERR_INVALID, "an async graph launch is already pending");  // one in flight, lib.rs:57,695
    FK_HIP(hipEventRecord(ds->ev0, ds->stream));
    FK_HIP(hipGraphLaunch(g->exec, ds->stream));
    FK_HIP(hipEventRecord(ds->ev1, ds->stream));
    ds->pending = true;
    ds->pending_graph = g;
    return FK_OK;
}

fk_status fk_wait_pending(fk_handle h, double* gpu_seconds) {
    DispatcherState* ds;
    FK_TRY(get_dispatcher(h, &ds));
    std::lock_guard<std::mutex> lk(ds->mu);
    if (!ds->pending) {
        if (gpu_seconds) *gpu_seconds = 0.0;
        return FK_OK;
    }
    FK_HIP(hipEventSynchronize(ds->ev1));
    float ms = 0.f;
    FK_HIP(hipEventElapsedTime(&ms, ds->ev0, ds->ev1));
    if (gpu_seconds) *gpu_seconds = ms * 1e-3;
    ds->pending = false;
    Graph* g = ds->pending_graph;
    ds->pending_graph = nullptr;
    return g ? check_abort(g) : FK_OK;
}

fk_status fk_decode_chunk(fk_handle h, uint32_t graph_id, const fk_decode_uniforms* u, uint32_t start_offset,
                          uint32_t seed_token, uint32_t count, uint32_t* out_tokens, double* gpu_seconds) {
    DispatcherState* ds;
    FK_TRY(get_dispatcher(h, &ds));
    if (!u || !u->token || !u->step_counter || !u->hist_counter || !u->history)
        return set_error(FK_ERR_INVALID, "decode uniforms: null pointer");
    if (count == 0 || count > u->hist_capacity) return set_error(FK_ERR_INVALID, "decode chunk: count outside (0, history capacity]");
    if (!out_tokens) return set_error(FK_ERR_INVALID, "null out_tokens");
    std::lock_guard<std::mutex> lk(ds->mu);
    Graph* g;
    FK_TRY(get_graph(ds, graph_id, &g));
    if (ds->pending) return set_error(FK_ERR_INVALID, "an async graph launch is pending; call fk_wait_pending first");
    // host seeds the counters and the first token (lib.rs:1299-1303) ...
    const uint32_t zero = 0;
    FK_HIP(hipMemcpyAsync(u->step_counter, &start_offset, 4, hipMemcpyHostToDevice, ds->stream));
    FK_HIP(hipMemcpyAsync(u->hist_counter, &zero, 4, hipMemcpyHostToDevice, ds->stream));
    FK_HIP(hipMemcpyAsync(u->token, &seed_token, 4, hipMemcpyHostToDevice, ds->stream));
    FK_HIP(hipStreamSynchronize(ds->stream));
    // ... then replays the graph back to back and waits only for the last (lib.rs:1351-1392)
    FK_TRY(timed(ds, gpu_seconds, [&]() -> fk_status {
        for (uint32_t i = 0; i < count; ++i) FK_HIP(hipGraphLaunch(g->exec, ds->stream));
        return FK_OK;
    }));
    FK_TRY(check_abort(g));
    FK_HIP(hipMemcpy(out_tokens, u->history, (size_t)count * 4, hipMemcpyDeviceToHost));
    return FK_OK;
}

fk_status fk_decode_chunk_host_loop(fk_handle h, uint32_t graph_id, const fk_decode_uniforms* u,
                                    uint32_t start_offset, const uint32_t* tokens_in, uint32_t count,
                                    uint32_t* out_next, double* gpu_seconds) {
    DispatcherState* ds;
    FK_TRY(get_dispatcher(h, &ds));
    if (!u || !u->token || !u->step_counter || !u->hist_counter)
        return set_error(FK_ERR_INVALID, "decode uniforms: null pointer");
    if (!tokens_in || !out_next || count == 0) return set_error(FK_ERR_INVALID, "host loop: null tokens or zero count");
    std::lock_guard<std::mutex> lk(ds->mu);
    Graph* g;
    FK_TRY(get_graph(ds, graph_id, &g));
    if (ds->pending) return set_error(FK_ERR_INVALID, "an async graph launch is pending; call fk_wait_pending first");
    double total = 0.0;
    for (uint32_t i = 0; i < count; ++i) {
        const uint32_t off = start_offset + i, hist = 0;
        FK_HIP(hipMemcpyAsync(u->token, &tokens_in[i], 4, hipMemcpyHostToDevice, ds->stream));
        FK_HIP(hipMemcpyAsync(u->step_counter, &off, 4, hipMemcpyHostToDevice, ds->stream));
        FK_HIP(hipMemcpyAsync(u->hist_counter, &hist, 4, hipMemcpyHostToDevice, ds->stream));
        FK_HIP(hipStreamSynchronize(ds->stream));
        double t = 0.0;
        FK_TRY(timed(ds, &t, [&]() -> fk_status {
            FK_HIP(hipGraphLaunch(g->exec, ds->stream));
            return FK_OK;
        }));
        total += t;
        FK_TRY(check_abort(g));
        FK_HIP(hipMemcpy(&out_next[i], u->token, 4, hipMemcpyDeviceToHost));
    }
    if (gpu_seconds) *gpu_seconds = total;
    return FK_OK;
}

}  // extern "C"
