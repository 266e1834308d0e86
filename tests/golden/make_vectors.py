#!/usr/bin/env python3
"""Writes tests/golden/hot_path_vectors.npz: small input / expected-output vectors for every
operator of the decode hot path.

Origin of the expected outputs: the CPU oracle (oracle/fk_oracle.c) at the commit that wrote the
file -- the reference (Rust -> Metal + MLX) can neither be built nor imported here and holds no
golden vectors of its own for this path, so these fixtures pin the ORACLE (any later change of
its arithmetic shows up as a diff against the committed file) and give the GPU tests fixed
cases that do not depend on the oracle being built.  The hand-derived known answers that pin
the oracle itself live in known_answers.json next to this script.

    python tests/golden/make_vectors.py        # rewrites the .npz (deterministic)
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
sys.path.insert(0, os.path.dirname(HERE))

import oracle  # noqa: E402
from helpers import make_qweight, normal_bf16, rng  # noqa: E402


def weight_arrays(prefix, W, out):
    out[prefix + "_w"] = W.w
    if W.scales is not None:
        out[prefix + "_scales"], out[prefix + "_biases"] = W.scales, W.biases


def build():
    v = {}
    # Q0 quantiser + unpack (bit-exact)
    for bits in (4, 8):
        w = (rng(1).standard_normal((6, 128), dtype=np.float32) * 0.05).astype(np.float32)
        w[0, :64] = 0.25            # constant group
        w[1, :64] = np.linspace(-1, 0.5, 64, dtype=np.float32)
        Q = oracle.quantize(w, bits, 64)
        v[f"quant{bits}_in"] = w
        weight_arrays(f"quant{bits}", Q, v)
        v[f"quant{bits}_codes"] = oracle.unpack_codes(Q)
    # K1 / K1r / N / K2 / K3a / H on one small set of matrices per storage kind
    hidden, inter, nq, nkv = 128, 192, 96, 32
    x = normal_bf16(2, hidden)
    gamma = normal_bf16(3, hidden, 0.1, 1.0)
    v["x"], v["gamma"] = x, gamma
    v["rmsnorm_out"] = oracle.rmsnorm(x, gamma, 1e-6)
    for bits in (4, 8, 16):
        t = f"b{bits}"
        Wq, Wk, Wv = make_qweight(10, nq, hidden, bits), make_qweight(11, nkv, hidden, bits), make_qweight(12, nkv, hidden, bits)
        Wg, Wu, Wd = make_qweight(13, inter, hidden, bits), make_qweight(14, inter, hidden, bits), make_qweight(15, hidden, inter, bits)
        for nm, W in (("wq", Wq), ("wk", Wk), ("wv", Wv), ("wg", Wg), ("wu", Wu), ("wd", Wd)):
            weight_arrays(f"{t}_{nm}", W, v)
        bq, bk, bv = normal_bf16(16, nq), normal_bf16(17, nkv), normal_bf16(18, nkv)
        v[f"{t}_bq"], v[f"{t}_bk"], v[f"{t}_bv"] = bq, bk, bv
        v[f"{t}_qgemv"] = oracle.qgemv(Wg, x)
        q, k, vv = oracle.rmsnorm_qkv(x, gamma, 1e-6, Wq, Wk, Wv, bq, bk, bv)
        v[f"{t}_q"], v[f"{t}_k"], v[f"{t}_v"] = q, k, vv
        for variant in (0, 1, 2):
            v[f"{t}_swiglu{variant}"] = oracle.gateup_swiglu(x, gamma, 1e-6, Wg, Wu, variant)
        mid = oracle.gateup_swiglu(x, gamma, 1e-6, Wg, Wu, 1)
        res, res2 = normal_bf16(19, hidden), normal_bf16(20, hidden)
        v["res"], v["res2"] = res, res2
        v[f"{t}_down"] = oracle.linear_residual(Wd, mid, res, None)
        v[f"{t}_down2"] = oracle.linear_residual(Wd, mid, res, res2)
        v[f"{t}_lm_head"] = oracle.final_rmsnorm_lm_head(x, gamma, 1e-6, Wg)
        v[f"{t}_embed_row5"] = oracle.embed_lookup(Wd, 5, 1.0)
    # R: rope / kv store
    n_heads, n_kv, dim, cap = 4, 2, 64, 16
    qh, kh, vh = normal_bf16(21, n_heads * dim), normal_bf16(22, n_kv * dim), normal_bf16(23, n_kv * dim)
    v["rope_q_in"], v["rope_k_in"], v["rope_v_in"] = qh, kh, vh
    for pos in (0, 7, 4097):
        v[f"rope_q_pos{pos}"] = oracle.rope_q(qh, n_heads, dim, dim, 1e6, pos)
    ck, cv = np.zeros(n_kv * cap * dim, np.uint16), np.zeros(n_kv * cap * dim, np.uint16)
    oracle.rope_kv_store(kh, vh, n_kv, dim, dim, 1e6, 21, 21, cap, ck, cv)   # row 21 % 16 = 5
    v["rope_cache_k"], v["rope_cache_v"] = ck, cv
    v["headnorm_rope_q"] = oracle.headnorm_rope(qh, normal_bf16(24, dim, 0.1, 1.0), n_heads, dim, 32, 1e-6, 1e4, 9)
    v["headnorm_w"] = normal_bf16(24, dim, 0.1, 1.0)
    # K4: attention
    kv_len = 37
    q = normal_bf16(25, n_heads * dim)
    ck, cv = normal_bf16(26, n_kv * 64 * dim), normal_bf16(27, n_kv * 64 * dim)
    v["sdpa_q"], v["sdpa_k"], v["sdpa_v"] = q, ck, cv
    v["sdpa_out"] = oracle.sdpa_decode(q, ck, cv, n_heads, n_kv, dim, dim, kv_len, 64, 0.125)
    # A: argmax (ties -> lowest index, NaN never wins)
    logits = normal_bf16(28, 1000)
    logits[[17, 503]] = 0x4120      # 10.0 twice
    logits[3] = 0x7FC0              # NaN
    v["argmax_logits"] = logits
    v["argmax_out"] = np.array([oracle.argmax(logits)], np.uint32)
    # M1 / M2: routed experts
    E, top_k = 4, 3
    Sg = oracle.StackedWeight([make_qweight(30 + e, inter, hidden, 4) for e in range(E)])
    Su = oracle.StackedWeight([make_qweight(40 + e, inter, hidden, 4) for e in range(E)])
    Sd = oracle.StackedWeight([make_qweight(50 + e, hidden, inter, 4) for e in range(E)])
    for nm, W in (("moe_wg", Sg), ("moe_wu", Su), ("moe_wd", Sd)):
        weight_arrays(nm, W, v)
    eidx, rw = np.array([2, 0, 3], np.uint32), normal_bf16(29, top_k, 0.2, 0.3)
    v["moe_expert_idx"], v["moe_route_weight"] = eidx, rw
    h = oracle.routed_qmv_swiglu(x.reshape(1, -1), Sg, Su, np.zeros(top_k, np.uint32), eidx, None)
    v["moe_h"] = h
    v["moe_out"] = oracle.routed_qmv_reduce(h, Sd, eidx, rw, res.reshape(1, -1), 1, top_k)
    # G: multi-row matmul
    xm = normal_bf16(31, (5, hidden))
    v["qgemm_x"] = xm
    v["qgemm_out"] = oracle.qgemm(make_qweight(13, inter, hidden, 4), xm)
    return v


if __name__ == "__main__":
    vec = build()
    path = os.path.join(HERE, "hot_path_vectors.npz")
    np.savez_compressed(path, **vec)
    print(f"wrote {path}: {len(vec)} arrays, {os.path.getsize(path)} bytes")
