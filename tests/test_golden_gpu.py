"""The HIP kernels against the committed operator vectors (tests/golden/hot_path_vectors.npz),
through the C ABI.  Integer results (quantiser codes, argmax, cache addressing) must be equal;
bf16 results may differ from the stored ones only by a rounding-edge flip of one ulp on a small
fraction of elements (K = 128..192 here, so flips are rare)."""
import ctypes as C
import os

import numpy as np
import pytest

from helpers import bf16_mismatch

pytestmark = pytest.mark.gpu

V = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "hot_path_vectors.npz"))
HIDDEN, INTER, NQ, NKV = 128, 192, 96, 32


def _dev(fk, a):
    return fk.DeviceBuffer.from_numpy(np.ascontiguousarray(a))


def _w(fk, prefix, n, k, bits):
    if bits == 16:
        return fk.DeviceWeight(V[prefix + "_w"], None, None, n, k, 16, 0)
    return fk.DeviceWeight(V[prefix + "_w"], V[prefix + "_scales"], V[prefix + "_biases"], n, k, bits, 64)


def _close(got, want):
    frac, ulps = bf16_mismatch(got, want)
    assert frac <= 0.02 and ulps <= 1.0, (frac, ulps)


@pytest.mark.parametrize("bits", [4, 8])
def test_quantizer_vectors(fk, bits):
    w = V[f"quant{bits}_in"]
    n, k = w.shape
    packed, sc, bi = fk.DeviceBuffer(n * k * bits // 8), fk.DeviceBuffer(n * (k // 64) * 2), fk.DeviceBuffer(n * (k // 64) * 2)
    fk.check(fk.lib.fk_quantize_affine(C.c_void_p(_dev(fk, w).ptr), C.c_size_t(n), C.c_size_t(k), C.c_uint32(bits),
                                       C.c_uint32(64), C.c_void_p(packed.ptr), C.c_void_p(sc.ptr), C.c_void_p(bi.ptr), None))
    fk.sync()
    assert np.array_equal(packed.to_numpy(np.uint32, (n, k * bits // 32)), V[f"quant{bits}_w"])
    assert np.array_equal(sc.to_numpy(np.uint16, (n, k // 64)), V[f"quant{bits}_scales"])
    assert np.array_equal(bi.to_numpy(np.uint16, (n, k // 64)), V[f"quant{bits}_biases"])


@pytest.mark.parametrize("bits", [4, 8, 16])
def test_projection_vectors(fk, bits):
    t = f"b{bits}"
    x, gamma = _dev(fk, V["x"]), _dev(fk, V["gamma"])
    Wq, Wk, Wv = _w(fk, t + "_wq", NQ, HIDDEN, bits), _w(fk, t + "_wk", NKV, HIDDEN, bits), _w(fk, t + "_wv", NKV, HIDDEN, bits)
    Wg, Wu, Wd = _w(fk, t + "_wg", INTER, HIDDEN, bits), _w(fk, t + "_wu", INTER, HIDDEN, bits), _w(fk, t + "_wd", HIDDEN, INTER, bits)
    y = fk.DeviceBuffer(INTER * 2)
    fk.qgemv(Wg, x, None, y)
    _close(y.to_numpy(np.uint16), V[t + "_qgemv"])
    q, k, v = fk.DeviceBuffer(NQ * 2), fk.DeviceBuffer(NKV * 2), fk.DeviceBuffer(NKV * 2)
    fk.rmsnorm_qkv(x, gamma, 1e-6, Wq, Wk, Wv, _dev(fk, V[t + "_bq"]), _dev(fk, V[t + "_bk"]), _dev(fk, V[t + "_bv"]), q, k, v)
    for buf, key in ((q, "_q"), (k, "_k"), (v, "_v")):
        _close(buf.to_numpy(np.uint16), V[t + key])
    mid = fk.DeviceBuffer(INTER * 2)
    for variant in (0, 2, 1):   # variant 1 last: it feeds the down projection below
        fk.gateup_swiglu(x, gamma, 1e-6, Wg, Wu, variant, mid)
        _close(mid.to_numpy(np.uint16), V[f"{t}_swiglu{variant}"])
    mid = _dev(fk, V[t + "_swiglu1"])   # the stored activations, so one flip upstream cannot spread
    out = fk.DeviceBuffer(HIDDEN * 2)
    fk.linear_residual(Wd, mid, _dev(fk, V["res"]), None, out)
    _close(out.to_numpy(np.uint16), V[t + "_down"])
    fk.linear_residual(Wd, mid, _dev(fk, V["res"]), _dev(fk, V["res2"]), out)
    _close(out.to_numpy(np.uint16), V[t + "_down2"])
    logits = fk.DeviceBuffer(INTER * 2)
    fk.final_rmsnorm_lm_head(x, gamma, 1e-6, Wg, logits)
    _close(logits.to_numpy(np.uint16), V[t + "_lm_head"])
    row = fk.DeviceBuffer(INTER * 2)
    fk.embed_lookup_decode(Wd, None, 5, 1.0, row)
    assert np.array_equal(row.to_numpy(np.uint16), V[t + "_embed_row5"])


def test_rope_and_cache_vectors(fk):
    n_heads, n_kv, dim, cap = 4, 2, 64, 16
    for pos in (0, 7, 4097):
        q = _dev(fk, V["rope_q_in"])
        fk.rope_q_decode(q, None, n_heads, dim, dim, 1e6, offset=pos)
        _close(q.to_numpy(np.uint16), V[f"rope_q_pos{pos}"])
    ck, cv = fk.zeros(n_kv * cap * dim * 2), fk.zeros(n_kv * cap * dim * 2)
    fk.rope_kv_cache_store_decode(_dev(fk, V["rope_k_in"]), _dev(fk, V["rope_v_in"]), None, n_kv, dim, dim, dim, 1e6, 0.0,
                                  None, 21, None, 21, cap, ck, cv)
    got_k, want_k = ck.to_numpy(np.uint16), V["rope_cache_k"]
    assert np.array_equal(got_k == 0, want_k == 0)            # same rows written (row 21 % 16 = 5), nothing else touched
    _close(got_k, want_k)
    assert np.array_equal(cv.to_numpy(np.uint16), V["rope_cache_v"])
    q = _dev(fk, V["rope_q_in"])
    fk.rope_q_decode(q, _dev(fk, V["headnorm_w"]), n_heads, dim, 32, 1e4, eps=1e-6, offset=9)
    _close(q.to_numpy(np.uint16), V["headnorm_rope_q"])


def test_attention_and_argmax_vectors(fk):
    n_heads, n_kv, dim = 4, 2, 64
    out = fk.DeviceBuffer(n_heads * dim * 2)
    pb, cb = fk.sdpa_workspace_bytes(n_heads, n_kv, dim, dim, 64)
    fk.sdpa_decode(_dev(fk, V["sdpa_q"]), _dev(fk, V["sdpa_k"]), _dev(fk, V["sdpa_v"]), out, None, 37, 64, n_heads, n_kv,
                   dim, dim, 64, 0.125, fk.DeviceBuffer(max(pb, 16)), fk.zeros(max(cb, 16)))
    got, want = out.to_numpy(np.uint16), V["sdpa_out"]
    frac, ulps = bf16_mismatch(got, want)
    assert frac <= 0.05 and ulps <= 2.0, (frac, ulps)   # fp32 softmax in a different order: a few 1-ulp flips
    tok = fk.zeros(4)
    fk.argmax_logits_decode(_dev(fk, V["argmax_logits"]), 1000, tok, None, None, 0, fk.zeros(fk.ARGMAX_WORKSPACE_BYTES))
    assert int(tok.to_numpy(np.uint32)[0]) == int(V["argmax_out"][0]) == 17


def test_moe_and_multirow_vectors(fk):
    E, top_k = 4, 3

    def stacked(prefix, n, k):
        return fk.DeviceWeight(V[prefix + "_w"], V[prefix + "_scales"], V[prefix + "_biases"], n, k, 4, 64)
    Sg, Su, Sd = stacked("moe_wg", INTER, HIDDEN), stacked("moe_wu", INTER, HIDDEN), stacked("moe_wd", HIDDEN, INTER)
    eidx = _dev(fk, V["moe_expert_idx"])
    h = fk.DeviceBuffer(top_k * INTER * 2)
    fk.routed_qmv_swiglu(_dev(fk, V["x"]), 1, Sg, Su, E, _dev(fk, np.zeros(top_k, np.uint32)), eidx, None, top_k, h)
    _close(h.to_numpy(np.uint16), V["moe_h"].ravel())
    out = fk.DeviceBuffer(HIDDEN * 2)
    ws = fk.DeviceBuffer(fk.routed_reduce_workspace_bytes(1, top_k, HIDDEN))
    fk.routed_qmv_reduce(_dev(fk, V["moe_h"]), top_k, Sd, E, None, eidx, _dev(fk, V["moe_route_weight"]), None, None,
                         _dev(fk, V["res"]), 1, top_k, out, ws)
    _close(out.to_numpy(np.uint16), V["moe_out"].ravel())
    W = _w(fk, "b4_wg", INTER, HIDDEN, 4)
    y = fk.DeviceBuffer(5 * INTER * 2)
    fk.qgemm(W, _dev(fk, V["qgemm_x"]), 5, None, None, y, fk.DeviceBuffer(fk.qgemm_workspace_bytes(5, INTER, HIDDEN)))
    _close(y.to_numpy(np.uint16), V["qgemm_out"].ravel())
