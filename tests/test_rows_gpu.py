"""Several active token rows per launch (multi-token verification / chunked prefill): the row forms
of RMSNorm, embedding, RoPE + KV store and causal attention against the oracle applied row by row,
and the batched prompt path of the decoder against its token-by-token path."""
import numpy as np
import pytest

import oracle
from helpers import OracleDecoder, bf16_mismatch, make_qweight, normal_bf16, rel_l2, rng, to_device

pytestmark = pytest.mark.gpu


def _dev(fk, a):
    return None if a is None else fk.DeviceBuffer.from_numpy(np.ascontiguousarray(a))


def _close(got, want, frac_bar=0.02, ulp_bar=1.0):
    frac, ulps = bf16_mismatch(got, want)
    assert frac <= frac_bar and ulps <= ulp_bar, (frac, ulps)


def test_rmsnorm_and_embed_rows(fk):
    rows, hidden = 7, 896
    x, w = normal_bf16(1, (rows, hidden)), normal_bf16(2, hidden, 0.1, 1.0)
    y = fk.DeviceBuffer(rows * hidden * 2)
    fk.rmsnorm_rows(_dev(fk, x), _dev(fk, w), 1e-6, rows, hidden, y)
    got = y.to_numpy(np.uint16, (rows, hidden))
    for r in range(rows):
        _close(got[r], oracle.rmsnorm(x[r], w, 1e-6))
    for bits in (16, 4):
        E = make_qweight(3, 500, 256, bits)
        toks = np.array([0, 499, 17, 17, 250], np.uint32)
        out = fk.DeviceBuffer(toks.size * 256 * 2)
        fk.embed_lookup_rows(to_device(fk, E), _dev(fk, toks), toks.size, 1.0, out)
        got = out.to_numpy(np.uint16, (toks.size, 256))
        for r, t in enumerate(toks):
            assert np.array_equal(got[r], oracle.embed_lookup(E, int(t)))


@pytest.mark.parametrize("rows,n_heads,n_kv,dim", [(6, 8, 2, 64), (12, 8, 2, 64), (21, 6, 3, 128), (9, 5, 1, 128)])
@pytest.mark.parametrize("norm", [False, True])
def test_rope_store_rows(fk, norm, rows, n_heads, n_kv, dim):
    cap, off = 32, 29     # the rows wrap around the cache
    q, k, v = normal_bf16(4, (rows, n_heads * dim)), normal_bf16(5, (rows, n_kv * dim)), normal_bf16(6, (rows, n_kv * dim))
    qn, kn = (normal_bf16(7, dim, 0.1, 1.0), normal_bf16(8, dim, 0.1, 1.0)) if norm else (None, None)
    dq, ck, cv = _dev(fk, q), fk.zeros(n_kv * cap * dim * 2), fk.zeros(n_kv * cap * dim * 2)
    fk.qkv_rope_store_rows(dq, _dev(fk, k), _dev(fk, v), _dev(fk, qn), _dev(fk, kn), n_heads, n_kv, dim, dim, 1e4, 1e-6,
                           rows, off, cap, ck, cv)
    got_q = dq.to_numpy(np.uint16, (rows, n_heads * dim))
    rk, rv = np.zeros(n_kv * cap * dim, np.uint16), np.zeros(n_kv * cap * dim, np.uint16)
    for r in range(rows):
        pos = off + r
        want_q = oracle.headnorm_rope(q[r], qn, n_heads, dim, dim, 1e-6, 1e4, pos) if norm else oracle.rope_q(q[r], n_heads, dim, dim, 1e4, pos)
        _close(got_q[r], want_q, ulp_bar=2.0)
        kr = oracle.headnorm_rope(k[r], kn, n_kv, dim, 0, 1e-6, 1e4, pos) if norm else k[r]   # norm only, rotation below
        oracle.rope_kv_store(kr, v[r], n_kv, dim, dim, 1e4, pos, pos, cap, rk, rv)
    assert np.array_equal(cv.to_numpy(np.uint16), rv)
    gk = ck.to_numpy(np.uint16)
    assert np.array_equal(gk == 0, rk == 0)
    _close(gk, rk, ulp_bar=2.0)
    # with the rotary table of the pass (filled once, reused by every layer): the same bits
    tab = fk.DeviceBuffer(rows * dim * 4)
    fk.rope_table_rows(tab, dim, 1e4, off, rows)
    dq2, ck2, cv2 = _dev(fk, q), fk.zeros(n_kv * cap * dim * 2), fk.zeros(n_kv * cap * dim * 2)
    fk.qkv_rope_store_rows(dq2, _dev(fk, k), _dev(fk, v), _dev(fk, qn), _dev(fk, kn), n_heads, n_kv, dim, dim, 1e4, 1e-6,
                           rows, off, cap, ck2, cv2, rope_tab=tab)
    q2, k2 = dq2.to_numpy(np.uint16, (rows, n_heads * dim)), ck2.to_numpy(np.uint16)
    if rows < 8:      # the same kernel with and without the table: the same bits
        assert np.array_equal(q2, got_q) and np.array_equal(k2, gk)
    else:             # from 8 rows the table selects the 16-bytes-per-lane form (other summation order in the norm)
        for r in range(rows):
            pos = off + r
            want_q = oracle.headnorm_rope(q[r], qn, n_heads, dim, dim, 1e-6, 1e4, pos) if norm else oracle.rope_q(q[r], n_heads, dim, dim, 1e4, pos)
            _close(q2[r], want_q, ulp_bar=2.0)
        assert np.array_equal(k2 == 0, rk == 0)
        _close(k2, rk, ulp_bar=2.0)
    assert np.array_equal(cv2.to_numpy(np.uint16), rv)
    t = tab.to_numpy(np.float32, (rows, dim // 2, 2)).astype(np.float64)
    ang = (off + np.arange(rows))[:, None] * (1e4 ** (-np.arange(dim // 2) / (dim // 2)))[None, :]
    assert np.allclose(t[..., 0], np.cos(ang), atol=2e-5) and np.allclose(t[..., 1], np.sin(ang), atol=2e-5)   # fp32 angles


@pytest.mark.parametrize("kv_len,rows", [(1, 5), (60, 8), (500, 32)])
def test_sdpa_rows_are_causal_single_row_calls(fk, kv_len, rows):
    n_heads, n_kv, dim, cap = 32, 8, 128, 1024
    q = normal_bf16(9, (rows, n_heads * dim))
    ck, cv = normal_bf16(10, n_kv * cap * dim), normal_bf16(11, n_kv * cap * dim)
    dck, dcv = _dev(fk, ck), _dev(fk, cv)
    pb, cb = fk.sdpa_workspace_bytes(n_heads, n_kv, dim, dim, kv_len + rows - 1)
    out = fk.DeviceBuffer(rows * n_heads * dim * 2)
    scale = 1.0 / np.sqrt(dim)
    fk.sdpa_decode_rows(_dev(fk, q), dck, dcv, out, rows, kv_len, n_heads, n_kv, dim, dim, cap, scale,
                        fk.DeviceBuffer(max(pb, 16) * rows), fk.zeros(max(cb, 16) * rows))
    got = out.to_numpy(np.uint16, (rows, n_heads * dim))
    one = fk.DeviceBuffer(n_heads * dim * 2)
    part, cnt = fk.DeviceBuffer(max(pb, 16)), fk.zeros(max(cb, 16))
    for r in range(rows):
        fk.sdpa_decode(_dev(fk, q[r]), dck, dcv, one, None, kv_len + r, kv_len + rows - 1, n_heads, n_kv, dim, dim, cap,
                       scale, part, cnt)
        # same kernel; with several rows the planner needs fewer key ranges per row to fill the chip, so the partial
        # softmaxes are cut differently: equal up to the last bit of a few outputs
        single = one.to_numpy(np.uint16)
        frac, ulps = bf16_mismatch(got[r], single)
        assert frac <= 0.05 and rel_l2(got[r], oracle.bf16_to_f32(single)) <= 2e-3, (r, frac, ulps)
        ref = oracle.sdpa_decode(q[r], ck, cv, n_heads, n_kv, dim, dim, kv_len + r, cap, scale)
        assert rel_l2(got[r], oracle.bf16_to_f32(ref)) <= 1e-2


@pytest.mark.parametrize("bits,prompt_len,rows_per_pass", [(4, 45, 128), (8, 7, 128), (4, 300, 256), (4, 333, 100), (16, 45, 128),
                                                          (16, 300, 4096)])
def test_batched_prefill_matches_token_by_token(fk, bits, prompt_len, rows_per_pass):
    """prefill_rows (32 tokens per weight pass on the matrix cores) leaves the caches of the
    token-by-token path and continues with the same tokens.  The two paths sum in different
    orders, so the caches agree to rounding flips and the greedy continuation is compared with
    the oracle's margins in view."""
    from fusekit_amd.decoder import DecoderConfig, DecoderRuntime, DecoderWeights
    cfg = DecoderConfig(n_layers=3, hidden=256, n_heads=4, n_kv=2, head_dim=64, inter=512, vocab=2000, capacity=512,
                        bits=bits, qk_norm=True, qkv_bias=(bits == 8), swiglu_variant=2)
    W = DecoderWeights.random_init(cfg, seed=41)
    prompt = rng(42).integers(0, cfg.vocab, prompt_len).tolist()
    a, b = DecoderRuntime(cfg, W), DecoderRuntime(cfg, W)
    first_a = a.prefill(prompt)
    first_b = b.prefill_rows(prompt, rows_per_pass=rows_per_pass)
    for l in range(cfg.n_layers):
        for ca, cb_ in ((a.cache_k[l], b.cache_k[l]), (a.cache_v[l], b.cache_v[l])):
            ga, gb = ca.to_numpy(np.uint16), cb_.to_numpy(np.uint16)
            assert np.array_equal(ga == 0, gb == 0)
            assert rel_l2(gb, oracle.bf16_to_f32(ga)) <= 1e-2, l
    ref, margins = OracleDecoder(cfg, W).generate(prompt, 9)
    assert first_a == ref[0]
    if margins[0] > 0.05:
        assert first_b == ref[0]
    if first_b == first_a:
        ta, _ = a.d.decode_chunk(a.graph, a.uniforms, prompt_len, first_a, 8)
        tb, _ = b.d.decode_chunk(b.graph, b.uniforms, prompt_len, first_b, 8)
        clear = next((i for i, m in enumerate(margins[1:]) if m <= 0.05), 8)
        assert ta[:clear] == tb[:clear] == ref[1:1 + clear]


@pytest.mark.parametrize("bits", [4, 8])
def test_prefill_with_resident_bf16_weights_is_bit_identical(fk, bits):
    """keep_bf16_weights: passes of at least 256 rows multiply with a resident bf16 copy of every projection
    (fk_dequantize_bf16) instead of dequantising in every pass: the caches and logits of the dequantise + library route
    (taken here from 256 rows, as the copy is; by default only from 1024), bit for bit; and the copy itself is
    T(code * scale + bias) of the oracle."""
    from fusekit_amd.decoder import DecoderConfig, DecoderRuntime, DecoderWeights
    cfg = DecoderConfig(n_layers=2, hidden=256, n_heads=4, n_kv=2, head_dim=64, inter=512, vocab=2000, capacity=1024,
                        bits=bits, qk_norm=True, swiglu_variant=1)
    W = DecoderWeights.random_init(cfg, seed=43)
    prompt = rng(44).integers(0, cfg.vocab, 600).tolist()
    a, b = DecoderRuntime(cfg, W), DecoderRuntime(cfg, W)
    fk.set_gemm_library_rows(256)
    try:
        ta = a.prefill_rows(prompt, rows_per_pass=512)
        tb = b.prefill_rows(prompt, rows_per_pass=512, keep_bf16_weights=True)
    finally:
        fk.set_gemm_library_rows(fk.GEMM_LIBRARY_ROWS_DEFAULT)
    assert len(b._bf16_weights) == 7 * cfg.n_layers and not a._bf16_weights
    assert ta == tb and np.array_equal(a.logits.to_numpy(np.uint16), b.logits.to_numpy(np.uint16))
    for l in range(cfg.n_layers):
        assert np.array_equal(a.cache_k[l].to_numpy(np.uint16), b.cache_k[l].to_numpy(np.uint16))
        assert np.array_equal(a.cache_v[l].to_numpy(np.uint16), b.cache_v[l].to_numpy(np.uint16))
    name = "layers.1.mlp.down_proj"
    from helpers import host_weight
    want = oracle.f32_to_bf16(oracle.dequantize(host_weight(W.mats[name])))
    assert np.array_equal(b._bf16_weights[name].w.to_numpy(np.uint16, want.shape), want)
