"""Quantised KV cache (kv_bits 4 / 8) through the C-ABI: the store (RoPE + optional head norm in
fp32, per-group affine quantisation) and attention over the packed cache, against the oracle."""
import numpy as np
import pytest

import oracle
from helpers import normal_bf16, rel_l2, rng

pytestmark = pytest.mark.gpu


def _dev(fk, a):
    return None if a is None else fk.DeviceBuffer.from_numpy(np.ascontiguousarray(a))


def _caches(fk, n_kv, cap, dim, bits, group):
    return fk.QuantKvCache(n_kv, cap, dim, bits, group), fk.QuantKvCache(n_kv, cap, dim, bits, group)


def _host(c, oc):
    """Device cache -> the oracle's container."""
    oc.packed[:] = c.packed.to_numpy(np.uint32, oc.packed.shape)
    oc.scales[:] = c.scales.to_numpy(np.uint16, oc.scales.shape)
    oc.biases[:] = c.biases.to_numpy(np.uint16, oc.biases.shape)
    return oc


def _upload(fk, oc, c):
    c.packed.upload(np.ascontiguousarray(oc.packed))
    c.scales.upload(np.ascontiguousarray(oc.scales))
    c.biases.upload(np.ascontiguousarray(oc.biases))


@pytest.mark.parametrize("bits,group,dim", [(4, 64, 128), (8, 64, 128), (4, 32, 64), (8, 128, 256)])
def test_store_without_rotation_is_bit_exact(fk, bits, group, dim):
    """No rotation, no norm: K and V are bf16 values quantised by integer-exact arithmetic, so the
    packed codes, scales and biases equal the oracle's bit for bit; rows wrap around the cache and
    nothing else is written."""
    rows, n_kv, cap, off = 5, 3, 8, 6                               # rows 6,7,0,1,2
    k, v = normal_bf16(1, (rows, n_kv * dim)), normal_bf16(2, (rows, n_kv * dim))
    K, V = _caches(fk, n_kv, cap, dim, bits, group)
    fk.kv_cache_store_quant(_dev(fk, k), _dev(fk, v), None, n_kv, dim, 0, 1e4, 0.0, None, off, rows, K, V)
    oK, oV = oracle.QuantCache(n_kv, cap, dim, bits, group), oracle.QuantCache(n_kv, cap, dim, bits, group)
    for r in range(rows):
        oracle.rope_kv_store_quant(k[r], v[r], None, n_kv, dim, 0, 1e4, 0.0, off + r, off + r, oK, oV)
    gK = _host(K, oracle.QuantCache(n_kv, cap, dim, bits, group))
    gV = _host(V, oracle.QuantCache(n_kv, cap, dim, bits, group))
    for g, o in ((gK, oK), (gV, oV)):
        assert np.array_equal(g.packed, o.packed) and np.array_equal(g.scales, o.scales)
        assert np.array_equal(g.biases, o.biases)
    assert not gK.packed[:, 3:6].any() and not gV.scales[:, 3:6].any()


@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("norm", [False, True])
def test_store_with_rotation(fk, bits, norm):
    """With RoPE the value quantised is an fp32 product of sin / cos: V stays bit-exact; K's scale and
    bias may differ from the oracle's in the last bf16 place and a code by one where the value sits on
    a rounding boundary, so the dequantised rows are compared (a fraction of a quantisation step)."""
    rows, n_kv, dim, cap, group = 4, 2, 128, 64, 64
    k, v = normal_bf16(3, (rows, n_kv * dim)), normal_bf16(4, (rows, n_kv * dim))
    kn = normal_bf16(5, dim, 0.1, 1.0) if norm else None
    off = np.array([37], np.uint32)
    K, V = _caches(fk, n_kv, cap, dim, bits, group)
    fk.kv_cache_store_quant(_dev(fk, k), _dev(fk, v), _dev(fk, kn), n_kv, dim, dim, 1e6, 1e-6, _dev(fk, off), 0, rows, K, V)
    oK, oV = oracle.QuantCache(n_kv, cap, dim, bits, group), oracle.QuantCache(n_kv, cap, dim, bits, group)
    for r in range(rows):
        oracle.rope_kv_store_quant(k[r], v[r], kn, n_kv, dim, dim, 1e6, 1e-6, 37 + r, 37 + r, oK, oV)
    gK = _host(K, oracle.QuantCache(n_kv, cap, dim, bits, group))
    gV = _host(V, oracle.QuantCache(n_kv, cap, dim, bits, group))
    assert np.array_equal(gV.packed, oV.packed) and np.array_equal(gV.scales, oV.scales) and np.array_equal(gV.biases, oV.biases)
    written = slice(37, 37 + rows)
    got, want = gK.dequantize()[:, written], oK.dequantize()[:, written]
    step = np.abs(oracle.bf16_to_f32(oK.scales[:, written])).repeat(group, axis=-1)
    err = np.abs(got - want)
    assert np.all(err <= 1.01 * step + 2.0 ** -7 * np.abs(want)), float((err / step).max())
    assert np.mean(err > 0.26 * step) <= 0.02                       # nearly every element: identical code, scale within an ulp
    assert np.mean(gK.packed[:, written] != oK.packed[:, written]) <= 0.05
    assert not gK.packed[:, :37].any() and not gK.packed[:, 37 + rows:].any()


@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("n_heads,n_kv,dim,group,kv_len,cap", [
    (8, 2, 128, 64, 1, 64),
    (8, 2, 128, 64, 77, 128),
    (32, 8, 128, 64, 700, 1024),
    (4, 4, 64, 32, 300, 512),
    (16, 2, 256, 128, 130, 256),
    (14, 2, 64, 64, 4500, 8192),
])
def test_attention_over_quantised_cache(fk, bits, n_heads, n_kv, dim, group, kv_len, cap):
    rs = rng(bits * 1000 + kv_len)
    oK, oV = oracle.QuantCache(n_kv, cap, dim, bits, group), oracle.QuantCache(n_kv, cap, dim, bits, group)
    for c in (oK, oV):
        c.packed[:] = rs.integers(0, 2 ** 32, c.packed.shape, dtype=np.uint32)
        c.scales[:] = oracle.f32_to_bf16((rs.standard_normal(c.scales.shape) * 0.02 + (0.1 if bits == 4 else 0.008)).astype(np.float32))
        c.biases[:] = oracle.f32_to_bf16((rs.standard_normal(c.biases.shape) * 0.3 - (0.7 if bits == 4 else 1.0)).astype(np.float32))
    q = normal_bf16(9, n_heads * dim)
    scale = dim ** -0.5
    K, V = _caches(fk, n_kv, cap, dim, bits, group)
    _upload(fk, oK, K), _upload(fk, oV, V)
    out = fk.DeviceBuffer(n_heads * dim * 2)
    pb, cb = fk.sdpa_workspace_bytes(n_heads, n_kv, dim, dim, cap)
    ws, counters = fk.DeviceBuffer(max(256, pb)), fk.zeros(max(256, cb))
    want = oracle.sdpa_decode_quant(q, oK, oV, n_heads, kv_len, scale)
    for d_len in (None, _dev(fk, np.array([kv_len], np.uint32))):     # immediate and device-resident length
        fk.fill_u32(out, 0, n_heads * dim // 2)
        fk.sdpa_decode_quant(_dev(fk, q), K, V, out, d_len, kv_len, cap, 1, n_heads, scale, ws, counters)
        got = out.to_numpy(np.uint16)
        assert rel_l2(got, oracle.bf16_to_f32(want)) <= 1e-2, rel_l2(got, oracle.bf16_to_f32(want))
        assert np.max(np.abs(oracle.bf16_to_f32(got) - oracle.bf16_to_f32(want))) <= 2.0 ** -6 * np.max(np.abs(oracle.bf16_to_f32(want)))


@pytest.mark.parametrize("bits,group,dim", [(4, 64, 128), (8, 64, 128), (4, 32, 64)])
def test_dequantised_prefix_and_prefill_attention(fk, bits, group, dim):
    """fk_kv_cache_dequant gives T(code * scale + bias) bit for bit (rows past the prefix untouched), and the
    matrix-core prefill attention over it agrees with the quantised-cache oracle row by row."""
    n_heads, n_kv, cap, rows, kv_len = 8, 2, 96, 40, 70
    rs = rng(17)
    oK, oV = oracle.QuantCache(n_kv, cap, dim, bits, group), oracle.QuantCache(n_kv, cap, dim, bits, group)
    for c in (oK, oV):
        c.packed[:] = rs.integers(0, 2 ** 32, c.packed.shape, dtype=np.uint32)
        c.scales[:] = oracle.f32_to_bf16((rs.standard_normal(c.scales.shape) * 0.02 + (0.1 if bits == 4 else 0.008)).astype(np.float32))
        c.biases[:] = oracle.f32_to_bf16((rs.standard_normal(c.biases.shape) * 0.3 - (0.7 if bits == 4 else 1.0)).astype(np.float32))
    K, V = _caches(fk, n_kv, cap, dim, bits, group)
    _upload(fk, oK, K), _upload(fk, oV, V)
    kdq, vdq = fk.zeros(n_kv * cap * dim * 2), fk.zeros(n_kv * cap * dim * 2)
    fk.kv_cache_dequant(K, kv_len, kdq, cap)
    fk.kv_cache_dequant(V, kv_len, vdq, cap)
    got_k = kdq.to_numpy(np.uint16).reshape(n_kv, cap, dim)
    want_k = oracle.f32_to_bf16(oK.dequantize().astype(np.float32)).reshape(n_kv, cap, dim)
    assert np.array_equal(got_k[:, :kv_len], want_k[:, :kv_len]) and not got_k[:, kv_len:].any()
    q = normal_bf16(19, (rows, n_heads * dim))
    out = fk.DeviceBuffer(rows * n_heads * dim * 2)
    scale = dim ** -0.5
    fk.sdpa_prefill(_dev(fk, q), kdq, vdq, out, rows, kv_len, n_heads, n_kv, dim, cap, scale)
    got = out.to_numpy(np.uint16).reshape(rows, n_heads * dim)
    for r in range(rows):
        want = oracle.sdpa_decode_quant(q[r], oK, oV, n_heads, kv_len - rows + r + 1, scale)
        assert rel_l2(got[r], oracle.bf16_to_f32(want)) <= 1e-2, r
    with pytest.raises(fk.FusekitError):
        fk.kv_cache_dequant(K, cap + 1, kdq, cap)


def test_store_then_attend_matches_bf16_cache(fk):
    """Round trip at 8 bits: rows stored quantised and attended give the plain bf16-cache attention to
    within the quantisation noise (a size-independent property: no oracle involved)."""
    n_heads, n_kv, dim, cap, rows = 16, 4, 128, 256, 200
    k, v = normal_bf16(11, (rows, n_kv * dim)), normal_bf16(12, (rows, n_kv * dim))
    q = normal_bf16(13, (rows, n_heads * dim))
    K, V = _caches(fk, n_kv, cap, dim, 8, 64)
    fk.kv_cache_store_quant(_dev(fk, k), _dev(fk, v), None, n_kv, dim, dim, 1e4, 0.0, None, 0, rows, K, V)
    dq, ck, cv = _dev(fk, q[-1:].copy()), fk.zeros(n_kv * cap * dim * 2), fk.zeros(n_kv * cap * dim * 2)
    dummy_q = _dev(fk, np.zeros((rows, n_heads * dim), np.uint16))
    fk.qkv_rope_store_rows(dummy_q, _dev(fk, k), _dev(fk, v), None, None, n_heads, n_kv, dim, dim, 1e4, 0.0, rows, 0, cap, ck, cv)
    pb, cb = fk.sdpa_workspace_bytes(n_heads, n_kv, dim, dim, cap)
    ws, counters = fk.DeviceBuffer(max(256, pb)), fk.zeros(max(256, cb))
    o1, o2 = fk.DeviceBuffer(n_heads * dim * 2), fk.DeviceBuffer(n_heads * dim * 2)
    fk.sdpa_decode_quant(dq, K, V, o1, None, rows, cap, 1, n_heads, dim ** -0.5, ws, counters)
    fk.sdpa_decode(dq, ck, cv, o2, None, rows, cap, n_heads, n_kv, dim, dim, cap, dim ** -0.5, ws, counters)
    assert rel_l2(o1.to_numpy(np.uint16), oracle.bf16_to_f32(o2.to_numpy(np.uint16))) <= 2e-2


def test_rejects_bad_geometry(fk):
    K, V = _caches(fk, 2, 16, 128, 4, 64)
    k = _dev(fk, normal_bf16(1, 256))
    with pytest.raises(fk.FusekitError):
        K3 = fk.QuantKvCache(2, 16, 128, 4, 64)
        K3.bits = 3
        fk.kv_cache_store_quant(k, k, None, 2, 128, 128, 1e4, 0.0, None, 0, 1, K3, V)
    with pytest.raises(fk.FusekitError):
        K48 = fk.QuantKvCache(2, 16, 128, 4, 64)
        K48.group = 48
        fk.kv_cache_store_quant(k, k, None, 2, 128, 128, 1e4, 0.0, None, 0, 1, K48, V)
    out = fk.DeviceBuffer(8 * 128 * 2)
    ws, counters = fk.DeviceBuffer(1 << 20), fk.zeros(4096)
    with pytest.raises(fk.FusekitError):
        K.bits = 2
        fk.sdpa_decode_quant(k, K, V, out, None, 4, 16, 1, 8, 0.1, ws, counters)


@pytest.mark.parametrize("kv_bits,qk_norm", [(8, True), (4, False), (4, True)])
def test_decoder_with_quantised_cache(fk, kv_bits, qk_norm):
    """The decode graph with a quantised KV cache, teacher-forced on the oracle's tokens: logits within
    the bf16 bar at every step, the greedy token identical wherever the oracle's top-2 margin is clear,
    and the batched prompt path leaves the same cache as the token-by-token path."""
    from fusekit_amd.decoder import DecoderConfig, DecoderRuntime, DecoderWeights
    from helpers import OracleDecoder
    cfg = DecoderConfig(n_layers=3, hidden=256, n_heads=4, n_kv=2, head_dim=64, inter=512, vocab=2000, capacity=128,
                        bits=4, qk_norm=qk_norm, qkv_bias=not qk_norm, kv_bits=kv_bits, kv_group=32 if kv_bits == 4 else 64)
    W = DecoderWeights.random_init(cfg, seed=21)
    rt, od = DecoderRuntime(cfg, W), OracleDecoder(cfg, W)
    tok = 11
    for i in range(40):
        rt.d.decode_host_loop(rt.graph, rt.uniforms, i, [tok])
        nxt, margin, ref_logits = od.step(tok, i, want_logits=True)
        got = rt.logits.to_numpy(np.uint16)
        assert rel_l2(got, oracle.bf16_to_f32(ref_logits)) <= 1e-2, i
        if margin > 0.05:
            assert int(np.argmax(oracle.bf16_to_f32(got))) == nxt, i
        tok = nxt
    prompt = rng(5).integers(0, cfg.vocab, 37).tolist()
    a, b = DecoderRuntime(cfg, W), DecoderRuntime(cfg, W)
    a.prefill(prompt)
    b.prefill_rows(prompt)
    for l in range(cfg.n_layers):
        for ca, cb_ in ((a.cache_k[l], b.cache_k[l]), (a.cache_v[l], b.cache_v[l])):
            ha = _host(ca, oracle.QuantCache(cfg.n_kv, cfg.capacity, cfg.head_dim, kv_bits, cfg.kv_group)).dequantize()
            hb = _host(cb_, oracle.QuantCache(cfg.n_kv, cfg.capacity, cfg.head_dim, kv_bits, cfg.kv_group)).dequantize()
            assert not ha[:, len(prompt):].any() and not hb[:, len(prompt):].any()
            assert np.linalg.norm(ha - hb) <= (0.02 if kv_bits == 8 else 0.08) * np.linalg.norm(ha), l
