"""GPU parity of RoPE / per-head norm / KV store (R), SDPA decode (K4), embedding (E),
argmax (A) and the step counter (U) against the CPU oracle."""
import numpy as np
import pytest

import oracle
from helpers import bf16_mismatch, make_qweight, normal_bf16, rel_l2, rng

pytestmark = pytest.mark.gpu

REL_L2_BAR = 1e-2


def _u32(fk, v):
    return fk.DeviceBuffer.from_numpy(np.array([v], dtype=np.uint32))


@pytest.mark.parametrize("n_heads,head_dim,rope_dims", [(14, 64, 64), (32, 128, 128), (16, 192, 64)])
@pytest.mark.parametrize("pos", [0, 1, 511, 32767])
def test_rope_q(fk, n_heads, head_dim, rope_dims, pos):
    q = normal_bf16(3, n_heads * head_dim)
    dq = fk.DeviceBuffer.from_numpy(q)
    fk.rope_q_decode(dq, None, n_heads, head_dim, rope_dims, 1e6, 0.0, _u32(fk, pos), 0)
    got = dq.to_numpy(np.uint16)
    ref = oracle.rope_q(q, n_heads, head_dim, rope_dims, 1e6, pos)
    frac, ulps = bf16_mismatch(got, ref)
    assert ulps <= 1.0 and frac <= 0.02
    if pos == 0:
        assert np.array_equal(got, q)  # rotation by zero is the identity
    # same result from the immediate
    dq2 = fk.DeviceBuffer.from_numpy(q)
    fk.rope_q_decode(dq2, None, n_heads, head_dim, rope_dims, 1e6, 0.0, None, pos)
    assert np.array_equal(dq2.to_numpy(np.uint16), got)


@pytest.mark.parametrize("norm", [False, True])
def test_rope_kv_store_and_fused(fk, norm):
    n_heads, n_kv, D, cap, pos = 32, 8, 128, 64, 70  # 70 % 64 = row 6: ring-buffer modulo
    q, k, v = normal_bf16(1, n_heads * D), normal_bf16(2, n_kv * D), normal_bf16(3, n_kv * D)
    qw, kw = normal_bf16(4, D, 0.1, 1.0), normal_bf16(5, D, 0.1, 1.0)
    ck0, cv0 = normal_bf16(6, n_kv * cap * D), normal_bf16(7, n_kv * cap * D)
    eps = 1e-6
    # oracle
    ck, cv = ck0.copy(), cv0.copy()
    if norm:
        rq = oracle.headnorm_rope(q, qw, n_heads, D, D, eps, 1e6, pos)
        rk = oracle.headnorm_rope(k, kw, n_kv, D, D, eps, 1e6, pos)
        oracle.kv_store(rk, v, n_kv, D, D, pos, cap, ck, cv)
    else:
        rq = oracle.rope_q(q, n_heads, D, D, 1e6, pos)
        oracle.rope_kv_store(k, v, n_kv, D, D, 1e6, pos, pos, cap, ck, cv)
    # separate launches
    dq, dck, dcv = (fk.DeviceBuffer.from_numpy(t) for t in (q, ck0, cv0))
    dqw, dkw = (fk.DeviceBuffer.from_numpy(t) if norm else None for t in (qw, kw))
    dpos = _u32(fk, pos)
    fk.rope_q_decode(dq, dqw, n_heads, D, D, 1e6, eps, dpos, 0)
    fk.rope_kv_cache_store_decode(fk.DeviceBuffer.from_numpy(k), fk.DeviceBuffer.from_numpy(v), dkw, n_kv, D, D, D,
                                  1e6, eps, dpos, 0, dpos, 0, cap, dck, dcv)
    for got, ref in ((dq, rq), (dck, ck), (dcv, cv)):
        frac, ulps = bf16_mismatch(got.to_numpy(np.uint16), ref)
        assert ulps <= 1.0 and frac <= 0.02
    assert np.array_equal(dcv.to_numpy(np.uint16), cv)  # V is a pure copy: bit-exact
    # untouched cache rows stay untouched
    gk = dck.to_numpy(np.uint16).reshape(n_kv, cap, D)
    keep = np.ones(cap, bool); keep[pos % cap] = False
    assert np.array_equal(gk[:, keep], ck0.reshape(n_kv, cap, D)[:, keep])
    # fused single launch gives the same bits as the separate launches
    fq, fck, fcv = (fk.DeviceBuffer.from_numpy(t) for t in (q, ck0, cv0))
    fk.qkv_rope_store_decode(fq, fk.DeviceBuffer.from_numpy(k), fk.DeviceBuffer.from_numpy(v), dqw, dkw, n_heads,
                             n_kv, D, D, 1e6, eps, dpos, 0, cap, fck, fcv)
    for a, b in ((fq, dq), (fck, dck), (fcv, dcv)):
        assert np.array_equal(a.to_numpy(np.uint16), b.to_numpy(np.uint16))


def test_kv_store_mla_dims(fk):
    """qk_dim != v_dim, no rotation (prepared K rows)."""
    n_kv, kd, vd, cap, pos = 16, 192, 128, 32, 5
    k, v = normal_bf16(1, n_kv * kd), normal_bf16(2, n_kv * vd)
    ck0, cv0 = np.zeros(n_kv * cap * kd, np.uint16), np.zeros(n_kv * cap * vd, np.uint16)
    ck, cv = ck0.copy(), cv0.copy()
    oracle.kv_store(k, v, n_kv, kd, vd, pos, cap, ck, cv)
    dck, dcv = fk.DeviceBuffer.from_numpy(ck0), fk.DeviceBuffer.from_numpy(cv0)
    fk.rope_kv_cache_store_decode(fk.DeviceBuffer.from_numpy(k), fk.DeviceBuffer.from_numpy(v), None, n_kv, kd, vd, 0,
                                  1e6, 0.0, None, pos, None, pos, cap, dck, dcv)
    assert np.array_equal(dck.to_numpy(np.uint16), ck) and np.array_equal(dcv.to_numpy(np.uint16), cv)


def _sdpa_case(fk, n_heads, n_kv, qk, vd, kv_len, cap, seed=0, max_len=None):
    q = normal_bf16(seed, n_heads * qk)
    ck, cv = normal_bf16(seed + 1, n_kv * cap * qk), normal_bf16(seed + 2, n_kv * cap * vd)
    scale = 1.0 / np.sqrt(qk)
    max_len = max_len or kv_len
    pb, cb = fk.sdpa_workspace_bytes(n_heads, n_kv, qk, vd, max_len)
    part, cnt = fk.DeviceBuffer(max(pb, 4)), fk.zeros(max(cb, 4))
    out = fk.DeviceBuffer(2 * n_heads * vd)
    dq, dck, dcv = (fk.DeviceBuffer.from_numpy(t) for t in (q, ck, cv))
    fk.sdpa_decode(dq, dck, dcv, out, _u32(fk, kv_len), 0, max_len, n_heads, n_kv, qk, vd, cap, scale, part, cnt)
    got = out.to_numpy(np.uint16)
    ref = oracle.sdpa_decode(q, ck, cv, n_heads, n_kv, qk, vd, kv_len, cap, scale)
    assert rel_l2(got, oracle.bf16_to_f32(ref)) <= REL_L2_BAR
    # element-wise: 2 bf16 ulps, or -- where an output is a near-total cancellation of
    # sum p_j v_j -- the fp32 reordering bound taken relative to the typical output size
    g, r = oracle.bf16_to_f32(got).astype(np.float64), oracle.bf16_to_f32(ref).astype(np.float64)
    tol = 2 * 2.0 ** -8 * np.abs(r) + 1e-4 * np.sqrt(np.mean(r * r))
    assert np.all(np.abs(g - r) <= tol), float(np.max(np.abs(g - r) - tol))
    assert np.mean(got != ref) <= 0.05
    assert not cnt.to_numpy(np.uint32).any()  # counters are left zero for the next launch
    # a second launch on the same workspace gives the same bits (ordered merge, reset counters)
    fk.sdpa_decode(dq, dck, dcv, out, None, kv_len, max_len, n_heads, n_kv, qk, vd, cap, scale, part, cnt)
    assert np.array_equal(out.to_numpy(np.uint16), got)
    return q, ck, cv, got


@pytest.mark.parametrize("kv_len", [1, 2, 31, 32, 33, 512, 1000])
def test_sdpa_gqa_small(fk, kv_len):
    _sdpa_case(fk, 32, 8, 128, 128, kv_len, 1024)


def test_sdpa_kv_len_one_returns_v0(fk):
    q, ck, cv, got = _sdpa_case(fk, 32, 8, 128, 128, 1, 16)
    v0 = cv.reshape(8, 16, 128)[:, 0]          # softmax over one key is 1
    assert np.array_equal(got.reshape(8, 4, 128), np.repeat(v0[:, None], 4, 1))


@pytest.mark.parametrize("n_heads,n_kv,qk,vd", [(14, 2, 64, 64), (16, 16, 192, 128), (8, 8, 64, 64), (6, 2, 128, 128)])
def test_sdpa_other_head_layouts(fk, n_heads, n_kv, qk, vd):
    _sdpa_case(fk, n_heads, n_kv, qk, vd, 300, 512)


@pytest.mark.parametrize("kv_len", [4096, 32768])
def test_sdpa_long_context(fk, kv_len):
    _sdpa_case(fk, 32, 8, 128, 128, kv_len, kv_len)


def test_sdpa_split_invariance(fk):
    """Any split of the context gives the same result to fp32 rounding: run one kv_len
    with two different max_len (hence different range sizes)."""
    a = _sdpa_case(fk, 32, 8, 128, 128, 700, 32768, max_len=700)[3]
    b = _sdpa_case(fk, 32, 8, 128, 128, 700, 32768, max_len=32768)[3]
    frac, ulps = bf16_mismatch(a, b)
    assert ulps <= 1.0 and frac <= 0.02


@pytest.mark.parametrize("bits", [16, 4, 8])
def test_embed_lookup(fk, bits):
    vocab, hidden = 1000, 896
    E = make_qweight(9, vocab, hidden, bits)
    dE = fk.DeviceWeight(E.w, E.scales, E.biases, E.n, E.k, E.bits, E.group)
    x = fk.DeviceBuffer(2 * hidden)
    for tok, sc in ((0, 1.0), (999, 1.0), (123, 29.93)):
        fk.embed_lookup_decode(dE, _u32(fk, tok), 0, sc, x)
        assert np.array_equal(x.to_numpy(np.uint16), oracle.embed_lookup(E, tok, sc))  # bit-exact
    with pytest.raises(fk.FusekitError):
        fk.embed_lookup_decode(dE, None, vocab, 1.0, x)


def test_argmax_ties_nan_and_history(fk):
    n = 151936
    vals = rng(0).standard_normal(n).astype(np.float32)
    logits = oracle.f32_to_bf16(vals)
    top = oracle.bf16_to_f32(logits).max()
    # plant exact ties of the maximum at several indices; lowest must win
    logits[[140000, 77, 5000]] = oracle.f32_to_bf16(np.array([top], np.float32))[0]
    logits[3] = 0x7FC0  # NaN never wins
    ws = fk.zeros(fk.ARGMAX_WORKSPACE_BYTES)
    nxt, hist, hc = fk.zeros(4), fk.zeros(4 * 8), fk.zeros(4)
    dl = fk.DeviceBuffer.from_numpy(logits)
    for step in range(3):
        fk.argmax_logits_decode(dl, n, nxt, hist, hc, 8, ws)
        assert int(nxt.to_numpy(np.uint32)[0]) == oracle.argmax(logits)
    assert int(hc.to_numpy(np.uint32)[0]) == 3
    assert list(hist.to_numpy(np.uint32)[:3]) == [oracle.argmax(logits)] * 3
    # brute force on small ragged sizes, negative-only rows, single element
    for m in (1, 2, 63, 64, 65, 2049, 4097):
        sub = oracle.f32_to_bf16(-np.abs(rng(m).standard_normal(m)).astype(np.float32) - 1.0)
        fk.argmax_logits_decode(fk.DeviceBuffer.from_numpy(sub), m, nxt, None, None, 0, ws)
        f = oracle.bf16_to_f32(sub)
        assert int(nxt.to_numpy(np.uint32)[0]) == int(np.flatnonzero(f == f.max())[0]) == oracle.argmax(sub)


def test_step_init(fk):
    sc, off, kvl = fk.DeviceBuffer.from_numpy(np.array([41], np.uint32)), fk.zeros(4), fk.zeros(4)
    for i in range(3):
        fk.step_init(sc, off, kvl)
    assert int(sc.to_numpy(np.uint32)[0]) == 44
    assert int(off.to_numpy(np.uint32)[0]) == 43 and int(kvl.to_numpy(np.uint32)[0]) == 44


@pytest.mark.parametrize("norm,table", [(False, False), (True, True), (True, False)])
@pytest.mark.parametrize("n_heads,n_kv,dim,rope_dims,cap,kv_len", [
    (32, 8, 128, 128, 1024, 1),       # first token: the only row is the new one
    (32, 8, 128, 128, 1024, 100),     # one range
    (32, 8, 128, 128, 1024, 577),     # several ranges, the new row in the last one
    (14, 2, 64, 64, 4096, 2049),      # group of 7 heads (tile of 8), the new row opens a range
    (16, 16, 192, 64, 256, 256),      # partial rotation, cache exactly full
    (4, 1, 128, 128, 16384, 9000),    # blocks that walk several ranges
])
def test_rope_store_sdpa_in_one_launch(fk, norm, table, n_heads, n_kv, dim, rope_dims, cap, kv_len):
    """fk_rope_store_sdpa_decode against the launch pair it replaces (fk_qkv_rope_store_decode, then
    fk_sdpa_decode): the same arithmetic in the same order, so the attention output and both caches
    are identical bit for bit; and the attention output against the oracle."""
    theta, eps, scale, pos = 1e6, 1e-6, dim ** -0.5, kv_len - 1
    q, k, v = normal_bf16(1, n_heads * dim), normal_bf16(2, n_kv * dim), normal_bf16(3, n_kv * dim)
    qw, kw = (normal_bf16(4, dim, 0.1, 1.0), normal_bf16(5, dim, 0.1, 1.0)) if norm else (None, None)
    ck, cv = normal_bf16(6, n_kv * cap * dim), normal_bf16(7, n_kv * cap * dim)
    dev = lambda a: None if a is None else fk.DeviceBuffer.from_numpy(a)
    pb, cb = fk.sdpa_workspace_bytes(n_heads, n_kv, dim, dim, cap)
    part, cnt = fk.DeviceBuffer(max(pb, 16)), fk.zeros(max(cb, 16))
    # the pair
    dq, ck1, cv1, out1 = dev(q), dev(ck), dev(cv), fk.DeviceBuffer(n_heads * dim * 2)
    fk.qkv_rope_store_decode(dq, dev(k), dev(v), dev(qw), dev(kw), n_heads, n_kv, dim, rope_dims, theta, eps,
                             _u32(fk, pos), 0, cap, ck1, cv1)
    fk.sdpa_decode(dq, ck1, cv1, out1, _u32(fk, kv_len), 0, cap, n_heads, n_kv, dim, dim, cap, scale, part, cnt)
    # one launch
    ck2, cv2, out2 = dev(ck), dev(cv), fk.DeviceBuffer(n_heads * dim * 2)
    tab = None
    if table:
        tab = fk.DeviceBuffer(rope_dims * 4)
        ctr, off, kvl = _u32(fk, pos), fk.zeros(4), fk.zeros(4)
        fk.step_init_rope(ctr, off, kvl, tab, rope_dims, theta)
        assert (ctr.to_numpy(np.uint32)[0], off.to_numpy(np.uint32)[0], kvl.to_numpy(np.uint32)[0]) == (pos + 1, pos, pos + 1)
    fk.rope_store_sdpa_decode(dev(q), dev(k), dev(v), dev(qw), dev(kw), ck2, cv2, out2, _u32(fk, kv_len), 0, cap, n_heads,
                              n_kv, dim, rope_dims, theta, eps, cap, scale, tab, part, cnt)
    assert np.array_equal(ck2.to_numpy(np.uint16), ck1.to_numpy(np.uint16))
    assert np.array_equal(cv2.to_numpy(np.uint16), cv1.to_numpy(np.uint16))
    assert np.array_equal(out2.to_numpy(np.uint16), out1.to_numpy(np.uint16))
    assert not np.array_equal(ck2.to_numpy(np.uint16), ck)          # the row was appended
    ref = oracle.sdpa_decode(dq.to_numpy(np.uint16), ck1.to_numpy(np.uint16), cv1.to_numpy(np.uint16), n_heads, n_kv,
                             dim, dim, kv_len, cap, scale)
    assert rel_l2(out2.to_numpy(np.uint16), oracle.bf16_to_f32(ref)) <= REL_L2_BAR
    # immediate kv_len gives the same result
    ck3, cv3, out3 = dev(ck), dev(cv), fk.DeviceBuffer(n_heads * dim * 2)
    fk.rope_store_sdpa_decode(dev(q), dev(k), dev(v), dev(qw), dev(kw), ck3, cv3, out3, None, kv_len, cap, n_heads,
                              n_kv, dim, rope_dims, theta, eps, cap, scale, tab, part, cnt)
    assert np.array_equal(out3.to_numpy(np.uint16), out1.to_numpy(np.uint16))
    assert np.array_equal(ck3.to_numpy(np.uint16), ck1.to_numpy(np.uint16))


@pytest.mark.parametrize("kv_len", [512, 4096, 32768])
def test_config3_rope_append_attention_chain_against_the_oracle(fk, kv_len):
    """configs[2] as stated: 32 q / 8 kv heads x 128, bf16 cache ~ N(0, 1) of kv_len - 1 positions, RoPE (theta 1e6) on
    q and on the new k, the new k / v rows appended at position kv_len - 1, then attention over kv_len rows --
    the one-launch form against the ORACLE's chain (rope_q, rope + cache store, attention), cache rows included."""
    n_heads, n_kv, dim, theta, eps = 32, 8, 128, 1e6, 1e-6
    cap, pos, scale = kv_len, kv_len - 1, dim ** -0.5
    q, k, v = normal_bf16(11, n_heads * dim), normal_bf16(12, n_kv * dim), normal_bf16(13, n_kv * dim)
    ck, cv = normal_bf16(14, n_kv * cap * dim), normal_bf16(15, n_kv * cap * dim)
    dev = lambda a: fk.DeviceBuffer.from_numpy(a)
    pb, cb = fk.sdpa_workspace_bytes(n_heads, n_kv, dim, dim, cap)
    part, cnt = fk.DeviceBuffer(max(pb, 16)), fk.zeros(max(cb, 16))
    dck, dcv, out = dev(ck), dev(cv), fk.DeviceBuffer(n_heads * dim * 2)
    tab = fk.DeviceBuffer(dim * 4)
    fk.step_init_rope(_u32(fk, pos), fk.zeros(4), fk.zeros(4), tab, dim, theta)
    fk.rope_store_sdpa_decode(dev(q), dev(k), dev(v), None, None, dck, dcv, out, _u32(fk, kv_len), 0, cap, n_heads, n_kv,
                              dim, dim, theta, eps, cap, scale, tab, part, cnt)
    # the oracle's chain on the same inputs
    rq = oracle.rope_q(q, n_heads, dim, dim, theta, pos)
    ock, ocv = ck.copy(), cv.copy()
    oracle.rope_kv_store(k, v, n_kv, dim, dim, theta, pos, pos, cap, ock, ocv)
    got_ck, got_cv = dck.to_numpy(np.uint16), dcv.to_numpy(np.uint16)
    assert np.array_equal(got_cv, ocv)                                    # V is a pure copy: bit-exact
    rows = lambda a: a.reshape(n_kv, cap, dim)
    keep = np.arange(cap) != pos
    assert np.array_equal(rows(got_ck)[:, keep], rows(ock)[:, keep])      # no other row touched
    frac, ulps = bf16_mismatch(rows(got_ck)[:, pos], rows(ock)[:, pos])
    assert ulps <= 1.0 and frac <= 0.02                                   # fp32 sin / cos products on a rounding edge
    ref = oracle.sdpa_decode(rq, ock, ocv, n_heads, n_kv, dim, dim, kv_len, cap, scale)
    assert rel_l2(out.to_numpy(np.uint16), oracle.bf16_to_f32(ref)) <= REL_L2_BAR
    assert not cnt.to_numpy(np.uint32).any()


def test_rope_store_sdpa_rejects_bad_arguments(fk):
    b = fk.DeviceBuffer(1 << 16)
    args = dict(n_heads=8, n_kv=2, dim=64)
    with pytest.raises(fk.FusekitError):      # q norm without k norm
        fk.rope_store_sdpa_decode(b, b, b, b, None, b, b, b, None, 4, 16, 8, 2, 64, 64, 1e4, 1e-6, 16, 0.1, None, b, b)
    with pytest.raises(fk.FusekitError):      # odd rope_dims
        fk.rope_store_sdpa_decode(b, b, b, None, None, b, b, b, None, 4, 16, 8, 2, 64, 33, 1e4, 1e-6, 16, 0.1, None, b, b)
    with pytest.raises(fk.FusekitError):      # kv_len beyond max_len
        fk.rope_store_sdpa_decode(b, b, b, None, None, b, b, b, None, 17, 16, 8, 2, 64, 64, 1e4, 1e-6, 16, 0.1, None, b, b)
    with pytest.raises(fk.FusekitError):      # table requested with rope_dims 0
        fk.step_init_rope(b, b, b, b, 0, 1e4)
