"""GPU parity of the glue a mixture-of-experts decoder with low-rank keys needs: the cache store of a
key given as [K0 | K1] (K1 rotated while written, shared head, packed K0 / V source; plus the in-place
rotation of the query's second part) and the softmax top-k router, against the CPU oracle through
the C ABI and through the dispatcher families."""
import numpy as np
import pytest

import oracle
from helpers import bf16_mismatch, normal_bf16, rel_l2

pytestmark = pytest.mark.gpu


def _dev(fk, a):
    return fk.DeviceBuffer.from_numpy(np.ascontiguousarray(a))


class _Slice:
    """A device pointer `elems` bf16 elements into a buffer (packed K0 / V sources)."""
    def __init__(self, buf, elems):
        self.ptr = buf.ptr + 2 * elems

    def __int__(self):
        return self.ptr


@pytest.mark.parametrize("traditional", [False, True])
@pytest.mark.parametrize("n_heads,n_kv,k0d,k1d,vd,k1_heads,packed,rope", [
    (16, 16, 128, 64, 128, 1, True, 64),     # config-5 heads: nope 128 | rope 64, values 128, one rotary key head
    (4, 4, 32, 16, 24, 4, False, 8),         # own rotary head per key head, partial rotation
    (0, 2, 64, 64, 64, 1, False, 64),        # no query part
])
def test_split_key_store(fk, n_heads, n_kv, k0d, k1d, vd, k1_heads, packed, rope, traditional):
    cap, pos, theta = 32, 37, 1e4
    if packed:
        src = normal_bf16(1, (n_kv, k0d + vd))
        d_src = _dev(fk, src)
        k0, v, k0s, vs = src.reshape(-1), src.reshape(-1)[k0d:], k0d + vd, k0d + vd
        d_k0, d_v = d_src, _Slice(d_src, k0d)
    else:
        k0, v, k0s, vs = normal_bf16(1, n_kv * k0d), normal_bf16(2, n_kv * vd), k0d, vd
        d_k0, d_v = _dev(fk, k0), _dev(fk, v)
    k1 = normal_bf16(3, (k1_heads, k1d))
    q = normal_bf16(4, (max(n_heads, 1), k0d + k1d))
    ck0, cv0 = normal_bf16(5, n_kv * cap * (k0d + k1d)), normal_bf16(6, n_kv * cap * vd)
    ck, cv = ck0.copy(), cv0.copy()
    oracle.kv_store_split(k0, k0s, k1, k1_heads, v, vs, n_kv, k0d, k1d, vd, rope, traditional, theta, pos, pos, cap, ck, cv)
    d_q, d_ck, d_cv, d_pos = _dev(fk, q), _dev(fk, ck0), _dev(fk, cv0), _dev(fk, np.array([pos], np.uint32))
    fk.kv_cache_store_split_decode(d_q if n_heads else None, n_heads, k0d, k1d, d_k0, k0s, _dev(fk, k1), k1_heads, d_v, vs,
                                   n_kv, k0d, k1d, vd, rope, traditional, theta, d_pos, 0, d_pos, 0, cap, d_ck, d_cv)
    got_k, got_v = d_ck.to_numpy(np.uint16), d_cv.to_numpy(np.uint16)
    assert np.array_equal(got_v, cv)                                   # copies: bit-exact
    gk, rk = got_k.reshape(n_kv, cap, -1), ck.reshape(n_kv, cap, -1)
    keep = np.ones(cap, bool); keep[pos % cap] = False
    assert np.array_equal(gk[:, keep], rk[:, keep])                    # other rows untouched
    assert np.array_equal(gk[:, pos % cap, :k0d], rk[:, pos % cap, :k0d])
    assert np.array_equal(gk[:, pos % cap, k0d + rope:], rk[:, pos % cap, k0d + rope:])
    frac, ulps = bf16_mismatch(gk[:, pos % cap, k0d:k0d + rope], rk[:, pos % cap, k0d:k0d + rope])
    assert ulps <= 1.0 and frac <= 0.02, (frac, ulps)
    if n_heads:
        # Q1 in place = the same rotation (the oracle's store of one-row "caches" rotates it)
        gq = d_q.to_numpy(np.uint16).reshape(n_heads, -1)
        assert np.array_equal(gq[:, :k0d], q[:, :k0d])
        for h in range(n_heads):
            row_k, row_v = np.zeros(k0d + k1d, np.uint16), np.zeros(1, np.uint16)
            oracle.kv_store_split(q[h, :k0d].copy(), k0d, q[h, k0d:].copy(), 1, np.zeros(1, np.uint16), 1, 1, k0d, k1d, 1,
                                  rope, traditional, theta, pos, 0, 1, row_k, row_v)
            frac, ulps = bf16_mismatch(gq[h], row_k)
            assert ulps <= 1.0 and frac <= 0.05, (h, frac, ulps)


def test_split_query_attention_close_to_the_fp32_form(fk):
    """Store + rotate on the GPU, then the attention kernel at 192 / 128: within the bar of the oracle's
    split-query attention, which keeps the rotated Q1 in fp32 as the reference's fused kernel does."""
    n_heads, k0d, k1d, vd, cap, kv_len, theta = 16, 128, 64, 128, 64, 40, 1e4
    q = normal_bf16(10, (n_heads, k0d + k1d))
    ck, cv = normal_bf16(11, n_heads * cap * (k0d + k1d)), normal_bf16(12, n_heads * cap * vd)
    src, k1 = normal_bf16(13, (n_heads, k0d + vd)), normal_bf16(14, (1, k1d))
    pos = kv_len - 1
    rck, rcv = ck.copy(), cv.copy()
    oracle.kv_store_split(src.reshape(-1), k0d + vd, k1, 1, src.reshape(-1)[k0d:], k0d + vd, n_heads, k0d, k1d, vd, k1d, True,
                          theta, pos, pos, cap, rck, rcv)
    scale = 1.0 / np.sqrt(k0d + k1d)
    ref = oracle.sdpa_decode_split_q(q, n_heads, k0d, k1d, k1d, True, theta, rck, rcv, n_heads, vd, kv_len, cap, scale)
    d_q, d_ck, d_cv, d_src = _dev(fk, q), _dev(fk, ck), _dev(fk, cv), _dev(fk, src)
    fk.kv_cache_store_split_decode(d_q, n_heads, k0d, k1d, d_src, k0d + vd, _dev(fk, k1), 1, _Slice(d_src, k0d), k0d + vd,
                                   n_heads, k0d, k1d, vd, k1d, True, theta, None, pos, None, pos, cap, d_ck, d_cv)
    pb, cb = fk.sdpa_workspace_bytes(n_heads, n_heads, k0d + k1d, vd, cap)
    out = fk.DeviceBuffer(2 * n_heads * vd)
    fk.sdpa_decode(d_q, d_ck, d_cv, out, None, kv_len, cap, n_heads, n_heads, k0d + k1d, vd, cap, scale,
                   fk.DeviceBuffer(max(pb, 4)), fk.zeros(max(cb, 4)))
    assert rel_l2(out.to_numpy(np.uint16), oracle.bf16_to_f32(ref)) <= 1e-2


@pytest.mark.parametrize("traditional,table", [(True, True), (False, False), (True, False)])
@pytest.mark.parametrize("n_heads,k0d,k1d,vd,rope,kv_len,cap", [(16, 128, 64, 128, 64, 40, 64), (16, 128, 64, 128, 64, 700, 1024),
                                                             (4, 64, 32, 64, 16, 1, 16), (2, 128, 64, 128, 64, 64, 64)])
def test_split_store_and_attention_in_one_launch(fk, n_heads, k0d, k1d, vd, rope, kv_len, cap, traditional, table):
    """fk_split_store_sdpa_decode == fk_kv_cache_store_split_decode followed by fk_sdpa_decode, bit for bit:
    output, cache rows, and the query left untouched."""
    theta, pos = 1e4, kv_len - 1
    qk = k0d + k1d
    q = normal_bf16(50, (n_heads, qk))
    ck, cv = normal_bf16(51, n_heads * cap * qk), normal_bf16(52, n_heads * cap * vd)
    src, k1 = normal_bf16(53, (n_heads, k0d + vd)), normal_bf16(54, (1, k1d))
    scale = 1.0 / np.sqrt(qk)
    pb, cb = fk.sdpa_workspace_bytes(n_heads, n_heads, qk, vd, cap)

    d_q, d_ck, d_cv, d_src, d_k1 = (_dev(fk, a) for a in (q, ck, cv, src, k1))
    fk.kv_cache_store_split_decode(d_q, n_heads, k0d, k1d, d_src, k0d + vd, d_k1, 1, _Slice(d_src, k0d), k0d + vd, n_heads, k0d,
                                   k1d, vd, rope, traditional, theta, None, pos, None, pos, cap, d_ck, d_cv)
    ref = fk.DeviceBuffer(2 * n_heads * vd)
    fk.sdpa_decode(d_q, d_ck, d_cv, ref, None, kv_len, cap, n_heads, n_heads, qk, vd, cap, scale, fk.DeviceBuffer(max(pb, 4)),
                   fk.zeros(max(cb, 4)))

    f_q, f_ck, f_cv = (_dev(fk, a) for a in (q, ck, cv))
    tab = None
    if table:
        tab = fk.DeviceBuffer(4 * rope)
        fk.step_init_rope(fk.zeros(4), fk.zeros(4), fk.zeros(4), tab, rope, theta)     # position 0 ...
        cnt = _dev(fk, np.array([pos], np.uint32))
        fk.step_init_rope(cnt, fk.zeros(4), fk.zeros(4), tab, rope, theta)             # ... then this token's
    out = fk.DeviceBuffer(2 * n_heads * vd)
    d_len = _dev(fk, np.array([kv_len], np.uint32))
    for _ in range(2):   # counters are left zero: a second launch gives the same bits
        fk.split_store_sdpa_decode(f_q, n_heads, k0d, k1d, d_src, k0d + vd, d_k1, 1, _Slice(d_src, k0d), k0d + vd, n_heads, vd,
                                   rope, traditional, theta, tab, f_ck, f_cv, out, d_len, 0, cap, cap, scale,
                                   fk.DeviceBuffer(max(pb, 4)), fk.zeros(max(cb, 4)))
        assert np.array_equal(out.to_numpy(np.uint16), ref.to_numpy(np.uint16))
    assert np.array_equal(f_ck.to_numpy(np.uint16), d_ck.to_numpy(np.uint16))
    assert np.array_equal(f_cv.to_numpy(np.uint16), d_cv.to_numpy(np.uint16))
    assert np.array_equal(f_q.to_numpy(np.uint16), q.reshape(-1))


@pytest.mark.parametrize("rows,row_n,top_k,per_route", [(1, 64, 6, False), (8, 64, 6, True), (3, 256, 32, False),
                                                        (5, 2, 1, False), (2, 128, 8, True)])
def test_softmax_topk_route(fk, rows, row_n, top_k, per_route):
    logits = normal_bf16(20 + row_n, (rows, row_n), 1.5)
    scale = normal_bf16(21, (rows, top_k), 0.1, 1.0) if per_route else oracle.f32_to_bf16(np.array([1.0], np.float32))
    ref_idx, ref_w = oracle.softmax_topk_route(logits, top_k, scale)
    idx, w = fk.zeros(4 * rows * top_k), fk.zeros(2 * rows * top_k)
    fk.softmax_topk_route(_dev(fk, logits), _dev(fk, scale), per_route, rows, row_n, top_k, idx, w)
    got_idx, got_w = idx.to_numpy(np.uint32, (rows, top_k)), w.to_numpy(np.uint16, (rows, top_k))
    # the fp32 exp / sum may differ in the last place from the oracle's; a probability on a bf16
    # rounding edge can then move one step and swap two neighbours of the order: the selected SET
    # and every weight agree to one step, and all but a few positions agree exactly
    for r in range(rows):
        assert len(set(got_idx[r].tolist())) == top_k
        frac, ulps = bf16_mismatch(got_w[r], ref_w[r])
        assert ulps <= 1.0, (r, ulps)
    assert np.mean(got_idx == ref_idx) >= 0.97, (got_idx, ref_idx)
    assert np.mean(got_w == ref_w) >= 0.97


def test_softmax_topk_route_ties_take_the_lower_index(fk):
    logits = oracle.f32_to_bf16(np.full((2, 64), -0.5, np.float32))
    logits[1, 40] = logits[1, 9] = 0x3F80      # two equal maxima, then the tie of all others
    one = oracle.f32_to_bf16(np.array([1.0], np.float32))
    idx, w = fk.zeros(4 * 2 * 6), fk.zeros(2 * 2 * 6)
    fk.softmax_topk_route(_dev(fk, logits), _dev(fk, one), False, 2, 64, 6, idx, w)
    got = idx.to_numpy(np.uint32, (2, 6))
    assert got[0].tolist() == [0, 1, 2, 3, 4, 5]
    assert got[1].tolist() == [9, 40, 0, 1, 2, 3]
    ref_idx, ref_w = oracle.softmax_topk_route(logits, 6, one)
    assert np.array_equal(got, ref_idx) and np.array_equal(w.to_numpy(np.uint16, (2, 6)), ref_w)


@pytest.mark.parametrize("hidden,experts,top_k,norm", [(2048, 64, 6, True), (512, 8, 2, True), (1024, 256, 32, False),
                                                       (3072, 16, 3, True)])
def test_router_in_one_launch(fk, hidden, experts, top_k, norm):
    """fk_moe_router = rmsnorm -> bf16 linear -> softmax top-k route of the oracle, outputs included."""
    from helpers import make_qweight
    x, nw = normal_bf16(40, hidden), normal_bf16(41, hidden, 0.1, 1.0)
    W = make_qweight(42, experts, hidden, 16, std=0.05)
    scale = oracle.f32_to_bf16(np.array([1.25], np.float32))
    xn_ref = oracle.rmsnorm(x, nw, 1e-6) if norm else x
    lg_ref = oracle.qgemv(W, xn_ref)
    idx_ref, w_ref = oracle.softmax_topk_route(lg_ref, top_k, scale)
    xn, lg, idx, w = fk.zeros(2 * hidden), fk.zeros(2 * experts), fk.zeros(4 * top_k), fk.zeros(2 * top_k)
    ws = fk.zeros(4 * (experts + 1))
    for _ in range(2):    # the second launch finds the counter back at zero
        fk.moe_router(_dev(fk, x), _dev(fk, nw) if norm else None, 1e-6, _dev(fk, W.w), _dev(fk, scale), hidden, experts, top_k,
                      xn, lg, idx, w, ws)
        fk.sync()
    assert ws.to_numpy(np.uint32)[experts] == 0
    frac, ulps = bf16_mismatch(xn.to_numpy(np.uint16), xn_ref)
    assert ulps <= 1.0 and frac <= 0.01
    got_lg = lg.to_numpy(np.uint16)
    frac, ulps = bf16_mismatch(got_lg, lg_ref)
    assert ulps <= 1.0 and frac <= 0.1, (frac, ulps)
    # the route is exactly the oracle's route of the logits the GPU produced (up to an edge flip of a probability)
    idx2, w2 = oracle.softmax_topk_route(got_lg, top_k, scale)
    got_idx, got_w = idx.to_numpy(np.uint32), w.to_numpy(np.uint16)
    assert np.mean(got_idx == idx2.reshape(-1)) >= 0.9 and set(got_idx.tolist()) == set(idx2.reshape(-1).tolist())
    assert bf16_mismatch(got_w, w2.reshape(-1))[1] <= 1.0
    assert len(set(got_idx.tolist()) & set(idx_ref.reshape(-1).tolist())) >= top_k - 1


def test_rejects(fk):
    b = fk.zeros(4096)
    with pytest.raises(fk.FusekitError):
        fk.softmax_topk_route(b, b, False, 1, 48, 4, b, b)          # not a power of two
    with pytest.raises(fk.FusekitError):
        fk.softmax_topk_route(b, b, False, 1, 64, 64, b, b)         # top_k must stay below row_n
    with pytest.raises(fk.InvalidArgument):
        fk.kv_cache_store_split_decode(None, 0, 0, 0, b, 8, b, 3, b, 8, 4, 8, 8, 8, 8, False, 1e4, None, 0, None, 0, 4, b, b)
    with pytest.raises(fk.InvalidArgument):
        fk.kv_cache_store_split_decode(None, 0, 0, 0, b, 4, b, 1, b, 8, 4, 8, 8, 8, 8, False, 1e4, None, 0, None, 0, 4, b, b)


def test_families_in_a_graph(fk):
    """fusekit_kv_cache_store_decode with split_k = 1 and fusekit_softmax_topk_route give the direct calls' bytes."""
    from fusekit_amd.runtime import Dispatch, Dispatcher, arg
    n_heads, k0d, k1d, vd, cap, pos, theta, E, top_k = 4, 32, 16, 32, 8, 5, 1e4, 64, 6
    q, src, k1 = normal_bf16(30, (n_heads, k0d + k1d)), normal_bf16(31, (n_heads, k0d + vd)), normal_bf16(32, (1, k1d))
    logits, one = normal_bf16(33, (1, E)), oracle.f32_to_bf16(np.array([1.0], np.float32))
    d_pos = _dev(fk, np.array([pos], np.uint32))

    def run(direct):
        d_q, d_src, d_k1 = _dev(fk, q), _dev(fk, src), _dev(fk, k1)
        d_ck, d_cv = fk.zeros(2 * n_heads * cap * (k0d + k1d)), fk.zeros(2 * n_heads * cap * vd)
        d_l, d_one, idx, w = _dev(fk, logits), _dev(fk, one), fk.zeros(4 * top_k), fk.zeros(2 * top_k)
        if direct:
            fk.kv_cache_store_split_decode(d_q, n_heads, k0d, k1d, d_src, k0d + vd, d_k1, 1, _Slice(d_src, k0d), k0d + vd,
                                           n_heads, k0d, k1d, vd, k1d, True, theta, d_pos, 0, d_pos, 0, cap, d_ck, d_cv)
            fk.softmax_topk_route(d_l, d_one, False, 1, E, top_k, idx, w)
        else:
            tail = (n_heads * (k0d + vd) - k0d) * 2
            tasks = [
                Dispatch("fusekit_kv_cache_store_decode_f1",
                         [arg(d_q), arg(d_src), arg(d_k1), arg(d_src, tail, k0d * 2), arg(d_ck), arg(d_cv), arg(d_pos), arg(d_pos)],
                         dict(split_k=1, has_q=1, n_heads=n_heads, q0_dim=k0d, q1_dim=k1d, n_kv=n_heads, k0_dim=k0d, k1_dim=k1d,
                              v_dim=vd, k1_n_kv=1, k0_stride=k0d + vd, v_stride=k0d + vd, rope_dims=k1d, traditional=1,
                              theta=theta, capacity=cap)),
                Dispatch("fusekit_softmax_topk_route_f2", [arg(d_l), arg(d_one), arg(idx), arg(w)],
                         dict(row_n=E, top_k=top_k, rows=1)),
            ]
            d = Dispatcher()
            g = d.build_graph(tasks)
            d.execute_graph(g)
        fk.sync()
        return [b.to_numpy(np.uint16) for b in (d_q, d_ck, d_cv, w)] + [idx.to_numpy(np.uint32)]

    for a, b in zip(run(True), run(False)):
        assert np.array_equal(a, b)


def test_split_key_store_rows_wrap_around_the_cache(fk):
    """Row form: token r at position offset + r lands in cache row (offset + r) % capacity with its own rotation;
    the oracle stores the rows one by one."""
    n_heads, k0d, k1d, vd, cap, rows, offset, theta = 4, 64, 32, 64, 8, 5, 6, 1e4
    kvb = normal_bf16(70, (rows, n_heads, k0d + vd))
    kpe = normal_bf16(71, (rows, k1d))
    q = normal_bf16(72, (rows, n_heads, k0d + k1d))
    ck0, cv0 = normal_bf16(73, n_heads * cap * (k0d + k1d)), normal_bf16(74, n_heads * cap * vd)
    ck, cv = ck0.copy(), cv0.copy()
    for r in range(rows):
        flat = kvb[r].reshape(-1)
        oracle.kv_store_split(flat, k0d + vd, kpe[r:r + 1], 1, flat[k0d:], k0d + vd, n_heads, k0d, k1d, vd, k1d, True, theta,
                              offset + r, offset + r, cap, ck, cv)
    d_kvb, d_q, d_ck, d_cv = _dev(fk, kvb), _dev(fk, q), _dev(fk, ck0), _dev(fk, cv0)
    fk.kv_cache_store_split_rows(d_q, n_heads, k0d, k1d, d_kvb, k0d + vd, n_heads * (k0d + vd), _dev(fk, kpe), 1, k1d,
                                 _Slice(d_kvb, k0d), k0d + vd, n_heads * (k0d + vd), n_heads, k0d, k1d, vd, k1d, True, theta, rows,
                                 offset, cap, d_ck, d_cv)
    assert np.array_equal(d_cv.to_numpy(np.uint16), cv)
    frac, ulps = bf16_mismatch(d_ck.to_numpy(np.uint16), ck)
    assert ulps <= 1.0 and frac <= 0.01, (frac, ulps)
    gq = d_q.to_numpy(np.uint16).reshape(rows, n_heads, -1)
    assert np.array_equal(gq[:, :, :k0d], q[:, :, :k0d]) and not np.array_equal(gq[1:, :, k0d:], q[1:, :, k0d:])
