"""GPU parity of the mixture-of-experts routed projections (M1 gate/up + SwiGLU, M2 down +
weighted reduction) against the CPU oracle, through the C ABI.

Same bars as the dense GEMV family: rel-L2 <= 1e-2 against an fp32 reference, and
element-wise equality with the oracle except for bf16 rounding-edge flips.
"""
import numpy as np
import pytest

import oracle
from helpers import bf16_mismatch, make_qweight, normal_bf16, rel_l2, rng, to_device
from test_gemv_gpu import FLIP_FRACTION_BAR, REL_L2_BAR, _check_swiglu

pytestmark = pytest.mark.gpu


def _stack(seed, n_experts, n, k, bits):
    return oracle.StackedWeight([make_qweight(seed + e, n, k, bits) for e in range(n_experts)])


def _dev(fk, a):
    return None if a is None else fk.DeviceBuffer.from_numpy(np.ascontiguousarray(a))


def _swiglu_fp32(x_row, Wg, Wu, rw):
    g, u = oracle.linear_acc(Wg, x_row).astype(np.float64), oracle.linear_acc(Wu, x_row).astype(np.float64)
    return g / (1 + np.exp(-g)) * u * rw


def _run_m1(fk, x, Wg, Wu, row_idx, expert_idx, route_weight):
    n_routes = expert_idx.size
    out = fk.DeviceBuffer(2 * n_routes * Wg.n)
    fk.routed_qmv_swiglu(_dev(fk, x), x.shape[0], to_device(fk, Wg), to_device(fk, Wu), Wg.n_experts,
                         _dev(fk, row_idx), _dev(fk, expert_idx), _dev(fk, route_weight), n_routes, out)
    return out.to_numpy(np.uint16, (n_routes, Wg.n))


@pytest.mark.parametrize("bits", [4, 8, 16])
@pytest.mark.parametrize("weighted", [False, True])
def test_routed_swiglu_one_token(fk, bits, weighted):
    E, O, K, top_k = 8, 352, 512, 6          # O not a multiple of the tile rows
    Wg, Wu = _stack(100, E, O, K, bits), _stack(200, E, O, K, bits)
    x = normal_bf16(3, (1, K))
    expert_idx = np.array([5, 0, 7, 2, 2, 6], np.uint32)   # an expert may be picked twice
    row_idx = np.zeros(top_k, np.uint32)
    rw = normal_bf16(4, top_k, 0.1, 0.3) if weighted else None
    got = _run_m1(fk, x, Wg, Wu, row_idx, expert_idx, rw)
    ref = oracle.routed_qmv_swiglu(x, Wg, Wu, row_idx, expert_idx, rw)
    for r in range(top_k):
        e = int(expert_idx[r])
        scale = float(oracle.bf16_to_f32(rw[r:r + 1])[0]) if weighted else 1.0
        assert rel_l2(got[r], _swiglu_fp32(x[0], Wg.expert(e), Wu.expert(e), scale)) <= REL_L2_BAR
        if weighted:
            frac, ulps = bf16_mismatch(got[r], ref[r])
            assert frac <= FLIP_FRACTION_BAR and ulps <= 2.0, (r, frac, ulps)
        else:
            _check_swiglu(got[r], ref[r], x[0], Wg.expert(e), Wu.expert(e), 1)


def test_routed_swiglu_rows_and_clamp(fk):
    """Several tokens with their own activation rows; expert and row indices beyond the range clamp."""
    E, O, K, tokens, top_k = 4, 128, 256, 5, 2
    Wg, Wu = _stack(300, E, O, K, 4), _stack(400, E, O, K, 4)
    x = normal_bf16(5, (tokens, K))
    expert_idx = rng(6).integers(0, E, tokens * top_k).astype(np.uint32)
    expert_idx[3] = 1000                     # clamps to E - 1 (routed_qmv_swiglu.rs:138)
    row_idx = np.repeat(np.arange(tokens, dtype=np.uint32), top_k)
    got = _run_m1(fk, x, Wg, Wu, row_idx, expert_idx, None)
    ref = oracle.routed_qmv_swiglu(x, Wg, Wu, row_idx, expert_idx, None)
    for r in range(tokens * top_k):
        e = min(int(expert_idx[r]), E - 1)
        _check_swiglu(got[r], ref[r], x[row_idx[r]], Wg.expert(e), Wu.expert(e), 1)
    # a row index past the end reads the last row instead of faulting
    far = row_idx.copy()
    far[-1] = 77
    got2 = _run_m1(fk, x, Wg, Wu, far, expert_idx, None)
    assert np.array_equal(got2[:-1], got[:-1])
    assert np.array_equal(got2[-1], got[-1])  # the last route already read the last row


@pytest.mark.parametrize("bits", [4, 8])
def test_routed_swiglu_with_shared_experts_riding_along(fk, bits):
    """fk_routed_qmv_swiglu_shared: the routed outputs are the plain routed launch's bits, the shared outputs
    the dense gate/up + SwiGLU pair's (variant B, no norm) on the same activation row."""
    E, O, K, top_k, n_shared = 8, 192, 256, 3, 2
    Wg, Wu = _stack(2200, E, O, K, bits), _stack(2300, E, O, K, bits)
    Sg, Su = make_qweight(2400, n_shared * O, K, bits), make_qweight(2500, n_shared * O, K, bits)
    x = normal_bf16(40, (1, K))
    expert_idx = np.array([5, 0, 7], np.uint32)
    rw = normal_bf16(41, top_k, 0.2, 0.4)
    out0, shared = fk.DeviceBuffer(2 * top_k * O), fk.DeviceBuffer(2 * n_shared * O)
    fk.routed_qmv_swiglu_shared(_dev(fk, x), to_device(fk, Wg), to_device(fk, Wu), E, _dev(fk, expert_idx), _dev(fk, rw), top_k,
                                out0, to_device(fk, Sg), to_device(fk, Su), shared)
    plain = _run_m1(fk, x, Wg, Wu, np.zeros(top_k, np.uint32), expert_idx, rw)
    assert np.array_equal(out0.to_numpy(np.uint16, (top_k, O)), plain)
    ref = oracle.gateup_swiglu(x.reshape(-1), None, 0.0, Sg, Su, 1)
    frac, ulps = bf16_mismatch(shared.to_numpy(np.uint16), ref)
    assert frac <= FLIP_FRACTION_BAR and ulps <= 2.0, (frac, ulps)
    with pytest.raises(fk.InvalidArgument):    # shared matrices must be whole row blocks of the expert shape
        fk.routed_qmv_swiglu_shared(_dev(fk, x), to_device(fk, Wg), to_device(fk, Wu), E, _dev(fk, expert_idx), None, top_k,
                                    out0, to_device(fk, make_qweight(1, O + 64, K, bits)), to_device(fk, make_qweight(2, O + 64, K, bits)), shared)


@pytest.mark.parametrize("apply_weight,shared", [(False, True), (True, False)])
def test_routed_swiglu_routing_for_itself(fk, apply_weight, shared):
    """fk_routed_qmv_swiglu_routing: the route written out is the oracle's router on the same logits, and the
    outputs are the plain routed launch's bits for that route."""
    E, O, K, top_k = 16, 192, 256, 4
    Wg, Wu = _stack(2800, E, O, K, 4), _stack(2900, E, O, K, 4)
    Sg, Su = make_qweight(3000, 2 * O, K, 4), make_qweight(3100, 2 * O, K, 4)
    x = normal_bf16(60, (1, K))
    logits = normal_bf16(61, E, 1.5)
    scale = oracle.f32_to_bf16(np.array([1.5], np.float32))
    ref_idx, ref_w = oracle.softmax_topk_route(logits, top_k, scale)
    idx, w = fk.zeros(4 * top_k), fk.zeros(2 * top_k)
    out0, sh = fk.DeviceBuffer(2 * top_k * O), fk.zeros(2 * 2 * O)
    fk.routed_qmv_swiglu_routing(_dev(fk, x), to_device(fk, Wg), to_device(fk, Wu), E, _dev(fk, logits), _dev(fk, scale), top_k,
                                 apply_weight, idx, w, out0, to_device(fk, Sg) if shared else None,
                                 to_device(fk, Su) if shared else None, sh if shared else None)
    got_idx, got_w = idx.to_numpy(np.uint32), w.to_numpy(np.uint16)
    assert np.array_equal(got_idx, ref_idx.reshape(-1)) and np.array_equal(got_w, ref_w.reshape(-1))
    plain = _run_m1(fk, x, Wg, Wu, np.zeros(top_k, np.uint32), got_idx, got_w if apply_weight else None)
    assert np.array_equal(out0.to_numpy(np.uint16, (top_k, O)), plain)
    if shared:
        ref = oracle.gateup_swiglu(x.reshape(-1), None, 0.0, Sg, Su, 1)
        frac, ulps = bf16_mismatch(sh.to_numpy(np.uint16), ref)
        assert frac <= FLIP_FRACTION_BAR and ulps <= 2.0


def test_routed_swiglu_routing_ties_and_the_largest_admitted_shape(fk):
    """256 experts, 32 routes: equal logits route to experts 0 .. 31 in order (ties to the lower index), each with
    probability 1/256; then a seeded row against the oracle's router."""
    E, O, K, top_k = 256, 64, 128, 32
    Wg, Wu = _stack(3200, E, O, K, 4), _stack(3300, E, O, K, 4)
    x = normal_bf16(62, (1, K))
    one = oracle.f32_to_bf16(np.array([1.0], np.float32))
    idx, w, out0 = fk.zeros(4 * top_k), fk.zeros(2 * top_k), fk.DeviceBuffer(2 * top_k * O)
    dWg, dWu = to_device(fk, Wg), to_device(fk, Wu)
    flat = oracle.f32_to_bf16(np.full(E, 0.25, np.float32))
    fk.routed_qmv_swiglu_routing(_dev(fk, x), dWg, dWu, E, _dev(fk, flat), _dev(fk, one), top_k, False, idx, w, out0)
    assert idx.to_numpy(np.uint32).tolist() == list(range(top_k))
    assert np.array_equal(w.to_numpy(np.uint16), oracle.f32_to_bf16(np.full(top_k, 1.0 / E, np.float32)))
    logits = normal_bf16(63, E, 2.0)
    fk.routed_qmv_swiglu_routing(_dev(fk, x), dWg, dWu, E, _dev(fk, logits), _dev(fk, one), top_k, False, idx, w, out0)
    ref_idx, ref_w = oracle.softmax_topk_route(logits, top_k, one)
    got_idx = idx.to_numpy(np.uint32)
    assert set(got_idx.tolist()) == set(ref_idx.reshape(-1).tolist()) and np.mean(got_idx == ref_idx.reshape(-1)) >= 0.9
    assert bf16_mismatch(w.to_numpy(np.uint16), ref_w.reshape(-1))[1] <= 1.0
    plain = _run_m1(fk, x, Wg, Wu, np.zeros(top_k, np.uint32), got_idx, None)
    assert np.array_equal(out0.to_numpy(np.uint16, (top_k, O)), plain)


def _run_m2(fk, h, Wd, row_idx, expert_idx, rw, shared_x, Ws, res, tokens, top_k):
    out = fk.DeviceBuffer(2 * tokens * Wd.n)
    ws = fk.DeviceBuffer(fk.routed_reduce_workspace_bytes(tokens, top_k, Wd.n))
    fk.routed_qmv_reduce(_dev(fk, h), h.shape[0], to_device(fk, Wd), Wd.n_experts, _dev(fk, row_idx),
                         _dev(fk, expert_idx), _dev(fk, rw), _dev(fk, shared_x),
                         None if Ws is None else to_device(fk, Ws), _dev(fk, res), tokens, top_k, out, ws)
    return out.to_numpy(np.uint16, (tokens, Wd.n))


def _m2_fp32(h, Wd, expert_idx, rw, shared_x, Ws, res, tokens, top_k):
    ref = np.zeros((tokens, Wd.n))
    for t in range(tokens):
        for s in range(top_k):
            r = t * top_k + s
            w = float(oracle.bf16_to_f32(rw[r:r + 1])[0]) if rw is not None else 1.0
            ref[t] += w * oracle.linear_acc(Wd.expert(int(expert_idx[r])), h[r]).astype(np.float64)
        if Ws is not None:
            ref[t] += oracle.linear_acc(Ws, shared_x[t]).astype(np.float64)
        if res is not None:
            ref[t] += oracle.bf16_to_f32(res[t]).astype(np.float64)
    return ref


@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("preweighted", [False, True])
@pytest.mark.parametrize("shared,residual", [(False, False), (False, True), (True, True)])
def test_routed_reduce_one_token(fk, bits, preweighted, shared, residual):
    E, O, K, top_k = 8, 320, 448, 6
    Wd = _stack(500, E, O, K, bits)
    h = normal_bf16(7, (top_k, K), 0.0, 0.5)
    expert_idx = np.array([1, 4, 4, 0, 7, 3], np.uint32)
    rw = None if preweighted else normal_bf16(8, top_k, 0.15, 0.2)
    Ws = make_qweight(600, O, 256, bits) if shared else None
    sx = normal_bf16(9, (1, 256)) if shared else None
    res = normal_bf16(10, (1, O)) if residual else None
    got = _run_m2(fk, h, Wd, None, expert_idx, rw, sx, Ws, res, 1, top_k)
    ref = oracle.routed_qmv_reduce(h, Wd, expert_idx, rw, res, 1, top_k, shared_x=sx, Wshared=Ws)
    assert rel_l2(got, _m2_fp32(h, Wd, expert_idx, rw, sx, Ws, res, 1, top_k)) <= REL_L2_BAR
    frac, ulps = bf16_mismatch(got, ref)
    assert frac <= FLIP_FRACTION_BAR and ulps <= 2.0, (frac, ulps)


@pytest.mark.parametrize("fused", [True, False])
@pytest.mark.parametrize("E,O,K,top_k,SK,with_rows", [(16, 2048, 1408, 6, 2816, False), (8, 320, 448, 6, 256, True),
                                                      (4, 64, 2048, 8, 4096, False), (4, 128, 64, 1, 0, False)])
def test_routed_reduce_one_launch_and_three(fk, fused, E, O, K, top_k, SK, with_rows):
    """One token of int4 weights: the single-launch form (a wave per output row, routes added in slot order)
    and the three-launch form both meet the oracle; fk_set_routed_fused_reduce picks."""
    Wd = _stack(2000, E, O, K, 4)
    n_rows = top_k + 2 if with_rows else top_k
    h = normal_bf16(30, (n_rows, K), 0.0, 0.5)
    row_idx = rng(31).permutation(n_rows)[:top_k].astype(np.uint32) if with_rows else None
    expert_idx = rng(32).integers(0, E + 2, top_k).astype(np.uint32)      # some beyond E: clamped
    rw = normal_bf16(33, top_k, 0.15, 0.2)
    Ws = make_qweight(2100, O, SK, 4) if SK else None
    sx = normal_bf16(34, (1, SK)) if SK else None
    res = normal_bf16(35, (1, O))
    fk.set_routed_fused_reduce(fused)
    try:
        got = _run_m2(fk, h, Wd, row_idx, expert_idx, rw, sx, Ws, res, 1, top_k)
    finally:
        fk.set_routed_fused_reduce(True)
    clamped = np.minimum(expert_idx, E - 1)
    ref = oracle.routed_qmv_reduce(h, Wd, clamped, rw, res, 1, top_k, row_idx=row_idx, shared_x=sx, Wshared=Ws)
    hh = h if row_idx is None else h[row_idx]
    assert rel_l2(got, _m2_fp32(hh, Wd, clamped, rw, sx, Ws, res, 1, top_k)) <= REL_L2_BAR
    frac, ulps = bf16_mismatch(got, ref)
    assert frac <= FLIP_FRACTION_BAR and ulps <= 2.0, (frac, ulps)


def test_routed_reduce_several_tokens_with_a_shared_expert(fk):
    """tokens > 1 with a shared expert: its rows go through the multi-row matmul, T(dot) per token, and enter
    the ordered sum after the routes (workspace sized by fk_routed_reduce_workspace_bytes_shared)."""
    E, O, K, SK, tokens, top_k = 8, 256, 192, 384, 5, 3
    Wd, Ws = _stack(2600, E, O, K, 4), make_qweight(2700, O, SK, 4)
    h = normal_bf16(50, (tokens * top_k, K), 0.0, 0.5)
    expert_idx = rng(51).integers(0, E, tokens * top_k).astype(np.uint32)
    rw = normal_bf16(52, tokens * top_k, 0.2, 0.3)
    sx, res = normal_bf16(53, (tokens, SK)), normal_bf16(54, (tokens, O))
    out = fk.DeviceBuffer(2 * tokens * O)
    ws = fk.DeviceBuffer(fk.routed_reduce_workspace_bytes(tokens, top_k, O, SK, 64))
    fk.routed_qmv_reduce(_dev(fk, h), tokens * top_k, to_device(fk, Wd), E, None, _dev(fk, expert_idx), _dev(fk, rw), _dev(fk, sx),
                         to_device(fk, Ws), _dev(fk, res), tokens, top_k, out, ws)
    got = out.to_numpy(np.uint16, (tokens, O))
    assert rel_l2(got, _m2_fp32(h, Wd, expert_idx, rw, sx, Ws, res, tokens, top_k)) <= REL_L2_BAR
    ref = np.stack([oracle.routed_qmv_reduce(h[t * top_k:(t + 1) * top_k], Wd, expert_idx[t * top_k:(t + 1) * top_k],
                                             rw[t * top_k:(t + 1) * top_k], res[t:t + 1], 1, top_k, shared_x=sx[t:t + 1], Wshared=Ws)[0]
                    for t in range(tokens)])
    frac, ulps = bf16_mismatch(got, ref)
    assert frac <= FLIP_FRACTION_BAR and ulps <= 2.0, (frac, ulps)


def test_routed_reduce_tokens_and_row_idx(fk):
    E, O, K, tokens, top_k = 4, 192, 256, 3, 2
    Wd = _stack(700, E, O, K, 4)
    h = normal_bf16(11, (tokens * top_k, K), 0.0, 0.5)
    expert_idx = rng(12).integers(0, E, tokens * top_k).astype(np.uint32)
    row_idx = rng(13).permutation(tokens * top_k).astype(np.uint32)
    rw = normal_bf16(14, tokens * top_k, 0.3, 0.2)
    res = normal_bf16(15, (tokens, O))
    got = _run_m2(fk, h, Wd, row_idx, expert_idx, rw, None, None, res, tokens, top_k)
    ref = oracle.routed_qmv_reduce(h, Wd, expert_idx, rw, res, tokens, top_k, row_idx=row_idx)
    frac, ulps = bf16_mismatch(got, ref)
    assert frac <= FLIP_FRACTION_BAR and ulps <= 2.0, (frac, ulps)


def test_routes_served_in_expert_order_give_the_same_bits(fk):
    """Several tokens whose routes share experts (config-5 widths, 8 tokens x top-6 over 16 experts): fk_route_order
    is numpy's stable sort by (clamped) expert, and the routed launches served in that order -- an expert's slice
    then comes from HBM once -- give the listed order's results (to rounding-edge flips: the tiles differ) and the
    oracle's, for M1 and for M2 with a shared expert and a residual.  The launches that rank the routes themselves
    (no order array) give the bits of the launches that read the array."""
    E, O, K, tokens, top_k = 16, 1408, 2048, 8, 6
    routes = tokens * top_k
    Wg, Wu, Wd = _stack(3100, E, O, K, 4), _stack(3200, E, O, K, 4), _stack(3300, E, K, O, 4)
    Ws = make_qweight(3400, K, 2816, 4)
    x = normal_bf16(60, (tokens, K))
    expert_idx = rng(61).integers(0, E, routes).astype(np.uint32)
    expert_idx[5] = 4000                                       # clamps to E - 1, and sorts as E - 1
    row_idx = np.repeat(np.arange(tokens, dtype=np.uint32), top_k)
    rw = normal_bf16(62, routes, 0.2, 0.2)
    d_e, order = _dev(fk, expert_idx), fk.zeros(4 * routes)
    fk.route_order(d_e, routes, E, order)
    fk.sync()
    want_order = np.argsort(np.minimum(expert_idx, E - 1), kind="stable").astype(np.uint32)
    assert np.array_equal(order.to_numpy(np.uint32), want_order)
    dWg, dWu, dWd, dWs = (to_device(fk, W) for W in (Wg, Wu, Wd, Ws))
    dx, dr, dw = _dev(fk, x), _dev(fk, row_idx), _dev(fk, rw)
    h0, h1 = fk.DeviceBuffer(2 * routes * O), fk.DeviceBuffer(2 * routes * O)
    fk.routed_qmv_swiglu(dx, tokens, dWg, dWu, E, dr, d_e, None, routes, h0)
    fk.routed_qmv_swiglu_ordered(dx, tokens, dWg, dWu, E, dr, d_e, None, routes, order, h1)
    fk.sync()
    a, b = h0.to_numpy(np.uint16, (routes, O)), h1.to_numpy(np.uint16, (routes, O))
    # same chunks, same products; the tile geometry follows the blocks a route gets (a multiple of eight when
    # served in order), and with it the order in which a row's partial sums are added: rounding-edge flips only
    frac, ulps = bf16_mismatch(b, a)
    print("ordered against listed: %.4f of the outputs differ, by at most %.1f ulp" % (frac, ulps))
    assert frac <= FLIP_FRACTION_BAR, (frac, ulps)
    ref = oracle.routed_qmv_swiglu(x, Wg, Wu, row_idx, expert_idx, None)
    for r in range(routes):
        e = min(int(expert_idx[r]), E - 1)
        _check_swiglu(b[r], ref[r], x[row_idx[r]], Wg.expert(e), Wu.expert(e), 1)
    sx, res = normal_bf16(63, (tokens, 2816)), normal_bf16(64, (tokens, K))
    outs = []
    for ordered in (False, True):
        out = fk.DeviceBuffer(2 * tokens * K)
        ws = fk.DeviceBuffer(fk.routed_reduce_workspace_bytes(tokens, top_k, K, 2816, 64))
        args = (h0, routes, dWd, E, None, d_e, dw, _dev(fk, sx), dWs, _dev(fk, res), tokens, top_k)
        if ordered:
            fk.routed_qmv_reduce_ordered(*args, order, out, ws)
        else:
            fk.routed_qmv_reduce(*args, out, ws)
        fk.sync()
        outs.append(out.to_numpy(np.uint16, (tokens, K)))
    frac, ulps = bf16_mismatch(outs[1], outs[0])
    assert frac <= FLIP_FRACTION_BAR, (frac, ulps)
    ref2 = np.stack([oracle.routed_qmv_reduce(a[t * top_k:(t + 1) * top_k], Wd, expert_idx[t * top_k:(t + 1) * top_k],
                                              rw[t * top_k:(t + 1) * top_k], res[t:t + 1], 1, top_k, shared_x=sx[t:t + 1], Wshared=Ws)[0]
                     for t in range(tokens)])
    frac, ulps = bf16_mismatch(outs[1], ref2)
    assert frac <= FLIP_FRACTION_BAR and ulps <= 2.0, (frac, ulps)
    # without an order array (up to 64 routes) every wave of the launch ranks the routes itself: the same order,
    # the same grid, hence the same bits as with the array
    h2 = fk.DeviceBuffer(2 * routes * O)
    fk.routed_qmv_swiglu_ordered(dx, tokens, dWg, dWu, E, dr, d_e, None, routes, None, h2)
    out2 = fk.DeviceBuffer(2 * tokens * K)
    ws2 = fk.DeviceBuffer(fk.routed_reduce_workspace_bytes(tokens, top_k, K, 2816, 64))
    fk.routed_qmv_reduce_ordered(h0, routes, dWd, E, None, d_e, dw, _dev(fk, sx), dWs, _dev(fk, res), tokens, top_k, None, out2, ws2)
    fk.sync()
    assert np.array_equal(h2.to_numpy(np.uint16, (routes, O)), b)
    assert np.array_equal(out2.to_numpy(np.uint16, (tokens, K)), outs[1])
    # more than 64 routes need the array
    many = 66
    with pytest.raises(fk.FusekitError):
        fk.routed_qmv_swiglu_ordered(dx, tokens, dWg, dWu, E, _dev(fk, np.zeros(many, np.uint32)), _dev(fk, np.zeros(many, np.uint32)),
                                     None, many, None, fk.DeviceBuffer(2 * many * O))


def test_moe_block_full_size(fk):
    """Config-5 shapes (hidden 2048, expert width 1408, 6 of 16 experts, int4): M1 feeds M2."""
    E, hidden, inter, top_k = 16, 2048, 1408, 6
    Wg, Wu, Wd = _stack(800, E, inter, hidden, 4), _stack(900, E, inter, hidden, 4), _stack(1000, E, hidden, inter, 4)
    x = normal_bf16(16, (1, hidden))
    expert_idx = rng(17).permutation(E)[:top_k].astype(np.uint32)
    row_idx = np.zeros(top_k, np.uint32)
    rw = oracle.f32_to_bf16(np.full(top_k, 1.0 / top_k, np.float32))
    res = normal_bf16(18, (1, hidden))
    h = _run_m1(fk, x, Wg, Wu, row_idx, expert_idx, None)
    h_ref = oracle.routed_qmv_swiglu(x, Wg, Wu, row_idx, expert_idx, None)
    frac, ulps = bf16_mismatch(h, h_ref)
    assert frac <= FLIP_FRACTION_BAR, frac
    got = _run_m2(fk, h, Wd, None, expert_idx, rw, None, None, res, 1, top_k)   # on the GPU's own h
    ref = oracle.routed_qmv_reduce(h, Wd, expert_idx, rw, res, 1, top_k)
    frac, ulps = bf16_mismatch(got, ref)
    assert frac <= FLIP_FRACTION_BAR and ulps <= 2.0, (frac, ulps)


def test_routed_rejects_bad_arguments(fk):
    Wg, Wu = _stack(1100, 2, 64, 128, 4), _stack(1200, 2, 64, 128, 4)
    x = _dev(fk, normal_bf16(1, (1, 128)))
    idx = _dev(fk, np.zeros(2, np.uint32))
    out = fk.DeviceBuffer(2 * 2 * 64)
    with pytest.raises(fk.InvalidArgument):
        fk.routed_qmv_swiglu(x, 1, to_device(fk, Wg), to_device(fk, Wu), 2, idx, None, None, 2, out)
    with pytest.raises(fk.InvalidArgument):
        fk.routed_qmv_swiglu(x, 1, to_device(fk, Wg), to_device(fk, Wu), 0, idx, idx, None, 2, out)
    with pytest.raises(fk.InvalidArgument):
        fk.routed_qmv_reduce(x, 1, to_device(fk, Wg), 2, None, idx, None, x, None, None, 1, 2, out, out)


def test_routed_families_in_a_graph(fk):
    """The dispatcher families (reference buffer order) give the direct calls' bytes, replay after replay."""
    from fusekit_amd.runtime import Dispatch, Dispatcher, arg
    E, hidden, inter, top_k = 8, 256, 192, 4
    Wg, Wu, Wd = _stack(1300, E, inter, hidden, 4), _stack(1400, E, inter, hidden, 4), _stack(1500, E, hidden, inter, 4)
    Ws = make_qweight(1600, hidden, 128, 4)
    x, sx, res = normal_bf16(20, (1, hidden)), normal_bf16(21, (1, 128)), normal_bf16(22, (1, hidden))
    eidx, rw = np.array([3, 0, 7, 5], np.uint32), normal_bf16(23, top_k, 0.25, 0.1)
    h_direct = _run_m1(fk, x, Wg, Wu, np.zeros(top_k, np.uint32), eidx, None)
    out_direct = _run_m2(fk, h_direct, Wd, None, eidx, rw, sx, Ws, res, 1, top_k)

    dWg, dWu, dWd, dWs = (to_device(fk, w) for w in (Wg, Wu, Wd, Ws))
    bx, bsx, bres, beidx, brw = (_dev(fk, a) for a in (x, sx, res, eidx, rw))
    rows0, rows = _dev(fk, np.zeros(top_k, np.uint32)), _dev(fk, np.arange(top_k, dtype=np.uint32))
    h, out = fk.DeviceBuffer(2 * top_k * inter), fk.DeviceBuffer(2 * hidden)
    ws = fk.DeviceBuffer(fk.routed_reduce_workspace_bytes(1, top_k, hidden))
    common = {"bits": 4, "group": 64, "experts": E}
    tasks = [
        Dispatch("fusekit_routed_qmv_swiglu_f1",
                 [arg(bx), arg(dWg.w), arg(dWg.scales), arg(dWg.biases), arg(dWu.w), arg(dWu.scales), arg(dWu.biases),
                  arg(rows0), arg(beidx), arg(h)], dict(common, k=hidden, o=inter, routes=top_k, x_rows=1)),
        Dispatch("fusekit_routed_qmv_reduce_f2",
                 [arg(h), arg(dWd.w), arg(dWd.scales), arg(dWd.biases), arg(rows), arg(beidx), arg(brw),
                  arg(bsx), arg(dWs.w), arg(dWs.scales), arg(dWs.biases), arg(bres), arg(out), arg(ws)],
                 dict(common, k=inter, o=hidden, tokens=1, top_k=top_k, x_rows=top_k, has_shared=1, shared_k=128,
                      has_extra=1)),
    ]
    d = Dispatcher()
    g = d.build_graph(tasks)
    assert d.node_deps(g, 1) == [0]
    for _ in range(3):
        fk.fill_u32(out, 0, hidden // 2)
        fk.sync()
        d.execute_graph(g)
        assert np.array_equal(h.to_numpy(np.uint16, (top_k, inter)), h_direct)
        assert np.array_equal(out.to_numpy(np.uint16, (1, hidden)), out_direct)
