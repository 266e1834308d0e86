"""Pins the CPU oracle (oracle/fk_oracle.c) without any GPU: every function is checked against
something the mathematics fixes -- closed forms, invariants, brute force on tiny inputs, or an
independent numpy formulation (float64 library matmul / softmax) -- chosen so that a dropped
term, a wrong sign, a transposed operand or a wrong nibble order fails.  The reference holds no
golden vectors for this path (its 39 unit tests are structural), so these are the pins."""
import numpy as np
import pytest

import oracle
from helpers import make_qweight, normal_bf16, rng


# ---------------------------------------------------------------- independent bf16 in numpy
def np_bf16_round(x):
    """fp32 -> bf16 (round to nearest even) -> fp32, by integer arithmetic on the bits."""
    u = np.asarray(x, dtype=np.float32).view(np.uint32).astype(np.uint64)
    u = (u + 0x7FFF + ((u >> 16) & 1)) & 0xFFFF0000
    return u.astype(np.uint32).view(np.float32)


def test_bf16_round_to_nearest_even_and_specials():
    cases = {1.0: 0x3F80, 1.00390625: 0x3F80,  # 1 + 2^-8: tie -> even (down)
             1.01171875: 0x3F82,               # 1 + 3*2^-8: tie -> even (up)
             1.0 + 2 ** -8 + 2 ** -20: 0x3F81, -2.5: 0xC020, 0.0: 0x0000, float("inf"): 0x7F80}
    for v, bits in cases.items():
        assert int(oracle.f32_to_bf16(np.array([v], np.float32))[0]) == bits
    nan = oracle.f32_to_bf16(np.array([np.nan], np.float32))[0]
    assert (nan & 0x7F80) == 0x7F80 and (nan & 0x7F) != 0
    x = rng(0).standard_normal(10000).astype(np.float32) * 100
    assert np.array_equal(oracle.bf16_to_f32(oracle.f32_to_bf16(x)), np_bf16_round(x))


# ---------------------------------------------------------------- packing (bit-exact)
@pytest.mark.parametrize("bits", [4, 8])
def test_unpack_every_value_in_every_lane(bits):
    per, top = 32 // bits, (1 << bits)
    for lane in range(per):
        words = (np.arange(top, dtype=np.uint32) << np.uint32(lane * bits)).reshape(top, 1)
        W = oracle.QWeight(np.ascontiguousarray(words), np.zeros((top, 1), np.uint16), np.zeros((top, 1), np.uint16),
                           top, per, bits, per)
        codes = oracle.unpack_codes(W)
        expect = np.zeros((top, per), np.uint8)
        expect[:, lane] = np.arange(top)
        assert np.array_equal(codes, expect)  # value v sits at bits [lane*bits, (lane+1)*bits): LSB first


@pytest.mark.parametrize("bits", [4, 8])
def test_pack_roundtrip_against_numpy_shifts(bits):
    per = 32 // bits
    W = make_qweight(1, 33, 256, bits)
    shifts = (np.arange(per, dtype=np.uint32) * bits)
    ref = ((W.w[..., None] >> shifts) & ((1 << bits) - 1)).reshape(33, 256).astype(np.uint8)
    codes = oracle.unpack_codes(W)
    assert np.array_equal(codes, ref)
    repack = (codes.reshape(33, -1, per).astype(np.uint32) << shifts).sum(axis=2, dtype=np.uint32)
    assert np.array_equal(repack, W.w)


# ---------------------------------------------------------------- quantiser
def np_quantize_group(x, bits):
    """The quantiser formula written independently, one group, float32 numpy scalars."""
    f = np.float32
    mask = f((1 << bits) - 1)
    vmin, vmax = f(x.min()), f(x.max())
    scale_abs = max(f((vmax - vmin) / mask), f(1e-7))
    lo = abs(vmin) > abs(vmax)
    scale, edge = (scale_abs, vmin) if lo else (f(-scale_abs), vmax)
    q0 = np.round(f(edge / scale))  # ties do not occur on the test data (np.round is half-even)
    if q0 != 0:
        scale, bias = f(edge / q0), edge
    else:
        bias = f(0)
    inv = f(1) / scale if scale != 0 else f(0)
    q = np.clip(np.floor(np.abs((x - bias) * inv) + f(0.5)) * np.sign((x - bias) * inv), 0, mask)
    return q.astype(np.uint8), scale, bias


@pytest.mark.parametrize("bits,group", [(4, 64), (8, 64), (4, 32), (4, 128)])
def test_quantizer_matches_independent_formula_and_invariants(bits, group):
    n, k = 24, 4 * group
    w = (rng(bits * 1000 + group).standard_normal((n, k), dtype=np.float32) * 0.02).astype(np.float32)
    Q = oracle.quantize(w, bits, group)
    codes = oracle.unpack_codes(Q)
    assert codes.max() <= (1 << bits) - 1
    deq = oracle.dequantize(Q)
    for r in range(n):
        for g in range(k // group):
            x = w[r, g * group:(g + 1) * group]
            q, s, b = np_quantize_group(x, bits)
            assert np.array_equal(codes[r, g * group:(g + 1) * group], q)
            assert Q.scales[r, g] == oracle.f32_to_bf16(np.array([s]))[0]
            assert Q.biases[r, g] == oracle.f32_to_bf16(np.array([b]))[0]
            # reconstruction error: half a step, plus the shortfall at the far edge when the
            # scale is re-derived as edge / q0 (|q0| >= mask/2, so at most ~one step), plus
            # the bf16 rounding of scale and bias
            lim = 1.6 * abs(s) + ((1 << bits) - 1) * abs(s) * 2.0 ** -8 + abs(b) * 2.0 ** -8
            assert np.all(np.abs(deq[r, g * group:(g + 1) * group] - x) <= lim * 1.001)


def test_quantizer_closed_forms():
    s = np.float32(2.0 ** -6)
    q = np.tile(np.arange(16, dtype=np.float32), 4)
    lo = (q - 8) * s                  # range [-8s, 7s]: low edge has the larger magnitude
    hi = (8 - q) * s                  # range [-7s, 8s]: high edge has the larger magnitude
    const = np.full(64, 0.25, np.float32)
    zero = np.zeros(64, np.float32)
    Q = oracle.quantize(np.stack([lo, hi, const, zero]), 4, 64)
    codes = oracle.unpack_codes(Q)
    sc, bi = oracle.bf16_to_f32(Q.scales)[:, 0], oracle.bf16_to_f32(Q.biases)[:, 0]
    assert np.array_equal(codes[0], q) and sc[0] == s and bi[0] == -8 * s
    assert np.array_equal(codes[1], q) and sc[1] == -s and bi[1] == 8 * s        # scale takes the sign
    assert np.array_equal(oracle.dequantize(Q)[:2], np.stack([lo, hi]))          # both reconstruct exactly
    assert not codes[2].any() and bi[2] == 0.25 and abs(sc[2]) < 2e-7            # constant group: 1e-7 clamp
    assert not codes[3].any() and bi[3] == 0.0                                   # all zero: q0 == 0 branch


# ---------------------------------------------------------------- linear / qgemv
@pytest.mark.parametrize("bits", [4, 8, 16])
def test_qgemv_is_matmul_on_dequantized_weights(bits):
    n, k = 77, 320
    W = make_qweight(3, n, k, bits)
    x = normal_bf16(4, k)
    xf = oracle.bf16_to_f32(x).astype(np.float64)
    ref = oracle.dequantize(W).astype(np.float64) @ xf            # library matmul, float64
    acc = oracle.linear_acc(W, x)
    assert np.allclose(acc, ref, rtol=1e-6, atol=1e-7)
    y = oracle.bf16_to_f32(oracle.qgemv(W, x))
    assert np.array_equal(y, np_bf16_round(acc))                  # exactly one final rounding
    if bits != 16:
        # algebraic identity: sum x (q s + b) = s sum(x q) + b sum(x), per group
        q = oracle.unpack_codes(W).astype(np.float64).reshape(n, -1, 64)
        s, b = oracle.bf16_to_f32(W.scales).astype(np.float64), oracle.bf16_to_f32(W.biases).astype(np.float64)
        xg = xf.reshape(-1, 64)
        alt = (s * (q * xg).sum(-1) + b * xg.sum(-1)).sum(-1)
        assert np.allclose(acc, alt, rtol=1e-6, atol=1e-7)
    # transposed-operand / wrong-row mistakes: a one-hot x selects one dequantised column
    e = np.zeros(k, np.float32); e[37] = 1.0
    assert np.allclose(oracle.linear_acc(W, oracle.f32_to_bf16(e)), oracle.dequantize(W)[:, 37])


def test_bias_and_residual_rounding_order():
    n, k = 40, 128
    W = make_qweight(5, n, k)
    x, b, r1, r2 = normal_bf16(1, k), normal_bf16(2, n), normal_bf16(3, n), normal_bf16(4, n)
    acc = oracle.linear_acc(W, x)
    f = oracle.bf16_to_f32
    assert np.array_equal(f(oracle.qgemv(W, x, b)), np_bf16_round(acc + f(b)))            # bias before the round
    y1 = np_bf16_round(acc + f(r1))
    assert np.array_equal(f(oracle.linear_residual(W, x, r1)), y1)
    assert np.array_equal(f(oracle.linear_residual(W, x, r1, r2)), np_bf16_round(y1 + f(r2)))  # rounds twice


# ---------------------------------------------------------------- rms norm
def test_rmsnorm_closed_forms_and_rounding_boundaries():
    h, eps = 64, 1e-6
    one = np.full(h, 0x3F80, np.uint16)
    r = np.float32(1.0) / np.sqrt(np.float32(1.0) + np.float32(eps))
    assert np.array_equal(oracle.bf16_to_f32(oracle.rmsnorm(one, one, eps)), np.full(h, np_bf16_round(r)))
    spike = np.zeros(h, np.float32); spike[5] = 8.0
    out = oracle.bf16_to_f32(oracle.rmsnorm(oracle.f32_to_bf16(spike), one, eps))
    assert out[5] == np_bf16_round(np.float32(8.0) / np.sqrt(np.float32(64.0 / h + eps))) and not np.delete(out, 5).any()
    # general case against the formula with the two roundings, T(w * T(x * r)), written in numpy
    x, w = normal_bf16(1, 896, 3.0), normal_bf16(2, 896, 0.1, 1.0)
    xf, wf = oracle.bf16_to_f32(x), oracle.bf16_to_f32(w)
    rr = np.float32(1.0) / np.sqrt(np.float32((xf.astype(np.float64) ** 2).sum()) / np.float32(896) + np.float32(eps))
    ref = np_bf16_round(wf * np_bf16_round(xf * rr))
    assert np.array_equal(oracle.bf16_to_f32(oracle.rmsnorm(x, w, eps)), ref)
    single = np_bf16_round(wf * xf * rr)                      # a single rounding is a different function
    assert not np.array_equal(single, ref)


# ---------------------------------------------------------------- rope
def test_rope_invariants():
    H, D = 4, 128
    q = normal_bf16(1, H * D)
    assert np.array_equal(oracle.rope_q(q, H, D, D, 1e6, 0), q)                        # position 0: identity
    f = lambda a: oracle.bf16_to_f32(a).astype(np.float64).reshape(H, D)
    r = f(oracle.rope_q(q, H, D, D, 1e6, 1234))
    n0 = f(q)[:, :64] ** 2 + f(q)[:, 64:] ** 2                                         # pair (d, d + D/2)
    n1 = r[:, :64] ** 2 + r[:, 64:] ** 2
    assert np.allclose(n0, n1, rtol=2e-2, atol=1e-4)                                   # rotation preserves pair norms
    # explicit formula in float64
    d = np.arange(64)
    ang = 1234 * np.exp2(-(d / 64.0) * np.log2(1e6))
    lo, hi = f(q)[:, :64], f(q)[:, 64:]
    ref = np.concatenate([lo * np.cos(ang) - hi * np.sin(ang), hi * np.cos(ang) + lo * np.sin(ang)], axis=1)
    assert np.allclose(r, ref, rtol=2 ** -7, atol=2e-3)
    # composition: R(a) R(b) = R(a + b) up to the intermediate bf16 rounding
    ab = f(oracle.rope_q(oracle.rope_q(q, H, D, D, 1e6, 300), H, D, D, 1e6, 500))
    assert np.allclose(ab, f(oracle.rope_q(q, H, D, D, 1e6, 800)), rtol=3e-2, atol=3e-2)
    # partial rotation leaves the tail untouched
    part = oracle.rope_q(q, H, D, 64, 1e6, 77).reshape(H, D)
    assert np.array_equal(part[:, 64:], q.reshape(H, D)[:, 64:]) and not np.array_equal(part[:, :64], q.reshape(H, D)[:, :64])


def test_kv_store_addressing_and_headnorm():
    n_kv, D, cap = 2, 64, 8
    k, v = normal_bf16(1, n_kv * D), normal_bf16(2, n_kv * D)
    ck, cv = np.zeros(n_kv * cap * D, np.uint16), np.zeros(n_kv * cap * D, np.uint16)
    oracle.rope_kv_store(k, v, n_kv, D, D, 1e6, 11, 11, cap, ck, cv)                  # row 11 % 8 = 3
    ck, cv = ck.reshape(n_kv, cap, D), cv.reshape(n_kv, cap, D)
    assert np.array_equal(cv[:, 3], v.reshape(n_kv, D)) and not np.delete(cv, 3, axis=1).any()
    assert np.array_equal(ck[:, 3].ravel(), oracle.rope_q(k, n_kv, D, D, 1e6, 11)) and not np.delete(ck, 3, axis=1).any()
    w = normal_bf16(3, D, 0.1, 1.0)
    hn = oracle.headnorm_rope(k, w, n_kv, D, D, 1e-6, 1e6, 0)                         # pos 0: norm only
    assert np.array_equal(hn.reshape(n_kv, D)[1], oracle.rmsnorm(k.reshape(n_kv, D)[1].copy(), w, 1e-6))


# ---------------------------------------------------------------- swiglu
def test_swiglu_variants():
    g = rng(1).standard_normal(2000).astype(np.float32) * 3
    u = rng(2).standard_normal(2000).astype(np.float32) * 2
    exact = (np_bf16_round(g).astype(np.float64) / (1 + np.exp(-np_bf16_round(g).astype(np.float64)))) * np_bf16_round(u)
    R = np_bf16_round
    gb, ub = R(g), R(u)
    sig_y = R(np.float32(1) / R(np.float32(1) + R(np.exp(np.abs(gb)))))
    sigA = np.where(gb < 0, sig_y, R(np.float32(1) - sig_y))
    refA = R(R(gb * sigA) * ub)
    sig = (np.float32(1) / (np.float32(1) + np.exp(-gb))).astype(np.float32)
    refB = R((sig * gb) * ub)
    refC = R(R(R(sig) * gb) * ub)
    for variant, ref in ((0, refA), (1, refB), (2, refC)):
        got = oracle.bf16_to_f32(np.array([oracle.swiglu_scalar(float(a), float(b), variant) for a, b in zip(g, u)],
                                          dtype=np.uint16))
        # libm expf and numpy exp may differ in the last fp32 bit, which can move a bf16 rounding edge
        assert np.mean(got != ref) < 0.01 and np.allclose(got, ref, rtol=2 ** -6, atol=1e-6)
        assert np.allclose(got, exact, rtol=3 * 2 ** -7, atol=1e-3)       # all three are silu(g) * u in bf16
    assert oracle.swiglu_scalar(0.0, 5.0, 0) in (0x0000, 0x8000) and oracle.swiglu_scalar(-100.0, 1.0, 1) in (0x0000, 0x8000)


# ---------------------------------------------------------------- sdpa
def test_sdpa_against_float64_attention_and_gqa_mapping():
    n_heads, n_kv, D, L, cap = 6, 2, 64, 37, 64
    q = normal_bf16(1, n_heads * D)
    ck, cv = normal_bf16(2, n_kv * cap * D), normal_bf16(3, n_kv * cap * D)
    out = oracle.bf16_to_f32(oracle.sdpa_decode(q, ck, cv, n_heads, n_kv, D, D, L, cap, D ** -0.5)).reshape(n_heads, D)
    f = lambda a: oracle.bf16_to_f32(a).astype(np.float64)
    K, V, Q = f(ck).reshape(n_kv, cap, D)[:, :L], f(cv).reshape(n_kv, cap, D)[:, :L], f(q).reshape(n_heads, D)
    for h in range(n_heads):
        kvh = h // (n_heads // n_kv)                              # GQA: consecutive heads share a kv head
        s = K[kvh] @ Q[h] * D ** -0.5
        p = np.exp(s - s.max()); p /= p.sum()
        assert np.allclose(out[h], p @ V[kvh], rtol=2 ** -7, atol=2e-3)
    # kv_len = 1: softmax of one score is 1 -> output is v_0 of the head's kv head, bit for bit
    one = oracle.sdpa_decode(q, ck, cv, n_heads, n_kv, D, D, 1, cap, D ** -0.5).reshape(n_heads, D)
    v0 = cv.reshape(n_kv, cap, D)[:, 0]
    assert np.array_equal(one, np.repeat(v0, n_heads // n_kv, axis=0))
    # rows at or beyond kv_len are ignored
    cv2 = cv.copy().reshape(n_kv, cap, D); cv2[:, L:] = 0x7FC0
    assert np.array_equal(oracle.sdpa_decode(q, ck, cv2.ravel(), n_heads, n_kv, D, D, L, cap, D ** -0.5).reshape(n_heads, D),
                          oracle.f32_to_bf16(out))


def test_sdpa_prefill_rows_are_causal_decode_attention():
    n_heads, n_kv, D, cap = 6, 2, 64, 96
    f = lambda a: oracle.bf16_to_f32(a).astype(np.float64)
    for rows, kv_len in ((1, 1), (5, 5), (7, 40), (33, 70)):
        q = normal_bf16(10 + rows, rows * n_heads * D)
        ck, cv = normal_bf16(2, n_kv * cap * D), normal_bf16(3, n_kv * cap * D)
        got = oracle.sdpa_prefill(q, ck, cv, rows, n_heads, n_kv, D, kv_len, cap, D ** -0.5).reshape(rows, n_heads, D)
        K, V, Q = f(ck).reshape(n_kv, cap, D), f(cv).reshape(n_kv, cap, D), f(q).reshape(rows, n_heads, D)
        for r in range(rows):
            sees = kv_len - rows + r + 1                          # sdpa_prefill.rs:95: q_kv = (kv_len - L) + l_q, kv <= q_kv
            # the pinned single-row attention over exactly those positions; the two differ only in where
            # the division by the sum of exponentials happens -> at most one bf16 step apart
            dec = oracle.sdpa_decode(q.reshape(rows, -1)[r], ck, cv, n_heads, n_kv, D, D, sees, cap, D ** -0.5).reshape(n_heads, D)
            a, b = oracle.bf16_to_f32(got[r]), oracle.bf16_to_f32(dec)
            assert np.mean(got[r] != dec) < 0.02 and np.allclose(a, b, rtol=2 ** -7, atol=1e-6)
            for h in range(n_heads):                              # and an independent float64 statement
                kvh = h // (n_heads // n_kv)
                s = K[kvh, :sees] @ Q[r, h] * D ** -0.5
                p = np.exp(s - s.max()); p /= p.sum()
                assert np.allclose(a[h], p @ V[kvh, :sees], rtol=2 ** -7, atol=2e-3)
        if kv_len == rows:                                        # a fresh group: row 0 sees one position -> v_0 bit for bit
            assert np.array_equal(got[0], np.repeat(cv.reshape(n_kv, cap, D)[:, 0], n_heads // n_kv, axis=0))
        # positions after a row's own never reach it: poison everything row r must not see
        r = rows // 2
        sees = kv_len - rows + r + 1
        ck2, cv2 = ck.copy().reshape(n_kv, cap, D), cv.copy().reshape(n_kv, cap, D)
        ck2[:, sees:] = 0x7FC0; cv2[:, sees:] = 0x7FC0
        poisoned = oracle.sdpa_prefill(q, ck2.ravel(), cv2.ravel(), rows, n_heads, n_kv, D, kv_len, cap, D ** -0.5)
        assert np.array_equal(poisoned.reshape(rows, n_heads, D)[: r + 1], got[: r + 1])
    # identical keys: uniform probabilities, the output is the mean of the visible V rows
    rows, kv_len = 4, 9
    q = normal_bf16(5, rows * n_heads * D)
    ck = np.tile(normal_bf16(6, D), n_kv * cap)
    cv = normal_bf16(7, n_kv * cap * D)
    got = oracle.bf16_to_f32(oracle.sdpa_prefill(q, ck, cv, rows, n_heads, n_kv, D, kv_len, cap, D ** -0.5)).reshape(rows, n_heads, D)
    V = f(cv).reshape(n_kv, cap, D)
    for r in range(rows):
        sees = kv_len - rows + r + 1
        for h in range(n_heads):
            assert np.allclose(got[r, h], V[h // (n_heads // n_kv), :sees].mean(axis=0), rtol=2 ** -7, atol=2e-3)


# ---------------------------------------------------------------- embed / lm head / argmax
def test_embed_lm_head_argmax():
    E = make_qweight(1, 50, 128, 4)
    deq = oracle.dequantize(E)
    assert np.array_equal(oracle.bf16_to_f32(oracle.embed_lookup(E, 17, 1.0)), np_bf16_round(deq[17]))
    assert np.array_equal(oracle.bf16_to_f32(oracle.embed_lookup(E, 49, 11.3)), np_bf16_round(deq[49] * np.float32(11.3)))
    x, w = normal_bf16(2, 128), normal_bf16(3, 128, 0.1, 1.0)
    logits = oracle.final_rmsnorm_lm_head(x, w, 1e-6, E)
    assert np.array_equal(logits, oracle.qgemv(E, oracle.rmsnorm(x, w, 1e-6)))
    vals = np.array([1.0, 3.0, -2.0, 3.0, np.nan, 3.0], np.float32)
    assert oracle.argmax(oracle.f32_to_bf16(vals)) == 1                    # lowest index among ties, NaN never wins
    assert oracle.argmax(oracle.f32_to_bf16(np.array([-5.0, -1.0, -3.0], np.float32))) == 1
    assert oracle.top2_margin(oracle.f32_to_bf16(vals[:4])) == 0.0
    for seed in range(5):
        l = oracle.f32_to_bf16(rng(seed).standard_normal(999).astype(np.float32))
        f = oracle.bf16_to_f32(l)
        assert oracle.argmax(l) == int(np.flatnonzero(f == f.max())[0])


# ---------------------------------------------------------------- whole step = composition of the parts
def test_decoder_step_is_the_composition_of_its_parts():
    import ctypes as C
    hid, nh, nkv, D, inter, vocab, cap = 128, 4, 2, 32, 256, 300, 16
    u16p = C.POINTER(C.c_uint16)
    W = {n: make_qweight(10 + i, r, c) for i, (n, r, c) in enumerate(
        [("q", nh * D, hid), ("k", nkv * D, hid), ("v", nkv * D, hid), ("o", hid, nh * D),
         ("gate", inter, hid), ("up", inter, hid), ("down", hid, inter)])}
    emb = oracle.dense(normal_bf16(30, (vocab, hid), 0.02))
    n1, n2, nf = (normal_bf16(40 + i, hid, 0.1, 1.0) for i in range(3))
    qn, kn = normal_bf16(50, D, 0.1, 1.0), normal_bf16(51, D, 0.1, 1.0)
    bq = normal_bf16(52, nh * D, 0.5)
    ck, cv = np.zeros(nkv * cap * D, np.uint16), np.zeros(nkv * cap * D, np.uint16)
    p = lambda a: a.ctypes.data_as(u16p)
    null = C.cast(None, u16p)
    for use_norm in (False, True):
        ck[:] = 0; cv[:] = 0
        L = (oracle.Layer * 1)()
        L[0].input_norm, L[0].post_norm = p(n1), p(n2)
        L[0].wq, L[0].wk, L[0].wv, L[0].wo = W["q"].c, W["k"].c, W["v"].c, W["o"].c
        L[0].wgate, L[0].wup, L[0].wdown = W["gate"].c, W["up"].c, W["down"].c
        L[0].bq, L[0].bk, L[0].bv = p(bq), null, null
        L[0].q_norm, L[0].k_norm = (p(qn), p(kn)) if use_norm else (null, null)
        L[0].cache_k, L[0].cache_v = p(ck), p(cv)
        M = oracle.Model(1, hid, nh, nkv, D, inter, vocab, 1e-6, 1e6, D ** -0.5, 1.0, 0, cap, emb.c, emb.c, p(nf), L)
        logits = np.empty(vocab, np.uint16)
        tok, margin = oracle.decoder_step(M, 7, 0, logits)
        # the same step, composed by hand from the pinned parts
        x = oracle.embed_lookup(emb, 7, 1.0)
        q, k, v = oracle.rmsnorm_qkv(x, n1, 1e-6, W["q"], W["k"], W["v"], bq, None, None)
        ck2, cv2 = np.zeros_like(ck), np.zeros_like(cv)
        if use_norm:
            q = oracle.headnorm_rope(q, qn, nh, D, D, 1e-6, 1e6, 0)
            oracle.kv_store(oracle.headnorm_rope(k, kn, nkv, D, D, 1e-6, 1e6, 0), v, nkv, D, D, 0, cap, ck2, cv2)
        else:
            q = oracle.rope_q(q, nh, D, D, 1e6, 0)
            oracle.rope_kv_store(k, v, nkv, D, D, 1e6, 0, 0, cap, ck2, cv2)
        att = oracle.sdpa_decode(q, ck2, cv2, nh, nkv, D, D, 1, cap, D ** -0.5)
        x1 = oracle.linear_residual(W["o"], att, x)
        mid = oracle.gateup_swiglu(x1, n2, 1e-6, W["gate"], W["up"], 0)
        x2 = oracle.linear_residual(W["down"], mid, x1)
        ref = oracle.final_rmsnorm_lm_head(x2, nf, 1e-6, emb)
        assert np.array_equal(logits, ref) and tok == oracle.argmax(ref)
        assert np.array_equal(ck, ck2) and np.array_equal(cv, cv2)
        assert margin == pytest.approx(oracle.top2_margin(ref))


def test_routed_swiglu_is_the_dense_pair_on_the_selected_expert():
    """M1: route r must equal the pinned dense gate/up SwiGLU (variant B) run on expert
    min(expert_idx[r], E-1)'s slice and activation row row_idx[r]; the route weight scales the fp32
    product before the single round (powers of two make that exact)."""
    E, O, K = 5, 48, 128
    experts_g = [make_qweight(100 + e, O, K, 4) for e in range(E)]
    experts_u = [make_qweight(200 + e, O, K, 4) for e in range(E)]
    Wg, Wu = oracle.StackedWeight(experts_g), oracle.StackedWeight(experts_u)
    x = normal_bf16(1, (3, K))
    row_idx = np.array([2, 0, 1, 1], np.uint32)
    expert_idx = np.array([4, 0, 99, 3], np.uint32)           # 99 clamps to E-1 (routed_qmv_swiglu.rs:138)
    out = oracle.routed_qmv_swiglu(x, Wg, Wu, row_idx, expert_idx)
    for r in range(4):
        e = min(int(expert_idx[r]), E - 1)
        assert np.array_equal(out[r], oracle.gateup_swiglu(x[row_idx[r]], None, 0.0, experts_g[e], experts_u[e], 1))
    rw = oracle.f32_to_bf16(np.array([0.5, 2.0, 0.25, 1.0], np.float32))
    scaled = oracle.routed_qmv_swiglu(x, Wg, Wu, row_idx, expert_idx, rw)
    want = oracle.bf16_to_f32(out) * oracle.bf16_to_f32(rw)[:, None]
    assert np.array_equal(oracle.bf16_to_f32(scaled), want)
    # the stacked layout itself: expert e starts e * O rows into the [E * O, K/8] matrix
    flat = oracle.QWeight(Wg.w.reshape(E * O, -1), Wg.scales.reshape(E * O, -1), Wg.biases.reshape(E * O, -1), E * O, K, 4, 64)
    assert np.array_equal(oracle.dequantize(flat)[3 * O:4 * O], oracle.dequantize(experts_g[3]))


def test_routed_reduce_closed_forms():
    """M2: one route with weight 1 is the pinned qGEMV; the sum runs in slot order in fp32 over the
    ROUNDED per-route results times the route weight; the shared expert adds its rounded result last;
    the residual is added before the single final round."""
    E, O, K, top_k = 4, 40, 192, 3
    experts = [make_qweight(300 + e, O, K, 4) for e in range(E)]
    Wd = oracle.StackedWeight(experts)
    h = normal_bf16(2, (top_k, K), 0.0, 0.5)
    eidx = np.array([1, 3, 1], np.uint32)
    one = oracle.routed_qmv_reduce(h[:1], Wd, eidx[:1], None, None, 1, 1)
    assert np.array_equal(one[0], oracle.qgemv(experts[1], h[0]))
    rw = normal_bf16(3, top_k, 0.3, 0.2)
    res = normal_bf16(4, (1, O))
    shared_w, shared_x = make_qweight(400, O, 64, 4), normal_bf16(5, (1, 64))
    got = oracle.routed_qmv_reduce(h, Wd, eidx, rw, res, 1, top_k, shared_x=shared_x, Wshared=shared_w)
    acc = np.zeros(O, np.float32)
    for s in range(top_k):
        part = oracle.bf16_to_f32(oracle.qgemv(experts[int(eidx[s])], h[s]))          # T(dot), pinned
        acc = (acc + (oracle.bf16_to_f32(rw[s:s + 1])[0] * part).astype(np.float32)).astype(np.float32)
    acc = (acc + oracle.bf16_to_f32(oracle.qgemv(shared_w, shared_x[0]))).astype(np.float32)
    acc = (acc + oracle.bf16_to_f32(res[0])).astype(np.float32)
    assert np.array_equal(got[0], oracle.f32_to_bf16(acc))
    # pre-weighted input (route_weight absent) is weight 1; row_idx permutes the rows of h
    perm = np.array([2, 0, 1], np.uint32)
    a = oracle.routed_qmv_reduce(h, Wd, eidx, None, None, 1, top_k, row_idx=perm)
    b = oracle.routed_qmv_reduce(h[perm], Wd, eidx, None, None, 1, top_k)
    assert np.array_equal(a, b)
    # two tokens are two independent reductions
    h2 = normal_bf16(6, (2 * top_k, K), 0.0, 0.5)
    e2 = np.array([0, 1, 2, 3, 2, 1], np.uint32)
    both = oracle.routed_qmv_reduce(h2, Wd, e2, None, None, 2, top_k)
    assert np.array_equal(both[1], oracle.routed_qmv_reduce(h2[top_k:], Wd, e2[top_k:], None, None, 1, top_k)[0])


def test_qgemm_rows_are_qgemv():
    W = make_qweight(500, 72, 256, 8)
    x = normal_bf16(7, (4, 256))
    bias = normal_bf16(8, 72)
    y = oracle.qgemm(W, x, bias)
    for r in range(4):
        assert np.array_equal(y[r], oracle.qgemv(W, x[r], bias))


@pytest.mark.parametrize("bits", [4, 8])
def test_quantised_kv_store_and_attention(bits):
    """Quantised KV cache.  Store: V codes are the pinned quantiser applied to the V row; K without
    rotation likewise; with rotation the dequantised row stays within half a quantisation step of the
    fp32 rotation (which agrees with the pinned bf16 RoPE to one bf16 rounding); only the addressed
    row is written.  Attention: float64 softmax attention over the dequantised cache."""
    n_kv, dim, cap, group = 2, 128, 16, 64
    k, v = normal_bf16(1, n_kv * dim), normal_bf16(2, n_kv * dim)
    K, V = oracle.QuantCache(n_kv, cap, dim, bits, group), oracle.QuantCache(n_kv, cap, dim, bits, group)
    oracle.rope_kv_store_quant(k, v, None, n_kv, dim, 0, 1e4, 0.0, 21, 21, K, V)        # rope_dims 0: plain
    row = 21 % cap
    for h in range(n_kv):
        for src, cache in ((k, K), (v, V)):
            Q = oracle.quantize(oracle.bf16_to_f32(src[h * dim:(h + 1) * dim]).reshape(1, dim), bits, group)
            assert np.array_equal(cache.packed[h, row], Q.w[0]) and np.array_equal(cache.scales[h, row], Q.scales[0])
            assert np.array_equal(cache.biases[h, row], Q.biases[0])
    untouched = np.ones(cap, bool)
    untouched[row] = False
    assert not K.packed[:, untouched].any() and not V.scales[:, untouched].any()
    K2, V2 = oracle.QuantCache(n_kv, cap, dim, bits, group), oracle.QuantCache(n_kv, cap, dim, bits, group)
    oracle.rope_kv_store_quant(k, v, None, n_kv, dim, dim, 1e4, 0.0, 7, 3, K2, V2)      # rotate at pos 7, row 3
    ck, cv = np.zeros(n_kv * cap * dim, np.uint16), np.zeros(n_kv * cap * dim, np.uint16)
    oracle.rope_kv_store(k, v, n_kv, dim, dim, 1e4, 7, 3, cap, ck, cv)
    want = oracle.bf16_to_f32(ck).reshape(n_kv, cap, dim)[:, 3]
    got = K2.dequantize()[:, 3]
    step = np.abs(oracle.bf16_to_f32(K2.scales[:, 3])).repeat(group, axis=-1)
    # half a step inside the range; the edge opposite the anchor may fall short by up to ~1.6 steps
    # because the scale is re-derived from the anchor (same bound as the weight quantiser's pin)
    err = np.abs(got - want)
    assert np.all(err <= 1.6 * step + 2.0 ** -8 * np.abs(want) + 1e-6)
    assert np.mean(err / (step + 2.0 ** -7 * np.abs(want))) <= 0.3   # `want` itself carries one bf16 rounding
    # attention over a filled cache
    rs = rng(3)
    for c in (K, V):
        c.packed[:] = rs.integers(0, 2 ** 32, c.packed.shape, dtype=np.uint32)
        c.scales[:] = oracle.f32_to_bf16((rs.standard_normal(c.scales.shape) * 0.02 + 0.1).astype(np.float32))
        c.biases[:] = oracle.f32_to_bf16((rs.standard_normal(c.biases.shape) * 0.3).astype(np.float32))
    n_heads, kv_len, scale = 4, 11, 0.09
    q = normal_bf16(4, n_heads * dim)
    out = oracle.bf16_to_f32(oracle.sdpa_decode_quant(q, K, V, n_heads, kv_len, scale)).reshape(n_heads, dim)
    kd, vd = K.dequantize().astype(np.float64), V.dequantize().astype(np.float64)
    qf = oracle.bf16_to_f32(q).astype(np.float64).reshape(n_heads, dim)
    for h in range(n_heads):
        kvh = h // (n_heads // n_kv)
        sc = (kd[kvh, :kv_len] @ qf[h]) * scale
        p = np.exp(sc - sc.max())
        ref = (p / p.sum()) @ vd[kvh, :kv_len]
        assert np.all(np.abs(out[h] - ref) <= 2.0 ** -8 * np.abs(ref) + 1e-6)


@pytest.mark.parametrize("bits", [4, 8])
def test_qgemm_with_weights_rounded_to_bf16(bits):
    """Large-M form: w = T(s * q + b) per element, then a float64 matmul on those bf16 weights; a
    one-hot activation row returns the rounded weights themselves; the rounding is visible (the
    result differs from the exact-weight form on some outputs) and small (rel-L2 << 1e-2)."""
    n, k, m = 48, 256, 5
    W = make_qweight(90 + bits, n, k, bits)
    x = normal_bf16(91, (m, k))
    x[0] = 0
    x[0, 17] = 0x3F80                                    # one-hot row: 1.0 at k = 17
    y, acc = oracle.qgemm_bf16w(W, x, want_acc=True)
    wq = oracle.bf16_to_f32(oracle.f32_to_bf16(oracle.dequantize(W)))   # dequantise, then one bf16 rounding
    ref = oracle.bf16_to_f32(x).astype(np.float64) @ wq.astype(np.float64).T
    assert np.allclose(acc, ref, rtol=1e-6, atol=1e-6)
    assert np.array_equal(y, oracle.f32_to_bf16(acc))
    assert np.array_equal(y[0], oracle.f32_to_bf16(wq[:, 17].copy()))
    exact = oracle.qgemm(W, x)
    assert not np.array_equal(y, exact)
    fe = oracle.bf16_to_f32(exact).astype(np.float64)
    assert np.linalg.norm(oracle.bf16_to_f32(y) - fe) / np.linalg.norm(fe) < 5e-3
    bias = normal_bf16(92, n)
    yb = oracle.qgemm_bf16w(W, x, bias)
    assert np.array_equal(yb, oracle.f32_to_bf16(acc + oracle.bf16_to_f32(bias)))


# ---------------------------------------------------------------- MLA glue and the router
def _split_case(seed, n_kv, k0d, k1d, vd, k1_heads, packed):
    if packed:
        src = normal_bf16(seed, (n_kv, k0d + vd))
        k0, v, k0s, vs = src.reshape(-1), src.reshape(-1)[k0d:], k0d + vd, k0d + vd
        k0_rows, v_rows = src[:, :k0d], src[:, k0d:]
    else:
        k0_rows, v_rows = normal_bf16(seed, (n_kv, k0d)), normal_bf16(seed + 1, (n_kv, vd))
        k0, v, k0s, vs = k0_rows.reshape(-1), v_rows.reshape(-1), k0d, vd
    k1 = normal_bf16(seed + 2, (k1_heads, k1d))
    return k0, k0s, k0_rows, k1, v, vs, v_rows


@pytest.mark.parametrize("k1_heads,packed", [(1, True), (4, False), (1, False)])
def test_split_key_store_equals_rope_and_plain_store_on_the_assembled_row(k1_heads, packed):
    """Half-split pairs: [K0 | K1] with K1 rotated == the pinned rope + store applied to a key whose
    FIRST dims are K1 (the pinned function rotates the leading dims), after moving the parts back."""
    n_kv, k0d, k1d, vd, cap, pos, rope = 4, 32, 16, 24, 8, 13, 16
    k0, k0s, k0_rows, k1, v, vs, v_rows = _split_case(300, n_kv, k0d, k1d, vd, k1_heads, packed)
    ck, cv = np.zeros(n_kv * cap * (k0d + k1d), np.uint16), np.zeros(n_kv * cap * vd, np.uint16)
    oracle.kv_store_split(k0, k0s, k1, k1_heads, v, vs, n_kv, k0d, k1d, vd, rope, False, 1e4, pos, pos + cap, cap, ck, cv)
    k1_rows = np.repeat(k1, n_kv, 0) if k1_heads == 1 else k1
    rot = oracle.rope_q(k1_rows.reshape(-1), n_kv, k1d, rope, 1e4, pos).reshape(n_kv, k1d)
    want_k = np.concatenate([k0_rows, rot], 1)
    got_k = ck.reshape(n_kv, cap, k0d + k1d)
    assert np.array_equal(got_k[:, pos % cap], want_k)
    assert np.array_equal(cv.reshape(n_kv, cap, vd)[:, pos % cap], v_rows)
    keep = np.ones(cap, bool); keep[pos % cap] = False
    assert not got_k[:, keep].any() and not cv.reshape(n_kv, cap, vd)[:, keep].any()


def test_split_key_store_traditional_pairs_are_complex_rotations():
    """Traditional pairs (2i, 2i+1): (lo + i hi) * exp(i pos theta^(-i/half)) in float64; dims beyond
    rope_dims are copied; position 0 is the identity."""
    n_kv, k0d, k1d, vd, cap, rope = 2, 8, 12, 8, 4, 8
    k0, k0s, k0_rows, k1, v, vs, v_rows = _split_case(310, n_kv, k0d, k1d, vd, 1, False)
    for pos in (0, 7):
        ck, cv = np.zeros(n_kv * cap * (k0d + k1d), np.uint16), np.zeros(n_kv * cap * vd, np.uint16)
        oracle.kv_store_split(k0, k0s, k1, 1, v, vs, n_kv, k0d, k1d, vd, rope, True, 100.0, pos, pos, cap, ck, cv)
        got = oracle.bf16_to_f32(ck.reshape(n_kv, cap, k0d + k1d)[:, pos % cap, k0d:])
        x = oracle.bf16_to_f32(k1[0]).astype(np.float64)
        z = (x[0:rope:2] + 1j * x[1:rope:2]) * np.exp(1j * pos * 100.0 ** (-np.arange(rope // 2) / (rope // 2)))
        want = x.copy()
        want[0:rope:2], want[1:rope:2] = z.real, z.imag
        for h in range(n_kv):
            assert np.all(np.abs(got[h] - want) <= 2.0 ** -8 * np.abs(want) + 1e-6)
            assert np.array_equal(got[h, rope:], oracle.bf16_to_f32(k1[0, rope:]))
            if pos == 0:
                assert np.array_equal(got[h], oracle.bf16_to_f32(k1[0]))


@pytest.mark.parametrize("traditional", [False, True])
def test_split_query_attention_is_attention_on_the_rotated_query(traditional):
    """[Q0 | rope(Q1)] at position kv_len - 1 through the pinned sdpa_decode: equal up to the one bf16
    rounding of the rotated elements that the split form does not make; with rope_dims = 0 bit-equal."""
    n_heads, n_kv, q0d, q1d, vd, cap, kv_len, rope = 4, 2, 16, 8, 16, 16, 9, 8
    q = normal_bf16(320, (n_heads, q0d + q1d))
    ck, cv = normal_bf16(321, n_kv * cap * (q0d + q1d)), normal_bf16(322, n_kv * cap * vd)
    scale = 0.2
    got = oracle.sdpa_decode_split_q(q, n_heads, q0d, q1d, rope, traditional, 1e4, ck, cv, n_kv, vd, kv_len, cap, scale)
    # rotate Q1 through the split store (one shared "key head" per query head, cache of one row)
    qr = q.copy()
    for h in range(n_heads):
        row_k, row_v = np.zeros(q0d + q1d, np.uint16), np.zeros(1, np.uint16)
        oracle.kv_store_split(q[h, :q0d].copy(), q0d, q[h, q0d:].copy(), 1, np.zeros(1, np.uint16), 1, 1, q0d, q1d, 1, rope,
                              traditional, 1e4, kv_len - 1, 0, 1, row_k, row_v)
        qr[h] = row_k
    ref = oracle.sdpa_decode(qr.reshape(-1), ck, cv, n_heads, n_kv, q0d + q1d, vd, kv_len, cap, scale)
    g, r = oracle.bf16_to_f32(got).astype(np.float64), oracle.bf16_to_f32(ref).astype(np.float64)
    assert np.linalg.norm(g - r) / np.linalg.norm(r) < 4e-3
    plain = oracle.sdpa_decode_split_q(q, n_heads, q0d, q1d, 0, traditional, 1e4, ck, cv, n_kv, vd, kv_len, cap, scale)
    assert np.array_equal(plain, oracle.sdpa_decode(q.reshape(-1), ck, cv, n_heads, n_kv, q0d + q1d, vd, kv_len, cap, scale))


def test_softmax_topk_route_closed_forms_and_brute_force():
    one = oracle.f32_to_bf16(np.array([1.0], np.float32))
    # equal logits: every probability is 1/N exactly, ties resolve to the lowest indices in order
    idx, w = oracle.softmax_topk_route(oracle.f32_to_bf16(np.full(64, 0.75, np.float32)), 6,
                                       oracle.f32_to_bf16(np.array([2.5], np.float32)))
    assert idx.tolist() == [[0, 1, 2, 3, 4, 5]]
    assert np.array_equal(w, oracle.f32_to_bf16(np.full((1, 6), 2.5 / 64, np.float32)))
    # logits 0 and ln 3 (bf16): probabilities 1/4 and 3/4 up to the logit's own rounding
    l = oracle.f32_to_bf16(np.array([0.0, np.log(3.0)], np.float32))
    idx, w = oracle.softmax_topk_route(l, 1, one)
    assert idx.tolist() == [[1]] and abs(float(oracle.bf16_to_f32(w)[0, 0]) - 0.75) < 4e-3
    # brute force: float64 softmax rounded to bf16, stable descending sort, per-route scales
    rows, n, k = 7, 32, 5
    logits = normal_bf16(330, (rows, n), 2.0)
    scale = normal_bf16(331, (rows, k), 0.1, 1.0)
    idx, w = oracle.softmax_topk_route(logits, k, scale)
    f = oracle.bf16_to_f32(logits).astype(np.float64)
    p = np.exp(f - f.max(1, keepdims=True)); p /= p.sum(1, keepdims=True)
    pt = oracle.bf16_to_f32(oracle.f32_to_bf16(p.astype(np.float32)))
    for r in range(rows):
        order = sorted(range(n), key=lambda i: (-pt[r, i], i))[:k]
        assert idx[r].tolist() == order
        want = oracle.f32_to_bf16((pt[r, order] * oracle.bf16_to_f32(scale[r])).astype(np.float32))
        assert np.array_equal(w[r], want)
    # rounding to T comes before the ordering: two logits whose probabilities differ in fp32 but
    # round to the same bf16 value are ordered by index
    l = oracle.f32_to_bf16(np.array([0.0, 2.0 ** -10, -3.0, -3.0], np.float32))   # p = 0.47607 and 0.47653 -> 244 / 512 both
    idx, w = oracle.softmax_topk_route(l, 2, one)
    assert w[0, 0] == w[0, 1] and idx.tolist() == [[0, 1]]
