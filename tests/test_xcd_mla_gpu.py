"""The attention half of a layer with low-rank keys as ONE XCD-resident launch (family fusekit_xcd_mla_block: input row,
RMSNorm, q and kv_a projections, latent norm + kv_b, rotations, cache append, attention over the growing context, o_proj
into a sum row) against the oracle's composition of the reference's kernels, step by step through the C ABI.

Bars as for fusekit_xcd_attn_block: projection rows equal to the oracle's except where the fp32 summation order crosses a
rounding edge; V cache rows bit-equal, K rows within one bf16 step of the row's largest magnitude on <= 1 %; the o_proj
sums within 1e-2 relative L2 of the oracle's chain on the GPU's own rows."""
import numpy as np
import pytest

import oracle
from helpers import make_qweight, normal_bf16, rng, to_device
from test_xcd_layer_gpu import _close_rows, _dev, _kslice_args, _row_values, _sum_row
from test_xcd_moe_gpu import _row_f32

pytestmark = pytest.mark.gpu

EPS = 1e-6


def _normed(x, w, rows, W):
    """RMSNorm of x as the launch staged it.  1 / rms is an fp32 value; where x * (1 / rms) lies on rounding ties for
    several elements at once (bf16 inputs share few mantissa patterns), its last bit decides them all, and the oracle's
    double-precision sum of squares may land on the other side of that bit than an fp32 sum: then the normalised row
    is taken with 1 / rms one fp32 step to either side -- whichever reproduces the projection rows `rows` the launch
    wrote from it."""
    ref = oracle.rmsnorm(x, w, EPS)
    if np.mean(rows != oracle.qgemv(W, ref)) <= 0.02:
        return ref
    xf = oracle.bf16_to_f32(x)
    r = np.float32(1.0 / np.sqrt(np.mean(xf.astype(np.float64) ** 2) + EPS))
    best = ref
    for r32 in (np.nextafter(r, np.float32(0)), r, np.nextafter(r, np.float32(2))):
        t = oracle.f32_to_bf16((oracle.bf16_to_f32(w) * oracle.bf16_to_f32(oracle.f32_to_bf16((xf * r32).astype(np.float32)))).astype(np.float32))
        if np.mean(rows != oracle.qgemv(W, t)) < np.mean(rows != oracle.qgemv(W, best)):
            best = t
    return best


@pytest.mark.parametrize("hidden,n_heads,rank,capacity,steps,traditional,two_rows",
                         [(512, 8, 128, 128, 100, True, False), (512, 8, 128, 128, 40, False, True),
                          (2048, 16, 512, 1024, 600, True, False), (1024, 32, 256, 256, 150, True, True)])
def test_xcd_mla_block(fk, hidden, n_heads, rank, capacity, steps, traditional, two_rows):
    from fusekit_amd.runtime import Dispatch, Dispatcher, arg
    rope, nope, vd, theta = 64, 128, 128, 1e4
    assert fk.xcd_mla_supported(hidden, n_heads, rank, rope, nope, vd, capacity, 4, 64), fk.lib.fk_last_error().decode()
    d = Dispatcher()
    qk, n_a, packed = nope + rope, rank + rope, nope + vd
    n_b = n_heads * packed
    Wq, Wa = make_qweight(1, n_heads * qk, hidden, 4, std=0.05), make_qweight(2, n_a, hidden, 4, std=0.05)
    Wb, Wo = make_qweight(3, n_b, rank, 4, std=0.05), make_qweight(4, hidden, n_heads * vd, 4)
    norm_w, a_norm = normal_bf16(5, hidden, 0.1, 1.0), normal_bf16(6, rank, 0.1, 1.0)
    dW = [to_device(fk, W) for W in (Wq, Wa, Wb, Wo)]
    ctl = fk.zeros(fk.xcd_workspace_bytes(32, 128)[0])
    lat_bytes, ap_bytes = fk.xcd_mla_workspace_bytes(n_heads, rank, rope, vd)
    assert lat_bytes == 8 * n_a * 2
    zero_row = _sum_row(fk, hidden)
    junk = np.full_like(zero_row, 0x0123456789abcdef)
    b = dict(res=fk.DeviceBuffer(hidden * 2), x=fk.DeviceBuffer(hidden * 2), nw=_dev(fk, norm_w), an=_dev(fk, a_norm),
             q=fk.DeviceBuffer(2 * n_heads * qk * 2), kva=fk.zeros(lat_bytes), kvb=fk.DeviceBuffer(n_b * 2),
             ck=fk.zeros(n_heads * capacity * qk * 2), cv=fk.zeros(n_heads * capacity * vd * 2), kv_len=fk.zeros(4), off=fk.zeros(4),
             step=fk.zeros(4), tab=fk.DeviceBuffer(rope * 4), ap=fk.DeviceBuffer(ap_bytes), out=_dev(fk, zero_row),
             clr=_dev(fk, junk), clr2=_dev(fk, junk), p1=_dev(fk, zero_row), p2=_dev(fk, zero_row))
    a = ([arg(b["p1"]), arg(b["p2"])] if two_rows else []) + [arg(b["res"]), arg(b["x"]), arg(b["nw"])]
    for W in dW[:2]:
        a += [arg(W.w), arg(W.scales), arg(W.biases)]
    a += [arg(b["an"]), arg(dW[2].w), arg(dW[2].scales), arg(dW[2].biases)]
    keep = []
    a += _kslice_args(fk, arg, dW[3], keep)
    a += [arg(b["q"]), arg(b["kva"]), arg(b["kvb"]), arg(b["ck"]), arg(b["cv"]), arg(b["kv_len"]), arg(b["tab"]), arg(b["ap"])]
    a += ([arg(b["clr2"])] if two_rows else []) + [arg(b["out"]), arg(b["clr"]), arg(ctl)]
    task = Dispatch("fusekit_xcd_mla_block_f1", a,
                    dict(hidden=hidden, n_heads=n_heads, rank=rank, rope_dim=rope, nope_dim=nope, v_dim=vd, capacity=capacity,
                         bits=4, group=64, eps=EPS, theta=theta, traditional=int(traditional), has_sums=2 if two_rows else 0,
                         has_clear2=int(two_rows)))
    step = Dispatch("fusekit_step_init", [arg(b["step"]), arg(b["off"]), arg(b["kv_len"]), arg(b["tab"])],
                    dict(rope_dims=rope, theta=theta))
    ck = np.zeros(n_heads * capacity * qk, np.uint16)
    cv = np.zeros(n_heads * capacity * vd, np.uint16)
    scale = 1.0 / np.sqrt(qk)
    worst = 0.0
    for pos in range(steps):
        res = normal_bf16(100 + pos, hidden)
        b["res"].upload(res)
        b["out"].upload(zero_row)
        x = res
        if two_rows:   # the rows an expert launch leaves: the routes' weighted outputs and the shared expert's dot products
            r1 = _sum_row(fk, hidden, (rng(300 + pos).standard_normal((6, hidden), dtype=np.float32) * 0.2).astype(np.float32))
            r2 = _sum_row(fk, hidden, (rng(400 + pos).standard_normal((2, hidden), dtype=np.float32) * 0.3).astype(np.float32))
            b["p1"].upload(r1)
            b["p2"].upload(r2)
            b["clr"].upload(junk)
            b["clr2"].upload(junk)
            shared = oracle.bf16_to_f32(oracle.f32_to_bf16(_row_f32(fk, r2, hidden)))
            x = oracle.f32_to_bf16(((_row_f32(fk, r1, hidden) + shared).astype(np.float32) + oracle.bf16_to_f32(res)).astype(np.float32))
        d.dispatch_batch([step, task])
        sampled = pos % 16 == 0 or pos >= steps - 10
        q2 = b["q"].to_numpy(np.uint16, (2, n_heads * qk))    # raw rows, then the rows with their second part rotated
        qg, ag, bg = q2[0], b["kva"].to_numpy(np.uint16, (8, n_a)), b["kvb"].to_numpy(np.uint16)
        k_pe = ag[0, rank:].copy().reshape(1, rope)
        if not sampled:   # the oracle still appends this position's rows: it follows the GPU's own, checked when sampled
            oracle.kv_store_split(bg, packed, k_pe, 1, bg[nope:], packed, n_heads, nope, rope, vd, rope, traditional, theta, pos, pos,
                                  capacity, ck, cv)
            continue
        fk.xcd_check(ctl)
        assert np.array_equal(b["x"].to_numpy(np.uint16), x), "the launch's input row differs"
        if two_rows:
            assert not b["clr"].to_numpy(np.int64).any() and not b["clr2"].to_numpy(np.int64).any()
        xn_bits = _normed(x, norm_w, qg, Wq)
        xn = oracle.bf16_to_f32(xn_bits).astype(np.float64)
        _close_rows(qg, oracle.qgemv(Wq, xn_bits), xn, Wq)
        for c in range(1, 8):
            assert np.array_equal(ag[c], ag[0]), "every XCD must form the same latent row"
        _close_rows(ag[0], oracle.qgemv(Wa, xn_bits), xn, Wa)
        lat = _normed(ag[0, :rank].copy(), a_norm, bg, Wb)
        _close_rows(bg, oracle.qgemv(Wb, lat), oracle.bf16_to_f32(lat).astype(np.float64), Wb)
        # downstream of the GPU's own projection rows, as the per-kernel tests do
        oracle.kv_store_split(bg, packed, k_pe, 1, bg[nope:], packed, n_heads, nope, rope, vd, rope, traditional, theta, pos, pos,
                              capacity, ck, cv)
        gck, gcv = b["ck"].to_numpy(np.uint16), b["cv"].to_numpy(np.uint16)
        assert np.array_equal(gcv, cv), "V cache rows differ"
        fg, fo = oracle.bf16_to_f32(gck).reshape(-1, qk), oracle.bf16_to_f32(ck).reshape(-1, qk)
        row_ulp = 2.0 ** (np.floor(np.log2(np.maximum(np.abs(fo).max(axis=1, keepdims=True), 1e-30))) - 7)
        assert np.all(np.abs(fg - fo) <= row_ulp), float(np.max(np.abs(fg - fo) / row_ulp))
        assert np.mean(gck != ck) <= 0.01
        ck = gck.copy()                                  # keep both sides on the same cache bits
        qh = qg.reshape(n_heads, qk).copy()
        for h in range(n_heads):                        # the rotation of q's second part, rounded to T
            row_k, row_v = np.zeros(qk, np.uint16), np.zeros(1, np.uint16)
            oracle.kv_store_split(qh[h, :nope].copy(), nope, qh[h, nope:].copy(), 1, np.zeros(1, np.uint16), 1, 1, nope, rope, 1, rope,
                                  traditional, theta, pos, 0, 1, row_k, row_v)
            qh[h] = row_k
        fq, fr = oracle.bf16_to_f32(q2[1]).reshape(n_heads, qk), oracle.bf16_to_f32(qh.reshape(-1)).reshape(n_heads, qk)
        q_ulp = 2.0 ** (np.floor(np.log2(np.maximum(np.abs(fr).max(axis=1, keepdims=True), 1e-30))) - 7)
        assert np.all(np.abs(fq - fr) <= q_ulp) and np.mean(q2[1] != qh.reshape(-1)) <= 0.01
        assert np.array_equal(q2[1].reshape(n_heads, qk)[:, :nope], qg.reshape(n_heads, qk)[:, :nope])
        att = oracle.sdpa_decode(q2[1].copy(), ck, cv, n_heads, n_heads, qk, vd, pos + 1, capacity, scale)
        y_ref_acc = oracle.linear_acc(Wo, att)
        acc = _row_values(fk, b["out"].to_numpy(np.int64), hidden)
        rel = float(np.linalg.norm(acc - y_ref_acc) / np.linalg.norm(y_ref_acc))
        worst = max(worst, rel)
        assert rel <= 1e-2, (pos, rel)
    print("worst rel-L2 of the o_proj sums over the sampled positions: %.3e" % worst)
