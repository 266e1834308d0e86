"""XCD-resident layer launches (families fusekit_xcd_attn_block / fusekit_xcd_mlp_block / fusekit_xcd_reduce)
against the oracle, through the C ABI (dispatcher).

Bar: the outputs are sums of 8 K-slices in fp32 added in a fixed order, so they are held to the per-kernel
bar of the streaming GEMV: relative L2 <= 1e-2 against the oracle's fp32 values, element-wise equal to the
oracle's bf16 except where the summation order crosses a rounding edge (<= 1 ulp on <= 2 % of elements)."""
import numpy as np
import pytest

import oracle
from helpers import OracleDecoder, bf16_mismatch, make_qweight, normal_bf16, rel_l2, rng, to_device

pytestmark = pytest.mark.gpu

EPS = 1e-6


def _dev(fk, a):
    return fk.DeviceBuffer.from_numpy(np.ascontiguousarray(a))


def _wargs(arg, W):
    return [arg(W.w)] + ([] if W.bits == 16 else [arg(W.scales), arg(W.biases)])


def _kslice_args(fk, arg, W, keep):
    """o_proj / down_proj slots: the weights as they are, scales and biases re-laid out per K-slice
    (fk_xcd_kslice_meta), checked here against the plain numpy statement of that layout."""
    if W.bits == 16:
        return [arg(W.w)]
    out = [arg(W.w)]
    groups = W.k // W.group
    for src in (W.scales, W.biases):
        dst = fk.xcd_kslice_meta(src, W.n, groups)
        fk.sync()
        want = src.to_numpy(np.uint16, (W.n, 8, groups // 8)).transpose(1, 0, 2)
        assert np.array_equal(dst.to_numpy(np.uint16, (8, W.n, groups // 8)), want)
        keep.append(dst)
        out.append(arg(dst))
    return out


def _sum_row(fk, hidden, contributions=None):
    """A sum row as the launches keep it: 64-bit fixed point (2^-32 units), elements permuted (fk.xcd_sum_index),
    padded to whole 512-element sections; `contributions` [n][hidden] fp32 are added the way a launch adds its
    outputs (each rounded to the nearest unit)."""
    row = np.zeros(fk.xcd_sum_row_bytes(hidden) // 8, np.int64)
    if contributions is not None:
        q = np.rint(np.asarray(contributions, np.float32).astype(np.float64) * 2.0 ** 32).astype(np.int64)
        row[fk.xcd_sum_index(hidden)] = q.sum(axis=0)
    return row


def _row_values(fk, row, hidden):
    """The sums of a row as exact doubles, in vector order."""
    return row[fk.xcd_sum_index(hidden)].astype(np.float64) / 2.0 ** 32


def _input_ref(fk, row, hidden, residual):
    """x = T(f32(sum) + float(res)), f32(sum) = fma(f32(low word), 2^-32, f32(high word)): the launches' input."""
    v = row[fk.xcd_sum_index(hidden)]
    lo = (v & 0xffffffff).astype(np.uint32).astype(np.float32).astype(np.float64)
    hi = (v >> 32).astype(np.int32).astype(np.float32).astype(np.float64)
    f = (lo * 2.0 ** -32 + hi).astype(np.float32)            # exact in double, one rounding: the fma
    return oracle.f32_to_bf16((f + oracle.bf16_to_f32(residual)).astype(np.float32))


def _close_bf16(got, ref_bits, ref_f32=None, frac=0.02, ulps=1.0):
    f, u = bf16_mismatch(got, ref_bits)
    assert f <= frac and u <= ulps, (f, u)
    if ref_f32 is not None:
        assert rel_l2(got, ref_f32) <= 1e-2


def _close_rows(got, ref_bits, x64, W, frac=0.02):
    """Projection rows against the oracle's: equal bits except where the fp32 summation order crosses a rounding
    edge (one ulp, at most `frac` of the elements) or where the row's terms nearly cancel -- there the difference is
    bounded by 2e-6 of the sum of the terms' magnitudes, whatever it is in ulps of the small result."""
    g, r = oracle.bf16_to_f32(got).astype(np.float64), oracle.bf16_to_f32(ref_bits).astype(np.float64)
    differ = np.asarray(got) != np.asarray(ref_bits)
    assert differ.mean() <= frac, differ.mean()
    if not differ.any():
        return
    mag = np.maximum(np.abs(g), np.abs(r))
    ulp = 2.0 ** (np.floor(np.log2(np.maximum(mag, 1e-38))) - 7)
    far = differ & (np.abs(g - r) > ulp)
    if far.any():
        w = oracle.dequantize(W).astype(np.float64) if W.bits != 16 else oracle.bf16_to_f32(W.w).astype(np.float64).reshape(W.n, W.k)
        terms = np.abs(w[far]) @ np.abs(x64)
        assert np.all(np.abs(g - r)[far] <= 2e-6 * terms + ulp[far]), (np.abs(g - r)[far], terms)


@pytest.mark.parametrize("bits,hidden,inter,variant",
                         [(b, h, i, v) for b in (4, 8, 16) for h, i, v in ((512, 1024, 0), (2560, 9728, 1), (1024, 3072, 2))] +
                         [(4, 4096, 14336, 1)])
def test_xcd_mlp_block(fk, bits, hidden, inter, variant):
    """(4096 x 14336 is the 8B class: in 4 bits its tiles hold up to 1792 quantisation groups and take the flavour with
    the pass loop; in 8 bits and bf16 two workgroups do not fit a CU and the shape is refused.)"""
    assert fk.xcd_layer_supported(hidden, inter, 32, 8, 128, 256, bits, 64), fk.lib.fk_last_error().decode()
    _run_mlp_block(fk, bits, hidden, inter, variant)


@pytest.mark.parametrize("gain,lo,hi", [(3.0e3, 2.0 ** 20, 2.0 ** 27), (1.5e-6, 0.0, 2.0 ** -26)])
def test_xcd_sum_row_carries_large_and_tiny_contributions(fk, gain, lo, hi):
    """The kernel's own add path at the ends of the fixed-point range: a norm weight scaled by `gain` puts the
    down_proj K-slice sums of the 4B-class shape near 2^26 (the range of one contribution ends at 2^27), resp. near
    the 2^-32 resolution.  Same checks as the plain test: the row equals the float64 product to 2e-6 of its
    absolute terms + 8 half-units, and the next input equals the oracle's down projection + residual."""
    peak = _run_mlp_block(fk, 4, 2560, 9728, 1, norm_gain=gain)
    assert lo <= peak <= hi, peak


def test_xcd_sum_row_reports_a_contribution_beyond_its_range(fk):
    """A K-slice sum of 2^27 or more cannot be carried by the fixed-point row: the launch clamps it, raises the
    overflow word, and the host reports an error instead of handing on a wrong row."""
    with pytest.raises(fk.FusekitError) as e:
        _run_mlp_block(fk, 4, 2560, 9728, 1, norm_gain=4.0e4)
    assert "fixed-point range" in str(e.value)


def _run_mlp_block(fk, bits, hidden, inter, variant, norm_gain=1.0):
    from fusekit_amd.runtime import Dispatch, Dispatcher, arg
    if not fk.xcd_layer_supported(hidden, inter, 32, 8, 128, 256, bits, 64):
        pytest.skip("shape not supported: " + fk.lib.fk_last_error().decode())
    d = Dispatcher()
    Wg, Wu, Wd = make_qweight(1, inter, hidden, bits), make_qweight(2, inter, hidden, bits), make_qweight(3, hidden, inter, bits)
    norm_w = oracle.f32_to_bf16((oracle.bf16_to_f32(normal_bf16(4, hidden, 0.1, 1.0)) * np.float32(norm_gain)).astype(np.float32))
    peak = 0.0
    partials = (rng(5).standard_normal((8, hidden), dtype=np.float32) * 0.3).astype(np.float32)
    res = normal_bf16(6, hidden)
    dWg, dWu, dWd = (to_device(fk, W) for W in (Wg, Wu, Wd))
    ctl_bytes, _ = fk.xcd_workspace_bytes(32, 128)
    ctl = fk.zeros(ctl_bytes)
    row_in = _sum_row(fk, hidden, partials)
    junk = np.full_like(row_in, 0x0123456789abcdef)
    b = dict(p=_dev(fk, row_in), res=_dev(fk, res), x=fk.DeviceBuffer(hidden * 2), nw=_dev(fk, norm_w),
             mid=fk.DeviceBuffer(inter * 2), out=_dev(fk, _sum_row(fk, hidden)), clr=_dev(fk, junk))
    a = [arg(b["p"]), arg(b["res"]), arg(b["x"]), arg(b["nw"]), arg(dWg.w), arg(dWu.w)]
    if bits != 16:
        a += [arg(dWg.scales), arg(dWu.scales), arg(dWg.biases), arg(dWu.biases)]
    keep = []
    a += _kslice_args(fk, arg, dWd, keep) + [arg(b["mid"]), arg(b["out"]), arg(b["clr"]), arg(ctl)]
    task = Dispatch("fusekit_xcd_mlp_block_f1", a,
                    dict(hidden=hidden, inter=inter, n_heads=32, n_kv=8, head_dim=128, capacity=256, bits=bits, group=64,
                         eps=EPS, variant=variant, has_sums=1))
    for rep in range(2):                                  # twice: the arrival words carry over between launches
        d.dispatch_kernel(task)
        fk.xcd_check(ctl)
        x1 = _input_ref(fk, row_in, hidden, res)
        assert np.array_equal(b["x"].to_numpy(np.uint16), x1), "the launch's input row differs"
        assert not b["clr"].to_numpy(np.int64).any(), "the third sum row was not cleared"
        mid_ref = oracle.gateup_swiglu(x1, norm_w, EPS, Wg, Wu, variant)
        got_mid = b["mid"].to_numpy(np.uint16)
        _close_bf16(got_mid, mid_ref, frac=0.03, ulps=2.0)   # gate and up may each sit on a rounding edge
        # the sum row holds W_down . mid (mid as the GPU produced it): eight fp32 K-slice sums per element
        row_out = b["out"].to_numpy(np.int64)
        out = _row_values(fk, row_out, hidden)
        wd = oracle.dequantize(Wd).astype(np.float64) if bits != 16 else oracle.bf16_to_f32(Wd.w).astype(np.float64)
        m64 = oracle.bf16_to_f32(got_mid).astype(np.float64)
        ref, scale = wd @ m64, np.abs(wd) @ np.abs(m64)
        assert np.all(np.abs(out - ref) <= 2e-6 * scale + 8 * 2.0 ** -33)
        peak = max(peak, float(np.abs(out).max()))
        pad = np.ones(row_out.size, bool)
        pad[fk.xcd_sum_index(hidden)] = False
        assert not row_out[pad].any()
        # and the next launch's input from it is the down projection + residual
        y = _input_ref(fk, row_out, hidden, x1)
        y_ref = oracle.linear_residual(Wd, got_mid, x1)
        _close_bf16(y, y_ref, oracle.linear_acc(Wd, got_mid) + oracle.bf16_to_f32(x1))
        partials = (partials * 0.5).astype(np.float32)   # second round on other inputs
        row_in = _sum_row(fk, hidden, partials)
        b["p"].upload(row_in)
        b["out"].upload(_sum_row(fk, hidden))
        b["clr"].upload(junk)
    return peak


@pytest.mark.parametrize("bits", [4, 16])
@pytest.mark.parametrize("n_heads,head_dim,qk_norm,hidden", [(32, 128, True, 1024), (16, 64, False, 1024), (8, 128, True, 1024),
                                                             (64, 64, True, 1024), (32, 128, True, 4096)])
def test_xcd_attn_block(fk, bits, n_heads, head_dim, qk_norm, hidden):
    """Several decode steps through the attention launch: q / k / v rows, head norm + RoPE, cache append,
    attention over the growing context, o_proj partial rows; against the oracle's composition of the same
    dispatches.  Context crosses several key ranges (capacity 256 -> ranges of 64 or 128 positions)."""
    from fusekit_amd.runtime import Dispatch, Dispatcher, arg
    n_kv, inter, capacity, theta = 8, 1024, 256, 1e6   # (hidden 4096: the 8B class, q / k / v tiles of 13 rows x 64 groups)
    if not fk.xcd_layer_supported(hidden, inter, n_heads, n_kv, head_dim, capacity, bits, 64):
        pytest.skip("shape not supported: " + fk.lib.fk_last_error().decode())
    d = Dispatcher()
    n_q, n_kvd = n_heads * head_dim, n_kv * head_dim
    Wq, Wk, Wv = make_qweight(1, n_q, hidden, bits, std=0.05), make_qweight(2, n_kvd, hidden, bits, std=0.05), make_qweight(3, n_kvd, hidden, bits, std=0.05)
    Wo = make_qweight(4, hidden, n_q, bits)
    norm_w = normal_bf16(5, hidden, 0.1, 1.0)
    qn, kn = (normal_bf16(6, head_dim, 0.1, 1.0), normal_bf16(7, head_dim, 0.1, 1.0)) if qk_norm else (None, None)
    dW = [to_device(fk, W) for W in (Wq, Wk, Wv, Wo)]
    ctl_bytes, ap_bytes = fk.xcd_workspace_bytes(n_heads, head_dim)
    ctl = fk.zeros(ctl_bytes)
    cache_bytes = n_kv * capacity * head_dim * 2
    zero_row = _sum_row(fk, hidden)
    b = dict(res=fk.DeviceBuffer(hidden * 2), x=fk.DeviceBuffer(hidden * 2), nw=_dev(fk, norm_w),
             q=fk.DeviceBuffer(n_q * 2), k=fk.DeviceBuffer(n_kvd * 2), v=fk.DeviceBuffer(n_kvd * 2),
             ck=fk.zeros(cache_bytes), cv=fk.zeros(cache_bytes), kv_len=fk.zeros(4), off=fk.zeros(4), step=fk.zeros(4),
             tab=fk.DeviceBuffer(head_dim * 4), ap=fk.DeviceBuffer(ap_bytes), out=_dev(fk, zero_row), clr=_dev(fk, zero_row))
    a = [arg(b["res"]), arg(b["x"]), arg(b["nw"]), arg(dW[0].w), arg(dW[1].w), arg(dW[2].w)]
    if bits != 16:
        a += [arg(m.scales) for m in dW[:3]] + [arg(m.biases) for m in dW[:3]]
    keep = []
    a += _kslice_args(fk, arg, dW[3], keep)
    if qk_norm:
        b["qn"], b["kn"] = _dev(fk, qn), _dev(fk, kn)
        a += [arg(b["qn"]), arg(b["kn"])]
    a += [arg(b["q"]), arg(b["k"]), arg(b["v"]), arg(b["ck"]), arg(b["cv"]), arg(b["kv_len"]), arg(b["tab"]), arg(b["ap"]),
          arg(b["out"]), arg(b["clr"]), arg(ctl)]
    task = Dispatch("fusekit_xcd_attn_block_f1", a,
                    dict(hidden=hidden, inter=inter, n_heads=n_heads, n_kv=n_kv, head_dim=head_dim, capacity=capacity,
                         bits=bits, group=64, eps=EPS, theta=theta, has_sums=0, has_norm=int(qk_norm)))
    step = Dispatch("fusekit_step_init", [arg(b["step"]), arg(b["off"]), arg(b["kv_len"]), arg(b["tab"])],
                    dict(rope_dims=head_dim, theta=theta))
    ck = np.zeros(n_kv * capacity * head_dim, np.uint16)
    cv = np.zeros(n_kv * capacity * head_dim, np.uint16)
    scale = 1.0 / np.sqrt(head_dim)
    worst = 0.0
    for pos in range(200):
        x = normal_bf16(100 + pos, hidden)
        b["res"].upload(x)
        b["out"].upload(zero_row)
        d.dispatch_batch([step, task])
        if pos % 16 and pos < 190:
            # the oracle still has to append this position's rows: it follows the GPU's own q/k/v rows, checked
            # against the oracle's at the sampled positions below
            qg, kg, vg = b["q"].to_numpy(np.uint16), b["k"].to_numpy(np.uint16), b["v"].to_numpy(np.uint16)
            kr = oracle.headnorm_rope(kg, kn, n_kv, head_dim, head_dim, EPS, theta, pos) if qk_norm else \
                oracle.rope_q(kg, n_kv, head_dim, head_dim, theta, pos)
            oracle.kv_store(kr, vg, n_kv, head_dim, head_dim, pos, capacity, ck, cv)
            continue
        fk.xcd_check(ctl)
        assert np.array_equal(b["x"].to_numpy(np.uint16), x)
        q_ref, k_ref, v_ref = oracle.rmsnorm_qkv(x, norm_w, EPS, Wq, Wk, Wv)
        qg, kg, vg = b["q"].to_numpy(np.uint16), b["k"].to_numpy(np.uint16), b["v"].to_numpy(np.uint16)
        xn = oracle.bf16_to_f32(oracle.rmsnorm(x, norm_w, EPS)).astype(np.float64)
        for g, r, W in ((qg, q_ref, Wq), (kg, k_ref, Wk), (vg, v_ref, Wv)):
            _close_rows(g, r, xn, W)
        # downstream of the GPU's own projection rows, as the per-kernel tests do
        if qk_norm:
            qr = oracle.headnorm_rope(qg, qn, n_heads, head_dim, head_dim, EPS, theta, pos)
            kr = oracle.headnorm_rope(kg, kn, n_kv, head_dim, head_dim, EPS, theta, pos)
        else:
            qr = oracle.rope_q(qg, n_heads, head_dim, head_dim, theta, pos)
            kr = oracle.rope_q(kg, n_kv, head_dim, head_dim, theta, pos)
        oracle.kv_store(kr, vg, n_kv, head_dim, head_dim, pos, capacity, ck, cv)
        gck, gcv = b["ck"].to_numpy(np.uint16), b["cv"].to_numpy(np.uint16)
        assert np.array_equal(gcv, cv), "V cache rows differ"
        # RoPE: a normalised value that sits on a rounding edge may differ by one bf16 ulp between the fp32 and
        # the double sum of squares, and the rotation (lo * cos - hi * sin) can nearly cancel: bound the difference by
        # one ulp of the ROW's largest magnitude, not of the element's
        fg, fo = oracle.bf16_to_f32(gck).reshape(-1, head_dim), oracle.bf16_to_f32(ck).reshape(-1, head_dim)
        row_ulp = 2.0 ** (np.floor(np.log2(np.maximum(np.abs(fo).max(axis=1, keepdims=True), 1e-30))) - 7)
        assert np.all(np.abs(fg - fo) <= row_ulp), float(np.max(np.abs(fg - fo) / row_ulp))
        assert np.mean(gck != ck) <= 0.01
        ck = gck.copy()                                  # keep both sides on the same cache bits
        att = oracle.sdpa_decode(qr, ck, cv, n_heads, n_kv, head_dim, head_dim, pos + 1, capacity, scale)
        y_ref_acc = oracle.linear_acc(Wo, att)
        acc = _row_values(fk, b["out"].to_numpy(np.int64), hidden)
        rel = float(np.linalg.norm(acc - y_ref_acc) / np.linalg.norm(y_ref_acc))
        worst = max(worst, rel)
        assert rel <= 1e-2, (pos, rel)
    print("worst rel-L2 of the o_proj sums over the sampled positions: %.3e" % worst)


@pytest.mark.parametrize("kv_len", [512, 4096, 32768])
def test_xcd_attn_block_at_the_config3_contexts(fk, kv_len):
    """The attention launch at 32 q / 8 kv heads x 128 over a cache ~ N(0, 1) of kv_len - 1 positions (blocks walk
    several key ranges at 4096 and 32768): cache append and o_proj sums against the oracle's chain."""
    from fusekit_amd.runtime import Dispatch, Dispatcher, arg
    n_heads, n_kv, head_dim, hidden, inter, bits, theta = 32, 8, 128, 1024, 1024, 4, 1e6
    capacity, pos = kv_len, kv_len - 1
    assert fk.xcd_layer_supported(hidden, inter, n_heads, n_kv, head_dim, capacity, bits, 64)
    d = Dispatcher()
    n_q, n_kvd = n_heads * head_dim, n_kv * head_dim
    Wq, Wk, Wv = (make_qweight(s_, n, hidden, bits, std=0.05) for s_, n in ((1, n_q), (2, n_kvd), (3, n_kvd)))
    Wo = make_qweight(4, hidden, n_q, bits)
    norm_w, x = normal_bf16(5, hidden, 0.1, 1.0), normal_bf16(6, hidden)
    ck, cv = normal_bf16(7, n_kv * capacity * head_dim), normal_bf16(8, n_kv * capacity * head_dim)
    dW = [to_device(fk, W) for W in (Wq, Wk, Wv, Wo)]
    ctl_bytes, ap_bytes = fk.xcd_workspace_bytes(n_heads, head_dim)
    ctl = fk.zeros(ctl_bytes)
    b = dict(res=_dev(fk, x), x=fk.DeviceBuffer(hidden * 2), nw=_dev(fk, norm_w), q=fk.DeviceBuffer(n_q * 2),
             k=fk.DeviceBuffer(n_kvd * 2), v=fk.DeviceBuffer(n_kvd * 2), ck=_dev(fk, ck), cv=_dev(fk, cv),
             kv_len=fk.zeros(4), off=fk.zeros(4), step=_dev(fk, np.array([pos], np.uint32)), tab=fk.DeviceBuffer(head_dim * 4),
             ap=fk.DeviceBuffer(ap_bytes), out=_dev(fk, _sum_row(fk, hidden)), clr=_dev(fk, _sum_row(fk, hidden)))
    a = [arg(b["res"]), arg(b["x"]), arg(b["nw"]), arg(dW[0].w), arg(dW[1].w), arg(dW[2].w)]
    keep = []
    a += [arg(m.scales) for m in dW[:3]] + [arg(m.biases) for m in dW[:3]] + _kslice_args(fk, arg, dW[3], keep)
    a += [arg(b["q"]), arg(b["k"]), arg(b["v"]), arg(b["ck"]), arg(b["cv"]), arg(b["kv_len"]), arg(b["tab"]), arg(b["ap"]),
          arg(b["out"]), arg(b["clr"]), arg(ctl)]
    task = Dispatch("fusekit_xcd_attn_block_f1", a,
                    dict(hidden=hidden, inter=inter, n_heads=n_heads, n_kv=n_kv, head_dim=head_dim, capacity=capacity,
                         bits=bits, group=64, eps=EPS, theta=theta, has_sums=0, has_norm=0))
    step = Dispatch("fusekit_step_init", [arg(b["step"]), arg(b["off"]), arg(b["kv_len"]), arg(b["tab"])],
                    dict(rope_dims=head_dim, theta=theta))
    d.dispatch_batch([step, task])
    fk.xcd_check(ctl)
    assert int(b["kv_len"].to_numpy(np.uint32)[0]) == kv_len
    qg, kg, vg = b["q"].to_numpy(np.uint16), b["k"].to_numpy(np.uint16), b["v"].to_numpy(np.uint16)
    q_ref, k_ref, v_ref = oracle.rmsnorm_qkv(x, norm_w, EPS, Wq, Wk, Wv)
    for g, r in ((qg, q_ref), (kg, k_ref), (vg, v_ref)):
        _close_bf16(g, r)
    qr = oracle.rope_q(qg, n_heads, head_dim, head_dim, theta, pos)
    ock, ocv = ck.copy(), cv.copy()
    oracle.rope_kv_store(kg, vg, n_kv, head_dim, head_dim, theta, pos, pos, capacity, ock, ocv)
    gck, gcv = b["ck"].to_numpy(np.uint16), b["cv"].to_numpy(np.uint16)
    assert np.array_equal(gcv, ocv)
    rows = lambda t: t.reshape(n_kv, capacity, head_dim)
    keep = np.arange(capacity) != pos
    assert np.array_equal(rows(gck)[:, keep], rows(ock)[:, keep])
    fg, fo = oracle.bf16_to_f32(rows(gck)[:, pos]), oracle.bf16_to_f32(rows(ock)[:, pos])
    row_ulp = 2.0 ** (np.floor(np.log2(np.abs(fo).max(axis=1, keepdims=True))) - 7)
    assert np.all(np.abs(fg - fo) <= row_ulp)
    att = oracle.sdpa_decode(qr, gck, gcv, n_heads, n_kv, head_dim, head_dim, kv_len, capacity, 1.0 / np.sqrt(head_dim))
    y_ref = oracle.linear_acc(Wo, att)
    acc = _row_values(fk, b["out"].to_numpy(np.int64), hidden)
    rel = float(np.linalg.norm(acc - y_ref) / np.linalg.norm(y_ref))
    print(f"kv_len {kv_len}: o_proj sums rel-L2 {rel:.3e}")
    assert rel <= 1e-2


def test_xcd_reduce(fk):
    from fusekit_amd.runtime import Dispatch, Dispatcher, arg
    d = Dispatcher()
    for hidden in (2560, 1088):                          # 1088: a row with a partly filled last section
        partials = (rng(1).standard_normal((8, hidden), dtype=np.float32) * 40).astype(np.float32)
        partials[:, :7] = [-3e5, 1e-9, -1e-9, 0.5, 2.0 ** -33, -2.0 ** -33, 70000.25]
        res = normal_bf16(2, hidden)
        row = _sum_row(fk, hidden, partials)
        bp, br, bx = _dev(fk, row), _dev(fk, res), fk.DeviceBuffer(hidden * 2)
        other = _dev(fk, np.full_like(row, -1))
        d.dispatch_kernel(Dispatch("fusekit_xcd_reduce_f1", [arg(bp), arg(br), arg(bx), arg(other)], dict(hidden=hidden)))
        assert np.array_equal(bx.to_numpy(np.uint16), _input_ref(fk, row, hidden, res))
        assert not other.to_numpy(np.int64)[fk.xcd_sum_index(hidden)].any()
        assert np.array_equal(bp.to_numpy(np.int64), row)
        # clearing the row that is read: read first, then cleared
        d.dispatch_kernel(Dispatch("fusekit_xcd_reduce_f1", [arg(bp), arg(br), arg(bx), arg(bp)], dict(hidden=hidden)))
        assert np.array_equal(bx.to_numpy(np.uint16), _input_ref(fk, row, hidden, res))
        assert not bp.to_numpy(np.int64)[fk.xcd_sum_index(hidden)].any()


def test_xcd_wait_gives_up_and_reports(fk):
    """A hand-over wait that exceeds its spin limit (forced from the host: one poll) must not hang: every
    block drains, the error is reported and the control block is reset."""
    from fusekit_amd.decoder import DecoderConfig, DecoderRuntime, DecoderWeights
    cfg = DecoderConfig(n_layers=2, hidden=512, n_heads=16, n_kv=8, head_dim=64, inter=1024, vocab=512, capacity=64,
                        qk_norm=True, xcd_spin_limit=1)
    rt = DecoderRuntime(cfg, DecoderWeights.random_init(cfg, seed=1))
    assert rt.xcd
    with pytest.raises(fk.FusekitError) as e:
        for _ in range(50):          # one poll may well succeed now and then: the limit has to bite within a few launches
            rt.d.decode_host_loop(rt.graph, rt.uniforms, 0, [5])
    assert "spin limit" in str(e.value)
    assert not rt.xcd_ctl.to_numpy(np.uint32).any()
    # the partial sums the failed launch left behind are gone as well: the next token starts from zero rows
    assert not any(row.to_numpy(np.int64).any() for row in rt.xcd_sums)
    # the asynchronous pair reports it too (the error belongs to the wait)
    with pytest.raises(fk.FusekitError) as e2:
        for _ in range(50):
            rt.d.submit_graph_async(rt.graph)
            rt.d.wait_pending()
    assert "spin limit" in str(e2.value)
    assert not any(row.to_numpy(np.int64).any() for row in rt.xcd_sums)


def test_placement_words_flip_together(fk):
    """Every block of a launch flips its bit of its XCD's placement word as it ends: after any number of launches
    each of the eight words is all zeros or all ones (one block per (XCD, slot)), which is what the host checks."""
    from fusekit_amd.decoder import DecoderConfig, DecoderRuntime, DecoderWeights
    cfg = DecoderConfig(n_layers=3, hidden=512, n_heads=16, n_kv=8, head_dim=64, inter=1024, vocab=512, capacity=64, qk_norm=True)
    rt = DecoderRuntime(cfg, DecoderWeights.random_init(cfg, seed=2))
    assert rt.xcd
    seen = set()
    for n in (1, 2, 5):
        rt.generate([7, 8, 9], n)
        ctl = rt.xcd_ctl.to_numpy(np.uint8)
        words = [int(np.frombuffer(ctl[2304 + 256 * x: 2304 + 256 * x + 8].tobytes(), np.uint64)[0]) for x in range(8)]
        assert all(w in (0, 2 ** 64 - 1) for w in words), [hex(w) for w in words]
        assert len(set(words)) == 1
        seen.add(words[0])
    # a word in any other state is reported
    ctl = rt.xcd_ctl.to_numpy(np.uint8).copy()
    ctl[2304 + 256 * 3] ^= 1
    rt.xcd_ctl.upload(ctl)
    with pytest.raises(fk.FusekitError) as e:
        fk.xcd_check(rt.xcd_ctl)
    assert "same (XCD, slot)" in str(e.value)
    assert not rt.xcd_ctl.to_numpy(np.uint8).any()


def test_shapes_whose_workgroups_cannot_all_be_resident_are_refused(fk):
    """Two workgroups per CU are a precondition of the hand-overs.  A bf16 8B-class layer (hidden 4096, intermediate
    14336) needs more than half a CU's LDS per workgroup in the MLP launch: refused at plan time, and the decoder
    takes the per-dispatch path.  Nothing of that shape is launched XCD-resident here."""
    from fusekit_amd.decoder import DecoderConfig, DecoderRuntime, DecoderWeights
    assert not fk.xcd_layer_supported(4096, 14336, 32, 8, 128, 1024, 16, 64)
    assert "resident" in fk.lib.fk_last_error().decode()
    cfg = DecoderConfig(n_layers=1, hidden=4096, n_heads=32, n_kv=8, head_dim=128, inter=14336, vocab=512, capacity=64,
                        qk_norm=True, bits=16)
    W = DecoderWeights.random_init(cfg, seed=3)
    rt = DecoderRuntime(cfg, W)
    assert not rt.xcd
    toks, _, _ = rt.generate([1, 2, 3], 4)
    ref, _ = OracleDecoder(cfg, W).generate([1, 2, 3], 4)
    assert toks == ref


@pytest.mark.parametrize("bits", [4, 8, 16])
@pytest.mark.parametrize("n_heads,head_dim,qk_norm", [(16, 64, True), (32, 128, False)])
def test_xcd_decoder_tokens_match_oracle_and_the_per_dispatch_path(fk, bits, n_heads, head_dim, qk_norm):
    from fusekit_amd.decoder import DecoderConfig, DecoderRuntime, DecoderWeights
    from helpers import OracleDecoder
    kw = dict(n_layers=3, hidden=512, n_heads=n_heads, n_kv=8, head_dim=head_dim, inter=1024, vocab=2000, capacity=128,
              qk_norm=qk_norm, bits=bits)
    cfg = DecoderConfig(**kw)
    W = DecoderWeights.random_init(cfg, seed=11)
    rt = DecoderRuntime(cfg, W)
    assert rt.xcd and len(rt.tasks) == 2 + 2 * cfg.n_layers + 3
    prompt = [7, 1500, 42, 3, 99]
    got, _, _ = rt.generate(prompt, 40)
    ref, margins = OracleDecoder(cfg, W).generate(prompt, 40)
    old = DecoderRuntime(DecoderConfig(**kw, xcd_layers=False), W)
    assert not old.xcd
    got_old, _, _ = old.generate(prompt, 40)
    print("margins:", ["%.3g" % m for m in margins])
    # identical tokens; the runs may part only at a step where the oracle's own top-2 margin is at most one bf16 ulp
    # of these logits (the two GPU paths and the oracle sum in different orders: at such a step any of them may
    # legitimately pick the other candidate, and the continuations then differ)
    for name_, seq in (("xcd", got), ("per-dispatch", got_old)):
        i = next((i for i, (g, r) in enumerate(zip(seq, ref)) if g != r), None)
        assert i is None or margins[i] < 0.01, f"{name_}: step {i}: gpu {seq[i]} oracle {ref[i]} at margin {margins[i]}"


def test_8b_class_int4_layers_run_the_two_launch_path(fk):
    """hidden 4096, intermediate 14336, 32 q / 8 kv heads x 128 in 4 bits: tiles of up to 1792 quantisation groups,
    served by the flavour with the pass loop (its metadata area holds 2048 groups per matrix).  Two layers decode the
    oracle's tokens (up to a step whose margin is within a bf16 ulp), as the per-dispatch list does."""
    from fusekit_amd.decoder import DecoderConfig, DecoderRuntime, DecoderWeights
    from helpers import OracleDecoder
    kw = dict(n_layers=2, hidden=4096, n_heads=32, n_kv=8, head_dim=128, inter=14336, vocab=3000, capacity=128, qk_norm=True, bits=4)
    cfg = DecoderConfig(**kw)
    W = DecoderWeights.random_init(cfg, seed=21)
    rt = DecoderRuntime(cfg, W)
    assert rt.xcd
    prompt = [5, 2900, 17, 333]
    got, _, _ = rt.generate(prompt, 16)
    ref, margins = OracleDecoder(cfg, W).generate(prompt, 16)
    got_old, _, _ = DecoderRuntime(DecoderConfig(**kw, xcd_layers=False), W).generate(prompt, 16)
    for name_, seq in (("two launches", got), ("per-dispatch", got_old)):
        i = next((i for i, (g, r) in enumerate(zip(seq, ref)) if g != r), None)
        assert i is None or margins[i] < 0.01, f"{name_}: step {i}: gpu {seq[i]} oracle {ref[i]} at margin {margins[i]}"


def test_artifact_round_trip_of_a_two_launch_layer_model(fk, tmp_path):
    """task_graph.json written from a runtime on the two-launch layer path (control words, sum rows, the
    per-K-slice copies of o_proj / down_proj scales and biases recorded as a parameter + transform) and replayed
    by a consumer that knows only the files and the parameter tree: same tokens."""
    import json
    from fusekit_amd.artifact import ArtifactRuntime, write_artifact
    from fusekit_amd.decoder import DecoderConfig, DecoderRuntime, DecoderWeights
    cfg = DecoderConfig(n_layers=2, hidden=512, n_heads=16, n_kv=8, head_dim=64, inter=1024, vocab=1000, capacity=128,
                        qk_norm=True)
    W = DecoderWeights.random_init(cfg, seed=9)
    rt = DecoderRuntime(cfg, W)
    assert rt.xcd
    prompt = [3, 700, 41, 12]
    want, _, _ = rt.generate(prompt, 12)
    write_artifact(rt, str(tmp_path), "tiny8")
    tg = json.load(open(tmp_path / "task_graph.json"))
    kinds = [t["kernel"].rsplit("_f", 1)[0] for t in tg["tasks"]]
    assert kinds.count("fusekit_xcd_attn_block") == 2 and kinds.count("fusekit_xcd_mlp_block") == 2
    attn = next(t for t in tg["tasks"] if t["kernel"].startswith("fusekit_xcd_attn_block"))
    moved = [b for b in attn["inputs"] if b.get("transform") == "xcd_kslice"]
    assert sorted(b["source_path"] for b in moved) == ["layers.0.self_attn.o_proj.biases", "layers.0.self_attn.o_proj.scales"]
    assert not any("@" in p["path"] for p in tg["model_params"])
    got = ArtifactRuntime(str(tmp_path), W).generate(prompt, 12)
    assert got == want


@pytest.mark.parametrize("bits", [4, 16])
def test_one_launch_per_layer_gives_the_same_tokens(fk, bits):
    """DecoderConfig.xcd_layer_launch: the dispatcher fuses each attention launch with the MLP launch behind it
    (attention phase, device-wide barrier, MLP phase; both argument blocks by value) where both take their one-pass
    flavour (the 4-bit model here; the bf16 one keeps its two launches).  Same tokens as the separate launches, same
    graph node list for the caller, and a rebinding of a member's buffer reaches the fused launch."""
    from fusekit_amd.decoder import DecoderConfig, DecoderRuntime, DecoderWeights
    kw = dict(n_layers=3, hidden=1024, n_heads=32, n_kv=8, head_dim=128, inter=2048, vocab=3000, capacity=128, qk_norm=True, bits=bits)
    W = DecoderWeights.random_init(DecoderConfig(**kw), seed=5)
    prompt = [11, 2222, 333, 4]
    want, _, _ = DecoderRuntime(DecoderConfig(**kw), W).generate(prompt, 24)
    rt = DecoderRuntime(DecoderConfig(**kw, xcd_layer_launch=True), W)
    assert rt.xcd
    got, _, _ = rt.generate(prompt, 24)
    assert got == want
    new_k, new_v = fk.zeros(rt.cache_k[1].nbytes), fk.zeros(rt.cache_v[1].nbytes)
    ups = []
    for i, t in enumerate(rt.tasks):
        for s_, (p, n) in enumerate(t.args):
            if p == rt.cache_k[1].ptr:
                ups.append((i, s_, new_k.ptr, n))
            if p == rt.cache_v[1].ptr:
                ups.append((i, s_, new_v.ptr, n))
    assert len(ups) == 2
    rt.d.update_graph_bindings(rt.graph, ups)
    old = rt.cache_k[1].to_numpy(np.uint16).copy()
    got2, _, _ = rt.generate(prompt, 24)
    assert got2 == want
    assert np.array_equal(rt.cache_k[1].to_numpy(np.uint16), old) and new_k.to_numpy(np.uint16).any()


@pytest.mark.parametrize("bits", [4, 16])
def test_one_launch_per_token_gives_the_same_tokens(fk, bits):
    """DecoderConfig.xcd_token_launch: the 2 x n_layers launches of a token fused by the dispatcher into ONE launch
    (device-wide barriers where the separate launches have kernel boundaries, per-layer argument blocks in device
    tables, the residual row kept in LDS).  Same tokens as the separate launches, same graph node list for the
    caller, and a rebinding of a member's buffer reaches the fused launch."""
    from fusekit_amd.decoder import DecoderConfig, DecoderRuntime, DecoderWeights
    kw = dict(n_layers=3, hidden=1024, n_heads=32, n_kv=8, head_dim=128, inter=2048, vocab=3000, capacity=128, qk_norm=True, bits=bits)
    W = DecoderWeights.random_init(DecoderConfig(**kw), seed=5)
    prompt = [11, 2222, 333, 4]
    want, _, _ = DecoderRuntime(DecoderConfig(**kw), W).generate(prompt, 24)
    rt = DecoderRuntime(DecoderConfig(**kw, xcd_token_launch=True), W)
    assert rt.xcd
    got, _, _ = rt.generate(prompt, 24)
    assert got == want
    # move layer 1's caches: the fused launch's device table entry is replaced
    new_k, new_v = fk.zeros(rt.cache_k[1].nbytes), fk.zeros(rt.cache_v[1].nbytes)
    ups = []
    for i, t in enumerate(rt.tasks):
        for s_, (p, n) in enumerate(t.args):
            if p == rt.cache_k[1].ptr:
                ups.append((i, s_, new_k.ptr, n))
            if p == rt.cache_v[1].ptr:
                ups.append((i, s_, new_v.ptr, n))
    assert len(ups) == 2
    rt.d.update_graph_bindings(rt.graph, ups)
    old = rt.cache_k[1].to_numpy(np.uint16).copy()
    got2, _, _ = rt.generate(prompt, 24)
    assert got2 == want
    assert np.array_equal(rt.cache_k[1].to_numpy(np.uint16), old) and new_k.to_numpy(np.uint16).any()
