"""The expert block of a mixture-of-experts layer as ONE XCD-resident launch (family fusekit_xcd_moe_block: router,
ranking, routed + shared gate / up with SwiGLU, routed + shared down_proj, weighted sum into a sum row) against the
oracle's composition of the reference's kernels, through the C ABI (dispatcher).

Bars: the router logits are fp32 dot products rounded once (equal to the oracle's except on a rounding edge); the routes
must be EXACTLY the oracle's ranking of the GPU's own logits; SwiGLU rows to the bar of the routed kernels (equal to the
oracle's except where gate or up sits on a rounding edge or nearly cancels); the block's output (sum row + residual, rounded once)
is bit for bit T((f32(routes' row) + T(f32(shared row))) + residual) and equals the oracle's reduction over the GPU's own
SwiGLU rows except where a term sat on a rounding edge (<= 2 % of the elements, by at most one step of that term)."""
import numpy as np
import pytest

import oracle
from helpers import bf16_mismatch, make_qweight, normal_bf16, rel_l2, rng, to_device
from test_gemv_gpu import _check_swiglu
from test_xcd_layer_gpu import _dev, _input_ref, _row_values, _sum_row

pytestmark = pytest.mark.gpu

EPS = 1e-6
SHAPES = [  # hidden, inter, shared_inter, experts, top_k
    (512, 128, 256, 16, 6),
    (1024, 256, 512, 64, 6),
    (512, 128, 128, 8, 7),          # one shared unit
    (512, 128, 128, 8, 4),          # three XCDs without a unit
    (2048, 1408, 2816, 64, 6),      # the benchmark model's expert layers
]


def _stack(seed, n_experts, n, k):
    return oracle.StackedWeight([make_qweight(seed + e, n, k, 4) for e in range(n_experts)])


def _wargs(arg, W):
    return [arg(W.w), arg(W.scales), arg(W.biases)]


@pytest.mark.parametrize("hidden,inter,shared,experts,top_k", SHAPES)
@pytest.mark.parametrize("has_sums", [0, 1])
def test_xcd_moe_block(fk, hidden, inter, shared, experts, top_k, has_sums):
    from fusekit_amd.runtime import Dispatch, Dispatcher, arg
    if not fk.xcd_moe_supported(hidden, inter, shared, experts, top_k, 4, 64):
        pytest.skip("shape not supported: " + fk.lib.fk_last_error().decode())
    d = Dispatcher()
    n_shared = shared // inter
    Eg, Eu, Ed = _stack(100, experts, inter, hidden), _stack(300, experts, inter, hidden), _stack(500, experts, hidden, inter)
    Sg, Su, Sd = make_qweight(701, shared, hidden, 4), make_qweight(702, shared, hidden, 4), make_qweight(703, hidden, shared, 4)
    Wr = normal_bf16(704, (experts, hidden), 0.05)
    norm_w = normal_bf16(705, hidden, 0.1, 1.0)
    scale = oracle.f32_to_bf16(np.array([1.5], np.float32))
    res = normal_bf16(706, hidden)
    partials = (rng(707).standard_normal((8, hidden), dtype=np.float32) * 0.3).astype(np.float32)
    dE = [to_device(fk, W) for W in (Eg, Eu, Ed, Sg, Su, Sd)]
    ctl_bytes, _ = fk.xcd_workspace_bytes(32, 128)
    ctl = fk.zeros(ctl_bytes)
    row_in = _sum_row(fk, hidden, partials)
    junk = np.full_like(row_in, 0x0123456789abcdef)
    scratch_bytes = fk.xcd_moe_scratch_bytes(inter)
    assert scratch_bytes == 8 * 64 * 4 + 8 * inter * 2
    b = dict(p=_dev(fk, row_in), res=_dev(fk, res), x=fk.DeviceBuffer(hidden * 2), nw=_dev(fk, norm_w), wr=_dev(fk, Wr),
             rs=_dev(fk, scale), lo=fk.zeros(experts * 2), io=fk.zeros(top_k * 4), wo=fk.zeros(top_k * 2),
             sc=fk.zeros(scratch_bytes), out=_dev(fk, _sum_row(fk, hidden)), out2=_dev(fk, _sum_row(fk, hidden)),
             clr=_dev(fk, junk), y=fk.DeviceBuffer(hidden * 2))
    a = ([arg(b["p"])] if has_sums else []) + [arg(b["res"]), arg(b["x"]), arg(b["nw"]), arg(b["wr"]), arg(b["rs"])]
    for W in dE:
        a += _wargs(arg, W)
    a += [arg(b["lo"]), arg(b["io"]), arg(b["wo"]), arg(b["sc"]), arg(b["out2"]), arg(b["out"]), arg(b["clr"]), arg(ctl)]
    task = Dispatch("fusekit_xcd_moe_block_f1", a,
                    dict(hidden=hidden, inter=inter, shared_inter=shared, experts=experts, top_k=top_k, bits=4, group=64,
                         eps=EPS, variant=1, has_sums=has_sums))
    for rep in range(2):                                  # twice: the arrival words carry over between launches
        d.dispatch_kernel(task)
        fk.xcd_check(ctl)
        x1 = _input_ref(fk, row_in, hidden, res) if has_sums else res
        assert np.array_equal(b["x"].to_numpy(np.uint16), x1), "the launch's input row differs"
        assert not b["clr"].to_numpy(np.int64).any(), "the third sum row was not cleared"
        xn = oracle.rmsnorm(x1, norm_w, EPS)
        # router logits: fp32 dot products of bf16 rows, rounded once
        logits = b["lo"].to_numpy(np.uint16)
        logits_ref = oracle.qgemv(oracle.dense(Wr), xn)
        f, u = bf16_mismatch(logits, logits_ref)
        assert f <= 0.1 and u <= 1.0, (f, u)
        # every XCD that ranks holds the same logits
        per_xcd = b["sc"].to_numpy(np.uint8)[:8 * 64 * 4].view(np.uint32).reshape(8, 64)
        for xcd in range(top_k):
            assert np.array_equal((per_xcd[xcd, :experts] >> 16).astype(np.uint16), logits)
            assert not (per_xcd[xcd, :experts] & 0xffff).any()
        # the routes: the oracle's ranking of the GPU's logits, bit for bit
        idx_ref, w_ref = oracle.softmax_topk_route(logits, top_k, scale)
        idx, rw = b["io"].to_numpy(np.uint32), b["wo"].to_numpy(np.uint16)
        assert np.array_equal(idx, idx_ref[0]) and np.array_equal(rw, w_ref[0])
        # SwiGLU rows of the eight units: the routes' experts, then the shared expert's rows in blocks of `inter`
        mid = b["sc"].to_numpy(np.uint8)[8 * 64 * 4:].view(np.uint16).reshape(8, inter)
        h = mid[:top_k]
        h_ref = oracle.routed_qmv_swiglu(xn.reshape(1, -1), Eg, Eu, np.zeros(top_k, np.uint32), idx, None)
        for r in range(top_k):
            _check_swiglu(h[r], h_ref[r], xn, Eg.expert(int(idx[r])), Eu.expert(int(idx[r])), 1)
        sh_ref = oracle.gateup_swiglu(xn, None, 0.0, Sg, Su, 1)
        sh = mid[top_k:top_k + n_shared].reshape(-1)
        _check_swiglu(sh, sh_ref, xn, Sg, Su, 1)
        # the routes' sum row: every term is w * T(dot), added exactly -- against float64 on the GPU's own rows
        row_out, row_out2 = b["out"].to_numpy(np.int64), b["out2"].to_numpy(np.int64)
        out, out2 = _row_values(fk, row_out, hidden), _row_values(fk, row_out2, hidden)
        ref64 = np.zeros(hidden)
        term_ulp = np.zeros(hidden)
        for r in range(top_k):
            w = float(oracle.bf16_to_f32(rw[r:r + 1])[0])
            dot = oracle.bf16_to_f32(oracle.qgemv(Ed.expert(int(idx[r])), h[r])).astype(np.float64)
            ref64 += w * dot
            term_ulp += w * 2.0 ** (np.floor(np.log2(np.maximum(np.abs(dot), 1e-30))) - 7)
        # a term whose dot product sat on a rounding edge may differ by one bf16 step of that term
        assert np.all(np.abs(out - ref64) <= term_ulp + 1e-6 * np.abs(ref64) + 8 * 2.0 ** -32)
        assert np.mean(np.abs(out - ref64) > 1e-6 * np.abs(ref64) + 8 * 2.0 ** -32) <= 0.05
        # the shared expert's row: K-slice sums of its down projection, unrounded
        wd = oracle.dequantize(Sd).astype(np.float64)
        s64 = oracle.bf16_to_f32(sh).astype(np.float64)
        assert np.all(np.abs(out2 - wd @ s64) <= 2e-6 * (np.abs(wd) @ np.abs(s64)) + 8 * 2.0 ** -33)
        pad = np.ones(row_out.size, bool)
        pad[fk.xcd_sum_index(hidden)] = False
        assert not row_out[pad].any() and not row_out2[pad].any()
        # what reads the rows (fusekit_xcd_reduce with six slots): T((f32(routes) + T(f32(shared))) + residual), rows cleared
        d.dispatch_kernel(Dispatch("fusekit_xcd_reduce_f2", [arg(b["out"]), arg(b["x"]), arg(b["y"]), arg(b["out"]), arg(b["out2"]),
                                                             arg(b["out2"])], dict(hidden=hidden)))
        fk.sync()
        y = b["y"].to_numpy(np.uint16)
        zero_res = np.zeros(hidden, np.uint16)
        f_routes = oracle.bf16_to_f32(zero_res) + _row_f32(fk, row_out, hidden)
        f_shared = oracle.bf16_to_f32(oracle.f32_to_bf16(_row_f32(fk, row_out2, hidden)))
        y_want = oracle.f32_to_bf16(((f_routes + f_shared).astype(np.float32) + oracle.bf16_to_f32(x1)).astype(np.float32))
        assert np.array_equal(y, y_want)
        assert not b["out"].to_numpy(np.int64).any() and not b["out2"].to_numpy(np.int64).any()
        # ... which is the reference's reduction (routes in slot order, shared expert, residual) over the GPU's SwiGLU rows
        y_ref = oracle.routed_qmv_reduce(h, Ed, idx, rw, x1.reshape(1, -1), 1, top_k, shared_x=sh.reshape(1, -1), Wshared=Sd)[0]
        # (a route whose dot product sat on a rounding edge moves the sum by one bf16 step of THAT TERM, which may exceed
        # a step of a smaller result; the same for the shared expert's)
        sdot = wd @ s64
        term_ulp += 2.0 ** (np.floor(np.log2(np.maximum(np.abs(sdot), 1e-30))) - 7)
        yf, rf = oracle.bf16_to_f32(y).astype(np.float64), oracle.bf16_to_f32(y_ref).astype(np.float64)
        step = 2.0 ** (np.floor(np.log2(np.maximum(np.maximum(np.abs(yf), np.abs(rf)), 1e-30))) - 7)
        assert np.mean(y != y_ref) <= 0.02 and np.all(np.abs(yf - rf) <= step + term_ulp)
        assert rel_l2(y, ref64 + sdot + oracle.bf16_to_f32(x1)) <= 1e-2
        # second round on other inputs
        partials = (partials * 0.5).astype(np.float32)
        row_in = _sum_row(fk, hidden, partials)
        res = normal_bf16(710 + rep, hidden)
        b["p"].upload(row_in)
        b["res"].upload(res)
        b["clr"].upload(junk)


def _row_f32(fk, row, hidden):
    """f32(sum) = fma(f32(low word), 2^-32, f32(high word)) of every element, in vector order."""
    v = row[fk.xcd_sum_index(hidden)]
    lo = (v & 0xffffffff).astype(np.uint32).astype(np.float32).astype(np.float64)
    hi = (v >> 32).astype(np.int32).astype(np.float32).astype(np.float64)
    return (lo * 2.0 ** -32 + hi).astype(np.float32)


