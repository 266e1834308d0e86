"""GPU parity of the multi-row quantised matmul on the matrix cores (G) against the CPU oracle.

Up to 64 activation rows the kernel keeps the single-row GEMV arithmetic (exact affine
dequantisation folded per group, fp32 accumulation, one round) and is compared with the oracle's
row-by-row form.  From 65 rows up it dequantises every weight to bf16 before the multiply, as the
reference's own multi-row path does (MLX QuantizedBlockLoader, not vendored in the reference), and
is compared with the oracle's restatement of that form.  Both agree with the fp32 result far inside
the rel-L2 <= 1e-2 bar.
"""
import numpy as np
import pytest

import oracle
from helpers import make_qweight, normal_bf16, to_device
from test_gemv_gpu import _check, _check_swiglu

pytestmark = pytest.mark.gpu


def _dev(fk, a):
    return None if a is None else fk.DeviceBuffer.from_numpy(np.ascontiguousarray(a))


def _run(fk, W, x, bias=None, res=None):
    m = x.shape[0]
    y = fk.DeviceBuffer(2 * m * W.n)
    ws = fk.DeviceBuffer(fk.qgemm_workspace_bytes(m, W.n, W.k, W.group))
    fk.qgemm(to_device(fk, W), _dev(fk, x), m, _dev(fk, bias), _dev(fk, res), y, ws)
    return y.to_numpy(np.uint16, (m, W.n))


SHAPES = [
    (8, 4096, 2560),    # batch-8 decode, 4B-class q projection
    (2, 333, 256),      # ragged N
    (32, 1152, 896),
    (33, 256, 512),     # one row into the second activation tile
    (5, 2560, 9728),    # long K: split over many blocks
    (70, 128, 128),     # three activation tiles, one weight block (weights rounded to bf16 from here up)
    (1, 64, 64),
    (64, 256, 320),     # last row count of the exact form; K not a multiple of the slab
    (65, 256, 320),     # first row count of the bf16-weight form
    (130, 512, 1024),   # two blocks of 128 rows, the second with two live rows
    (200, 333, 2560),   # ragged N, several slabs
    (512, 256, 512),
]


def _reference(W, x, bias=None):
    """(bits, unrounded sums) of the form the kernel uses for this row count."""
    if x.shape[0] > 64:
        return oracle.qgemm_bf16w(W, x, bias, want_acc=True)
    ref = oracle.qgemm(W, x, bias)
    acc = np.stack([oracle.linear_acc(W, x[r]) for r in range(x.shape[0])])
    return ref, acc


@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("m,n,k", SHAPES)
def test_qgemm_matches_oracle(fk, m, n, k, bits):
    W = make_qweight(50 + bits, n, k, bits)
    x = normal_bf16(51, (m, k))
    got = _run(fk, W, x)
    ref, acc = _reference(W, x)
    for r in range(m):
        _check(got[r], ref[r], acc[r], W, x[r])


# The shared-stream kernel for 2..10 activation rows (one launch, no split-k sums): every row count of its range,
# the projections of the 4B-class decoder and of the mixture-of-experts model (K = 1408 ends in half a slab),
# a ragged N, few weight rows with a long K (16 waves per block), bias and residual, and the split-k route on the
# same operands (both keep the single-row arithmetic: rounding-edge flips only).
WIDE_SHAPES = [(2, 2560, 2560), (3, 6144, 2560), (4, 333, 1408), (5, 2560, 9728), (6, 2048, 1408), (7, 1408, 2048),
               (8, 9728, 2560), (9, 70, 4096), (10, 2560, 4096),
               # K of one, three and five groups (a slab's second double group partly or wholly past the end), few rows
               (8, 48, 64), (3, 100, 192), (2, 17, 320), (8, 40000, 512)]


@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("m,n,k", WIDE_SHAPES)
def test_shared_stream_rows_match_oracle_and_the_split_k_route(fk, m, n, k, bits):
    W = make_qweight(150 + bits + m, n, k, bits)
    x = normal_bf16(151 + m, (m, k))
    bias, res = normal_bf16(152, n), normal_bf16(153, (m, n))
    got = _run(fk, W, x)
    ref, acc = _reference(W, x)
    for r in range(m):
        _check(got[r], ref[r], acc[r], W, x[r])
    got_b = _run(fk, W, x, bias=bias, res=res)
    fk.set_qgemm_wide(False)
    try:
        split_k = _run(fk, W, x)
        split_k_b = _run(fk, W, x, bias=bias, res=res)
    finally:
        fk.set_qgemm_wide(True)
    for r in range(m):
        _check(got[r], split_k[r], oracle.bf16_to_f32(split_k[r]), W, x[r])
        _check(got_b[r], split_k_b[r], oracle.bf16_to_f32(split_k_b[r]), W, x[r])
    assert not np.array_equal(got_b, got)


@pytest.mark.parametrize("variant", [0, 1, 2])
@pytest.mark.parametrize("m,hidden,inter,bits", [(2, 2560, 9728, 4), (10, 2048, 1408, 4), (5, 896, 4864, 8)])
def test_shared_stream_gate_up_swiglu(fk, m, hidden, inter, bits, variant):
    Wg, Wu = make_qweight(166, inter, hidden, bits), make_qweight(167, inter, hidden, bits)
    x = normal_bf16(168, (m, hidden))
    out = fk.DeviceBuffer(2 * m * inter)
    ws = fk.DeviceBuffer(2 * fk.qgemm_workspace_bytes(m, inter, hidden, 64))
    fk.qgemm_swiglu(to_device(fk, Wg), to_device(fk, Wu), _dev(fk, x), m, variant, out, ws)
    got = out.to_numpy(np.uint16, (m, inter))
    for r in range(m):
        _check_swiglu(got[r], oracle.gateup_swiglu(x[r], None, 0.0, Wg, Wu, variant), x[r], Wg, Wu, variant)


@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("m,hidden,ns,normed", [(8, 2048, (3072, 288, 288), True), (5, 512, (2048, 1024, 1024), True),
                                                (2, 896, (333, 64, None), False), (8, 2560, (4096, None, None), True)])
def test_norm_and_fan_out_of_several_rows_in_one_launch(fk, bits, m, hidden, ns, normed):
    """fk_rmsnorm_qkv_rows: 2..8 token rows, RMSNorm applied while the rows are staged, one to three matrices served by
    one launch, inputs and outputs with row strides (column blocks of wider rows).  Every row equals the oracle's
    RMSNorm followed by its single-row projection (to rounding-edge flips), and the launch equals the separate
    rmsnorm_rows + fk_qgemm launches to the same bar; what lies between the column blocks is not touched."""
    Ws = [make_qweight(700 + i + bits, n, hidden, bits) if n else None for i, n in enumerate(ns)]
    xs_, pad = hidden + 64, 40                       # activations are the first `hidden` columns of wider rows
    xw = normal_bf16(710 + m, (m, xs_))
    nw = normal_bf16(711, hidden, 0.1, 1.0) if normed else None
    outs = [fk.DeviceBuffer.from_numpy(np.full((m, n + pad), 0xAAAA, np.uint16)) if n else None for n in ns]
    dW = [to_device(fk, W) if W is not None else None for W in Ws]
    fk.rmsnorm_qkv_rows(_dev(fk, xw), m, xs_, _dev(fk, nw), 1e-6, dW[0], dW[1], dW[2],
                        outs[0], ns[0] + pad, outs[1], (ns[1] or 0) + pad, outs[2], (ns[2] or 0) + pad)
    fk.sync()
    x = np.ascontiguousarray(xw[:, :hidden])
    xn = np.stack([oracle.rmsnorm(x[r], nw, 1e-6) for r in range(m)]) if normed else x
    for W, o, n in zip(Ws, outs, ns):
        if W is None:
            continue
        got = o.to_numpy(np.uint16, (m, n + pad))
        assert (got[:, n:] == 0xAAAA).all()
        sep = _run(fk, W, xn)                         # the separate launches on the oracle's normalised rows
        for r in range(m):
            _check(got[r, :n], oracle.qgemv(W, xn[r], None), oracle.linear_acc(W, xn[r]), W, xn[r])
            _check(got[r, :n], sep[r], oracle.bf16_to_f32(sep[r]), W, xn[r])
    with pytest.raises(fk.FusekitError):               # nine rows take the plain matmul
        fk.rmsnorm_qkv_rows(_dev(fk, normal_bf16(1, (9, xs_))), 9, xs_, _dev(fk, nw), 1e-6, dW[0], None, None,
                            fk.DeviceBuffer(2 * 9 * (ns[0] + pad)), ns[0] + pad)


@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("m,hidden,inter,variant,normed", [(8, 2560, 9728, 1, True), (3, 896, 4864, 0, True), (2, 512, 1408, 2, False)])
def test_norm_gate_up_and_swiglu_of_several_rows_in_one_launch(fk, bits, m, hidden, inter, variant, normed):
    """fk_gateup_swiglu_rows: every row equals the oracle's single-row RMSNorm -> gate / up -> SwiGLU."""
    Wg, Wu = make_qweight(720 + bits, inter, hidden, bits), make_qweight(730 + bits, inter, hidden, bits)
    x = normal_bf16(740 + m, (m, hidden))
    nw = normal_bf16(741, hidden, 0.1, 1.0) if normed else None
    out = fk.DeviceBuffer(2 * m * inter)
    fk.gateup_swiglu_rows(_dev(fk, x), m, _dev(fk, nw), 1e-6, to_device(fk, Wg), to_device(fk, Wu), variant, out)
    got = out.to_numpy(np.uint16, (m, inter))
    for r in range(m):
        xn = oracle.rmsnorm(x[r], nw, 1e-6) if normed else x[r]
        _check_swiglu(got[r], oracle.gateup_swiglu(x[r], nw, 1e-6, Wg, Wu, variant), xn, Wg, Wu, variant)
    with pytest.raises(fk.FusekitError):
        fk.gateup_swiglu_rows(_dev(fk, normal_bf16(1, (9, hidden))), 9, _dev(fk, nw), 1e-6, to_device(fk, Wg), to_device(fk, Wu),
                              variant, fk.DeviceBuffer(2 * 9 * inter))


@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("m", [9, 100])
def test_qgemm_group_128(fk, bits, m):
    W = make_qweight(60, 384, 1024, bits, group=128)
    x = normal_bf16(61, (m, 1024))
    got = _run(fk, W, x)
    ref, acc = _reference(W, x)
    for r in range(m):
        _check(got[r], ref[r], acc[r], W, x[r])


def test_qgemm_bias_and_residual(fk):
    W = make_qweight(62, 896, 4864, 4)
    x = normal_bf16(63, (12, 4864))
    bias, res = normal_bf16(64, 896), normal_bf16(65, (12, 896))
    got = _run(fk, W, x, bias=bias)
    ref = oracle.qgemm(W, x, bias)
    for r in range(12):
        _check(got[r], ref[r], oracle.linear_acc(W, x[r]) + oracle.bf16_to_f32(bias), W, x[r])
    got = _run(fk, W, x, res=res)
    for r in range(12):
        ref_r = oracle.linear_residual(W, x[r], res[r], None)
        _check(got[r], ref_r, oracle.linear_acc(W, x[r]) + oracle.bf16_to_f32(res[r]), W, x[r])


@pytest.mark.parametrize("variant", [0, 1, 2])
def test_qgemm_swiglu(fk, variant):
    m, hidden, inter = 8, 896, 4864
    Wg, Wu = make_qweight(66, inter, hidden, 4), make_qweight(67, inter, hidden, 4)
    x = normal_bf16(68, (m, hidden))
    out = fk.DeviceBuffer(2 * m * inter)
    ws = fk.DeviceBuffer(2 * fk.qgemm_workspace_bytes(m, inter, hidden, 64))
    fk.qgemm_swiglu(to_device(fk, Wg), to_device(fk, Wu), _dev(fk, x), m, variant, out, ws)
    got = out.to_numpy(np.uint16, (m, inter))
    for r in range(m):
        _check_swiglu(got[r], oracle.gateup_swiglu(x[r], None, 0.0, Wg, Wu, variant), x[r], Wg, Wu, variant)


@pytest.mark.parametrize("route", ["kernel", "library"])
@pytest.mark.parametrize("bits,group", [(4, 64), (8, 64), (4, 128)])
@pytest.mark.parametrize("m,n,k", [(512, 333, 2560), (700, 1152, 896), (300, 512, 4864)])
def test_qgemm_many_rows_both_routes(fk, m, n, k, bits, group, route):
    """From a row threshold on (1024 by default; 256 here) direct calls dequantise the matrix to bf16 once and take
    the library GEMM; the fused kernel stays reachable (and is what a graph node runs).  Same arithmetic, same oracle form,
    with bias and residual in the epilogue."""
    fk.set_gemm_library_rows(0 if route == "kernel" else 256)
    try:
        W = make_qweight(70 + bits, n, k, bits, group=group)
        x = normal_bf16(71, (m, k))
        bias, res = normal_bf16(72, n), normal_bf16(73, (m, n))
        got = _run(fk, W, x)
        ref, acc = _reference(W, x)
        for r in range(0, m, 7):
            _check(got[r], ref[r], acc[r], W, x[r])
        got = _run(fk, W, x, bias=bias, res=res)
        full = acc + oracle.bf16_to_f32(bias)[None, :] + oracle.bf16_to_f32(res)
        want = oracle.f32_to_bf16(full.astype(np.float32))
        for r in range(0, m, 7):
            _check(got[r], want[r], full[r], W, x[r])
    finally:
        fk.set_gemm_library_rows(fk.GEMM_LIBRARY_ROWS_DEFAULT)


@pytest.mark.parametrize("bits,group", [(4, 64), (8, 64), (4, 128)])
def test_qgemm_tile_form_finishes_its_outputs_at_one_k_split(fk, bits, group):
    """From 65 rows the fused kernel stages both operands of a 256 x 128 tile in LDS; with enough tiles to fill the
    device it takes ONE k split and adds bias and residual and rounds in the same launch (no fp32 partial sums, no
    second kernel).  Ragged in both directions: 520 rows (a third row tile with 8 live rows), 9700 weight rows."""
    from fusekit_amd.runtime import Dispatch, Dispatcher, arg
    m, n, k = 520, 9700, 256
    W = make_qweight(80 + bits, n, k, bits, group=group)
    x = normal_bf16(81, (m, k))
    bias, res = normal_bf16(82, n), normal_bf16(83, (m, n))
    dW, bx, bb, br = to_device(fk, W), _dev(fk, x), _dev(fk, bias), _dev(fk, res)
    y, ws = fk.DeviceBuffer(2 * m * n), fk.DeviceBuffer(fk.qgemm_workspace_bytes(m, n, k, group))
    d = Dispatcher()
    params = {"bits": bits, "group": group, "m": k, "n": n, "rows": m}
    plain = Dispatch("fusekit_qgemm_f0", [arg(bx), arg(dW.w), arg(dW.scales), arg(dW.biases), arg(y), arg(ws)], params)
    geo = d.plan_geometry(plain)
    assert geo.n_kernels == 1 and tuple(geo.threadgroup[0]) == (512, 1, 1) and tuple(geo.grid[0]) == (76, 3, 1)
    y.upload(np.full(m * n, 0x7fc0, np.uint16))
    d.dispatch_kernel(plain)
    fk.sync()
    got = y.to_numpy(np.uint16, (m, n))
    ref, acc = _reference(W, x)
    rows = list(range(0, m, 37)) + [255, 256, 511, 512, 519]
    for r in rows:
        _check(got[r], ref[r], acc[r], W, x[r])
    full_d = Dispatch("fusekit_qgemm_f0", [arg(bx), arg(dW.w), arg(dW.scales), arg(dW.biases), arg(bb), arg(br), arg(y), arg(ws)],
                      dict(params, has_bias=1, has_residual=1))
    d.dispatch_kernel(full_d)
    fk.sync()
    got = y.to_numpy(np.uint16, (m, n))
    full = acc + oracle.bf16_to_f32(bias)[None, :] + oracle.bf16_to_f32(res)
    want = oracle.f32_to_bf16(full.astype(np.float32))
    for r in rows:
        _check(got[r], want[r], full[r], W, x[r])


@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("m,hidden,inter,kernels", [(512, 256, 9700, 1), (300, 1024, 1280, 2)])
@pytest.mark.parametrize("variant", [1, 2])
def test_qgemm_swiglu_tile_form_takes_the_pair_in_one_launch(fk, bits, m, hidden, inter, kernels, variant):
    """From 65 rows a gate / up pair (same shape, even count of 64-wide k slabs per split) is ONE launch of the tile
    form: the activations staged once, two sets of accumulators; with one k split SwiGLU is applied there (1 kernel),
    otherwise the partial sums of both go to the usual second kernel (2 kernels instead of 3)."""
    from fusekit_amd.runtime import Dispatch, Dispatcher, arg
    Wg, Wu = make_qweight(90 + bits, inter, hidden, bits), make_qweight(93 + bits, inter, hidden, bits)
    x = normal_bf16(96, (m, hidden))
    dg, du, bx = to_device(fk, Wg), to_device(fk, Wu), _dev(fk, x)
    out = fk.DeviceBuffer(2 * m * inter)
    ws = fk.DeviceBuffer(2 * fk.qgemm_workspace_bytes(m, inter, hidden, 64))
    d = Dispatcher()
    task = Dispatch("fusekit_qgemm_swiglu_f0", [arg(bx), arg(dg.w), arg(du.w), arg(dg.scales), arg(du.scales), arg(dg.biases),
                                                arg(du.biases), arg(out), arg(ws)],
                    {"bits": bits, "group": 64, "hidden": hidden, "inter": inter, "rows": m, "variant": variant})
    geo = d.plan_geometry(task)
    assert geo.n_kernels == kernels and tuple(geo.threadgroup[0]) == (512, 1, 1) and geo.lds_bytes[0] == 147456
    out.upload(np.full(m * inter, 0x7fc0, np.uint16))
    d.dispatch_kernel(task)
    fk.sync()
    got = out.to_numpy(np.uint16, (m, inter))
    _, g = oracle.qgemm_bf16w(Wg, x, None, want_acc=True)
    _, u = oracle.qgemm_bf16w(Wu, x, None, want_acc=True)
    rows = list(range(0, m, 41)) + [255, 256, m - 1]
    want = np.array([[oracle.swiglu_scalar(float(a), float(b), variant) for a, b in zip(g[r], u[r])] for r in rows], dtype=np.uint16)
    sel = got[rows]
    gf, wf = oracle.bf16_to_f32(sel).astype(np.float64), oracle.bf16_to_f32(want).astype(np.float64)
    assert np.linalg.norm(gf - wf) / np.linalg.norm(wf) <= 1e-2
    assert np.mean(sel != want) <= 0.05          # fp32 summation order may cross a bf16 rounding edge


@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("m,k,ns,with_bias", [(512, 256, (4096, 1024, 1024), False),   # one k split: finished in the launch
                                              (300, 1024, (1000, 520, 260), True),     # ragged, k split, the fan-out's second kernel
                                              (512, 512, (2048, 1024), True),          # two matrices
                                              (40, 256, (512, 256, 256), False)])      # too few rows for the tile form: one by one
def test_qgemm_fanout_of_the_prompt_projections(fk, bits, m, k, ns, with_bias):
    """fk_qgemm_fanout: up to three matrices over the same rows (q / k / v of a prompt pass) as one launch of the tile
    form whose blocks run through the matrices in turn; every output against the oracle form of its row count."""
    Ws = [make_qweight(110 + bits + 3 * i, n, k, bits) for i, n in enumerate(ns)]
    x = normal_bf16(120, (m, k))
    biases = [normal_bf16(121 + i, n) if (with_bias and i != 1) else None for i, n in enumerate(ns)]
    dWs, bx = [to_device(fk, W) for W in Ws], _dev(fk, x)
    dbs = [_dev(fk, b) for b in biases]
    ys = [fk.DeviceBuffer(2 * m * n) for n in ns]
    for y, n in zip(ys, ns):
        y.upload(np.full(m * n, 0x7fc0, np.uint16))
    ws = fk.DeviceBuffer(max(fk.qgemm_workspace_bytes(m, sum(ns), k, 64), max(fk.qgemm_workspace_bytes(m, n, k, 64) for n in ns)))
    fk.qgemm_fanout(dWs, bx, m, dbs if with_bias else None, ys, ws)
    fk.sync()
    rows = sorted(set(list(range(0, m, 53)) + [m - 1, min(255, m - 1), min(256, m - 1)]))
    for W, b, y, n in zip(Ws, biases, ys, ns):
        got = y.to_numpy(np.uint16, (m, n))
        ref, acc = _reference(W, x)
        full = acc if b is None else acc + oracle.bf16_to_f32(b)[None, :]
        want = ref if b is None else oracle.f32_to_bf16(full.astype(np.float32))
        for r in rows:
            _check(got[r], want[r], full[r], W, x[r])


@pytest.mark.parametrize("route,m", [("kernel", 512), ("library", 512), ("library", 2048)])
def test_qgemm_swiglu_many_rows_both_routes(fk, route, m):
    """From 2048 rows the library route lets the GEMM round gate and up to bf16 itself and runs SwiGLU over bf16."""
    hidden, inter, variant = 896, 1216, 2
    fk.set_gemm_library_rows(0 if route == "kernel" else 256)
    try:
        Wg, Wu = make_qweight(76, inter, hidden, 4), make_qweight(77, inter, hidden, 4)
        x = normal_bf16(78, (m, hidden))
        out = fk.DeviceBuffer(2 * m * inter)
        ws = fk.DeviceBuffer(2 * fk.qgemm_workspace_bytes(m, inter, hidden, 64))
        fk.qgemm_swiglu(to_device(fk, Wg), to_device(fk, Wu), _dev(fk, x), m, variant, out, ws)
        got = out.to_numpy(np.uint16, (m, inter))
        _, g = oracle.qgemm_bf16w(Wg, x, None, want_acc=True)
        _, u = oracle.qgemm_bf16w(Wu, x, None, want_acc=True)
        step = 37 * (m // 512)
        want = np.array([[oracle.swiglu_scalar(float(a), float(b), variant) for a, b in zip(g[r], u[r])] for r in range(0, m, step)],
                        dtype=np.uint16)
        sel = got[::step]
        gf, wf = oracle.bf16_to_f32(sel).astype(np.float64), oracle.bf16_to_f32(want).astype(np.float64)
        assert np.linalg.norm(gf - wf) / np.linalg.norm(wf) <= 1e-2
        assert np.mean(sel != want) <= 0.05          # fp32 summation order may cross a bf16 rounding edge
    finally:
        fk.set_gemm_library_rows(fk.GEMM_LIBRARY_ROWS_DEFAULT)


@pytest.mark.parametrize("m,n,k", [(1, 64, 64), (7, 333, 256), (100, 1152, 896), (512, 256, 4864)])
def test_qgemm_dense_bf16_weights(fk, m, n, k):
    """bits = 16: the plain library GEMM (fp32 accumulate) with this library's epilogue."""
    W = make_qweight(80, n, k, 16)
    x = normal_bf16(81, (m, k))
    bias, res = normal_bf16(82, n), normal_bf16(83, (m, n))
    got = _run(fk, W, x)
    for r in range(0, m, 5):
        _check(got[r], oracle.qgemv(W, x[r]), oracle.linear_acc(W, x[r]), W, x[r])
    got = _run(fk, W, x, bias=bias, res=res)
    for r in range(0, m, 5):
        full = oracle.linear_acc(W, x[r]) + oracle.bf16_to_f32(bias) + oracle.bf16_to_f32(res[r])
        _check(got[r], oracle.f32_to_bf16(full.astype(np.float32)), full, W, x[r])


def test_qgemm_rows_agree_with_gemv(fk):
    """Every row of the multi-row result lies within one rounding flip of the single-row kernel."""
    W = make_qweight(69, 1024, 2048, 4)
    x = normal_bf16(70, (6, 2048))
    got = _run(fk, W, x)
    dW = to_device(fk, W)
    for r in range(6):
        y = fk.DeviceBuffer(2 * 1024)
        fk.qgemv(dW, _dev(fk, x[r]), None, y)
        single = y.to_numpy(np.uint16)
        _check(got[r], single, oracle.linear_acc(W, x[r]), W, x[r])


def test_qgemm_rejects(fk):
    x = _dev(fk, normal_bf16(1, (2, 128)))
    y = fk.DeviceBuffer(2 * 2 * 64)
    ws = fk.DeviceBuffer(1 << 16)
    with pytest.raises(fk.FusekitError):
        fk.qgemm(to_device(fk, make_qweight(1, 64, 132, 16)), _dev(fk, normal_bf16(1, (2, 132))), 2, None, None, y, ws)  # dense rows not 16-byte aligned
    with pytest.raises(fk.InvalidArgument):
        fk.qgemm(to_device(fk, make_qweight(1, 64, 128, 16)), x, 2, None, None, y, None)     # dense weights need the workspace too
    with pytest.raises(fk.FusekitError):
        fk.qgemm(to_device(fk, make_qweight(1, 64, 128, 4, group=32)), x, 2, None, None, y, ws)
    with pytest.raises(fk.InvalidArgument):
        fk.qgemm(to_device(fk, make_qweight(1, 64, 128, 4)), x, 0, None, None, y, ws)
    with pytest.raises(fk.InvalidArgument):
        fk.qgemm(to_device(fk, make_qweight(1, 64, 128, 4)), x, 2, None, None, y, None)


def test_qgemm_family_in_a_graph_with_binding_update(fk):
    from fusekit_amd.runtime import Dispatch, Dispatcher, arg
    m, n, k = 8, 512, 1024
    W = make_qweight(71, n, k, 4)
    xa, xb = normal_bf16(72, (m, k)), normal_bf16(73, (m, k))
    res = normal_bf16(74, (m, n))
    dW, bxa, bxb, bres = to_device(fk, W), _dev(fk, xa), _dev(fk, xb), _dev(fk, res)
    y, ws = fk.DeviceBuffer(2 * m * n), fk.DeviceBuffer(fk.qgemm_workspace_bytes(m, n, k))
    d = Dispatcher()
    g = d.build_graph([Dispatch("fusekit_qgemm_f0", [arg(bxa), arg(dW.w), arg(dW.scales), arg(dW.biases), arg(bres),
                                                      arg(y), arg(ws)],
                                {"bits": 4, "group": 64, "m": k, "n": n, "rows": m, "has_residual": 1})])
    d.execute_graph(g)
    assert np.array_equal(y.to_numpy(np.uint16, (m, n)), _run(fk, W, xa, res=res))
    d.update_graph_bindings(g, [(0, 0, bxb.ptr, bxb.nbytes)])
    for _ in range(2):
        d.execute_graph(g)
        assert np.array_equal(y.to_numpy(np.uint16, (m, n)), _run(fk, W, xb, res=res))
