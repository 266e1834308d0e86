"""GPU parity of the streaming GEMV family (K1, K1r, N, K2, K3a, H) against the CPU oracle.

Bars: rel-L2 <= 1e-2 against the fp32 reference (north star); in practice the
kernel and the oracle share every bf16 rounding boundary, so outputs may differ
only where fp32 summation order moves a value across a bf16 rounding edge:
at most 1 bf16 ulp, on a small fraction of elements.
"""
import numpy as np
import pytest

import oracle
from helpers import bf16_mismatch, make_qweight, normal_bf16, rel_l2, rng, to_device

pytestmark = pytest.mark.gpu

REL_L2_BAR = 1e-2      # stated tolerance (bf16 output vs fp32 CPU reference)
ULP_BAR = 1.0          # rounding-edge flips only
FLIP_FRACTION_BAR = 0.02


def _check(got, ref_bits, ref_f32, W=None, x=None):
    """rel-L2 bar, then element-wise: equal to the oracle except for rounding-edge
    flips (<= 1 bf16 ulp).  An accumulator that is a near-total cancellation may
    differ by more ulps of its tiny value while staying inside the fp32 summation
    bound 2e-6 * sum|x*w| (checked when W and x are given)."""
    assert rel_l2(got, ref_f32) <= REL_L2_BAR
    frac, ulps = bf16_mismatch(got, ref_bits)
    assert frac <= FLIP_FRACTION_BAR, f"{frac:.4f} of outputs differ from oracle"
    if ulps <= ULP_BAR:
        return
    assert W is not None, f"differs from oracle by {ulps} bf16 ulps"
    gf, rf = oracle.bf16_to_f32(got).astype(np.float64), oracle.bf16_to_f32(ref_bits).astype(np.float64)
    mag = np.maximum(np.abs(gf), np.abs(rf))
    ulp = 2.0 ** (np.floor(np.log2(np.maximum(mag, 1e-38))) - 7)
    ax = np.abs(oracle.bf16_to_f32(x)).astype(np.float64)
    for i in np.nonzero(np.abs(gf - rf) > ULP_BAR * ulp)[0]:
        scale = float(np.abs(oracle.dequantize_rows(W, i, i + 1)[0]).astype(np.float64) @ ax)
        assert abs(gf[i] - rf[i]) <= 2e-6 * scale + 2.0 ** -8 * abs(rf[i]), \
            f"row {i}: got {gf[i]!r} ref {rf[i]!r} (sum|xw| = {scale!r})"


SHAPES = [
    (4864, 896),    # config 1 / gate, up at hidden 896
    (896, 4864),    # down projection at hidden 896
    (1152, 896),
    (2560, 9728),   # 4B-class down projection
    (4096, 2560),
    (333, 128),     # ragged N, small K
    (1, 64),        # single row, single group
    (70, 10944),    # long rows (MoE dense layer)
]


@pytest.mark.parametrize("bits", [4, 8, 16])
@pytest.mark.parametrize("n,k", SHAPES)
def test_qgemv_matches_oracle(fk, n, k, bits):
    W = make_qweight(100 + n + k, n, k, bits)
    x = normal_bf16(7, k)
    dW, dx = to_device(fk, W), fk.DeviceBuffer.from_numpy(x)
    dy = fk.DeviceBuffer(2 * n)
    fk.qgemv(dW, dx, None, dy)
    got = dy.to_numpy(np.uint16)
    acc = oracle.linear_acc(W, x)
    _check(got, oracle.qgemv(W, x), acc, W, x)
    # textbook x @ dequant(W)^T in float64 (library routine)
    ref64 = oracle.dequantize(W).astype(np.float64) @ oracle.bf16_to_f32(x).astype(np.float64)
    assert rel_l2(got, ref64) <= REL_L2_BAR


def test_qgemv_vocab_sized_matches_oracle(fk):
    """The 219 MB shape whose streaming rate the kernel bench reports (1536 blocks, many tiles per block)."""
    n, k = 151936, 2560
    W = make_qweight(4242, n, k, 4)
    x = normal_bf16(9, k)
    dW, dx = to_device(fk, W), fk.DeviceBuffer.from_numpy(x)
    dy = fk.DeviceBuffer(2 * n)
    fk.qgemv(dW, dx, None, dy)
    _check(dy.to_numpy(np.uint16), oracle.qgemv(W, x), oracle.linear_acc(W, x), W, x)


# Shapes of the row-group kernel form (sixteen lanes per row, four rows per wave and pass): batches of 5, 4 and 3
# column blocks, rows whose last batch has unused slots (9728 / int4: 19 column blocks in batches of 5; 9728 / int8:
# 38 in batches of 3; 2432 / bf16: 19 in batches of 5), a row count that is not a multiple of four.
ROW_GROUP_SHAPES = [
    (8201, 2560, 4), (8201, 9728, 4), (8196, 4096, 4), (8202, 2048, 8), (8201, 9728, 8), (8201, 2560, 16),
    (8199, 1536, 16), (8203, 2432, 16), (8201, 1536, 4),
]


@pytest.mark.parametrize("n,k,bits", ROW_GROUP_SHAPES)
def test_qgemv_row_group_form_matches_oracle_and_flat_form(fk, n, k, bits):
    assert fk.gemv_form(n, k, bits) == 1, "the planner is expected to pick the row-group form for this shape"
    W = make_qweight(300 + n + k, n, k, bits)
    x = normal_bf16(17, k)
    dW, dx = to_device(fk, W), fk.DeviceBuffer.from_numpy(x)
    dy = fk.DeviceBuffer(2 * n)
    fk.qgemv(dW, dx, None, dy)
    got = dy.to_numpy(np.uint16)
    _check(got, oracle.qgemv(W, x), oracle.linear_acc(W, x), W, x)
    # the flat form on the same operands: both forms share every rounding boundary and differ in summation order only
    fk.set_gemv_flat_only(True)
    try:
        assert fk.gemv_form(n, k, bits) == 0
        dz = fk.DeviceBuffer(2 * n)
        fk.qgemv(dW, dx, None, dz)
    finally:
        fk.set_gemv_flat_only(False)
    flat = dz.to_numpy(np.uint16)
    _check(got, flat, oracle.bf16_to_f32(flat), W, x)


def test_row_group_form_with_fused_final_norm(fk):
    hidden, vocab = 2560, 20011
    assert fk.gemv_form(vocab, hidden, 4) == 1
    W = make_qweight(61, vocab, hidden, 4)
    x = normal_bf16(1, hidden, 3.0)
    gamma = normal_bf16(2, hidden, 0.1, 1.0)
    dl = fk.DeviceBuffer(2 * vocab)
    fk.final_rmsnorm_lm_head(fk.DeviceBuffer.from_numpy(x), fk.DeviceBuffer.from_numpy(gamma), 1e-6,
                             to_device(fk, W), dl)
    ref = oracle.final_rmsnorm_lm_head(x, gamma, 1e-6, W)
    ny = oracle.rmsnorm(x, gamma, 1e-6)
    _check(dl.to_numpy(np.uint16), ref, oracle.linear_acc(W, ny), W, ny)


def _greedy(logits_bf16: np.ndarray) -> int:
    """Largest bf16 logit, lowest index on ties, NaN never wins (argmax_logits_decode.rs:63-95)."""
    v = oracle.bf16_to_f32(logits_bf16).astype(np.float64)
    v = np.where(np.isnan(v), -np.inf, v)
    return int(np.argmax(v)) if np.isfinite(v).any() or np.isinf(v).any() else 0


@pytest.mark.parametrize("bits,hidden", [(16, 2560), (4, 2560), (8, 1024), (4, 3072), (16, 2432), (4, 9728)])
def test_direct_head_argmax_matches_the_two_launches(fk, bits, hidden):
    """The LM head that selects the token itself: same logits, bit for bit, as the plain head, and the token the
    stand-alone argmax picks over them -- with the winning row repeated (lowest index must win, also against a copy
    in the last, partial group of four rows), twice in a row on one workspace, then with another winner."""
    vocab = 20011
    assert fk.gemv_form(vocab, hidden, bits) == 1
    W = make_qweight(62, vocab, hidden, bits)
    x = normal_bf16(1, hidden, 3.0)
    gamma = normal_bf16(2, hidden, 0.1, 1.0)
    dx, dg = fk.DeviceBuffer.from_numpy(x), fk.DeviceBuffer.from_numpy(gamma)
    base = oracle.final_rmsnorm_lm_head(x, gamma, 1e-6, W)
    win = _greedy(base)
    copies = sorted({win, (win + 4097) % vocab, vocab - 1, (win + 13) % vocab})
    for r in copies:                                      # identical rows -> identical logits
        W.w[r] = W.w[win]
        if bits != 16:
            W.scales[r], W.biases[r] = W.scales[win], W.biases[win]
    if bits == 16:
        W.w[(copies[0] + 1) % vocab, 5] = 0x7FC0         # a NaN logit never wins
    dW = to_device(fk, W)
    plain = fk.DeviceBuffer(2 * vocab)
    fk.final_rmsnorm_lm_head(dx, dg, 1e-6, dW, plain)
    want_logits = plain.to_numpy(np.uint16)
    tok2, ws2 = fk.zeros(4), fk.zeros(fk.ARGMAX_WORKSPACE_BYTES)
    fk.argmax_logits_decode(plain, vocab, tok2, None, None, 0, ws2)
    want = int(tok2.to_numpy(np.uint32)[0])
    assert want == copies[0] == _greedy(want_logits)

    ws = fk.zeros(fk.HEAD_ARGMAX_WORKSPACE_BYTES)
    tok, hist, cnt = fk.zeros(4), fk.zeros(4 * 4), fk.zeros(4)
    for rep in range(2):
        dl = fk.DeviceBuffer(2 * vocab)
        fk.final_rmsnorm_lm_head_argmax(dx, dg, 1e-6, dW, dl, tok, hist, cnt, 4, ws)
        assert np.array_equal(dl.to_numpy(np.uint16), want_logits)
        assert int(tok.to_numpy(np.uint32)[0]) == want
        assert int(cnt.to_numpy(np.uint32)[0]) == rep + 1
    assert hist.to_numpy(np.uint32).tolist() == [want, want, 0, 0]
    assert int(ws.to_numpy(np.uint32)[0]) == 0           # the block counter is back at zero

    # another activation vector: another winner through the same workspace, no history
    x2 = normal_bf16(9, hidden, 3.0)
    dl = fk.DeviceBuffer(2 * vocab)
    fk.final_rmsnorm_lm_head_argmax(fk.DeviceBuffer.from_numpy(x2), dg, 1e-6, dW, dl, tok, None, None, 0, ws)
    assert int(tok.to_numpy(np.uint32)[0]) == _greedy(dl.to_numpy(np.uint16))
    assert int(cnt.to_numpy(np.uint32)[0]) == 2


def test_direct_head_argmax_refuses_shapes_of_the_flat_form(fk):
    W = make_qweight(63, 2000, 896, 4)
    assert fk.gemv_form(2000, 896, 4) == 0
    with pytest.raises(fk.FusekitError) as e:
        fk.final_rmsnorm_lm_head_argmax(fk.DeviceBuffer(896 * 2), fk.DeviceBuffer(896 * 2), 1e-6, to_device(fk, W),
                                        fk.DeviceBuffer(4000), fk.zeros(4), None, None, 0,
                                        fk.zeros(fk.HEAD_ARGMAX_WORKSPACE_BYTES))
    assert e.value.status == 5 and "row-group" in str(e.value)
    with pytest.raises(fk.InvalidArgument):
        fk.final_rmsnorm_lm_head_argmax(fk.DeviceBuffer(896 * 2), fk.DeviceBuffer(896 * 2), 1e-6, to_device(fk, W),
                                        fk.DeviceBuffer(4000), None, None, None, 0, None)


def test_row_group_form_is_kept_for_the_shapes_it_was_built_for(fk):
    assert fk.gemv_form(151936, 2560, 4) == 1 and fk.gemv_form(151936, 2560, 16) == 1
    assert fk.gemv_form(2560, 2560, 4) == 0          # too few rows to fill the chip four rows a wave
    assert fk.gemv_form(20000, 896, 4) == 0          # rows are not whole 256-byte blocks
    assert fk.gemv_form(20000, 2560, 4, 32) == 0     # group size
    assert fk.gemv_form(20000, 12288, 4) == 0        # longer than the staging registers cover


@pytest.mark.parametrize("group", [32, 128])
@pytest.mark.parametrize("bits", [4, 8])
def test_qgemv_other_group_sizes(fk, bits, group):
    n, k = 512, 1024
    W = make_qweight(5, n, k, bits, group)
    x = normal_bf16(8, k)
    dy = fk.DeviceBuffer(2 * n)
    fk.qgemv(to_device(fk, W), fk.DeviceBuffer.from_numpy(x), None, dy)
    _check(dy.to_numpy(np.uint16), oracle.qgemv(W, x), oracle.linear_acc(W, x), W, x)


def test_qgemv_bias(fk):
    n, k = 1152, 896
    W = make_qweight(11, n, k)
    x, b = normal_bf16(1, k), normal_bf16(2, n, 0.5)
    dy = fk.DeviceBuffer(2 * n)
    fk.qgemv(to_device(fk, W), fk.DeviceBuffer.from_numpy(x), fk.DeviceBuffer.from_numpy(b), dy)
    _check(dy.to_numpy(np.uint16), oracle.qgemv(W, x, b), oracle.linear_acc(W, x) + oracle.bf16_to_f32(b), W, x)


@pytest.mark.parametrize("bits", [4, 8, 16])
@pytest.mark.parametrize("two", [False, True])
def test_linear_residual(fk, bits, two):
    n, k = 896, 4864
    W = make_qweight(12, n, k, bits)
    x, r1, r2 = normal_bf16(1, k), normal_bf16(2, n), normal_bf16(3, n)
    dy = fk.DeviceBuffer(2 * n)
    fk.linear_residual(to_device(fk, W), fk.DeviceBuffer.from_numpy(x), fk.DeviceBuffer.from_numpy(r1),
                       fk.DeviceBuffer.from_numpy(r2) if two else None, dy)
    ref = oracle.linear_residual(W, x, r1, r2 if two else None)
    f = oracle.linear_acc(W, x) + oracle.bf16_to_f32(r1) + (oracle.bf16_to_f32(r2) if two else 0)
    _check(dy.to_numpy(np.uint16), ref, f, W, x)


@pytest.mark.parametrize("bits", [4, 8, 16])
@pytest.mark.parametrize("hidden,nq,nkv,bias", [(896, 896, 128, True), (2560, 4096, 1024, False)])
def test_rmsnorm_qkv(fk, hidden, nq, nkv, bias, bits):
    Wq, Wk, Wv = (make_qweight(20 + i, n, hidden, bits) for i, n in enumerate((nq, nkv, nkv)))
    x = normal_bf16(1, hidden)
    gamma = normal_bf16(2, hidden, 0.1, 1.0)
    bs = [normal_bf16(30 + i, n, 0.5) if bias else None for i, n in enumerate((nq, nkv, nkv))]
    dq, dk, dv = fk.DeviceBuffer(2 * nq), fk.DeviceBuffer(2 * nkv), fk.DeviceBuffer(2 * nkv)
    dbs = [fk.DeviceBuffer.from_numpy(b) if bias else None for b in bs]
    fk.rmsnorm_qkv(fk.DeviceBuffer.from_numpy(x), fk.DeviceBuffer.from_numpy(gamma), 1e-6, to_device(fk, Wq),
                   to_device(fk, Wk), to_device(fk, Wv), dbs[0], dbs[1], dbs[2], dq, dk, dv)
    rq, rk, rv = oracle.rmsnorm_qkv(x, gamma, 1e-6, Wq, Wk, Wv, *bs)
    ny = oracle.rmsnorm(x, gamma, 1e-6)
    for got, ref, W, b in ((dq, rq, Wq, bs[0]), (dk, rk, Wk, bs[1]), (dv, rv, Wv, bs[2])):
        f = oracle.linear_acc(W, ny) + (oracle.bf16_to_f32(b) if bias else 0)
        _check(got.to_numpy(np.uint16), ref, f, W, ny)


@pytest.mark.parametrize("variant", [0, 1, 2])
@pytest.mark.parametrize("bits", [4, 8, 16])
@pytest.mark.parametrize("norm", [True, False])
def test_gateup_swiglu(fk, variant, bits, norm):
    hidden, inter = 896, 4864
    Wg, Wu = make_qweight(40, inter, hidden, bits), make_qweight(41, inter, hidden, bits)
    x = normal_bf16(1, hidden)
    gamma = normal_bf16(2, hidden, 0.1, 1.0)
    dout = fk.DeviceBuffer(2 * inter)
    fk.gateup_swiglu(fk.DeviceBuffer.from_numpy(x), fk.DeviceBuffer.from_numpy(gamma) if norm else None, 1e-6,
                     to_device(fk, Wg), to_device(fk, Wu), variant, dout)
    ref = oracle.gateup_swiglu(x, gamma if norm else None, 1e-6, Wg, Wu, variant)
    got = dout.to_numpy(np.uint16)
    # fp32 reference of silu(g) * u on unrounded accumulators
    ny = oracle.rmsnorm(x, gamma, 1e-6) if norm else x
    g, u = oracle.linear_acc(Wg, ny).astype(np.float64), oracle.linear_acc(Wu, ny).astype(np.float64)
    assert rel_l2(got, g / (1 + np.exp(-g)) * u) <= REL_L2_BAR
    _check_swiglu(got, ref, ny, Wg, Wu, variant)


def _check_swiglu(got, ref, ny, Wg, Wu, variant):
    """Outputs equal the oracle's except where fp32 summation order matters.

    Two legitimate causes: (1) gate or up crosses a bf16 rounding edge -- then the
    kernel must equal the oracle's epilogue evaluated on one of the two bf16
    neighbours of each accumulator; (2) an accumulator is a near-total
    cancellation, so its relative error is large though its absolute error stays
    within the fp32 summation bound ~1e-6 * sum|x*w|; then the output may move by
    that bound propagated through silu(g)*u, plus a few ulps of rounding."""
    bad = np.nonzero(got != ref)[0]
    assert bad.size <= FLIP_FRACTION_BAR * got.size
    if bad.size == 0:
        return
    ag, au = oracle.linear_acc(Wg, ny), oracle.linear_acc(Wu, ny)
    ax = np.abs(oracle.bf16_to_f32(ny)).astype(np.float64)

    def neighbours(v):
        lo = np.float32(v).view(np.uint32) & np.uint32(0xFFFF0000)
        return [np.uint32(lo).view(np.float32), np.uint32(lo + 0x10000).view(np.float32)]

    gf, rf = oracle.bf16_to_f32(got).astype(np.float64), oracle.bf16_to_f32(ref).astype(np.float64)
    for i in bad:
        cands = {oracle.swiglu_scalar(float(g), float(u), variant)
                 for g in neighbours(ag[i]) for u in neighbours(au[i])}
        if int(got[i]) in cands:
            continue
        sg = float(np.abs(oracle.dequantize_rows(Wg, i, i + 1)[0]).astype(np.float64) @ ax)
        su = float(np.abs(oracle.dequantize_rows(Wu, i, i + 1)[0]).astype(np.float64) @ ax)
        g, u = float(ag[i]), float(au[i])
        silu = g / (1.0 + np.exp(-g))
        tol = 4 * 2.0 ** -8 * abs(rf[i]) + 1e-6 * (1.1 * sg * (abs(u) + 1e-3) + su * (abs(silu) + 1e-3))
        assert abs(gf[i] - rf[i]) <= tol, f"row {i}: got {gf[i]!r} ref {rf[i]!r} tol {tol!r}"


def test_swiglu_4b_shape(fk):
    hidden, inter = 2560, 9728
    Wg, Wu = make_qweight(50, inter, hidden), make_qweight(51, inter, hidden)
    x = normal_bf16(1, hidden)
    gamma = normal_bf16(2, hidden, 0.1, 1.0)
    dout = fk.DeviceBuffer(2 * inter)
    fk.gateup_swiglu(fk.DeviceBuffer.from_numpy(x), fk.DeviceBuffer.from_numpy(gamma), 1e-6, to_device(fk, Wg),
                     to_device(fk, Wu), 0, dout)
    ref = oracle.gateup_swiglu(x, gamma, 1e-6, Wg, Wu, 0)
    _check_swiglu(dout.to_numpy(np.uint16), ref, oracle.rmsnorm(x, gamma, 1e-6), Wg, Wu, 0)


@pytest.mark.parametrize("bits", [16, 4])
def test_final_rmsnorm_lm_head(fk, bits):
    hidden, vocab = 896, 20011   # ragged vocabulary
    W = make_qweight(60, vocab, hidden, bits)
    x = normal_bf16(1, hidden, 3.0)
    gamma = normal_bf16(2, hidden, 0.1, 1.0)
    dl = fk.DeviceBuffer(2 * vocab)
    fk.final_rmsnorm_lm_head(fk.DeviceBuffer.from_numpy(x), fk.DeviceBuffer.from_numpy(gamma), 1e-6,
                             to_device(fk, W), dl)
    ref = oracle.final_rmsnorm_lm_head(x, gamma, 1e-6, W)
    ny = oracle.rmsnorm(x, gamma, 1e-6)
    _check(dl.to_numpy(np.uint16), ref, oracle.linear_acc(W, ny), W, ny)


def test_rejects_bad_shapes(fk):
    W = make_qweight(1, 8, 64)
    dW = to_device(fk, W)
    dW.k = 96  # not a multiple of 64
    with pytest.raises(fk.FusekitError):
        fk.qgemv(dW, fk.DeviceBuffer(256), None, fk.DeviceBuffer(16))
    dW.k, dW.bits = 64, 3
    with pytest.raises(fk.FusekitError):
        fk.qgemv(dW, fk.DeviceBuffer(256), None, fk.DeviceBuffer(16))


def test_plain_read_kernel_returns_the_xor_of_what_it_read(fk):
    """fk_read_reduce (the measurement aid behind bench.py's hbm_read_ceiling): every 16-byte piece is read exactly
    once -- the XOR over the per-workgroup words equals numpy's over the buffer, for sizes around the unrolled
    loop's edges."""
    for nbytes in (16, 4096 * 16, (256 * 8 * 256 * 8 + 3) * 16, 3 * 1000 * 1000 * 16):
        a = rng(nbytes % 1000).integers(0, 2 ** 32, nbytes // 4, dtype=np.uint32)
        src = fk.DeviceBuffer.from_numpy(a)
        out = fk.zeros(fk.read_reduce_out_bytes())
        fk.read_reduce(src, nbytes, out)
        fk.sync()
        q = a.reshape(-1, 4)
        x, y, z, w = (int(np.bitwise_xor.reduce(q[:, i])) for i in range(4))
        want = ((x ^ z) << 32) | (y ^ w)
        got = int(np.bitwise_xor.reduce(out.to_numpy(np.uint64)))
        assert got == want, nbytes
