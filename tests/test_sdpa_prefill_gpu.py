"""Causal attention of a group of rows on the matrix cores (fk_sdpa_prefill) against the oracle's
restatement of the reference's prefill kernel (src/codegen/kernels/sdpa_prefill.rs).
Tolerance: rel-L2 <= 1e-2 against the oracle (bf16 activations, fp32 softmax; the probabilities
enter the second matrix product rounded to bf16, which bounds each output's error by
2^-9 * sum_j p_j |v_j|)."""
import numpy as np
import pytest

import oracle
from helpers import normal_bf16, rel_l2

pytestmark = pytest.mark.gpu
REL_L2_BAR = 1e-2


def _case(fk, rows, kv_len, n_heads, n_kv, D, cap, seed=0, poison=True):
    q = normal_bf16(seed, rows * n_heads * D)
    ck, cv = normal_bf16(seed + 1, n_kv * cap * D), normal_bf16(seed + 2, n_kv * cap * D)
    if poison:  # cache rows that hold no token yet must never be read
        for c in (ck, cv):
            c.reshape(n_kv, cap, D)[:, kv_len:] = 0x7FC0
    scale = 1.0 / np.sqrt(D)
    dq, dck, dcv = (fk.DeviceBuffer.from_numpy(t) for t in (q, ck, cv))
    out = fk.DeviceBuffer(2 * rows * n_heads * D)
    fk.sdpa_prefill(dq, dck, dcv, out, rows, kv_len, n_heads, n_kv, D, cap, scale)
    fk.sync()
    got = out.to_numpy(np.uint16)
    ref = oracle.sdpa_prefill(q, ck, cv, rows, n_heads, n_kv, D, kv_len, cap, scale)
    g = oracle.bf16_to_f32(got).astype(np.float64).reshape(rows, n_heads, D)
    r = oracle.bf16_to_f32(ref).astype(np.float64).reshape(rows, n_heads, D)
    assert np.isfinite(g).all()
    assert rel_l2(got, r) <= REL_L2_BAR
    # per row and head as well (one wrong row of 128 would hide in the global norm)
    num = np.linalg.norm(g - r, axis=2)
    den = np.maximum(np.linalg.norm(r, axis=2), 1e-30)
    assert float((num / den).max()) <= REL_L2_BAR, np.unravel_index(np.argmax(num / den), num.shape)
    # element-wise: |v| <~ 4 for N(0,1) rows, so 2^-9 * 4 bounds the effect of rounding the probabilities
    assert float(np.abs(g - r).max()) <= 2.0 ** -8 * np.abs(r).max() + 2.0 ** -7
    return q, ck, cv, got


@pytest.mark.parametrize("rows,kv_len", [(1, 1), (2, 2), (5, 5), (31, 31), (32, 32), (33, 33), (64, 64), (100, 100), (128, 128)])
def test_fresh_group(fk, rows, kv_len):
    _case(fk, rows, kv_len, 32, 8, 128, 256)


@pytest.mark.parametrize("rows,kv_len", [(1, 300), (7, 300), (32, 64), (64, 65), (64, 1000), (128, 640), (128, 1024), (97, 513)])
def test_group_after_earlier_tokens(fk, rows, kv_len):
    _case(fk, rows, kv_len, 32, 8, 128, 1024, seed=3)


@pytest.mark.parametrize("n_heads,n_kv,D", [(14, 2, 64), (8, 8, 64), (6, 2, 128), (16, 1, 128), (3, 3, 64)])
def test_head_layouts(fk, n_heads, n_kv, D):
    _case(fk, 45, 333, n_heads, n_kv, D, 512, seed=7)


@pytest.mark.parametrize("rows,kv_len", [(65, 65), (129, 129), (200, 200), (256, 256), (300, 900), (512, 512), (512, 1536), (1000, 1000)])
@pytest.mark.parametrize("n_heads,n_kv,D", [(8, 2, 128), (6, 3, 64)])
def test_large_groups_few_heads(fk, rows, kv_len, n_heads, n_kv, D):
    """Many rows, few heads: still the form whose waves split the positions (one block per 32 rows)."""
    _case(fk, rows, kv_len, n_heads, n_kv, D, 1600, seed=13)


@pytest.mark.parametrize("rows,kv_len", [(129, 129), (200, 200), (300, 900), (512, 512), (512, 1536), (640, 700)])
@pytest.mark.parametrize("n_heads,n_kv,D", [(64, 8, 128), (48, 12, 64)])
def test_large_groups_many_heads(fk, rows, kv_len, n_heads, n_kv, D):
    """Enough (head, 32-row) tiles that the first form would need several rounds over the CUs: the
    library takes the form with one block per 128 rows, whose waves share K and V through LDS."""
    _case(fk, rows, kv_len, n_heads, n_kv, D, 1600, seed=17)


def test_first_row_of_fresh_group_is_v0(fk):
    q, ck, cv, got = _case(fk, 40, 40, 32, 8, 128, 64, seed=11)
    v0 = cv.reshape(8, 64, 128)[:, 0]  # softmax over the one visible position is 1
    assert np.array_equal(got.reshape(40, 8, 4, 128)[0], np.repeat(v0[:, None], 4, 1))


def test_long_context_against_oracle(fk):
    _case(fk, 128, 4096 + 128, 32, 8, 128, 4352, seed=5)


def test_full_context_rows_match_single_row_attention(fk):
    """At the cache's full length the oracle's causal attention over 128 rows takes minutes: check
    the rows against the single-row oracle (the same arithmetic over the positions a row sees, pinned
    to agree with the causal form) on a few rows, and all rows against the library's own
    single-row kernel."""
    rows, kv_len, n_heads, n_kv, D, cap = 128, 32768, 32, 8, 128, 32768
    q = normal_bf16(21, rows * n_heads * D)
    ck, cv = normal_bf16(22, n_kv * cap * D), normal_bf16(23, n_kv * cap * D)
    scale = 1.0 / np.sqrt(D)
    dq, dck, dcv = (fk.DeviceBuffer.from_numpy(t) for t in (q, ck, cv))
    out = fk.DeviceBuffer(2 * rows * n_heads * D)
    fk.sdpa_prefill(dq, dck, dcv, out, rows, kv_len, n_heads, n_kv, D, cap, scale)
    fk.sync()
    got = out.to_numpy(np.uint16).reshape(rows, n_heads * D)
    for r in (0, 63, 127):
        ref = oracle.sdpa_decode(q.reshape(rows, -1)[r], ck, cv, n_heads, n_kv, D, D, kv_len - rows + r + 1, cap, scale)
        assert rel_l2(got[r], oracle.bf16_to_f32(ref)) <= REL_L2_BAR
    pb, cb = fk.sdpa_workspace_bytes(n_heads, n_kv, D, D, kv_len)
    part, cnt = fk.DeviceBuffer(max(pb, 4) * rows), fk.zeros(max(cb, 4) * rows)
    out2 = fk.DeviceBuffer(2 * rows * n_heads * D)
    fk.sdpa_decode_rows(dq, dck, dcv, out2, rows, kv_len - rows + 1, n_heads, n_kv, D, D, cap, scale, part, cnt)
    fk.sync()
    assert rel_l2(got, oracle.bf16_to_f32(out2.to_numpy(np.uint16))) <= REL_L2_BAR


def test_same_bits_on_a_second_launch(fk):
    q, ck, cv, got = _case(fk, 70, 500, 32, 8, 128, 512, seed=9)
    dq, dck, dcv = (fk.DeviceBuffer.from_numpy(t) for t in (q, ck, cv))
    out = fk.DeviceBuffer(2 * 70 * 32 * 128)
    fk.sdpa_prefill(dq, dck, dcv, out, 70, 500, 32, 8, 128, 512, 1.0 / np.sqrt(128))
    fk.sync()
    assert np.array_equal(out.to_numpy(np.uint16), got)  # no dependence on block scheduling


def test_rejects_bad_arguments(fk):
    b = fk.zeros(1 << 16)
    ok = dict(rows=4, kv_len=8, n_heads=4, n_kv=2, head_dim=64, capacity=16)

    def call(**kw):
        a = dict(ok, **kw)
        fk.sdpa_prefill(b, b, b, b, a["rows"], a["kv_len"], a["n_heads"], a["n_kv"], a["head_dim"], a["capacity"], 0.125)

    call()
    fk.sync()
    for bad in (dict(rows=0), dict(kv_len=3), dict(kv_len=17), dict(n_heads=5), dict(head_dim=96), dict(head_dim=256)):
        with pytest.raises(fk.FusekitError):
            call(**bad)
    with pytest.raises(fk.FusekitError):
        fk.sdpa_prefill(None, b, b, b, 4, 8, 4, 2, 64, 16, 0.125)
