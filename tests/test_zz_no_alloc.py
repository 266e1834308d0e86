"""The entry point that allocates nothing (fk_sdpa_decode_static) against fk_sdpa_decode, through the C ABI.

The split-K workspace is the library's static device array; results must be bit-identical to the entry point that
takes a caller-provided workspace (same kernel, same split), on two calls in a row, the second with a smaller
input (the array keeps the first call's contents)."""
import numpy as np
import pytest

from helpers import normal_bf16

pytestmark = pytest.mark.gpu


def _case(fk, n_heads, n_kv, dim, capacity, kv_len, seed):
    q = fk.DeviceBuffer.from_numpy(normal_bf16(seed, n_heads * dim))
    ck = fk.DeviceBuffer.from_numpy(normal_bf16(seed + 1, n_kv * capacity * dim))
    cv = fk.DeviceBuffer.from_numpy(normal_bf16(seed + 2, n_kv * capacity * dim))
    scale = 1.0 / float(np.sqrt(dim))
    pb, cb = fk.sdpa_workspace_bytes(n_heads, n_kv, dim, dim, capacity)
    partials, counters = fk.DeviceBuffer(max(pb, 16)), fk.zeros(max(cb, 16))
    want, got = fk.DeviceBuffer(n_heads * dim * 2), fk.DeviceBuffer(n_heads * dim * 2)
    fk.sdpa_decode(q, ck, cv, want, None, kv_len, capacity, n_heads, n_kv, dim, dim, capacity, scale, partials, counters)
    fk.sdpa_decode_static(q, ck, cv, got, None, kv_len, capacity, n_heads, n_kv, dim, dim, capacity, scale)
    fk.sync()
    a, b = want.to_numpy(np.uint16), got.to_numpy(np.uint16)
    assert a.any()
    assert np.array_equal(a, b), f"{np.count_nonzero(a != b)} of {a.size} outputs differ"


def test_static_scratch_attention_matches_the_workspace_entry_point(fk):
    _case(fk, 32, 8, 128, 4096, 4096, seed=1)      # 64 ranges merged through the static array
    _case(fk, 16, 4, 64, 1024, 700, seed=7)        # smaller problem right after: stale partial rows must not matter
    _case(fk, 32, 8, 128, 4096, 37, seed=11)       # one range: the direct path, counters untouched


def test_static_scratch_refuses_what_does_not_fit(fk):
    q = fk.DeviceBuffer(64 * 256 * 2)
    c = fk.DeviceBuffer(8 * 1024 * 256 * 2)
    out = fk.DeviceBuffer(64 * 256 * 2)
    with pytest.raises(fk.FusekitError) as e:
        # max_len only sizes the split: 64 heads x 256 dims x 65536 positions need 67 MB of partial rows
        fk.sdpa_decode_static(q, c, c, out, None, 5, 65536, 64, 8, 256, 256, 65536, 0.0625)
    assert "static scratch" in str(e.value)
