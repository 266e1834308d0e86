"""The safetensors container reader / writer and config.json mapping (no GPU)."""
import json
import struct

import numpy as np
import pytest


def _module():
    # the reader itself needs no device; import it without loading the HIP library
    import importlib.util
    import os
    import sys
    import types
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    try:
        from fusekit_amd import checkpoint
        return checkpoint
    except ImportError:
        pytest.skip("fusekit_amd library not built")


def test_safetensors_round_trip_and_validation(tmp_path):
    ck = _module()
    a = np.arange(24, dtype=np.uint32).reshape(4, 6)
    b = np.arange(8, dtype=np.uint16)
    path = str(tmp_path / "t.safetensors")
    ck.write_safetensors(path, [("w.weight", "U32", (4, 6), a), ("w.scales", "BF16", (4, 2), b)])
    f = ck.SafetensorsFile(path)
    data, dtype, shape = f.raw("w.weight")
    assert dtype == "U32" and shape == (4, 6) and np.array_equal(data.view(np.uint32).reshape(shape), a)
    data, dtype, shape = f.raw("w.scales")
    assert dtype == "BF16" and np.array_equal(data.view(np.uint16), b)
    f.close()
    # header layout as the format defines it: u64 length, JSON, data
    raw = open(path, "rb").read()
    (hlen,) = struct.unpack("<Q", raw[:8])
    head = json.loads(raw[8:8 + hlen])
    assert head["w.weight"]["data_offsets"] == [0, 96] and head["w.scales"]["data_offsets"] == [96, 112]
    # a tensor whose offsets disagree with its shape is refused
    head["w.scales"]["shape"] = [4, 3]
    text = json.dumps(head).encode()
    bad = str(tmp_path / "bad.safetensors")
    open(bad, "wb").write(struct.pack("<Q", len(text)) + text + raw[8 + hlen:])
    with pytest.raises(ValueError):
        ck.SafetensorsFile(bad)
    open(bad, "wb").write(b"\x01\x02")
    with pytest.raises(ValueError):
        ck.SafetensorsFile(bad)


def test_config_mapping():
    ck = _module()
    cfg = ck.config_from_json(dict(model_type="qwen3", hidden_size=2560, num_hidden_layers=36, num_attention_heads=32,
                                   num_key_value_heads=8, head_dim=128, intermediate_size=9728, vocab_size=151936,
                                   rms_norm_eps=1e-6, rope_theta=1000000, quantization=dict(group_size=64, bits=4)))
    assert (cfg.n_layers, cfg.hidden, cfg.n_heads, cfg.n_kv, cfg.head_dim, cfg.inter, cfg.vocab) == (36, 2560, 32, 8, 128, 9728, 151936)
    assert cfg.bits == 4 and cfg.group == 64 and cfg.theta == 1e6 and cfg.qk_norm and not cfg.qkv_bias
    dense = ck.config_from_json(dict(model_type="qwen2", hidden_size=896, num_hidden_layers=24, num_attention_heads=14,
                                     num_key_value_heads=2, intermediate_size=4864, vocab_size=151936))
    assert dense.bits == 16 and dense.head_dim == 64 and dense.qkv_bias
