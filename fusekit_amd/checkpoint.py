"""MLX-format checkpoints: `config.json` + `*.safetensors` as mlx-lm writes them for its quantised
models (`*.weight` uint32 packed, `*.scales`, `*.biases`, `config.json: quantization{group_size, bits}`;
the reference reads the same files, src/fusion/ir.rs:600-700, 1033-1080).

The safetensors container is read here directly (8-byte little-endian header length, a JSON header
of name -> {dtype, shape, data_offsets}, then the raw bytes), through a memory map, tensor by tensor
straight into HBM: nothing is unpickled, no array the size of the model is ever held on the host,
and bf16 needs no numpy dtype.  The writer exists for tests and for exporting a random-init model.
"""
from __future__ import annotations

import json
import os
import struct
from typing import Dict, Iterable, Tuple

import numpy as np

from . import native
from .decoder import DecoderConfig, DecoderWeights
from .native import DeviceBuffer, DeviceWeight

_ITEM = {"U32": 4, "BF16": 2, "F16": 2, "F32": 4, "I32": 4, "U8": 1}


class SafetensorsFile:
    """Read-only view of one .safetensors file."""

    def __init__(self, path: str):
        self.path = path
        with open(path, "rb") as f:
            head = f.read(8)
            if len(head) != 8:
                raise ValueError(f"{path}: truncated safetensors header")
            (hlen,) = struct.unpack("<Q", head)
            if hlen > 128 * 1024 * 1024:                 # same sanity bound as src/fusion/ir.rs:1063
                raise ValueError(f"{path}: implausible header length {hlen}")
            self.header = json.loads(f.read(hlen))
        self.base = 8 + hlen
        self.tensors = {k: v for k, v in self.header.items() if k != "__metadata__"}
        size = os.path.getsize(path)
        for name, t in self.tensors.items():
            a, b = t["data_offsets"]
            n = int(np.prod(t["shape"], dtype=np.int64)) * _ITEM.get(t["dtype"], 0)
            if t["dtype"] not in _ITEM or b - a != n or self.base + b > size:
                raise ValueError(f"{path}: tensor {name} has inconsistent dtype / shape / offsets")

    def raw(self, name: str) -> Tuple[np.ndarray, str, Tuple[int, ...]]:
        """(bytes of the tensor as a read-only memory-mapped uint8 array, dtype label, shape)."""
        t = self.tensors[name]
        a, b = t["data_offsets"]
        data = np.memmap(self.path, dtype=np.uint8, mode="r", offset=self.base + a, shape=(b - a,))
        return data, t["dtype"], tuple(t["shape"])

    def close(self) -> None:
        pass  # every tensor view owns its own mapping


def write_safetensors(path: str, tensors: Iterable[Tuple[str, str, Tuple[int, ...], np.ndarray]]) -> None:
    """tensors: (name, dtype label, shape, array whose bytes are the data)."""
    header, blobs, off = {}, [], 0
    for name, dtype, shape, arr in tensors:
        data = np.ascontiguousarray(arr).view(np.uint8).ravel()
        assert data.size == int(np.prod(shape, dtype=np.int64)) * _ITEM[dtype], name
        header[name] = {"dtype": dtype, "shape": list(shape), "data_offsets": [off, off + data.size]}
        blobs.append(data)
        off += data.size
    header["__metadata__"] = {"format": "mlx"}
    text = json.dumps(header, separators=(",", ":")).encode()
    text += b" " * (-len(text) % 8)
    with open(path, "wb") as f:
        f.write(struct.pack("<Q", len(text)))
        f.write(text)
        for b in blobs:
            f.write(b.tobytes())


def config_from_json(cfg_json: dict, capacity: int = 1024) -> DecoderConfig:
    """DecoderConfig from an mlx-lm / HF `config.json` of a dense llama/qwen-style decoder."""
    c = cfg_json.get("text_config", cfg_json)
    q = cfg_json.get("quantization") or {}
    heads = int(c["num_attention_heads"])
    hidden = int(c["hidden_size"])
    return DecoderConfig(
        n_layers=int(c["num_hidden_layers"]), hidden=hidden, n_heads=heads,
        n_kv=int(c.get("num_key_value_heads", heads)), head_dim=int(c.get("head_dim", hidden // heads)),
        inter=int(c["intermediate_size"]), vocab=int(c["vocab_size"]), eps=float(c.get("rms_norm_eps", 1e-6)),
        theta=float(c.get("rope_theta", 10000.0)), bits=int(q.get("bits", 16)), group=int(q.get("group_size", 64)),
        qk_norm=bool(c.get("qk_norm", c.get("model_type") in ("qwen3",))), qkv_bias=bool(c.get("attention_bias", c.get("model_type") in ("qwen2",))),
        swiglu_variant=1, capacity=capacity)


_LAYER_MATS = ("self_attn.q_proj", "self_attn.k_proj", "self_attn.v_proj", "self_attn.o_proj",
               "mlp.gate_proj", "mlp.up_proj", "mlp.down_proj")


def load_mlx_checkpoint(model_dir: str, capacity: int = 1024) -> Tuple[DecoderConfig, DecoderWeights]:
    """Reads config.json and every *.safetensors of `model_dir` into HBM.  Names follow mlx-lm
    (`model.layers.N.self_attn.q_proj.weight|scales|biases|bias`, `model.embed_tokens.*`,
    `model.norm.weight`, optional `lm_head.*`)."""
    cfg = config_from_json(json.load(open(os.path.join(model_dir, "config.json"))), capacity)
    files = [SafetensorsFile(os.path.join(model_dir, f)) for f in sorted(os.listdir(model_dir)) if f.endswith(".safetensors")]
    if not files:
        raise FileNotFoundError(f"no .safetensors file in {model_dir}")
    where: Dict[str, SafetensorsFile] = {}
    for f in files:
        for name in f.tensors:
            where[name] = f

    def upload(name: str, want_dtype: str) -> Tuple[DeviceBuffer, Tuple[int, ...]]:
        if name not in where:
            raise KeyError(f"checkpoint has no tensor {name}")
        data, dtype, shape = where[name].raw(name)
        if dtype != want_dtype:
            raise ValueError(f"{name}: dtype {dtype}, this backend needs {want_dtype} "
                             "(activations and quantisation metadata are bfloat16)")
        return DeviceBuffer.from_numpy(data), shape

    def matrix(prefix: str, n: int, k: int) -> DeviceWeight:
        W = DeviceWeight.__new__(DeviceWeight)
        quantised = (prefix + ".scales") in where
        W.n, W.k = n, k
        if quantised:
            W.bits, W.group = cfg.bits, cfg.group
            W.w, shape = upload(prefix + ".weight", "U32")
            if tuple(shape) != (n, k * cfg.bits // 32):
                raise ValueError(f"{prefix}.weight: shape {shape}, expected {(n, k * cfg.bits // 32)}")
            W.scales, sshape = upload(prefix + ".scales", "BF16")
            W.biases, _ = upload(prefix + ".biases", "BF16")
            if tuple(sshape) != (n, k // cfg.group):
                raise ValueError(f"{prefix}.scales: shape {sshape}, expected {(n, k // cfg.group)}")
        else:
            W.bits, W.group, W.scales, W.biases = 16, 0, None, None
            W.w, shape = upload(prefix + ".weight", "BF16")
            if tuple(shape) != (n, k):
                raise ValueError(f"{prefix}.weight: shape {shape}, expected {(n, k)}")
        return W

    w = DecoderWeights(cfg)
    dims = {"self_attn.q_proj": (cfg.n_q, cfg.hidden), "self_attn.k_proj": (cfg.n_kvd, cfg.hidden),
            "self_attn.v_proj": (cfg.n_kvd, cfg.hidden), "self_attn.o_proj": (cfg.hidden, cfg.n_q),
            "mlp.gate_proj": (cfg.inter, cfg.hidden), "mlp.up_proj": (cfg.inter, cfg.hidden),
            "mlp.down_proj": (cfg.hidden, cfg.inter)}
    w.mats["embed_tokens"] = matrix("model.embed_tokens", cfg.vocab, cfg.hidden)
    if "lm_head.weight" in where:
        w.mats["lm_head"] = matrix("lm_head", cfg.vocab, cfg.hidden)
    w.vecs["final_norm"], _ = upload("model.norm.weight", "BF16")
    cfg.qkv_bias = "model.layers.0.self_attn.q_proj.bias" in where
    cfg.qk_norm = "model.layers.0.self_attn.q_norm.weight" in where
    for l in range(cfg.n_layers):
        src, dst = f"model.layers.{l}.", f"layers.{l}."
        for m in _LAYER_MATS:
            w.mats[dst + m] = matrix(src + m, *dims[m])
        w.vecs[dst + "input_layernorm"], _ = upload(src + "input_layernorm.weight", "BF16")
        w.vecs[dst + "post_attention_layernorm"], _ = upload(src + "post_attention_layernorm.weight", "BF16")
        if cfg.qk_norm:
            w.vecs[dst + "self_attn.q_norm"], _ = upload(src + "self_attn.q_norm.weight", "BF16")
            w.vecs[dst + "self_attn.k_norm"], _ = upload(src + "self_attn.k_norm.weight", "BF16")
        if cfg.qkv_bias:
            for n in "qkv":
                w.vecs[dst + f"self_attn.{n}_proj.bias"], _ = upload(src + f"self_attn.{n}_proj.bias", "BF16")
    for f in files:
        f.close()
    native.sync()
    return cfg, w


def save_mlx_checkpoint(model_dir: str, cfg: DecoderConfig, w: DecoderWeights, model_type: str = "qwen3") -> None:
    """Writes `w` (downloaded from HBM) as config.json + model.safetensors in the mlx-lm layout."""
    os.makedirs(model_dir, exist_ok=True)
    tensors = []

    def matrix(name: str, W: DeviceWeight):
        if W.bits == 16:
            tensors.append((name + ".weight", "BF16", (W.n, W.k), W.w.to_numpy(np.uint16)))
        else:
            tensors.append((name + ".weight", "U32", (W.n, W.k * W.bits // 32), W.w.to_numpy(np.uint32)))
            tensors.append((name + ".scales", "BF16", (W.n, W.k // W.group), W.scales.to_numpy(np.uint16)))
            tensors.append((name + ".biases", "BF16", (W.n, W.k // W.group), W.biases.to_numpy(np.uint16)))

    def vector(name: str, v: DeviceBuffer):
        tensors.append((name, "BF16", (v.nbytes // 2,), v.to_numpy(np.uint16)))

    matrix("model.embed_tokens", w.mats["embed_tokens"])
    if "lm_head" in w.mats:
        matrix("lm_head", w.mats["lm_head"])
    vector("model.norm.weight", w.vecs["final_norm"])
    for l in range(cfg.n_layers):
        src, dst = f"layers.{l}.", f"model.layers.{l}."
        for m in _LAYER_MATS:
            matrix(dst + m, w.mats[src + m])
        vector(dst + "input_layernorm.weight", w.vecs[src + "input_layernorm"])
        vector(dst + "post_attention_layernorm.weight", w.vecs[src + "post_attention_layernorm"])
        if cfg.qk_norm:
            vector(dst + "self_attn.q_norm.weight", w.vecs[src + "self_attn.q_norm"])
            vector(dst + "self_attn.k_norm.weight", w.vecs[src + "self_attn.k_norm"])
        if cfg.qkv_bias:
            for n in "qkv":
                vector(dst + f"self_attn.{n}_proj.bias", w.vecs[src + f"self_attn.{n}_proj.bias"])
    write_safetensors(os.path.join(model_dir, "model.safetensors"), tensors)
    conf = dict(model_type=model_type, hidden_size=cfg.hidden, num_hidden_layers=cfg.n_layers,
                num_attention_heads=cfg.n_heads, num_key_value_heads=cfg.n_kv, head_dim=cfg.head_dim,
                intermediate_size=cfg.inter, vocab_size=cfg.vocab, rms_norm_eps=cfg.eps, rope_theta=cfg.theta,
                tie_word_embeddings="lm_head" not in w.mats)
    if cfg.bits != 16:
        conf["quantization"] = dict(group_size=cfg.group, bits=cfg.bits)
    json.dump(conf, open(os.path.join(model_dir, "config.json"), "w"), indent=1)
