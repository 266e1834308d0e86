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


# ---------------------------------------------------------------- mixture-of-experts layout (mlx-lm deepseek_v2)
#
# config.json keys as in DeepSeek-V2-Lite checkpoints: kv_lora_rank, qk_rope_head_dim, qk_nope_head_dim, v_head_dim,
# n_routed_experts, num_experts_per_tok, moe_intermediate_size, n_shared_experts, intermediate_size (dense layers),
# first_k_dense_replace, routed_scaling_factor; q_lora_rank must be absent / null (direct q_proj).  Expert matrices
# are the stacked `mlp.switch_mlp.{gate,up,down}_proj` tensors [E, n, k*bits/32] mlx-lm writes; the router
# `mlp.gate.weight` stays bf16.  The embedding is tied unless `lm_head.*` is present (then it must be bf16 too).

def moe_config_from_json(c: dict, capacity: int = 1024):
    from .moe_decoder import MoeConfig
    if c.get("q_lora_rank"):
        raise ValueError("low-rank query projections (q_lora_rank) are not supported: the model needs a direct q_proj")
    q = c.get("quantization") or {}
    return MoeConfig(
        n_layers=int(c["num_hidden_layers"]), hidden=int(c["hidden_size"]), n_heads=int(c["num_attention_heads"]),
        kv_lora_rank=int(c["kv_lora_rank"]), rope_dim=int(c["qk_rope_head_dim"]), nope_dim=int(c["qk_nope_head_dim"]),
        v_dim=int(c["v_head_dim"]), n_experts=int(c["n_routed_experts"]), top_k=int(c["num_experts_per_tok"]),
        moe_inter=int(c["moe_intermediate_size"]), n_shared=int(c.get("n_shared_experts") or 0),
        dense_inter=int(c["intermediate_size"]), first_dense=int(c.get("first_k_dense_replace", 0)), vocab=int(c["vocab_size"]),
        eps=float(c.get("rms_norm_eps", 1e-6)), theta=float(c.get("rope_theta", 1e4)),
        rope_traditional=bool(c.get("rope_traditional", True)), route_scale=float(c.get("routed_scaling_factor", 1.0)),
        bits=int(q.get("bits", 16)), group=int(q.get("group_size", 64)), capacity=capacity)


def save_moe_checkpoint(model_dir: str, cfg, w) -> None:
    """Writes a MoeWeights (downloaded from HBM) as config.json + model.safetensors in the mlx-lm deepseek_v2 layout."""
    os.makedirs(model_dir, exist_ok=True)
    tensors = []
    for path, W in w.mats.items():
        name = "model." + path
        lead = (W.n_experts,) if getattr(W, "n_experts", 0) else ()
        if W.bits == 16:
            tensors.append((name + ".weight", "BF16", lead + (W.n, W.k), W.w.to_numpy(np.uint16)))
        else:
            tensors.append((name + ".weight", "U32", lead + (W.n, W.k * W.bits // 32), W.w.to_numpy(np.uint32)))
            tensors.append((name + ".scales", "BF16", lead + (W.n, W.k // W.group), W.scales.to_numpy(np.uint16)))
            tensors.append((name + ".biases", "BF16", lead + (W.n, W.k // W.group), W.biases.to_numpy(np.uint16)))
    for path, v in w.vecs.items():
        if path.startswith("mlp.route_"):
            continue   # constants of the task list, rebuilt from the config on load
        name = "model.norm.weight" if path == "final_norm" else "model." + path + ".weight"
        tensors.append((name, "BF16", (v.nbytes // 2,), v.to_numpy(np.uint16)))
    write_safetensors(os.path.join(model_dir, "model.safetensors"), tensors)
    conf = dict(model_type="deepseek_v2", hidden_size=cfg.hidden, num_hidden_layers=cfg.n_layers, num_attention_heads=cfg.n_heads,
                num_key_value_heads=cfg.n_heads, kv_lora_rank=cfg.kv_lora_rank, q_lora_rank=None, qk_rope_head_dim=cfg.rope_dim,
                qk_nope_head_dim=cfg.nope_dim, v_head_dim=cfg.v_dim, n_routed_experts=cfg.n_experts,
                num_experts_per_tok=cfg.top_k, moe_intermediate_size=cfg.moe_inter, n_shared_experts=cfg.n_shared,
                intermediate_size=cfg.dense_inter, first_k_dense_replace=cfg.first_dense, vocab_size=cfg.vocab,
                rms_norm_eps=cfg.eps, rope_theta=cfg.theta, rope_traditional=cfg.rope_traditional,
                routed_scaling_factor=cfg.route_scale, tie_word_embeddings=True)
    if cfg.bits != 16:
        conf["quantization"] = dict(group_size=cfg.group, bits=cfg.bits)
    json.dump(conf, open(os.path.join(model_dir, "config.json"), "w"), indent=1)


def load_moe_checkpoint(model_dir: str, capacity: int = 1024):
    """config.json (model_type deepseek_v2, no q_lora_rank) and every *.safetensors of `model_dir` into a
    (MoeConfig, MoeWeights) pair in HBM; shapes are checked against the config tensor by tensor."""
    from .moe_decoder import MoeWeights, _bf16
    cfg = moe_config_from_json(json.load(open(os.path.join(model_dir, "config.json"))), capacity)
    if cfg.bits == 16:
        raise ValueError("the mixture-of-experts decoder takes 4- or 8-bit projections (config.json has no quantization block)")
    files = [SafetensorsFile(os.path.join(model_dir, f)) for f in sorted(os.listdir(model_dir)) if f.endswith(".safetensors")]
    if not files:
        raise FileNotFoundError(f"no .safetensors file in {model_dir}")
    where = {name: f for f in files for name in f.tensors}

    def upload(name: str, want_dtype: str, want_shape) -> DeviceBuffer:
        if name not in where:
            raise KeyError(f"checkpoint has no tensor {name}")
        data, dtype, shape = where[name].raw(name)
        if dtype != want_dtype:
            raise ValueError(f"{name}: dtype {dtype}, this backend needs {want_dtype}")
        if tuple(shape) != tuple(want_shape):
            raise ValueError(f"{name}: shape {tuple(shape)}, expected {tuple(want_shape)}")
        return DeviceBuffer.from_numpy(data)

    c, w = cfg, MoeWeights(cfg)

    def matrix(path: str, n: int, k: int, experts: int = 0, dense: bool = False):
        W = DeviceWeight.__new__(DeviceWeight)
        W.n, W.k = n, k
        lead = (experts,) if experts else ()
        if dense:
            W.bits, W.group, W.scales, W.biases = 16, 0, None, None
            W.w = upload("model." + path + ".weight", "BF16", lead + (n, k))
        else:
            W.bits, W.group = c.bits, c.group
            W.w = upload("model." + path + ".weight", "U32", lead + (n, k * c.bits // 32))
            W.scales = upload("model." + path + ".scales", "BF16", lead + (n, k // c.group))
            W.biases = upload("model." + path + ".biases", "BF16", lead + (n, k // c.group))
        if experts:
            W.n_experts = experts
        w.mats[path] = W

    def vector(path: str, n: int, name: str = None):
        w.vecs[path] = upload(name or "model." + path + ".weight", "BF16", (n,))

    matrix("embed_tokens", c.vocab, c.hidden, dense=True)
    vector("final_norm", c.hidden, "model.norm.weight")
    for l in range(c.n_layers):
        p = f"layers.{l}."
        vector(p + "input_layernorm", c.hidden)
        vector(p + "post_attention_layernorm", c.hidden)
        matrix(p + "self_attn.q_proj", c.n_heads * c.qk_dim, c.hidden)
        matrix(p + "self_attn.kv_a_proj_with_mqa", c.kv_lora_rank + c.rope_dim, c.hidden)
        vector(p + "self_attn.kv_a_layernorm", c.kv_lora_rank)
        matrix(p + "self_attn.kv_b_proj", c.n_heads * (c.nope_dim + c.v_dim), c.kv_lora_rank)
        matrix(p + "self_attn.o_proj", c.hidden, c.n_heads * c.v_dim)
        if l < c.first_dense:
            matrix(p + "mlp.gate_proj", c.dense_inter, c.hidden)
            matrix(p + "mlp.up_proj", c.dense_inter, c.hidden)
            matrix(p + "mlp.down_proj", c.hidden, c.dense_inter)
        else:
            matrix(p + "mlp.gate", c.n_experts, c.hidden, dense=True)
            for nm in ("gate_proj", "up_proj"):
                matrix(p + f"mlp.switch_mlp.{nm}", c.moe_inter, c.hidden, c.n_experts)
                matrix(p + f"mlp.shared_experts.{nm}", c.shared_inter, c.hidden)
            matrix(p + "mlp.switch_mlp.down_proj", c.hidden, c.moe_inter, c.n_experts)
            matrix(p + "mlp.shared_experts.down_proj", c.hidden, c.shared_inter)
    w.vecs["mlp.route_scale"] = DeviceBuffer.from_numpy(_bf16(np.array([c.route_scale], np.float32)))
    w.vecs["mlp.route_rows"] = DeviceBuffer.from_numpy(np.arange(c.top_k, dtype=np.uint32))
    for f in files:
        f.close()
    native.sync()
    return cfg, w
