"""Dense decoder on the MI355X backend: random-init weights in HBM, the per-token task
list in the reference's decode_pipeline order and the generation loop.

Task order follows the reference's decode pipeline (src/codegen/task_graph_json.rs:54-65):
  step_init -> embed_lookup -> L x [ rmsnorm_qkv | rope(+head-norm) + KV store | sdpa |
  linear_residual(o_proj) | rmsnorm_gateup_swiglu | linear_residual(down_proj) ]
  -> final_rmsnorm_lm_head -> argmax (+ history).
The generation loop mirrors `_fast_generate_step`
(python/fusekit_runtime/__init__.py:4782-5141): prompt through the graph with forced
tokens, greedy first token, then native chunks of FK_CHUNK tokens with the argmax fed
back on the GPU.
"""
from __future__ import annotations

import ctypes as C
from dataclasses import dataclass
from typing import Dict, List, Optional, Sequence

import numpy as np

from . import native
from .native import DeviceBuffer, DeviceWeight, check, lib
from .runtime import FK_CHUNK, Dispatch, Dispatcher, arg, make_uniforms


@dataclass
class DecoderConfig:
    n_layers: int
    hidden: int
    n_heads: int
    n_kv: int
    head_dim: int
    inter: int
    vocab: int
    eps: float = 1e-6
    theta: float = 1e6
    bits: int = 4            # 4 / 8: MLX-affine projections; 16: dense bf16
    group: int = 64
    qk_norm: bool = False    # per-head q/k RMSNorm
    qkv_bias: bool = False
    swiglu_variant: int = 0
    capacity: int = 1024     # KV-cache rows per layer
    fuse_rope_store: bool = True   # one launch for rope_q + rope_kv_store (False: the reference's two)
    fuse_attention: bool = True    # graph mode, bf16 cache: rope/store + attention of a layer in one launch
    kv_bits: int = 0         # 0: bf16 KV cache; 4 / 8: quantised cache (mlx-lm QuantizedKVCache layout)
    kv_group: int = 64
    embed_scale: float = 1.0  # output_scale of the embedding lookup (embed_lookup_decode.rs:74-99)
    xcd_layers: bool = True   # graph mode: run a layer as two XCD-resident launches where the shape allows it
    xcd_spin_limit: int = 0   # bound of the XCD hand-over waits in polls (0: the library's default)
    direct_head_argmax: bool = True  # graph mode: the LM head selects the greedy token itself where its shape allows
    xcd_token_launch: bool = False  # the layers' launches of a token as ONE launch (device-wide barriers between them); slower at present
    xcd_layer_launch: bool = False  # a layer's two launches as ONE launch (attention phase, device-wide barrier, MLP phase)

    @property
    def n_q(self) -> int:
        return self.n_heads * self.head_dim

    @property
    def n_kvd(self) -> int:
        return self.n_kv * self.head_dim

    def layer_param_bytes(self) -> int:
        """Algorithmic weight bytes one token streams per layer (packed + scales + biases)."""
        per = self.bits / 8 + (0 if self.bits == 16 else 4 / self.group)
        params = self.hidden * (self.n_q + 2 * self.n_kvd) + self.n_q * self.hidden + 3 * self.inter * self.hidden
        return int(params * per)

    def token_bytes(self, ctx: int) -> int:
        """Algorithmic HBM bytes per decoded token at context `ctx`: layer weights + tied bf16
        LM head + K/V rows read by attention."""
        per_elem = 2.0 if not self.kv_bits else self.kv_bits / 8 + 4 / self.kv_group
        kv = int(self.n_layers * 2 * self.n_kv * self.head_dim * per_elem * ctx)
        return self.n_layers * self.layer_param_bytes() + self.vocab * self.hidden * 2 + kv


QWEN25_05B_LIKE = dict(n_layers=24, hidden=896, n_heads=14, n_kv=2, head_dim=64, inter=4864, vocab=151936,
                       qkv_bias=True)
DENSE_4B = dict(n_layers=36, hidden=2560, n_heads=32, n_kv=8, head_dim=128, inter=9728, vocab=151936, qk_norm=True)


def _synth(buf: DeviceBuffer, count: int, seed: int, mean: float, std: float, kind: int, bound: int = 0,
           row_len: int = 0, tau: float = 0.0, loud_rows: int = 0, loud_gain: float = 1.0) -> None:
    """kind 0 / 1: fp32 / bf16 normal, 2: uniform uint32 below `bound`; 3 / 4: fp32 / bf16 values a host can
    reproduce bit for bit (fk_synth_fill_exact), optionally with a log-normal-like spread of the row norms."""
    if kind >= 3:
        check(lib.fk_synth_fill_exact(C.c_void_p(buf.ptr), C.c_size_t(count), C.c_uint64(seed), C.c_float(mean),
                                      C.c_float(std), C.c_uint32(kind), C.c_size_t(row_len), C.c_float(tau),
                                      C.c_size_t(loud_rows), C.c_float(loud_gain), None))
        return
    check(lib.fk_synth_fill(C.c_void_p(buf.ptr), C.c_size_t(count), C.c_uint64(seed), C.c_float(mean),
                            C.c_float(std), C.c_uint32(kind), C.c_uint32(bound), None))


def quantize_on_device(w_f32: DeviceBuffer, n: int, k: int, bits: int, group: int) -> DeviceWeight:
    """fp32 [n, k] in HBM -> MLX-affine DeviceWeight (fk_quantize_affine)."""
    W = DeviceWeight.__new__(DeviceWeight)
    W.n, W.k, W.bits, W.group = n, k, bits, group
    W.w = DeviceBuffer(n * k * bits // 8)
    W.scales = DeviceBuffer(n * (k // group) * 2)
    W.biases = DeviceBuffer(n * (k // group) * 2)
    check(lib.fk_quantize_affine(C.c_void_p(w_f32.ptr), C.c_size_t(n), C.c_size_t(k), C.c_uint32(bits),
                                 C.c_uint32(group), C.c_void_p(W.w.ptr), C.c_void_p(W.scales.ptr),
                                 C.c_void_p(W.biases.ptr), None))
    return W


class DecoderWeights:
    """Weights of one model resident in HBM, keyed by the reference's parameter paths
    (`layers.<l>.self_attn.q_proj` ..., src/codegen/kernels/mod.rs:4907-4939)."""

    def __init__(self, cfg: DecoderConfig):
        self.cfg = cfg
        self.mats: Dict[str, DeviceWeight] = {}
        self.vecs: Dict[str, DeviceBuffer] = {}

    @classmethod
    def random_init(cls, cfg: DecoderConfig, seed: int = 0, std: float = 0.02, exact: bool = False,
                    embed_seed: Optional[int] = None, embed_tau: float = 0.0, embed_loud_rows: int = 0,
                    embed_loud_gain: float = 1.0) -> "DecoderWeights":
        """Projections ~ N(0, std^2) quantised on the device; norm weights ~ 1 + N(0, 0.1^2);
        tied bf16 embedding ~ N(0, std^2); biases ~ N(0, 0.5^2).
        exact: draw every value with the host-reproducible generator (fk_synth_fill_exact), so a CPU
        build of the same model from the same seeds holds the same bytes.  embed_seed / embed_tau /
        embed_loud_rows / embed_loud_gain (exact only): own seed of the embedding, the spread of its row
        norms, and a few dominant rows (token ids 0 .. loud_rows - 1)."""
        self = cls(cfg)
        f32_kind, bf16_kind = (3, 4) if exact else (0, 1)
        biggest = max(cfg.inter * cfg.hidden, cfg.n_q * cfg.hidden)
        tmp = DeviceBuffer(biggest * 4) if cfg.bits != 16 else None
        counter = [seed * 100003 + 1]

        def next_seed() -> int:
            counter[0] += 1
            return counter[0]

        def matrix(name: str, n: int, k: int) -> None:
            if cfg.bits == 16:
                W = DeviceWeight.__new__(DeviceWeight)
                W.n, W.k, W.bits, W.group = n, k, 16, 0
                W.w, W.scales, W.biases = DeviceBuffer(n * k * 2), None, None
                _synth(W.w, n * k, next_seed(), 0.0, std, bf16_kind)
            else:
                _synth(tmp, n * k, next_seed(), 0.0, std, f32_kind)
                W = quantize_on_device(tmp, n, k, cfg.bits, cfg.group)
            self.mats[name] = W

        def vector(name: str, n: int, mean: float, sd: float) -> None:
            b = DeviceBuffer(n * 2)
            _synth(b, n, next_seed(), mean, sd, bf16_kind)
            self.vecs[name] = b

        emb = DeviceWeight.__new__(DeviceWeight)
        emb.n, emb.k, emb.bits, emb.group = cfg.vocab, cfg.hidden, 16, 0
        emb.w, emb.scales, emb.biases = DeviceBuffer(cfg.vocab * cfg.hidden * 2), None, None
        es = next_seed()
        if exact:
            _synth(emb.w, cfg.vocab * cfg.hidden, es if embed_seed is None else embed_seed, 0.0, std, 4,
                   row_len=cfg.hidden, tau=embed_tau, loud_rows=embed_loud_rows, loud_gain=embed_loud_gain)
        else:
            _synth(emb.w, cfg.vocab * cfg.hidden, es, 0.0, std, 1)
        self.mats["embed_tokens"] = emb
        vector("final_norm", cfg.hidden, 1.0, 0.1)
        for l in range(cfg.n_layers):
            p = f"layers.{l}."
            matrix(p + "self_attn.q_proj", cfg.n_q, cfg.hidden)
            matrix(p + "self_attn.k_proj", cfg.n_kvd, cfg.hidden)
            matrix(p + "self_attn.v_proj", cfg.n_kvd, cfg.hidden)
            matrix(p + "self_attn.o_proj", cfg.hidden, cfg.n_q)
            matrix(p + "mlp.gate_proj", cfg.inter, cfg.hidden)
            matrix(p + "mlp.up_proj", cfg.inter, cfg.hidden)
            matrix(p + "mlp.down_proj", cfg.hidden, cfg.inter)
            vector(p + "input_layernorm", cfg.hidden, 1.0, 0.1)
            vector(p + "post_attention_layernorm", cfg.hidden, 1.0, 0.1)
            if cfg.qk_norm:
                vector(p + "self_attn.q_norm", cfg.head_dim, 1.0, 0.1)
                vector(p + "self_attn.k_norm", cfg.head_dim, 1.0, 0.1)
            if cfg.qkv_bias:
                vector(p + "self_attn.q_proj.bias", cfg.n_q, 0.0, 0.5)
                vector(p + "self_attn.k_proj.bias", cfg.n_kvd, 0.0, 0.5)
                vector(p + "self_attn.v_proj.bias", cfg.n_kvd, 0.0, 0.5)
        native.sync()
        return self

    def nbytes(self) -> int:
        return sum(m.nbytes for m in self.mats.values()) + sum(v.nbytes for v in self.vecs.values())


class DecoderRuntime:
    """Scratch arena, KV caches, uniforms and the captured decode graph of one model."""

    def __init__(self, cfg: DecoderConfig, weights: DecoderWeights, dispatcher: Optional[Dispatcher] = None,
                 hist_capacity: int = 4096, persistent: bool = False, spin_limit: int = 0):
        self.cfg, self.w = cfg, weights
        self.d = dispatcher or Dispatcher()
        z = native.zeros
        self.token, self.step_counter = z(4), z(4)
        self.offset, self.kv_len, self.hist_counter = z(4), z(4), z(4)
        self.history = z(4 * hist_capacity)
        self.x = [DeviceBuffer(cfg.hidden * 2), DeviceBuffer(cfg.hidden * 2)]
        self.q, self.k, self.v = DeviceBuffer(cfg.n_q * 2), DeviceBuffer(cfg.n_kvd * 2), DeviceBuffer(cfg.n_kvd * 2)
        self.att, self.mid = DeviceBuffer(cfg.n_q * 2), DeviceBuffer(cfg.inter * 2)
        self.logits = DeviceBuffer(cfg.vocab * 2)
        if cfg.kv_bits:
            if persistent:
                raise ValueError("the whole-token kernel reads a bf16 KV cache; use the graph mode with kv_bits")
            mk = lambda: native.QuantKvCache(cfg.n_kv, cfg.capacity, cfg.head_dim, cfg.kv_bits, cfg.kv_group)
            self.cache_k = [mk() for _ in range(cfg.n_layers)]
            self.cache_v = [mk() for _ in range(cfg.n_layers)]
        else:
            cache_bytes = cfg.n_kv * cfg.capacity * cfg.head_dim * 2
            self.cache_k = [z(cache_bytes) for _ in range(cfg.n_layers)]
            self.cache_v = [z(cache_bytes) for _ in range(cfg.n_layers)]
        pb, cb = native.sdpa_workspace_bytes(cfg.n_heads, cfg.n_kv, cfg.head_dim, cfg.head_dim, cfg.capacity)
        self.sdpa_partials, self.sdpa_counters = DeviceBuffer(max(pb, 4)), z(max(cb, 4))
        self.argmax_ws = z(native.ARGMAX_WORKSPACE_BYTES)
        self.head_argmax_ws = z(native.HEAD_ARGMAX_WORKSPACE_BYTES)
        self.uniforms = make_uniforms(self.token, self.step_counter, self.hist_counter, self.history)
        self.persistent = persistent
        # one launch per layer for rope/store + attention: the task graph only (the whole-token kernel
        # fuses them itself and is built from the plain task list)
        self.fused_attention = bool(cfg.fuse_attention and not persistent and not cfg.kv_bits)
        self.rope_tab = DeviceBuffer(cfg.head_dim * 4) if self.fused_attention else None
        # a layer as two XCD-resident launches (8 KV heads, one per XCD): graph mode, bf16 cache, no projection bias
        self.xcd = bool(cfg.xcd_layers and self.fused_attention and not cfg.qkv_bias and
                        native.xcd_layer_supported(cfg.hidden, cfg.inter, cfg.n_heads, cfg.n_kv, cfg.head_dim, cfg.capacity,
                                                   cfg.bits, cfg.group))
        if self.xcd:
            ctl, ap = native.xcd_workspace_bytes(cfg.n_heads, cfg.head_dim)
            self.xcd_ctl = z(ctl)
            self.xcd_att_partials = DeviceBuffer(ap)
            self.xcd_xa, self.xcd_xb = DeviceBuffer(cfg.hidden * 2), DeviceBuffer(cfg.hidden * 2)
            # one launch per token: every layer needs its own q / k / v rows (read with ordinary loads inside the launch)
            if cfg.xcd_token_launch:
                self.xcd_qkv = [(DeviceBuffer(cfg.n_q * 2), DeviceBuffer(cfg.n_kvd * 2), DeviceBuffer(cfg.n_kvd * 2))
                                for _ in range(cfg.n_layers)]
            # three rotating sum rows: a launch reads one, adds into the next and clears the third
            self.xcd_sums = [z(native.xcd_sum_row_bytes(cfg.hidden)) for _ in range(3)]
            # scales / biases of o_proj and down_proj, one contiguous copy per K-slice (once, at load time)
            self.xcd_kmeta: Dict[str, tuple] = {}
            if cfg.bits != 16:
                for l in range(cfg.n_layers):
                    for name in (f"layers.{l}.self_attn.o_proj", f"layers.{l}.mlp.down_proj"):
                        W = weights.mats[name]
                        self.xcd_kmeta[name] = (native.xcd_kslice_meta(W.scales, W.n, W.k // W.group),
                                                native.xcd_kslice_meta(W.biases, W.n, W.k // W.group))
        self._bf16_weights: Dict[str, DeviceWeight] = {}   # resident bf16 copies for prompt passes (prefill_rows)
        self.tasks = self.build_tasks()
        # persistent: the same task list, run by one whole-token kernel per replay
        self.graph = (self.d.build_decode_graph(self.tasks, True, spin_limit) if persistent
                      else self.d.build_decode_graph(self.tasks, False))

    # -- task list -------------------------------------------------------------------
    def _wargs(self, W: DeviceWeight):
        return [arg(W.w)] if W.bits == 16 else [arg(W.w), arg(W.scales), arg(W.biases)]

    def build_tasks(self) -> List[Dispatch]:
        c, w = self.cfg, self.w
        q = dict(bits=c.bits, group=c.group)
        t: List[Dispatch] = []
        fid = [0]

        def name(kind: str) -> str:
            fid[0] += 1
            return f"fusekit_{kind}_f{fid[0]}"

        if self.fused_attention:   # step_init also fills this token's (cos, sin) table, shared by all layers
            t.append(Dispatch("fusekit_step_init", [arg(self.step_counter), arg(self.offset), arg(self.kv_len),
                                                    arg(self.rope_tab)], dict(rope_dims=c.head_dim, theta=c.theta)))
        else:
            t.append(Dispatch("fusekit_step_init", [arg(self.step_counter), arg(self.offset), arg(self.kv_len)]))
        emb = w.mats["embed_tokens"]       # dense bf16 or MLX-affine (4-bit checkpoints quantise it too)
        head = w.mats.get("lm_head", emb)  # untied output projection when the checkpoint has one
        t.append(Dispatch(name("embed_lookup_decode"), [arg(self.token)] + self._wargs(emb) + [arg(self.x[0])],
                          dict(bits=emb.bits, group=emb.group or 64, hidden=c.hidden, vocab=c.vocab,
                               output_scale=c.embed_scale)))
        if self.xcd:
            self._xcd_layer_tasks(t, name)
        for l in range(0 if not self.xcd else c.n_layers, c.n_layers):
            p = f"layers.{l}."
            Wq, Wk, Wv = (w.mats[p + f"self_attn.{n}_proj"] for n in "qkv")
            qkv_args = [arg(self.x[0]), arg(w.vecs[p + "input_layernorm"]), arg(Wq.w), arg(Wk.w), arg(Wv.w)]
            if c.bits != 16:
                qkv_args += [arg(m.scales) for m in (Wq, Wk, Wv)] + [arg(m.biases) for m in (Wq, Wk, Wv)]
            if c.qkv_bias:
                qkv_args += [arg(w.vecs[p + f"self_attn.{n}_proj.bias"]) for n in "qkv"]
            qkv_args += [arg(self.q), arg(self.k), arg(self.v)]
            t.append(Dispatch(name("rmsnorm_qkv"), qkv_args,
                              dict(q, hidden=c.hidden, n_q=c.n_q, n_kv=c.n_kvd, eps=c.eps, has_norm=1,
                                   has_bias=int(c.qkv_bias))))
            rope = dict(n_heads=c.n_heads, n_kv=c.n_kv, head_dim=c.head_dim, rope_dims=c.head_dim, theta=c.theta,
                        capacity=c.capacity, eps=c.eps)
            if self.fused_attention:
                a = [arg(self.q), arg(self.k), arg(self.v)]
                if c.qk_norm:
                    a += [arg(w.vecs[p + "self_attn.q_norm"]), arg(w.vecs[p + "self_attn.k_norm"])]
                a += [arg(self.cache_k[l]), arg(self.cache_v[l]), arg(self.kv_len), arg(self.att),
                      arg(self.sdpa_partials), arg(self.sdpa_counters), arg(self.rope_tab)]
                t.append(Dispatch(name("rope_store_sdpa_decode"), a,
                                  dict(rope, has_norm=int(c.qk_norm), has_table=1, max_len=c.capacity)))
            elif c.kv_bits:
                # quantised cache: rotate q in place, then quantise the rotated K row and the V row
                qa = [arg(self.q)] + ([arg(w.vecs[p + "self_attn.q_norm"])] if c.qk_norm else []) + [arg(self.offset)]
                t.append(Dispatch(name("rmsnorm_rope_q_decode" if c.qk_norm else "rope_q_decode"), qa, rope))
                K, V = self.cache_k[l], self.cache_v[l]
                ka = [arg(self.k), arg(self.v)] + ([arg(w.vecs[p + "self_attn.k_norm"])] if c.qk_norm else [])
                ka += [arg(b) for b in (K.packed, K.scales, K.biases, V.packed, V.scales, V.biases)]
                ka += [arg(self.offset), arg(self.offset)]
                t.append(Dispatch(name(f"rope_kv_cache_store_decode_q{c.kv_bits}"), ka,
                                  dict(rope, has_norm=int(c.qk_norm), group=c.kv_group)))
            elif c.fuse_rope_store:
                a = [arg(self.q), arg(self.k), arg(self.v)]
                if c.qk_norm:
                    a += [arg(w.vecs[p + "self_attn.q_norm"]), arg(w.vecs[p + "self_attn.k_norm"])]
                a += [arg(self.cache_k[l]), arg(self.cache_v[l]), arg(self.offset)]
                t.append(Dispatch(name("qkv_rope_store_decode"), a, dict(rope, has_norm=int(c.qk_norm))))
            elif c.qk_norm:
                t.append(Dispatch(name("rmsnorm_rope_q_decode"),
                                  [arg(self.q), arg(w.vecs[p + "self_attn.q_norm"]), arg(self.offset)], rope))
                t.append(Dispatch(name("rmsnorm_rope_kv_cache_store_decode"),
                                  [arg(self.k), arg(self.v), arg(w.vecs[p + "self_attn.k_norm"]),
                                   arg(self.cache_k[l]), arg(self.cache_v[l]), arg(self.offset), arg(self.offset)],
                                  rope))
            else:
                t.append(Dispatch(name("rope_q_decode"), [arg(self.q), arg(self.offset)], rope))
                t.append(Dispatch(name("rope_kv_cache_store_decode"),
                                  [arg(self.k), arg(self.v), arg(self.cache_k[l]), arg(self.cache_v[l]),
                                   arg(self.offset), arg(self.offset)], rope))
            if self.fused_attention:
                pass
            elif c.kv_bits:
                K, V = self.cache_k[l], self.cache_v[l]
                t.append(Dispatch(name(f"sdpa_decode_q{c.kv_bits}"),
                                  [arg(self.q)] + [arg(b) for b in (K.packed, K.scales, K.biases, V.packed, V.scales, V.biases)]
                                  + [arg(self.kv_len), arg(self.att), arg(self.sdpa_partials), arg(self.sdpa_counters)],
                                  dict(n_heads=c.n_heads, n_kv=c.n_kv, head_dim=c.head_dim, capacity=c.capacity,
                                       max_len=c.capacity, group=c.kv_group)))
            else:
                t.append(Dispatch(name("sdpa_decode"),
                                  [arg(self.q), arg(self.cache_k[l]), arg(self.cache_v[l]), arg(self.kv_len),
                                   arg(self.att), arg(self.sdpa_partials), arg(self.sdpa_counters)],
                                  dict(n_heads=c.n_heads, n_kv=c.n_kv, head_dim=c.head_dim, capacity=c.capacity,
                                       max_len=c.capacity)))
            Wo = w.mats[p + "self_attn.o_proj"]
            t.append(Dispatch(name("linear_residual"),
                              [arg(self.att)] + self._wargs(Wo) + [arg(self.x[0]), arg(self.x[1])],
                              dict(q, m=c.n_q, n=c.hidden)))
            Wg, Wu = w.mats[p + "mlp.gate_proj"], w.mats[p + "mlp.up_proj"]
            ga = [arg(self.x[1]), arg(w.vecs[p + "post_attention_layernorm"]), arg(Wg.w), arg(Wu.w)]
            if c.bits != 16:
                ga += [arg(Wg.scales), arg(Wu.scales), arg(Wg.biases), arg(Wu.biases)]
            ga += [arg(self.mid)]
            t.append(Dispatch(name("rmsnorm_gateup_swiglu"), ga,
                              dict(q, hidden=c.hidden, inter=c.inter, eps=c.eps, variant=c.swiglu_variant,
                                   has_norm=1)))
            Wd = w.mats[p + "mlp.down_proj"]
            t.append(Dispatch(name("linear_residual"),
                              [arg(self.mid)] + self._wargs(Wd) + [arg(self.x[1]), arg(self.x[0])],
                              dict(q, m=c.inter, n=c.hidden)))
        head_args = [arg(self.x[0]), arg(w.vecs["final_norm"])] + self._wargs(head) + [arg(self.logits)]
        head_params = dict(bits=head.bits, group=head.group or 64, hidden=c.hidden, vocab=c.vocab, eps=c.eps)
        # The direct head (the reference's `<head>_argmax` + `_argmax_finalize`, dispatch.py:3458-3505, greedy
        # decode only) as one launch; the whole-token kernel keeps the canonical two tasks.
        self.direct_head = bool(c.direct_head_argmax and not self.persistent and
                                native.gemv_form(c.vocab, c.hidden, head.bits, head.group or 64) == 1)
        if self.direct_head:
            t.append(Dispatch(name("final_rmsnorm_lm_head_argmax"),
                              head_args + [arg(self.token), arg(self.head_argmax_ws), arg(self.history),
                                           arg(self.hist_counter)], head_params))
            return t
        t.append(Dispatch(name("final_rmsnorm_lm_head"), head_args, head_params))
        t.append(Dispatch(name("argmax_logits_decode"),
                          [arg(self.logits), arg(self.token), arg(self.argmax_ws), arg(self.history),
                           arg(self.hist_counter)], dict(vocab=c.vocab)))
        return t

    def _xcd_kslice_args(self, name: str, W: DeviceWeight):
        if W.bits == 16:
            return [arg(W.w)]
        sc, bi = self.xcd_kmeta[name]
        return [arg(W.w), arg(sc), arg(bi)]

    def _xcd_layer_tasks(self, t: List[Dispatch], name) -> None:
        """Two launches per layer (families fusekit_xcd_attn_block / fusekit_xcd_mlp_block), then the last layer's
        sum row + residual into x[0] for the LM head.  Launch i of the token reads sum row i % 3, adds into row
        (i + 1) % 3 and clears row (i + 2) % 3; the first launch adds into row 1, which the closing reduction
        leaves cleared for the next token."""
        c, w = self.cfg, self.w
        shape = dict(hidden=c.hidden, inter=c.inter, n_heads=c.n_heads, n_kv=c.n_kv, head_dim=c.head_dim,
                     capacity=c.capacity, bits=c.bits, group=c.group, eps=c.eps, theta=c.theta,
                     spin_limit=c.xcd_spin_limit, token_launch=1 if c.xcd_token_launch else (2 if c.xcd_layer_launch else 0))
        quant = c.bits != 16
        for l in range(c.n_layers):
            p = f"layers.{l}."
            Wq, Wk, Wv, Wo = (w.mats[p + f"self_attn.{n}_proj"] for n in "qkvo")
            S = lambda i: arg(self.xcd_sums[i % 3])
            a = [] if l == 0 else [S(2 * l)]
            a += [arg(self.x[0]) if l == 0 else arg(self.xcd_xb), arg(self.xcd_xa), arg(w.vecs[p + "input_layernorm"]),
                  arg(Wq.w), arg(Wk.w), arg(Wv.w)]
            if quant:
                a += [arg(m.scales) for m in (Wq, Wk, Wv)] + [arg(m.biases) for m in (Wq, Wk, Wv)]
            a += self._xcd_kslice_args(p + "self_attn.o_proj", Wo)
            if c.qk_norm:
                a += [arg(w.vecs[p + "self_attn.q_norm"]), arg(w.vecs[p + "self_attn.k_norm"])]
            q_, k_, v_ = self.xcd_qkv[l] if c.xcd_token_launch else (self.q, self.k, self.v)
            a += [arg(q_), arg(k_), arg(v_), arg(self.cache_k[l]), arg(self.cache_v[l]), arg(self.kv_len),
                  arg(self.rope_tab), arg(self.xcd_att_partials), S(2 * l + 1), S(2 * l + 2), arg(self.xcd_ctl)]
            # the first launch of a token also flips the placement words (the watch on how workgroups are dealt)
            t.append(Dispatch(name("xcd_attn_block"), a, dict(shape, has_sums=int(l > 0), has_norm=int(c.qk_norm),
                                                              mark_placement=int(l == 0))))
            Wg, Wu, Wd = (w.mats[p + f"mlp.{n}_proj"] for n in ("gate", "up", "down"))
            m = [S(2 * l + 1), arg(self.xcd_xa), arg(self.xcd_xb), arg(w.vecs[p + "post_attention_layernorm"]),
                 arg(Wg.w), arg(Wu.w)]
            if quant:
                m += [arg(Wg.scales), arg(Wu.scales), arg(Wg.biases), arg(Wu.biases)]
            m += self._xcd_kslice_args(p + "mlp.down_proj", Wd) + [arg(self.mid), S(2 * l + 2), S(2 * l + 3), arg(self.xcd_ctl)]
            t.append(Dispatch(name("xcd_mlp_block"), m, dict(shape, has_sums=1, variant=c.swiglu_variant)))
        t.append(Dispatch(name("xcd_reduce"), [arg(self.xcd_sums[(2 * c.n_layers) % 3]), arg(self.xcd_xb), arg(self.x[0]),
                                               arg(self.xcd_sums[1])], dict(hidden=c.hidden)))

    # -- generation ------------------------------------------------------------------
    def reset(self) -> None:
        for b in (self.step_counter, self.offset, self.kv_len, self.hist_counter):
            b.upload(np.zeros(1, np.uint32))
        if self.xcd:
            for b in self.xcd_sums:
                b.upload(np.zeros(b.nbytes, np.uint8))

    def prefill(self, prompt: Sequence[int], start_offset: int = 0) -> int:
        """Feeds the prompt through the decode graph with forced tokens; returns the greedy
        first token (the argmax after the last prompt token)."""
        nxt, _ = self.d.decode_host_loop(self.graph, self.uniforms, start_offset, list(prompt))
        return nxt[-1]

    def prefill_rows(self, prompt: Sequence[int], start_offset: int = 0, rows_per_pass: int = 4096,
                     keep_bf16_weights: bool = False) -> int:
        """Prompt processing with several active rows per pass (the reference's `prefill_mN` /
        active_m > 1 variants): the projections of up to `rows_per_pass` (<= 4096) tokens share ONE pass over each weight
        matrix on the matrix cores (fk_qgemm; from 65 rows up in its bf16-weight form, which is LDS-tiled, from 1024 rows -- fk_set_gemm_library_rows -- as a dequantisation to bf16 followed by a library GEMM), attention is
        causal inside the group (fk_sdpa_prefill for the bf16 cache with head dimension 64 or 128,
        else the single-row kernel once per row).  Leaves the KV
        caches, step counter and history as token-by-token `prefill` would, and returns the greedy
        first token.  Dense bf16 weights take the library GEMM for every row count.
        keep_bf16_weights: passes of at least 256 rows multiply with a bf16 copy of every projection that stays
        resident after its first use (2 bytes per weight: 7.3 GB for the 4B-class model) instead of
        dequantising each matrix again in every pass; the results of the dequantise + library route, bit for bit."""
        c, w = self.cfg, self.w
        prompt = list(prompt)
        if start_offset + len(prompt) > c.capacity:
            raise ValueError("prompt exceeds the KV-cache capacity")
        # buffers follow the prompt (next power of two), so a short prompt does not allocate for 4096 rows
        R = max(1, min(rows_per_pass, 4096, 1 << max(5, (len(prompt) - 1).bit_length())))
        if getattr(self, "_rows_R", 0) != R:
            self._rows_R = R
            # the split of k differs between the kernel forms (<= 32, <= 64, more rows) and with the
            # number of 128-row tiles; the last pass of a prompt may have any row count up to R
            ws = max(native.qgemm_workspace_bytes(m, n, k, 0 if c.bits == 16 else c.group)
                     for m in {R} | {v for v in (*range(512, 4096, 128), 384, 256, 128, 64, 32) if v < R}
                     for n, k in ((c.n_q, c.hidden), (c.n_q + 2 * c.n_kvd, c.hidden), (c.hidden, c.n_q), (c.inter, c.hidden),
                                  (c.hidden, c.inter)))
            # only the single-row attention kernel (quantised cache, other head dimensions) needs a workspace
            pb, cb = (native.sdpa_workspace_bytes(c.n_heads, c.n_kv, c.head_dim, c.head_dim, c.capacity)
                      if c.head_dim not in (64, 128) else (0, 0))
            self._rows = dict(
                tok=DeviceBuffer(4 * R), x=DeviceBuffer(R * c.hidden * 2), x2=DeviceBuffer(R * c.hidden * 2),
                xn=DeviceBuffer(R * c.hidden * 2), q=DeviceBuffer(R * c.n_q * 2), k=DeviceBuffer(R * c.n_kvd * 2),
                v=DeviceBuffer(R * c.n_kvd * 2), att=DeviceBuffer(R * c.n_q * 2), mid=DeviceBuffer(R * c.inter * 2),
                ws=DeviceBuffer(2 * ws), part=DeviceBuffer(max(pb, 4) * R), cnt=native.zeros(max(cb, 4) * R),
                rope=DeviceBuffer(R * c.head_dim * 4))
            if c.kv_bits and c.head_dim in (64, 128):  # the dequantised prefix of one layer's cache, reused by every layer
                self._rows["kdq"] = DeviceBuffer(c.n_kv * c.capacity * c.head_dim * 2)
                self._rows["vdq"] = DeviceBuffer(c.n_kv * c.capacity * c.head_dim * 2)
        b = self._rows
        emb = w.mats["embed_tokens"]
        head = w.mats.get("lm_head", emb)
        pos = start_offset
        scale = 1.0 / float(np.sqrt(c.head_dim))

        def mat(name: str, m: int):
            W = w.mats[name]
            if not keep_bf16_weights or W.bits == 16 or m < 256 or not native.gemm_library_available():
                return W
            if name not in self._bf16_weights:
                self._bf16_weights[name] = native.dequantize_bf16(W)
            return self._bf16_weights[name]

        while pos < start_offset + len(prompt):
            chunk = prompt[pos - start_offset: pos - start_offset + R]
            m = len(chunk)
            b["tok"].upload(np.asarray(chunk, np.uint32))
            native.embed_lookup_rows(emb, b["tok"], m, c.embed_scale, b["x"])
            native.rope_table_rows(b["rope"], c.head_dim, c.theta, pos, m)  # once per pass, for every layer and head
            for l in range(c.n_layers):
                p = f"layers.{l}."
                native.rmsnorm_rows(b["x"], w.vecs[p + "input_layernorm"], c.eps, m, c.hidden, b["xn"])
                # q, k and v over the same rows: one call (one launch of the fused kernel where its tile form applies)
                qkv = [mat(p + f"self_attn.{nm}_proj", m) for nm in "qkv"]
                qkv_bias = [w.vecs.get(p + f"self_attn.{nm}_proj.bias") for nm in "qkv"] if c.qkv_bias else None
                if all(W.bits != 16 for W in qkv):
                    native.qgemm_fanout(qkv, b["xn"], m, qkv_bias, [b["q"], b["k"], b["v"]], b["ws"])
                else:
                    for i, dst in enumerate((b["q"], b["k"], b["v"])):
                        native.qgemm(qkv[i], b["xn"], m, qkv_bias[i] if qkv_bias else None, None, dst, b["ws"])
                qn = w.vecs.get(p + "self_attn.q_norm") if c.qk_norm else None
                kn = w.vecs.get(p + "self_attn.k_norm") if c.qk_norm else None
                if c.kv_bits:
                    native.qkv_rope_store_rows(b["q"], None, None, qn, None, c.n_heads, 0, c.head_dim, c.head_dim,
                                               c.theta, c.eps, m, pos, c.capacity, None, None, rope_tab=b["rope"])
                    native.kv_cache_store_quant(b["k"], b["v"], kn, c.n_kv, c.head_dim, c.head_dim, c.theta, c.eps,
                                                None, pos, m, self.cache_k[l], self.cache_v[l])
                    if c.head_dim in (64, 128):
                        # the visible prefix as bf16 (a few MB per layer), then the matrix-core attention
                        native.kv_cache_dequant(self.cache_k[l], pos + m, b["kdq"], c.capacity)
                        native.kv_cache_dequant(self.cache_v[l], pos + m, b["vdq"], c.capacity)
                        native.sdpa_prefill(b["q"], b["kdq"], b["vdq"], b["att"], m, pos + m, c.n_heads, c.n_kv, c.head_dim,
                                            c.capacity, scale)
                    else:
                        native.sdpa_decode_quant(b["q"], self.cache_k[l], self.cache_v[l], b["att"], None, pos + 1,
                                                 pos + m, m, c.n_heads, scale, b["part"], b["cnt"])
                else:
                    native.qkv_rope_store_rows(b["q"], b["k"], b["v"], qn, kn, c.n_heads, c.n_kv, c.head_dim, c.head_dim,
                                               c.theta, c.eps, m, pos, c.capacity, self.cache_k[l], self.cache_v[l],
                                               rope_tab=b["rope"])
                    if c.head_dim in (64, 128):  # causal attention of the whole group on the matrix cores
                        native.sdpa_prefill(b["q"], self.cache_k[l], self.cache_v[l], b["att"], m, pos + m, c.n_heads,
                                            c.n_kv, c.head_dim, c.capacity, scale)
                    else:
                        native.sdpa_decode_rows(b["q"], self.cache_k[l], self.cache_v[l], b["att"], m, pos + 1, c.n_heads,
                                                c.n_kv, c.head_dim, c.head_dim, c.capacity, scale, b["part"], b["cnt"])
                native.qgemm(mat(p + "self_attn.o_proj", m), b["att"], m, None, b["x"], b["x2"], b["ws"])
                native.rmsnorm_rows(b["x2"], w.vecs[p + "post_attention_layernorm"], c.eps, m, c.hidden, b["xn"])
                native.qgemm_swiglu(mat(p + "mlp.gate_proj", m), mat(p + "mlp.up_proj", m), b["xn"], m, c.swiglu_variant,
                                    b["mid"], b["ws"])
                native.qgemm(mat(p + "mlp.down_proj", m), b["mid"], m, None, b["x2"], b["x"], b["ws"])
            pos += m
        # the last row's hidden state -> logits -> greedy token, and the decode loop's uniforms
        last = DeviceBuffer(c.hidden * 2)
        native.copy(last, b["x"].ptr + (m - 1) * c.hidden * 2, c.hidden * 2)
        native.final_rmsnorm_lm_head(last, w.vecs["final_norm"], c.eps, head, self.logits)
        native.argmax_logits_decode(self.logits, c.vocab, self.token, None, None, 0, self.argmax_ws)
        native.sync()
        total = start_offset + len(prompt)
        self.step_counter.upload(np.array([total], np.uint32))
        return int(self.token.to_numpy(np.uint32)[0])

    def generate(self, prompt: Sequence[int], max_tokens: int):
        """Greedy decode.  Returns (tokens, gpu_seconds of the decode chunks, decode steps timed)."""
        if len(prompt) + max_tokens > self.cfg.capacity:
            raise ValueError("prompt + max_tokens exceeds the KV-cache capacity")  # __init__.py:5017-5037
        first = self.prefill(prompt)
        out = [first]
        offset = len(prompt)
        gpu_s, steps = 0.0, 0
        while len(out) < max_tokens:
            n = min(FK_CHUNK, max_tokens - len(out), self.uniforms.hist_capacity)
            toks, sec = self.d.decode_chunk(self.graph, self.uniforms, offset, out[-1], n)
            out += toks
            offset += n
            gpu_s += sec
            steps += n
        return out, gpu_s, steps
