"""Mixture-of-experts decoder with low-rank (MLA-style) keys and values on the MI355X backend:
random-init weights in HBM, the per-token task list and the captured decode graph.

The architecture is the DeepSeek-V2-Lite-like model of the reference's MoE benchmarks: per layer
  RMSNorm -> q_proj [n_heads x (nope + rope)] and kv_a_proj [kv_lora_rank + rope] (one launch)
  RMSNorm(latent) -> kv_b_proj [n_heads x (nope + v)]                              (one launch)
  cache K row = [k_nope | rope(k_pe)] with ONE rotary key head shared by all heads, V row, and the
  rotation of the query's rope part (the reference's split-key KvCacheStoreDecode,
  src/codegen/kernels/kv_cache_store_decode.rs:84-352, and the Q1 rotation of its attention kernel,
  sdpa_decode.rs:592-660)
  attention at qk_dim = nope + rope, v_dim (sdpa_decode.rs:133-408) -> o_proj + residual
  RMSNorm -> router logits -> SoftmaxTopKRoute (single.rs:2615-2760)
  RoutedQmvSwiglu over the top_k experts (routed_qmv_swiglu.rs:20-452), the shared experts' gate/up,
  RoutedQmvReduce + shared down projection + residual (routed_qmv_reduce.rs:11-543)
with the first `first_dense` layers carrying a dense SwiGLU MLP instead of the experts.
Every dispatch is a kernel family of the task-graph contract, so the list captures into one hipGraph
and replays per token like the dense decoder's.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, List, Optional, Sequence

import numpy as np

from . import native
from .decoder import _synth, quantize_on_device
from .native import DeviceBuffer, DeviceWeight
from .runtime import FK_CHUNK, Dispatch, Dispatcher, arg, make_uniforms


@dataclass
class MoeConfig:
    n_layers: int = 27
    hidden: int = 2048
    n_heads: int = 16
    kv_lora_rank: int = 512
    rope_dim: int = 64
    nope_dim: int = 128
    v_dim: int = 128
    n_experts: int = 64
    top_k: int = 6
    moe_inter: int = 1408
    n_shared: int = 2
    dense_inter: int = 10944
    first_dense: int = 1
    vocab: int = 102400
    eps: float = 1e-6
    theta: float = 1e4
    rope_traditional: bool = True
    route_scale: float = 1.0
    bits: int = 4
    group: int = 64
    swiglu_variant: int = 1
    capacity: int = 1024
    fuse_topk: bool = True        # the expert launch ranks the router logits itself (needs fuse_router and fuse_shared)
    fuse_attention: bool = True   # split-key cache store + attention of a layer in one launch
    fuse_shared: bool = True   # the shared experts' gate/up pair as further routes of the routed launch
    fuse_router: bool = True   # norm + router projection + top-k route as one launch (hidden % 512 == 0)
    direct_head_argmax: bool = True  # the LM head selects the greedy token itself where its shape allows
    xcd_moe: bool = True       # router + routed / shared experts + reduction of a layer as ONE XCD-resident launch, where
                               # the shape admits it (MoeRuntime.xcd tells); off: the per-dispatch families
    xcd_attn: bool = True      # with xcd_moe: the attention half of every layer as ONE launch too (two launches per layer)
    xcd_spin_limit: int = 0    # hand-over wait bound of these launches (0: the library's default)

    @property
    def qk_dim(self) -> int:
        return self.nope_dim + self.rope_dim

    @property
    def shared_inter(self) -> int:
        return self.n_shared * self.moe_inter

    def token_bytes(self, ctx: int) -> int:
        """Algorithmic HBM bytes per decoded token at context `ctx`: the weights one token touches
        (attention, top_k + shared experts or the dense MLP, bf16 router), the tied bf16 LM head and
        the K / V rows attention reads."""
        per = self.bits / 8 + 4 / self.group
        attn = self.hidden * (self.n_heads * self.qk_dim + self.kv_lora_rank + self.rope_dim) \
            + self.kv_lora_rank * self.n_heads * (self.nope_dim + self.v_dim) + self.n_heads * self.v_dim * self.hidden
        moe = 3 * self.hidden * self.moe_inter * (self.top_k + self.n_shared)
        dense = 3 * self.hidden * self.dense_inter
        n_moe = self.n_layers - self.first_dense
        weights = per * (self.n_layers * attn + n_moe * moe + self.first_dense * dense) + n_moe * self.n_experts * self.hidden * 2
        kv = self.n_layers * self.n_heads * (self.qk_dim + self.v_dim) * 2 * ctx
        return int(weights + self.vocab * self.hidden * 2 + kv)


MOE_16B_LIKE = dict()   # the defaults above: 27 layers, hidden 2048, 64 experts of 1408, top-6, 2 shared


class MoeWeights:
    """Weights of one model in HBM, keyed by mlx-lm's parameter paths for this architecture."""

    def __init__(self, cfg: MoeConfig):
        self.cfg = cfg
        self.mats: Dict[str, DeviceWeight] = {}
        self.vecs: Dict[str, DeviceBuffer] = {}

    @classmethod
    def random_init(cls, cfg: MoeConfig, seed: int = 0, std: float = 0.02, exact: bool = False,
                    embed_loud_rows: int = 0, embed_loud_gain: float = 1.0) -> "MoeWeights":
        """Projections ~ N(0, std^2) quantised on the device (experts stacked [E, n, k]); the router and
        the tied embedding stay bf16; norm weights ~ 1 + N(0, 0.1^2).
        exact: every value from the host-reproducible generator (fk_synth_fill_exact), so that a CPU build of the
        same model from the same seeds holds the same bytes; embed_loud_rows / embed_loud_gain (exact only): a few
        dominant embedding rows (token ids 0 .. loud_rows - 1)."""
        self = cls(cfg)
        c = cfg
        f32_kind, bf16_kind = (3, 4) if exact else (0, 1)
        biggest = max(c.n_experts * c.moe_inter * c.hidden if c.n_layers > c.first_dense else 0,
                      c.dense_inter * c.hidden if c.first_dense else 0, c.n_heads * c.qk_dim * c.hidden)
        tmp = DeviceBuffer(biggest * 4)
        counter = [seed * 100003 + 7]

        def next_seed() -> int:
            counter[0] += 1
            return counter[0]

        def matrix(name: str, n: int, k: int, experts: int = 0, sd: float = std) -> None:
            rows = n * max(experts, 1)
            _synth(tmp, rows * k, next_seed(), 0.0, sd, f32_kind)
            W = quantize_on_device(tmp, rows, k, c.bits, c.group)
            if experts:
                W.n, W.n_experts = n, experts
            self.mats[name] = W

        def dense_bf16(name: str, n: int, k: int, sd: float) -> None:
            W = DeviceWeight.__new__(DeviceWeight)
            W.n, W.k, W.bits, W.group = n, k, 16, 0
            W.w, W.scales, W.biases = DeviceBuffer(n * k * 2), None, None
            if exact and name == "embed_tokens":
                _synth(W.w, n * k, next_seed(), 0.0, sd, 4, row_len=k, loud_rows=embed_loud_rows, loud_gain=embed_loud_gain)
            else:
                _synth(W.w, n * k, next_seed(), 0.0, sd, bf16_kind)
            self.mats[name] = W

        def vector(name: str, n: int, mean: float, sd: float) -> None:
            b = DeviceBuffer(n * 2)
            _synth(b, n, next_seed(), mean, sd, bf16_kind)
            self.vecs[name] = b

        dense_bf16("embed_tokens", c.vocab, c.hidden, std)
        vector("final_norm", c.hidden, 1.0, 0.1)
        for l in range(c.n_layers):
            p = f"layers.{l}."
            vector(p + "input_layernorm", c.hidden, 1.0, 0.1)
            vector(p + "post_attention_layernorm", c.hidden, 1.0, 0.1)
            matrix(p + "self_attn.q_proj", c.n_heads * c.qk_dim, c.hidden)
            matrix(p + "self_attn.kv_a_proj_with_mqa", c.kv_lora_rank + c.rope_dim, c.hidden)
            vector(p + "self_attn.kv_a_layernorm", c.kv_lora_rank, 1.0, 0.1)
            matrix(p + "self_attn.kv_b_proj", c.n_heads * (c.nope_dim + c.v_dim), c.kv_lora_rank)
            matrix(p + "self_attn.o_proj", c.hidden, c.n_heads * c.v_dim)
            if l < c.first_dense:
                matrix(p + "mlp.gate_proj", c.dense_inter, c.hidden)
                matrix(p + "mlp.up_proj", c.dense_inter, c.hidden)
                matrix(p + "mlp.down_proj", c.hidden, c.dense_inter)
            else:
                dense_bf16(p + "mlp.gate", c.n_experts, c.hidden, 0.05)   # wider spread: distinct routes
                for nm in ("gate_proj", "up_proj"):
                    matrix(p + f"mlp.switch_mlp.{nm}", c.moe_inter, c.hidden, c.n_experts)
                    matrix(p + f"mlp.shared_experts.{nm}", c.shared_inter, c.hidden)
                matrix(p + "mlp.switch_mlp.down_proj", c.hidden, c.moe_inter, c.n_experts)
                matrix(p + "mlp.shared_experts.down_proj", c.hidden, c.shared_inter)
        # two constants the task list binds like parameters: the routing scale (bf16) and the identity map from
        # a route to its row of expert outputs (uint32 0 .. top_k - 1)
        self.vecs["mlp.route_scale"] = DeviceBuffer.from_numpy(_bf16(np.array([c.route_scale], np.float32)))
        self.vecs["mlp.route_rows"] = DeviceBuffer.from_numpy(np.arange(c.top_k, dtype=np.uint32))
        native.sync()
        return self

    def nbytes(self) -> int:
        return sum(m.nbytes for m in self.mats.values()) + sum(v.nbytes for v in self.vecs.values())


def _rows(W: DeviceWeight, r0: int, r1: int):
    """(packed, scales, biases) argument slices of rows r0 .. r1 of a quantised matrix."""
    wb, sb = W.k * W.bits // 8, (W.k // W.group) * 2
    return (arg(W.w, (r1 - r0) * wb, r0 * wb), arg(W.scales, (r1 - r0) * sb, r0 * sb), arg(W.biases, (r1 - r0) * sb, r0 * sb))


class MoeRuntime:
    """Scratch arena, KV caches, uniforms and the captured decode graph of one MoE model."""

    def __init__(self, cfg: MoeConfig, weights: MoeWeights, dispatcher: Optional[Dispatcher] = None,
                 hist_capacity: int = 4096, route_order: bool = False):
        c = cfg
        self.route_order = route_order   # passes over several token rows serve their routes sorted by expert
        if c.kv_lora_rank % 64 or c.hidden % 64 or c.moe_inter % 64 or (c.kv_lora_rank + c.rope_dim) % 2:
            raise ValueError("widths must be multiples of the quantisation group")
        self.cfg, self.w = cfg, weights
        self.d = dispatcher or Dispatcher()
        z, B = native.zeros, DeviceBuffer
        self.token, self.step_counter = z(4), z(4)
        self.offset, self.kv_len, self.hist_counter = z(4), z(4), z(4)
        self.history = z(4 * hist_capacity)
        self.x = [B(c.hidden * 2), B(c.hidden * 2)]
        self.xn = B(c.hidden * 2)
        self.q = B(c.n_heads * c.qk_dim * 2)
        self.kva = B((c.kv_lora_rank + c.rope_dim) * 2)            # [latent | k_pe]
        self.kvb = B(c.n_heads * (c.nope_dim + c.v_dim) * 2)       # per head [k_nope | v]
        self.att = B(c.n_heads * c.v_dim * 2)
        self.mid = B(max(c.dense_inter, c.shared_inter) * 2)
        self.route_logits = z(c.n_experts * 2 * c.n_layers)   # one slot per layer, like the routes
        # one slot per layer, so that the routes of a whole step can be read back after it
        self.route_idx, self.route_weight = z(4 * c.top_k * c.n_layers), z(2 * c.top_k * c.n_layers)
        self.route_scale = weights.vecs["mlp.route_scale"]
        self.rows_x = z(4 * c.top_k)                                # every route reads activation row 0
        self.rows_h = weights.vecs["mlp.route_rows"]
        self.h = B(c.top_k * c.moe_inter * 2)
        self.moe_ws = B(max(native.routed_reduce_workspace_bytes(1, c.top_k, c.hidden), 4))
        self.logits = B(c.vocab * 2)
        self.cache_k = [z(c.n_heads * c.capacity * c.qk_dim * 2) for _ in range(c.n_layers)]
        self.cache_v = [z(c.n_heads * c.capacity * c.v_dim * 2) for _ in range(c.n_layers)]
        pb, cb = native.sdpa_workspace_bytes(c.n_heads, c.n_heads, c.qk_dim, c.v_dim, c.capacity)
        self.sdpa_partials, self.sdpa_counters = B(max(pb, 4)), z(max(cb, 4))
        self.argmax_ws = z(native.ARGMAX_WORKSPACE_BYTES)
        self.head_argmax_ws = z(native.HEAD_ARGMAX_WORKSPACE_BYTES)
        self.rope_tab = B(c.rope_dim * 4)
        self.uniforms = make_uniforms(self.token, self.step_counter, self.hist_counter, self.history)
        # the single-launch router holds the hidden row in registers, 512 elements per piece, at most 8
        self.fused_router = bool(c.fuse_router and c.hidden % 512 == 0 and c.hidden <= 4096)
        self.router_ws = z(4 * (c.n_experts + 1))
        # the expert block as one launch, cut by route over the XCDs (where the shape admits it)
        self.xcd = bool(c.xcd_moe and c.swiglu_variant == 1 and c.first_dense < c.n_layers and
                        native.xcd_moe_supported(c.hidden, c.moe_inter, c.shared_inter, c.n_experts, c.top_k, c.bits, c.group))
        # ... and the attention half (low-rank keys) as one launch: then a layer is two launches
        self.xcd_attn = bool(self.xcd and c.xcd_attn and c.fuse_attention and
                             native.xcd_mla_supported(c.hidden, c.n_heads, c.kv_lora_rank, c.rope_dim, c.nope_dim, c.v_dim,
                                                      c.capacity, c.bits, c.group))
        if self.xcd:
            self.xcd_ctl = z(native.xcd_workspace_bytes(c.n_heads, c.qk_dim)[0])
            # expert launch alone: routes, shared expert, a row to clear; with the attention launch six rows rotate:
            # P0, P1 (attention outputs), then the (routes, shared expert) pairs of even and of odd layers
            self.xcd_sums = [z(native.xcd_sum_row_bytes(c.hidden)) for _ in range(6 if self.xcd_attn else 3)]
            self.xcd_x = B(c.hidden * 2)
            self.xcd_scratch = z(native.xcd_moe_scratch_bytes(c.moe_inter))
        self.xcd_kmeta: Dict[str, tuple] = {}
        if self.xcd_attn:
            lat, part = native.xcd_mla_workspace_bytes(c.n_heads, c.kv_lora_rank, c.rope_dim, c.v_dim)
            self.xcd_kva, self.xcd_att_partials = z(lat), B(part)
            self.xcd_q = B(2 * c.n_heads * c.qk_dim * 2)     # raw q rows, then the rows with q_pe rotated
            self.xcd_xb = B(c.hidden * 2)
            for l in range(c.n_layers):   # o_proj's scales and biases per K-slice, once per matrix
                name = f"layers.{l}.self_attn.o_proj"
                Wo = weights.mats[name]
                self.xcd_kmeta[name] = (native.xcd_kslice_meta(Wo.scales, Wo.n, Wo.k // Wo.group),
                                        native.xcd_kslice_meta(Wo.biases, Wo.n, Wo.k // Wo.group))
            native.sync()
        self._rows_variants: Dict[int, "MoeRowsVariant"] = {}
        self.tasks = self.build_tasks()
        self.graph = self.d.build_decode_graph(self.tasks, False)

    def build_tasks(self) -> List[Dispatch]:
        c, w = self.cfg, self.w
        quant = dict(bits=c.bits, group=c.group)
        t: List[Dispatch] = []
        fid = [0]

        def name(kind: str) -> str:
            fid[0] += 1
            return f"fusekit_{kind}_f{fid[0]}"

        def wargs(W):
            return [arg(W.w)] if W.bits == 16 else [arg(W.w), arg(W.scales), arg(W.biases)]

        def fanout3(x, norm_w, hidden, parts, outs):
            """RMSNorm + three row blocks of projections in one launch (the rmsnorm_qkv family)."""
            (w0, s0, b0), (w1, s1, b1), (w2, s2, b2) = (p[0] for p in parts)
            n_q, n_kv = parts[0][1], parts[1][1]
            assert parts[2][1] == n_kv
            t.append(Dispatch(name("rmsnorm_qkv"), [x, arg(norm_w), w0, w1, w2, s0, s1, s2, b0, b1, b2] + outs,
                              dict(quant, hidden=hidden, n_q=n_q, n_kv=n_kv, eps=c.eps, has_norm=1, has_bias=0)))

        if c.fuse_attention:   # step_init also fills this token's (cos, sin) table, shared by all layers
            t.append(Dispatch("fusekit_step_init", [arg(self.step_counter), arg(self.offset), arg(self.kv_len), arg(self.rope_tab)],
                              dict(rope_dims=c.rope_dim, theta=c.theta)))
        else:
            t.append(Dispatch("fusekit_step_init", [arg(self.step_counter), arg(self.offset), arg(self.kv_len)]))
        emb = w.mats["embed_tokens"]
        t.append(Dispatch(name("embed_lookup_decode"), [arg(self.token)] + wargs(emb) + [arg(self.x[0])],
                          dict(bits=16, group=64, hidden=c.hidden, vocab=c.vocab, output_scale=1.0)))
        n_a, half_a = c.kv_lora_rank + c.rope_dim, (c.kv_lora_rank + c.rope_dim) // 2
        n_b = c.n_heads * (c.nope_dim + c.v_dim)
        if self.xcd_attn:
            self._two_launch_tasks(t, name, wargs, quant)
            return self._head_tasks(t, name, wargs, emb)
        for l in range(c.n_layers):
            p = f"layers.{l}."
            Wq, Wa, Wb = (w.mats[p + f"self_attn.{n}"] for n in ("q_proj", "kv_a_proj_with_mqa", "kv_b_proj"))
            # q and the two halves of kv_a (latent | k_pe lands contiguously in kva)
            fanout3(arg(self.x[0]), w.vecs[p + "input_layernorm"], c.hidden,
                    [(_rows(Wq, 0, Wq.n), Wq.n), (_rows(Wa, 0, half_a), half_a), (_rows(Wa, half_a, n_a), half_a)],
                    [arg(self.q), arg(self.kva, half_a * 2, 0), arg(self.kva, half_a * 2, half_a * 2)])
            # kv_b on the normalised latent, as row blocks of one half and two quarters
            fanout3(arg(self.kva, c.kv_lora_rank * 2, 0), w.vecs[p + "self_attn.kv_a_layernorm"], c.kv_lora_rank,
                    [(_rows(Wb, 0, n_b // 2), n_b // 2), (_rows(Wb, n_b // 2, 3 * n_b // 4), n_b // 4),
                     (_rows(Wb, 3 * n_b // 4, n_b), n_b // 4)],
                    [arg(self.kvb, n_b, 0), arg(self.kvb, n_b // 2, n_b), arg(self.kvb, n_b // 2, n_b + n_b // 2)])
            packed = c.nope_dim + c.v_dim
            split = dict(n_heads=c.n_heads, q0_dim=c.nope_dim, q1_dim=c.rope_dim, n_kv=c.n_heads, v_dim=c.v_dim, k1_n_kv=1,
                         k0_stride=packed, v_stride=packed, rope_dims=c.rope_dim, traditional=int(c.rope_traditional),
                         theta=c.theta, capacity=c.capacity)
            k0, k1 = arg(self.kvb), arg(self.kva, c.rope_dim * 2, c.kv_lora_rank * 2)
            vv = arg(self.kvb, self.kvb.nbytes - c.nope_dim * 2, c.nope_dim * 2)
            if c.fuse_attention:   # store + attention in one launch; the rotary table comes from step_init
                t.append(Dispatch(name("split_store_sdpa_decode"),
                                  [arg(self.q), k0, k1, vv, arg(self.cache_k[l]), arg(self.cache_v[l]), arg(self.kv_len),
                                   arg(self.att), arg(self.sdpa_partials), arg(self.sdpa_counters), arg(self.rope_tab)],
                                  dict(split, has_table=1, max_len=c.capacity)))
            else:
                t.append(Dispatch(name("kv_cache_store_decode"),
                                  [arg(self.q), k0, k1, vv, arg(self.cache_k[l]), arg(self.cache_v[l]), arg(self.offset),
                                   arg(self.offset)], dict(split, split_k=1, has_q=1, k0_dim=c.nope_dim, k1_dim=c.rope_dim)))
                t.append(Dispatch(name("sdpa_decode"),
                                  [arg(self.q), arg(self.cache_k[l]), arg(self.cache_v[l]), arg(self.kv_len), arg(self.att),
                                   arg(self.sdpa_partials), arg(self.sdpa_counters)],
                                  dict(n_heads=c.n_heads, n_kv=c.n_heads, qk_dim=c.qk_dim, head_dim=c.qk_dim, v_dim=c.v_dim,
                                       capacity=c.capacity, max_len=c.capacity)))
            Wo = w.mats[p + "self_attn.o_proj"]
            t.append(Dispatch(name("linear_residual"), [arg(self.att)] + wargs(Wo) + [arg(self.x[0]), arg(self.x[1])],
                              dict(quant, m=Wo.k, n=c.hidden)))
            post = w.vecs[p + "post_attention_layernorm"]
            if l < c.first_dense:
                Wg, Wu, Wd = (w.mats[p + f"mlp.{n}_proj"] for n in ("gate", "up", "down"))
                t.append(Dispatch(name("rmsnorm_gateup_swiglu"),
                                  [arg(self.x[1]), arg(post), arg(Wg.w), arg(Wu.w), arg(Wg.scales), arg(Wu.scales),
                                   arg(Wg.biases), arg(Wu.biases), arg(self.mid, c.dense_inter * 2)],
                                  dict(quant, hidden=c.hidden, inter=c.dense_inter, eps=c.eps, variant=c.swiglu_variant,
                                       has_norm=1)))
                t.append(Dispatch(name("linear_residual"),
                                  [arg(self.mid, c.dense_inter * 2)] + wargs(Wd) + [arg(self.x[1]), arg(self.x[0])],
                                  dict(quant, m=c.dense_inter, n=c.hidden)))
                continue
            Wr = w.mats[p + "mlp.gate"]
            ridx = arg(self.route_idx, 4 * c.top_k, 4 * c.top_k * l)
            rlg = arg(self.route_logits, 2 * c.n_experts, 2 * c.n_experts * l)
            rwt = arg(self.route_weight, 2 * c.top_k, 2 * c.top_k * l)
            route_in_consumer = self.fused_router and c.fuse_topk and c.fuse_shared and c.swiglu_variant == 1
            if self.xcd:            # the expert launch below forms and ranks the logits itself
                pass
            elif self.fused_router:   # norm + router projection (+ top-k route unless the expert launch ranks the logits itself)
                t.append(Dispatch(name("moe_router"),
                                  [arg(self.x[1]), arg(post), arg(Wr.w), arg(self.route_scale), arg(self.xn), rlg,
                                   ridx, rwt, arg(self.router_ws)],
                                  dict(hidden=c.hidden, experts=c.n_experts, top_k=0 if route_in_consumer else c.top_k, eps=c.eps,
                                       has_norm=1)))
            else:
                t.append(Dispatch(name("rmsnorm_rows"), [arg(self.x[1]), arg(post), arg(self.xn)],
                                  dict(rows=1, hidden=c.hidden, eps=c.eps)))
                t.append(Dispatch(name("qgemv"), [arg(self.xn), arg(Wr.w), rlg],
                                  dict(bits=16, group=64, m=c.hidden, n=c.n_experts)))
                t.append(Dispatch(name("softmax_topk_route"),
                                  [rlg, arg(self.route_scale), ridx, rwt],
                                  dict(row_n=c.n_experts, top_k=c.top_k, rows=1)))
            Eg, Eu, Ed = (w.mats[p + f"mlp.switch_mlp.{n}_proj"] for n in ("gate", "up", "down"))
            Sg, Su, Sd = (w.mats[p + f"mlp.shared_experts.{n}_proj"] for n in ("gate", "up", "down"))
            if self.xcd:   # one launch into a sum row, then sum row + residual -> x[0]
                a = [arg(self.x[1]), arg(self.xcd_x), arg(post), arg(Wr.w), arg(self.route_scale)]
                for W in (Eg, Eu, Ed, Sg, Su, Sd):
                    a += wargs(W)
                a += [rlg, ridx, rwt, arg(self.xcd_scratch), arg(self.xcd_sums[1]), arg(self.xcd_sums[0]), arg(self.xcd_sums[2]),
                      arg(self.xcd_ctl)]
                t.append(Dispatch(name("xcd_moe_block"), a,
                                  dict(quant, hidden=c.hidden, inter=c.moe_inter, shared_inter=c.shared_inter, experts=c.n_experts,
                                       top_k=c.top_k, eps=c.eps, variant=c.swiglu_variant, has_sums=0,
                                       spin_limit=c.xcd_spin_limit, mark_placement=int(l == c.first_dense))))
                t.append(Dispatch(name("xcd_reduce"), [arg(self.xcd_sums[0]), arg(self.x[1]), arg(self.x[0]), arg(self.xcd_sums[0]),
                                                       arg(self.xcd_sums[1]), arg(self.xcd_sums[1])], dict(hidden=c.hidden)))
                continue
            routed = [arg(self.xn), arg(Eg.w), arg(Eg.scales), arg(Eg.biases), arg(Eu.w), arg(Eu.scales), arg(Eu.biases),
                      arg(self.rows_x), ridx, arg(self.h)]
            rparams = dict(quant, k=c.hidden, o=c.moe_inter, experts=c.n_experts, routes=c.top_k, x_rows=1)
            shared_slots = [arg(Sg.w), arg(Sg.scales), arg(Sg.biases), arg(Su.w), arg(Su.scales), arg(Su.biases),
                            arg(self.mid, c.shared_inter * 2)]
            if route_in_consumer:   # the expert launch ranks the logits itself and writes the route for the reduction
                t.append(Dispatch(name("routed_qmv_swiglu"),
                                  [arg(self.xn), arg(Eg.w), arg(Eg.scales), arg(Eg.biases), arg(Eu.w), arg(Eu.scales), arg(Eu.biases),
                                   rlg, arg(self.route_scale), ridx, rwt, arg(self.h)] + shared_slots,
                                  dict(quant, k=c.hidden, o=c.moe_inter, experts=c.n_experts, routes=c.top_k, route_in_kernel=1,
                                       has_shared=1, shared_o=c.shared_inter)))
            elif c.fuse_shared and c.swiglu_variant == 1:   # the shared pair as further routes of the routed launch
                t.append(Dispatch(name("routed_qmv_swiglu"),
                                  routed + [arg(Sg.w), arg(Sg.scales), arg(Sg.biases), arg(Su.w), arg(Su.scales), arg(Su.biases),
                                            arg(self.mid, c.shared_inter * 2)],
                                  dict(rparams, has_shared=1, shared_o=c.shared_inter)))
            else:
                t.append(Dispatch(name("routed_qmv_swiglu"), routed, rparams))
                t.append(Dispatch(name("qmv_swiglu"),
                                  [arg(self.xn), arg(Sg.w), arg(Su.w), arg(Sg.scales), arg(Su.scales), arg(Sg.biases), arg(Su.biases),
                                   arg(self.mid, c.shared_inter * 2)],
                                  dict(quant, hidden=c.hidden, inter=c.shared_inter, eps=c.eps, variant=c.swiglu_variant, has_norm=0)))
            t.append(Dispatch(name("routed_qmv_reduce"),
                              [arg(self.h), arg(Ed.w), arg(Ed.scales), arg(Ed.biases), arg(self.rows_h), ridx,
                               rwt, arg(self.mid, c.shared_inter * 2), arg(Sd.w), arg(Sd.scales), arg(Sd.biases),
                               arg(self.x[1]), arg(self.x[0]), arg(self.moe_ws)],
                              dict(quant, k=c.moe_inter, o=c.hidden, experts=c.n_experts, tokens=1, top_k=c.top_k, x_rows=c.top_k,
                                   has_shared=1, shared_k=c.shared_inter, has_extra=1)))
        return self._head_tasks(t, name, wargs, emb)

    def _two_launch_tasks(self, t, name, wargs, quant) -> None:
        """A layer as TWO launches (families fusekit_xcd_mla_block / fusekit_xcd_moe_block; a dense layer keeps its
        per-dispatch MLP behind fusekit_xcd_reduce).  Sum rows: the attention launch of layer l adds into P[l % 2] and
        clears the pair Q[l % 2] its expert launch adds into; the expert launch reads P[l % 2], adds into Q[l % 2] and
        clears P[(l + 1) % 2]; the next attention launch reads Q[l % 2].  The closing fusekit_xcd_reduce clears what the
        last layer left, so that every row a token's first launches add into holds zeros."""
        c, w = self.cfg, self.w
        P = lambda i: arg(self.xcd_sums[i % 2])
        Q = lambda i: (arg(self.xcd_sums[2 + 2 * (i % 2)]), arg(self.xcd_sums[3 + 2 * (i % 2)]))
        mla = dict(quant, hidden=c.hidden, n_heads=c.n_heads, rank=c.kv_lora_rank, rope_dim=c.rope_dim, nope_dim=c.nope_dim,
                   v_dim=c.v_dim, capacity=c.capacity, eps=c.eps, theta=c.theta, traditional=int(c.rope_traditional),
                   spin_limit=c.xcd_spin_limit)
        from_experts = False          # the previous layer ended in an expert launch (two sum rows + the row in xcd_xb)
        for l in range(c.n_layers):
            p = f"layers.{l}."
            Wq, Wa, Wb, Wo = (w.mats[p + f"self_attn.{n}"] for n in ("q_proj", "kv_a_proj_with_mqa", "kv_b_proj", "o_proj"))
            sc, bi = self.xcd_kmeta[p + "self_attn.o_proj"]
            a = list(Q(l - 1)) if from_experts else []
            a += [arg(self.xcd_xb) if from_experts else arg(self.x[0]), arg(self.xcd_x), arg(w.vecs[p + "input_layernorm"])]
            a += wargs(Wq) + wargs(Wa) + [arg(w.vecs[p + "self_attn.kv_a_layernorm"])] + wargs(Wb) + [arg(Wo.w), arg(sc), arg(bi)]
            a += [arg(self.xcd_q), arg(self.xcd_kva), arg(self.kvb), arg(self.cache_k[l]), arg(self.cache_v[l]), arg(self.kv_len),
                  arg(self.rope_tab), arg(self.xcd_att_partials)]
            qr, qs = Q(l)
            a += [qs, P(l), qr, arg(self.xcd_ctl)]      # clear2 = the shared row, out, clear = the routes' row
            t.append(Dispatch(name("xcd_mla_block"), a, dict(mla, has_sums=2 if from_experts else 0, has_clear2=1,
                                                            mark_placement=int(l == 0))))
            post = w.vecs[p + "post_attention_layernorm"]
            if l < c.first_dense:   # x1 = T(P + x) as a row, then the per-dispatch MLP
                t.append(Dispatch(name("xcd_reduce"), [P(l), arg(self.xcd_x), arg(self.x[1]), P(l)], dict(hidden=c.hidden)))
                Wg, Wu, Wd = (w.mats[p + f"mlp.{n}_proj"] for n in ("gate", "up", "down"))
                t.append(Dispatch(name("rmsnorm_gateup_swiglu"),
                                  [arg(self.x[1]), arg(post), arg(Wg.w), arg(Wu.w), arg(Wg.scales), arg(Wu.scales),
                                   arg(Wg.biases), arg(Wu.biases), arg(self.mid, c.dense_inter * 2)],
                                  dict(quant, hidden=c.hidden, inter=c.dense_inter, eps=c.eps, variant=c.swiglu_variant,
                                       has_norm=1)))
                t.append(Dispatch(name("linear_residual"),
                                  [arg(self.mid, c.dense_inter * 2)] + wargs(Wd) + [arg(self.x[1]), arg(self.x[0])],
                                  dict(quant, m=c.dense_inter, n=c.hidden)))
                from_experts = False
                continue
            Wr = w.mats[p + "mlp.gate"]
            Eg, Eu, Ed = (w.mats[p + f"mlp.switch_mlp.{n}_proj"] for n in ("gate", "up", "down"))
            Sg, Su, Sd = (w.mats[p + f"mlp.shared_experts.{n}_proj"] for n in ("gate", "up", "down"))
            m = [P(l), arg(self.xcd_x), arg(self.xcd_xb), arg(post), arg(Wr.w), arg(self.route_scale)]
            for W in (Eg, Eu, Ed, Sg, Su, Sd):
                m += wargs(W)
            m += [arg(self.route_logits, 2 * c.n_experts, 2 * c.n_experts * l), arg(self.route_idx, 4 * c.top_k, 4 * c.top_k * l),
                  arg(self.route_weight, 2 * c.top_k, 2 * c.top_k * l), arg(self.xcd_scratch), qs, qr, P(l + 1), arg(self.xcd_ctl)]
            t.append(Dispatch(name("xcd_moe_block"), m,
                              dict(quant, hidden=c.hidden, inter=c.moe_inter, shared_inter=c.shared_inter, experts=c.n_experts,
                                   top_k=c.top_k, eps=c.eps, variant=c.swiglu_variant, has_sums=1, spin_limit=c.xcd_spin_limit)))
            from_experts = True
        if from_experts:   # the last layer's rows + its residual row -> x[0] for the LM head; leaves every row zero
            qr, qs = Q(c.n_layers - 1)
            t.append(Dispatch(name("xcd_reduce"), [qr, arg(self.xcd_xb), arg(self.x[0]), qr, qs, qs, P(c.n_layers - 1)],
                              dict(hidden=c.hidden)))

    def _head_tasks(self, t, name, wargs, emb) -> List[Dispatch]:
        c, w = self.cfg, self.w
        head_args = [arg(self.x[0]), arg(w.vecs["final_norm"])] + wargs(emb) + [arg(self.logits)]
        head_params = dict(bits=16, group=64, hidden=c.hidden, vocab=c.vocab, eps=c.eps)
        # the direct head (dispatch.py:3458-3505) as one launch where the vocabulary matrix takes the row-group GEMV
        self.direct_head = bool(c.direct_head_argmax and native.gemv_form(c.vocab, c.hidden, 16, 64) == 1)
        if self.direct_head:
            t.append(Dispatch(name("final_rmsnorm_lm_head_argmax"),
                              head_args + [arg(self.token), arg(self.head_argmax_ws), arg(self.history), arg(self.hist_counter)],
                              head_params))
            return t
        t.append(Dispatch(name("final_rmsnorm_lm_head"), head_args, head_params))
        t.append(Dispatch(name("argmax_logits_decode"),
                          [arg(self.logits), arg(self.token), arg(self.argmax_ws), arg(self.history), arg(self.hist_counter)],
                          dict(vocab=c.vocab)))
        return t

    def scratch_symbols(self):
        """name -> (buffer, dtype, zero-initialised) of every arena buffer, as the artifact describes them."""
        out = {}
        for name in ("token", "step_counter", "offset", "kv_len", "hist_counter", "history", "sdpa_counters", "argmax_ws",
                     "head_argmax_ws", "route_idx", "rows_x", "router_ws"):
            out[name] = (getattr(self, name), "uint32", True)
        out["x.0"], out["x.1"] = (self.x[0], "bfloat16", False), (self.x[1], "bfloat16", False)
        for name in ("xn", "q", "kva", "kvb", "att", "mid", "h", "logits", "moe_ws"):
            out[name] = (getattr(self, name), "bfloat16", False)
        for name in ("route_logits", "route_weight"):
            out[name] = (getattr(self, name), "bfloat16", True)
        out["sdpa_partials"], out["rope_tab"] = (self.sdpa_partials, "float32", False), (self.rope_tab, "float32", False)
        for l in range(self.cfg.n_layers):
            out[f"cache_k.{l}"], out[f"cache_v.{l}"] = (self.cache_k[l], "bfloat16", True), (self.cache_v[l], "bfloat16", True)
        if self.xcd:
            out["xcd.control"], out["xcd.scratch"] = (self.xcd_ctl, "uint32", True), (self.xcd_scratch, "uint32", True)
            out["xcd.x"] = (self.xcd_x, "bfloat16", False)
            if self.xcd_attn:
                out["xcd.x.1"], out["xcd.kva"] = (self.xcd_xb, "bfloat16", False), (self.xcd_kva, "bfloat16", True)
                out["xcd.attention_partials"], out["xcd.q"] = (self.xcd_att_partials, "float32", False), (self.xcd_q, "bfloat16", False)
            for i, b in enumerate(self.xcd_sums):
                out[f"xcd.sums.{i}"] = (b, "uint32", True)
        return out

    def routes(self) -> np.ndarray:
        """Expert indices the last replay chose, [n_layers, top_k] (rows of dense layers stay zero)."""
        return self.route_idx.to_numpy(np.uint32, (self.cfg.n_layers, self.cfg.top_k))

    def router_logits(self) -> np.ndarray:
        """bf16 router logits of the last replay, [n_layers, n_experts]."""
        return self.route_logits.to_numpy(np.uint16, (self.cfg.n_layers, self.cfg.n_experts))

    # -- several active token rows (the reference's active_m > 1: multi-token verification, chunked prefill)
    def forward_rows(self, tokens: Sequence[int], offset: int = 0) -> int:
        """Processes len(tokens) rows at positions offset .. in ONE pass over the weights: the replay of a
        `MoeRowsVariant` graph for that row count (built on first use).  Fills the KV caches and returns the
        greedy token after the last row."""
        m = len(tokens)
        v = self._rows_variants.get(m)
        if v is None:
            v = self._rows_variants[m] = MoeRowsVariant(self, m)
        nxt = v.run(tokens, offset)
        self.rows_routes = v.ridx.to_numpy(np.uint32, (self.cfg.n_layers, m, self.cfg.top_k))[-1]   # of the last expert layer
        return nxt

    # -- generation (the dense runtime's loop: prompt with forced tokens, then chunks fed back on the GPU)
    def reset(self) -> None:
        for b in (self.step_counter, self.offset, self.kv_len, self.hist_counter):
            b.upload(np.zeros(1, np.uint32))
        if self.xcd:
            for b in self.xcd_sums:
                b.upload(np.zeros(b.nbytes, np.uint8))

    def prefill(self, prompt: Sequence[int], start_offset: int = 0) -> int:
        preds, _ = self.d.decode_host_loop(self.graph, self.uniforms, start_offset, list(prompt))
        return preds[-1]

    def generate(self, prompt: Sequence[int], max_tokens: int):
        """Greedy decode: returns (tokens, seconds on the GPU for the decode chunks, decode steps)."""
        if len(prompt) + max_tokens > self.cfg.capacity:
            raise ValueError("prompt + max_tokens exceeds the KV-cache capacity")
        out = [self.prefill(prompt)]
        gpu_s, steps, offset = 0.0, 0, len(prompt)
        while len(out) < max_tokens:
            n = min(FK_CHUNK, max_tokens - len(out), self.uniforms.hist_capacity)
            toks, sec = self.d.decode_chunk(self.graph, self.uniforms, offset, out[-1], n)
            out += toks
            gpu_s += sec
            steps += n
            offset += n
        return out, gpu_s, steps


class MoeRowsVariant:
    """The whole MoE model for `m` active token rows as ONE task list / hipGraph (the reference's `active_m = m`
    variants, src/commands/patch.rs:112-150): multi-row matmuls for the dense projections and the shared experts,
    the row forms of the norm, the split-key store, the attention and the router, routed experts over
    m x top_k routes, the ordered reduction with the shared expert's rows.  `offset` (position of row 0) and
    `kv_len` (= offset + 1, row 0's) are device words the host writes before a replay; caches, token, history
    and logits are the decode graph's."""

    def __init__(self, rt: "MoeRuntime", m: int):
        c = rt.cfg
        if not 1 <= m <= c.capacity:
            raise ValueError("rows must lie in 1 .. capacity")
        if c.hidden % 512 or c.hidden > 4096:
            raise ValueError("the row form of the router needs hidden to be a multiple of 512 of at most 4096")
        self.rt, self.m, self.name = rt, m, f"prefill_m{m}"
        B, z = DeviceBuffer, native.zeros
        n_q, n_b = c.n_heads * c.qk_dim, c.n_heads * (c.nope_dim + c.v_dim)
        self.tokens, self.offset, self.kv_len = z(4 * m), z(4), z(4)
        self.x = [B(m * c.hidden * 2), B(m * c.hidden * 2)]
        self.xn = B(m * c.hidden * 2)
        self.q, self.lat, self.kpe, self.latn = B(m * n_q * 2), B(m * c.kv_lora_rank * 2), B(m * c.rope_dim * 2), B(m * c.kv_lora_rank * 2)
        self.kvb, self.att = B(m * n_b * 2), B(m * c.n_heads * c.v_dim * 2)
        # 2..8 rows: RMSNorm + q / kv_a, and RMSNorm(latent) + kv_b, are ONE launch each (the row form of the
        # rmsnorm_qkv family); kv_a's output rows are [latent | k_pe], as in the single-token list
        self.fan = 2 <= m <= 8 and c.bits in (4, 8) and c.group == 64
        self.kva = B(m * (c.kv_lora_rank + c.rope_dim) * 2)
        self.mid = B(m * max(c.dense_inter, c.shared_inter) * 2)
        routes = m * c.top_k
        self.ridx, self.rwt = z(4 * routes * c.n_layers), z(2 * routes * c.n_layers)
        self.rlg = z(2 * m * c.n_experts)
        self.rows_x = DeviceBuffer.from_numpy(np.repeat(np.arange(m, dtype=np.uint32), c.top_k))
        self.rows_h = DeviceBuffer.from_numpy(np.arange(routes, dtype=np.uint32))
        # the routes of a layer in the order the routed launches serve them: sorted by expert (fusekit_route_order)
        self.rank_in_launch = rt.route_order and 1 < routes <= 64      # the routed launches rank the routes themselves
        self.order = z(4 * routes) if (rt.route_order and 64 < routes <= 2048) else None
        self.h = B(routes * c.moe_inter * 2)
        self.router_ws = z(4 * m * (c.n_experts + 1))
        shapes = [(n_q, c.hidden), (c.kv_lora_rank, c.hidden), (c.rope_dim, c.hidden), (n_b, c.kv_lora_rank),
                  (c.hidden, c.n_heads * c.v_dim), (c.shared_inter, c.hidden), (c.dense_inter, c.hidden), (c.hidden, c.dense_inter)]
        self.qws = B(2 * max(native.qgemm_workspace_bytes(m, n, k, c.group) for n, k in shapes))
        self.moe_ws = B(native.routed_reduce_workspace_bytes(m, c.top_k, c.hidden, c.shared_inter, c.group))
        pb, cb = native.sdpa_workspace_bytes(c.n_heads, c.n_heads, c.qk_dim, c.v_dim, c.capacity)
        self.parts, self.counters = B(max(pb, 4) * m), z(max(cb, 4) * m)
        self.tasks = self._build()
        self.graph = rt.d.build_decode_graph(self.tasks, False)

    def _build(self) -> List[Dispatch]:
        rt, c, w, m = self.rt, self.rt.cfg, self.rt.w, self.m
        quant = dict(bits=c.bits, group=c.group)
        t: List[Dispatch] = []
        fid = [0]

        def name(kind: str) -> str:
            fid[0] += 1
            return f"fusekit_{kind}_f{fid[0]}"

        def matmul(x, wargs, k, n, out, res=None):
            a = [arg(x)] + list(wargs) + ([arg(res)] if res is not None else []) + [arg(out), arg(self.qws)]
            t.append(Dispatch(name("qgemm"), a, dict(quant, m=k, n=n, rows=m, has_bias=0, has_residual=int(res is not None))))

        def full(W):
            return [arg(W.w), arg(W.scales), arg(W.biases)]

        def norm_rows(x, nw, hidden, out):
            t.append(Dispatch(name("rmsnorm_rows"), [arg(x), arg(nw), arg(out)], dict(rows=m, hidden=hidden, eps=c.eps)))

        def fan3(x, x_stride, norm_w, hidden, parts, outs):
            """RMSNorm + three row blocks of projections of the m rows in one launch (row form of rmsnorm_qkv);
            outs: (buffer, first column, row stride in elements) per block."""
            (w0, s0, b0), (w1, s1, b1), (w2, s2, b2) = (pt[0] for pt in parts)
            n0, n1 = parts[0][1], parts[1][1]
            assert parts[2][1] == n1
            o = [arg(buf, ((m - 1) * st + n) * 2, col * 2) for (buf, col, st), n in zip(outs, (n0, n1, n1))]
            t.append(Dispatch(name("rmsnorm_qkv"), [x, arg(norm_w), w0, w1, w2, s0, s1, s2, b0, b1, b2] + o,
                              dict(quant, hidden=hidden, n_q=n0, n_kv=n1, eps=c.eps, has_norm=1, has_bias=0, rows=m,
                                   x_row_stride=x_stride, q_row_stride=outs[0][2], k_row_stride=outs[1][2], v_row_stride=outs[2][2])))

        def swiglu(Wg, Wu, inter):
            t.append(Dispatch(name("qgemm_swiglu"),
                              [arg(self.xn), arg(Wg.w), arg(Wu.w), arg(Wg.scales), arg(Wu.scales), arg(Wg.biases), arg(Wu.biases),
                               arg(self.mid, m * inter * 2), arg(self.qws)],
                              dict(quant, hidden=c.hidden, inter=inter, rows=m, variant=c.swiglu_variant)))

        emb = w.mats["embed_tokens"]
        t.append(Dispatch(name("embed_lookup_decode"), [arg(self.tokens), arg(emb.w), arg(self.x[0])],
                          dict(bits=16, group=64, hidden=c.hidden, vocab=c.vocab, output_scale=1.0, rows=m)))
        n_q, n_a, n_b = c.n_heads * c.qk_dim, c.kv_lora_rank + c.rope_dim, c.n_heads * (c.nope_dim + c.v_dim)
        packed, routes = c.nope_dim + c.v_dim, m * c.top_k
        for l in range(c.n_layers):
            p = f"layers.{l}."
            Wq, Wa, Wb, Wo = (w.mats[p + f"self_attn.{n}"] for n in ("q_proj", "kv_a_proj_with_mqa", "kv_b_proj", "o_proj"))
            if self.fan:
                half_a = n_a // 2
                fan3(arg(self.x[0]), c.hidden, w.vecs[p + "input_layernorm"], c.hidden,
                     [(_rows(Wq, 0, n_q), n_q), (_rows(Wa, 0, half_a), half_a), (_rows(Wa, half_a, n_a), half_a)],
                     [(self.q, 0, n_q), (self.kva, 0, n_a), (self.kva, half_a, n_a)])
                fan3(arg(self.kva, ((m - 1) * n_a + c.kv_lora_rank) * 2, 0), n_a, w.vecs[p + "self_attn.kv_a_layernorm"], c.kv_lora_rank,
                     [(_rows(Wb, 0, n_b // 2), n_b // 2), (_rows(Wb, n_b // 2, 3 * n_b // 4), n_b // 4),
                      (_rows(Wb, 3 * n_b // 4, n_b), n_b // 4)],
                     [(self.kvb, 0, n_b), (self.kvb, n_b // 2, n_b), (self.kvb, 3 * n_b // 4, n_b)])
                kpe, kpe_stride = arg(self.kva, ((m - 1) * n_a + c.rope_dim) * 2, c.kv_lora_rank * 2), n_a
            else:
                norm_rows(self.x[0], w.vecs[p + "input_layernorm"], c.hidden, self.xn)
                matmul(self.xn, full(Wq), c.hidden, n_q, self.q)
                matmul(self.xn, _rows(Wa, 0, c.kv_lora_rank), c.hidden, c.kv_lora_rank, self.lat)
                matmul(self.xn, _rows(Wa, c.kv_lora_rank, n_a), c.hidden, c.rope_dim, self.kpe)
                norm_rows(self.lat, w.vecs[p + "self_attn.kv_a_layernorm"], c.kv_lora_rank, self.latn)
                matmul(self.latn, full(Wb), c.kv_lora_rank, n_b, self.kvb)
                kpe, kpe_stride = arg(self.kpe), c.rope_dim
            t.append(Dispatch(name("kv_cache_store_decode"),
                              [arg(self.q), arg(self.kvb), kpe, arg(self.kvb, self.kvb.nbytes - c.nope_dim * 2, c.nope_dim * 2),
                               arg(rt.cache_k[l]), arg(rt.cache_v[l]), arg(self.offset), arg(self.offset)],
                              dict(split_k=1, has_q=1, n_heads=c.n_heads, q0_dim=c.nope_dim, q1_dim=c.rope_dim, n_kv=c.n_heads,
                                   k0_dim=c.nope_dim, k1_dim=c.rope_dim, v_dim=c.v_dim, k1_n_kv=1, k0_stride=packed, v_stride=packed,
                                   rope_dims=c.rope_dim, traditional=int(c.rope_traditional), theta=c.theta, capacity=c.capacity,
                                   rows=m, k0_row_stride=n_b, k1_row_stride=kpe_stride, v_row_stride=n_b)))
            t.append(Dispatch(name("sdpa_decode"),
                              [arg(self.q), arg(rt.cache_k[l]), arg(rt.cache_v[l]), arg(self.kv_len), arg(self.att), arg(self.parts),
                               arg(self.counters)],
                              dict(n_heads=c.n_heads, n_kv=c.n_heads, qk_dim=c.qk_dim, head_dim=c.qk_dim, v_dim=c.v_dim,
                                   capacity=c.capacity, max_len=c.capacity, rows=m)))
            matmul(self.att, full(Wo), c.n_heads * c.v_dim, c.hidden, self.x[1], res=self.x[0])
            post = w.vecs[p + "post_attention_layernorm"]
            if l < c.first_dense:
                Wg, Wu = w.mats[p + "mlp.gate_proj"], w.mats[p + "mlp.up_proj"]
                if self.fan:    # the norm rides in the gate / up launch (row form of rmsnorm_gateup_swiglu)
                    t.append(Dispatch(name("rmsnorm_gateup_swiglu"),
                                      [arg(self.x[1]), arg(post), arg(Wg.w), arg(Wu.w), arg(Wg.scales), arg(Wu.scales), arg(Wg.biases),
                                       arg(Wu.biases), arg(self.mid, m * c.dense_inter * 2)],
                                      dict(quant, hidden=c.hidden, inter=c.dense_inter, eps=c.eps, variant=c.swiglu_variant,
                                           has_norm=1, rows=m)))
                else:
                    norm_rows(self.x[1], post, c.hidden, self.xn)
                    swiglu(Wg, Wu, c.dense_inter)
                matmul(self.mid, full(w.mats[p + "mlp.down_proj"]), c.dense_inter, c.hidden, self.x[0], res=self.x[1])
                continue
            ridx = arg(self.ridx, 4 * routes, 4 * routes * l)
            rwt = arg(self.rwt, 2 * routes, 2 * routes * l)
            t.append(Dispatch(name("moe_router"),
                              [arg(self.x[1]), arg(post), arg(w.mats[p + "mlp.gate"].w), arg(rt.route_scale), arg(self.xn), arg(self.rlg),
                               ridx, rwt, arg(self.router_ws)],
                              dict(hidden=c.hidden, experts=c.n_experts, top_k=c.top_k, eps=c.eps, has_norm=1, rows=m)))
            Eg, Eu, Ed = (w.mats[p + f"mlp.switch_mlp.{n}_proj"] for n in ("gate", "up", "down"))
            Sg, Su, Sd = (w.mats[p + f"mlp.shared_experts.{n}_proj"] for n in ("gate", "up", "down"))
            order, ordered = ([arg(self.order)], dict(has_order=1)) if self.order is not None else ([], {})
            if self.rank_in_launch:
                ordered = dict(expert_order=1)
            if order:
                t.append(Dispatch(name("route_order"), [ridx, arg(self.order)], dict(routes=routes, experts=c.n_experts)))
            t.append(Dispatch(name("routed_qmv_swiglu"),
                              [arg(self.xn), arg(Eg.w), arg(Eg.scales), arg(Eg.biases), arg(Eu.w), arg(Eu.scales), arg(Eu.biases),
                               arg(self.rows_x), ridx, arg(self.h)] + order,
                              dict(quant, k=c.hidden, o=c.moe_inter, experts=c.n_experts, routes=routes, x_rows=m, **ordered)))
            swiglu(Sg, Su, c.shared_inter)
            t.append(Dispatch(name("routed_qmv_reduce"),
                              [arg(self.h), arg(Ed.w), arg(Ed.scales), arg(Ed.biases), arg(self.rows_h), ridx, rwt,
                               arg(self.mid, m * c.shared_inter * 2), arg(Sd.w), arg(Sd.scales), arg(Sd.biases), arg(self.x[1]),
                               arg(self.x[0]), arg(self.moe_ws)] + order,
                              dict(quant, k=c.moe_inter, o=c.hidden, experts=c.n_experts, tokens=m, top_k=c.top_k, x_rows=routes,
                                   has_shared=1, shared_k=c.shared_inter, has_extra=1, **ordered)))
        last = arg(self.x[0], c.hidden * 2, (m - 1) * c.hidden * 2)
        t.append(Dispatch(name("final_rmsnorm_lm_head"), [last, arg(w.vecs["final_norm"]), arg(emb.w), arg(rt.logits)],
                          dict(bits=16, group=64, hidden=c.hidden, vocab=c.vocab, eps=c.eps)))
        t.append(Dispatch(name("argmax_logits_decode"),
                          [arg(rt.logits), arg(rt.token), arg(rt.argmax_ws), arg(rt.history), arg(rt.hist_counter)], dict(vocab=c.vocab)))
        return t

    def run(self, tokens: Sequence[int], offset: int) -> int:
        rt = self.rt
        tokens = list(tokens)
        if len(tokens) != self.m:
            raise ValueError(f"a variant of {self.m} rows processes exactly {self.m} tokens")
        if offset + self.m > rt.cfg.capacity:
            raise ValueError("rows exceed the KV-cache capacity")
        self.tokens.upload(np.asarray(tokens, np.uint32))
        self.offset.upload(np.array([offset], np.uint32))
        self.kv_len.upload(np.array([offset + 1], np.uint32))     # row 0's length; row r attends to kv_len + r positions
        rt.d.execute_graph(self.graph)
        return int(rt.token.to_numpy(np.uint32)[0])


class _View:
    """`nbytes` bytes at `offset` into a DeviceBuffer, usable wherever the bindings take a buffer."""

    def __init__(self, buf, offset: int, nbytes: int):
        self.ptr, self.nbytes = buf.ptr + offset, nbytes

    def __int__(self) -> int:
        return self.ptr


def _bf16(a: np.ndarray) -> np.ndarray:
    u = np.ascontiguousarray(a, np.float32).view(np.uint32)
    return ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)
