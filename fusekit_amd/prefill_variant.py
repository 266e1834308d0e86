"""`prefill_mN` variants: the whole model for N active token rows as ONE task list / hipGraph.

The reference compiles, next to the decode artifact, variants with `active_m = N` under
`variants/prefill_mN` (src/commands/patch.rs:112-150) and its runtime takes one when exactly N prompt
tokens are to be processed (python/fusekit_runtime/__init__.py:4866).  Here a variant is the list of
multi-row dispatches over a private activation arena, sharing the KV caches, the token / history
uniforms and the logits with the decode graph:

    embed rows -> per layer [RMSNorm rows, q / k / v matmul, RoPE + cache store of the N rows,
    causal attention (kv_len read on the device), o matmul + residual, RMSNorm rows,
    gate/up matmul + SwiGLU, down matmul + residual] -> final norm + LM head on the last row -> argmax

(for 2..8 rows of 4- / 8-bit weights the norms ride in the launches behind them: RMSNorm + q / k / v is one launch,
RMSNorm + gate/up + SwiGLU another)

`offset` (position of row 0) and `kv_len` (= offset + N) are device words the host writes before a
replay, so one graph serves any position.  Every node is a kernel of this library (the fused
multi-row matmul; a library GEMM cannot be a node), quantised weights and a bf16 KV cache only.
"""
from __future__ import annotations

from typing import Dict, List, Sequence

import numpy as np

from . import native
from .native import DeviceBuffer
from .runtime import Dispatch, arg


class PrefillVariant:
    def __init__(self, rt, m: int):
        c = rt.cfg
        if c.bits == 16 or c.kv_bits or c.head_dim not in (64, 128):
            raise ValueError("prefill variants need quantised weights, a bf16 KV cache and head_dim 64 or 128")
        if not 1 <= m <= c.capacity:
            raise ValueError("active_m must lie in 1 .. capacity")
        self.rt, self.m = rt, m
        self.name = f"prefill_m{m}"
        B = DeviceBuffer
        self.tokens, self.offset, self.kv_len = native.zeros(4 * m), native.zeros(4), native.zeros(4)
        self.x = [B(m * c.hidden * 2), B(m * c.hidden * 2)]
        self.xn = B(m * c.hidden * 2)
        self.q, self.k, self.v = B(m * c.n_q * 2), B(m * c.n_kvd * 2), B(m * c.n_kvd * 2)
        self.att, self.mid = B(m * c.n_q * 2), B(m * c.inter * 2)
        ws = max(native.qgemm_workspace_bytes(m, n, k, c.group)
                 for n, k in ((c.n_q, c.hidden), (c.n_q + 2 * c.n_kvd, c.hidden), (c.n_kvd, c.hidden), (c.hidden, c.n_q),
                              (c.inter, c.hidden), (c.hidden, c.inter)))
        self.ws = B(2 * ws)
        self.tasks = self._build()
        self.graph = rt.d.build_decode_graph(self.tasks, False)

    def scratch(self) -> Dict[str, DeviceBuffer]:
        """Buffers private to the variant, by the role name the artifact gives them."""
        p = self.name + "."
        return {p + "tokens": self.tokens, p + "offset": self.offset, p + "kv_len": self.kv_len, p + "x.0": self.x[0],
                p + "x.1": self.x[1], p + "xn": self.xn, p + "q": self.q, p + "k": self.k, p + "v": self.v, p + "att": self.att,
                p + "mid": self.mid, p + "ws": self.ws}

    def _fanout_applies(self, task: Dispatch) -> bool:
        """Whether the family fusekit_qgemm_fanout plans this dispatch (its tile form needs 65 rows or more)."""
        if getattr(self, "_fanout", None) is None:
            try:
                self.rt.d.plan_geometry(task)
                self._fanout = True
            except native.FusekitError:
                self._fanout = False
        return self._fanout

    def _build(self) -> List[Dispatch]:
        rt, c, w, m = self.rt, self.rt.cfg, self.rt.w, self.m
        quant = dict(bits=c.bits, group=c.group)
        t: List[Dispatch] = []
        fid = [0]

        def name(kind: str) -> str:
            fid[0] += 1
            return f"fusekit_{kind}_f{fid[0]}"

        def wargs(W):
            return [arg(W.w), arg(W.scales), arg(W.biases)]

        def matmul(x, W, out, bias=None, res=None):
            a = [arg(x)] + wargs(W) + ([arg(bias)] if bias is not None else []) + ([arg(res)] if res is not None else [])
            t.append(Dispatch(name("qgemm"), a + [arg(out), arg(self.ws)],
                              dict(quant, m=W.k, n=W.n, rows=m, has_bias=int(bias is not None), has_residual=int(res is not None))))

        emb = w.mats["embed_tokens"]
        head = w.mats.get("lm_head", emb)
        t.append(Dispatch(name("embed_lookup_decode"), [arg(self.tokens)] + rt._wargs(emb) + [arg(self.x[0])],
                          dict(bits=emb.bits, group=emb.group or 64, hidden=c.hidden, vocab=c.vocab, output_scale=c.embed_scale, rows=m)))
        # 2..8 rows of 4- / 8-bit weights: the norm and the projections behind it are ONE launch (row forms of the
        # rmsnorm_qkv and rmsnorm_gateup_swiglu families: the norm is applied while the rows are staged)
        fused = 2 <= m <= 8 and c.bits in (4, 8) and c.group == 64
        for l in range(c.n_layers):
            p = f"layers.{l}."
            if fused and not c.qkv_bias:
                Wq, Wk, Wv = (w.mats[p + f"self_attn.{nm}_proj"] for nm in "qkv")
                t.append(Dispatch(name("rmsnorm_qkv"),
                                  [arg(self.x[0]), arg(w.vecs[p + "input_layernorm"]), arg(Wq.w), arg(Wk.w), arg(Wv.w),
                                   arg(Wq.scales), arg(Wk.scales), arg(Wv.scales), arg(Wq.biases), arg(Wk.biases), arg(Wv.biases),
                                   arg(self.q), arg(self.k), arg(self.v)],
                                  dict(quant, hidden=c.hidden, n_q=Wq.n, n_kv=Wk.n, eps=c.eps, has_norm=1, has_bias=0, rows=m)))
            else:
                t.append(Dispatch(name("rmsnorm_rows"), [arg(self.x[0]), arg(w.vecs[p + "input_layernorm"]), arg(self.xn)],
                                  dict(rows=m, hidden=c.hidden, eps=c.eps)))
                Wq, Wk, Wv = (w.mats[p + f"self_attn.{nm}_proj"] for nm in "qkv")
                qkv_bias = [w.vecs.get(p + f"self_attn.{nm}_proj.bias") for nm in "qkv"] if c.qkv_bias else []
                fan = Dispatch(name("qgemm_fanout"),
                               [arg(self.xn), arg(Wq.w), arg(Wk.w), arg(Wv.w), arg(Wq.scales), arg(Wk.scales), arg(Wv.scales),
                                arg(Wq.biases), arg(Wk.biases), arg(Wv.biases)] + [arg(b_) for b_ in qkv_bias] +
                               [arg(self.q), arg(self.k), arg(self.v), arg(self.ws)],
                               dict(quant, hidden=c.hidden, n_q=Wq.n, n_kv=Wk.n, rows=m, has_bias=int(c.qkv_bias)))
                if self._fanout_applies(fan):      # q, k and v as one launch of the fused kernel's tile form
                    t.append(fan)
                else:
                    fid[0] -= 1
                    for nm, dst in (("q", self.q), ("k", self.k), ("v", self.v)):
                        matmul(self.xn, w.mats[p + f"self_attn.{nm}_proj"], dst,
                               bias=w.vecs.get(p + f"self_attn.{nm}_proj.bias") if c.qkv_bias else None)
            a = [arg(self.q), arg(self.k), arg(self.v)]
            if c.qk_norm:
                a += [arg(w.vecs[p + "self_attn.q_norm"]), arg(w.vecs[p + "self_attn.k_norm"])]
            a += [arg(rt.cache_k[l]), arg(rt.cache_v[l]), arg(self.offset)]
            t.append(Dispatch(name("qkv_rope_store_decode"), a,
                              dict(n_heads=c.n_heads, n_kv=c.n_kv, head_dim=c.head_dim, rope_dims=c.head_dim, theta=c.theta,
                                   capacity=c.capacity, eps=c.eps, has_norm=int(c.qk_norm), rows=m)))
            t.append(Dispatch(name("sdpa_prefill"),
                              [arg(self.q), arg(rt.cache_k[l]), arg(rt.cache_v[l]), arg(self.kv_len), arg(self.att)],
                              dict(n_heads=c.n_heads, n_kv=c.n_kv, head_dim=c.head_dim, capacity=c.capacity, rows=m)))
            matmul(self.att, w.mats[p + "self_attn.o_proj"], self.x[1], res=self.x[0])
            Wg, Wu = w.mats[p + "mlp.gate_proj"], w.mats[p + "mlp.up_proj"]
            if fused:
                t.append(Dispatch(name("rmsnorm_gateup_swiglu"),
                                  [arg(self.x[1]), arg(w.vecs[p + "post_attention_layernorm"]), arg(Wg.w), arg(Wu.w), arg(Wg.scales),
                                   arg(Wu.scales), arg(Wg.biases), arg(Wu.biases), arg(self.mid)],
                                  dict(quant, hidden=c.hidden, inter=c.inter, eps=c.eps, variant=c.swiglu_variant, has_norm=1, rows=m)))
            else:
                t.append(Dispatch(name("rmsnorm_rows"), [arg(self.x[1]), arg(w.vecs[p + "post_attention_layernorm"]), arg(self.xn)],
                                  dict(rows=m, hidden=c.hidden, eps=c.eps)))
                t.append(Dispatch(name("qgemm_swiglu"),
                                  [arg(self.xn), arg(Wg.w), arg(Wu.w), arg(Wg.scales), arg(Wu.scales), arg(Wg.biases), arg(Wu.biases),
                                   arg(self.mid), arg(self.ws)],
                                  dict(quant, hidden=c.hidden, inter=c.inter, rows=m, variant=c.swiglu_variant)))
            matmul(self.mid, w.mats[p + "mlp.down_proj"], self.x[0], res=self.x[1])
        last = arg(self.x[0], c.hidden * 2, (m - 1) * c.hidden * 2)  # the last row's hidden state
        t.append(Dispatch(name("final_rmsnorm_lm_head"), [last, arg(w.vecs["final_norm"])] + rt._wargs(head) + [arg(rt.logits)],
                          dict(bits=head.bits, group=head.group or 64, hidden=c.hidden, vocab=c.vocab, eps=c.eps)))
        t.append(Dispatch(name("argmax_logits_decode"),
                          [arg(rt.logits), arg(rt.token), arg(rt.argmax_ws), arg(rt.history), arg(rt.hist_counter)],
                          dict(vocab=c.vocab)))
        return t

    def run(self, tokens: Sequence[int], offset: int) -> int:
        """Processes exactly `m` tokens at positions offset .. offset + m - 1; returns the greedy next token."""
        return run_variant(self.rt.d, self.graph, self.m, self.tokens, self.offset, self.kv_len, self.rt.token, tokens, offset,
                           self.rt.cfg.capacity)


def run_variant(d, graph, m, tokens_buf, offset_buf, kv_len_buf, token_buf, tokens, offset, capacity) -> int:
    tokens = list(tokens)
    if len(tokens) != m:
        raise ValueError(f"a prefill_m{m} variant processes exactly {m} tokens")
    if offset + m > capacity:
        raise ValueError("prompt exceeds the KV-cache capacity")
    tokens_buf.upload(np.asarray(tokens, np.uint32))
    offset_buf.upload(np.array([offset], np.uint32))
    kv_len_buf.upload(np.array([offset + m], np.uint32))
    d.execute_graph(graph)
    return int(token_buf.to_numpy(np.uint32)[0])
