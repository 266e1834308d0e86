"""The per-model artifact of the decode path: `task_graph.json` (schema version 2) and `manifest.json`.

The reference's compiler writes these next to `kernel.metallib` (src/codegen/task_graph_json.rs:31-227,
src/manifest.rs:26-100) and its Python runtime resolves every task's buffer slots from them
(python/fusekit_runtime/dispatch.py).  For the HIP target the kernels live in the library, so the
artifact is the task list only.  `write_artifact` serialises a DecoderRuntime's task list in that
schema -- kernel name, grid_threads / threadgroup as the launch planners decide them, every slot as
an `external` (model parameter, by `source_path`) or `scratch` binding, `depends_on` from the graph's
hazard edges, `layer_groups`, `decode_pipeline` -- plus the per-task `params` object the HIP kernels
take instead of constants baked into generated source.  `load_artifact` is the consumer: it
allocates what the file describes, binds the parameters of a DecoderWeights by path and returns a
runtime whose graph replays the same decode.
"""
from __future__ import annotations

import dataclasses
import json
import os
import re
import time
from typing import Dict, List, Optional

import numpy as np

from . import native
from .decoder import DecoderConfig, DecoderRuntime, DecoderWeights
from .native import DeviceBuffer
from .runtime import Dispatch, Dispatcher, make_uniforms

SCHEMA_VERSION = 2
BACKEND_VERSION = "fusekit_amd-0.1"


def _symbols(rt: DecoderRuntime) -> Dict[int, dict]:
    """Device pointer -> how the slot is described in the artifact."""
    sym: Dict[int, dict] = {}

    def scratch(name: str, buf: DeviceBuffer, dtype: str, zero: bool = False):
        sym[buf.ptr] = dict(role="scratch", role_name=name, dtype=dtype, size_bytes=buf.nbytes, zero=zero)

    if hasattr(rt, "scratch_symbols"):   # a runtime that names its own arena (the mixture-of-experts decoder)
        for name, (buf, dtype, zero) in rt.scratch_symbols().items():
            scratch(name, buf, dtype, zero)
        _parameter_symbols(rt, sym)
        _kslice_symbols(rt, sym)
        return sym
    for name in ("token", "step_counter", "offset", "kv_len", "hist_counter", "history", "sdpa_counters", "argmax_ws",
                 "head_argmax_ws"):
        scratch(name, getattr(rt, name), "uint32", zero=True)
    scratch("x.0", rt.x[0], "bfloat16")
    scratch("x.1", rt.x[1], "bfloat16")
    for name in ("q", "k", "v", "att", "mid", "logits"):
        scratch(name, getattr(rt, name), "bfloat16")
    scratch("sdpa_partials", rt.sdpa_partials, "float32")
    if rt.rope_tab is not None:
        scratch("rope_tab", rt.rope_tab, "float32")
    if getattr(rt, "xcd", False):   # a layer as two launches: control words, sum rows, the rows between the launches
        scratch("xcd.control", rt.xcd_ctl, "uint32", zero=True)
        scratch("xcd.attention_partials", rt.xcd_att_partials, "float32")
        scratch("xcd.x.0", rt.xcd_xa, "bfloat16")
        scratch("xcd.x.1", rt.xcd_xb, "bfloat16")
        for i, b in enumerate(rt.xcd_sums):
            scratch(f"xcd.sums.{i}", b, "uint32", zero=True)
        for l, bufs in enumerate(getattr(rt, "xcd_qkv", [])):
            for nm, b in zip("qkv", bufs):
                scratch(f"xcd.{nm}.{l}", b, "bfloat16")
    for l in range(rt.cfg.n_layers):
        if rt.cfg.kv_bits:
            for nm, c in (("cache_k", rt.cache_k[l]), ("cache_v", rt.cache_v[l])):
                scratch(f"{nm}.{l}.packed", c.packed, "uint32", zero=True)
                scratch(f"{nm}.{l}.scales", c.scales, "bfloat16", zero=True)
                scratch(f"{nm}.{l}.biases", c.biases, "bfloat16", zero=True)
        else:
            scratch(f"cache_k.{l}", rt.cache_k[l], "bfloat16", zero=True)
            scratch(f"cache_v.{l}", rt.cache_v[l], "bfloat16", zero=True)
    _parameter_symbols(rt, sym)
    _kslice_symbols(rt, sym)
    return sym


def _kslice_symbols(rt, sym: Dict[int, dict]) -> None:
    """Scales / biases of o_proj and down_proj as the XCD-resident launches bind them: a parameter behind a load-time
    re-layout, named by the parameter and the transform."""
    for path, (sc, bi) in getattr(rt, "xcd_kmeta", {}).items():
        W = rt.w.mats[path]
        for buf, leaf in ((sc, ".scales"), (bi, ".biases")):
            sym[buf.ptr] = dict(role="external", source_path=path + leaf, dtype="bfloat16", transform="xcd_kslice",
                                shape=[W.n, W.k // W.group], size_bytes=buf.nbytes)


def _parameter_symbols(rt, sym: Dict[int, dict]) -> None:
    for path, W in rt.w.mats.items():
        lead = [W.n_experts] if getattr(W, "n_experts", 0) else []   # expert-stacked tensors [E, n, ...]
        sym[W.w.ptr] = dict(role="external", source_path=path + ".weight", dtype="uint32" if W.bits != 16 else "bfloat16",
                            shape=lead + ([W.n, W.k * W.bits // 32] if W.bits != 16 else [W.n, W.k]), size_bytes=W.w.nbytes)
        if W.bits != 16:
            sym[W.scales.ptr] = dict(role="external", source_path=path + ".scales", dtype="bfloat16",
                                     shape=lead + [W.n, W.k // W.group], size_bytes=W.scales.nbytes)
            sym[W.biases.ptr] = dict(role="external", source_path=path + ".biases", dtype="bfloat16",
                                     shape=lead + [W.n, W.k // W.group], size_bytes=W.biases.nbytes)
    for path, v in rt.w.vecs.items():
        sym[v.ptr] = dict(role="external", source_path=path, dtype="bfloat16", shape=[v.nbytes // 2], size_bytes=v.nbytes)


def _resolve(sym: Dict[int, dict], ptr: int):
    """The symbol a slot points into, and the byte offset inside it (a slot may be a slice of a buffer:
    part of an arena, or a block of rows of a parameter)."""
    s = sym.get(ptr)
    if s is not None:
        return s, 0
    for base, cand in sym.items():
        if base < ptr < base + cand["size_bytes"]:
            return cand, ptr - base
    return None, 0


def _graph_dict(rt: DecoderRuntime, task_list: List[Dispatch], graph_id: int, sym: Dict[int, dict], active_m: int,
                uniforms: Dict[str, str]) -> dict:
    scratch_ids: Dict[str, int] = {}
    scratch_buffers: List[dict] = []
    tasks: List[dict] = []
    groups: Dict[str, List[int]] = {}
    for tid, d in enumerate(task_list):
        geo = rt.d.plan_geometry(d)
        bindings = []
        for slot, (ptr, nbytes) in enumerate(d.args):
            s, off = _resolve(sym, ptr)
            if s is None:
                raise ValueError(f"task {tid} ({d.kernel}) slot {slot}: buffer is not a known parameter or scratch")
            access = geo.slot_access[slot]
            b = dict(slot=slot, role=s["role"], access=("rw" if access == 3 else "w" if access == 2 else "r"),
                     nbytes=nbytes, dtype=s["dtype"])
            if off:
                b["offset_bytes"] = off
            if s["role"] == "external":
                b.update(source_path=s["source_path"], shape=s["shape"], role_name=s["source_path"].rsplit(".", 1)[-1])
                if s.get("transform"):
                    b["transform"] = s["transform"]
            else:
                name = s["role_name"]
                if name not in scratch_ids:
                    scratch_ids[name] = len(scratch_buffers)
                    scratch_buffers.append(dict(id=scratch_ids[name], role_name=name, dtype=s["dtype"],
                                                shape=[s["size_bytes"] // (4 if s["dtype"] != "bfloat16" else 2)],
                                                size_bytes=s["size_bytes"], zero_init=s["zero"]))
                b.update(scratch_id=scratch_ids[name], role_name=name)
            bindings.append(b)
        m = re.search(r"cache_k\.(\d+)", " ".join(b.get("role_name", "") for b in bindings))
        lm = [re.match(r"layers\.(\d+)\.", b.get("source_path", "")) for b in bindings]
        layer = next((int(x.group(1)) for x in lm if x), int(m.group(1)) if m else None)
        kernels = [dict(grid=list(geo.grid[i]), threadgroup=list(geo.threadgroup[i]), lds_bytes=geo.lds_bytes[i])
                   for i in range(geo.n_kernels)]
        task = dict(id=tid, fusion_id=tid, kernel=d.kernel,
                    grid_threads=[kernels[0]["grid"][a] * kernels[0]["threadgroup"][a] for a in range(3)],
                    threadgroup=kernels[0]["threadgroup"],
                    inputs=[b for b in bindings if b["access"] == "r"],
                    outputs=[b for b in bindings if b["access"] != "r"],
                    params={k: float(v) for k, v in d.params.items()},
                    kernels=kernels, depends_on=rt.d.node_deps(graph_id, tid), trigger_event=tid)
        if layer is not None:
            task["layer_idx"] = layer
        tasks.append(task)
        region = "embed" if layer is None and tid < 2 else (f"layer.{layer}" if layer is not None else "post")
        groups.setdefault(region, []).append(tid)
    c = rt.cfg
    return dict(
        version=SCHEMA_VERSION, active_m=active_m, backend="hip-gfx950", tasks=tasks,
        events=[dict(id=t["id"], num_triggers=1, fires=[u["id"] for u in tasks if t["id"] in u["depends_on"]]) for t in tasks],
        scratch_buffers=scratch_buffers, initial_tasks=[t["id"] for t in tasks if not t["depends_on"]],
        model_params=[dict(path=s["source_path"], shape=s["shape"], dtype=s["dtype"]) for s in sym.values()
                      if s["role"] == "external" and not s.get("transform")],
        layer_groups=[dict(region=r, task_ids=ids) for r, ids in groups.items()],
        decode_pipeline=[t["id"] for t in tasks],
        decode_capabilities=dict(dispatchable=True, reasons=[]),
        uniforms=uniforms,
        model_config=dict(dataclasses.asdict(c), config_class=type(c).__name__))


def write_artifact(rt: DecoderRuntime, out_dir: str, model_name: str = "synthetic", prefill_variants=()) -> None:
    """`prefill_variants`: PrefillVariant objects of this runtime; each is written as
    `variants/prefill_mN/task_graph.json` and listed in the manifest (src/commands/patch.rs:112-150)."""
    if getattr(rt, "persistent", False):
        raise ValueError("write the artifact from a task-graph runtime (persistent=False)")
    os.makedirs(out_dir, exist_ok=True)
    sym = _symbols(rt)
    graph = _graph_dict(rt, rt.tasks, rt.graph, sym, 1,
                        dict(token="token", step_counter="step_counter", hist_counter="hist_counter", history="history"))
    with open(os.path.join(out_dir, "task_graph.json"), "w") as f:
        json.dump(graph, f, indent=1)
    tasks = graph["tasks"]
    variants = []
    for v in prefill_variants:
        vsym = dict(sym)
        for name, buf in v.scratch().items():
            u32 = name.rsplit(".", 1)[-1] in ("tokens", "offset", "kv_len")
            vsym[buf.ptr] = dict(role="scratch", role_name=name, dtype="uint32" if u32 else ("float32" if name.endswith(".ws") else "bfloat16"),
                                 size_bytes=buf.nbytes, zero=u32)
        vg = _graph_dict(rt, v.tasks, v.graph, vsym, v.m,
                         dict(token="token", tokens=v.name + ".tokens", offset=v.name + ".offset", kv_len=v.name + ".kv_len",
                              hist_counter="hist_counter", history="history"))
        vdir = os.path.join(out_dir, "variants", v.name)
        os.makedirs(vdir, exist_ok=True)
        with open(os.path.join(vdir, "task_graph.json"), "w") as f:
            json.dump(vg, f, indent=1)
        variants.append(dict(name=v.name, path="variants/" + v.name, active_m=v.m, tasks=len(vg["tasks"])))
    c = rt.cfg
    manifest = dict(
        schema_version=SCHEMA_VERSION, fusekit_version=BACKEND_VERSION,
        compiled_at=time.strftime("%Y-%m-%dT%H:%M:%SZ", time.gmtime()),
        model=dict(name=model_name, model_type="moe-decoder" if hasattr(c, "n_experts") else "dense-decoder",
                   hidden_size=c.hidden, num_hidden_layers=c.n_layers, num_kv_shared_layers=0, num_attention_heads=c.n_heads,
                   num_key_value_heads=getattr(c, "n_kv", c.n_heads), head_dim=getattr(c, "head_dim", None) or c.qk_dim,
                   vocab_size=c.vocab),
        stats=dict(ops=len(tasks), fusions=len(tasks), tasks=len(tasks),
                   unique_kernels=len({re.sub(r"_f\d+$", "", t["kernel"]) for t in tasks})),
        variants=variants)
    with open(os.path.join(out_dir, "manifest.json"), "w") as f:
        json.dump(manifest, f, indent=1)


class ArtifactRuntime:
    """A decode loop built from an artifact directory alone (plus the parameters it names)."""

    def __init__(self, art_dir: str, weights: DecoderWeights, dispatcher: Optional[Dispatcher] = None):
        manifest = json.load(open(os.path.join(art_dir, "manifest.json")))
        if manifest.get("schema_version") != SCHEMA_VERSION:
            raise ValueError(f"manifest schema {manifest.get('schema_version')} is not {SCHEMA_VERSION}")  # manifest.rs:108-112
        path = os.path.join(art_dir, "task_graph.json")
        graph = json.load(open(path))
        # the native loader validates version and kernel names before the device is used
        self.d = dispatcher or Dispatcher(None, path)
        self.scratch: Dict[str, DeviceBuffer] = {}
        for s in graph["scratch_buffers"]:
            self.scratch[s["role_name"]] = native.zeros(s["size_bytes"]) if s["zero_init"] else DeviceBuffer(s["size_bytes"])
        params: Dict[str, DeviceBuffer] = {}
        for p, W in weights.mats.items():
            params[p + ".weight"] = W.w
            if W.bits != 16:
                params[p + ".scales"], params[p + ".biases"] = W.scales, W.biases
        params.update(weights.vecs)
        self._params = params
        self.tasks = self._tasks_of(graph)
        u = graph["uniforms"]
        self.uniforms = make_uniforms(self.scratch[u["token"]], self.scratch[u["step_counter"]],
                                      self.scratch[u["hist_counter"]], self.scratch[u["history"]])
        self.graph = self.d.build_decode_graph(self.tasks, False)
        self.model_config = graph["model_config"]
        self._weights = weights  # keeps the parameter buffers alive
        # prefill_mN variants (manifest `variants`, one task graph each): scratch buffers are shared by role
        # name with the decode graph (KV caches, token, history, logits), the rest is the variant's own
        self.variants: Dict[int, dict] = {}
        for v in manifest.get("variants", []):
            if not str(v.get("name", "")).startswith("prefill_m"):
                continue
            vg = json.load(open(os.path.join(art_dir, v["path"], "task_graph.json")))
            if vg.get("version") != SCHEMA_VERSION or int(vg.get("active_m", 0)) != int(v["active_m"]):
                raise ValueError(f"variant {v['name']}: task graph does not match the manifest entry")
            for sb in vg["scratch_buffers"]:
                have = self.scratch.get(sb["role_name"])
                if have is None:
                    self.scratch[sb["role_name"]] = native.zeros(sb["size_bytes"]) if sb["zero_init"] else DeviceBuffer(sb["size_bytes"])
                elif have.nbytes < sb["size_bytes"]:
                    raise ValueError(f"variant {v['name']}: scratch {sb['role_name']} is larger than in the decode graph")
            vu = vg["uniforms"]
            self.variants[int(v["active_m"])] = dict(
                graph=self.d.build_decode_graph(self._tasks_of(vg), False), tokens=self.scratch[vu["tokens"]],
                offset=self.scratch[vu["offset"]], kv_len=self.scratch[vu["kv_len"]], token=self.scratch[vu["token"]])

    def _tasks_of(self, graph: dict) -> List[Dispatch]:
        out: List[Dispatch] = []
        for tid in graph["decode_pipeline"]:
            t = graph["tasks"][tid]
            slots = sorted(t["inputs"] + t["outputs"], key=lambda b: b["slot"])
            args = []
            for b in slots:
                if b["role"] == "external" and b.get("transform") == "xcd_kslice":
                    key = b["source_path"] + "@xcd_kslice"
                    if key not in self._params:   # [n, groups] -> [8][n][groups / 8], once per parameter
                        n, groups = b["shape"]
                        self._params[key] = native.xcd_kslice_meta(self._params[b["source_path"]], n, groups)
                    buf = self._params[key]
                elif b["role"] == "external" and b.get("transform"):
                    raise ValueError(f"task {tid} slot {b['slot']}: unknown parameter transform {b['transform']}")
                else:
                    buf = self._params[b["source_path"]] if b["role"] == "external" else self.scratch[b["role_name"]]
                off = int(b.get("offset_bytes", 0))
                if off + b["nbytes"] > buf.nbytes:
                    raise ValueError(f"task {tid} slot {b['slot']}: binding wants {off + b['nbytes']} bytes, buffer has {buf.nbytes}")
                args.append((buf.ptr + off, b["nbytes"]))
            out.append(Dispatch(t["kernel"], args, dict(t["params"])))
        return out

    def prefill(self, prompt) -> int:
        """Prompt processing: whole blocks of N tokens through the largest `prefill_mN` variant that fits
        what is left (the reference takes a variant when exactly N tokens are to be processed,
        python/fusekit_runtime/__init__.py:4866), the rest token by token through the decode graph."""
        from .prefill_variant import run_variant
        prompt = list(prompt)
        pos, nxt = 0, None
        cap = int(self.model_config["capacity"])
        while pos < len(prompt):
            fit = [m for m in self.variants if m <= len(prompt) - pos]
            if not fit:
                toks, _ = self.d.decode_host_loop(self.graph, self.uniforms, pos, prompt[pos:])
                return toks[-1]
            m = max(fit)
            v = self.variants[m]
            nxt = run_variant(self.d, v["graph"], m, v["tokens"], v["offset"], v["kv_len"], v["token"], prompt[pos:pos + m], pos, cap)
            pos += m
        return nxt

    def generate(self, prompt, max_tokens: int) -> List[int]:
        out = [self.prefill(prompt)]
        offset = len(prompt)
        while len(out) < max_tokens:
            n = min(64, max_tokens - len(out), self.uniforms.hist_capacity)
            toks, _ = self.d.decode_chunk(self.graph, self.uniforms, offset, out[-1], n)
            out += toks
            offset += n
        return out
