#!/usr/bin/env python3
"""Per-kernel measurements of the decode hot path on one MI355X.

    python -m fusekit_amd.kernel_bench [--case NAME ...] [--reps N]

Every case builds one hipGraph whose nodes run the same kernel over a pool of DISTINCT
operands larger than the 256 MB last-level cache, so each launch streams its bytes from HBM
("cold"); a second graph re-runs one operand set ("warm", cache resident where it fits).
Nodes are serialised (a barrier between each) so that the figure is the kernel's own
duration plus the ~1.6 us a dependent graph node costs; `parallel` lets the graph overlap
independent nodes instead.  GPU time comes from HIP events around whole graph launches on the
dispatcher's stream.  One JSON line per case; bytes are the ALGORITHMIC bytes of the call
(weights + scales + biases + activations in and out, KV rows read), peak is 8 TB/s.

Weights are random bits / random bf16 scales written straight into HBM: timing does not
depend on the values.
"""
import argparse
import json
import sys

from . import native as fk
from .decoder import _synth
from .runtime import Dispatch, Dispatcher, arg

HBM_PEAK = 8.0e12
MFMA_BF16_PEAK = 2.5e15


def _rand_weight(n, k, bits, seed, group=64, experts=1):
    """Random-valued weight of the right byte sizes (timing only)."""
    W = fk.DeviceWeight.__new__(fk.DeviceWeight)
    W.n, W.k, W.bits, W.group = n, k, bits, group
    words = experts * n * k * bits // 32
    W.w = fk.DeviceBuffer(words * 4)
    _synth(W.w, words, seed, 0.0, 0.0, 2, 0xFFFFFFFF)
    if bits == 16:
        W.scales = W.biases = None
        # random words may hold NaN/Inf bf16 patterns; fill with small normals instead
        _synth(W.w, words * 2, seed, 0.0, 0.02, 1)
    else:
        meta = experts * n * (k // group)
        W.scales, W.biases = fk.DeviceBuffer(meta * 2), fk.DeviceBuffer(meta * 2)
        _synth(W.scales, meta, seed + 1, 0.002, 0.0005, 1)
        _synth(W.biases, meta, seed + 2, -0.015, 0.004, 1)
    return W


def _bf16(count, seed, std=1.0):
    b = fk.DeviceBuffer(count * 2)
    _synth(b, count, seed, 0.0, std, 1)
    return b


def _wargs(W):
    return [arg(W.w)] + ([] if W.bits == 16 else [arg(W.scales), arg(W.biases)])


def _time_graph(d, tasks, reps, serial=True):
    g = d.build_graph(tasks, barriers=[serial] * len(tasks))
    d.execute_graph(g)                      # warm-up (first launch uploads the graph)
    sec = d.execute_graph(g, repeat=reps)
    return sec / (reps * len(tasks))


def _emit(case, per_call_s, nbytes, flops=None, **extra):
    out = {"case": case, "us_per_call": round(per_call_s * 1e6, 3), "bytes_per_call": int(nbytes),
           "GBps": round(nbytes / per_call_s / 1e9, 1), "frac_of_hbm_peak": round(nbytes / per_call_s / HBM_PEAK, 4)}
    if flops is not None:
        out["TFLOPs"] = round(flops / per_call_s / 1e12, 2)
        out["frac_of_mfma_bf16_peak"] = round(flops / per_call_s / MFMA_BF16_PEAK, 4)
    out.update(extra)
    print(json.dumps(out), flush=True)


def case_qgemv(d, reps, n, k, bits, pool, tag):
    per = bits / 8 + (0 if bits == 16 else 4 / 64)
    nbytes = n * k * per + k * 2 + n * 2
    Ws = [_rand_weight(n, k, bits, 100 + 3 * i) for i in range(pool)]
    x, ys = _bf16(k, 7), [fk.DeviceBuffer(n * 2) for _ in range(pool)]
    mk = lambda W, y: Dispatch("fusekit_qgemv_f0", [arg(x)] + _wargs(W) + [arg(y)], {"bits": bits, "group": 64, "m": k, "n": n})
    cold = [mk(W, y) for W, y in zip(Ws, ys)]
    warm = [mk(Ws[0], ys[i]) for i in range(min(pool, 64))]
    _emit(f"qgemv_{tag}_q{bits}_cold_serial", _time_graph(d, cold, reps), nbytes, n=n, k=k, pool=pool)
    _emit(f"qgemv_{tag}_q{bits}_cold_parallel", _time_graph(d, cold, reps, serial=False), nbytes, n=n, k=k, pool=pool)
    _emit(f"qgemv_{tag}_q{bits}_warm_serial", _time_graph(d, warm, reps), nbytes, n=n, k=k, pool=1)


def case_sdpa_quant(d, reps, length, bits):
    """Attention over a quantised KV cache (group 64): algorithmic bytes = packed codes + scales + biases."""
    import numpy as np
    n_heads, n_kv, dim, group = 32, 8, 128, 64
    rows = n_kv * length
    kv_bytes = 2 * rows * (dim * bits // 8 + (dim // group) * 4)
    pool = max(2, min(256, int(600e6 // kv_bytes) + 1))
    q, out = _bf16(n_heads * dim, 3), fk.DeviceBuffer(n_heads * dim * 2)
    kv_len = fk.DeviceBuffer.from_numpy(np.array([length], np.uint32))
    pb, cb = fk.sdpa_workspace_bytes(n_heads, n_kv, dim, dim, length)
    partials, counters = fk.DeviceBuffer(max(pb, 16)), fk.zeros(max(cb, 16))
    tasks, keep = [], []
    for i in range(pool):
        c = []
        for j in range(2):
            packed = fk.DeviceBuffer(rows * dim * bits // 8)
            _synth(packed, rows * dim * bits // 32, 100 + 2 * i + j, 0.0, 0.0, 2, 0xFFFFFFFF)
            sc, bi = fk.DeviceBuffer(rows * (dim // group) * 2), fk.DeviceBuffer(rows * (dim // group) * 2)
            _synth(sc, rows * (dim // group), 300 + 2 * i + j, 0.1 if bits == 4 else 0.008, 0.01, 1)
            _synth(bi, rows * (dim // group), 500 + 2 * i + j, -0.7, 0.2, 1)
            c += [packed, sc, bi]
        keep.append(c)
        tasks.append(Dispatch(f"fusekit_sdpa_decode_q{bits}_f0", [arg(q)] + [arg(b) for b in c] +
                              [arg(kv_len), arg(out), arg(partials), arg(counters)],
                              {"n_heads": n_heads, "n_kv": n_kv, "head_dim": dim, "capacity": length, "max_len": length,
                               "group": group}))
    nbytes = kv_bytes + 2 * n_heads * dim * 2
    _emit(f"sdpa_decode_q{bits}_L{length}_cold_serial", _time_graph(d, tasks, reps), nbytes,
          flops=4 * n_heads * length * dim, pool=pool)


def case_sdpa(d, reps, length):
    n_heads, n_kv, dim = 32, 8, 128
    kv_bytes = 2 * n_kv * length * dim * 2
    pool = max(2, min(256, int(600e6 // kv_bytes) + 1))
    q, out = _bf16(n_heads * dim, 3), fk.DeviceBuffer(n_heads * dim * 2)
    import numpy as np
    kv_len = fk.DeviceBuffer.from_numpy(np.array([length], np.uint32))
    pb, cb = fk.sdpa_workspace_bytes(n_heads, n_kv, dim, dim, length)
    partials, counters = fk.DeviceBuffer(max(pb, 16)), fk.zeros(max(cb, 16))
    tasks = []
    keep = []
    for i in range(pool):
        ck, cv = _bf16(n_kv * length * dim, 10 + 2 * i), _bf16(n_kv * length * dim, 11 + 2 * i)
        keep.append((ck, cv))
        tasks.append(Dispatch("fusekit_sdpa_decode_f0", [arg(q), arg(ck), arg(cv), arg(kv_len), arg(out), arg(partials),
                                                         arg(counters)],
                              {"n_heads": n_heads, "n_kv": n_kv, "head_dim": dim, "capacity": length, "max_len": length}))
    nbytes = kv_bytes + 2 * n_heads * dim * 2
    _emit(f"sdpa_decode_L{length}_cold_serial", _time_graph(d, tasks, reps), nbytes, flops=4 * n_heads * length * dim,
          pool=pool)
    _emit(f"sdpa_decode_L{length}_warm_serial", _time_graph(d, [tasks[0]] * 16, reps), nbytes,
          flops=4 * n_heads * length * dim, pool=1)


def case_sdpa_prefill(d, reps, rows, kv_len):
    """Causal attention of `rows` rows whose last one sits at position kv_len - 1 (one layer's worth)."""
    n_heads, n_kv, dim = 32, 8, 128
    kv_bytes = 2 * n_kv * kv_len * dim * 2
    pool = max(2, min(64, int(600e6 // kv_bytes) + 1))
    q, out = _bf16(rows * n_heads * dim, 3), fk.DeviceBuffer(rows * n_heads * dim * 2)
    tasks, keep = [], []
    for i in range(pool):
        ck, cv = _bf16(n_kv * kv_len * dim, 10 + 2 * i), _bf16(n_kv * kv_len * dim, 11 + 2 * i)
        keep.append((ck, cv))
        tasks.append(Dispatch("fusekit_sdpa_prefill_f0", [arg(q), arg(ck), arg(cv), arg(out)],
                              {"n_heads": n_heads, "n_kv": n_kv, "head_dim": dim, "capacity": kv_len, "rows": rows,
                               "kv_len": kv_len}))
    nbytes = kv_bytes + 2 * rows * n_heads * dim * 2
    # row r sees kv_len - rows + r + 1 positions: 4 flops per (head, position, dimension)
    seen = rows * (kv_len - rows) + rows * (rows + 1) // 2
    _emit(f"sdpa_prefill_rows{rows}_L{kv_len}", _time_graph(d, tasks, reps), nbytes, flops=4.0 * n_heads * seen * dim,
          pool=pool)


def case_moe(d, reps, bits=4, tokens=1):
    """Config 5 routed experts: `tokens` active rows, top-6 of 64 experts each (tokens = 8: up to 48 distinct experts)."""
    import numpy as np
    E, hidden, inter, top_k, layers = 64, 2048, 1408, 6, 2
    routes = tokens * top_k
    per = bits / 8 + 4 / 64
    rng = np.random.Generator(np.random.PCG64(5))
    x, res = _bf16(tokens * hidden, 1), _bf16(tokens * hidden, 2)
    row_idx = fk.DeviceBuffer.from_numpy(np.repeat(np.arange(tokens, dtype=np.uint32), top_k))  # route r reads its token's row
    h_rows = fk.DeviceBuffer.from_numpy(np.arange(routes, dtype=np.uint32))  # route r reads row r of the SwiGLU output
    m1, m2, o1, o2, keep = [], [], [], [], []
    for L in range(layers):
        Wg, Wu = _rand_weight(inter, hidden, bits, 300 + 10 * L, experts=E), _rand_weight(inter, hidden, bits, 303 + 10 * L, experts=E)
        Wd = _rand_weight(hidden, inter, bits, 306 + 10 * L, experts=E)
        keep.append((Wg, Wu, Wd))
    distinct = []
    for i in range(16):
        Wg, Wu, Wd = keep[i % layers]
        ids = np.concatenate([rng.permutation(E)[:top_k] for _ in range(tokens)]).astype(np.uint32)
        distinct.append(len(set(ids.tolist())))
        eidx = fk.DeviceBuffer.from_numpy(ids)
        rwt = _bf16(routes, 50 + i, 0.2)
        h, out = fk.DeviceBuffer(routes * inter * 2), fk.DeviceBuffer(tokens * hidden * 2)
        ws = fk.DeviceBuffer(fk.routed_reduce_workspace_bytes(tokens, top_k, hidden))
        keep.append((eidx, rwt, h, out, ws))
        m1.append(Dispatch("fusekit_routed_qmv_swiglu_f0",
                           [arg(x), arg(Wg.w), arg(Wg.scales), arg(Wg.biases), arg(Wu.w), arg(Wu.scales), arg(Wu.biases),
                            arg(row_idx), arg(eidx), arg(h)],
                           {"bits": bits, "k": hidden, "o": inter, "experts": E, "routes": routes, "x_rows": tokens}))
        m2.append(Dispatch("fusekit_routed_qmv_reduce_f0",
                           [arg(h), arg(Wd.w), arg(Wd.scales), arg(Wd.biases), arg(h_rows), arg(eidx), arg(rwt),
                            arg(res), arg(out), arg(ws)],
                           {"bits": bits, "k": inter, "o": hidden, "experts": E, "tokens": tokens, "top_k": top_k,
                            "x_rows": routes, "has_extra": 1}))
        if tokens > 1:   # the same launches with the routes served in expert order (fusekit_route_order)
            order = fk.zeros(4 * routes)
            fk.route_order(eidx, routes, E, order)
            keep.append(order)
            o1.append(Dispatch(m1[-1].kernel, list(m1[-1].args) + [arg(order)], dict(m1[-1].params, has_order=1)))
            o2.append(Dispatch(m2[-1].kernel, list(m2[-1].args) + [arg(order)], dict(m2[-1].params, has_order=1)))
    uniq = sum(distinct) / len(distinct)  # an expert chosen by several rows is streamed once per route here
    b1 = routes * 2 * inter * hidden * per + tokens * hidden * 2 + routes * inter * 2
    b2 = routes * hidden * inter * per + routes * inter * 2 + 2 * tokens * hidden * 2
    tag = f"cfg5_q{bits}" + (f"_rows{tokens}" if tokens > 1 else "")
    _emit(f"routed_qmv_swiglu_{tag}", _time_graph(d, m1, reps), b1, flops=2.0 * routes * 2 * inter * hidden, routes=routes,
          experts=E, distinct_experts=round(uniq, 1))
    _emit(f"routed_qmv_reduce_{tag}", _time_graph(d, m2, reps), b2, flops=2.0 * routes * inter * hidden, routes=routes, experts=E,
          note="three kernels: routed GEMV, ordered reduction")
    if o1:
        fk.sync()
        _emit(f"routed_qmv_swiglu_{tag}_expert_order", _time_graph(d, o1, reps), b1, routes=routes, experts=E,
              distinct_experts=round(uniq, 1), note="bytes as if every route streamed its slice")
        _emit(f"routed_qmv_reduce_{tag}_expert_order", _time_graph(d, o2, reps), b2, routes=routes, experts=E)


def measure_qgemm(d, reps, rows, n=9728, k=2560, bits=4):
    """Seconds per call of the family fusekit_qgemm on `rows` activation rows (a serialised graph over a pool of
    matrices larger than the last-level cache), the algorithmic bytes and flops of one call, the pool size."""
    per = bits / 8 + 4 / 64
    pool = max(2, int(600e6 // (n * k * per)) + 1)
    x = _bf16(rows * k, 1)
    ws_bytes = fk.qgemm_workspace_bytes(rows, n, k, 64)
    tasks, keep = [], []
    for i in range(pool):
        W, y, ws = _rand_weight(n, k, bits, 500 + 3 * i), fk.DeviceBuffer(rows * n * 2), fk.DeviceBuffer(ws_bytes)
        keep.append((W, y, ws))
        tasks.append(Dispatch("fusekit_qgemm_f0", [arg(x)] + _wargs(W) + [arg(y), arg(ws)],
                              {"bits": bits, "group": 64, "m": k, "n": n, "rows": rows}))
    nbytes = n * k * per + rows * k * 2 + rows * n * 2
    return _time_graph(d, tasks, reps), nbytes, 2.0 * rows * n * k, pool


def case_qgemm(d, reps, rows, n=9728, k=2560, bits=4):
    sec, nbytes, flops, pool = measure_qgemm(d, reps, rows, n, k, bits)
    _emit(f"qgemm_rows{rows}_{n}x{k}_q{bits}", sec, nbytes, flops=flops, pool=pool,
          note="2..10 rows: one shared-stream launch; 11..64 rows: MFMA main + split-k reduction; from 65 rows the "
               "LDS-tiled form (finished outputs at one k split)")


def case_qgemm_swiglu(d, reps, rows, hidden=2560, inter=9728, bits=4):
    """The gate / up pair with SwiGLU of the family fusekit_qgemm_swiglu on `rows` activation rows (from 65 rows one
    launch of the tile form); flops of both products."""
    per = bits / 8 + 4 / 64
    pool = max(2, int(600e6 // (2 * inter * hidden * per)) + 1)
    x = _bf16(rows * hidden, 1)
    ws_bytes = 2 * fk.qgemm_workspace_bytes(rows, inter, hidden, 64)
    tasks, keep = [], []
    for i in range(pool):
        Wg, Wu = _rand_weight(inter, hidden, bits, 700 + 5 * i), _rand_weight(inter, hidden, bits, 702 + 5 * i)
        y, ws = fk.DeviceBuffer(rows * inter * 2), fk.DeviceBuffer(ws_bytes)
        keep.append((Wg, Wu, y, ws))
        tasks.append(Dispatch("fusekit_qgemm_swiglu_f0", [arg(x), arg(Wg.w), arg(Wu.w), arg(Wg.scales), arg(Wu.scales),
                                                          arg(Wg.biases), arg(Wu.biases), arg(y), arg(ws)],
                              {"bits": bits, "group": 64, "hidden": hidden, "inter": inter, "rows": rows, "variant": 1}))
    nbytes = 2 * inter * hidden * per + rows * hidden * 2 + rows * inter * 2
    _emit(f"qgemm_swiglu_rows{rows}_{inter}x{hidden}_q{bits}", _time_graph(d, tasks, reps), nbytes, flops=4.0 * rows * inter * hidden,
          pool=pool)


def case_prefill(d, reps, prompt_len=512, rows_per_pass=4096, capacity=1024, kv_bits=0, keep=False):
    """Chunked prefill of the 4B-class model: `rows_per_pass` prompt tokens per pass over the weights."""
    import time
    import numpy as np
    from .decoder import DENSE_4B, DecoderConfig, DecoderRuntime, DecoderWeights
    cfg = DecoderConfig(**DENSE_4B, bits=4, capacity=capacity, swiglu_variant=1, kv_bits=kv_bits)
    W = DecoderWeights.random_init(cfg, seed=0)
    rt = DecoderRuntime(cfg, W, dispatcher=d)
    prompt = np.random.Generator(np.random.PCG64(0)).integers(0, cfg.vocab, prompt_len).tolist()
    rt.prefill_rows(prompt, rows_per_pass=rows_per_pass, keep_bf16_weights=keep)
    t0 = time.perf_counter()
    rt.prefill_rows(prompt, rows_per_pass=rows_per_pass, keep_bf16_weights=keep)
    rows_s = time.perf_counter() - t0
    t0 = time.perf_counter()
    rt.prefill(prompt[:64])
    single_s = (time.perf_counter() - t0) / 64 * prompt_len
    flops = 2.0 * prompt_len * (cfg.n_layers * (cfg.hidden * (cfg.n_q + 2 * cfg.n_kvd) + cfg.n_q * cfg.hidden + 3 * cfg.inter * cfg.hidden))
    print(json.dumps({"case": f"prefill_4b_q4_{prompt_len}_tokens" + (f"_kv{kv_bits}" if kv_bits else "") + ("_bf16_copy" if keep else ""), "rows_per_pass": rows_per_pass,
                      "prompt_tok_per_s": round(prompt_len / rows_s, 1), "ms": round(rows_s * 1e3, 2),
                      "token_by_token_tok_per_s": round(prompt_len / single_s, 1),
                      "TFLOPs": round(flops / rows_s / 1e12, 2)}), flush=True)


def case_moe_decode(d, reps, prompt_len=32, decode=512, xcd_moe=True):
    """Decode loop of the MoE benchmark model (27 layers, 64 experts top-6 + 2 shared, low-rank keys, int4):
    a 32-token prompt, then 512 greedy tokens from the captured graph; per-node times of one replay."""
    import numpy as np
    from .moe_decoder import MoeConfig, MoeRuntime, MoeWeights
    cfg = MoeConfig(capacity=1024, xcd_moe=xcd_moe)
    W = MoeWeights.random_init(cfg, seed=0)
    rt = MoeRuntime(cfg, W, dispatcher=d)
    prompt = np.random.Generator(np.random.PCG64(0)).integers(0, cfg.vocab, prompt_len).tolist()
    rt.generate(prompt, 9)
    toks, gpu_s, steps = rt.generate(prompt, decode + 1)
    ctx = prompt_len + decode // 2
    roof = 8e12 / cfg.token_bytes(ctx)
    per_node = rt.d.profile_graph_nodes(rt.graph)
    kinds = {}
    for t, sec in zip(rt.tasks, per_node):
        k = t.kernel.rsplit("_f", 1)[0].replace("fusekit_", "")
        kinds[k] = kinds.get(k, 0.0) + sec * 1e6
    print(json.dumps({"case": "moe_cfg5_decode_q4" + ("" if xcd_moe else "_per_dispatch"), "tok_per_s": round(steps / gpu_s, 1), "ms_per_token": round(gpu_s / steps * 1e3, 3),
                      "graph_nodes": len(rt.tasks), "token_MB": round(cfg.token_bytes(ctx) / 1e6, 1),
                      "roofline_tok_per_s": round(roof, 1), "frac": round(steps / gpu_s / roof, 4),
                      "weights_GB": round(W.nbytes() / 1e9, 2),
                      "us_by_family_serialised": {k: round(v, 1) for k, v in sorted(kinds.items(), key=lambda kv: -kv[1])}}),
          flush=True)


def case_moe_rows(d, reps, rows=8, offset=32):
    """`rows` active token rows of the MoE benchmark model in one pass over the weights (direct calls)."""
    import time
    import numpy as np
    from .moe_decoder import MoeConfig, MoeRuntime, MoeWeights
    cfg = MoeConfig(capacity=1024)
    W = MoeWeights.random_init(cfg, seed=0)
    rt = MoeRuntime(cfg, W, dispatcher=d)
    toks = np.random.Generator(np.random.PCG64(0)).integers(0, cfg.vocab, offset + rows).tolist()
    rt.prefill(toks[:offset])
    rt.forward_rows(toks[offset:], offset)
    n = 5
    t0 = time.perf_counter()
    for _ in range(n):
        rt.forward_rows(toks[offset:], offset)
    sec = (time.perf_counter() - t0) / n
    print(json.dumps({"case": f"moe_cfg5_rows{rows}_pass_q4", "rows": rows, "ms_per_pass": round(sec * 1e3, 3),
                      "rows_per_s": round(rows / sec, 1), "note": "one graph replay per pass, wall clock"}), flush=True)


def case_dense_rows(d, reps, rows=8, offset=32):
    """`rows` active token rows of the 4B-class dense model (int4) in one pass: its prefill_m<rows> variant."""
    import time
    from .decoder import DENSE_4B, DecoderConfig, DecoderRuntime, DecoderWeights
    from .prefill_variant import PrefillVariant
    cfg = DecoderConfig(**DENSE_4B, bits=4, capacity=1024)
    rt = DecoderRuntime(cfg, DecoderWeights.random_init(cfg, seed=0), dispatcher=d)
    v = PrefillVariant(rt, rows)
    rt.prefill(list(range(200, 200 + offset)))
    toks = list(range(100, 100 + rows))
    v.run(toks, offset)
    n = 10
    t0 = time.perf_counter()
    for _ in range(n):
        v.run(toks, offset)
    sec = (time.perf_counter() - t0) / n
    print(json.dumps({"case": f"dense4b_rows{rows}_pass_q4", "rows": rows, "ms_per_pass": round(sec * 1e3, 3), "launches": len(v.tasks),
                      "rows_per_s": round(rows / sec, 1), "note": "one graph replay per pass, wall clock"}), flush=True)


CASES = {
    "dense4b_rows8_pass": lambda d, r: case_dense_rows(d, r, 8),
    "moe_cfg5_rows8_pass": lambda d, r: case_moe_rows(d, r, 8),
    "moe_cfg5_rows64_pass": lambda d, r: case_moe_rows(d, r, 64),
    "moe_cfg5_decode": lambda d, r: case_moe_decode(d, r),
    "moe_cfg5_decode_per_dispatch": lambda d, r: case_moe_decode(d, r, xcd_moe=False),
    "qgemv_cfg1": lambda d, r: case_qgemv(d, r, 4864, 896, 4, 512, "cfg1_4864x896"),
    "qgemv_big_q4": lambda d, r: case_qgemv(d, r, 9728, 2560, 4, 48, "9728x2560"),
    "qgemv_big_q8": lambda d, r: case_qgemv(d, r, 9728, 2560, 8, 28, "9728x2560"),
    "qgemv_big_bf16": lambda d, r: case_qgemv(d, r, 9728, 2560, 16, 14, "9728x2560"),
    # Vocabulary-sized matrices: hundreds of MB per launch, so the start-up chain of a launch is
    # amortised and the figure is the kernel's steady streaming rate.
    "qgemv_vocab_q4": lambda d, r: case_qgemv(d, r, 151936, 2560, 4, 3, "151936x2560"),
    "qgemv_vocab_q8": lambda d, r: case_qgemv(d, r, 151936, 2560, 8, 2, "151936x2560"),
    "qgemv_wide_q4": lambda d, r: case_qgemv(d, r, 65536, 8192, 4, 2, "65536x8192"),
    "sdpa_512": lambda d, r: case_sdpa(d, r, 512),
    "sdpa_4096": lambda d, r: case_sdpa(d, r, 4096),
    "sdpa_32768": lambda d, r: case_sdpa(d, r, 32768),
    "sdpa_q4_4096": lambda d, r: case_sdpa_quant(d, r, 4096, 4),
    "sdpa_q8_4096": lambda d, r: case_sdpa_quant(d, r, 4096, 8),
    "sdpa_q4_32768": lambda d, r: case_sdpa_quant(d, r, 32768, 4),
    "sdpa_q8_32768": lambda d, r: case_sdpa_quant(d, r, 32768, 8),
    "sdpa_prefill_128": lambda d, r: case_sdpa_prefill(d, r, 128, 128),
    "sdpa_prefill_512": lambda d, r: case_sdpa_prefill(d, r, 128, 512),
    "sdpa_prefill_4096": lambda d, r: case_sdpa_prefill(d, r, 128, 4096),
    "sdpa_prefill_32768": lambda d, r: case_sdpa_prefill(d, r, 128, 32768),
    "sdpa_prefill_r32_4096": lambda d, r: case_sdpa_prefill(d, r, 32, 4096),
    "sdpa_prefill_r512_512": lambda d, r: case_sdpa_prefill(d, r, 512, 512),
    "sdpa_prefill_r512_4096": lambda d, r: case_sdpa_prefill(d, r, 512, 4096),
    "moe_cfg5": lambda d, r: case_moe(d, r),
    "moe_cfg5_rows8": lambda d, r: case_moe(d, r, tokens=8),
    "qgemm_8": lambda d, r: case_qgemm(d, r, 8),
    "qgemm_32": lambda d, r: case_qgemm(d, r, 32),
    "qgemm_128": lambda d, r: case_qgemm(d, r, 128),
    "qgemm_512": lambda d, r: case_qgemm(d, r, 512),
    "qgemm_2048": lambda d, r: case_qgemm(d, r, 2048),
    "qgemm_swiglu_512": lambda d, r: case_qgemm_swiglu(d, r, 512),
    "qgemm_swiglu_2048": lambda d, r: case_qgemm_swiglu(d, r, 2048),
    "prefill_4b_32": lambda d, r: case_prefill(d, r, 512, 32),
    "prefill_4b": lambda d, r: case_prefill(d, r),
    "prefill_4b_128": lambda d, r: case_prefill(d, r, 512, 128),
    "prefill_4b_256": lambda d, r: case_prefill(d, r, 512, 256),
    "prefill_4b_4096_tokens": lambda d, r: case_prefill(d, r, 4096, 512, 4608),
    "prefill_4b_4096_tokens_1024": lambda d, r: case_prefill(d, r, 4096, 1024, 4608),
    "prefill_4b_4096_tokens_4096": lambda d, r: case_prefill(d, r, 4096, 4096, 4608),
    "prefill_4b_4096_tokens_bf16_copy": lambda d, r: case_prefill(d, r, 4096, 4096, 4608, keep=True),
    "prefill_4b_512_tokens_bf16_copy": lambda d, r: case_prefill(d, r, 512, 512, 1024, keep=True),
    "prefill_4b_4096_tokens_kv4": lambda d, r: case_prefill(d, r, 4096, 4096, 4608, kv_bits=4),
}


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--case", action="append", choices=sorted(CASES), help="default: all")
    ap.add_argument("--reps", type=int, default=20)
    args = ap.parse_args()
    d = Dispatcher()
    for name in (args.case or list(CASES)):
        print(f"[kernel_bench] {name}", file=sys.stderr, flush=True)
        CASES[name](d, args.reps)
        fk.sync()
    return 0


if __name__ == "__main__":
    sys.exit(main())
