#!/usr/bin/env python3
"""Headline benchmark: hipGraph-replayed batch-1 greedy decode of the 4B-class dense model
(configs[3]: 36 layers, hidden 2560, 4-bit g64 MLX-affine weights) at context 512, on one MI355X.

One "step" = one decoded token = one replay of the captured decode graph: step_init, embedding, 36 x
[attention launch | MLP launch] (the XCD-resident layer: RMSNorm + q/k/v + head norm + RoPE + cache append +
attention + o_proj, then RMSNorm + gate/up + SwiGLU + down_proj, residuals folded into the next launch's
input), the last layer's reduction, final norm + LM head, argmax.  Weights are random-init (seeded,
generated and quantised in HBM); everything is resident before the timed region.

The K timed steps always sit around context 512: after the 32-token prompt the script decodes
untimed (at least --warmup steps) until the cache holds 512 - K/2 positions, then times exactly K
steps, so the window is [512 - K/2, 512 + K/2] whatever K is (K <= 960).

Prints ONE JSON line: value = generated tokens/s (wall clock around the K timed steps), plus
  roofline     -- the kernel symbol that holds the largest share of a token's GPU time: algorithmic
                  bytes of its launches / their summed average durations, measured here with HIP
                  events on the launch stream over serialised graphs of the 36 layers' own nodes
                  (distinct weights, 2 GB in all: nothing stays in a cache); `by_launch` lists every
                  launch shape of the token the same way,
  qgemv_cfg1   -- configs[0]/[1]'s int4 qGEMV (4864 x 896, g64) over a rotating pool of 512 weight
                  sets (1.26 GB), GB/s and fraction of the 8 TB/s peak,
  qgemv_steady -- the same kernel family on a vocabulary-sized int4 matrix (151936 x 2560, 219 MB per
                  launch, three sets in rotation): the steady streaming rate of the int4 qGEMV,
  hbm_read_ceiling -- a plain read-and-XOR kernel over 1 GiB buffers: what a read-only kernel gets from
                  HBM on this device, the bound the GEMV figures are also stated against,
  qgemm_rows   -- the multi-row matmul of the prompt path (9728 x 2560 int4 as a graph node, 512 and 2048
                  activation rows): TFLOP/s and fraction of the dense bf16 MFMA peak,
  moe_cfg5_decode -- configs[4]'s mixture-of-experts decoder: tokens/s of its decode loop,
  cpu_baseline -- the CPU oracle (C restatement of the reference semantics) decoding the same
                  model at the same context on the host cores, bounded to --cpu-tokens steps.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0  # MI355X HBM3E published peak
CONTEXT = 512

# task family -> (HIP kernel symbol as rocprofv3 prints it, short label)
SYMBOLS = {
    "rmsnorm_qkv": "gemv_stream_kernel<Q4, 1 segment>",
    "linear_residual": "gemv_stream_kernel<Q4, 1 segment>",
    "rmsnorm_gateup_swiglu": "gemv_stream_kernel<Q4, gate/up pair>",
    "rope_store_sdpa_decode": "sdpa_rope_store_kernel",
    "xcd_attn_block": "xcd_attn_kernel<Q4>",
    "xcd_mlp_block": "xcd_mlp_kernel<Q4>",
    "xcd_reduce": "xcd_reduce_kernel",
    "final_rmsnorm_lm_head": "gemv_rows_kernel<BF16, batches of 5 column blocks>",
    "final_rmsnorm_lm_head_argmax": "gemv_rows_kernel<BF16, batches of 5 column blocks, greedy token>",
    "argmax_logits_decode": "argmax_kernel",
    "embed_lookup_decode": "embed_lookup_kernel",
    "step_init": "step_init_kernel",
}


def family(kernel: str) -> str:
    name = kernel[len("fusekit_"):] if kernel.startswith("fusekit_") else kernel
    return name.rsplit("_f", 1)[0] if "_f" in name else name


# HBM bytes per launch from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE (each scaled by what the counter reads for a plain
# 256 MiB copy); the runs and their commands are kept in profiles/xcd_layer_q4_4b.pmc_traffic.md.  Counters cannot be
# read inside this process, so the figure is the recorded one for the kernel as built there.
TRAFFIC_BYTES = {"xcd_mlp_kernel<Q4>": 44944500, "xcd_attn_kernel<Q4>": 18298100}  # the latter at context 505..520


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=512)
    ap.add_argument("--warmup", type=int, default=32)
    ap.add_argument("--bits", type=int, default=4, choices=[4, 8, 16])
    ap.add_argument("--prompt", type=int, default=32)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-kernels", action="store_true", help="skip the per-launch measurements (roofline, qgemv_cfg1)")
    ap.add_argument("--cpu-tokens", type=int, default=48,
                    help="decode steps the CPU oracle runs for cpu_baseline (10-30 s on the box's cores)")
    ap.add_argument("--per-kernel", action="store_true", help="print per-family GPU time of one token to stderr")
    ap.add_argument("--layers", type=int, default=0, help="experiment only: override the layer count (not the headline config)")
    ap.add_argument("--sync-steps", action="store_true",
                    help="counter runs: one synchronised graph launch per token instead of chunks of queued launches "
                         "(a profiler that rewrites every dispatch packet needs the queue kept short); the rate "
                         "printed is then not the headline figure")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run 4 plain 256 MiB device copies (outside the timed region): the known-traffic "
                         "kernel that rocprofv3 byte counters of the same run are scaled by")
    ap.add_argument("--layer-launch", action="store_true",
                    help="a layer's attention and MLP launches as ONE launch with a device-wide barrier between the phases")
    ap.add_argument("--five-launches", action="store_true",
                    help="experiment only: the per-dispatch task list (five launches per layer) instead of the two-launch layer")
    ap.add_argument("--mode", choices=["persistent", "graph"], default="graph",
                    help="persistent: one whole-token kernel per replay; graph: one kernel node per task")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on ONE GPU; the decode path has no multi-GPU mode (--gpus must be 1)",
              file=sys.stderr)
        return 2

    import numpy as np

    import fusekit_amd.native as fk
    from fusekit_amd.decoder import DENSE_4B, DecoderConfig, DecoderRuntime, DecoderWeights
    from fusekit_amd.runtime import Dispatch, arg

    props = fk.device_props()
    start = max(args.prompt + args.warmup, CONTEXT - args.steps // 2)   # context of the first timed step
    total = start + args.steps
    capacity = max(1024, 1 << (total - 1).bit_length())
    cfg = DecoderConfig(**DENSE_4B, bits=args.bits, capacity=capacity, xcd_layers=not args.five_launches,
                        xcd_layer_launch=args.layer_launch)
    if args.layers:
        cfg.n_layers = args.layers
    t0 = time.time()
    W = DecoderWeights.random_init(cfg, seed=0)
    rt = DecoderRuntime(cfg, W, hist_capacity=max(4096, total),
                        persistent=(args.mode == "persistent"))
    setup_s = time.time() - t0

    if args.calibrate_copy:
        src, dst = fk.DeviceBuffer(256 << 20), fk.DeviceBuffer(256 << 20)
        fk.fill_u32(src, 0x3f803f80, (256 << 20) // 4)
        for _ in range(4):
            fk.copy(dst, src, 256 << 20)
        fk.sync()
        del src, dst

    rng = np.random.Generator(np.random.PCG64(0))
    prompt = rng.integers(0, cfg.vocab, args.prompt).tolist()
    first = rt.prefill(prompt)
    offset = len(prompt)
    tok = first
    # untimed: decode until the cache holds `start` positions (>= W steps; this is the warm-up)
    def chunk(offset, tok, n):
        if not args.sync_steps:
            return rt.d.decode_chunk(rt.graph, rt.uniforms, offset, tok, n)
        out, sec = [], 0.0
        for i in range(n):
            nxt, s1 = rt.d.decode_host_loop(rt.graph, rt.uniforms, offset + i, [tok])
            tok = nxt[0]
            out.append(tok)
            sec += s1
        return out, sec

    while offset < start:
        n = min(64, start - offset)
        toks, _ = chunk(offset, tok, n)
        tok, offset = toks[-1], offset + n
    fk.sync()
    # timed: exactly K steps, all chunks enqueued by the native loop, sync on both sides
    gpu_s = 0.0
    t0 = time.perf_counter()
    done = 0
    while done < args.steps:
        n = min(rt.uniforms.hist_capacity, args.steps - done)
        toks, sec = chunk(offset, tok, n)
        tok, offset, done, gpu_s = toks[-1], offset + n, done + n, gpu_s + sec
    fk.sync()
    wall_s = time.perf_counter() - t0
    tok_s = args.steps / wall_s
    ctx_mid = start + args.steps // 2
    bytes_per_token = cfg.token_bytes(ctx_mid)
    roofline_tok_s = HBM_PEAK_GBPS * 1e9 / bytes_per_token

    out = {
        "metric": "decode tok/s, 4B-class %d-bit @ L=%d (int4 qGEMV HBM GB/s in qgemv_cfg1 and roofline)" % (cfg.bits, ctx_mid),
        "value": round(tok_s, 2),
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(wall_s / args.steps * 1e3, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16 activations, int%d g64 weights, fp32 accumulate" % cfg.bits if cfg.bits != 16 else "bf16",
        "data": "synthetic (seeded random-init weights and prompt)",
        "config": {
            "workload": "configs[3]: 36-layer dense decoder, hidden 2560, inter 9728, 32q/8kv heads x128, vocab 151936 "
                        "tied bf16 head, %d-token prompt, greedy decode, one hipGraph per token" % args.prompt,
            "weights": "%d-bit g%d MLX-affine" % (cfg.bits, cfg.group) if cfg.bits != 16 else "bf16",
            "context": ctx_mid,
            "context_range": [start, start + args.steps],
            "untimed_steps_before": start - args.prompt,
            "graph_nodes": len(rt.tasks),
        },
        "gpu_ms_per_step": round(gpu_s / args.steps * 1e3, 4),
        "bytes_per_token": bytes_per_token,
        "weight_streaming_roofline_tok_s": round(roofline_tok_s, 1),
        "frac_of_roofline_tok_s": round(tok_s / roofline_tok_s, 4),
        "device": props.name.decode().strip() or props.arch.decode(),
        "setup_s": round(setup_s, 1),
    }

    # ---- per launch shape: serialised graphs of the token's own nodes, HIP events on the dispatcher's stream ----
    if not args.no_kernels and args.mode == "graph":
        # the attention launches read kv_len from the device: hold the measurement at context 512
        rt.kv_len.upload(np.array([CONTEXT], np.uint32))
        rt.offset.upload(np.array([CONTEXT - 1], np.uint32))
        rt.step_counter.upload(np.array([CONTEXT - 1], np.uint32))
        kv_row_bytes = 2 * cfg.n_kv * cfg.head_dim * 2
        groups = {}   # (family, position of the launch among its family inside a layer) -> tasks
        seen = {}
        for t in rt.tasks:
            fam = family(t.kernel)
            if fam in ("step_init",):
                continue
            idx = seen.get(fam, 0)
            seen[fam] = idx + 1
            per_layer = 2 if fam == "linear_residual" else 1
            groups.setdefault((fam, idx % per_layer), []).append(t)
        by_launch, by_symbol = [], {}
        cache_bytes = cfg.n_kv * cfg.capacity * cfg.head_dim * 2
        for (fam, pos), tasks in groups.items():
            if fam == "rope_store_sdpa_decode" or fam.startswith("sdpa_decode"):
                nbytes = kv_row_bytes * CONTEXT + 2 * (cfg.n_q * 2)          # K/V rows read + q in, out
                label = "rope/store + attention @%d" % CONTEXT
            elif fam == "xcd_attn_block":
                # q/k/v/o weights + vectors + partial rows, and the K/V rows of the context instead of the whole caches
                nbytes = sum(n for _, n in tasks[0].args if n != cache_bytes) + kv_row_bytes * CONTEXT
                label = "attention launch (norm, q/k/v, rope, append, attention @%d, o_proj)" % CONTEXT
            elif fam == "xcd_mlp_block":
                nbytes = sum(n for _, n in tasks[0].args)
                label = "MLP launch (norm, gate/up, SwiGLU, down_proj)"
            elif fam == "embed_lookup_decode":
                nbytes = 4 + 2 * cfg.hidden * 2                               # the token, one table row in, one row out
                label = fam
            else:
                nbytes = sum(n for _, n in tasks[0].args)                    # weights + scales + biases + vectors in/out
                label = {("linear_residual", 0): "o_proj + residual", ("linear_residual", 1): "down_proj + residual"}.get(
                    (fam, pos), fam)
            # a launch that occurs once per token is chained 32 times, so that the cost of starting a graph is not
            # charged to one small kernel
            chain = tasks if len(tasks) > 1 else tasks * 32
            reps = max(2, 720 // len(chain))
            g = rt.d.build_graph(chain, barriers=[True] * len(chain))
            rt.d.execute_graph(g)
            us = rt.d.execute_graph(g, repeat=reps) / (reps * len(chain)) * 1e6
            sym = SYMBOLS.get(fam, fam)
            e = {"launch": label, "kernel": sym, "per_token": len(tasks), "bytes_per_launch": int(nbytes),
                 "avg_launch_us": round(us, 3), "GBps": round(nbytes / us / 1e3, 1),
                 "frac": round(nbytes / us / 1e3 / HBM_PEAK_GBPS, 4)}
            by_launch.append(e)
            s = by_symbol.setdefault(sym, {"us": 0.0, "bytes": 0, "launches": 0})
            s["us"] += us * len(tasks)
            s["bytes"] += nbytes * len(tasks)
            s["launches"] += len(tasks)
        dom = max(by_symbol, key=lambda k: by_symbol[k]["us"])
        s = by_symbol[dom]
        achieved = s["bytes"] / s["us"] / 1e3
        out["roofline"] = {
            "kernel": dom,
            "bound": "hbm",
            "achieved": round(achieved, 1),
            "peak": HBM_PEAK_GBPS,
            "unit": "GB/s",
            "frac": round(achieved / HBM_PEAK_GBPS, 4),
            "traffic": TRAFFIC_BYTES.get(dom),
            "bytes_per_launch": int(s["bytes"] / s["launches"]),
            "avg_launch_us": round(s["us"] / s["launches"], 3),
            "launches_per_token": s["launches"],
            "share_of_token_gpu_time": round(s["us"] / sum(v["us"] for v in by_symbol.values()), 4),
            "by_launch": sorted(by_launch, key=lambda e: -e["avg_launch_us"] * e["per_token"]),
        }
        if args.per_kernel:
            for e in out["roofline"]["by_launch"]:
                print("[bench:launch] %-34s x%-3d %8.2f us  %7.1f GB/s  %.3f of peak" % (
                    e["launch"], e["per_token"], e["avg_launch_us"], e["GBps"], e["frac"]), file=sys.stderr)

        # ---- configs[0]/[1]: the single int4 qGEMV 4864 x 896 over a rotating pool of 512 weight sets ----
        if cfg.bits == 4:
            from fusekit_amd.kernel_bench import _bf16, _rand_weight, _wargs
            n, k, pool = 4864, 896, 512
            nbytes = int(n * k * 0.5625) + k * 2 + n * 2
            Ws = [_rand_weight(n, k, 4, 100 + 3 * i) for i in range(pool)]
            x, ys = _bf16(k, 7), [fk.DeviceBuffer(n * 2) for _ in range(pool)]
            tasks = [Dispatch("fusekit_qgemv_f0", [arg(x)] + _wargs(Wi) + [arg(y)], {"bits": 4, "group": 64, "m": k, "n": n})
                     for Wi, y in zip(Ws, ys)]
            res = {}
            for name, serial in (("serial", True), ("overlapped", False)):
                g = rt.d.build_graph(tasks, barriers=[serial] * pool)
                rt.d.execute_graph(g)
                us = rt.d.execute_graph(g, repeat=4) / (4 * pool) * 1e6
                res[name] = us
            out["qgemv_cfg1"] = {
                "shape": "4864 x 896 int4 g64, bf16 x and y", "pool": pool, "bytes_per_launch": nbytes,
                "serial_us": round(res["serial"], 3), "serial_GBps": round(nbytes / res["serial"] / 1e3, 1),
                "serial_frac": round(nbytes / res["serial"] / 1e3 / HBM_PEAK_GBPS, 4),
                "overlapped_us": round(res["overlapped"], 3), "overlapped_GBps": round(nbytes / res["overlapped"] / 1e3, 1),
                "overlapped_frac": round(nbytes / res["overlapped"] / 1e3 / HBM_PEAK_GBPS, 4),
                "note": "serial: dependent graph nodes, launch to launch; overlapped: independent nodes of one graph",
            }
            del Ws, ys, tasks

            # ---- the same kernel family at steady state: a vocabulary-sized int4 matrix (151936 x 2560, 219 MB per
            # launch), three weight sets in rotation (657 MB: past the 256 MB last-level cache), dependent graph
            # nodes, launch to launch; median and best of nine graph executions ----
            n, k, pool, rounds = 151936, 2560, 3, 8
            nbytes = int(n * k * 0.5625) + k * 2 + n * 2
            Ws = [_rand_weight(n, k, 4, 900 + 3 * i) for i in range(pool)]
            x, ys = _bf16(k, 8), [fk.DeviceBuffer(n * 2) for _ in range(pool)]
            tasks = [Dispatch("fusekit_qgemv_f0", [arg(x)] + _wargs(Wi) + [arg(y)], {"bits": 4, "group": 64, "m": k, "n": n})
                     for Wi, y in zip(Ws, ys)] * rounds
            g = rt.d.build_graph(tasks, barriers=[True] * len(tasks))
            rt.d.execute_graph(g)
            runs = sorted(rt.d.execute_graph(g) / len(tasks) * 1e6 for _ in range(9))
            med, best = runs[len(runs) // 2], runs[0]
            out["qgemv_steady"] = {
                "shape": "151936 x 2560 int4 g64, bf16 x and y", "pool": pool, "bytes_per_launch": nbytes,
                "median_us": round(med, 2), "median_GBps": round(nbytes / med / 1e3, 1),
                "median_frac": round(nbytes / med / 1e3 / HBM_PEAK_GBPS, 4),
                "best_us": round(best, 2), "best_frac": round(nbytes / best / 1e3 / HBM_PEAK_GBPS, 4),
                "note": "gemv_rows_kernel<Q4>; dependent graph nodes, launch to launch, %d launches per graph execution" % len(tasks),
            }
            del Ws, ys, tasks

        # ---- what a plain read-only kernel gets from HBM on this device: 16 bytes per lane, 1 KiB contiguous per wave
        # instruction, eight requests in flight per lane, XOR only; two 1 GiB buffers in rotation ----
        gib = 1 << 30
        bufs = [fk.DeviceBuffer(gib) for _ in range(2)]
        for i, b in enumerate(bufs):
            fk.fill_u32(b, 0x3f803f80 + i, gib // 4)
        sink = fk.DeviceBuffer(fk.read_reduce_out_bytes())
        tasks = [Dispatch("fusekit_read_reduce_f0", [arg(b), arg(sink)], {}) for b in bufs] * 4
        g = rt.d.build_graph(tasks, barriers=[True] * len(tasks))
        rt.d.execute_graph(g)
        runs = sorted(rt.d.execute_graph(g) / len(tasks) * 1e6 for _ in range(5))
        med = runs[len(runs) // 2]
        out["hbm_read_ceiling"] = {
            "kernel": "read_reduce_kernel (plain 16-byte loads, XOR)", "bytes_per_launch": gib,
            "median_us": round(med, 2), "GBps": round(gib / med / 1e3, 1), "frac_of_published_peak": round(gib / med / 1e3 / HBM_PEAK_GBPS, 4),
            "best_us": round(runs[0], 2),
        }
        if "qgemv_steady" in out:
            out["qgemv_steady"]["median_frac_of_read_ceiling"] = round(out["qgemv_steady"]["median_GBps"] / out["hbm_read_ceiling"]["GBps"], 4)
        del bufs

        # ---- the multi-row matmul on the matrix cores (the prompt path's projection: 9728 x 2560 int4 g64 as a graph
        # node, 512 and 2048 activation rows), against the dense bf16 MFMA peak ----
        from fusekit_amd.kernel_bench import measure_qgemm
        out["qgemm_rows"] = {}
        for rows in (512, 2048):
            q_s, _, q_flops, _ = measure_qgemm(rt.d, 20, rows)
            out["qgemm_rows"][str(rows)] = {"us_per_call": round(q_s * 1e6, 2), "TFLOPs": round(q_flops / q_s / 1e12, 1),
                                            "frac_of_mfma_bf16_peak": round(q_flops / q_s / 2.5e15, 4)}
        out["qgemm_rows"]["workload"] = "family fusekit_qgemm, 9728 x 2560 int4 g64, 512 / 2048 activation rows, peak 2.5 PFLOP/s"

        # ---- the mixture-of-experts benchmark model (BASELINE configs[4]: 27 layers, hidden 2048, 64 experts of 1408
        # top-6 + 2 shared, low-rank keys 16 heads x 192 / 128, vocab 102400, int4 g64; 9 GB of weights): 32-token
        # prompt, 512 greedy tokens at context 32..544, one hipGraph replay per token (two launches per layer) ----
        from fusekit_amd.moe_decoder import MoeConfig, MoeRuntime, MoeWeights
        mcfg = MoeConfig(capacity=1024)
        mW = MoeWeights.random_init(mcfg, seed=0)
        mrt = MoeRuntime(mcfg, mW)
        mprompt = np.random.Generator(np.random.PCG64(0)).integers(0, mcfg.vocab, 32).tolist()
        mrt.generate(mprompt, 9)
        mrt.reset()
        _, m_s, m_steps = mrt.generate(mprompt, 513)
        m_bytes = mcfg.token_bytes(32 + 256)
        out["moe_cfg5_decode"] = {
            "workload": "configs[4]: 27-layer mixture-of-experts decoder, 64 experts top-6 + 2 shared, int4 g64, context 32..544",
            "tok_per_s": round(m_steps / m_s, 1), "ms_per_token": round(m_s / m_steps * 1e3, 4), "graph_nodes": len(mrt.tasks),
            "launches_per_expert_layer": 2 if mrt.xcd_attn else (5 if mrt.xcd else 7),
            "bytes_per_token": m_bytes, "weight_streaming_roofline_tok_s": round(HBM_PEAK_GBPS * 1e9 / m_bytes, 1),
            "frac_of_roofline_tok_s": round(m_steps / m_s / (HBM_PEAK_GBPS * 1e9 / m_bytes), 4),
        }
        del mrt, mW

    if args.per_kernel and args.mode == "persistent":
        per_kernel = {}
        tr = rt.d.graph_phase_trace(rt.graph)
        names = ["embed"] + ["qkv", "attention", "o_proj", "gateup", "down"] * cfg.n_layers + ["lm_head", "argmax_scan", "argmax_final"]
        for nm, s_ in zip(names, tr):
            per_kernel[nm] = per_kernel.get(nm, 0.0) + s_
        print("[bench:per-phase] " + " ".join(f"{k}={v * 1e3:.3f}ms" for k, v in per_kernel.items()), file=sys.stderr)

    if not args.no_cpu_baseline:
        sys.path.insert(0, os.path.join(ROOT, "tests"))
        import oracle
        from helpers import OracleDecoder
        od = OracleDecoder(cfg, W)
        threads = oracle.num_threads()
        od.step(prompt[0], CONTEXT - 1)                    # untimed: pages the weights in
        t0 = time.perf_counter()
        t = prompt[0]
        for i in range(args.cpu_tokens):
            t, _, _ = od.step(t, CONTEXT + i)
        cpu_s = time.perf_counter() - t0
        out["cpu_baseline"] = {
            "value": round(args.cpu_tokens / cpu_s, 4),
            "unit": "tokens/s",
            "cores": threads,
            "kind": "port",
            "sample": "%d decode steps of the same model at context %d..%d with the CPU oracle (OpenMP over rows / heads; "
                      "the cache rows before the sample are zeros, which costs the same arithmetic)"
                      % (args.cpu_tokens, CONTEXT + 1, CONTEXT + args.cpu_tokens),
        }
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
