#!/usr/bin/env python3
"""Headline benchmark: hipGraph-replayed batch-1 greedy decode of the 4B-class dense model,
4-bit g64 MLX-affine weights, 512 generated tokens, on one MI355X.

One "step" = one decoded token = one replay of the captured decode graph (step_init, embed,
36 x [rmsnorm_qkv, rope + kv-store + sdpa (one launch), o_proj+residual,
rmsnorm_gateup_swiglu, down_proj+residual], final norm + LM head, argmax).  Weights are random-init (seeded, generated
and quantised in HBM); inputs are resident before the timed region.

Prints ONE JSON line: value = generated tokens/s (wall clock around the K timed steps), plus
  roofline     -- the dominant kernel (int4 gate/up SwiGLU qGEMV): algorithmic bytes per launch /
                  its average launch duration, measured here with HIP events on the launch stream
                  over the 36 layers' distinct weights (985 MB, larger than any cache),
  cpu_baseline -- the CPU oracle (C restatement of the reference semantics) decoding the same
                  model on the host cores, bounded to --cpu-tokens decode steps (about 10 s of CPU work).
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0  # MI355X HBM3E published peak
# HBM bytes per launch of the int4 gate/up kernel of the 4B-class model, from rocprofv3 FETCH_SIZE and
# WRITE_SIZE (two counter runs of this script, each scaled by what the same counter reads for the plain
# 256 MiB copies of --calibrate-copy: 1.99989 and 1.0).  Counters cannot be read from inside this process.
GATEUP_Q4_4B_TRAFFIC_BYTES = 28590500


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=512)
    ap.add_argument("--warmup", type=int, default=32)
    ap.add_argument("--bits", type=int, default=4, choices=[4, 8, 16])
    ap.add_argument("--prompt", type=int, default=32)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--cpu-tokens", type=int, default=24,
                    help="decode steps the CPU oracle runs for cpu_baseline (about 10 s on 16 cores)")
    ap.add_argument("--per-kernel", action="store_true", help="print per-family GPU time of one token to stderr")
    ap.add_argument("--layers", type=int, default=0, help="experiment only: override the layer count (not the headline config)")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run 4 plain 256 MiB device copies (outside the timed region): the known-traffic "
                         "kernel that rocprofv3 byte counters of the same run are scaled by")
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
    total = args.prompt + args.warmup + args.steps
    capacity = max(1024, 1 << (total - 1).bit_length())
    cfg = DecoderConfig(**DENSE_4B, bits=args.bits, capacity=capacity)
    if args.layers:
        cfg.n_layers = args.layers
    t0 = time.time()
    W = DecoderWeights.random_init(cfg, seed=0)
    rt = DecoderRuntime(cfg, W, hist_capacity=max(4096, args.steps + args.warmup),
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
    # warm-up: W untimed decode steps
    done = 0
    while done < args.warmup:
        n = min(64, args.warmup - done)
        toks, _ = rt.d.decode_chunk(rt.graph, rt.uniforms, offset, tok, n)
        tok, offset, done = toks[-1], offset + n, done + n
    fk.sync()
    # timed: exactly K steps, all chunks enqueued by the native loop, sync on both sides
    gpu_s = 0.0
    t0 = time.perf_counter()
    done = 0
    while done < args.steps:
        n = min(rt.uniforms.hist_capacity, args.steps - done)
        toks, sec = rt.d.decode_chunk(rt.graph, rt.uniforms, offset, tok, n)
        tok, offset, done, gpu_s = toks[-1], offset + n, done + n, gpu_s + sec
    fk.sync()
    wall_s = time.perf_counter() - t0
    tok_s = args.steps / wall_s
    ctx_mid = args.prompt + args.warmup + args.steps // 2
    bytes_per_token = cfg.token_bytes(ctx_mid)
    roofline_tok_s = HBM_PEAK_GBPS * 1e9 / bytes_per_token

    # ---- dominant kernel: gate/up SwiGLU qGEMV over the 36 layers' distinct weights ----
    gateup = [t for t in rt.tasks if t.kernel.startswith("fusekit_rmsnorm_gateup_swiglu")]
    per = cfg.bits / 8 + (0 if cfg.bits == 16 else 4 / cfg.group)
    gateup_bytes = int(2 * cfg.inter * cfg.hidden * per) + 2 * cfg.hidden * 2 + cfg.inter * 2
    g2 = rt.d.build_graph(gateup, barriers=[True] * len(gateup))   # serialised, one launch after another
    rt.d.execute_graph(g2)
    reps = 20
    sec = rt.d.execute_graph(g2, repeat=reps)
    gateup_us = sec / (reps * len(gateup)) * 1e6
    achieved = gateup_bytes / (gateup_us * 1e-6) / 1e9

    per_kernel = {}
    if args.per_kernel and args.mode == "persistent":
        tr = rt.d.graph_phase_trace(rt.graph)
        names = ["embed"] + ["qkv", "attention", "o_proj", "gateup", "down"] * cfg.n_layers + ["lm_head", "argmax_scan", "argmax_final"]
        for nm, s_ in zip(names, tr):
            per_kernel[nm] = per_kernel.get(nm, 0.0) + s_
        print("[bench:per-phase] " + " ".join(f"{k}={v * 1e3:.3f}ms" for k, v in per_kernel.items())
              + f" | layer0: " + " ".join(f"{n}={t * 1e6:.1f}us" for n, t in zip(names[1:6], tr[1:6])), file=sys.stderr)
    elif args.per_kernel:
        times = rt.d.profile_graph_nodes(rt.graph)
        for t, s in zip(rt.tasks, times):
            fam = t.kernel.rsplit("_f", 1)[0]
            per_kernel[fam] = per_kernel.get(fam, 0.0) + s
        print("[bench:per-kernel] " + " ".join(f"{k}={v * 1e3:.3f}ms" for k, v in per_kernel.items()),
              file=sys.stderr)

    out = {
        "metric": "decode tok/s, 4B-class %d-bit @ L=%d (int4 qGEMV HBM GB/s in roofline)" % (cfg.bits, args.steps),
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
            "context_range": [args.prompt + args.warmup, args.prompt + args.warmup + args.steps],
            "graph_nodes": len(rt.tasks),
        },
        "gpu_ms_per_step": round(gpu_s / args.steps * 1e3, 4),
        "bytes_per_token": bytes_per_token,
        "weight_streaming_roofline_tok_s": round(roofline_tok_s, 1),
        "frac_of_roofline_tok_s": round(tok_s / roofline_tok_s, 4),
        "device": props.name.decode().strip() or props.arch.decode(),
        "setup_s": round(setup_s, 1),
        "roofline": {
            "kernel": "gemv_stream_kernel<Q4, gate/up SwiGLU, fused RMSNorm> (fusekit_rmsnorm_gateup_swiglu)",
            "bound": "hbm",
            "achieved": round(achieved, 1),
            "peak": HBM_PEAK_GBPS,
            "unit": "GB/s",
            "frac": round(achieved / HBM_PEAK_GBPS, 4),
            "traffic": GATEUP_Q4_4B_TRAFFIC_BYTES if (cfg.bits == 4 and not args.layers) else None,
            "bytes_per_launch": gateup_bytes,
            "avg_launch_us": round(gateup_us, 3),
            "launches_timed": reps * len(gateup),
        },
    }

    if not args.no_cpu_baseline:
        sys.path.insert(0, os.path.join(ROOT, "tests"))
        import oracle
        from helpers import OracleDecoder
        od = OracleDecoder(cfg, W)
        threads = oracle.num_threads()
        t0 = time.perf_counter()
        t = prompt[0]
        for i in range(args.cpu_tokens):
            t, _, _ = od.step(t, i)
        cpu_s = time.perf_counter() - t0
        out["cpu_baseline"] = {
            "value": round(args.cpu_tokens / cpu_s, 4),
            "unit": "tokens/s",
            "cores": threads,
            "kind": "port",
            "sample": "%d decode steps of the same model at context 1..%d with the CPU oracle (OpenMP over rows/heads)"
                      % (args.cpu_tokens, args.cpu_tokens),
        }
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
