"""python -m fusekit_amd <command>

  info                                   the device as the backend sees it (fk_target_describe)
  generate --model DIR --ids 1,2,3 [--max-tokens N] [--capacity C]
                                         greedy decode of an mlx-lm format checkpoint (token ids in,
                                         token ids out; no tokenizer is bundled)
  export-random --out DIR [--bits 4] [--layers 2] [--moe] ...
                                         write a small random-init model in the mlx-lm file layout (--moe: a
                                         mixture-of-experts model in the deepseek_v2 layout; generate / patch
                                         recognise it by config.json's model_type)
  patch --model DIR [--out DIR/.fusekit] [--prefill-m 32,128] [--capacity C]
                                         the reference's `fusekit patch`: write task_graph.json, manifest.json and
                                         variants/prefill_mN/task_graph.json for a checkpoint
  generate --model DIR --artifact DIR ... decode from the artifact's task graphs instead of a fresh runtime
  bench DIR [--tokens 64] [--prompt TEXT | --ids 1,2,3] [--repeat 1] [--max-kv-size N] [--kv-bits 4|8]
        [--kv-group-size 64] [--per-kernel] [--dump-tokens]
                                         the reference's `fusekit bench`: fixed-length generation, `[bench:N] key=value`
                                         lines (prompt_tokens, generated_tokens, stream_tps, wall_s, wall_tps, peak_gb)
"""
import argparse
import json
import sys


def main() -> int:
    ap = argparse.ArgumentParser(prog="python -m fusekit_amd")
    sub = ap.add_subparsers(dest="cmd", required=True)
    sub.add_parser("info")
    g = sub.add_parser("generate")
    g.add_argument("--model", required=True)
    g.add_argument("--ids", required=True, help="comma-separated prompt token ids")
    g.add_argument("--max-tokens", type=int, default=32)
    g.add_argument("--capacity", type=int, default=1024)
    g.add_argument("--artifact", default=None, help="directory written by `patch`")
    pa = sub.add_parser("patch")
    pa.add_argument("--model", required=True)
    pa.add_argument("--out", default=None)
    pa.add_argument("--prefill-m", default="", help="comma-separated active row counts of the prefill variants")
    pa.add_argument("--capacity", type=int, default=1024)
    e = sub.add_parser("export-random")
    e.add_argument("--out", required=True)
    e.add_argument("--bits", type=int, default=4, choices=[4, 8, 16])
    e.add_argument("--layers", type=int, default=2)
    e.add_argument("--hidden", type=int, default=256)
    e.add_argument("--heads", type=int, default=4)
    e.add_argument("--kv-heads", type=int, default=2)
    e.add_argument("--head-dim", type=int, default=64)
    e.add_argument("--inter", type=int, default=512)
    e.add_argument("--vocab", type=int, default=2000)
    e.add_argument("--seed", type=int, default=0)
    e.add_argument("--moe", action="store_true", help="a small mixture-of-experts model with low-rank keys (deepseek_v2 layout)")
    from . import bench_cli
    bench_cli.add_arguments(sub)
    args = ap.parse_args()

    if args.cmd == "bench":
        return bench_cli.run(args)
    from . import native as fk
    if args.cmd == "info":
        t = fk.target_describe()
        print(json.dumps({f: (getattr(t, f).decode() if isinstance(getattr(t, f), bytes) else getattr(t, f))
                          for f, _ in t._fields_}, indent=1))
        return 0
    from .decoder import DecoderConfig, DecoderRuntime, DecoderWeights
    if args.cmd == "export-random" and args.moe:
        from .checkpoint import save_moe_checkpoint
        from .moe_decoder import MoeConfig, MoeWeights
        mc = MoeConfig(n_layers=max(args.layers, 2), hidden=512, n_heads=args.heads, kv_lora_rank=128, rope_dim=64, nope_dim=128,
                       v_dim=128, n_experts=8, top_k=2, moe_inter=128, n_shared=1, dense_inter=args.inter, first_dense=1,
                       vocab=args.vocab, bits=args.bits if args.bits != 16 else 4)
        save_moe_checkpoint(args.out, mc, MoeWeights.random_init(mc, seed=args.seed))
        print(f"wrote {args.out}/config.json and model.safetensors (deepseek_v2 layout)")
        return 0
    if args.cmd == "export-random":
        from .checkpoint import save_mlx_checkpoint
        cfg = DecoderConfig(n_layers=args.layers, hidden=args.hidden, n_heads=args.heads, n_kv=args.kv_heads,
                            head_dim=args.head_dim, inter=args.inter, vocab=args.vocab, bits=args.bits, qk_norm=True,
                            swiglu_variant=1)
        save_mlx_checkpoint(args.out, cfg, DecoderWeights.random_init(cfg, seed=args.seed))
        print(f"wrote {args.out}/config.json and model.safetensors")
        return 0
    import os
    model_type = json.load(open(os.path.join(args.model, "config.json"))).get("model_type", "")
    if model_type.startswith("deepseek"):   # mixture-of-experts decoder with low-rank keys
        from .artifact import ArtifactRuntime, write_artifact
        from .checkpoint import load_moe_checkpoint
        from .moe_decoder import MoeRuntime
        cfg, w = load_moe_checkpoint(args.model, capacity=args.capacity)
        if args.cmd == "patch":
            rt = MoeRuntime(cfg, w)
            out = args.out or os.path.join(args.model, ".fusekit")
            write_artifact(rt, out, os.path.basename(os.path.normpath(args.model)))
            print(json.dumps({"artifact": out, "tasks": len(rt.tasks), "variants": []}))
            return 0
        prompt = [int(t) for t in args.ids.split(",") if t.strip()]
        if args.artifact:
            print(json.dumps({"tokens": ArtifactRuntime(args.artifact, w).generate(prompt, args.max_tokens)}))
            return 0
        toks, gpu_s, steps = MoeRuntime(cfg, w).generate(prompt, args.max_tokens)
        print(json.dumps({"tokens": toks, "decode_tok_per_s": round(steps / gpu_s, 1) if gpu_s else None}))
        return 0
    from .checkpoint import load_mlx_checkpoint
    cfg, w = load_mlx_checkpoint(args.model, capacity=args.capacity)
    if args.cmd == "patch":
        import os
        from .artifact import write_artifact
        from .prefill_variant import PrefillVariant
        rt = DecoderRuntime(cfg, w)
        out = args.out or os.path.join(args.model, ".fusekit")
        ms = [int(v) for v in args.prefill_m.split(",") if v.strip()]
        write_artifact(rt, out, os.path.basename(os.path.normpath(args.model)), prefill_variants=[PrefillVariant(rt, m) for m in ms])
        print(json.dumps({"artifact": out, "tasks": len(rt.tasks), "variants": [f"prefill_m{m}" for m in ms]}))
        return 0
    prompt = [int(t) for t in args.ids.split(",") if t.strip()]
    if args.artifact:
        from .artifact import ArtifactRuntime
        art = ArtifactRuntime(args.artifact, w)
        print(json.dumps({"tokens": art.generate(prompt, args.max_tokens), "variants": sorted(art.variants)}))
        return 0
    rt = DecoderRuntime(cfg, w)
    toks, gpu_s, steps = rt.generate(prompt, args.max_tokens)
    print(json.dumps({"tokens": toks, "decode_tok_per_s": round(steps / gpu_s, 1) if gpu_s else None}))
    return 0


if __name__ == "__main__":
    sys.exit(main())
