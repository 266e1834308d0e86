"""`python -m fusekit_amd bench MODEL ...`: the reference's fixed-length benchmark driver for this backend.

Same arguments and the same `[bench:N] key=value` lines as `fusekit bench` (src/main.rs:74-107,
src/commands/bench.rs:13-37, scripts/bench.py:131-150): --tokens, --prompt, --repeat, --max-kv-size, --kv-bits,
--kv-group-size, --raw, --per-kernel, --dump-tokens.  Differences a caller has to know:

  * MODEL is a checkpoint directory (mlx-lm file layout), not a name in a model registry.
  * The prompt is tokenised with MODEL/tokenizer.json when it is there (the `tokenizers` package); without one
    the prompt's UTF-8 bytes are the token ids (every vocabulary here has at least 256 entries), or --ids gives
    them directly.
  * --raw (the reference: the same model through plain mlx-lm) has no counterpart on this platform: refused.
  * --per-kernel prints, after the run, the GPU time of every node of ONE decode step's graph
    (`[fusekit-profile]` lines, aggregate by kernel family first; python/fusekit_runtime/dispatch.py:4732-4790).
"""
import json
import os
import time
from typing import List


def add_arguments(sub) -> None:
    b = sub.add_parser("bench")
    b.add_argument("model", help="checkpoint directory (config.json + *.safetensors)")
    b.add_argument("--tokens", type=int, default=64, help="number of generated tokens")
    b.add_argument("--prompt", default="Repeat the word token forever: token token token")
    b.add_argument("--ids", default="", help="comma-separated prompt token ids (instead of --prompt)")
    b.add_argument("--repeat", type=int, default=1)
    b.add_argument("--max-kv-size", type=int, default=None, help="KV-cache capacity in positions")
    b.add_argument("--kv-bits", type=int, default=None, choices=[4, 8], help="quantised KV cache")
    b.add_argument("--kv-group-size", type=int, default=64)
    b.add_argument("--raw", action="store_true", help="(reference: plain mlx-lm) not available here")
    b.add_argument("--per-kernel", action="store_true", help="GPU time per graph node of one decode step")
    b.add_argument("--dump-tokens", action="store_true")


def _prompt_ids(args, vocab: int) -> List[int]:
    if args.ids:
        return [int(t) for t in args.ids.split(",") if t.strip()]
    tok_file = os.path.join(args.model, "tokenizer.json")
    if os.path.exists(tok_file):
        from tokenizers import Tokenizer
        return list(Tokenizer.from_file(tok_file).encode(args.prompt).ids)
    ids = list(args.prompt.encode("utf-8"))
    if vocab < 256:
        raise SystemExit("bench: no tokenizer.json and a vocabulary below 256 entries: pass --ids")
    return ids


def _family(kernel: str) -> str:
    name = kernel[len("fusekit_"):] if kernel.startswith("fusekit_") else kernel
    head, sep, tail = name.rpartition("_f")
    return head if sep and tail.isdigit() else name


def _per_kernel(rt) -> None:
    """One more decode step, node by node (events around every node of the step's graph)."""
    us = [t * 1e6 for t in rt.d.profile_graph_nodes(rt.graph)]
    rows = [(u, i, t.kernel) for i, (u, t) in enumerate(zip(us, rt.tasks))]
    print("[fusekit-profile] per-kernel decode step", flush=True)
    print(f"[fusekit-profile] kernels={len(rows)} total_gpu_us={sum(us):.1f}", flush=True)
    fam = {}
    for u, _, k in rows:
        a = fam.setdefault(_family(k), [0.0, 0])
        a[0] += u
        a[1] += 1
    print("[fusekit-profile] aggregate by kernel family:", flush=True)
    for f, (u, n) in sorted(fam.items(), key=lambda kv: -kv[1][0]):
        print(f"[fusekit-profile] {u:9.2f} us  count={n:>4} family={f}", flush=True)
    print("[fusekit-profile] top by gpu_us:", flush=True)
    for u, i, k in sorted(rows, reverse=True)[:40]:
        print(f"[fusekit-profile] {u:9.2f} us  task={i:>4} kernel={k}", flush=True)


def run(args) -> int:
    if args.raw and args.per_kernel:
        raise SystemExit("--raw and --per-kernel are mutually exclusive")      # src/commands/bench.rs:27-29
    if args.raw:
        raise SystemExit("bench: --raw measures the model through plain mlx-lm; there is no such path on this platform")
    from . import native as fk
    cfg_json = json.load(open(os.path.join(args.model, "config.json")))
    moe = cfg_json.get("model_type", "").startswith("deepseek")
    free0, total = fk.mem_info()
    vocab = int(cfg_json.get("text_config", cfg_json)["vocab_size"])
    prompt = _prompt_ids(args, vocab)
    capacity = args.max_kv_size or max(1024, 1 << (len(prompt) + args.tokens - 1).bit_length())
    if len(prompt) + args.tokens > capacity:
        raise SystemExit(f"bench: prompt ({len(prompt)}) + tokens ({args.tokens}) exceed --max-kv-size {capacity}")
    print(f"[bench] model={os.path.abspath(args.model)} mode=fusekit"
          + (" + per-kernel profile" if args.per_kernel else ""), flush=True)
    if moe:
        if args.kv_bits:
            raise SystemExit("bench: the mixture-of-experts runtime keeps a bf16 KV cache (--kv-bits is for dense models)")
        from .checkpoint import load_moe_checkpoint
        from .moe_decoder import MoeRuntime
        cfg, w = load_moe_checkpoint(args.model, capacity=capacity)
        rt = MoeRuntime(cfg, w)
    else:
        from .checkpoint import load_mlx_checkpoint
        from .decoder import DecoderRuntime
        cfg, w = load_mlx_checkpoint(args.model, capacity=capacity)
        if args.kv_bits:
            cfg.kv_bits, cfg.kv_group = args.kv_bits, args.kv_group_size
        rt = DecoderRuntime(cfg, w)
    for rep in range(args.repeat):
        rt.reset()
        fk.sync()
        started = time.perf_counter()
        toks, gpu_s, steps = rt.generate(prompt, args.tokens)
        fk.sync()
        wall_s = time.perf_counter() - started
        free1, _ = fk.mem_info()
        print(f"[bench:{rep}] prompt_tokens={len(prompt)}", flush=True)
        print(f"[bench:{rep}] generated_tokens={len(toks)}", flush=True)
        print(f"[bench:{rep}] stream_tps={steps / gpu_s if gpu_s else 0:.3f}", flush=True)
        print(f"[bench:{rep}] wall_s={wall_s:.3f}", flush=True)
        print(f"[bench:{rep}] wall_tps={len(toks) / wall_s if wall_s else 0:.3f}", flush=True)
        print(f"[bench:{rep}] peak_gb={(free0 - free1) / 1e9:.3f}", flush=True)
        if args.dump_tokens:
            print(f"[bench:{rep}] tokens={toks}", flush=True)
    if args.per_kernel:
        _per_kernel(rt)
    return 0
