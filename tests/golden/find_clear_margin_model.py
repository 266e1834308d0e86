#!/usr/bin/env python3
"""CPU search for a full-size dense decoder whose greedy continuation is decided by clear margins.

Random-init weights give near-uniform logits: among 151936 candidates the two largest are within a few
bf16 ulps at roughly one step in ten, and no arithmetic (fp32 in any order, double) agrees with another
across such a step.  A trained model has peaked logits.  This script instantiates configs[3] (36 layers,
hidden 2560, 32 q / 8 kv heads x 128, intermediate 9728, vocab 151936, int4 g64) ON THE HOST with the
oracle's copy of the library's host-reproducible generator, gives the tied embedding either a
log-normal-like spread of row norms (rowscale = 2^(tau z)) or a few dominant rows (row j < loud_rows scaled by
loud_gain * 2^-j; see fko_synth_fill) and an embedding output scale, and keeps a candidate (embedding seed,
tau, embed_scale) when, over the 32-token prompt + 32 greedy steps of the double-accumulating oracle,

  * at every step, for each of the 16 leading competitors j of the chosen token t, the gap
    logit[t] - logit[j] is at least `--safety` times the largest change of that gap that the two fp32
    summation orders of the oracle (fko_set_accum_mode 1 and 2) produce, teacher-forced on the same
    tokens (and at least 3 bf16 ulps of the top logit), and both fp32 orders pick the same token;
  * the continuation is not one repeated token.

The winner is written to clear_margin_4b.json (parameters, prompt, the 32 expected tokens, margins and the
fp32 envelope per step); tests/test_decoder_gpu.py builds the same model in HBM from the same seeds and
asserts plain free-running equality.  Runs only the oracle: no GPU, no reference code.

The committed fixtures came from

    python tests/golden/find_clear_margin_model.py --bits 4  --grid 0:0.004 --loud-rows 12 --loud-gain 256 \
        --first-seed 6328 --seeds 1 --safety 2 --min-distinct 4          # clear_margin_4b.json
    python tests/golden/find_clear_margin_model.py --bits 8  ... --first-seed 5511 --seeds 1 ...   # clear_margin_4b_q8.json
    python tests/golden/find_clear_margin_model.py --bits 16 ... --first-seed 5600 --seeds 1 ...   # clear_margin_4b_bf16.json

(configs[3] names the 4-bit, 8-bit and bf16 variants; the seed each fixture took is in its file).  About one candidate
in fifteen passes -- most hold at least one near-tie among their 32 steps -- and a candidate costs one to three minutes
on 8 cores, so the seeds tried were ranked beforehand with the library itself: the GPU decoder ran thousands of seeds
through the two-launch and the five-launch task lists and sorted them by the smallest ratio of a logit gap to what the
other list changes it by.  That ranking only chose WHICH seeds this script examined; every number in a fixture is the
CPU oracle's, and the commands above reproduce the files without a GPU.
"""
import argparse
import json
import os
import sys
import time

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

import numpy as np  # noqa: E402

import oracle  # noqa: E402
from fusekit_amd.decoder import DENSE_4B, DecoderConfig  # noqa: E402  (a plain dataclass: no GPU needed)
from helpers import HostDecoderWeights, OracleDecoder, loud_rows_equal, rng  # noqa: E402

N_PROMPT, N_GEN = 32, 32


def run(cfg, W, prompt, forced=None, want_logits=False):
    """Greedy run (or teacher-forced along `forced`); returns tokens, margins, logits of the N_GEN decisions."""
    od = OracleDecoder(cfg, W)
    seq = list(prompt)
    toks, margins, logits = [], [], []
    for i in range(N_PROMPT + N_GEN - 1):
        dec = i >= N_PROMPT - 1
        nxt, m, lg = od.step(seq[i], i, want_logits=want_logits and dec)
        if dec:
            toks.append(nxt); margins.append(m); logits.append(lg)
            seq.append(forced[len(toks) - 1] if forced is not None else nxt)
    return toks, margins, logits


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--model-seed", type=int, default=0)
    ap.add_argument("--grid", nargs="+", default=["0:0.02"], help="tau:embed_scale pairs")
    ap.add_argument("--loud-rows", type=int, default=0, help="token ids 0 .. N-1 get the row gain instead of the spread")
    ap.add_argument("--loud-gain", type=float, default=1.0)
    ap.add_argument("--loud-equal", action="store_true",
                    help="the loud rows all get the gain (a power of two; applied on the host, helpers.loud_rows_equal) "
                         "instead of the generator's gain * 2^-j")
    ap.add_argument("--seeds", type=int, default=8, help="embedding seeds tried per (tau, scale)")
    ap.add_argument("--first-seed", type=int, default=1000)
    ap.add_argument("--safety", type=float, default=3.0)
    ap.add_argument("--min-distinct", type=int, default=3)
    ap.add_argument("--layers", type=int, default=0, help="experiments only: fewer layers")
    ap.add_argument("--bits", type=int, default=4, choices=[4, 8, 16], help="weights: 4- / 8-bit g64 MLX-affine, or bf16")
    ap.add_argument("--out", default="", help="default: clear_margin_4b.json (4-bit), clear_margin_4b_q8.json, clear_margin_4b_bf16.json")
    ap.add_argument("--log", default="")
    args = ap.parse_args()

    if not args.out:
        args.out = os.path.join(HERE, {4: "clear_margin_4b.json", 8: "clear_margin_4b_q8.json", 16: "clear_margin_4b_bf16.json"}[args.bits])
    cfg = DecoderConfig(**DENSE_4B, bits=args.bits, capacity=128)
    if args.layers:
        cfg.n_layers = args.layers
    t0 = time.time()
    W = HostDecoderWeights(cfg, seed=args.model_seed, with_embedding=False)
    print("model built in %.0f s" % (time.time() - t0), flush=True)
    prompt = rng(0).integers(0, cfg.vocab, N_PROMPT).tolist()
    log = open(args.log, "a") if args.log else None

    for pair in args.grid:
        tau, scale = (float(v) for v in pair.split(":"))
        if True:
            for es in range(args.first_seed, args.first_seed + args.seeds):
                cfg.embed_scale = scale
                if args.loud_equal:
                    W.set_embedding(es, tau, 0, 1.0)
                    loud_rows_equal(W, args.loud_rows, args.loud_gain)
                else:
                    W.set_embedding(es, tau, args.loud_rows, args.loud_gain)
                oracle.set_accum_mode(0)
                t0 = time.time()
                toks, margins, lg0 = run(cfg, W, prompt, want_logits=True)
                distinct = len(set(toks))
                rec = dict(tau=tau, embed_scale=scale, embed_seed=es, loud_rows=args.loud_rows, loud_gain=args.loud_gain,
                           loud_equal=bool(args.loud_equal),
                           tokens=toks, distinct=distinct,
                           min_margin=float(min(margins)), margins=[float(m) for m in margins])
                line = "tau %.2f scale %.3g seed %d: distinct %d, min margin %.4g, %.0f s" % (
                    tau, scale, es, distinct, min(margins), time.time() - t0)
                ulps = []
                for i in range(N_GEN):
                    top = float(oracle.bf16_to_f32(lg0[i]).max())
                    ulps.append(margins[i] / 2.0 ** (np.floor(np.log2(abs(top))) - 7))
                rec["min_margin_ulps"] = float(min(ulps))
                line += ", min margin %.1f ulps" % min(ulps)
                if distinct < args.min_distinct or min(ulps) < 3:
                    print(line + "  -> skip", flush=True)
                    if log:
                        log.write(json.dumps(rec) + "\n"); log.flush()
                    continue
                # envelope of the two fp32 orders, teacher-forced on the double run's tokens
                env = np.zeros(N_GEN)
                ratio_steps = np.full(N_GEN, np.inf)
                same = True
                for mode in (1, 2):
                    oracle.set_accum_mode(mode)
                    t_m, _, lg_m = run(cfg, W, prompt, forced=toks, want_logits=True)
                    same = same and t_m == toks
                    for i in range(N_GEN):
                        f0 = oracle.bf16_to_f32(lg0[i]).astype(np.float64)
                        fm = oracle.bf16_to_f32(lg_m[i]).astype(np.float64)
                        lead = np.argsort(-f0)[:17]
                        gap0 = f0[lead[0]] - f0[lead[1:]]
                        gapm = fm[lead[0]] - fm[lead[1:]]
                        r_i = float((gap0 / np.maximum(np.abs(gapm - gap0), 1e-30)).min())
                        ratio_steps[i] = min(ratio_steps[i], r_i)
                        env[i] = max(env[i], float(np.abs(gapm - gap0).max()))
                oracle.set_accum_mode(0)
                ratio = ratio_steps
                rec.update(envelope=[float(e) for e in env], fp32_orders_agree=bool(same), min_ratio=float(ratio.min()))
                print(line + "  fp32 agree %s, min margin/envelope %.2f" % (same, ratio.min()), flush=True)
                if log:
                    log.write(json.dumps(rec) + "\n"); log.flush()
                if same and ratio.min() >= args.safety and not args.layers:
                    rec.update(model_seed=args.model_seed, std=0.02, prompt=prompt, n_layers=cfg.n_layers,
                               safety=args.safety, bits=args.bits,
                               note="written by tests/golden/find_clear_margin_model.py (oracle only)")
                    with open(args.out, "w") as f:
                        json.dump(rec, f, indent=1)
                    print("wrote", args.out, flush=True)
                    return 0
    print("no candidate passed")
    return 1


if __name__ == "__main__":
    sys.exit(main())
