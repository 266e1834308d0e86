#!/usr/bin/env python3
"""CPU search for a full-size mixture-of-experts decoder whose greedy continuation AND whose expert routes are
decided by clear margins -- with routes that differ from layer to layer and from step to step, and a continuation
of several distinct tokens.

The benchmark model of configs[5] (27 layers, hidden 2048, 64 experts of 1408 top-6 + 2 shared, 16 heads of
128 + 64 / 128, vocab 102400, int4 g64) with random weights routes on near-uniform router logits: among 64 experts
the sixth and seventh are within the stack's rounding drift in a few layers of every step, and a different expert
changes a layer's output by far more than a rounding.  A trained model has what a random one lacks: persistent
large activations in a few hidden channels and routers with structure.  This script builds the model ON THE HOST
with the oracle's copy of the library's host-reproducible generator (helpers.HostMoeWeights) and gives it that
structure (helpers.moe_class_channels): a token's class (id modulo the class count) lights one of a few hidden
channels, every layer's router maps each class to its own six experts through a per-layer permutation, and a few
embedding rows dominate the head.  The routes then depend on the token being processed and on the layer -- the
32 random prompt tokens alone walk through every class -- and the expert outputs a class selects decide the next
token, so the continuation moves between classes.  A parameter set is kept when, over the 32-token prompt + 32
greedy steps of the double-accumulating oracle,

  * in every mixture-of-experts layer of every step the gap between the sixth and the seventh router logit is at
    least `--safety` times the largest change the two fp32 summation orders of the oracle (fko_set_accum_mode 1 / 2)
    produce in any router logit of that layer, teacher-forced on the same tokens, and the fp32 runs choose the same
    experts everywhere;
  * at every step each gap of the chosen token to its 16 leading competitors is at least `--safety` times what the
    fp32 orders change it by, and at least 3 bf16 ulps; both fp32 orders pick the same token;
  * the 32 generated tokens hold at least `--min-distinct` different values (the last 16 at least
    `--min-distinct-tail`: the continuation has not settled on one token), and the route sets of the 63 steps hold at
    least `--min-route-sets` different ones in every layer.

The winner is written to clear_margin_moe.json: parameters, prompt, the 32 expected tokens, EVERY step's routes
(63 steps x 26 layers x 6 experts), the worst margins.  tests/test_moe_decoder_gpu.py builds the same model in HBM
and asserts plain free-running equality of the tokens and of all the routes.  Runs only the oracle: no GPU, no
reference code.

The committed fixture came from

    python tests/golden/find_clear_margin_moe.py --loud-rows 64 --gains 4 --ratios 1.0 --perm-seeds 17 --min-distinct 4

after a sweep over permutation seeds 1 .. 20 at that gain (about 20 s per candidate on 8 cores, a minute with the two
fp32 runs).  With 64 embedding rows at gain 4 the expert outputs of a class, not the token's own embedding row, decide
the next token: about half the seeds fall into a fixed point within eight tokens and are dropped at once, the others
cycle through three to five tokens; seed 17 cycles through four (63, 22, 24, 3) with every margin clear.
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
from fusekit_amd.moe_decoder import MoeConfig  # noqa: E402  (a plain dataclass: no GPU needed)
from helpers import HostMoeWeights, OracleMoeDecoder, moe_class_channels, rng  # noqa: E402

N_PROMPT, N_GEN = 32, 32


class Recorder(OracleMoeDecoder):
    """The oracle decoder, keeping every layer's router logits of the last step."""

    def __init__(self, cfg, W):
        super().__init__(cfg, W)
        self.router_logits = []
        real = oracle.softmax_topk_route

        def spy(logits, top_k, scale):
            if top_k == cfg.top_k:
                self.router_logits.append(np.array(logits, copy=True))
            return real(logits, top_k, scale)
        self._spy, self._real = spy, real

    def step(self, token, offset, **kw):
        self.router_logits = []
        oracle.softmax_topk_route = self._spy
        try:
            return super().step(token, offset, **kw)
        finally:
            oracle.softmax_topk_route = self._real


def run(cfg, W, prompt, forced=None, stop_when=None):
    """Greedy (or teacher-forced) run: tokens, margins, logits of the N_GEN decisions; router logits and routes of
    every step [steps][moe layers].  stop_when(tokens so far) -> True ends a hopeless greedy run early."""
    od = Recorder(cfg, W)
    seq = list(prompt)
    toks, margins, logits, rl, routes = [], [], [], [], []
    for i in range(N_PROMPT + N_GEN - 1):
        dec = i >= N_PROMPT - 1
        nxt, m, lg = od.step(seq[i], i, want_logits=dec)
        rl.append([oracle.bf16_to_f32(x).astype(np.float64) for x in od.router_logits])
        routes.append([sorted(int(e) for e in r.tolist()) for r in od.routes])
        if dec:
            toks.append(nxt); margins.append(m); logits.append(lg)
            seq.append(forced[len(toks) - 1] if forced is not None else nxt)
            if stop_when is not None and stop_when(toks):
                return toks, margins, logits, rl, routes, False
    return toks, margins, logits, rl, routes, True


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--model-seed", type=int, default=0)
    ap.add_argument("--classes", type=int, default=8)
    ap.add_argument("--first-channel", type=int, default=8)
    ap.add_argument("--level", type=float, default=2048.0, help="embedding value of a token's class channel")
    ap.add_argument("--ladder", default="12:2", help="top:step -> router logits top, top-step, ... of a class's six experts")
    ap.add_argument("--noise", type=float, default=0.05, help="scale of the routers' random part")
    ap.add_argument("--loud-rows", type=int, nargs="+", default=[64])
    ap.add_argument("--gains", type=float, nargs="+", default=[64.0], help="gain of embedding row 0")
    ap.add_argument("--ratios", type=float, nargs="+", default=[1.25], help="gain of row j = gain * ratio^-j")
    ap.add_argument("--perm-seeds", type=int, nargs="+", default=[1])
    ap.add_argument("--safety", type=float, default=2.0)
    ap.add_argument("--min-distinct", type=int, default=4)
    ap.add_argument("--min-route-sets", type=int, default=4)
    ap.add_argument("--min-distinct-tail", type=int, default=3, help="distinct values among the last 16 generated tokens")
    ap.add_argument("--layers", type=int, default=0, help="experiments only: fewer layers")
    ap.add_argument("--out", default=os.path.join(HERE, "clear_margin_moe.json"))
    args = ap.parse_args()

    cfg = MoeConfig(capacity=128)
    if args.layers:
        cfg.n_layers = args.layers
    prompt = rng(0).integers(0, cfg.vocab, N_PROMPT).tolist()
    top, step = (float(v) for v in args.ladder.split(":"))
    ladder = [top - step * j for j in range(cfg.top_k)]
    t0 = time.time()
    base = HostMoeWeights(cfg, seed=args.model_seed)
    print("model built in %.0f s" % (time.time() - t0), flush=True)
    keep = {"embed_tokens": np.array(base.mats["embed_tokens"].w, copy=True), "final_norm": base.vecs["final_norm"].copy()}
    for l in range(cfg.first_dense, cfg.n_layers):
        keep[f"layers.{l}.mlp.gate"] = np.array(base.mats[f"layers.{l}.mlp.gate"].w, copy=True)

    def restore():
        for name, a in keep.items():
            if name in base.vecs:
                base.vecs[name][:] = a
            else:
                np.asarray(base.mats[name].w)[...] = a

    for loud_rows in args.loud_rows:
        for gain in args.gains:
            for ratio in args.ratios:
                for ps in args.perm_seeds:
                    restore()
                    W = base
                    _, expected = moe_class_channels(cfg, W.mats, W.vecs, args.classes, args.first_channel, args.level, ladder,
                                                     args.noise, ps, loud_rows, gain, ratio)
                    oracle.set_accum_mode(0)
                    t0 = time.time()

                    def hopeless(toks):   # a fixed point reached
                        return len(toks) >= 8 and len(set(toks[-4:])) == 1 and args.min_distinct_tail > 1
                    toks, margins, lg0, rl0, routes0, whole = run(cfg, W, prompt, stop_when=hopeless)
                    tag = "rows %d gain %g ratio %g perm %d" % (loud_rows, gain, ratio, ps)
                    if not whole:
                        print("%s: fixed point %s after %d tokens, %.0f s  -> skip" % (tag, toks[-1], len(toks), time.time() - t0), flush=True)
                        continue
                    gap67 = min(np.sort(x)[-cfg.top_k] - np.sort(x)[-cfg.top_k - 1] for st in rl0 for x in st)
                    ulps = []
                    for i in range(N_GEN):
                        topv = float(oracle.bf16_to_f32(lg0[i]).max())
                        ulps.append(margins[i] / 2.0 ** (np.floor(np.log2(abs(topv))) - 7))
                    n_layers_moe = cfg.n_layers - cfg.first_dense
                    sets_per_layer = [len({tuple(st[l]) for st in routes0}) for l in range(n_layers_moe)]
                    seq = list(prompt) + toks[:-1]
                    as_built = all(routes0[i][l] == expected[cfg.first_dense + l][seq[i] % args.classes]
                                   for i in range(len(routes0)) for l in range(n_layers_moe))
                    line = "%s: distinct %d, min logit margin %.1f ulps, min 6th-7th router gap %.3g, route sets per layer %d..%d, as built %s, %.0f s" % (
                        tag, len(set(toks)), min(ulps), gap67, min(sets_per_layer), max(sets_per_layer), as_built, time.time() - t0)
                    if (len(set(toks)) < args.min_distinct or len(set(toks[-16:])) < args.min_distinct_tail or min(ulps) < 3 or gap67 <= 0
                            or min(sets_per_layer) < args.min_route_sets):
                        print(line + "  -> skip  tokens %s" % toks, flush=True)
                        continue
                    same_tok, same_routes, ratio_tok, ratio_route = True, True, np.inf, np.inf
                    for mode in (1, 2):
                        oracle.set_accum_mode(mode)
                        t_m, _, lg_m, rl_m, routes_m, _ = run(cfg, W, prompt, forced=toks)
                        same_tok = same_tok and t_m == toks
                        same_routes = same_routes and routes_m == routes0
                        for i in range(N_GEN):
                            f0 = oracle.bf16_to_f32(lg0[i]).astype(np.float64)
                            fm = oracle.bf16_to_f32(lg_m[i]).astype(np.float64)
                            lead = np.argsort(-f0)[:17]
                            g0, gm = f0[lead[0]] - f0[lead[1:]], fm[lead[0]] - fm[lead[1:]]
                            ratio_tok = min(ratio_tok, float((g0 / np.maximum(np.abs(gm - g0), 1e-30)).min()))
                        for st0, stm in zip(rl0, rl_m):
                            for x0, xm in zip(st0, stm):
                                s = np.sort(x0)
                                ratio_route = min(ratio_route, float((s[-cfg.top_k] - s[-cfg.top_k - 1]) / max(np.abs(xm - x0).max(), 1e-30)))
                    oracle.set_accum_mode(0)
                    print(line + "  fp32: same tokens %s, same routes %s, logit margin / envelope %.2f, router gap / envelope %.2f  tokens %s" % (
                        same_tok, same_routes, ratio_tok, ratio_route, toks), flush=True)
                    if same_tok and same_routes and min(ratio_tok, ratio_route) >= args.safety and not args.layers:
                        rec = dict(model_seed=args.model_seed, std=0.02, classes=args.classes, first_channel=args.first_channel,
                                   level=args.level, ladder=ladder, route_noise=args.noise, perm_seed=ps, loud_rows=loud_rows,
                                   loud_gain=gain, loud_ratio=ratio, prompt=prompt, tokens=toks, n_layers=cfg.n_layers,
                                   min_margin_ulps=float(min(ulps)), min_router_gap=float(gap67), min_ratio=float(ratio_tok),
                                   min_router_ratio=float(ratio_route), safety=args.safety, distinct=len(set(toks)),
                                   route_sets_per_layer=sets_per_layer, routes=routes0,
                                   note="written by tests/golden/find_clear_margin_moe.py (oracle only); routes[step][layer] for the "
                                        "63 steps (32 prompt tokens, then the generated ones) and the 26 expert layers")
                        with open(args.out, "w") as f:
                            json.dump(rec, f)
                        print("wrote", args.out, flush=True)
                        return 0
    print("no candidate passed")
    return 1


if __name__ == "__main__":
    sys.exit(main())
