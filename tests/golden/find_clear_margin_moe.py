#!/usr/bin/env python3
"""CPU search for a full-size mixture-of-experts decoder whose greedy continuation AND whose expert routes are
decided by clear margins.

The benchmark model of configs[5] (27 layers, hidden 2048, 64 experts of 1408 top-6 + 2 shared, 16 heads of
128 + 64 / 128, vocab 102400, int4 g64) with random weights routes on near-uniform router logits: among 64 experts
the sixth and seventh are within the stack's rounding drift in a few layers of every step, and a different expert
changes a layer's output by far more than a rounding.  A trained model has what a random one lacks: a persistent
large activation in one hidden channel and routers with structure.  This script builds the model ON THE HOST with
the oracle's copy of the library's host-reproducible generator (helpers.HostMoeWeights), gives it that structure
(helpers.moe_stable_channel: one embedding column at a constant level, router columns that read it, the routers'
random part scaled down; a few dominant embedding rows as in find_clear_margin_model.py), and keeps a parameter
set when, over a 32-token prompt + 32 greedy steps of the double-accumulating oracle,

  * in every mixture-of-experts layer of every step the gap between the sixth and the seventh router logit is at
    least `--safety` times the largest change the two fp32 summation orders of the oracle (fko_set_accum_mode 1 / 2)
    produce in any router logit of that layer, teacher-forced on the same tokens, and the fp32 runs choose the same
    experts everywhere;
  * at every step each gap of the chosen token to its 16 leading competitors is at least `--safety` times what the
    fp32 orders change it by, and at least 3 bf16 ulps; both fp32 orders pick the same token;
  * the continuation is not one repeated token.

The winner is written to clear_margin_moe.json (parameters, prompt, the 32 expected tokens, the routes' and the
logits' worst margins); tests/test_moe_decoder_gpu.py builds the same model in HBM and asserts plain free-running
equality.  Runs only the oracle: no GPU, no reference code.

    python tests/golden/find_clear_margin_moe.py --levels 8 --patterns 12:2 --noises 0.05 --embed-scales 1
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
from helpers import HostMoeWeights, OracleMoeDecoder, moe_stable_channel, rng  # noqa: E402

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


def run(cfg, W, prompt, forced=None):
    """Greedy (or teacher-forced) run: tokens, margins, logits of the N_GEN decisions; router logits and routes of
    every step [steps][moe layers]."""
    od = Recorder(cfg, W)
    seq = list(prompt)
    toks, margins, logits, rl, routes = [], [], [], [], []
    for i in range(N_PROMPT + N_GEN - 1):
        dec = i >= N_PROMPT - 1
        nxt, m, lg = od.step(seq[i], i, want_logits=dec)
        rl.append([oracle.bf16_to_f32(x).astype(np.float64) for x in od.router_logits])
        routes.append([frozenset(r.tolist()) for r in od.routes])
        if dec:
            toks.append(nxt); margins.append(m); logits.append(lg)
            seq.append(forced[len(toks) - 1] if forced is not None else nxt)
    return toks, margins, logits, rl, routes


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--model-seed", type=int, default=0)
    ap.add_argument("--channel", type=int, default=7)
    ap.add_argument("--levels", type=float, nargs="+", default=[8.0], help="embedding column level")
    ap.add_argument("--patterns", nargs="+", default=["12:2"], help="top:step -> router logits top, top-step, ... for the six chosen experts, 0 for the rest")
    ap.add_argument("--noises", type=float, nargs="+", default=[0.05], help="scale of the routers' random part")
    ap.add_argument("--loud-rows", type=int, default=12)
    ap.add_argument("--loud-gain", type=float, default=256.0)
    ap.add_argument("--safety", type=float, default=2.0)
    ap.add_argument("--min-distinct", type=int, default=2)
    ap.add_argument("--layers", type=int, default=0, help="experiments only: fewer layers")
    ap.add_argument("--out", default=os.path.join(HERE, "clear_margin_moe.json"))
    args = ap.parse_args()

    cfg = MoeConfig(capacity=128)
    if args.layers:
        cfg.n_layers = args.layers
    prompt = rng(0).integers(0, cfg.vocab, N_PROMPT).tolist()
    for level in args.levels:
        for pat in args.patterns:
            for noise in args.noises:
                t0 = time.time()
                W = HostMoeWeights(cfg, seed=args.model_seed, embed_loud_rows=args.loud_rows, embed_loud_gain=args.loud_gain)
                top, step = (float(v) for v in pat.split(":"))
                route_logits = [top - step * j if j < cfg.top_k else 0.0 for j in range(cfg.n_experts)]
                moe_stable_channel(cfg, W.mats, W.vecs, args.channel, level, route_logits, noise)
                print("model built in %.0f s" % (time.time() - t0), flush=True)
                oracle.set_accum_mode(0)
                t0 = time.time()
                toks, margins, lg0, rl0, routes0 = run(cfg, W, prompt)
                gap67 = min(np.sort(x)[-cfg.top_k] - np.sort(x)[-cfg.top_k - 1] for st in rl0 for x in st)
                ulps = []
                for i in range(N_GEN):
                    topv = float(oracle.bf16_to_f32(lg0[i]).max())
                    ulps.append(margins[i] / 2.0 ** (np.floor(np.log2(abs(topv))) - 7))
                line = "level %g pattern %s noise %g: distinct %d, min logit margin %.1f ulps, min 6th-7th router gap %.3g, %.0f s" % (
                    level, pat, noise, len(set(toks)), min(ulps), gap67, time.time() - t0)
                if len(set(toks)) < args.min_distinct or min(ulps) < 3 or gap67 <= 0:
                    print(line + "  -> skip", flush=True)
                    continue
                same_tok, same_routes, ratio_tok, ratio_route = True, True, np.inf, np.inf
                for mode in (1, 2):
                    oracle.set_accum_mode(mode)
                    t_m, _, lg_m, rl_m, routes_m = run(cfg, W, prompt, forced=toks)
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
                print(line + "  fp32: same tokens %s, same routes %s, logit margin / envelope %.2f, router gap / envelope %.2f" % (
                    same_tok, same_routes, ratio_tok, ratio_route), flush=True)
                if same_tok and same_routes and min(ratio_tok, ratio_route) >= args.safety and not args.layers:
                    rec = dict(model_seed=args.model_seed, std=0.02, channel=args.channel, level=level, route_logits=route_logits,
                               route_noise=noise, loud_rows=args.loud_rows, loud_gain=args.loud_gain, prompt=prompt, tokens=toks,
                               n_layers=cfg.n_layers, min_margin_ulps=float(min(ulps)), min_router_gap=float(gap67),
                               min_ratio=float(ratio_tok), min_router_ratio=float(ratio_route), safety=args.safety,
                               distinct=len(set(toks)),
                               routes_last_step=[sorted(r) for r in routes0[-1]],
                               note="written by tests/golden/find_clear_margin_moe.py (oracle only)")
                    with open(args.out, "w") as f:
                        json.dump(rec, f, indent=1)
                    print("wrote", args.out, flush=True)
                    return 0
    print("no candidate passed")
    return 1


if __name__ == "__main__":
    sys.exit(main())
