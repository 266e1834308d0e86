"""What the committed clear-margin fixtures promise, checked on their own numbers (no model is built here: the
search scripts beside them wrote these files from the CPU oracle alone, and the GPU tests decode against them)."""
import json
import os

import pytest

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


@pytest.mark.parametrize("name,bits", [("clear_margin_4b.json", 4), ("clear_margin_4b_q8.json", 8),
                                       ("clear_margin_4b_bf16.json", 16)])
def test_dense_fixture_decides_every_token_clearly(name, bits):
    fx = json.load(open(os.path.join(GOLDEN, name)))
    assert fx.get("bits", 4) == bits and fx["n_layers"] == 36
    assert len(fx["prompt"]) == 32 and len(fx["tokens"]) == 32 and len(fx["margins"]) == 32 and len(fx["envelope"]) == 32
    assert len(set(fx["tokens"])) == fx["distinct"] >= 4          # a continuation that moves
    assert fx["fp32_orders_agree"] is True                        # both fp32 summation orders pick these tokens
    assert fx["min_ratio"] >= fx["safety"] >= 2.0                 # every gap >= safety x what the orders change it by
    assert fx["min_margin_ulps"] >= 3.0
    assert min(fx["margins"]) == pytest.approx(fx["min_margin"])


def test_moe_fixture_varies_tokens_and_routes():
    fx = json.load(open(os.path.join(GOLDEN, "clear_margin_moe.json")))
    assert len(fx["tokens"]) == 32 and len(set(fx["tokens"])) >= 4
    routes = fx["routes"]                                          # [position][expert layer] -> sorted expert ids
    assert len(routes) == 63 and all(len(r) == 26 for r in routes) and all(len(e) == 6 for r in routes for e in r)
    for layer in range(26):
        sets = {tuple(routes[p][layer]) for p in range(63)}
        assert len(sets) >= 4, (layer, len(sets))                  # routes differ from step to step
    per_layer = [{tuple(routes[p][layer]) for p in range(63)} for layer in range(26)]
    assert len({frozenset(s) for s in per_layer}) >= 20            # and from layer to layer
    used = {e for r in routes for layer in r for e in layer}
    assert len(used) >= 40                                         # most of the 64 experts are read
