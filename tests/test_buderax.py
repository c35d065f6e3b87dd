"""Buderax without a GPU: the configuration reader, the layout it makes, the plain implementation's
own properties, and the plain PyTorch twins of the new kernels against the plain implementation."""

from __future__ import annotations

import copy

import pytest
import torch

from fastgen_amd.config import ConfigError, get_architecture
from fastgen_amd.engine.model import build_parts
from fastgen_amd.kernels import twins

from plain_buderax import (ALL_LOOP, ONE_PASS, PLAIN_STACK, SMALL_LOOP, plain_buderax_forward, plain_buderax_weights,
                           plain_causal_attention, plain_expert, plain_linear_frequencies, plain_mixture, plain_rotate_pairs,
                           plain_route, plain_run_order, plain_zero_centred_rmsnorm)

CONFIGS = {"small_loop": SMALL_LOOP, "plain_stack": PLAIN_STACK, "all_loop": ALL_LOOP, "one_pass": ONE_PASS}


@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_configuration_round_trip_and_tensor_names(name):
    config = CONFIGS[name]
    arch = get_architecture(config)
    assert arch.name == "Buderax"
    args = arch.parse(config)
    assert arch.parse(arch.to_hf_config(args)) == args
    layout = arch.layout(args)
    specs = {s.name: tuple(s.shape) for s in build_parts(layout).tensor_specs()}
    weights = plain_buderax_weights(config, 0)
    assert specs == {k: tuple(v.shape) for k, v in weights.items()}
    # the run order is the plain one, and a pass begins where the plain order says
    assert [(e.layer, e.inject[1] if e.inject else None) for e in layout.order] == plain_run_order(
        len(config["layers"]), config.get("loop"))


def test_configuration_errors_name_the_key():
    for path, value, word in [(("layers", 0, "mixer", "kv_heads"), 3, "kv_heads"), (("layers", 0, "mixer", "vdim"), 8, "vdim"),
                              (("layers", 0, "mlp", "router", "top"), 9, "top"), (("loop", "stop"), 7, "loop"),
                              (("layers", 0, "type"), "other", "type"), (("layers", 0, "mlp", "kind"), "dense", "kind")]:
        config = copy.deepcopy(SMALL_LOOP)
        node = config
        for key in path[:-1]:
            node = node[key]
        node[path[-1]] = value
        with pytest.raises(ConfigError, match=word):
            get_architecture(config).parse(config)
    config = copy.deepcopy(SMALL_LOOP)
    del config["norm"]
    with pytest.raises(ConfigError, match="norm.eps"):
        get_architecture(config).parse(config)


def test_plain_model_is_causal_and_its_streams_add_up():
    w = plain_buderax_weights(SMALL_LOOP, 3, sharpen=4.0)
    toks = torch.randint(0, SMALL_LOOP["vocab"], (40,), generator=torch.Generator().manual_seed(1)).tolist()
    streams = []
    full = plain_buderax_forward(w, SMALL_LOOP, toks, streams=streams)
    assert len(streams) == len(plain_run_order(3, SMALL_LOOP["loop"])) == 5
    assert torch.equal(full[:25], plain_buderax_forward(w, SMALL_LOOP, toks[:25]))
    other = toks[:30] + [(t + 1) % SMALL_LOOP["vocab"] for t in toks[30:]]
    assert torch.equal(full[:30], plain_buderax_forward(w, SMALL_LOOP, other)[:30])
    assert not torch.allclose(full[30:], plain_buderax_forward(w, SMALL_LOOP, other)[30:])


def test_plain_rotation_scores_depend_on_the_distance_only():
    f = plain_linear_frequencies(8, 100.0, 4.0)
    assert torch.allclose(f, torch.tensor([1.0, 100 ** -0.25, 100 ** -0.5, 100 ** -0.75]) / 4)
    g = torch.Generator().manual_seed(2)
    q, k = torch.randn(1, 1, 12, generator=g), torch.randn(1, 1, 12, generator=g)
    def score(i, j):
        return float((plain_rotate_pairs(q, torch.tensor([i]), f) * plain_rotate_pairs(k, torch.tensor([j]), f)).sum())
    assert abs(score(9, 4) - score(105, 100)) < 1e-4
    assert abs(score(9, 4) - score(9, 5)) > 1e-3
    # the dimensions behind the rotated ones pass unchanged
    assert torch.equal(plain_rotate_pairs(q, torch.tensor([7]), f)[..., 8:], q[..., 8:])


def test_plain_norm_router_and_attention_special_cases():
    x = torch.tensor([[3.0, 4.0]])
    assert torch.allclose(plain_zero_centred_rmsnorm(x, torch.zeros(2), 0.0), x / (12.5 ** 0.5))
    assert torch.allclose(plain_zero_centred_rmsnorm(x, torch.tensor([1.0, -1.0]), 0.0), torch.tensor([[6.0 / 12.5 ** 0.5, 0.0]]))
    idx, wt = plain_route(torch.eye(3), torch.tensor([[1.0, 0, 0], [0, 2.0, 0], [0, 0, 0.5], [0.9, 1.9, 0.4]]),
                          torch.zeros(4), 2)
    assert idx.tolist() == [[0, 3], [1, 3], [2, 3]]
    assert torch.allclose(wt.sum(-1), torch.ones(3)) and torch.allclose(wt[0, 0] / wt[0, 1], torch.exp(torch.tensor(0.1)))
    # one key: the output is its value; the values here are the keys before the rotation
    q, k = torch.randn(1, 2, 4), torch.randn(1, 1, 4)
    assert torch.allclose(plain_causal_attention(q, k, k, 0.3), k.expand(1, 2, 4))


def test_twins_of_the_routed_experts_are_the_plain_mixture():
    config = PLAIN_STACK
    w = plain_buderax_weights(config, 5)
    m = config["layers"][1]["mlp"]
    E, top = m["router"]["experts"], m["router"]["top"]
    n = torch.randn(19, config["width"], generator=torch.Generator().manual_seed(4))
    want = plain_mixture(n, w, "l1.mlp", m)
    choice, weight = twins.moe_route(n, w["l1.mlp.router"], w["l1.mlp.router.b"], top)
    idx, wt = plain_route(n, w["l1.mlp.router"], w["l1.mlp.router.b"], top)
    assert torch.equal(choice.long(), idx) and torch.allclose(weight, wt)
    stack = lambda which: torch.stack([w[f"l1.mlp.e{e}.{which}"] for e in range(E)])
    for tile_rows in (16, 32):
        sorted_, tiles = twins.moe_sort(choice, E, tile_rows)
        assert sorted(sorted_.tolist()) == list(range(19 * top)) and int(tiles[:, 2].sum()) == 19 * top
        act = twins.moe_gate_up(n, stack("gate"), stack("up"), sorted_, tiles, top, tile_rows)
        y = twins.moe_down(act, stack("down"), sorted_, tiles, tile_rows)
        plus = torch.randn(19, config["width"])
        got = twins.moe_combine(y, weight, plus)
        torch.testing.assert_close(got[0], want + plus, rtol=1e-5, atol=1e-5)
    assert torch.allclose(plain_expert(n[:1], w["l1.mlp.e0.gate"], w["l1.mlp.e0.up"], w["l1.mlp.e0.down"]),
                          (torch.nn.functional.silu(n[:1] @ w["l1.mlp.e0.gate"].T) * (n[:1] @ w["l1.mlp.e0.up"].T))
                          @ w["l1.mlp.e0.down"].T)
