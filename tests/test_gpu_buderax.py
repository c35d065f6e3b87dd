"""Buderax on the GPU against the plain implementation (``tests/plain_buderax.py``): each new
mechanism alone, then whole models of several shapes under every way of cutting requests into steps,
with small pools so that pages and slots change hands, in float32 (strict) and bfloat16."""

from __future__ import annotations

from typing import Dict, List

import pytest
import torch

import traces
from helpers import assert_close, make_runner, run_trace, save_model_folder
from plain_buderax import (ALL_LOOP, ONE_PASS, PLAIN_STACK, SMALL_LOOP, plain_buderax_forward, plain_buderax_greedy,
                           plain_buderax_weights, plain_mixture, plain_route, plain_scaled_embedding,
                           plain_zero_centred_rmsnorm)

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
CONFIGS = {"small_loop": SMALL_LOOP, "plain_stack": PLAIN_STACK, "all_loop": ALL_LOOP, "one_pass": ONE_PASS}


def _tokens(config, lengths: Dict[str, int], seed: int) -> Dict[str, List[int]]:
    g = torch.Generator().manual_seed(seed)
    return {r: torch.randint(0, config["vocab"], (n,), generator=g).tolist() for r, n in lengths.items()}


def _mostly_close(got, want, noise, what):
    """bfloat16: a routing decision that lies within rounding of a tie may fall the other way than in the
    plain bfloat16 run, and the positions that read that token then differ by more than rounding.  Nine in
    ten positions of a request keep to the tolerance of ``assert_close`` (twice the plain bfloat16 run's
    worst error), none is off by more than a routing decision can explain, and all are finite."""
    for rid, w in want.items():
        g = got[rid]
        assert g.shape == w.shape and torch.isfinite(g).all(), f"{what} {rid}"
        err = (g - w).abs().amax(-1)
        tol = 2.0 * float((noise[rid] - w).abs().max()) + 1e-3 * float(w.abs().max())
        assert float((err <= tol).float().mean()) >= 0.9, f"{what} {rid}: {(err > tol).nonzero().flatten().tolist()} over {tol:.3e}"
        assert float(err.max()) <= 0.5 * float(w.abs().max()), f"{what} {rid}: {float(err.max()):.3e}"


# ------------------------------------------------------------ mechanisms alone
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_embedding_scale_offset_norm_and_stream_additions(dtype):
    from fastgen_amd.config import PartSpec
    from fastgen_amd.kernels import ops
    from fastgen_amd.parts import build_part

    g = torch.Generator().manual_seed(0)
    V, D, T = 37, 72, 9
    table = (torch.randn(V, D, generator=g)).to(torch.bfloat16).float()
    tok = torch.randint(0, V, (T,), generator=g)
    emb = build_part("embedding", PartSpec("embedding", "embed", dict(vocab_size=V, dim=D, scale=3.5, names={"weight": ""})))
    emb.load({"embed": table}, dtype, DEV)
    h = emb.forward(tok.to(DEV, torch.int32))
    want = plain_scaled_embedding(table, tok, 3.5)
    torch.testing.assert_close(h.cpu(), want, rtol=0, atol=0)
    # the norm's weight is stored around zero
    w = (torch.randn(D, generator=g) * 0.3).to(torch.bfloat16).float()
    norm = build_part("norm", PartSpec("rmsnorm", "n", dict(dim=D, eps=1e-5, unit_offset=True, names={"weight": ""})))
    norm.load({"n": w}, dtype, DEV)
    delta = torch.randn(T, D, generator=g).to(dtype)
    out = norm.forward(h, delta.to(DEV), dtype)
    want_h = want + delta.float()
    torch.testing.assert_close(h.cpu(), want_h, rtol=1e-6, atol=1e-6)
    tol = dict(rtol=1e-5, atol=1e-5) if dtype == torch.float32 else dict(rtol=1e-2, atol=1e-2)
    torch.testing.assert_close(out.float().cpu(), plain_zero_centred_rmsnorm(want_h, w, 1e-5), **tol)
    # what enters the stream at the start of a pass: what was left to add, the embedding again, the pass's vector
    step = torch.randn(3, D, generator=g)
    loop = build_part("injection", PartSpec("loop_input", "loop", dict(dim=D, times=3)))
    loop.load({"loop.step": step}, dtype, DEV)
    parts = torch.randn(2, T, D, generator=g)
    for index, pending in ((0, None), (2, delta.to(DEV)), (1, parts.to(DEV))):
        hh = want_h.clone().to(DEV)
        loop.forward(hh, pending, want.to(DEV), index)
        ref = want_h.clone()
        if pending is not None:
            ref = ref + (delta.float() if pending.dim() == 2 else parts[0] + parts[1])
        if index > 0:
            ref = ref + want
        torch.testing.assert_close(hh.cpu(), ref + step[index], rtol=1e-6, atol=1e-5)
    # the gate on the heads' outputs, from columns of a wider tensor
    x, wide = torch.randn(T, 48, generator=g).to(dtype), torch.randn(T, 80, generator=g).to(dtype)
    xd = x.to(DEV)
    ops.gate_mul(xd, wide.to(DEV)[:, 32:])
    torch.testing.assert_close(xd.float().cpu(), (x.float() * torch.sigmoid(wide[:, 32:].float())).to(dtype).float(), **tol)
    a, b = torch.randn(T, D, generator=g).to(dtype), torch.randn(T, D, generator=g).to(dtype)
    torch.testing.assert_close(ops.add_rows(a.to(DEV), b.to(DEV)).cpu()[0], a.float() + b.float(), rtol=1e-6, atol=1e-6)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("D,E,top,F,T", [(64, 5, 2, 24, 70), (96, 4, 1, 20, 7), (40, 6, 6, 16, 33), (128, 3, 2, 64, 300),
                                         (64, 70, 3, 8, 1), (72, 4, 2, 44, 230), (64, 2, 1, 40, 90), (48, 3, 2, 20, 400)])
def test_routed_experts_alone(dtype, D, E, top, F, T):
    """Router, sort, the experts' products and the weighted sum against the plain mixture: few rows (tiles of
    16) and many rows an expert (larger tiles, and those that go through LDS), all experts chosen, one
    chosen, more experts than a wave has lanes, widths that are no multiple of 8 or of 32."""
    from fastgen_amd.config import PartSpec
    from fastgen_amd.kernels import ops
    from fastgen_amd.parts import build_part

    config = {"width": D, "vocab": 8, "layers": [{"mixer": dict(heads=1, kv_heads=1, dim=8, vdim=8),
                                                   "mlp": {"router": {"experts": E, "top": top}, "expert": {"ff": F}}}]}
    w = plain_buderax_weights(config, D + E)
    g = torch.Generator().manual_seed(T)
    n = torch.randn(T, D, generator=g).to(torch.bfloat16).float()
    plus = torch.randn(T, D, generator=g).to(torch.bfloat16).float()
    part = build_part("feed_forward", PartSpec("moe", "l0.mlp", dict(
        dim=D, hidden_dim=F, n_experts=E, top=top,
        names={"router.weight": "router", "router.bias": "router.b", "expert": "e{}", "gate_proj.weight": "gate",
               "up_proj.weight": "up", "down_proj.weight": "down"})))
    part.load(w, dtype, DEV)
    choice, weight = ops.moe_route(n.to(DEV, dtype), part.router, part.bias, top)
    idx, wt = plain_route(n, w["l0.mlp.router"], w["l0.mlp.router.b"], top)
    assert torch.equal(choice.cpu().long(), idx)
    torch.testing.assert_close(weight.cpu(), wt, rtol=1e-5, atol=1e-6)
    got = part.forward(n.to(DEV, dtype), plus=plus.to(DEV, dtype)).cpu()[0]
    want = plain_mixture(n, w, "l0.mlp", config["layers"][0]["mlp"]) + plus
    if dtype == torch.float32:
        torch.testing.assert_close(got, want, rtol=2e-5, atol=2e-5)
    else:
        low = plain_mixture(n.to(dtype), {k: v.to(dtype) for k, v in w.items()}, "l0.mlp", config["layers"][0]["mlp"]) + plus
        assert float((got - want).abs().max()) <= 2.0 * float((low - want).abs().max()) + 1e-3 * float(want.abs().max())
    alone = part.forward(n.to(DEV, dtype)).cpu()[0]
    torch.testing.assert_close(alone + plus, got, rtol=1e-5, atol=1e-5)


# ----------------------------------------------------------------- whole models
LENGTHS = {"a": 150, "b": 37, "c": 2, "d": 1, "e": 70, "f": 19}


@pytest.fixture(scope="module")
def cases(tmp_path_factory):
    out = {}
    for name, config in CONFIGS.items():
        weights = plain_buderax_weights(config, seed=len(name), sharpen=5.0)
        folder = save_model_folder(tmp_path_factory.mktemp(name), config, weights)
        toks = _tokens(config, LENGTHS, seed=7)
        out[name] = (config, weights, folder, toks, {r: plain_buderax_forward(weights, config, t) for r, t in toks.items()})
    return out


def _all_traces(lengths):
    return {"whole": traces.whole(lengths), "tail": traces.tail(lengths, 40), "chunks": traces.chunks(lengths),
            "mixed": traces.mixed(lengths, seed=3), "mixed2": traces.mixed(lengths, max_live=3, seed=11, budget=23)}


@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_float32_every_cut_batch_and_reuse(cases, name):
    """Whole prompts, prompts then single tokens, portions down to two tokens and one, mixed batches of
    unequal requests: the same logits as the plain run, and the same bits whatever the cut.  Pages of 16
    tokens and a pool that holds the live requests only: pages and slots are used again."""
    config, weights, folder, toks, want = cases[name]
    runner = make_runner(folder, torch.float32, page_size=16, max_tokens=304, max_requests=4)
    first = None
    for kind, tr in _all_traces(LENGTHS).items():
        got = run_trace(runner, tr, toks)
        assert_close(got, want, torch.float32, None, f"buderax {name} {kind}")
        if first is None:
            first = got
        else:
            for r in got:
                assert torch.equal(got[r], first[r]), f"{name} {kind}: request {r} depends on the cut"
        assert runner.cache.free_pages() == 304 // 16 and runner.cache.free_slots() == 4


@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_bfloat16_every_cut_batch_and_reuse(cases, name):
    config, weights, folder, toks, want = cases[name]
    noise = {r: plain_buderax_forward(weights, config, t, torch.bfloat16) for r, t in toks.items()}
    runner = make_runner(folder, torch.bfloat16, page_size=16, max_tokens=304, max_requests=4)
    for kind, tr in _all_traces(LENGTHS).items():
        _mostly_close(run_trace(runner, tr, toks), want, noise, f"buderax {name} {kind} bfloat16")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_streams_after_every_layer_run(cases, dtype):
    """The residual stream after each run of a layer (a looped layer counts each time), read from the
    engine by stopping the run order there."""
    import dataclasses

    from fastgen_amd.engine import Model, ModelRunner, StepEntry
    from fastgen_amd.weights.source import SafetensorsSource

    config, weights, folder, toks, _ = cases["small_loop"]
    streams: list = []
    plain_buderax_forward(weights, config, toks["b"], dtype, streams=streams)
    full = Model.from_folder(folder, dtype, DEV)
    for n_runs in range(1, len(full.layout.order) + 1):
        layout = dataclasses.replace(full.layout, order=full.layout.order[:n_runs])
        model = Model(layout, dtype, DEV, args=full.args, architecture=full.architecture)
        model.load(SafetensorsSource(folder))
        seen = {}
        norm = model.parts.final_norm
        keep = norm.forward
        norm.forward = lambda h, pending, dt, rows=None: (seen.update(h=h.clone(), pending=pending), keep(h, pending, dt, rows))[1]
        runner = ModelRunner(model, page_size=16, max_tokens=64, max_requests=1)
        runner.step([StepEntry("b", toks["b"], [0])])
        h, pending = seen["h"], seen["pending"]
        h = h + (pending.sum(0) if pending.dim() == 3 else pending.float())
        want = streams[n_runs - 1]
        tol = 2e-5 if dtype == torch.float32 else 4e-2
        assert float((h.cpu() - want).abs().max()) <= tol * float(want.abs().max()), f"after {n_runs} layer runs"


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_long_decoding_across_pages(cases, dtype):
    """A short prompt, then 140 tokens one by one over nine pages (bfloat16: from recorded steps)."""
    config, weights, folder, _, _ = cases["one_pass"]
    toks = _tokens(config, {"z": 150}, seed=5)
    want = {"z": plain_buderax_forward(weights, config, toks["z"])}
    runner = make_runner(folder, dtype, page_size=16, max_tokens=160, max_requests=2)
    got = run_trace(runner, traces.tail({"z": 150}, 140), toks)
    if dtype == torch.float32:
        assert_close(got, want, dtype, None, "buderax long decoding")
    else:
        _mostly_close(got, want, {"z": plain_buderax_forward(weights, config, toks["z"], torch.bfloat16)}, "long decoding")
        assert runner.use_graphs and runner.graphs, "decode steps of this model are recorded"


def test_a_far_key_decides(tmp_path):
    """One query and one key, hundreds of tokens apart and on different pages, are scaled so that their
    score stands out: the logits at the query follow that key's value, in a prompt, in portions and
    decoded alone; losing the key would change them by far more than the tolerance."""
    config = {"architecture": "Buderax", "width": 32, "vocab": 50, "embedding": {"scale": 1.0}, "norm": {"eps": 1e-6},
              "layers": [{"type": "attention", "mlp": None,
                          "mixer": {"heads": 2, "kv_heads": 1, "dim": 16, "vdim": 16, "scale": 0.25,
                                    "rot": {"base": 10000.0, "dims": 4, "scaling": {"factor": 2.0}}}}]}
    w = plain_buderax_weights(config, 9)
    # token 1 is the far key, token 2 the query.  The key's embedding has one large component, which only
    # the key projection reads, the query's another, which only the query projection reads, both into the
    # head dimensions that are not rotated: their score towers over all others, the query's own included
    w["embed"][1] = 0.0
    w["embed"][1, 1] = 6.0
    w["embed"][2] = 0.0
    w["embed"][2, 0] = 6.0
    w["l0.norm1"][:] = 0.0
    w["l0.mix.q"][:, :2] = 0.0
    w["l0.mix.k"][:, :2] = 0.0
    w["l0.mix.q"][4:16, 0] = 3.0
    w["l0.mix.q"][20:32, 0] = 3.0
    w["l0.mix.k"][4:16, 1] = 3.0
    n = 420
    toks = torch.randint(3, 50, (n,), generator=torch.Generator().manual_seed(2)).tolist()
    toks[33] = 1          # just behind a page's edge (pages of 16 tokens)
    toks[400] = toks[419] = 2
    want = {"s": plain_buderax_forward(w, config, toks)}
    without = list(toks)
    without[33] = 7
    gap = float((plain_buderax_forward(w, config, without)[400] - want["s"][400]).abs().max())
    assert gap > 0.05 * float(want["s"].abs().max()), "the test's weights do not make the far key count"
    folder = save_model_folder(tmp_path / "m", config, w)
    for dtype in (torch.float32, torch.bfloat16):
        runner = make_runner(folder, dtype, page_size=16, max_tokens=432, max_requests=1)
        for tr in (traces.whole({"s": n}), traces.tail({"s": n}, 25), traces.chunks({"s": n})):
            got = run_trace(runner, tr, {"s": toks})
            if dtype == torch.float32:
                assert_close(got, want, dtype, None, "far key")
            else:
                assert float((got["s"] - want["s"]).abs().max()) < 0.2 * gap


def test_greedy_generation_through_the_engine(cases):
    from fastgen_amd.engine import Engine
    from fastgen_amd.sampling import SamplingParams

    config, weights, folder, toks, _ = cases["small_loop"]
    prompts = [toks["b"], toks["f"], toks["c"], toks["e"][:40], toks["d"]]
    want = [plain_buderax_greedy(weights, config, p, 9) for p in prompts]
    engine = Engine.from_folder(folder, torch.float32, DEV, page_size=16, max_tokens=320, max_batch=3, max_step_tokens=24)
    assert engine.generate(prompts, SamplingParams(temperature=0.0, max_new_tokens=9)) == want
    low = Engine.from_folder(folder, torch.bfloat16, DEV, page_size=16, max_tokens=320, max_batch=3, max_step_tokens=24)
    got = low.generate(prompts, SamplingParams(temperature=0.0, max_new_tokens=9))
    assert [len(g) for g in got] == [9] * len(prompts)


def test_command_lines(cases, tmp_path):
    """The trace runner and the chat tool take the model by its folder, as they take any other."""
    import json
    import subprocess
    import sys
    from pathlib import Path

    config, weights, folder, toks, want = cases["plain_stack"]
    root = Path(__file__).resolve().parents[1]
    steps = [{"step": 0, "entries": [{"id": "x", "tokens": toks["b"][:20], "want": [19]}], "end": []},
             {"step": 1, "entries": [{"id": "x", "tokens": toks["b"][20:], "want": [0, 16]}], "end": ["x"]}]
    out = tmp_path / "out"
    run = subprocess.run([sys.executable, str(root / "bin" / "trace_run"), "--model", str(folder), "--dtype", "float32",
                          "--out", str(out), "--max-tokens", "64"], input="\n".join(json.dumps(s) for s in steps) + "\n",
                         capture_output=True, text=True, timeout=600)
    assert run.returncode == 0, run.stderr[-2000:]
    assert [l for l in run.stdout.splitlines() if l.startswith("done")] == ["done 0", "done 1"]
    import numpy as np
    got = np.fromfile(out / "1.f32", dtype="<f4").reshape(2, -1)
    assert np.abs(got - want["b"][[20, 36]].numpy()).max() <= 2e-5 * float(want["b"].abs().max())
    chat = subprocess.run([sys.executable, str(root / "bin" / "fgchat"), str(folder), "--prompt-ids", "1,2,3", "--max-tokens",
                           "5", "--temperature", "0"], capture_output=True, text=True, timeout=600)
    assert chat.returncode == 0, chat.stderr[-2000:]
