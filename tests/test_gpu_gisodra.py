"""Gisodra on the GPU against the plain implementation (``tests/plain_gisodra.py``) and the kernels' plain
twins: each new kernel alone, each mixer alone inside the engine, then whole models of several shapes
under every way of cutting requests into steps, with small pools so that pages and slots change hands,
in float32 (strict, and the same bits whatever the cut) and bfloat16."""

from __future__ import annotations

import copy
from typing import Dict, List

import pytest
import torch

import traces
from helpers import assert_close, make_runner, run_trace, save_model_folder
from plain_gisodra import (ODD_SIZES, ONLY_ATTENTION, ONLY_GLA, ONLY_LATENT, TRIO, WIDE_VALUES, plain_gisodra_forward,
                           plain_gisodra_greedy, plain_gisodra_weights)

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
CONFIGS = {"trio": TRIO, "wide_values": WIDE_VALUES, "only_attention": ONLY_ATTENTION, "only_gla": ONLY_GLA,
           "only_latent": ONLY_LATENT, "odd_sizes": ODD_SIZES}


def _tokens(config, lengths: Dict[str, int], seed: int) -> Dict[str, List[int]]:
    g = torch.Generator().manual_seed(seed)
    return {r: torch.randint(0, config["vocab"], (n,), generator=g).tolist() for r, n in lengths.items()}


def _close(got, want, dtype, what=""):
    tol = dict(rtol=2e-5, atol=2e-5) if dtype == torch.float32 else dict(rtol=2e-2, atol=2e-2)
    torch.testing.assert_close(got.float().cpu(), want.float().cpu(), msg=lambda m: f"{what}: {m}", **tol)


# ------------------------------------------------------------------ kernels alone
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("T,D,S", [(5, 40, 0), (3, 200, 2), (17, 1000, 0), (2, 4104, 3)])
def test_post_add_rmsnorm_gelu_and_softcap_kernels(dtype, T, D, S):
    from fastgen_amd.kernels import ops, twins

    g = torch.Generator().manual_seed(T + D)
    h = torch.randn(T, D, generator=g)
    delta = torch.randn(S, T, D, generator=g) if S else torch.randn(T, D, generator=g).to(dtype)
    wp, w = (1 + 0.1 * torch.randn(D, generator=g)).to(dtype), (1 + 0.1 * torch.randn(D, generator=g)).to(dtype)
    rows = torch.tensor([T - 1, 0, T - 1], dtype=torch.int32)
    for use_rows, use_w in ((False, True), (True, True), (False, False)):
        hc, hg = h.clone(), h.clone().to(DEV)
        n = 3 if use_rows else T
        oc = torch.empty(n, D, dtype=dtype) if use_w else None
        og = torch.empty(n, D, dtype=dtype, device=DEV) if use_w else None
        twins.post_add_rmsnorm(hc, delta, wp, 1e-5, w if use_w else None, 1e-6, oc, rows if use_rows else None)
        ops.post_add_rmsnorm(hg, delta.to(DEV), wp.to(DEV), 1e-5, w.to(DEV) if use_w else None, 1e-6, og,
                             rows.to(DEV) if use_rows else None)
        torch.testing.assert_close(hg.cpu(), hc, rtol=1e-5, atol=1e-5)
        if use_w:
            _close(og, oc, dtype, "post_add_rmsnorm")
    F = 8 * ((D + 15) // 16)
    gu = torch.randn(T, 2 * F, generator=g).to(dtype)
    _close(ops.gelu_mul(gu.to(DEV)), twins.gelu_mul(gu), dtype, "gelu_mul")
    x = 20 * torch.randn(T, D, generator=g)
    torch.testing.assert_close(ops.softcap(x.clone().to(DEV), 9.0).cpu(), twins.softcap(x.clone(), 9.0), rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("M,N,K", [(3, 64, 64), (16, 96, 128), (40, 176, 72), (100, 128, 256), (300, 256, 128)])
def test_products_with_the_gelu_epilogue(M, N, K):
    """Every kernel that can take a gate/up product applies the tanh form of GELU where it stores."""
    from fastgen_amd.kernels import linear, ops, twins

    g = torch.Generator().manual_seed(M)
    x = torch.randn(M, K, generator=g).to(torch.bfloat16)
    w = (torch.randn(N, K, generator=g) / K ** 0.5).to(torch.bfloat16)
    want = twins.gemm_skinny(x, w, None, "gelu_tanh")
    xd, wd = x.to(DEV), w.to(DEV)
    if M <= 16:
        _close(ops.gemm_skinny(xd, wd, None, "gelu_tanh", wide=False), want, torch.bfloat16, "narrow")
    if M <= 128:
        _close(ops.gemm_skinny(xd, wd, None, "gelu_tanh", wide=True), want, torch.bfloat16, "wide")
        _close(ops.gemm_skinny(xd, ops.pack_weight(wd), None, "gelu_tanh", wide=True), want, torch.bfloat16, "wide packed")
    for tile_rows in ops.TILED_TILE_ROWS:
        _close(ops.gemm_tiled(xd, wd, None, "gelu_tanh", tile_rows=tile_rows), want, torch.bfloat16, "tiled")
    _close(linear.linear(xd, wd, epilogue="gelu_tanh_mul"), want, torch.bfloat16, "linear")
    _close(linear.linear(xd.float(), wd.float(), epilogue="gelu_tanh_mul"), twins.gelu_mul(x.float() @ w.float().T),
           torch.float32, "linear float32")


def _paged(T, n_kv, hc, P, dtype, seed):
    """Pages poisoned with NaN, a shuffled block table for one sequence of ``T`` tokens, and its slots."""
    n_pages = -(-T // P) + 2
    perm = torch.randperm(n_pages, generator=torch.Generator().manual_seed(seed))
    table = perm[: -(-T // P)].to(torch.int32)[None]
    slots = torch.tensor([int(table[0, t // P]) * P + t % P for t in range(T)], dtype=torch.int32)
    kp = torch.full((n_pages, n_kv, P, hc), float("nan"), dtype=dtype)
    vp = torch.full((n_pages, n_kv, hc, P), float("nan"), dtype=dtype)
    return kp, vp, table, slots


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,G,d,e,hc,rot,P", [(4, 2, 6, 4, 8, 0, 8), (5, 1, 80, 48, 80, 0, 64), (2, 2, 16, 48, 48, 8, 16),
                                              (3, 1, 130, 130, 144, 64, 32)])
def test_heads_prepare_kernel(dtype, H, G, d, e, hc, rot, P):
    from fastgen_amd.kernels import ops, twins

    g = torch.Generator().manual_seed(H * d)
    T = 37
    for src_dtype in {torch.float32, dtype}:
        src = torch.randn(T, H * d + G * d + G * e + 2, generator=g).to(src_dtype)
        bias = torch.randn(src.shape[1], generator=g)
        qn, kn = 1 + 0.2 * torch.randn(d, generator=g), 1 + 0.2 * torch.randn(d, generator=g)
        table = twins.rope_table(torch.arange(5, 5 + T, dtype=torch.int32), torch.rand(rot // 2, generator=g)) if rot else None
        for from_key in (False, True):
            if from_key and e > d:
                continue
            kp, vp, _, slots = _paged(T, G, hc, P, dtype, 1)
            slots[3] = -1  # a token that writes nothing
            kw = dict(n_q=H, q_col=0, q_width=d, q_norm=qn, q_norm_dims=d - 2, q_out_width=hc, n_kv=G, k_col=H * d, k_width=d,
                      k_norm=kn, k_norm_dims=d - 2, v_col=-1 if from_key else H * d + G * d, v_width=e, rot_start=2,
                      rotary_dim=rot, rotate_q=True, rotate_k=True)
            qc = torch.full((T, H * hc), float("nan"), dtype=dtype)
            kc, vc = kp.clone(), vp.clone()
            twins.heads_prepare(src, bias, 1e-5, q_out=qc, table=table, slots=slots, k_pages=kc, v_pages=vc, **kw)
            qg = torch.full((T, H * hc), float("nan"), dtype=dtype, device=DEV)
            kg, vg = kp.to(DEV), vp.to(DEV)
            ops.heads_prepare(src.to(DEV), bias.to(DEV), 1e-5, q_out=qg, table=table.to(DEV) if rot else None,
                              slots=slots.to(DEV), k_pages=kg, v_pages=vg, q_norm=kw.pop("q_norm").to(DEV),
                              k_norm=kw.pop("k_norm").to(DEV), **kw)
            _close(qg, qc, dtype, "queries")
            for got, want in ((kg, kc), (vg, vc)):
                assert torch.equal(torch.isnan(got.cpu()), torch.isnan(want)), "another set of cache elements was written"
                _close(torch.nan_to_num(got), torch.nan_to_num(want), dtype, "pages")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("T,H,N,K,tail,pad", [(5, 3, 7, 6, 2, 3), (70, 6, 128, 32, 32, 0), (130, 2, 40, 136, 0, 8),
                                              (1, 16, 24, 48, 8, 0), (9, 1, 200, 1024, 0, 0)])
def test_head_linear_kernel(dtype, T, H, N, K, tail, pad):
    from fastgen_amd.kernels import ops, twins

    g = torch.Generator().manual_seed(T + N)
    xs, ys = K + tail + (8 if K % 8 == 0 else 1), N + tail + pad
    x = torch.randn(T, H * xs + 8, generator=g).to(dtype)
    w = (torch.randn(H, N, K, generator=g) / K ** 0.5).to(dtype)
    gate = torch.randn(T, H + 3, generator=g)
    for use_gate in (False, True):
        yc = torch.full((T, H * ys), float("nan"), dtype=dtype)
        yg = yc.to(DEV)
        twins.head_linear(x, xs, w, yc, ys, tail, gate if use_gate else None)
        ops.head_linear(x.to(DEV), xs, w.to(DEV), yg, ys, tail, gate.to(DEV) if use_gate else None)
        _close(yg, yc, dtype, "head_linear")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,d,e,lens", [(2, 6, 5, [5, 1, 8]), (4, 48, 32, [70, 1, 1, 33]), (1, 256, 24, [9]),
                                        (3, 20, 130, [2, 40]), (2, 64, 40, [300, 1, 520, 5, 128, 129]), (1, 384, 16, [21, 3])])
def test_decay_scan_and_head_norm_gate_kernels(dtype, H, d, e, lens):
    """The last case brings runs of hundreds of tokens: with the sequences' starts on the host the kernels scan
    them in chunks side by side, which must give the token-by-token result within rounding."""
    from fastgen_amd.kernels import ops, twins

    g = torch.Generator().manual_seed(d + e)
    T, B = sum(lens), len(lens)
    rows = torch.randn(T, 2 * H * d + 2 * H * e + 8, generator=g).to(dtype)
    z, zb = 2 * torch.randn(T, H * d + 4, generator=g), 1 + torch.randn(H * d, generator=g)
    state = torch.randn(B + 2, H, d, e, generator=g)
    slots = torch.randperm(B + 2, generator=g)[:B].to(torch.int32)
    q_start = torch.tensor([0] + torch.tensor(lens).cumsum(0).tolist(), dtype=torch.int32)
    oc, sc = torch.empty(T, H * e), state.clone()
    twins.decay_scan(rows, 0, H * d, 2 * H * d, z, zb, 4.0, d ** -0.5, sc, slots, q_start, B, oc)
    og, sg = torch.empty(T, H * e, device=DEV), state.to(DEV)
    ops.decay_scan(rows.to(DEV), 0, H * d, 2 * H * d, z.to(DEV), zb.to(DEV), 4.0, d ** -0.5, sg, slots.to(DEV),
                   q_start.to(DEV), B, og)
    torch.testing.assert_close(og.cpu(), oc, rtol=1e-4, atol=1e-4)
    torch.testing.assert_close(sg.cpu(), sc, rtol=1e-4, atol=1e-4)
    if max(lens) >= ops.SCAN_CHUNKED_FROM:
        og2, sg2 = torch.empty(T, H * e, device=DEV), state.to(DEV)
        ops.decay_scan(rows.to(DEV), 0, H * d, 2 * H * d, z.to(DEV), zb.to(DEV), 4.0, d ** -0.5, sg2, slots.to(DEV),
                       q_start.to(DEV), B, og2, q_start_host=q_start.numpy())
        assert not torch.equal(og2, og), "the chunked scan did not run"
        torch.testing.assert_close(og2.cpu(), oc, rtol=1e-4, atol=1e-4)
        torch.testing.assert_close(sg2.cpu(), sc, rtol=1e-4, atol=1e-4)
    wn = torch.rand(e, generator=g) + 0.5
    rc, rg = torch.empty(T, H * e, dtype=dtype), torch.empty(T, H * e, dtype=dtype, device=DEV)
    g_col = 2 * H * d + H * e
    twins.head_norm_gate(oc, wn, 1e-5, rows[:, g_col:], H, rc)
    ops.head_norm_gate(oc.to(DEV), wn.to(DEV), 1e-5, rows.to(DEV)[:, g_col:], H, rg)
    _close(rg, rc, dtype, "head_norm_gate")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,G,hd,P,window,n", [(4, 2, 16, 16, 9, 70), (5, 1, 80, 64, 110, 300), (2, 2, 48, 32, 33, 150),
                                               (12, 1, 176, 64, 56, 200), (3, 3, 24, 8, 0, 50)])
def test_attention_kernels_with_a_sink_and_a_window_edge_that_decides(dtype, H, G, hd, P, window, n):
    """Every attention kernel (general; on the matrix cores: prompt tiles, decode chunks and their merge) with
    sinks, against the twin.  One key just inside the window and one just outside it are made to score far
    above the rest for the last query, and one head's sink is made to outweigh all its scores: a window off
    by one, or a sink left out, would change the result by far more than the tolerance."""
    from fastgen_amd.kernels import ops, twins
    from fastgen_amd.cache.layout import pack_k, pack_v

    g = torch.Generator().manual_seed(n + hd)
    q = torch.randn(n, H * hd, generator=g)
    k, v = torch.randn(n, G, hd, generator=g), torch.randn(n, G, hd, generator=g)
    last = n - 1
    if window:
        inside, outside = last - window + 1, last - window
        for kv in range(G):
            k[inside, kv] = 10 * q[last].view(H, hd)[kv * (H // G)] / hd ** 0.5
            k[outside, kv] = 14 * q[last].view(H, hd)[kv * (H // G)] / hd ** 0.5
    sinks = torch.randn(H, generator=g)
    sinks[H - 1] = 25.0
    q, k, v = q.to(dtype), k.to(dtype), v.to(dtype)
    kp, vp, table, _ = _paged(n, G, hd, P, dtype, 3)
    pad = -n % P
    kn = torch.nn.functional.pad(k, (0, 0, 0, 0, 0, pad)).view(-1, P, G, hd).permute(0, 2, 1, 3)
    vn = torch.nn.functional.pad(v, (0, 0, 0, 0, 0, pad)).view(-1, P, G, hd).permute(0, 2, 1, 3)
    for i, page in enumerate(table[0].tolist()):
        kp[page], vp[page] = pack_k(kn[i]), pack_v(vn[i])
    seq, pos = torch.zeros(n, dtype=torch.int32), torch.arange(n, dtype=torch.int32)
    want = twins.paged_attention_general(q, torch.empty(n, H * hd, dtype=dtype), kp, vp, table, seq, pos, H, hd ** -0.5,
                                         window, sinks)
    if window:  # the test's keys do decide
        for w_off in (window - 1, window + 1):
            other = twins.paged_attention_general(q[last:], torch.empty(1, H * hd, dtype=dtype), kp, vp, table, seq[last:],
                                                  pos[last:], H, hd ** -0.5, w_off, sinks)
            assert float((other.float() - want[last:].float())[:, :hd].abs().max()) > 0.3  # the first head follows the marked key
    assert float(want.float()[:, (H - 1) * hd :].abs().max()) < 1e-3  # the heavy sink takes all the weight
    dev = lambda t: t.to(DEV)
    got = ops.paged_attention_general(dev(q), torch.empty(n, H * hd, dtype=dtype, device=DEV), dev(kp), dev(vp), dev(table),
                                      dev(seq), dev(pos), H, hd ** -0.5, window, dev(sinks))
    _close(got, want, dtype, "general")
    if dtype == torch.bfloat16 and hd % 16 == 0:
        for exact in (False, True):
            tile_rows = ops.attention_tile_rows(hd, False, exact)
            # the prompt's first part as tiles, its last tokens as single decoded ones (chunks and their merge)
            head = n - 5
            per_tile = max(1, tile_rows // (H // G))
            big = [(0, i, min(per_tile, head - i), i) for i in range(0, head, per_tile)]
            small = [(0, t, 1, t) for t in range(head, n)]
            items = torch.tensor(small + big, dtype=torch.int32).reshape(-1).to(DEV)
            out = torch.empty(n, H * hd, dtype=dtype, device=DEV)
            ops.paged_attention_mfma(dev(q), out, dev(kp), dev(vp), dev(table), items[: 4 * len(small)], items[4 * len(small):],
                                     H, hd ** -0.5, window, min_tiles=1, max_rows=H // G, tile_rows=tile_rows,
                                     exact_weights=exact, sinks=dev(sinks))
            _close(out, want, dtype, f"matrix cores, exact={exact}")


# ----------------------------------------------------------------- whole models
LENGTHS = {"a": 150, "b": 37, "c": 2, "d": 1, "e": 70, "f": 19}


@pytest.fixture(scope="module")
def cases(tmp_path_factory):
    out = {}
    for name, config in CONFIGS.items():
        weights = plain_gisodra_weights(config, seed=len(name))
        folder = save_model_folder(tmp_path_factory.mktemp(name), config, weights)
        toks = _tokens(config, LENGTHS, seed=7)
        out[name] = (config, weights, folder, toks, {r: plain_gisodra_forward(weights, config, t) for r, t in toks.items()})
    return out


@pytest.fixture(scope="module")
def exact(cases):
    """The float64 runs of the same requests: what float32 results are measured against where sums are long."""
    return {name: {r: plain_gisodra_forward(c[1], c[0], t, torch.float64) for r, t in c[3].items()} for name, c in cases.items()}


def _all_traces(lengths):
    return {"whole": traces.whole(lengths), "tail": traces.tail(lengths, 60), "chunks": traces.chunks(lengths),
            "mixed": traces.mixed(lengths, seed=3), "mixed2": traces.mixed(lengths, max_live=3, seed=11, budget=23)}


@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_float32_every_cut_batch_and_reuse(cases, exact, name):
    """Whole prompts, prompts then single tokens (windows pass over decoded tokens), portions down to two
    tokens and one, mixed batches of unequal requests: the same logits as the plain run, and the same bits
    whatever the cut.  Pages of 16 tokens and a pool that holds the live requests only: pages and state
    slots are used again."""
    config, weights, folder, toks, want = cases[name]
    runner = make_runner(folder, torch.float32, page_size=16, max_tokens=304, max_requests=4)
    first = None
    for kind, tr in _all_traces(LENGTHS).items():
        got = run_trace(runner, tr, toks)
        assert_close(got, exact[name], torch.float32, want, f"gisodra {name} {kind}")  # three times the plain run's error
        if first is None:
            first = got
        else:
            for r in got:
                assert torch.equal(got[r], first[r]), f"{name} {kind}: request {r} depends on the cut"
        assert all(runner.cache.free_pages(g) == 304 // 16 for g in range(runner.cache.n_groups))
        assert runner.cache.free_slots() == 4


@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_bfloat16_every_cut_batch_and_reuse(cases, name):
    config, weights, folder, toks, want = cases[name]
    noise = {r: plain_gisodra_forward(weights, config, t, torch.bfloat16) for r, t in toks.items()}
    runner = make_runner(folder, torch.bfloat16, page_size=16, max_tokens=304, max_requests=4)
    for kind, tr in _all_traces(LENGTHS).items():
        assert_close(run_trace(runner, tr, toks), want, torch.bfloat16, noise, f"gisodra {name} {kind} bfloat16")
    assert runner.use_graphs and runner.graphs, "decode steps of this model are recorded"


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_streams_after_every_layer(cases, dtype):
    """The residual stream after each layer, read from the engine by stopping the run order there."""
    import dataclasses

    from fastgen_amd.engine import Model, ModelRunner, StepEntry
    from fastgen_amd.kernels import ops
    from fastgen_amd.weights.source import SafetensorsSource

    config, weights, folder, toks, _ = cases["wide_values"]
    _, streams = plain_gisodra_forward(weights, config, toks["b"], dtype, return_layers=True)
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
        ops.post_add_rmsnorm(h, pending.rows, pending.weight, pending.eps, None, 0.0, None)
        want = streams[n_runs - 1]
        tol = 2e-5 if dtype == torch.float32 else 4e-2
        assert float((h.cpu() - want).abs().max()) <= tol * float(want.abs().max()), f"after {n_runs} layers"


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("name", ["trio", "only_gla"])
def test_long_decoding_across_pages_and_windows(cases, dtype, name):
    """A short prompt, then 190 tokens one by one over a dozen pages: every window passes over decoded tokens,
    windowed pages go back to the pool on the way, the recurrence runs 190 steps (bfloat16: recorded steps)."""
    config, weights, folder, _, _ = cases[name]
    toks = _tokens(config, {"z": 200}, seed=5)
    want = {"z": plain_gisodra_forward(weights, config, toks["z"])}
    runner = make_runner(folder, dtype, page_size=16, max_tokens=208, max_requests=2)
    got = run_trace(runner, traces.tail({"z": 200}, 190), toks)
    noise = {"z": plain_gisodra_forward(weights, config, toks["z"], torch.bfloat16)} if dtype == torch.bfloat16 else None
    assert_close(got, want, dtype, noise, f"gisodra {name} long decoding")


@pytest.mark.parametrize("name", ["trio", "only_gla", "odd_sizes"])
def test_long_prompts_whose_recurrence_is_scanned_in_chunks(cases, name):
    """Prompts of several hundred tokens in one step (the recurrence then runs chunk by chunk, side by side),
    in two steps and in small portions (token by token): the plain logits, in both precisions, and in float32
    the cuts agree within rounding."""
    config, weights, folder, _, _ = cases[name]
    lengths = {"p": 700, "q": 260, "r": 3}
    toks = _tokens(config, lengths, seed=13)
    want = {r: plain_gisodra_forward(weights, config, t) for r, t in toks.items()}
    exact = {r: plain_gisodra_forward(weights, config, t, torch.float64) for r, t in toks.items()}
    noise = {r: plain_gisodra_forward(weights, config, t, torch.bfloat16) for r, t in toks.items()}
    together = [([("p", 0, 700), ("q", 0, 260), ("r", 0, 3)], ["p", "q", "r"])]
    for dtype in (torch.float32, torch.bfloat16):
        runner = make_runner(folder, dtype, page_size=16, max_tokens=1024, max_requests=3)
        for kind, tr in (("whole", traces.whole(lengths)), ("together", together),
                         ("halves", traces.chunks(lengths, sizes=(390, 310))), ("portions", traces.chunks(lengths))):
            got = run_trace(runner, tr, toks)
            if dtype == torch.float32:
                assert_close(got, exact, dtype, want, f"gisodra {name} long {kind}")
            else:
                assert_close(got, want, dtype, noise, f"gisodra {name} long {kind} bfloat16")


def test_the_recurrence_remembers_a_far_token(tmp_path):
    """With a decay close to one the state carries a token for hundreds of steps: the logits at the end follow a
    token 300 positions back, in a prompt, in portions and decoded alone, and through a slot that another
    request held before; losing the state (or starting from another request's) would change them by far more
    than the tolerance."""
    config = copy.deepcopy(ONLY_GLA)
    w = plain_gisodra_weights(config, 3)
    w["l0.mix.a2.b"] += 6.0  # sigmoid(8)^(1/16): a decay of 0.99998 a step
    # token 1 is the far token, token 2 asks for it: only token 1's embedding has the component that the key
    # projection reads, only token 2's the one that the query projection reads, so the state holds token 1's
    # value alone and only token 2 reads it
    w["embed"][:, :2] = 0.0
    w["embed"][1, 1] = 4.0
    w["embed"][2, 0] = 4.0
    w["l0.mix.q"][:, 1:] = 0.0
    w["l0.mix.q"][:, 0] = 1.0
    w["l0.mix.k"][:] = 0.0
    w["l0.mix.k"][:, 1] = 1.0
    n = 330
    toks = {r: [3 + t % (config["vocab"] - 3) for t in ts] for r, ts in _tokens(config, {"s": n, "other": 50}, seed=2).items()}
    toks["s"][20], toks["s"][-1], toks["other"][5], toks["other"][-1] = 1, 2, 1, 2
    want = {r: plain_gisodra_forward(w, config, t) for r, t in toks.items()}
    without = list(toks["s"])
    without[20] = (without[20] + 1) % config["vocab"]
    gap = float((plain_gisodra_forward(w, config, without)[-1] - want["s"][-1]).abs().max())
    assert gap > 0.02 * float(want["s"].abs().max()), "the test's weights do not make the far token count"
    folder = save_model_folder(tmp_path / "m", config, w)
    for dtype in (torch.float32, torch.bfloat16):
        runner = make_runner(folder, dtype, page_size=16, max_tokens=64, max_requests=1)  # one slot: it is used again
        for tr in (traces.whole({"other": 50, "s": n}), traces.tail({"other": 50, "s": n}, 25), traces.chunks({"other": 50, "s": n})):
            got = run_trace(runner, tr, toks)
            if dtype == torch.float32:
                assert_close(got, want, dtype, None, "far token")
            else:
                assert float((got["s"][-1] - want["s"][-1]).abs().max()) < 0.25 * gap


def test_window_edges_in_prompts_and_decoding(tmp_path):
    """One layer of attention whose marked keys score far above all others: a query sees the marked key at
    distance window - 1 and not the one at distance window, in a whole prompt, in portions that cut the
    window anywhere, decoded alone, and at page borders (windows of 9, 16 and 33 with pages of 16)."""
    for window in (9, 16, 33):
        config = copy.deepcopy(ONLY_ATTENTION)
        config["layers"][0]["mixer"]["mask"]["size"] = window
        w = plain_gisodra_weights(config, window)
        # token 1 marks a key, token 2 asks for it: only their embeddings have the component that the key (the
        # query) projection reads, so every other key and query is zero and the marked score, after the norms
        # per head the largest there can be, towers over the rest of its window and the sink
        w["embed"][:, :2] = 0.0
        for tok, col in ((1, 1), (2, 0)):
            w["embed"][tok] = 0.0
            w["embed"][tok, col] = 8.0
        for name in ("q", "k", "q.b", "k.b", "sink"):
            w[f"l0.mix.{name}"][:] = 0.0
        w["l0.mix.q"][:, 0] = 1.0
        w["l0.mix.k"][:, 1] = 1.0
        w["l0.mix.q.norm"][:] = 2.5
        w["l0.mix.k.norm"][:] = 2.5
        n = 200
        toks = torch.randint(3, config["vocab"], (n,), generator=torch.Generator().manual_seed(window)).tolist()
        queries = [39, 79, 119, 159, 199]  # farther apart than a window: each sees its own marked key or none
        sees, misses = queries[0::2], queries[1::2]
        for p in queries:
            toks[p] = 2
        for p in sees:
            toks[p - window + 1] = 1  # just inside
        for p in misses:
            toks[p - window] = 1      # just outside
        want = {"s": plain_gisodra_forward(w, config, toks)}
        for off, edge in ((-1, sees), (1, misses)):
            c2 = copy.deepcopy(config)
            c2["layers"][0]["mixer"]["mask"]["size"] = window + off
            moved = (plain_gisodra_forward(w, c2, toks) - want["s"]).abs().amax(-1)
            assert float(moved[edge].min()) > 0.2 * float(want["s"].abs().max()), "the marked keys do not decide"
        folder = save_model_folder(tmp_path / f"w{window}", config, w)
        for dtype in (torch.float32, torch.bfloat16):
            runner = make_runner(folder, dtype, page_size=16, max_tokens=208, max_requests=1)
            noise = {"s": plain_gisodra_forward(w, config, toks, torch.bfloat16)} if dtype == torch.bfloat16 else None
            for tr in (traces.whole({"s": n}), traces.tail({"s": n}, 130), traces.chunks({"s": n}),
                       traces.chunks({"s": n}, sizes=(2, 3, 2, 5))):
                assert_close(run_trace(runner, tr, {"s": toks}), want, dtype, noise, f"window {window}")


def test_greedy_generation_through_the_engine(cases):
    from fastgen_amd.engine import Engine
    from fastgen_amd.sampling import SamplingParams

    config, weights, folder, toks, _ = cases["trio"]
    prompts = [toks["b"], toks["f"], toks["c"], toks["e"][:40], toks["d"]]
    want = [plain_gisodra_greedy(weights, config, p, 9) for p in prompts]
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

    import numpy as np

    config, weights, folder, toks, want = cases["wide_values"]
    root = Path(__file__).resolve().parents[1]
    steps = [{"step": 0, "entries": [{"id": "x", "tokens": toks["b"][:20], "want": [19]}], "end": []},
             {"step": 1, "entries": [{"id": "x", "tokens": toks["b"][20:], "want": [0, 16]}], "end": ["x"]}]
    out = tmp_path / "out"
    run = subprocess.run([sys.executable, str(root / "bin" / "trace_run"), "--model", str(folder), "--dtype", "float32",
                          "--out", str(out), "--max-tokens", "64"], input="\n".join(json.dumps(s) for s in steps) + "\n",
                         capture_output=True, text=True, timeout=600)
    assert run.returncode == 0, run.stderr[-2000:]
    assert [l for l in run.stdout.splitlines() if l.startswith("done")] == ["done 0", "done 1"]
    got = np.fromfile(out / "1.f32", dtype="<f4").reshape(2, -1)
    assert np.abs(got - want["b"][[20, 36]].numpy()).max() <= 2e-5 * float(want["b"].abs().max())
    chat = subprocess.run([sys.executable, str(root / "bin" / "fgchat"), str(folder), "--prompt-ids", "1,2,3", "--max-tokens",
                           "5", "--temperature", "0"], capture_output=True, text=True, timeout=600)
    assert chat.returncode == 0, chat.stderr[-2000:]
