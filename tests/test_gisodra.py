"""Gisodra without a GPU: its configuration reader and layout, the plain implementation's own
mechanisms against hand-made cases, and the kernels' plain twins against the plain mechanisms."""

from __future__ import annotations

import copy
import math

import pytest
import torch

from fastgen_amd.config import ConfigError, get_architecture
from fastgen_amd.engine.model import build_parts
from fastgen_amd.kernels import twins
from plain_gisodra import (ODD_SIZES, ONLY_ATTENTION, ONLY_GLA, ONLY_LATENT, TRIO, WIDE_VALUES, plain_decay, plain_decayed_state_scan,
                           plain_gelu_tanh, plain_gisodra_forward, plain_gisodra_shapes, plain_gisodra_weights,
                           plain_rms, plain_rotate_halves, plain_window_sink_attention)

CONFIGS = {"trio": TRIO, "wide_values": WIDE_VALUES, "only_attention": ONLY_ATTENTION, "only_gla": ONLY_GLA,
           "only_latent": ONLY_LATENT, "odd_sizes": ODD_SIZES}


# ------------------------------------------------------------------ configuration
@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_layout_names_every_tensor_and_the_configuration_round_trips(name):
    config = CONFIGS[name]
    arch = get_architecture(config)
    assert arch.name == "Gisodra"
    args = arch.parse(config)
    assert arch.parse(arch.to_hf_config(args)) == args
    specs = {s.name: tuple(s.shape) for s in build_parts(arch.layout(args)).tensor_specs()}
    assert specs == plain_gisodra_shapes(config)


def test_sizes_that_only_the_tensors_give():
    config = copy.deepcopy(ONLY_GLA)
    arch = get_architecture(config)
    assert arch.parse(config).layers[0].mixer.decay_rank == 16
    config["layers"][0]["mixer"]["decay_rank"] = 6
    assert arch.parse(config).layers[0].mixer.decay_rank == 6
    args = arch.parse(config, lambda name: (24, 48) if name == "l0.mix.a1" else None)  # the tensor's shape wins
    assert args.layers[0].mixer.decay_rank == 24
    specs = {s.name: tuple(s.shape) for s in build_parts(arch.layout(args)).tensor_specs()}
    assert specs["l0.mix.a1"] == (24, 48) and specs["l0.mix.a2"] == (2 * 24, 24)


def test_a_cache_keeps_keys_for_the_longest_window_that_reads_it():
    arch = get_architecture(TRIO)
    layout = arch.layout(arch.parse(TRIO))
    assert [e.reads_cache_of for e in layout.order] == [None, None, 0, None]
    own, reader = layout.layers[0].mixer.options, layout.layers[2].mixer.options
    assert (own["window"], own["cache_window"]) == (24, 40) and reader["window"] == 40 and not reader["has_kv"]
    parts = build_parts(layout)
    assert parts.mixers[0].paged_need().window == 40
    assert parts.mixers[1].state_need().shape == (2, 16, 32) and parts.mixers[1].paged_need() is None
    # keys of 32 and values of 16 share pages of one width; the latent's row is latent + rotated part, padded
    assert parts.mixers[0].paged_need().head_dim == 32 and parts.mixers[3].paged_need().head_dim == 64
    assert parts.mixers[3].paged_need().n_kv_heads == 1


@pytest.mark.parametrize("change,match", [
    (lambda c: c["layers"][0].update(type="conv"), "not supported"),
    (lambda c: c["layers"][2]["mixer"].update(kv_from=1), "earlier attention layer"),
    (lambda c: c["layers"][2]["mixer"].update(kv_from=2), "earlier attention layer"),
    (lambda c: c["layers"][2]["mixer"].update(dim=16), "must equal layer 0"),
    (lambda c: c["layers"][0]["mixer"].pop("scale"), "layers|scale"),
    (lambda c: c["layers"][0]["mixer"].update(heads=3), "multiple of kv_heads"),
    (lambda c: c["layers"][1]["mixer"].update(tau=0.0), "tau"),
    (lambda c: c["layers"][3]["mixer"]["rot"].update(dims=8), "rot.dims"),
    (lambda c: c["layers"][0]["mlp"].update(kind="moe"), "not supported"),
    (lambda c: c["norm"].pop("eps"), "norm.eps"),
    (lambda c: c.update(logit_softcap=-1.0), "logit_softcap"),
])
def test_configuration_errors_name_what_is_wrong(change, match):
    config = copy.deepcopy(TRIO)
    change(config)
    with pytest.raises(ConfigError, match=match):
        get_architecture(config).parse(config)


# ------------------------------------------------- the plain mechanisms on hand-made cases
def test_plain_norm_activation_and_decay():
    x = torch.tensor([[3.0, -4.0, 0.0, 0.0]])
    torch.testing.assert_close(plain_rms(x, torch.tensor([1.0, 2.0, 1.0, 1.0]), 0.0), torch.tensor([[1.2, -3.2, 0.0, 0.0]]))
    assert float(plain_rms(torch.zeros(1, 4), None, 1e-6).abs().max()) == 0.0  # eps is inside the root
    z = torch.tensor([-3.0, 0.0, 0.5, 4.0])
    torch.testing.assert_close(plain_gelu_tanh(z), torch.nn.functional.gelu(z, approximate="tanh"))
    torch.testing.assert_close(plain_decay(torch.tensor([0.0, 2.0]), 1.0), torch.sigmoid(torch.tensor([0.0, 2.0])))
    torch.testing.assert_close(plain_decay(torch.tensor([0.0]), 4.0), torch.tensor([0.5 ** 0.25]))


def test_plain_window_and_sink():
    T, d = 7, 4
    g = torch.Generator().manual_seed(1)
    q, k, v = torch.randn(T, 1, d, generator=g), torch.randn(T, 1, d, generator=g), torch.randn(T, 1, 3, generator=g)
    # window 1: every position sees itself only; without a sink its weight is 1
    torch.testing.assert_close(plain_window_sink_attention(q, k, v, 0.5, 1, None), v)
    # a sink as large as the one score halves the weight
    s = (q[:, 0] * k[:, 0]).sum(-1) * 0.5
    for t in range(T):
        got = plain_window_sink_attention(q[: t + 1], k[: t + 1], v[: t + 1], 0.5, 1, s[t].reshape(1))[t]
        torch.testing.assert_close(got, 0.5 * v[t])
    # window 3 against the definition, position by position
    sink = torch.tensor([0.3])
    got = plain_window_sink_attention(q, k, v, 0.7, 3, sink)
    for i in range(T):
        lo = max(0, i - 2)
        sc = (k[lo : i + 1, 0] @ q[i, 0]) * 0.7
        w = torch.exp(sc) / (torch.exp(sc).sum() + torch.exp(sink[0]))
        torch.testing.assert_close(got[i, 0], w @ v[lo : i + 1, 0])


def test_plain_rotation_pairs_halves_and_keeps_scores_relative():
    g = torch.Generator().manual_seed(2)
    x = torch.randn(5, 2, 12, generator=g)
    pos = torch.tensor([0, 1, 2, 50, 51])
    y = plain_rotate_halves(x, pos, 100.0, 8)
    torch.testing.assert_close(y[0], x[0])  # position 0 turns nothing
    torch.testing.assert_close(y[..., 8:], x[..., 8:])  # dimensions from `dims` on pass
    torch.testing.assert_close(y.norm(dim=-1), x.norm(dim=-1))
    a = 1.0 * 100.0 ** (-2.0 * 1 / 8)  # dimension 1 is paired with 1 + 4
    torch.testing.assert_close(y[1, 0, 1], x[1, 0, 1] * math.cos(a) - x[1, 0, 5] * math.sin(a))
    torch.testing.assert_close(y[1, 0, 5], x[1, 0, 5] * math.cos(a) + x[1, 0, 1] * math.sin(a))
    # a score depends on the distance only
    u, w = torch.randn(1, 1, 8, generator=g), torch.randn(1, 1, 8, generator=g)
    s1 = (plain_rotate_halves(u, torch.tensor([7]), 100.0, 8) * plain_rotate_halves(w, torch.tensor([3]), 100.0, 8)).sum()
    s2 = (plain_rotate_halves(u, torch.tensor([44]), 100.0, 8) * plain_rotate_halves(w, torch.tensor([40]), 100.0, 8)).sum()
    torch.testing.assert_close(s1, s2, rtol=1e-4, atol=1e-4)


def test_plain_scan_is_the_sum_it_stands_for_and_carries_its_state():
    g = torch.Generator().manual_seed(3)
    T, H, d, e = 9, 2, 3, 4
    q, k, v = torch.randn(T, H, d, generator=g), torch.randn(T, H, d, generator=g), torch.randn(T, H, e, generator=g)
    a = torch.rand(T, H, d, generator=g)
    o, S = plain_decayed_state_scan(q, k, v, a)
    for t in (0, 4, 8):
        want = torch.zeros(H, e)
        for s in range(t + 1):
            decay = a[s + 1 : t + 1].prod(0)  # [H, d]: every decay after s up to t
            want += torch.einsum("hd,hd,he->he", q[t] * decay, k[s], v[s])
        torch.testing.assert_close(o[t], want, rtol=1e-5, atol=1e-5)
    o1, S1 = plain_decayed_state_scan(q[:5], k[:5], v[:5], a[:5])
    o2, S2 = plain_decayed_state_scan(q[5:], k[5:], v[5:], a[5:], S1)
    torch.testing.assert_close(torch.cat([o1, o2]), o)
    torch.testing.assert_close(S2, S)


def test_every_mechanism_moves_the_logits():
    """The random weights of these tests are large enough that leaving a mechanism out shows."""
    toks = torch.randint(0, TRIO["vocab"], (70,), generator=torch.Generator().manual_seed(4)).tolist()
    w = plain_gisodra_weights(TRIO, 1)
    base = plain_gisodra_forward(w, TRIO, toks)
    scale = float(base.abs().max())

    def moved(change_w=None, change_c=None):
        w2, c2 = {k: v.clone() for k, v in w.items()}, copy.deepcopy(TRIO)
        if change_w:
            change_w(w2)
        if change_c:
            change_c(c2)
        return float((plain_gisodra_forward(w2, c2, toks) - base).abs().max()) / scale

    assert moved(lambda w2: w2["l0.mix.sink"].fill_(-30.0)) > 1e-3
    assert moved(lambda w2: w2["l3.mix.sink"].fill_(-30.0)) > 1e-3
    assert moved(lambda w2: w2["l0.mix.q.b"].zero_()) > 1e-3
    assert moved(lambda w2: w2["l0.mix.k.norm"].fill_(1.0)) > 1e-3
    assert moved(lambda w2: w2["l1.mix.a2.b"].add_(3.0)) > 1e-3
    assert moved(lambda w2: w2["l3.mix.g"].zero_()) > 1e-3
    assert moved(change_c=lambda c: c["layers"][0]["mixer"]["mask"].update(size=23)) > 1e-3
    assert moved(change_c=lambda c: c["layers"][2]["mixer"]["mask"].update(size=41)) > 1e-3
    assert moved(change_c=lambda c: c["layers"][3]["mixer"]["mask"].update(size=19)) > 1e-3
    assert moved(change_c=lambda c: c["layers"][3]["mixer"]["rot"].update(base=5000.0)) > 1e-4
    assert moved(change_c=lambda c: c["layers"][1]["mixer"].update(tau=4.0)) > 1e-3
    assert moved(change_c=lambda c: c.update(logit_softcap=200.0)) > 1e-3


# ------------------------------------------------- the kernels' twins against the plain mechanisms
def test_twins_of_the_row_kernels():
    g = torch.Generator().manual_seed(5)
    T, D = 6, 40
    h, delta = torch.randn(T, D, generator=g), torch.randn(T, D, generator=g)
    wp, w = 1 + 0.1 * torch.randn(D, generator=g), 1 + 0.1 * torch.randn(D, generator=g)
    want_h = h + plain_rms(delta, wp, 1e-5)
    out = torch.empty(T, D)
    hh = h.clone()
    twins.post_add_rmsnorm(hh, delta, wp, 1e-5, w, 1e-6, out)
    torch.testing.assert_close(hh, want_h)
    torch.testing.assert_close(out, plain_rms(want_h, w, 1e-6))
    rows = torch.tensor([4, 1, 4], dtype=torch.int32)
    hh, some = h.clone(), torch.empty(3, D)
    twins.post_add_rmsnorm(hh, delta, wp, 1e-5, w, 1e-6, some, rows)
    torch.testing.assert_close(hh, h)
    torch.testing.assert_close(some, plain_rms(want_h, w, 1e-6)[rows.long()])
    parts = torch.randn(3, T, D, generator=g)
    hh = h.clone()
    twins.post_add_rmsnorm(hh, parts, wp, 1e-5, None, 0.0, None)
    torch.testing.assert_close(hh, h + plain_rms(parts.sum(0), wp, 1e-5))
    gate, up = torch.randn(T, 16, generator=g), torch.randn(T, 16, generator=g)
    gu = twins.interleave_gate_up(gate.T.contiguous(), up.T.contiguous()).T.contiguous()
    torch.testing.assert_close(twins.gelu_mul(gu), plain_gelu_tanh(gate) * up)
    x = 30 * torch.randn(4, 9, generator=g)
    torch.testing.assert_close(twins.softcap(x.clone(), 7.0), 7.0 * torch.tanh(x / 7.0))


def test_twin_of_the_recurrence():
    g = torch.Generator().manual_seed(6)
    H, d, e, tau = 2, 6, 5, 4.0
    lens = [5, 1, 8]
    T = sum(lens)
    rows = torch.randn(T, 2 * H * d + H * e + 3, generator=g)
    z, zb = torch.randn(T, H * d, generator=g), torch.randn(H * d, generator=g)
    state = torch.randn(4, H, d, e, generator=g)
    start = state.clone()
    slots = torch.tensor([2, 0, 3], dtype=torch.int32)
    q_start = torch.tensor([0, 5, 6, 14], dtype=torch.int32)
    out = torch.empty(T, H * e)
    twins.decay_scan(rows, 0, H * d, 2 * H * d, z, zb, tau, 0.5, state, slots, q_start, 3, out)
    for b, n in enumerate(lens):
        t0 = int(q_start[b])
        r = rows[t0 : t0 + n]
        q = r[:, : H * d].view(n, H, d) * 0.5
        k, v = r[:, H * d : 2 * H * d].view(n, H, d), r[:, 2 * H * d : 2 * H * d + H * e].view(n, H, e)
        a = plain_decay(z[t0 : t0 + n] + zb, tau).view(n, H, d)
        o, S = plain_decayed_state_scan(q, k, v, a, start[int(slots[b])])
        torch.testing.assert_close(out[t0 : t0 + n], o.reshape(n, -1), rtol=1e-5, atol=1e-5)
        torch.testing.assert_close(state[int(slots[b])], S, rtol=1e-5, atol=1e-5)
    torch.testing.assert_close(state[1], start[1])  # a slot that no sequence of the step holds stays


def test_twins_of_the_per_head_kernels_and_attention_with_a_sink():
    """The path of an attention layer through the twins: prepare (bias, norms per head, padding, pages), attention
    over the pages with window and sink; against the plain attention on the plain norms."""
    g = torch.Generator().manual_seed(7)
    T, H, G, d, e, hc, P, win = 21, 4, 2, 6, 4, 8, 8, 5
    src = torch.randn(T, H * d + G * d + G * e, generator=g)
    bias = torch.randn(src.shape[1], generator=g)
    qn, kn = 1 + 0.2 * torch.randn(d, generator=g), 1 + 0.2 * torch.randn(d, generator=g)
    sinks = torch.randn(H, generator=g)
    n_pages = 4
    kp, vp = torch.full((n_pages, G, P, hc), float("nan")), torch.full((n_pages, G, hc, P), float("nan"))
    table = torch.tensor([[3, 0, 2]], dtype=torch.int32)
    slots = torch.tensor([int(table[0, t // P]) * P + t % P for t in range(T)], dtype=torch.int32)
    q = torch.empty(T, H * hc)
    twins.heads_prepare(src, bias, 1e-5, n_q=H, q_col=0, q_width=d, q_norm=qn, q_norm_dims=d, q_out=q, q_out_width=hc,
                        n_kv=G, k_col=H * d, k_width=d, k_norm=kn, k_norm_dims=d, v_col=H * d + G * d, v_width=e,
                        slots=slots, k_pages=kp, v_pages=vp)
    out = torch.empty(T, H * hc)
    twins.paged_attention_general(q, out, kp, vp, table, torch.zeros(T, dtype=torch.int32),
                                  torch.arange(T, dtype=torch.int32), H, 0.4, win, sinks)
    x = src + bias
    pq = plain_rms(x[:, : H * d].view(T, H, d), qn, 1e-5)
    pk = plain_rms(x[:, H * d : H * d + G * d].view(T, G, d), kn, 1e-5)
    pv = x[:, H * d + G * d :].view(T, G, e)
    want = plain_window_sink_attention(pq, pk, pv, 0.4, win, sinks)
    got = out.view(T, H, hc)
    torch.testing.assert_close(got[..., :e], want, rtol=1e-5, atol=1e-5)
    assert float(got[..., e:].abs().max()) == 0.0
    # a product per head with a gate, copied columns and padding
    w = torch.randn(H, 3, d, generator=g)
    gate = torch.randn(T, H + 2, generator=g)
    y = torch.full((T, H * 7), float("nan"))
    twins.head_linear(q, hc, w, y, 7, tail=2, gate=gate)
    qq = q.view(T, H, hc)
    want_y = torch.einsum("hnk,thk->thn", w, qq[..., :d]) * torch.sigmoid(gate[:, :H])[:, :, None]
    yy = y.view(T, H, 7)
    torch.testing.assert_close(yy[..., :3], want_y)
    torch.testing.assert_close(yy[..., 3:5], qq[..., d : d + 2])
    assert float(yy[..., 5:].abs().max()) == 0.0
    # the norm per head with its gate
    o32, gt, wn = torch.randn(T, H * e, generator=g), torch.randn(T, H * e + 3, generator=g), torch.rand(e, generator=g)
    res = torch.empty(T, H * e)
    twins.head_norm_gate(o32, wn, 1e-5, gt, H, res)
    gg = gt[:, : H * e]
    torch.testing.assert_close(res, (plain_rms(o32.view(T, H, e), wn, 1e-5).reshape(T, -1) * gg * torch.sigmoid(gg)))
