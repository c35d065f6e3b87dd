"""A plain, slow Buderax: whole sequences, no cache, no batching, one function
per mechanism, sharing no code with ``fastgen_amd``.  It is what the engine is
compared with.

The model (notation of this file): tokens are embedded and scaled; layers are
*parallel* (``x <- x + mixer(n) + ff(n)`` with ``n = norm(x)`` the one norm of
the layer, whose weight is stored around zero); the mixer is causal softmax
attention with grouped heads whose values are its keys as projected (before
the rotation), rotated pairs ``(2i, 2i+1)`` on the first ``dims`` head
dimensions with every frequency divided by a factor, a score scale from the
configuration and a sigmoid gate on the concatenated heads; the feed-forward
is a mixture of gated experts, chosen by the largest router logits and
weighted by the softmax over the chosen logits; a stretch of layers may run
several times, each pass starting from ``x + embedding`` (not the first) plus
a learned vector of the pass.

``dtype`` is the precision of matrix products and activations; norms, the
residual stream, angles, scores and weights, and the router stay in float32
(float64 when the whole run is).
"""

from __future__ import annotations

import math
from typing import Dict, List, Mapping, Optional, Tuple

import torch


def _hi(x: torch.Tensor) -> torch.Tensor:
    return x if x.dtype == torch.float64 else x.float()


# ------------------------------------------------------------------ mechanisms
def plain_scaled_embedding(table: torch.Tensor, tokens: torch.Tensor, scale: float) -> torch.Tensor:
    return _hi(table[tokens]) * scale


def plain_zero_centred_rmsnorm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    """``x / sqrt(mean(x^2) + eps) * (1 + w)``: eps inside the root."""
    x = _hi(x)
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * (1.0 + _hi(w))


def plain_linear_frequencies(dims: int, base: float, factor: float) -> torch.Tensor:
    """``base^(-2i/dims) / factor`` for ``i < dims/2``."""
    i = torch.arange(dims // 2, dtype=torch.float32)
    return base ** (-2.0 * i / dims) / factor


def plain_rotate_pairs(x: torch.Tensor, pos: torch.Tensor, freqs: torch.Tensor) -> torch.Tensor:
    """``x [T, heads, hd]``: dimensions ``2i`` and ``2i+1`` (``i < len(freqs)``) turn by ``pos * freqs[i]``;
    the others pass."""
    out = _hi(x).clone()
    n = 2 * freqs.numel()
    if n == 0:
        return out.to(x.dtype)
    ang = pos.to(torch.float32)[:, None] * freqs[None, :]
    c, s = torch.cos(ang)[:, None, :].to(out.dtype), torch.sin(ang)[:, None, :].to(out.dtype)
    u, v = _hi(x[..., 0:n:2]), _hi(x[..., 1:n:2])
    out[..., 0:n:2] = u * c - v * s
    out[..., 1:n:2] = v * c + u * s
    return out.to(x.dtype)


def plain_causal_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float) -> torch.Tensor:
    """``q [T, H, d]``, ``k``, ``v`` ``[T, G, d]``; query head ``h`` reads kv head ``h // (H/G)``; position ``i``
    sees every ``j <= i``; plain softmax.  Scores and weights in the high precision."""
    T, H, _ = q.shape
    G = k.shape[1]
    out = torch.empty(T, H, v.shape[2], dtype=_hi(q).dtype)
    seen = torch.tril(torch.ones(T, T, dtype=torch.bool))
    for h in range(H):
        g = h // (H // G)
        s = (_hi(q[:, h]) @ _hi(k[:, g]).T) * scale
        s = s.masked_fill(~seen, float("-inf"))
        out[:, h] = torch.softmax(s, dim=-1) @ _hi(v[:, g])
    return out


def plain_gated_attention(n: torch.Tensor, wq, wk, wg, wo, m: Mapping, pos: torch.Tensor) -> torch.Tensor:
    """The whole mixer on normed rows ``n [T, width]``."""
    T = n.shape[0]
    H, G, d = m["heads"], m["kv_heads"], m["dim"]
    q = (n @ wq.T).view(T, H, d)
    k = (n @ wk.T).view(T, G, d)
    v = k  # the values are the keys as projected: before the rotation
    rot = m.get("rot") or {}
    dims = rot.get("dims", 0)
    freqs = plain_linear_frequencies(dims, rot.get("base", 10000.0), (rot.get("scaling") or {}).get("factor", 1.0))
    q, k = plain_rotate_pairs(q, pos, freqs), plain_rotate_pairs(k, pos, freqs)
    heads = plain_causal_attention(q, k, v, m["scale"]).reshape(T, H * m["vdim"])
    gate = torch.sigmoid(_hi(n @ wg.T))
    return (heads * gate).to(n.dtype) @ wo.T


def plain_route(n: torch.Tensor, wr: torch.Tensor, br: torch.Tensor, top: int) -> Tuple[torch.Tensor, torch.Tensor]:
    """Experts ``[T, top]`` with the largest logits ``n wr^T + br`` and the softmax over those logits alone."""
    z = _hi(n) @ _hi(wr).T + _hi(br)
    val, idx = torch.topk(z, top, dim=-1)
    return idx, torch.softmax(val, dim=-1)


def plain_expert(n: torch.Tensor, w_gate, w_up, w_down) -> torch.Tensor:
    a = n @ w_gate.T
    return ((a * torch.sigmoid(a)) * (n @ w_up.T)) @ w_down.T


def plain_mixture(n: torch.Tensor, W: Mapping[str, torch.Tensor], prefix: str, m: Mapping) -> torch.Tensor:
    idx, wt = plain_route(n, W[prefix + ".router"], W[prefix + ".router.b"], m["router"]["top"])
    out = torch.zeros(n.shape, dtype=_hi(n).dtype)
    for t in range(n.shape[0]):
        for j in range(idx.shape[1]):
            e = int(idx[t, j])
            y = plain_expert(n[t : t + 1], W[f"{prefix}.e{e}.gate"], W[f"{prefix}.e{e}.up"], W[f"{prefix}.e{e}.down"])
            out[t] += wt[t, j] * _hi(y[0])
    return out


def plain_run_order(n_layers: int, loop: Optional[Mapping]) -> List[Tuple[int, Optional[int]]]:
    """(layer, number of the pass that begins with it or None)."""
    if not loop:
        return [(i, None) for i in range(n_layers)]
    a, b, times = loop["start"], loop["stop"], loop["times"]
    order: List[Tuple[int, Optional[int]]] = [(i, None) for i in range(a)]
    for t in range(times):
        order += [(i, t if i == a else None) for i in range(a, b)]
    return order + [(i, None) for i in range(b, n_layers)]


# ------------------------------------------------------------------- the model
def plain_buderax_forward(weights: Mapping[str, torch.Tensor], config: Mapping, tokens, dtype=torch.float32,
                          streams: Optional[list] = None) -> torch.Tensor:
    """Logits ``[T, vocab]`` of one whole sequence; ``streams`` collects the residual stream after every
    layer run."""
    hi = torch.float64 if dtype == torch.float64 else torch.float32
    W = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in weights.items()}
    tok = torch.as_tensor(tokens, dtype=torch.long)
    pos = torch.arange(tok.numel())
    eps = config["norm"]["eps"]
    x = plain_scaled_embedding(W["embed"], tok, config["embedding"]["scale"]).to(hi)
    first = x.clone()
    for i, begins in plain_run_order(len(config["layers"]), config.get("loop")):
        if begins is not None:
            if begins > 0:
                x = x + first
            x = x + W["loop.step"][begins].to(hi)
        layer, p = config["layers"][i], f"l{i}"
        n = plain_zero_centred_rmsnorm(x, W[p + ".norm1"], eps).to(dtype)
        y = _hi(plain_gated_attention(n, W[p + ".mix.q"], W[p + ".mix.k"], W[p + ".mix.g"], W[p + ".mix.o"],
                                      layer["mixer"], pos)).to(hi)
        if layer.get("mlp") is not None:
            y = y + plain_mixture(n, W, p + ".mlp", layer["mlp"]).to(hi)
        x = x + y
        if streams is not None:
            streams.append(x.clone())
    n = plain_zero_centred_rmsnorm(x, W["final.norm"], eps).to(dtype)
    return _hi(n @ W["head"].T)


def plain_buderax_greedy(weights, config, prompt, n_new: int, dtype=torch.float32) -> List[int]:
    toks = list(prompt)
    for _ in range(n_new):
        toks.append(int(torch.argmax(plain_buderax_forward(weights, config, toks, dtype)[-1])))
    return toks[len(prompt):]


def plain_buderax_weights(config: Mapping, seed: int, sharpen: float = 1.0) -> Dict[str, torch.Tensor]:
    """Random weights under the checkpoint's names, every value one that bfloat16 holds.  ``sharpen``
    multiplies the query projections: the softmax then leans on few keys, and a key that is lost or
    misplaced shows in the logits."""
    g = torch.Generator().manual_seed(seed)
    D, V = config["width"], config["vocab"]

    def rnd(*shape, std):
        return (torch.randn(*shape, generator=g) * std).to(torch.bfloat16).float()

    w = {"embed": rnd(V, D, std=0.5), "final.norm": rnd(D, std=0.2), "head": rnd(V, D, std=D**-0.5)}
    if config.get("loop"):
        w["loop.step"] = rnd(config["loop"]["times"], D, std=0.5)
    for i, layer in enumerate(config["layers"]):
        m, p = layer["mixer"], f"l{i}"
        H, G, d = m["heads"], m["kv_heads"], m["dim"]
        w[p + ".norm1"] = rnd(D, std=0.2)
        w[p + ".mix.q"] = rnd(H * d, D, std=sharpen * D**-0.5)
        w[p + ".mix.k"] = rnd(G * d, D, std=D**-0.5)
        w[p + ".mix.g"] = rnd(H * m["vdim"], D, std=D**-0.5)
        w[p + ".mix.o"] = rnd(D, H * m["vdim"], std=(H * d) ** -0.5)
        if layer.get("mlp") is not None:
            E, F = layer["mlp"]["router"]["experts"], layer["mlp"]["expert"]["ff"]
            w[p + ".mlp.router"] = rnd(E, D, std=2.0 * D**-0.5)
            w[p + ".mlp.router.b"] = rnd(E, std=0.5)
            for e in range(E):
                w[f"{p}.mlp.e{e}.gate"] = rnd(F, D, std=D**-0.5)
                w[f"{p}.mlp.e{e}.up"] = rnd(F, D, std=D**-0.5)
                w[f"{p}.mlp.e{e}.down"] = rnd(D, F, std=F**-0.5)
    return w


# --------------------------------------------------------------- test models
def _attn(heads, kv, dim, dims, base, factor, scale):
    rot = {"base": base, "dims": dims}
    if factor is not None:
        rot["scaling"] = {"factor": factor}
    return {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": dim, "scale": scale, "rot": rot}


def _moe(experts, top, ff):
    return {"kind": "moe", "router": {"experts": experts, "top": top}, "expert": {"ff": ff}}


# layers that differ in every size, a layer without a feed-forward, all experts chosen in one layer, a loop
# over the two last layers
SMALL_LOOP = {
    "architecture": "Buderax", "width": 64, "vocab": 101, "embedding": {"scale": 2.5}, "norm": {"eps": 1e-5},
    "layers": [
        {"type": "attention", "mixer": _attn(4, 2, 16, 8, 10000.0, 2.0, 0.3), "mlp": _moe(5, 2, 24)},
        {"type": "attention", "mixer": _attn(2, 1, 32, 32, 500.0, None, 0.2), "mlp": None},
        {"type": "attention", "mixer": _attn(4, 4, 16, 16, 70000.0, 8.0, 0.25), "mlp": _moe(3, 3, 40)},
    ],
    "loop": {"start": 1, "stop": 3, "times": 2},
}
# no loop, one expert a token, expert widths that are no multiple of 8, embedding scale 1
PLAIN_STACK = {
    "architecture": "Buderax", "width": 96, "vocab": 77, "embedding": {"scale": 1.0}, "norm": {"eps": 1e-6},
    "layers": [
        {"type": "attention", "mixer": _attn(6, 3, 16, 4, 100.0, 1.5, 0.25), "mlp": _moe(4, 1, 20)},
        {"type": "attention", "mixer": _attn(3, 1, 32, 16, 1000.0, None, 0.18), "mlp": _moe(2, 2, 12)},
    ],
}
# one layer looped three times from the start; a width and a head size that are multiples of 8 only
ALL_LOOP = {
    "architecture": "Buderax", "width": 40, "vocab": 53, "embedding": {"scale": 0.7}, "norm": {"eps": 1e-5},
    "layers": [{"type": "attention", "mixer": _attn(3, 3, 24, 24, 3000.0, 3.0, 0.2), "mlp": _moe(6, 2, 16)}],
    "loop": {"start": 0, "stop": 1, "times": 3},
}
# a loop of one pass in the middle
ONE_PASS = {
    "architecture": "Buderax", "width": 64, "vocab": 67, "embedding": {"scale": 4.0}, "norm": {"eps": 1e-6},
    "layers": [
        {"type": "attention", "mixer": _attn(2, 2, 32, 32, 20000.0, 4.0, 0.17), "mlp": _moe(8, 2, 32)},
        {"type": "attention", "mixer": _attn(4, 1, 16, 16, 20000.0, 4.0, 0.25), "mlp": _moe(8, 2, 32)},
    ],
    "loop": {"start": 1, "stop": 2, "times": 1},
}
