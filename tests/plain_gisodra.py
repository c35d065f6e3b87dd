"""A plain, slow Gisodra: whole sequences, no cache, no batching, one function
per mechanism, sharing no code with ``fastgen_amd``.  It is what the engine is
compared with.

The model (notation of this file).  Tokens are embedded.  A layer is
*sandwiched*: ``x <- x + post1(mixer(pre1(x)))`` and, if it has a feed-forward,
``x <- x + post2(ff(pre2(x)))``; all four are RMS norms with a plain weight.
Three mixers exist:

* ``attention``: grouped heads with biases on q, k and v, an RMS norm per head
  on q and on k, no rotation, a sliding window, and a *sink*: one more term
  ``exp(sink_h)`` in the softmax's denominator that has no value.  Keys are
  ``dim`` wide, values ``vdim``.  A layer may name an earlier layer whose
  keys and values it reads instead of projecting its own.
* ``gla``: a recurrence per head on a ``dim x vdim`` state,
  ``S <- diag(a_t) S + k_t v_t^T``, ``o_t = S^T q_t``, with the decay
  ``a = sigmoid(z)^(1/tau)`` from a low-rank projection; the output is normed
  per head, gated by ``silu`` and projected.
* ``latent_attention``: queries and keys/values go through narrow latents; a
  key is ``[W_uk c ; r]`` with ``r`` one rotated part shared by all heads, a
  value ``W_uv c``; sliding window, sink, and a sigmoid gate per head.

The feed-forward is ``down(gelu_tanh(gate x) * up x)``.  The output is the
final norm, the embedding table as the head, and a soft cap on the logits.

``dtype`` is the precision of matrix products and activations; norms, the
residual stream, angles, scores and weights, the recurrence and all that
enters it but the projections stay in float32 (float64 when the whole run is).
"""

from __future__ import annotations

import math
from typing import Dict, List, Mapping, Optional, Tuple

import torch


def _hi(x: torch.Tensor) -> torch.Tensor:
    return x if x.dtype == torch.float64 else x.float()


def _mm(x: torch.Tensor, w: torch.Tensor, dtype: torch.dtype, bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``x W^T (+ b)`` with operands in ``dtype``, summed in the high precision, rounded once to ``dtype``."""
    y = _hi(x.to(dtype)) @ _hi(w.to(dtype)).T
    if bias is not None:
        y = y + _hi(bias)
    return y.to(dtype)


# ------------------------------------------------------------------ mechanisms
def plain_rms(x: torch.Tensor, w: Optional[torch.Tensor], eps: float) -> torch.Tensor:
    """``x / sqrt(mean(x^2) + eps) * w`` over the last axis (eps inside the root)."""
    x = _hi(x)
    y = x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)
    return y if w is None else y * _hi(w)


def plain_gelu_tanh(z: torch.Tensor) -> torch.Tensor:
    z = _hi(z)
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def plain_gated_ff(x: torch.Tensor, gate: torch.Tensor, up: torch.Tensor, down: torch.Tensor,
                   dtype: torch.dtype) -> torch.Tensor:
    a = (plain_gelu_tanh(_mm(x, gate, dtype)) * _hi(_mm(x, up, dtype))).to(dtype)
    return _mm(a, down, dtype)


def plain_rotate_halves(x: torch.Tensor, pos: torch.Tensor, base: float, dims: int) -> torch.Tensor:
    """``x [T, heads, >= dims]``: dimension ``i`` and ``i + dims/2`` (``i < dims/2``) turn by
    ``pos * base^(-2i/dims)``; dimensions from ``dims`` on pass."""
    out = _hi(x).clone()
    half = dims // 2
    if half == 0:
        return out
    f = base ** (-2.0 * torch.arange(half, dtype=torch.float64) / dims)
    ang = (pos.to(torch.float64)[:, None] * f[None, :]).to(torch.float32 if out.dtype != torch.float64 else torch.float64)
    c, s = torch.cos(ang)[:, None, :].to(out.dtype), torch.sin(ang)[:, None, :].to(out.dtype)
    u, v = _hi(x[..., :half]), _hi(x[..., half:dims])
    out[..., :half] = u * c - v * s
    out[..., half:dims] = v * c + u * s
    return out


def plain_window_sink_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float,
                                window: Optional[int], sink: Optional[torch.Tensor]) -> torch.Tensor:
    """``q [T, H, d]``, ``k [T, G, d]``, ``v [T, G, e]`` -> ``[T, H, e]``.  Query head ``h`` reads kv head
    ``h // (H/G)``; position ``i`` sees ``j`` with ``0 <= i - j < window``; the softmax's denominator has one
    more term ``exp(sink[h])`` that brings no value."""
    T, H, _ = q.shape
    G = k.shape[1]
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    seen = (j <= i) if window is None else (j <= i) & (i - j < window)
    out = torch.empty(T, H, v.shape[2], dtype=_hi(q).dtype)
    for h in range(H):
        g = h // (H // G)
        s = (_hi(q[:, h]) @ _hi(k[:, g]).T) * scale
        s = s.masked_fill(~seen, float("-inf"))
        top = s.max(-1, keepdim=True).values
        if sink is not None:
            top = torch.maximum(top, _hi(sink[h]).reshape(1, 1).to(s.dtype))
        e = torch.exp(s - top)
        den = e.sum(-1, keepdim=True)
        if sink is not None:
            den = den + torch.exp(_hi(sink[h]).to(s.dtype) - top)
        out[:, h] = (e / den) @ _hi(v[:, g])
    return out


def plain_decay(z: torch.Tensor, tau: float) -> torch.Tensor:
    """``sigmoid(z)^(1/tau)``."""
    return torch.exp(torch.nn.functional.logsigmoid(_hi(z)) / tau)


def plain_decayed_state_scan(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, a: torch.Tensor,
                             state: Optional[torch.Tensor] = None) -> Tuple[torch.Tensor, torch.Tensor]:
    """``q, k, a [T, H, d]``, ``v [T, H, e]``; per head ``S <- a_t[:, None] * S + k_t v_t^T`` and
    ``o_t = S^T q_t``.  Returns ``o [T, H, e]`` and the last state ``[H, d, e]``."""
    T, H, d = q.shape
    e = v.shape[2]
    hi = _hi(q).dtype
    S = torch.zeros(H, d, e, dtype=hi) if state is None else state.clone()
    out = torch.empty(T, H, e, dtype=hi)
    for t in range(T):
        S = _hi(a[t])[:, :, None] * S + _hi(k[t])[:, :, None] * _hi(v[t])[:, None, :]
        out[t] = torch.einsum("hde,hd->he", S, _hi(q[t]))
    return out, S


# ---------------------------------------------------------------------- mixers
def plain_attention_keys_values(x: torch.Tensor, w: Mapping[str, torch.Tensor], p: str, m: Mapping, eps: float,
                                dtype: torch.dtype) -> Tuple[torch.Tensor, torch.Tensor]:
    """The keys (after their norm) and values that an attention layer projects: what a later layer that names
    this one reads."""
    T = x.shape[0]
    G, d, e = m["kv_heads"], m["dim"], m["vdim"]
    k = _mm(x, w[f"{p}.k"], dtype, w[f"{p}.k.b"]).view(T, G, d)
    v = _mm(x, w[f"{p}.v"], dtype, w[f"{p}.v.b"]).view(T, G, e)
    return plain_rms(k, w[f"{p}.k.norm"], eps).to(dtype), v


def plain_attention_mixer(x: torch.Tensor, w: Mapping[str, torch.Tensor], p: str, m: Mapping, eps: float,
                          dtype: torch.dtype, kv: Tuple[torch.Tensor, torch.Tensor]) -> torch.Tensor:
    T = x.shape[0]
    H, d = m["heads"], m["dim"]
    q = _mm(x, w[f"{p}.q"], dtype, w[f"{p}.q.b"]).view(T, H, d)
    q = plain_rms(q, w[f"{p}.q.norm"], eps).to(dtype)
    window = (m.get("mask") or {}).get("size")
    o = plain_window_sink_attention(q, kv[0], kv[1], m["scale"], window, w.get(f"{p}.sink"))
    return _mm(o.reshape(T, -1), w[f"{p}.o"], dtype)


def plain_gla_mixer(x: torch.Tensor, w: Mapping[str, torch.Tensor], p: str, m: Mapping, eps: float,
                    dtype: torch.dtype) -> torch.Tensor:
    T = x.shape[0]
    H, d, e = m["heads"], m["dim"], m["vdim"]
    q = _hi(_mm(x, w[f"{p}.q"], dtype)).view(T, H, d) * d ** -0.5
    k = _mm(x, w[f"{p}.k"], dtype).view(T, H, d)
    v = _mm(x, w[f"{p}.v"], dtype).view(T, H, e)
    low = _mm(x, w[f"{p}.a1"], dtype)
    z = _hi(low.to(dtype)) @ _hi(w[f"{p}.a2"].to(dtype)).T + _hi(w[f"{p}.a2.b"])
    a = plain_decay(z, m["tau"]).view(T, H, d)
    o, _ = plain_decayed_state_scan(q, k, v, a)
    o = plain_rms(o, w[f"{p}.norm"], eps)
    g = _hi(_mm(x, w[f"{p}.g"], dtype))
    o = (o.reshape(T, -1) * (g * torch.sigmoid(g))).to(dtype)
    return _mm(o, w[f"{p}.o"], dtype)


def plain_latent_attention_mixer(x: torch.Tensor, w: Mapping[str, torch.Tensor], p: str, m: Mapping, eps: float,
                                 dtype: torch.dtype, pos: torch.Tensor) -> torch.Tensor:
    T = x.shape[0]
    H, d, r, e, R = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    base, dims = m["rot"]["base"], m["rot"]["dims"]
    cq = plain_rms(_mm(x, w[f"{p}.dq"], dtype), w[f"{p}.dq.norm"], eps).to(dtype)
    q = _mm(cq, w[f"{p}.uq"], dtype).view(T, H, d + r)
    both = _mm(x, w[f"{p}.dkv"], dtype)
    c = plain_rms(both[:, :R], w[f"{p}.dkv.norm"], eps).to(dtype)
    shared = plain_rotate_halves(both[:, None, R:], pos, base, dims).to(dtype)  # [T, 1, r]
    k_plain = _mm(c, w[f"{p}.uk"], dtype).view(T, H, d)
    v = _mm(c, w[f"{p}.uv"], dtype).view(T, H, e)
    q_turned = plain_rotate_halves(q[:, :, d:], pos, base, dims).to(dtype)
    q_full = torch.cat([q[:, :, :d], q_turned], dim=-1)
    k_full = torch.cat([k_plain, shared.expand(T, H, r)], dim=-1)
    window = (m.get("mask") or {}).get("size")
    o = plain_window_sink_attention(q_full, k_full, v, m["scale"], window, w.get(f"{p}.sink"))
    gate = torch.sigmoid(_hi(_mm(x, w[f"{p}.g"], dtype)))  # [T, H]
    o = (o * gate[:, :, None]).to(dtype)
    return _mm(o.reshape(T, -1), w[f"{p}.o"], dtype)


# ----------------------------------------------------------------------- model
def plain_gisodra_forward(weights: Mapping[str, torch.Tensor], config: Mapping, tokens: List[int],
                          dtype: torch.dtype = torch.float32, return_layers: bool = False):
    """Logits ``[T, vocab]`` of one whole sequence (and, with ``return_layers``, the residual stream after
    every layer ``[layers, T, width]``)."""
    hi = torch.float64 if dtype == torch.float64 else torch.float32
    w = {n: (t.to(torch.float64) if dtype == torch.float64 else t) for n, t in weights.items()}
    eps = config["norm"]["eps"]
    tok = torch.tensor(tokens, dtype=torch.long)
    pos = torch.arange(len(tokens))
    x = w["embed"][tok].to(hi)
    kept: Dict[int, Tuple[torch.Tensor, torch.Tensor]] = {}
    after = []
    for i, layer in enumerate(config["layers"]):
        p, m = f"l{i}.mix", layer["mixer"]
        n = plain_rms(x, w[f"l{i}.norm1"], eps).to(dtype)
        if layer["type"] == "attention":
            if m.get("kv_from") is None:
                kept[i] = plain_attention_keys_values(n, w, p, m, eps, dtype)
            y = plain_attention_mixer(n, w, p, m, eps, dtype, kept[i if m.get("kv_from") is None else m["kv_from"]])
        elif layer["type"] == "gla":
            y = plain_gla_mixer(n, w, p, m, eps, dtype)
        elif layer["type"] == "latent_attention":
            y = plain_latent_attention_mixer(n, w, p, m, eps, dtype, pos)
        else:
            raise ValueError(f"layer {i}: unknown type {layer['type']!r}")
        x = x + plain_rms(y, w[f"l{i}.norm1b"], eps)
        if layer.get("mlp") is not None:
            n = plain_rms(x, w[f"l{i}.norm2"], eps).to(dtype)
            y = plain_gated_ff(n, w[f"l{i}.mlp.gate"], w[f"l{i}.mlp.up"], w[f"l{i}.mlp.down"], dtype)
            x = x + plain_rms(y, w[f"l{i}.norm2b"], eps)
        after.append(x.clone())
    n = plain_rms(x, w["final.norm"], eps).to(dtype)
    logits = _hi(n) @ _hi(w["embed"].to(dtype)).T
    cap = config.get("logit_softcap")
    if cap:
        logits = cap * torch.tanh(logits / cap)
    logits = logits.to(hi)
    return (logits, torch.stack(after)) if return_layers else logits


def plain_gisodra_greedy(weights, config, prompt: List[int], n_new: int, dtype=torch.float32) -> List[int]:
    seq, out = list(prompt), []
    for _ in range(n_new):
        nxt = int(plain_gisodra_forward(weights, config, seq, dtype)[-1].argmax())
        out.append(nxt)
        seq.append(nxt)
    return out


# --------------------------------------------------------------------- weights
def plain_gisodra_shapes(config: Mapping) -> Dict[str, Tuple[int, ...]]:
    """Every tensor's name and shape for ``config``."""
    D, V = config["width"], config["vocab"]
    s: Dict[str, Tuple[int, ...]] = {"embed": (V, D), "final.norm": (D,)}
    for i, layer in enumerate(config["layers"]):
        p, m = f"l{i}.mix", layer["mixer"]
        s[f"l{i}.norm1"] = s[f"l{i}.norm1b"] = (D,)
        if layer["type"] == "attention":
            H, G, d, e = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            s.update({f"{p}.q": (H * d, D), f"{p}.q.b": (H * d,), f"{p}.q.norm": (d,), f"{p}.sink": (H,),
                      f"{p}.o": (D, H * e)})
            if m.get("kv_from") is None:
                s.update({f"{p}.k": (G * d, D), f"{p}.k.b": (G * d,), f"{p}.v": (G * e, D), f"{p}.v.b": (G * e,),
                          f"{p}.k.norm": (d,)})
        elif layer["type"] == "gla":
            H, d, e = m["heads"], m["dim"], m["vdim"]
            low = m.get("decay_rank", 16)
            s.update({f"{p}.q": (H * d, D), f"{p}.k": (H * d, D), f"{p}.v": (H * e, D), f"{p}.g": (H * e, D),
                      f"{p}.o": (D, H * e), f"{p}.norm": (e,), f"{p}.a1": (low, D), f"{p}.a2": (H * d, low),
                      f"{p}.a2.b": (H * d,)})
        else:
            H, d, r, e, R, Q = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"], m["q_rank"]
            s.update({f"{p}.dq": (Q, D), f"{p}.dq.norm": (Q,), f"{p}.uq": (H * (d + r), Q), f"{p}.dkv": (R + r, D),
                      f"{p}.dkv.norm": (R,), f"{p}.uk": (H * d, R), f"{p}.uv": (H * e, R), f"{p}.sink": (H,),
                      f"{p}.g": (H, D), f"{p}.o": (D, H * e)})
        if layer.get("mlp") is not None:
            F = layer["mlp"]["ff"]
            s[f"l{i}.norm2"] = s[f"l{i}.norm2b"] = (D,)
            s.update({f"l{i}.mlp.gate": (F, D), f"l{i}.mlp.up": (F, D), f"l{i}.mlp.down": (D, F)})
    return s


def plain_gisodra_weights(config: Mapping, seed: int) -> Dict[str, torch.Tensor]:
    """Random weights, representable in bfloat16, large enough that every mechanism moves the logits."""
    g = torch.Generator().manual_seed(seed)
    out: Dict[str, torch.Tensor] = {}
    for name, shape in plain_gisodra_shapes(config).items():
        if name.endswith("norm") or name.endswith("norm1") or name.endswith("norm2") or name.endswith("norm1b") \
                or name.endswith("norm2b"):
            t = 1.0 + 0.2 * torch.randn(shape, generator=g)
        elif name.endswith(".sink"):
            t = torch.randn(shape, generator=g)
        elif name.endswith(".a2.b"):
            t = 2.0 + torch.randn(shape, generator=g)
        elif name.endswith(".b"):
            t = 0.3 * torch.randn(shape, generator=g)
        elif name == "embed":
            t = torch.randn(shape, generator=g)
        else:
            t = torch.randn(shape, generator=g) * (1.5 / math.sqrt(shape[-1]))
        out[name] = t.to(torch.bfloat16).float()
    return out


def _attn(H, G, d, e, window, kv_from=None):
    m = {"heads": H, "kv_heads": G, "dim": d, "vdim": e, "scale": d ** -0.5, "mask": {"size": window}}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return m


def _latent(H, d, r, e, R, Q, window, base=10000.0):
    return {"heads": H, "dim": d, "rot_dim": r, "vdim": e, "kv_rank": R, "q_rank": Q, "scale": (d + r) ** -0.5,
            "mask": {"size": window}, "rot": {"base": base, "dims": r}}


def _config(width, vocab, layers, cap=20.0, eps=1e-5):
    return {"architecture": "Gisodra", "width": width, "vocab": vocab, "norm": {"eps": eps}, "logit_softcap": cap,
            "layers": layers}


# every mixer once, a shared cache, a layer without a feed-forward; windows shorter than a page
TRIO = _config(64, 97, [
    {"type": "attention", "mixer": _attn(4, 2, 32, 16, 24), "mlp": {"kind": "dense", "ff": 96}},
    {"type": "gla", "mixer": {"heads": 2, "dim": 16, "vdim": 32, "tau": 8.0}, "mlp": None},
    {"type": "attention", "mixer": _attn(4, 2, 32, 16, 40, kv_from=0), "mlp": {"kind": "dense", "ff": 96}},
    {"type": "latent_attention", "mixer": _latent(4, 16, 16, 24, 48, 40, 20), "mlp": {"kind": "dense", "ff": 80}},
])
# another order, values wider than keys, one kv head for all and one a head, windows longer than a page,
# a rotated part larger than the plain one, tau 1
WIDE_VALUES = _config(96, 130, [
    {"type": "latent_attention", "mixer": _latent(3, 8, 32, 16, 40, 24, 150, base=500.0), "mlp": None},
    {"type": "gla", "mixer": {"heads": 3, "dim": 32, "vdim": 16, "tau": 1.0}, "mlp": {"kind": "dense", "ff": 72}},
    {"type": "attention", "mixer": _attn(3, 3, 16, 48, 100), "mlp": {"kind": "dense", "ff": 64}},
    {"type": "attention", "mixer": _attn(6, 1, 24, 40, 70), "mlp": None},
    {"type": "gla", "mixer": {"heads": 1, "dim": 64, "vdim": 64, "tau": 4.0}, "mlp": {"kind": "dense", "ff": 40}},
], cap=8.0, eps=1e-6)
# one layer of a kind each, for tests of a mechanism inside the engine
ONLY_ATTENTION = _config(48, 61, [{"type": "attention", "mixer": _attn(2, 1, 16, 16, 9),
                                   "mlp": {"kind": "dense", "ff": 56}}])
ONLY_GLA = _config(48, 61, [{"type": "gla", "mixer": {"heads": 2, "dim": 24, "vdim": 8, "tau": 16.0}, "mlp": None}])
ONLY_LATENT = _config(48, 61, [{"type": "latent_attention", "mixer": _latent(2, 16, 8, 16, 32, 16, 33),
                                "mlp": None}])
# sizes that are no multiples of 8 or 16, head counts that are no powers of two, more heads a kv head than the
# matrix-core kernels take, a window of one token and one longer than any prompt of the tests, a cache read by two
# later layers through a shorter and a longer window than its owner's, a width that the streaming products refuse
ODD_SIZES = _config(100, 101, [
    {"type": "gla", "mixer": {"heads": 3, "dim": 20, "vdim": 12, "tau": 2.5, "decay_rank": 6}, "mlp": {"kind": "dense", "ff": 70}},
    {"type": "attention", "mixer": _attn(5, 5, 40, 24, 1), "mlp": None},
    {"type": "latent_attention", "mixer": _latent(7, 20, 6, 10, 30, 18, 1000), "mlp": {"kind": "dense", "ff": 36}},
    {"type": "attention", "mixer": _attn(34, 2, 8, 8, 50), "mlp": None},
    {"type": "attention", "mixer": _attn(34, 2, 8, 8, 7, kv_from=3), "mlp": {"kind": "dense", "ff": 24}},
    {"type": "latent_attention", "mixer": _latent(20, 8, 24, 56, 72, 64, 31, base=77.0), "mlp": None},
    {"type": "attention", "mixer": _attn(34, 2, 8, 8, 90, kv_from=3), "mlp": None},
], cap=50.0, eps=1e-4)
