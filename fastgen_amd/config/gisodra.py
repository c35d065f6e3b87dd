"""The Gisodra decoder as a layout of parts.

A Gisodra ``config.json`` is nested: ``width``, ``vocab``, ``norm.eps``,
``logit_softcap`` and a list ``layers`` whose entries name their mixer
(``type``: ``attention``, ``gla`` or ``latent_attention``), its sizes
(``mixer``) and their feed-forward (``mlp``: ``{"kind": "dense", "ff": n}`` or
null).  Every layer is a sandwich: an RMS norm before and one behind each
sublayer (``l<i>.norm1``, ``norm1b``, ``norm2``, ``norm2b``).  The head is the
embedding table; the logits are soft-capped.  Tensors are named ``embed``,
``l<i>.mix.*``, ``l<i>.mlp.{gate,up,down}``, ``final.norm``.

An attention layer whose mixer says ``kv_from: j`` has no keys and values of
its own: it reads layer ``j``'s cache.  The width of the narrow middle of a
``gla`` layer's decay projection is no key of the configuration: it is the
shape of ``l<i>.mix.a1`` (``parse`` takes the tensors' shapes), or the optional
key ``decay_rank`` where there are no tensors yet.
"""

from __future__ import annotations

from dataclasses import dataclass, field, replace
from typing import Any, Callable, Mapping, Optional, Tuple, Union

from .buderax import _get
from .layout import LayerSpec, ModelLayout, PartSpec, RunEntry
from .model_args import ConfigError
from .registry import register_architecture

DEFAULT_DECAY_RANK = 16


@dataclass(frozen=True)
class WindowAttentionArgs:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    window: Optional[int]
    kv_from: Optional[int]


@dataclass(frozen=True)
class GlaArgs:
    heads: int
    dim: int
    vdim: int
    tau: float
    decay_rank: int


@dataclass(frozen=True)
class LatentArgs:
    heads: int
    dim: int
    rot_dim: int
    vdim: int
    kv_rank: int
    q_rank: int
    scale: float
    window: Optional[int]
    rot_base: float


@dataclass(frozen=True)
class GisodraLayer:
    type: str
    mixer: Union[WindowAttentionArgs, GlaArgs, LatentArgs]
    ff: Optional[int]  # width of the dense feed-forward; None: the layer has none


@dataclass(frozen=True)
class GisodraArgs:
    architecture: str
    width: int
    vocab: int
    norm_eps: float
    logit_softcap: Optional[float]
    layers: Tuple[GisodraLayer, ...]
    extra: Mapping[str, Any] = field(default_factory=dict, compare=False)

    @property
    def vocab_size(self) -> int:
        return self.vocab


def _positive(where: str, **values: int) -> None:
    for name, v in values.items():
        if v <= 0:
            raise ConfigError(f"config.json: {where}.{name}={v} must be positive")


class GisodraArchitecture:
    name = "Gisodra"

    def parse(self, config: Mapping[str, Any], shape_of: Optional[Callable[[str], Optional[Tuple[int, ...]]]] = None
              ) -> GisodraArgs:
        """``shape_of(name)``: the shape of a tensor of the checkpoint (None if it has none of that name);
        sizes that only the tensors give are read from it."""
        layers = []
        raw = _get(config, "layers")
        for i, l in enumerate(raw):
            kind, m, where = _get(l, "type", str), _get(l, "mixer"), f"layers[{i}].mixer"
            window = _get(m, "mask.size", int, None)
            if window is not None and window <= 0:
                raise ConfigError(f"config.json: {where}.mask.size={window} must be positive")
            if kind == "attention":
                a = WindowAttentionArgs(_get(m, "heads", int), _get(m, "kv_heads", int), _get(m, "dim", int),
                                        _get(m, "vdim", int), _get(m, "scale", float), window,
                                        _get(m, "kv_from", int, None))
                _positive(where, heads=a.heads, kv_heads=a.kv_heads, dim=a.dim, vdim=a.vdim)
                if a.heads % a.kv_heads:
                    raise ConfigError(f"config.json: {where}: heads={a.heads} is not a multiple of kv_heads={a.kv_heads}")
                if a.kv_from is not None:
                    j = a.kv_from
                    if not 0 <= j < i or layers[j].type != "attention" or layers[j].mixer.kv_from is not None:
                        raise ConfigError(f"config.json: {where}.kv_from={j} must name an earlier attention layer"
                                          " with keys and values of its own")
                    o = layers[j].mixer
                    if (o.kv_heads, o.dim, o.vdim) != (a.kv_heads, a.dim, a.vdim):
                        raise ConfigError(f"config.json: {where}: kv_heads, dim and vdim must equal layer {j}'s")
            elif kind == "gla":
                rank = _get(m, "decay_rank", int, DEFAULT_DECAY_RANK)
                shape = shape_of(f"l{i}.mix.a1") if shape_of is not None else None
                if shape is not None:
                    rank = int(shape[0])
                a = GlaArgs(_get(m, "heads", int), _get(m, "dim", int), _get(m, "vdim", int), _get(m, "tau", float), rank)
                _positive(where, heads=a.heads, dim=a.dim, vdim=a.vdim, decay_rank=a.decay_rank)
                if not a.tau > 0:
                    raise ConfigError(f"config.json: {where}.tau must be positive")
            elif kind == "latent_attention":
                a = LatentArgs(_get(m, "heads", int), _get(m, "dim", int), _get(m, "rot_dim", int), _get(m, "vdim", int),
                               _get(m, "kv_rank", int), _get(m, "q_rank", int), _get(m, "scale", float), window,
                               _get(m, "rot.base", float))
                _positive(where, heads=a.heads, dim=a.dim, rot_dim=a.rot_dim, vdim=a.vdim, kv_rank=a.kv_rank, q_rank=a.q_rank)
                dims = _get(m, "rot.dims", int, a.rot_dim)
                if dims != a.rot_dim or a.rot_dim % 2:
                    raise ConfigError(f"config.json: {where}: rot.dims={dims} must equal rot_dim={a.rot_dim}, an even number")
            else:
                raise ConfigError(f"config.json: layers[{i}].type {kind!r} is not supported"
                                  " (supported: 'attention', 'gla', 'latent_attention')")
            mlp = l.get("mlp")
            ff = None
            if mlp is not None:
                if mlp.get("kind", "dense") != "dense":
                    raise ConfigError(f"config.json: layers[{i}].mlp.kind {mlp.get('kind')!r} is not supported (supported: 'dense')")
                ff = _get(mlp, "ff", int)
                _positive(f"layers[{i}].mlp", ff=ff)
            layers.append(GisodraLayer(kind, a, ff))
        cap = _get(config, "logit_softcap", float, None)
        if cap is not None and not cap > 0:
            raise ConfigError("config.json: logit_softcap must be positive")
        return GisodraArgs(
            architecture=self.name, width=_get(config, "width", int), vocab=_get(config, "vocab", int),
            norm_eps=_get(config, "norm.eps", float), logit_softcap=cap, layers=tuple(layers),
            extra={k: config[k] for k in ("bos_token_id", "eos_token_id") if k in config},
        )

    def to_hf_config(self, args: GisodraArgs) -> dict:
        def mixer(l: GisodraLayer) -> dict:
            m = l.mixer
            mask = {"mask": {"size": m.window}} if getattr(m, "window", None) is not None else {}
            if l.type == "attention":
                out = {"heads": m.heads, "kv_heads": m.kv_heads, "dim": m.dim, "vdim": m.vdim, "scale": m.scale, **mask}
                if m.kv_from is not None:
                    out["kv_from"] = m.kv_from
                return out
            if l.type == "gla":
                return {"heads": m.heads, "dim": m.dim, "vdim": m.vdim, "tau": m.tau, "decay_rank": m.decay_rank}
            return {"heads": m.heads, "dim": m.dim, "rot_dim": m.rot_dim, "vdim": m.vdim, "kv_rank": m.kv_rank,
                    "q_rank": m.q_rank, "scale": m.scale, "rot": {"base": m.rot_base, "dims": m.rot_dim}, **mask}

        out = {
            "architecture": self.name, "width": args.width, "vocab": args.vocab, "norm": {"eps": args.norm_eps},
            "layers": [{"type": l.type, "mixer": mixer(l),
                        "mlp": None if l.ff is None else {"kind": "dense", "ff": l.ff}} for l in args.layers],
        }
        if args.logit_softcap is not None:
            out["logit_softcap"] = args.logit_softcap
        out.update(args.extra)
        return out

    def layout(self, args: GisodraArgs) -> ModelLayout:
        bare = {"weight": ""}  # a part's one tensor is named by the prefix alone
        D, eps = args.width, args.norm_eps

        def norm(prefix: str) -> PartSpec:
            return PartSpec("rmsnorm", prefix, dict(dim=D, eps=eps, names=bare))

        # how long a layer's cache keeps a key: the longest window of the layers that read it
        keep = {}
        for i, l in enumerate(args.layers):
            if l.type == "attention":
                owner = i if l.mixer.kv_from is None else l.mixer.kv_from
                w = l.mixer.window
                keep[owner] = None if w is None or (owner in keep and keep[owner] is None) else max(w, keep.get(owner, 0))
        layers, order = [], []
        for i, l in enumerate(args.layers):
            m, p = l.mixer, f"l{i}.mix"
            reads = None
            if l.type == "attention":
                own = m.kv_from is None
                reads = None if own else m.kv_from
                mixer = PartSpec("attention", p, dict(
                    dim=D, n_heads=m.heads, n_kv_heads=m.kv_heads, head_dim=m.dim, v_head_dim=m.vdim, scale=m.scale,
                    window=m.window, cache_window=keep[i] if own else m.window, position=PartSpec("none"), bias=True,
                    qk_norm=True, qk_norm_eps=eps, sink=True, has_kv=own, exact_weights=True,
                    names={"q_proj.weight": "q", "k_proj.weight": "k", "v_proj.weight": "v", "o_proj.weight": "o",
                           "q_proj.bias": "q.b", "k_proj.bias": "k.b", "v_proj.bias": "v.b",
                           "q_norm.weight": "q.norm", "k_norm.weight": "k.norm", "sinks": "sink"}))
            elif l.type == "gla":
                mixer = PartSpec("gated_linear_attention", p, dict(
                    dim=D, n_heads=m.heads, head_dim=m.dim, v_head_dim=m.vdim, tau=m.tau, decay_rank=m.decay_rank, eps=eps,
                    names={"q_proj.weight": "q", "k_proj.weight": "k", "v_proj.weight": "v", "gate_proj.weight": "g",
                           "o_proj.weight": "o", "out_norm.weight": "norm", "decay_down.weight": "a1",
                           "decay_up.weight": "a2", "decay_up.bias": "a2.b"}))
            else:
                rope = PartSpec("rope", options=dict(head_dim=m.rot_dim, rotary_dim=m.rot_dim, theta=m.rot_base,
                                                     pairing="half"))
                mixer = PartSpec("latent_attention", p, dict(
                    dim=D, n_heads=m.heads, head_dim=m.dim, rot_dim=m.rot_dim, v_head_dim=m.vdim, kv_rank=m.kv_rank,
                    q_rank=m.q_rank, scale=m.scale, window=m.window, sink=True, head_gate=True, eps=eps, position=rope,
                    exact_weights=True,
                    names={"q_down.weight": "dq", "q_down_norm.weight": "dq.norm", "q_up.weight": "uq",
                           "kv_down.weight": "dkv", "kv_down_norm.weight": "dkv.norm", "k_up.weight": "uk",
                           "v_up.weight": "uv", "sinks": "sink", "gate_proj.weight": "g", "o_proj.weight": "o"}))
            ffn = None
            extra = {"post_mixer": norm(f"l{i}.norm1b")}
            if l.ff is not None:
                ffn = PartSpec("swiglu", f"l{i}.mlp", dict(
                    dim=D, hidden_dim=l.ff, activation="gelu_tanh",
                    names={"gate_proj.weight": "gate", "up_proj.weight": "up", "down_proj.weight": "down"}))
                extra["post_ffn"] = norm(f"l{i}.norm2b")
            layers.append(LayerSpec(mixer=mixer, ffn=ffn, mixer_norm=norm(f"l{i}.norm1"),
                                    ffn_norm=norm(f"l{i}.norm2") if ffn is not None else None,
                                    arrangement="sandwich", extra_norms=extra))
            order.append(RunEntry(i, reads_cache_of=reads))
        return ModelLayout(
            dim=D, vocab_size=args.vocab,
            embed=PartSpec("embedding", "embed", dict(vocab_size=args.vocab, dim=D, names=bare)),
            layers=tuple(layers), order=tuple(order), final_norm=norm("final.norm"),
            head=PartSpec("lm_head", "head", dict(vocab_size=args.vocab, dim=D, tied_to="embed", names=bare,
                                                  softcap=args.logit_softcap)),
        )


GISODRA = register_architecture(GisodraArchitecture())
