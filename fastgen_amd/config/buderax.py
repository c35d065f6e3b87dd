"""The Buderax decoder as a layout of parts.

A Buderax ``config.json`` is nested: ``width``, ``vocab``, ``embedding.scale``,
``norm.eps``, a list ``layers`` whose entries name their mixer (``type``), its
sizes (``mixer``) and their feed-forward (``mlp``, or null), and optionally
``loop``: layers ``start .. stop-1`` run ``times`` times in a row with the same
weights and a cache per pass.  Every layer is parallel: one norm, whose output
both the mixer and the feed-forward read, and their sum goes to the residual
stream.  Tensors are named ``l<i>.norm1``, ``l<i>.mix.*``, ``l<i>.mlp.*``,
``embed``, ``loop.step``, ``final.norm``, ``head``.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Mapping, Optional, Tuple

from .layout import LayerSpec, ModelLayout, PartSpec, RunEntry
from .model_args import ConfigError
from .registry import register_architecture


def _get(config: Mapping[str, Any], path: str, kind=None, default: Any = ...):
    """``config[a][b]...`` for ``path`` = "a.b..."; a missing key raises with the whole path
    unless a default is given."""
    node: Any = config
    for key in path.split("."):
        if not isinstance(node, Mapping) or key not in node or node[key] is None:
            if default is not ...:
                return default
            raise ConfigError(f"config.json: required key {path!r} is missing")
        node = node[key]
    return kind(node) if kind is not None else node


@dataclass(frozen=True)
class AttentionArgs:
    heads: int
    kv_heads: int
    dim: int  # per-head size of queries and keys
    vdim: int  # per-head size of values
    scale: float
    rot_dims: int
    rot_base: float
    rot_factor: float  # linear scaling: every frequency is divided by it (1: none)


@dataclass(frozen=True)
class MoeArgs:
    experts: int
    top: int
    ff: int


@dataclass(frozen=True)
class BuderaxLayer:
    type: str
    mixer: AttentionArgs
    mlp: Optional[MoeArgs]


@dataclass(frozen=True)
class LoopArgs:
    start: int
    stop: int
    times: int


@dataclass(frozen=True)
class BuderaxArgs:
    architecture: str
    width: int
    vocab: int
    embedding_scale: float
    norm_eps: float
    layers: Tuple[BuderaxLayer, ...]
    loop: Optional[LoopArgs]
    extra: Mapping[str, Any] = field(default_factory=dict, compare=False)

    @property
    def vocab_size(self) -> int:
        return self.vocab


def _attention_args(m: Mapping[str, Any], where: str) -> AttentionArgs:
    a = AttentionArgs(
        heads=_get(m, "heads", int), kv_heads=_get(m, "kv_heads", int), dim=_get(m, "dim", int),
        vdim=_get(m, "vdim", int), scale=_get(m, "scale", float),
        rot_dims=_get(m, "rot.dims", int, 0), rot_base=_get(m, "rot.base", float, 10000.0),
        rot_factor=_get(m, "rot.scaling.factor", float, 1.0),
    )
    if a.heads <= 0 or a.kv_heads <= 0 or a.heads % a.kv_heads:
        raise ConfigError(f"config.json: {where}: heads={a.heads} is not a multiple of kv_heads={a.kv_heads}")
    if a.vdim != a.dim:
        raise ConfigError(f"config.json: {where}: the values are the keys, so vdim={a.vdim} must equal dim={a.dim}")
    if a.rot_dims % 2 or not 0 <= a.rot_dims <= a.dim:
        raise ConfigError(f"config.json: {where}: rot.dims={a.rot_dims} must be even and at most dim={a.dim}")
    if not a.rot_factor > 0:
        raise ConfigError(f"config.json: {where}: rot.scaling.factor must be positive")
    return a


def _moe_args(m: Mapping[str, Any], where: str) -> MoeArgs:
    kind = m.get("kind", "moe")
    if kind != "moe":
        raise ConfigError(f"config.json: {where}: feed-forward kind {kind!r} is not supported (supported: 'moe')")
    a = MoeArgs(experts=_get(m, "router.experts", int), top=_get(m, "router.top", int), ff=_get(m, "expert.ff", int))
    if not 1 <= a.top <= a.experts:
        raise ConfigError(f"config.json: {where}: router.top={a.top} must be between 1 and experts={a.experts}")
    return a


class BuderaxArchitecture:
    name = "Buderax"

    def parse(self, config: Mapping[str, Any]) -> BuderaxArgs:
        layers = []
        for i, l in enumerate(_get(config, "layers")):
            kind = _get(l, "type", str)
            if kind != "attention":
                raise ConfigError(f"config.json: layers[{i}].type {kind!r} is not supported (supported: 'attention')")
            mlp = l.get("mlp")
            layers.append(BuderaxLayer(kind, _attention_args(_get(l, "mixer"), f"layers[{i}].mixer"),
                                       _moe_args(mlp, f"layers[{i}].mlp") if mlp is not None else None))
        loop = None
        if config.get("loop") is not None:
            loop = LoopArgs(_get(config, "loop.start", int), _get(config, "loop.stop", int),
                            _get(config, "loop.times", int))
            if not (0 <= loop.start < loop.stop <= len(layers)) or loop.times < 1:
                raise ConfigError(
                    f"config.json: loop start={loop.start} stop={loop.stop} times={loop.times} does not fit"
                    f" {len(layers)} layers")
        return BuderaxArgs(
            architecture=self.name, width=_get(config, "width", int), vocab=_get(config, "vocab", int),
            embedding_scale=_get(config, "embedding.scale", float, 1.0), norm_eps=_get(config, "norm.eps", float),
            layers=tuple(layers), loop=loop,
            extra={k: config[k] for k in ("bos_token_id", "eos_token_id") if k in config},
        )

    def to_hf_config(self, args: BuderaxArgs) -> dict:
        def layer(l: BuderaxLayer) -> dict:
            m = l.mixer
            rot: dict = {"base": m.rot_base, "dims": m.rot_dims}
            if m.rot_factor != 1.0:
                rot["scaling"] = {"factor": m.rot_factor}
            return {
                "type": l.type,
                "mixer": {"heads": m.heads, "kv_heads": m.kv_heads, "dim": m.dim, "vdim": m.vdim, "scale": m.scale,
                          "rot": rot},
                "mlp": None if l.mlp is None else {
                    "kind": "moe", "expert": {"ff": l.mlp.ff},
                    "router": {"experts": l.mlp.experts, "top": l.mlp.top}},
            }

        out = {
            "architecture": self.name, "width": args.width, "vocab": args.vocab,
            "embedding": {"scale": args.embedding_scale}, "norm": {"eps": args.norm_eps},
            "layers": [layer(l) for l in args.layers],
        }
        if args.loop is not None:
            out["loop"] = {"start": args.loop.start, "stop": args.loop.stop, "times": args.loop.times}
        out.update(args.extra)
        return out

    def layout(self, args: BuderaxArgs) -> ModelLayout:
        bare = {"weight": ""}  # a part's one tensor is named by the prefix alone

        def norm(prefix: str) -> PartSpec:
            return PartSpec("rmsnorm", prefix, dict(dim=args.width, eps=args.norm_eps, unit_offset=True, names=bare))

        layers = []
        for i, l in enumerate(args.layers):
            m = l.mixer
            rope = PartSpec("rope", options=dict(
                head_dim=m.dim, rotary_dim=m.rot_dims, theta=m.rot_base, pairing="interleaved",
                linear_factor=m.rot_factor))
            mixer = PartSpec("attention", f"l{i}.mix", dict(
                dim=args.width, n_heads=m.heads, n_kv_heads=m.kv_heads, head_dim=m.dim, scale=m.scale, window=None,
                position=rope, value_from_key=True, output_gate=True, exact_weights=True,
                names={"q_proj.weight": "q", "k_proj.weight": "k", "o_proj.weight": "o", "gate_proj.weight": "g"}))
            ffn = None
            if l.mlp is not None:
                ffn = PartSpec("moe", f"l{i}.mlp", dict(
                    dim=args.width, hidden_dim=l.mlp.ff, n_experts=l.mlp.experts, top=l.mlp.top,
                    names={"router.weight": "router", "router.bias": "router.b", "expert": "e{}",
                           "gate_proj.weight": "gate", "up_proj.weight": "up", "down_proj.weight": "down"}))
            layers.append(LayerSpec(mixer=mixer, ffn=ffn, mixer_norm=norm(f"l{i}.norm1"), ffn_norm=None,
                                    arrangement="parallel"))
        n = len(layers)
        injections: Tuple[PartSpec, ...] = ()
        if args.loop is None:
            order = [RunEntry(i) for i in range(n)]
        else:
            lp = args.loop
            injections = (PartSpec("loop_input", "loop", dict(dim=args.width, times=lp.times, names={"step": "step"})),)
            order = [RunEntry(i) for i in range(lp.start)]
            for t in range(lp.times):
                order += [RunEntry(i, inject=(0, t) if i == lp.start else None) for i in range(lp.start, lp.stop)]
            order += [RunEntry(i) for i in range(lp.stop, n)]
        return ModelLayout(
            dim=args.width, vocab_size=args.vocab,
            embed=PartSpec("embedding", "embed", dict(vocab_size=args.vocab, dim=args.width,
                                                      scale=args.embedding_scale, names=bare)),
            layers=tuple(layers), order=tuple(order), final_norm=norm("final.norm"),
            head=PartSpec("lm_head", "head", dict(vocab_size=args.vocab, dim=args.width, tied_to=None, names=bare)),
            injections=injections,
        )


BUDERAX = register_architecture(BuderaxArchitecture())
