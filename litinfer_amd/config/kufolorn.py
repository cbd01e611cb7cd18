"""Typed configuration of the Kufolorn decoder, read from config.json, and the model as data.

config.json: `vocab`, `width`, `norm.eps`, optional `logit_softcap`, and `layers`, a list whose entries have `type`
(`delta` or `parallel`), the mixer's sizes and constants under `mixer`, and `mlp` (null, {kind: dense, ff} or
{kind: moe, expert: {ff, limit}, router: {experts, top, identity, groups: {count, keep}}}).

The model: the token's embedding row; per layer x += norm1(mixer(x)) and, if the layer has one,
x += norm2(feed_forward(x)): the sublayers read the stream itself, and only their outputs are normed (RMS norms whose
weights are stored around zero, 1 + w); a final norm of the same kind, the embedding table as the head, and a tanh cap
on the logits.
`delta`: a gated delta-rule mixer (`parts/delta.py`).  `parallel`: softmax attention with biases, an RMS norm over the
whole query and key projections, half-split rotation with linear scaling of the frequencies, a sink a head and a
sigmoid gate a head (`parts/masked_attention.py`) beside a retention (`parts/retention.py`), added with factors.
Dense feed-forward: Wdown(gelu_tanh(Wgate x) * Wup x).  Routed: softmax over all router outputs, a correction of the
choice, groups of neighbours scored by their largest choice value, weights not renormalised, identity experts, experts
with a clamped activation (`parts/moe.py`).
Tensor names: embed, final.norm and per layer i `l<i>.norm1|norm2`, `l<i>.mix.*` (`.left.*`, `.right.*` for the two
mixers of a parallel layer), `l<i>.mlp.gate|up|down` or `l<i>.mlp.router|correction|e<j>.gate|up|down`.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Dict, Optional, Tuple

from .qwen2 import ConfigError
from .spec import ExecEntry, LayerSpec, ModelSpec, PartSpec
from .tovasun import DEFAULT_MAX_POSITIONS, _number, _pos_int

MIXER_TYPES = ("delta", "parallel")


def _obj(d: Any, where: str) -> Dict[str, Any]:
    if not isinstance(d, dict):
        raise ConfigError(f"config.json: {where} must be an object")
    return d


@dataclass(frozen=True)
class RotationConfig:
    base: float
    dims: int
    factor: float                       # every frequency is divided by it (1: no scaling)

    @classmethod
    def from_dict(cls, d: Any, where: str, head_dim: int) -> "RotationConfig":
        d = _obj(d, where)
        base, dims = _number(d, "base", where), _pos_int(d, "dims", where)
        if base <= 0 or dims % 2 or dims > head_dim:
            raise ConfigError(f"config.json: {where}: base must be positive, dims even and at most the head size {head_dim}")
        factor = 1.0
        if d.get("scaling") is not None:
            factor = _number(_obj(d["scaling"], where + ".scaling"), "factor", where + ".scaling")
            if factor <= 0:
                raise ConfigError(f"config.json: {where}.scaling.factor must be positive")
        return cls(base, dims, factor)


@dataclass(frozen=True)
class DeltaConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    conv: int

    @classmethod
    def from_dict(cls, d: Any, where: str) -> "DeltaConfig":
        d = _obj(d, where)
        heads, dim = _pos_int(d, "heads", where), _pos_int(d, "dim", where)
        kvh = _pos_int(d, "kv_heads", where) if d.get("kv_heads") is not None else heads
        if heads % kvh:
            raise ConfigError(f"config.json: {where}: {heads} heads are not a multiple of {kvh} kv heads")
        return cls(heads, kvh, dim, _pos_int(d, "vdim", where) if d.get("vdim") is not None else dim,
                   _pos_int(d, "conv", where) if d.get("conv") is not None else 1)


@dataclass(frozen=True)
class SinkAttentionConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    rot: RotationConfig

    @classmethod
    def from_dict(cls, d: Any, where: str) -> "SinkAttentionConfig":
        d = _obj(d, where)
        heads, dim = _pos_int(d, "heads", where), _pos_int(d, "dim", where)
        kvh = _pos_int(d, "kv_heads", where) if d.get("kv_heads") is not None else heads
        if heads % kvh:
            raise ConfigError(f"config.json: {where}: {heads} heads are not a multiple of {kvh} kv heads")
        return cls(heads, kvh, dim, _pos_int(d, "vdim", where) if d.get("vdim") is not None else dim,
                   _number(d, "scale", where), RotationConfig.from_dict(d.get("rot"), where + ".rot", dim))


@dataclass(frozen=True)
class RetentionConfig:
    heads: int
    dim: int
    vdim: int
    decay: Tuple[float, ...]
    rot: RotationConfig

    @classmethod
    def from_dict(cls, d: Any, where: str) -> "RetentionConfig":
        d = _obj(d, where)
        heads, dim = _pos_int(d, "heads", where), _pos_int(d, "dim", where)
        decay = d.get("decay")
        if not isinstance(decay, list) or len(decay) != heads or any(isinstance(x, bool) or not isinstance(x, (int, float)) for x in decay):
            raise ConfigError(f"config.json: {where}.decay must be a list of {heads} numbers, one a head")
        return cls(heads, dim, _pos_int(d, "vdim", where) if d.get("vdim") is not None else dim,
                   tuple(float(x) for x in decay), RotationConfig.from_dict(d.get("rot"), where + ".rot", dim))


@dataclass(frozen=True)
class ParallelConfig:
    left: SinkAttentionConfig
    right: RetentionConfig
    left_scale: float
    right_scale: float

    @classmethod
    def from_dict(cls, d: Any, where: str) -> "ParallelConfig":
        d = _obj(d, where)
        return cls(SinkAttentionConfig.from_dict(d.get("left"), where + ".left"), RetentionConfig.from_dict(d.get("right"), where + ".right"),
                   _number(d, "left_scale", where), _number(d, "right_scale", where))


@dataclass(frozen=True)
class FeedForwardConfig:
    kind: str                    # "dense" or "moe"
    ff: int
    limit: float = 0.0
    experts: int = 0
    identity: int = 0
    top: int = 0
    groups: int = 1
    keep_groups: int = 1

    @classmethod
    def from_dict(cls, d: Any, where: str) -> "FeedForwardConfig":
        d = _obj(d, where)
        kind = d.get("kind")
        if kind == "dense":
            return cls("dense", _pos_int(d, "ff", where))
        if kind != "moe":
            raise ConfigError(f"config.json: {where}.kind {kind!r} is not supported ('dense' or 'moe')")
        expert, router = _obj(d.get("expert"), where + ".expert"), _obj(d.get("router"), where + ".router")
        experts, top = _pos_int(router, "experts", where + ".router"), _pos_int(router, "top", where + ".router")
        identity = _pos_int(router, "identity", where + ".router", allow_zero=True) if router.get("identity") is not None else 0
        groups = keep = 1
        if router.get("groups") is not None:
            g = _obj(router["groups"], where + ".router.groups")
            groups, keep = _pos_int(g, "count", where + ".router.groups"), _pos_int(g, "keep", where + ".router.groups")
        n = experts + identity
        if n % groups or keep > groups:
            raise ConfigError(f"config.json: {where}.router: {n} router outputs in {groups} groups of which {keep} are kept")
        if top > keep * (n // groups):
            raise ConfigError(f"config.json: {where}.router: {top} choices among the {keep * (n // groups)} outputs of the kept groups")
        limit = _number(expert, "limit", where + ".expert")
        if limit <= 0:
            raise ConfigError(f"config.json: {where}.expert.limit must be positive")
        return cls("moe", _pos_int(expert, "ff", where + ".expert"), limit, experts, identity, top, groups, keep)


@dataclass(frozen=True)
class KufolornLayer:
    type: str
    mixer: Any                   # DeltaConfig | ParallelConfig
    mlp: Optional[FeedForwardConfig]


@dataclass(frozen=True)
class KufolornConfig:
    vocab: int
    width: int
    eps: float
    layers: Tuple[KufolornLayer, ...]
    logit_softcap: float
    max_positions: int
    eos_token_ids: Tuple[int, ...]
    raw: Any = None

    architecture = "Kufolorn"

    @classmethod
    def from_dict(cls, cfg: Dict[str, Any]) -> "KufolornConfig":
        vocab, width = _pos_int(cfg, "vocab", "config"), _pos_int(cfg, "width", "config")
        eps = _number(cfg.get("norm") or {}, "eps", "norm")
        if eps < 0:
            raise ConfigError("config.json: norm.eps must not be negative")
        raw_layers = cfg.get("layers")
        if not isinstance(raw_layers, list) or not raw_layers:
            raise ConfigError("config.json: 'layers' must be a list with at least one layer")
        layers = []
        for i, L in enumerate(raw_layers):
            where = f"layers[{i}]"
            L = _obj(L, where)
            kind = L.get("type")
            if kind not in MIXER_TYPES:
                raise ConfigError(f"config.json: {where}: unknown mixer type {kind!r} (known: {', '.join(MIXER_TYPES)})")
            mixer = (DeltaConfig if kind == "delta" else ParallelConfig).from_dict(L.get("mixer"), where + ".mixer")
            mlp = FeedForwardConfig.from_dict(L["mlp"], where + ".mlp") if L.get("mlp") is not None else None
            layers.append(KufolornLayer(kind, mixer, mlp))
        cap = cfg.get("logit_softcap")
        cap = 0.0 if cap is None else _number(cfg, "logit_softcap", "config")
        if cap < 0:
            raise ConfigError("config.json: logit_softcap must not be negative")
        eos = cfg.get("eos_token_id")
        eos_ids = () if eos is None else tuple(int(e) for e in (eos if isinstance(eos, list) else [eos]))
        maxpos = cfg.get("max_positions")
        maxpos = DEFAULT_MAX_POSITIONS if maxpos is None else _pos_int(cfg, "max_positions", "config")
        return cls(vocab=vocab, width=width, eps=eps, layers=tuple(layers), logit_softcap=cap, max_positions=maxpos,
                   eos_token_ids=tuple(e for e in eos_ids if e >= 0), raw=cfg)


def _rotation_spec(rot: RotationConfig, head_dim: int) -> PartSpec:
    args: Dict[str, Any] = {"head_dim": head_dim, "rotary_dim": rot.dims, "theta": rot.base, "layout": "half"}
    if rot.factor != 1.0:
        args["scaling"] = {"kind": "linear", "factor": rot.factor}
    return PartSpec("rope_pairs", "", args)


def _mixer_spec(c: KufolornConfig, L: KufolornLayer, prefix: str) -> PartSpec:
    m = L.mixer
    if L.type == "delta":
        return PartSpec("gated_delta", prefix, {"hidden_size": c.width, "num_heads": m.heads, "num_kv_heads": m.kv_heads,
                                                "head_dim": m.dim, "value_dim": m.vdim, "conv": m.conv, "eps": c.eps})
    a, r = m.left, m.right
    left = PartSpec("masked_attention", prefix + "left.", {
        "hidden_size": c.width, "num_heads": a.heads, "num_kv_heads": a.kv_heads, "head_dim": a.dim, "value_dim": a.vdim,
        "scale": a.scale, "qk_norm": True, "eps": c.eps, "bias": True, "sink": True, "head_gate": True,
        "position": _rotation_spec(a.rot, a.dim)})
    right = PartSpec("retention", prefix + "right.", {
        "hidden_size": c.width, "num_heads": r.heads, "head_dim": r.dim, "value_dim": r.vdim, "decay": list(r.decay),
        "eps": c.eps, "position": _rotation_spec(r.rot, r.dim)})
    return PartSpec("mixer_pair", prefix, {"left": left, "right": right, "left_scale": m.left_scale, "right_scale": m.right_scale})


def _mlp_spec(c: KufolornConfig, f: FeedForwardConfig, prefix: str) -> PartSpec:
    if f.kind == "dense":
        return PartSpec("gated_mlp", prefix, {"hidden_size": c.width, "intermediate_size": f.ff, "activation": "gelu_tanh",
                                              "names": {"gate": "gate", "up": "up", "down": "down"}})
    return PartSpec("routed_mlp", prefix, {
        "hidden_size": c.width, "intermediate_size": f.ff, "experts": f.experts, "identity": f.identity, "top": f.top,
        "activation": "clamped_swiglu", "limit": f.limit, "scores": "softmax", "correction": True, "router_bias": False,
        "groups": f.groups, "keep_groups": f.keep_groups, "group_score": "max", "normalize": False})


def kufolorn_model_spec(c: KufolornConfig) -> ModelSpec:
    layers = []
    for i, L in enumerate(c.layers):
        p = f"l{i}."

        def norm(name):
            return PartSpec("rmsnorm", p, {"size": c.width, "eps": c.eps, "param": name, "offset": 1.0})
        # no norm before a sublayer: the sandwich arrangement without its `norm1` and `norm2`
        parts: Dict[str, Optional[PartSpec]] = {"mixer": _mixer_spec(c, L, p + "mix."), "norm1b": norm("norm1")}
        if L.mlp is not None:
            parts["feed_forward"] = _mlp_spec(c, L.mlp, p + "mlp.")
            parts["norm2b"] = norm("norm2")
        layers.append(LayerSpec(block="sandwich", parts=parts))
    return ModelSpec(
        architecture=c.architecture, hidden_size=c.width, vocab_size=c.vocab, max_positions=c.max_positions,
        embedding=PartSpec("token_embedding", "", {"vocab_size": c.vocab, "hidden_size": c.width, "param": "embed"}),
        layers=tuple(layers), order=tuple(ExecEntry(i) for i in range(len(layers))),
        final_norm=PartSpec("rmsnorm", "final.", {"size": c.width, "eps": c.eps, "param": "norm", "offset": 1.0}),
        head=PartSpec("linear_head", "", {"vocab_size": c.vocab, "hidden_size": c.width, "tied_to": "embed",
                                          "softcap": c.logit_softcap}),
        eos_token_ids=c.eos_token_ids)
