"""Typed configuration of the Nusuvik decoder, read from config.json, and the model as data.

config.json: `vocab`, `width`, `norm.eps`, `embedding.bigram` {buckets, mul_prev, mul_cur} (optional), `layers` (a
list; each entry has `type` = `latent_attention`, the mixer's sizes and constants under `mixer`, and `mlp` = null,
{kind: dense, ff} or {kind: moe, expert: {ff}, router: {experts, top, groups: {count, keep}}}), optional `loop`
{start, stop, times} (layers start..stop-1 are passed `times` times with the same weights, every pass with a cache
of its own) and optional `logit_softcap`.

The model: the token's embedding row plus a row of a hashed table that the token and its predecessor choose; per
layer ONE layer norm (weight and bias) whose output both the mixer and the feed-forward read, their outputs added to
the stream together; before every pass of the loop the stream becomes `loop.in` [x ; embedding output]; a final layer
norm, a linear head and a tanh cap on the logits.  The mixer is attention over a compressed cache with queries that
go through a latent of their own, half-split rotation of the rotated part and a sigmoid gate a head.
Tensor names: embed, bigram, head, final.norm(.b), loop.in, and per layer i `l<i>.norm1(.b)`,
`l<i>.mix.dq|dq.norm|uq|dkv|dkv.norm|uk|uv|g|o`, `l<i>.mlp.up(.b)|down(.b)` or
`l<i>.mlp.router|correction|e<j>.gate|up|down`.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Dict, Optional, Tuple

from .qwen2 import ConfigError
from .spec import ExecEntry, LayerSpec, ModelSpec, PartSpec
from .tovasun import DEFAULT_MAX_POSITIONS, RotaryConfig, _number, _pos_int

MIXER_TYPES = ("latent_attention",)


@dataclass(frozen=True)
class LatentMixerConfig:
    heads: int
    dim: int
    rot_dim: int
    vdim: int
    kv_rank: int
    q_rank: int
    scale: float
    rot: RotaryConfig

    @classmethod
    def from_dict(cls, kind: str, d: Dict[str, Any], where: str) -> "LatentMixerConfig":
        if kind not in MIXER_TYPES:
            raise ConfigError(f"config.json: {where}: unknown mixer type {kind!r} (known: {', '.join(MIXER_TYPES)})")
        if not isinstance(d, dict):
            raise ConfigError(f"config.json: {where}.mixer must be an object")
        heads, dim = _pos_int(d, "heads", where), _pos_int(d, "dim", where)
        vdim = _pos_int(d, "vdim", where) if d.get("vdim") is not None else dim
        rot_dim, rank, q_rank = _pos_int(d, "rot_dim", where), _pos_int(d, "kv_rank", where), _pos_int(d, "q_rank", where)
        rot = RotaryConfig.from_dict(d.get("rot"), where + ".rot")
        if rot.dims != rot_dim:
            raise ConfigError(f"config.json: {where}: rot.dims ({rot.dims}) must equal rot_dim ({rot_dim})")
        if rot.scaling is not None:
            raise ConfigError(f"config.json: {where}.rot.scaling is not part of this design")
        return cls(heads=heads, dim=dim, rot_dim=rot_dim, vdim=vdim, kv_rank=rank, q_rank=q_rank,
                   scale=_number(d, "scale", where), rot=rot)


@dataclass(frozen=True)
class FeedForwardConfig:
    kind: str                    # "dense" or "moe"
    ff: int
    experts: int = 0
    top: int = 0
    groups: int = 1
    keep_groups: int = 1

    @classmethod
    def from_dict(cls, d: Dict[str, Any], where: str) -> "FeedForwardConfig":
        if not isinstance(d, dict):
            raise ConfigError(f"config.json: {where} must be an object or null")
        kind = d.get("kind")
        if kind == "dense":
            return cls("dense", _pos_int(d, "ff", where))
        if kind != "moe":
            raise ConfigError(f"config.json: {where}.kind {kind!r} is not supported ('dense' or 'moe')")
        expert, router = d.get("expert"), d.get("router")
        if not isinstance(expert, dict) or not isinstance(router, dict):
            raise ConfigError(f"config.json: {where} needs the objects 'expert' and 'router'")
        experts, top = _pos_int(router, "experts", where + ".router"), _pos_int(router, "top", where + ".router")
        groups = keep = 1
        if router.get("groups") is not None:
            g = router["groups"]
            if not isinstance(g, dict):
                raise ConfigError(f"config.json: {where}.router.groups must be an object")
            groups, keep = _pos_int(g, "count", where + ".router.groups"), _pos_int(g, "keep", where + ".router.groups")
        if experts % groups or keep > groups:
            raise ConfigError(f"config.json: {where}.router: {experts} experts in {groups} groups of which {keep} are kept")
        if top > keep * (experts // groups):
            raise ConfigError(f"config.json: {where}.router: {top} choices among the {keep * (experts // groups)} "
                              f"experts of the kept groups")
        return cls("moe", _pos_int(expert, "ff", where + ".expert"), experts, top, groups, keep)


@dataclass(frozen=True)
class NusuvikLayer:
    mixer: LatentMixerConfig
    mlp: Optional[FeedForwardConfig]


@dataclass(frozen=True)
class NusuvikConfig:
    vocab: int
    width: int
    eps: float
    layers: Tuple[NusuvikLayer, ...]
    loop: Optional[Tuple[int, int, int]]        # (start, stop, times)
    bigram: Optional[Tuple[int, int, int]]      # (buckets, mul_prev, mul_cur)
    logit_softcap: float
    max_positions: int
    eos_token_ids: Tuple[int, ...]
    raw: Any = None

    architecture = "Nusuvik"

    @classmethod
    def from_dict(cls, cfg: Dict[str, Any]) -> "NusuvikConfig":
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
            if not isinstance(L, dict):
                raise ConfigError(f"config.json: {where} must be an object")
            mixer = LatentMixerConfig.from_dict(L.get("type"), L.get("mixer"), where)
            mlp = FeedForwardConfig.from_dict(L["mlp"], where + ".mlp") if L.get("mlp") is not None else None
            layers.append(NusuvikLayer(mixer, mlp))
        loop = cfg.get("loop")
        if loop is not None:
            start = _pos_int(loop, "start", "loop", allow_zero=True)
            stop, times = _pos_int(loop, "stop", "loop", allow_zero=True), _pos_int(loop, "times", "loop")
            if not 0 <= start <= stop <= len(layers):
                raise ConfigError(f"config.json: loop {start}..{stop} lies outside the {len(layers)} layers")
            loop = (start, stop, times) if stop > start else None
        bigram = (cfg.get("embedding") or {}).get("bigram")
        if bigram is not None:
            bigram = (_pos_int(bigram, "buckets", "embedding.bigram"),
                      _pos_int(bigram, "mul_prev", "embedding.bigram", allow_zero=True),
                      _pos_int(bigram, "mul_cur", "embedding.bigram", allow_zero=True))
        cap = cfg.get("logit_softcap")
        cap = 0.0 if cap is None else _number(cfg, "logit_softcap", "config")
        if cap < 0:
            raise ConfigError("config.json: logit_softcap must not be negative")
        eos = cfg.get("eos_token_id")
        eos_ids = () if eos is None else tuple(int(e) for e in (eos if isinstance(eos, list) else [eos]))
        maxpos = cfg.get("max_positions")
        maxpos = DEFAULT_MAX_POSITIONS if maxpos is None else _pos_int(cfg, "max_positions", "config")
        return cls(vocab=vocab, width=width, eps=eps, layers=tuple(layers), loop=loop, bigram=bigram, logit_softcap=cap,
                   max_positions=maxpos, eos_token_ids=tuple(e for e in eos_ids if e >= 0), raw=cfg)


def _mixer_spec(c: NusuvikConfig, m: LatentMixerConfig, prefix: str) -> PartSpec:
    position = PartSpec("rope_pairs", "", {"head_dim": m.rot_dim, "rotary_dim": m.rot.dims, "theta": m.rot.base,
                                           "layout": "half"})
    return PartSpec("latent_attention", prefix, {
        "hidden_size": c.width, "num_heads": m.heads, "head_dim": m.dim, "rot_dim": m.rot_dim, "value_dim": m.vdim,
        "kv_rank": m.kv_rank, "q_rank": m.q_rank, "head_gate": True, "scale": m.scale, "eps": c.eps, "position": position})


def _mlp_spec(c: NusuvikConfig, f: FeedForwardConfig, prefix: str) -> PartSpec:
    if f.kind == "dense":
        return PartSpec("gelu_mlp", prefix, {"hidden_size": c.width, "intermediate_size": f.ff, "biases": True})
    return PartSpec("routed_mlp", prefix, {
        "hidden_size": c.width, "intermediate_size": f.ff, "experts": f.experts, "top": f.top, "activation": "swiglu",
        "scores": "sigmoid", "correction": True, "router_bias": False, "groups": f.groups, "keep_groups": f.keep_groups})


def nusuvik_model_spec(c: NusuvikConfig) -> ModelSpec:
    n = len(c.layers)
    layers = []
    for i, L in enumerate(c.layers):
        p = f"l{i}."
        parts: Dict[str, Optional[PartSpec]] = {
            "norm1": PartSpec("layernorm", p, {"size": c.width, "eps": c.eps, "param": "norm1"}),
            "mixer": _mixer_spec(c, L.mixer, p + "mix.")}
        if L.mlp is not None:
            parts["feed_forward"] = _mlp_spec(c, L.mlp, p + "mlp.")
        layers.append(LayerSpec(block="parallel", parts=parts))
    order, injections = [], ()
    if c.loop:
        start, stop, times = c.loop
        injections = (PartSpec("loop_mix", "loop.", {"times": times, "hidden_size": c.width, "param": "in"}),)
        order += [ExecEntry(i) for i in range(start)]
        for t in range(times):
            order += [ExecEntry(i, inject=(0, t) if i == start else None) for i in range(start, stop)]
        order += [ExecEntry(i) for i in range(stop, n)]
    else:
        order = [ExecEntry(i) for i in range(n)]
    emb_args = {"vocab_size": c.vocab, "hidden_size": c.width, "param": "embed"}
    if c.bigram:
        embedding = PartSpec("pair_hash_embedding", "", {**emb_args, "buckets": c.bigram[0], "mul_prev": c.bigram[1],
                                                         "mul_cur": c.bigram[2], "pair_param": "bigram"})
    else:
        embedding = PartSpec("token_embedding", "", emb_args)
    return ModelSpec(
        architecture=c.architecture, hidden_size=c.width, vocab_size=c.vocab, max_positions=c.max_positions,
        embedding=embedding, layers=tuple(layers), order=tuple(order),
        final_norm=PartSpec("layernorm", "final.", {"size": c.width, "eps": c.eps, "param": "norm"}),
        head=PartSpec("linear_head", "", {"vocab_size": c.vocab, "hidden_size": c.width, "param": "head",
                                          "softcap": c.logit_softcap}),
        eos_token_ids=c.eos_token_ids, injections=injections)
