"""Typed configuration of the Vovalix decoder, read from config.json.

The file lists the layers one by one; every size and every constant that can differ between
models comes from it (or, for the one size the file leaves out, from a tensor's shape):

    {"architecture": "Vovalix", "vocab": V, "width": H, "norm": {"eps": e}, "logit_scale": s,
     "layers": [{"type": "attention" | "gla" | "delta", "mixer": {...}, "mlp": {...} | null,
                 "weights_of": j (optional)}, ...]}

``attention`` mixers give ``heads, kv_heads, dim, vdim, scale`` and ``mask {size}``; ``gla``
mixers ``heads, dim, vdim, tau`` (``rank``, the width of the decay's low-rank product, is the
first size of the layer's ``mix.a1`` tensor unless the file names it); ``delta`` mixers ``heads,
kv_heads, dim, vdim, conv``.  A feed-forward is ``{"kind": "moe", "expert": {ff, limit}, "router":
{experts, top, groups {count, keep}}, "shared": {ff, limit}}``.  A layer with ``weights_of: j``
runs layer j's tensors with a cache or state of its own.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Callable, Mapping

from .model_config import ConfigError, _require


def _mapping(d: Mapping[str, Any], key: str, where: str) -> Mapping[str, Any]:
    value = d.get(key)
    if not isinstance(value, Mapping):
        raise ConfigError(f"config.json: {where}{key!r} must be an object")
    return value


@dataclass(frozen=True)
class ChunkedAttentionConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    chunk: int  # 0: every earlier token is seen

    @classmethod
    def from_dict(cls, d: Mapping[str, Any], where: str) -> "ChunkedAttentionConfig":
        heads, kv = _require(d, "heads", int), _require(d, "kv_heads", int)
        dim, vdim = _require(d, "dim", int), _require(d, "vdim", int)
        if min(heads, kv, dim, vdim) <= 0 or heads % kv:
            raise ConfigError(f"config.json: {where}sizes must be positive and heads a multiple of kv_heads "
                              f"(heads {heads}, kv_heads {kv}, dim {dim}, vdim {vdim})")
        chunk = 0
        if d.get("mask") is not None:
            chunk = _require(_mapping(d, "mask", where), "size", int)
            if chunk <= 0:
                raise ConfigError(f"config.json: {where}mask.size must be positive, got {chunk}")
        return cls(heads, kv, dim, vdim, _require(d, "scale", float), chunk)


@dataclass(frozen=True)
class GatedLinearAttentionConfig:
    heads: int
    dim: int
    vdim: int
    tau: float
    rank: int

    @classmethod
    def from_dict(cls, d: Mapping[str, Any], where: str) -> "GatedLinearAttentionConfig":
        heads, dim, vdim = _require(d, "heads", int), _require(d, "dim", int), _require(d, "vdim", int)
        tau = _require(d, "tau", float)
        if d.get("rank") is None:
            raise ConfigError(f"config.json: {where}rank is neither in the file nor given by a tensor's shape")
        rank = _require(d, "rank", int)
        if min(heads, dim, vdim, rank) <= 0 or not tau > 0:
            raise ConfigError(f"config.json: {where}sizes and tau must be positive: {dict(d)}")
        return cls(heads, dim, vdim, tau, rank)


@dataclass(frozen=True)
class DeltaRuleConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    conv: int

    @classmethod
    def from_dict(cls, d: Mapping[str, Any], where: str) -> "DeltaRuleConfig":
        c = cls(*(_require(d, k, int) for k in ("heads", "kv_heads", "dim", "vdim", "conv")))
        if min(c.heads, c.kv_heads, c.dim, c.vdim) <= 0 or c.heads % c.kv_heads or c.conv < 1:
            raise ConfigError(f"config.json: {where}sizes do not fit together: {dict(d)}")
        return c


@dataclass(frozen=True)
class RoutedFeedForwardConfig:
    experts: int
    top: int
    groups: int
    keep: int
    ff: int
    limit: float
    shared_ff: int  # 0: no shared expert
    shared_limit: float

    @classmethod
    def from_dict(cls, d: Mapping[str, Any], where: str) -> "RoutedFeedForwardConfig":
        if d.get("kind") != "moe":
            raise ConfigError(f"config.json: {where}kind {d.get('kind')!r} is not supported (supported: 'moe')")
        expert, router = _mapping(d, "expert", where), _mapping(d, "router", where)
        experts, top = _require(router, "experts", int), _require(router, "top", int)
        groups = keep = 1
        if router.get("groups") is not None:
            g = _mapping(router, "groups", where + "router.")
            groups, keep = _require(g, "count", int), _require(g, "keep", int)
        ff, limit = _require(expert, "ff", int), _require(expert, "limit", float)
        shared_ff, shared_limit = 0, limit
        if d.get("shared") is not None:
            sh = _mapping(d, "shared", where)
            shared_ff, shared_limit = _require(sh, "ff", int), _require(sh, "limit", float)
            if shared_ff <= 0:
                raise ConfigError(f"config.json: {where}shared.ff must be positive")
        if experts <= 0 or not 0 < top <= experts or ff <= 0 or groups <= 0 or experts % groups \
                or not 0 < keep <= groups:
            raise ConfigError(f"config.json: {where}router and expert sizes do not fit together: {dict(d)}")
        return cls(experts, top, groups, keep, ff, limit, shared_ff, shared_limit)


@dataclass(frozen=True)
class VovalixLayerConfig:
    type: str
    mixer: ChunkedAttentionConfig | GatedLinearAttentionConfig | DeltaRuleConfig
    mlp: RoutedFeedForwardConfig | None
    weights_of: int | None


_MIXERS = {"attention": ChunkedAttentionConfig, "gla": GatedLinearAttentionConfig, "delta": DeltaRuleConfig}


@dataclass(frozen=True)
class VovalixConfig:
    vocab: int
    width: int
    eps: float
    logit_scale: float
    layers: tuple[VovalixLayerConfig, ...]
    max_position_embeddings: int
    eos_token_ids: tuple[int, ...] = ()

    @classmethod
    def from_dict(cls, d: Mapping[str, Any]) -> "VovalixConfig":
        vocab, width = _require(d, "vocab", int), _require(d, "width", int)
        if vocab <= 0 or width <= 0:
            raise ConfigError("config.json: vocab and width must be positive")
        eps = _require(_mapping(d, "norm", ""), "eps", float)
        raw_layers = d.get("layers")
        if not isinstance(raw_layers, list) or not raw_layers:
            raise ConfigError("config.json: 'layers' must be a list of at least one layer")
        layers: list[VovalixLayerConfig] = []
        for i, raw in enumerate(raw_layers):
            where = f"layers[{i}]."
            kind = raw.get("type")
            if kind not in _MIXERS:
                raise ConfigError(f"config.json: {where}type {kind!r} is not supported (supported: {sorted(_MIXERS)})")
            source = raw.get("weights_of")
            if source is None:
                mixer = _MIXERS[kind].from_dict(_mapping(raw, "mixer", where), where + "mixer.")
                mlp = None if raw.get("mlp") is None else RoutedFeedForwardConfig.from_dict(raw["mlp"], where + "mlp.")
            else:
                source = int(source)
                if not 0 <= source < i:
                    raise ConfigError(f"config.json: {where}weights_of must name an earlier layer")
                if layers[source].weights_of is not None:  # a layer that borrows in turn: its owner
                    source = layers[source].weights_of
                # the tensors are the owner's, so the owner's sizes are the ones that count
                kind, mixer, mlp = layers[source].type, layers[source].mixer, layers[source].mlp
            layers.append(VovalixLayerConfig(kind, mixer, mlp, source))
        eos = d.get("eos_token_id")
        eos_ids = () if eos is None else tuple(int(e) for e in (eos if isinstance(eos, (list, tuple)) else [eos]))
        return cls(vocab, width, eps, float(d.get("logit_scale", 1.0)), tuple(layers),
                   int(d.get("max_position_embeddings") or 131072), eos_ids)


def complete_from_tensor_shapes(config: Mapping[str, Any],
                                shape_of: Callable[[str], "tuple[int, ...] | None"]) -> dict:
    """config.json with the sizes that only the checkpoint's tensor shapes give filled in: the
    ``rank`` of every ``gla`` mixer is the first size of ``l<i>.mix.a1`` (of the layer whose
    tensors it uses)."""
    out = dict(config)
    layers = []
    for i, raw in enumerate(config.get("layers") or []):
        raw = dict(raw)
        mixer = raw.get("mixer")
        if raw.get("type") == "gla" and isinstance(mixer, Mapping) and mixer.get("rank") is None:
            owner = raw.get("weights_of") if raw.get("weights_of") is not None else i
            shape = shape_of(f"l{owner}.mix.a1")
            if shape:
                raw["mixer"] = {**mixer, "rank": int(shape[0])}
        layers.append(raw)
    out["layers"] = layers
    return out
