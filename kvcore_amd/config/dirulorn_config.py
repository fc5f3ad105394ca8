"""Typed configuration of the Dirulorn decoder, read from config.json.

The file lists the layers one by one; every size and every constant that can differ between
models comes from it:

    {"architecture": "Dirulorn", "vocab": V, "width": H, "norm": {"eps": e},
     "layers": [{"type": "mamba2" | "parallel", "mixer": {...}, "mlp": {"kind": "dense",
                 "ff": F} | null}, ...],
     "loop": {"start": a, "stop": b, "times": n}}            (optional)

``mamba2`` mixers give ``heads, vdim, state, groups, conv, norm_groups``; ``parallel`` mixers
give ``left`` (attention: ``heads, kv_heads, dim, vdim, scale, rot {dims, base, scaling
{factor, low, high, original}}``) and ``right`` (recurrent block: ``width, blocks, conv``).
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Mapping

from .model_config import ConfigError, _require


def _mapping(d: Mapping[str, Any], key: str, where: str) -> Mapping[str, Any]:
    value = d.get(key)
    if not isinstance(value, Mapping):
        raise ConfigError(f"config.json: {where}{key!r} must be an object")
    return value


@dataclass(frozen=True)
class RotaryConfig:
    dims: int
    base: float
    scaling: tuple[float, float, float, int] | None  # factor, low, high, original

    @classmethod
    def from_dict(cls, d: Mapping[str, Any] | None, head_dim: int) -> "RotaryConfig | None":
        if not d:
            return None
        dims = _require(d, "dims", int)
        if dims <= 0 or dims % 2 or dims > head_dim:
            raise ConfigError(f"config.json: rot.dims must be even, positive and at most the head size, got {dims}")
        sc = d.get("scaling")
        scaling = None
        if sc:
            scaling = (_require(sc, "factor", float), _require(sc, "low", float), _require(sc, "high", float),
                       _require(sc, "original", int))
            if scaling[0] <= 0 or scaling[3] <= 0 or scaling[2] <= scaling[1]:
                raise ConfigError("config.json: rot.scaling needs a positive factor and original length and high > low")
        return cls(dims, _require(d, "base", float), scaling)


@dataclass(frozen=True)
class AttentionBranchConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    rot: RotaryConfig | None

    @classmethod
    def from_dict(cls, d: Mapping[str, Any]) -> "AttentionBranchConfig":
        heads, kv = _require(d, "heads", int), _require(d, "kv_heads", int)
        dim, vdim = _require(d, "dim", int), _require(d, "vdim", int)
        if min(heads, kv, dim, vdim) <= 0 or heads % kv:
            raise ConfigError(f"config.json: attention sizes must be positive and heads a multiple of kv_heads "
                              f"(heads {heads}, kv_heads {kv}, dim {dim}, vdim {vdim})")
        return cls(heads, kv, dim, vdim, _require(d, "scale", float), RotaryConfig.from_dict(d.get("rot"), dim))


@dataclass(frozen=True)
class RecurrentBranchConfig:
    width: int
    blocks: int
    conv: int

    @classmethod
    def from_dict(cls, d: Mapping[str, Any]) -> "RecurrentBranchConfig":
        width, blocks, conv = _require(d, "width", int), _require(d, "blocks", int), _require(d, "conv", int)
        if width <= 0 or blocks <= 0 or width % blocks or conv < 1:
            raise ConfigError(f"config.json: recurrent block of width {width} in {blocks} blocks with {conv} taps")
        return cls(width, blocks, conv)


@dataclass(frozen=True)
class ParallelMixerConfig:
    left: AttentionBranchConfig
    right: RecurrentBranchConfig


@dataclass(frozen=True)
class StateSpaceConfig:
    heads: int
    vdim: int
    state: int
    groups: int
    conv: int
    norm_groups: int

    @classmethod
    def from_dict(cls, d: Mapping[str, Any]) -> "StateSpaceConfig":
        c = cls(*(_require(d, k, int) for k in ("heads", "vdim", "state", "groups", "conv", "norm_groups")))
        if min(c.heads, c.vdim, c.state, c.groups, c.norm_groups) <= 0 or c.conv < 1 or c.heads % c.groups \
                or (c.heads * c.vdim) % c.norm_groups:
            raise ConfigError(f"config.json: state-space mixer sizes do not fit together: {dict(d)}")
        return c


@dataclass(frozen=True)
class DirulornLayerConfig:
    type: str
    mixer: ParallelMixerConfig | StateSpaceConfig
    ff: int | None  # None: the layer has no feed-forward


@dataclass(frozen=True)
class LoopConfig:
    start: int
    stop: int
    times: int


@dataclass(frozen=True)
class DirulornConfig:
    vocab: int
    width: int
    eps: float
    layers: tuple[DirulornLayerConfig, ...]
    loop: LoopConfig | None
    max_position_embeddings: int
    eos_token_ids: tuple[int, ...] = ()

    @classmethod
    def from_dict(cls, d: Mapping[str, Any]) -> "DirulornConfig":
        vocab, width = _require(d, "vocab", int), _require(d, "width", int)
        if vocab <= 0 or width <= 0:
            raise ConfigError("config.json: vocab and width must be positive")
        eps = _require(_mapping(d, "norm", ""), "eps", float)
        raw_layers = d.get("layers")
        if not isinstance(raw_layers, list) or not raw_layers:
            raise ConfigError("config.json: 'layers' must be a list of at least one layer")
        layers = []
        for i, raw in enumerate(raw_layers):
            where = f"layers[{i}]."
            kind = raw.get("type")
            mixer = _mapping(raw, "mixer", where)
            if kind == "parallel":
                parsed = ParallelMixerConfig(AttentionBranchConfig.from_dict(_mapping(mixer, "left", where + "mixer.")),
                                             RecurrentBranchConfig.from_dict(_mapping(mixer, "right", where + "mixer.")))
            elif kind == "mamba2":
                parsed = StateSpaceConfig.from_dict(mixer)
            else:
                raise ConfigError(f"config.json: {where}type {kind!r} is not supported (supported: 'mamba2', 'parallel')")
            mlp = raw.get("mlp")
            ff = None
            if mlp is not None:
                if mlp.get("kind") != "dense":
                    raise ConfigError(f"config.json: {where}mlp.kind {mlp.get('kind')!r} is not supported (supported: 'dense')")
                ff = _require(mlp, "ff", int)
                if ff <= 0:
                    raise ConfigError(f"config.json: {where}mlp.ff must be positive")
            layers.append(DirulornLayerConfig(kind, parsed, ff))
        loop = None
        if d.get("loop"):
            lp = d["loop"]
            loop = LoopConfig(_require(lp, "start", int), _require(lp, "stop", int), _require(lp, "times", int))
            if not 0 <= loop.start < loop.stop <= len(layers) or loop.times < 1:
                raise ConfigError(f"config.json: loop {dict(lp)} does not fit {len(layers)} layers")
        eos = d.get("eos_token_id")
        eos_ids = () if eos is None else tuple(int(e) for e in (eos if isinstance(eos, (list, tuple)) else [eos]))
        return cls(vocab, width, eps, tuple(layers), loop,
                   int(d.get("max_position_embeddings") or 131072), eos_ids)
