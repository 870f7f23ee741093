"""Typed configuration of the Darovik decoder, read from config.json.

The file lists the layers one by one; every size and every constant that can differ between
models comes from it:

    {"architecture": "Darovik", "vocab": V, "width": H, "norm": {"eps": e}, "residual_mult": m,
     "streams": c, "loop": {"start": a, "stop": b, "times": n},
     "layers": [{"type": "attention" | "latent_attention", "mixer": {...},
                 "mlp": {"kind": "dense", "ff": F}
                      | {"kind": "moe", "expert": {"ff": F}, "router": {"experts": E, "top": k, "scale": s,
                                                                         "groups": {"count": g, "keep": k'}}}
                      | null}, ...]}

``attention`` mixers (two softmax maps a head) give ``heads, kv_heads, dim, vdim, scale, diff`` and
``mask {size}``; ``latent_attention`` mixers ``heads, dim, vdim, kv_rank, scale``.  A missing
``mask`` means that every earlier token is seen, a missing ``loop`` that every layer runs once, a
missing ``residual_mult`` 1, a missing ``groups`` that every expert may be chosen.  A missing
``streams`` means the plain residual sum (one row a token and no link tensors); with it, every
sublayer has link tensors, also when it says 1.
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


def _window(d: Mapping[str, Any], where: str) -> int:
    if d.get("mask") is None:
        return 0
    size = _require(_mapping(d, "mask", where), "size", int)
    if size <= 0:
        raise ConfigError(f"config.json: {where}mask.size must be positive, got {size}")
    return size


@dataclass(frozen=True)
class DifferentialAttentionConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    diff: float
    window: int  # 0: every earlier token is seen

    @classmethod
    def from_dict(cls, d: Mapping[str, Any], where: str) -> "DifferentialAttentionConfig":
        heads, kv, dim = _require(d, "heads", int), _require(d, "kv_heads", int), _require(d, "dim", int)
        vdim = _require(d, "vdim", int)
        if min(heads, kv, dim, vdim) <= 0 or heads % kv:
            raise ConfigError(f"config.json: {where}sizes must be positive and heads a multiple of kv_heads "
                              f"(heads {heads}, kv_heads {kv}, dim {dim}, vdim {vdim})")
        return cls(heads, kv, dim, vdim, _require(d, "scale", float), _require(d, "diff", float),
                   _window(d, where))


@dataclass(frozen=True)
class SinkLatentAttentionConfig:
    heads: int
    dim: int
    vdim: int
    kv_rank: int
    scale: float
    window: int

    @classmethod
    def from_dict(cls, d: Mapping[str, Any], where: str) -> "SinkLatentAttentionConfig":
        heads, dim, vdim = _require(d, "heads", int), _require(d, "dim", int), _require(d, "vdim", int)
        kv_rank = _require(d, "kv_rank", int)
        if min(heads, dim, vdim, kv_rank) <= 0:
            raise ConfigError(f"config.json: {where}sizes must be positive: {dict(d)}")
        return cls(heads, dim, vdim, kv_rank, _require(d, "scale", float), _window(d, where))


@dataclass(frozen=True)
class DenseFeedForwardConfig:
    ff: int


@dataclass(frozen=True)
class ExpertsConfig:
    ff: int
    experts: int
    top: int
    scale: float
    groups: int  # 1 and 1: every expert may be chosen
    keep: int


def _feed_forward(d: Mapping[str, Any], where: str) -> DenseFeedForwardConfig | ExpertsConfig:
    kind = d.get("kind")
    if kind == "dense":
        ff = _require(d, "ff", int)
        if ff <= 0:
            raise ConfigError(f"config.json: {where}ff must be positive")
        return DenseFeedForwardConfig(ff)
    if kind == "moe":
        ff = _require(_mapping(d, "expert", where), "ff", int)
        router = _mapping(d, "router", where)
        experts, top = _require(router, "experts", int), _require(router, "top", int)
        scale = float(router.get("scale", 1.0))
        groups = keep = 1
        if router.get("groups") is not None:
            g = _mapping(router, "groups", where + "router.")
            groups, keep = _require(g, "count", int), _require(g, "keep", int)
        if ff <= 0 or experts <= 0 or not 0 < top <= experts or groups <= 0 or experts % groups \
                or not 0 < keep <= groups:
            raise ConfigError(f"config.json: {where}{top} of {experts} experts of {ff} units in {groups} equal "
                              f"groups of which {keep} are kept: sizes do not fit")
        return ExpertsConfig(ff, experts, top, scale, groups, keep)
    raise ConfigError(f"config.json: {where}kind {kind!r} is not supported (supported: 'dense', 'moe')")


@dataclass(frozen=True)
class DarovikLayerConfig:
    type: str
    mixer: DifferentialAttentionConfig | SinkLatentAttentionConfig
    mlp: DenseFeedForwardConfig | ExpertsConfig | None


_MIXERS = {"attention": DifferentialAttentionConfig, "latent_attention": SinkLatentAttentionConfig}


@dataclass(frozen=True)
class DarovikConfig:
    vocab: int
    width: int
    eps: float
    residual_mult: float
    streams: int | None  # None: the plain residual sum, no link tensors
    loop: tuple[int, int, int] | None  # (start, stop, times)
    layers: tuple[DarovikLayerConfig, ...]
    max_position_embeddings: int
    eos_token_ids: tuple[int, ...] = ()

    def layer_order(self) -> list[int]:
        """The layers in the order in which they run, a looped stretch as often as it says."""
        n = len(self.layers)
        if self.loop is None:
            return list(range(n))
        start, stop, times = self.loop
        return list(range(start)) + list(range(start, stop)) * times + list(range(stop, n))

    @classmethod
    def from_dict(cls, d: Mapping[str, Any]) -> "DarovikConfig":
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
            if not isinstance(raw, Mapping):
                raise ConfigError(f"config.json: layers[{i}] must be an object")
            kind = raw.get("type")
            if kind not in _MIXERS:
                raise ConfigError(f"config.json: {where}type {kind!r} is not supported (supported: {sorted(_MIXERS)})")
            mixer = _MIXERS[kind].from_dict(_mapping(raw, "mixer", where), where + "mixer.")
            mlp = None if raw.get("mlp") is None else _feed_forward(_mapping(raw, "mlp", where), where + "mlp.")
            layers.append(DarovikLayerConfig(kind, mixer, mlp))
        streams = d.get("streams")
        if streams is not None and (not isinstance(streams, int) or not 1 <= streams <= 8):
            raise ConfigError(f"config.json: streams must be 1 to 8, got {streams!r}")
        loop = None
        if d.get("loop") is not None:
            raw = _mapping(d, "loop", "")
            start, stop, times = _require(raw, "start", int), _require(raw, "stop", int), _require(raw, "times", int)
            if not 0 <= start <= stop <= len(layers) or times < 1:
                raise ConfigError(f"config.json: loop {dict(raw)} does not fit {len(layers)} layers")
            loop = (start, stop, times)
        mult = d.get("residual_mult")
        eos = d.get("eos_token_id")
        eos_ids = () if eos is None else tuple(int(e) for e in (eos if isinstance(eos, (list, tuple)) else [eos]))
        return cls(vocab, width, eps, 1.0 if mult is None else float(mult), streams, loop, tuple(layers),
                   int(d.get("max_position_embeddings") or 131072), eos_ids)
