"""Typed configuration of the Tazunex decoder, read from config.json.

The file lists the layers one by one; every size and every constant that can differ between
models comes from it:

    {"architecture": "Tazunex", "vocab": V, "width": H, "norm": {"eps": e}, "logit_softcap": c,
     "layers": [{"type": "attention" | "latent_attention" | "mlstm", "mixer": {...},
                 "mlp": {"kind": "dense", "ff": F} | null, "weights_of": j (optional)}, ...]}

``attention`` mixers give ``heads, kv_heads, dim, vdim, scale``, ``mask {size}`` and ``rot {base,
dims}``; ``latent_attention`` mixers ``heads, dim, rot_dim, vdim, kv_rank, q_rank, scale``, ``mask``
and ``rot``; ``mlstm`` mixers ``heads, dim, vdim, gate_cap``.  A missing ``mask`` means that every
earlier token is seen, a missing ``rot`` that nothing is rotated, a missing ``logit_softcap`` no
cap.  A layer with ``weights_of: j`` runs layer j's tensors with a cache or state of its own.
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


def _rotation(d: Mapping[str, Any], where: str, most: int) -> tuple[int, float]:
    """``(dims, base)``; ``(0, 1.0)`` without a ``rot`` entry."""
    if d.get("rot") is None:
        return 0, 1.0
    rot = _mapping(d, "rot", where)
    dims, base = _require(rot, "dims", int), _require(rot, "base", float)
    if dims < 0 or dims % 2 or dims > most or not base > 0:
        raise ConfigError(f"config.json: {where}rot.dims must be even and at most {most}, rot.base positive "
                          f"(dims {dims}, base {base})")
    return dims, base


@dataclass(frozen=True)
class SinkAttentionConfig:
    heads: int
    kv_heads: int
    dim: int
    scale: float
    window: int  # 0: every earlier token is seen
    rot_dims: int
    rot_base: float

    @classmethod
    def from_dict(cls, d: Mapping[str, Any], where: str) -> "SinkAttentionConfig":
        heads, kv, dim = _require(d, "heads", int), _require(d, "kv_heads", int), _require(d, "dim", int)
        if min(heads, kv, dim) <= 0 or heads % kv:
            raise ConfigError(f"config.json: {where}sizes must be positive and heads a multiple of kv_heads "
                              f"(heads {heads}, kv_heads {kv}, dim {dim})")
        if d.get("vdim") is not None and _require(d, "vdim", int) != dim:
            raise ConfigError(f"config.json: {where}vdim must equal dim: the values of this mixer are its keys")
        dims, base = _rotation(d, where, dim)
        return cls(heads, kv, dim, _require(d, "scale", float), _window(d, where), dims, base)


@dataclass(frozen=True)
class LatentAttentionConfig:
    heads: int
    dim: int
    rot_dim: int
    vdim: int
    kv_rank: int
    q_rank: int
    scale: float
    window: int
    rot_base: float

    @classmethod
    def from_dict(cls, d: Mapping[str, Any], where: str) -> "LatentAttentionConfig":
        heads, dim, vdim = _require(d, "heads", int), _require(d, "dim", int), _require(d, "vdim", int)
        rot_dim = _require(d, "rot_dim", int)
        kv_rank, q_rank = _require(d, "kv_rank", int), _require(d, "q_rank", int)
        if min(heads, dim, vdim, kv_rank, q_rank) <= 0 or rot_dim < 0 or rot_dim % 2:
            raise ConfigError(f"config.json: {where}sizes must be positive and rot_dim even: {dict(d)}")
        dims, base = _rotation(d, where, rot_dim)
        if rot_dim and dims != rot_dim:
            raise ConfigError(f"config.json: {where}rot.dims ({dims}) must equal rot_dim ({rot_dim})")
        return cls(heads, dim, rot_dim, vdim, kv_rank, q_rank, _require(d, "scale", float), _window(d, where), base)


@dataclass(frozen=True)
class MatrixMemoryConfig:
    heads: int
    dim: int
    vdim: int
    gate_cap: float

    @classmethod
    def from_dict(cls, d: Mapping[str, Any], where: str) -> "MatrixMemoryConfig":
        heads, dim, vdim = _require(d, "heads", int), _require(d, "dim", int), _require(d, "vdim", int)
        cap = _require(d, "gate_cap", float)
        if min(heads, dim, vdim) <= 0 or not cap > 0:
            raise ConfigError(f"config.json: {where}sizes and gate_cap must be positive: {dict(d)}")
        return cls(heads, dim, vdim, cap)


@dataclass(frozen=True)
class DenseFeedForwardConfig:
    ff: int

    @classmethod
    def from_dict(cls, d: Mapping[str, Any], where: str) -> "DenseFeedForwardConfig":
        if d.get("kind") != "dense":
            raise ConfigError(f"config.json: {where}kind {d.get('kind')!r} is not supported (supported: 'dense')")
        ff = _require(d, "ff", int)
        if ff <= 0:
            raise ConfigError(f"config.json: {where}ff must be positive")
        return cls(ff)


@dataclass(frozen=True)
class TazunexLayerConfig:
    type: str
    mixer: SinkAttentionConfig | LatentAttentionConfig | MatrixMemoryConfig
    mlp: DenseFeedForwardConfig | None
    weights_of: int | None


_MIXERS = {"attention": SinkAttentionConfig, "latent_attention": LatentAttentionConfig, "mlstm": MatrixMemoryConfig}


@dataclass(frozen=True)
class TazunexConfig:
    vocab: int
    width: int
    eps: float
    logit_softcap: float  # 0: none
    layers: tuple[TazunexLayerConfig, ...]
    max_position_embeddings: int
    eos_token_ids: tuple[int, ...] = ()

    @classmethod
    def from_dict(cls, d: Mapping[str, Any]) -> "TazunexConfig":
        vocab, width = _require(d, "vocab", int), _require(d, "width", int)
        if vocab <= 0 or width <= 0:
            raise ConfigError("config.json: vocab and width must be positive")
        eps = _require(_mapping(d, "norm", ""), "eps", float)
        raw_layers = d.get("layers")
        if not isinstance(raw_layers, list) or not raw_layers:
            raise ConfigError("config.json: 'layers' must be a list of at least one layer")
        for i, raw in enumerate(raw_layers):
            if not isinstance(raw, Mapping):
                raise ConfigError(f"config.json: layers[{i}] must be an object")
        slots: list[TazunexLayerConfig | None] = [None] * len(raw_layers)
        for i, raw in enumerate(raw_layers):  # the layers that own tensors
            if raw.get("weights_of") is not None:
                continue
            where = f"layers[{i}]."
            kind = raw.get("type")
            if kind not in _MIXERS:
                raise ConfigError(f"config.json: {where}type {kind!r} is not supported (supported: {sorted(_MIXERS)})")
            mixer = _MIXERS[kind].from_dict(_mapping(raw, "mixer", where), where + "mixer.")
            mlp = None if raw.get("mlp") is None else DenseFeedForwardConfig.from_dict(raw["mlp"], where + "mlp.")
            slots[i] = TazunexLayerConfig(kind, mixer, mlp, None)
        for i, raw in enumerate(raw_layers):  # the layers that borrow them, before or behind their owner
            if raw.get("weights_of") is None:
                continue
            where = f"layers[{i}]."
            source, seen = int(raw["weights_of"]), {i}
            while 0 <= source < len(raw_layers) and raw_layers[source].get("weights_of") is not None:
                if source in seen:
                    break
                seen.add(source)
                source = int(raw_layers[source]["weights_of"])  # a layer that borrows in turn: its owner
            owner = slots[source] if 0 <= source < len(raw_layers) and source not in seen else None
            if owner is None or owner.weights_of is not None:
                raise ConfigError(f"config.json: {where}weights_of must name a layer that has tensors of its own")
            # the tensors are the owner's, so the owner's sizes are the ones that count
            slots[i] = TazunexLayerConfig(owner.type, owner.mixer, owner.mlp, source)
        layers = [layer for layer in slots if layer is not None]
        assert len(layers) == len(raw_layers)
        cap = d.get("logit_softcap")
        cap = 0.0 if cap is None else float(cap)
        if cap < 0:
            raise ConfigError("config.json: logit_softcap must be positive when given")
        eos = d.get("eos_token_id")
        eos_ids = () if eos is None else tuple(int(e) for e in (eos if isinstance(eos, (list, tuple)) else [eos]))
        return cls(vocab, width, eps, cap, tuple(layers), int(d.get("max_position_embeddings") or 131072), eos_ids)
