"""The Tazunex decoder as a ``ModelSpec``.

Layers with a norm before and a norm behind each sublayer on a float32 stream: ``x += norm1b(
mixer(norm1(x))); x += norm2b(ff(norm2(x)))`` (``parts/block.py: sandwich_norm``), all RMS norms
with plain gains.  A layer's mixer is one of
* ``attention``: grouped-query attention whose values are the keys as projected (no value
  matrix), with one RMS norm over all query heads and one over all key heads before the
  rotation (half layout, on the first ``rot.dims`` elements of a head), a sliding window, and a
  learned sink per head in the softmax's denominator (options of ``parts/attention.py``);
* ``latent_attention``: keys and values from one cached latent a token, queries through a
  latent of their own, one rotated key part shared by the heads (neighbouring pairs), a sliding
  window, a sigmoid gate per head (``parts/latent_attention.py``);
* ``mlstm``: a matrix memory with log gates and a running maximum (``parts/linear_attention.py:
  max_gated_matrix_memory``).
The feed-forward is ``W_down(gelu_tanh(W_gate h) * (W_up h))`` or absent.  A layer may run
another layer's tensors (``weights_of``): the schedule then names that layer again, with a cache
plane or state of its own.  The head is the embedding's table, the logits softly capped.
Tensor names: ``embed``, ``final.norm``, ``l<i>.{norm1, norm1b, norm2, norm2b}``, ``l<i>.mix.*``,
``l<i>.mlp.{gate, up, down}``.
"""

from __future__ import annotations

from kvcore_amd.config.tazunex_config import (LatentAttentionConfig, MatrixMemoryConfig, SinkAttentionConfig,
                                              TazunexConfig)
from kvcore_amd.parts.base import PartSpec

from .spec import LayerSpec, ModelSpec, ScheduleEntry

DEN_EPS = 1e-6  # added to the matrix memory's denominator


def tazunex_spec(config: TazunexConfig) -> ModelSpec:
    H, eps = config.width, config.eps

    def norm() -> PartSpec:
        return PartSpec("rmsnorm", {"hidden_size": H, "eps": eps, "weight_name": ""})

    positions: list[PartSpec] = []
    position_index: dict[tuple, int] = {}

    def rotation(dims: int, base: float, interleaved: bool) -> int | None:
        """The index of the rotary encoding with these constants among ``positions``."""
        if dims <= 0:
            return None
        key = (dims, base, interleaved)
        if key not in position_index:
            position_index[key] = len(positions)
            positions.append(PartSpec("rotary", {"rot_dim": dims, "theta": base, "interleaved": interleaved}))
        return position_index[key]

    layers: list[LayerSpec] = []
    spec_index: dict[int, int] = {}  # config layer -> index among the layers that own tensors
    for i, layer in enumerate(config.layers):
        if layer.weights_of is not None:
            continue
        m = layer.mixer
        position = None
        if isinstance(m, SinkAttentionConfig):
            position = rotation(m.rot_dims, m.rot_base, False)
            mixer = PartSpec("paged_attention", {
                "hidden_size": H, "num_heads": m.heads, "num_kv_heads": m.kv_heads, "head_dim": m.dim,
                "scale": m.scale, "window": m.window, "qk_norm_eps": eps, "qk_norm_span": "projection",
                "values_are_keys": True, "sinks": True, "float32_result": True, "sized_buffers": True,
                "tensor_names": {"q": "q", "k": "k", "o": "o", "q_norm": "q.norm", "k_norm": "k.norm",
                                 "sink": "sink"}})
        elif isinstance(m, LatentAttentionConfig):
            position = rotation(m.rot_dim, m.rot_base, True)
            mixer = PartSpec("latent_attention", {
                "hidden_size": H, "heads": m.heads, "dim": m.dim, "rot_dim": m.rot_dim, "vdim": m.vdim,
                "kv_rank": m.kv_rank, "q_rank": m.q_rank, "scale": m.scale, "eps": eps, "window": m.window,
                "float32_result": True,
                "tensor_names": {"dq": "dq", "dq_norm": "dq.norm", "uq": "uq", "dkv": "dkv",
                                 "dkv_norm": "dkv.norm", "uk": "uk", "uv": "uv", "g": "g", "o": "o"}})
        else:
            assert isinstance(m, MatrixMemoryConfig)
            mixer = PartSpec("max_gated_matrix_memory", {
                "hidden_size": H, "heads": m.heads, "dim": m.dim, "vdim": m.vdim, "gate_cap": m.gate_cap,
                "eps": eps, "den_eps": DEN_EPS, "float32_result": True,
                "tensor_names": {"q": "q", "k": "k", "v": "v", "g": "g", "o": "o", "norm": "norm", "i": "i",
                                 "f": "f", "i_bias": "i.b", "f_bias": "f.b"}})
        if layer.mlp is None:
            ffn = PartSpec("none")
            norms = {"norm1": norm(), "norm1b": norm()}
        else:
            ffn = PartSpec("swiglu", {
                "hidden_size": H, "intermediate_size": layer.mlp.ff, "gate_name": "gate", "up_name": "up",
                "down_name": "down", "suffix": "", "sized_buffers": True, "activation": "gelu_tanh",
                "float32_result": True})
            norms = {"norm1": norm(), "norm1b": norm(), "norm2": norm(), "norm2b": norm()}
        spec_index[i] = len(layers)
        layers.append(LayerSpec(
            prefix=f"l{i}", mixer=mixer, ffn=ffn, norms=norms, position=position,
            block=PartSpec("sandwich_norm", {"mixer_name": "mix", "ffn_name": "mlp"})))

    # a layer that borrows names its owner again, whichever of the two comes first
    schedule = [ScheduleEntry(spec_index[i if layer.weights_of is None else layer.weights_of])
                for i, layer in enumerate(config.layers)]
    return ModelSpec(
        vocab_size=config.vocab, hidden_size=H, max_position_embeddings=config.max_position_embeddings,
        layers=tuple(layers), final_norm=norm(), positions=tuple(positions), schedule=tuple(schedule),
        embedding=PartSpec("token_embedding", {"vocab_size": config.vocab, "hidden_size": H, "weight_name": ""}),
        head=PartSpec("linear_head", {"vocab_size": config.vocab, "hidden_size": H, "tied": True,
                                      "soft_cap": config.logit_softcap}),
        tie_word_embeddings=True, eos_token_ids=config.eos_token_ids, embed_prefix="embed",
        final_norm_prefix="final.norm", head_prefix="head", ignored_suffixes=(),
    )
