"""The Darovik decoder as a ``ModelSpec``.

Pre-norm layers on a float32 stream that is kept as several copies a token, every sublayer hung
on it by learned weights (``parts/block.py: hyper_connections``); every sublayer's result is
multiplied by ``residual_mult`` on its way in.  Without ``streams`` in the configuration the same
block runs with one copy and no link tensors: ``x += m f(norm(x))``.  A layer's mixer is one of
* ``attention``: grouped-query attention with two softmax maps a head over the same values and a
  sliding window, no positions (``parts/attention.py: differential_attention``);
* ``latent_attention``: keys and values from one cached, normed latent a token, queries straight
  from the layer's input, no positions, a learned sink a head in the softmax's denominator
  (``parts/latent_attention.py`` with ``q_rank`` None, ``rot_dim`` 0, ``sinks``).
The feed-forward is ``W_down relu(W_up h + b)^2 + b`` (``parts/mlp.py: mlp``), or routed experts
with sigmoid scores, a correction for the choice, groups worth their best two and scaled weights
(``parts/moe.py``), or absent.  A stretch of layers may run several times in a row with the same
tensors and a cache of its own each time: the schedule names those layers again.  The head is the
embedding's table.  Tensor names: ``embed``, ``final.norm``, ``l<i>.{norm1, norm2}``,
``l<i>.{hc1, hc2}.{in, mix, out}``, ``l<i>.mix.*``, ``l<i>.mlp.*``.
"""

from __future__ import annotations

from kvcore_amd.config.darovik_config import (DarovikConfig, DenseFeedForwardConfig, DifferentialAttentionConfig,
                                              ExpertsConfig)
from kvcore_amd.parts.base import PartSpec

from .spec import LayerSpec, ModelSpec, ScheduleEntry

GROUP_BEST = 2  # a group of experts is worth the sum of its two best choice scores


def darovik_spec(config: DarovikConfig) -> ModelSpec:
    H, eps = config.width, config.eps

    def norm() -> PartSpec:
        return PartSpec("rmsnorm", {"hidden_size": H, "eps": eps, "weight_name": ""})

    layers: list[LayerSpec] = []
    unread: list[str] = []  # tensors of a second sublayer that a layer without a feed-forward may still carry
    for i, layer in enumerate(config.layers):
        m = layer.mixer
        if isinstance(m, DifferentialAttentionConfig):
            mixer = PartSpec("differential_attention", {
                "hidden_size": H, "num_heads": m.heads, "num_kv_heads": m.kv_heads, "head_dim": m.dim,
                "v_head_dim": m.vdim, "scale": m.scale, "diff": m.diff, "eps": eps, "window": m.window,
                "float32_result": True,
                "tensor_names": {"q": "q", "k": "k", "v": "v", "o": "o", "lq1": "lq1", "lk1": "lk1", "lq2": "lq2",
                                 "lk2": "lk2"}})
        else:
            mixer = PartSpec("latent_attention", {
                "hidden_size": H, "heads": m.heads, "dim": m.dim, "rot_dim": 0, "vdim": m.vdim,
                "kv_rank": m.kv_rank, "q_rank": None, "scale": m.scale, "eps": eps, "window": m.window,
                "gated": False, "sinks": True, "float32_result": True,
                "tensor_names": {"q": "q", "dkv": "dkv", "dkv_norm": "dkv.norm", "uk": "uk", "uv": "uv", "o": "o",
                                 "sink": "sink"}})
        norms = {"norm1": norm(), "norm2": norm()}
        if layer.mlp is None:
            ffn = PartSpec("none")
            norms = {"norm1": norm()}
            unread += [f"l{i}.norm2", f"l{i}.hc2.in", f"l{i}.hc2.mix", f"l{i}.hc2.out"]
        elif isinstance(layer.mlp, DenseFeedForwardConfig):
            ffn = PartSpec("mlp", {
                "hidden_size": H, "intermediate_size": layer.mlp.ff, "activation": "relu_squared", "bias": True,
                "up_name": "up", "down_name": "down", "suffix": "", "bias_suffix": ".b", "float32_result": True})
        else:
            assert isinstance(layer.mlp, ExpertsConfig)
            e = layer.mlp
            ffn = PartSpec("routed_experts", {
                "hidden_size": H, "experts": e.experts, "top": e.top, "expert_size": e.ff, "limit": None,
                "alpha": 1.0, "up_shift": 0.0, "groups": e.groups, "keep": e.keep, "score": "sigmoid",
                "correction": True, "group_best": GROUP_BEST, "weight_scale": e.scale,
                "tensor_names": {"router": "router", "correction": "correction", "expert": "e{e}", "gate": "gate",
                                 "up": "up", "down": "down"}})
        block = PartSpec("hyper_connections", {
            "copies": config.streams or 1, "learned": config.streams is not None, "mult": config.residual_mult,
            "mixer_name": "mix", "ffn_name": "mlp"})
        layers.append(LayerSpec(prefix=f"l{i}", mixer=mixer, ffn=ffn, norms=norms, block=block))

    schedule = tuple(ScheduleEntry(i) for i in config.layer_order())
    return ModelSpec(
        vocab_size=config.vocab, hidden_size=H, max_position_embeddings=config.max_position_embeddings,
        layers=tuple(layers), final_norm=norm(), schedule=schedule,
        embedding=PartSpec("token_embedding", {"vocab_size": config.vocab, "hidden_size": H, "weight_name": ""}),
        head=PartSpec("linear_head", {"vocab_size": config.vocab, "hidden_size": H, "tied": True}),
        tie_word_embeddings=True, eos_token_ids=config.eos_token_ids, embed_prefix="embed",
        final_norm_prefix="final.norm", head_prefix="head", ignored_suffixes=tuple(unread),
    )
