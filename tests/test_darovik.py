"""Darovik without a GPU: configuration, registry, the schedule of a looped stretch, the checkpoint
layout, caches as the model plans them, and the plain implementation's own consistency."""

from __future__ import annotations

import copy
import math
import random

import pytest
import torch

from tests.darovik_helpers import CONFIG_A, CONFIG_B, CONFIG_C, CONFIG_D, CONFIGS, random_config
from tests.plain import darovik as plain


def spec_of(config):
    from kvcore_amd.registry import resolve_architecture

    arch = resolve_architecture(config)
    return arch.build_spec(arch.parse_config(config))


def test_the_architecture_is_registered():
    from kvcore_amd.registry import resolve_architecture

    assert resolve_architecture(CONFIG_A).name == "Darovik"


def test_a_looped_stretch_is_run_again_with_caches_of_its_own():
    from kvcore_amd.models.decoder import DecoderModel

    spec = spec_of(CONFIG_A)
    assert [e.layer for e in spec.resolved_schedule()] == [0, 1, 2, 1, 2, 1, 2, 3]
    assert plain.layer_order(CONFIG_A) == [0, 1, 2, 1, 2, 1, 2, 3]
    model = DecoderModel(spec, torch.float32, "cpu")
    assert model.stream_copies == 3
    # the two maps' keys are one cached key of twice the size; values keep their own size
    needs = {g.need.planes: (g.need.window, g.num_planes) for g in model.cache_groups}
    assert needs[((2, 48), (2, 40))] == (24, 3)      # layer 1, three passes
    assert needs[((3, 32), (3, 16))] == (10, 1)      # layer 3
    assert needs[((1, 40), (1, 40))] == (0, 1)       # layer 0: one latent row a token
    assert needs[((1, 24), (1, 24))] == (0, 3)       # layer 2, three passes
    assert all(not c.state_indices for c in model.calls)
    # the whole model twice; a loop of one pass; no loop
    assert [e.layer for e in spec_of(CONFIG_B).resolved_schedule()] == [0, 1, 2, 3, 0, 1, 2, 3]
    assert [e.layer for e in spec_of(CONFIG_D).resolved_schedule()] == [0, 1, 2, 3]
    assert [e.layer for e in spec_of(CONFIG_C).resolved_schedule()] == [0, 1, 2, 3]
    empty = copy.deepcopy(CONFIG_A)
    empty["loop"] = {"start": 2, "stop": 2, "times": 5}  # an empty stretch is no layer at all
    assert [e.layer for e in spec_of(empty).resolved_schedule()] == [0, 1, 2, 3]


def test_checkpoint_layout_has_the_design_s_names_and_shapes():
    from kvcore_amd.weights.loader import checkpoint_layout

    layout = {k: v[0] for k, v in checkpoint_layout(spec_of(CONFIG_A)).items()}
    assert layout["embed"] == (211, 96) and layout["final.norm"] == (96,)
    assert layout["l0.mix.q"] == (48, 96) and layout["l0.mix.dkv"] == (40, 96) and layout["l0.mix.dkv.norm"] == (40,)
    assert layout["l0.mix.uk"] == (48, 40) and layout["l0.mix.uv"] == (72, 40) and layout["l0.mix.sink"] == (3,)
    assert layout["l0.mix.o"] == (96, 72)
    assert layout["l0.mlp.up"] == (80, 96) and layout["l0.mlp.up.b"] == (80,) and layout["l0.mlp.down.b"] == (96,)
    assert layout["l1.mix.q"] == (4 * 2 * 24, 96) and layout["l1.mix.k"] == (2 * 2 * 24, 96)
    assert layout["l1.mix.v"] == (80, 96) and layout["l1.mix.o"] == (96, 160) and layout["l1.mix.lq2"] == (24,)
    assert layout["l1.mlp.router"] == (12, 96) and layout["l1.mlp.correction"] == (12,)
    assert layout["l1.mlp.e11.gate"] == (24, 96) and layout["l1.mlp.e0.down"] == (96, 24)
    assert layout["l1.hc1.in"] == (3,) and layout["l1.hc2.mix"] == (3, 3) and layout["l3.hc2.out"] == (3,)
    assert "l2.norm2" not in layout and "l2.hc2.in" not in layout and "l2.norm1" in layout  # no feed-forward there
    assert not any(k.startswith("head") for k in layout)  # the head is the embedding's table
    # without `streams` there are no link tensors; with `streams: 1` there are
    plain_layout = checkpoint_layout(spec_of(CONFIG_C))
    assert not any(".hc" in k for k in plain_layout)
    assert checkpoint_layout(spec_of(CONFIG_D))["l0.hc1.mix"][0] == (1, 1)


def test_wrong_configurations_are_refused_by_name():
    from kvcore_amd.config.model_config import ConfigError

    def broken(change):
        config = copy.deepcopy(CONFIG_A)
        change(config)
        with pytest.raises(ConfigError) as info:
            spec_of(config)
        return str(info.value)

    assert "kv_heads" in broken(lambda c: c["layers"][1]["mixer"].update(kv_heads=3))
    assert "diff" in broken(lambda c: c["layers"][1]["mixer"].pop("diff"))
    assert "kv_rank" in broken(lambda c: c["layers"][0]["mixer"].pop("kv_rank"))
    assert "type" in broken(lambda c: c["layers"][0].update(type="mamba"))
    assert "kind" in broken(lambda c: c["layers"][0]["mlp"].update(kind="glu"))
    assert "groups" in broken(lambda c: c["layers"][1]["mlp"]["router"]["groups"].update(count=5))
    assert "loop" in broken(lambda c: c["loop"].update(stop=9))
    assert "streams" in broken(lambda c: c.update(streams=0))
    assert "mask" in broken(lambda c: c["layers"][1]["mixer"]["mask"].update(size=0))


def test_every_drawn_configuration_builds():
    from kvcore_amd.models.decoder import DecoderModel

    for seed in range(30):
        config = random_config(random.Random(seed))
        model = DecoderModel(spec_of(config), torch.float32, "cpu")
        assert len(model.calls) == len(plain.layer_order(config))
        assert model.stream_copies == (config.get("streams") or 1)


def _weights(config, seed=0, std=0.3):
    from kvcore_amd.weights.loader import checkpoint_layout

    gen = torch.Generator().manual_seed(seed)
    out = {}
    for name, (shape, _, _) in checkpoint_layout(spec_of(config)).items():
        out[name] = torch.randn(shape, generator=gen, dtype=torch.float64) * std
        if name.endswith("mix") and ".hc" in name:
            out[name] += torch.eye(shape[0], dtype=torch.float64)
    return out


def test_plain_model_is_causal_and_its_windows_end_where_they_say():
    """A token's logits depend on earlier tokens only; an attention layer alone forgets a token once
    it is `mask.size` positions back, and the latent layer never does."""
    config = {"architecture": "Darovik", "vocab": 50, "width": 32, "norm": {"eps": 1e-5}, "streams": 2,
              "layers": [{"type": "attention", "mlp": None,
                          "mixer": {"heads": 2, "kv_heads": 1, "dim": 8, "vdim": 8, "scale": 0.3, "diff": 0.5,
                                    "mask": {"size": 5}}}]}
    w = _weights(config)
    a = [3, 7, 1, 9, 4, 4, 8, 2, 6, 5]
    b = [11] + a[1:]
    la, lb = plain.forward(config, w, a), plain.forward(config, w, b)
    assert (la[:0] == lb[:0]).all() and not torch.allclose(la[4], lb[4])  # position 4 still sees position 0
    assert torch.allclose(la[5:], lb[5:], atol=1e-12)                      # position 5 does not
    c = a[:6] + [12] + a[7:]
    assert torch.allclose(plain.forward(config, w, c)[:6], la[:6], atol=1e-12)  # nothing looks ahead
    config["layers"][0] = {"type": "latent_attention", "mlp": None,
                           "mixer": {"heads": 2, "dim": 8, "vdim": 4, "kv_rank": 6, "scale": 0.3}}
    w = _weights(config)
    la, lb = plain.forward(config, w, a), plain.forward(config, w, b)
    assert not torch.allclose(la[9], lb[9])


def test_plain_routing_by_hand():
    """Sigmoid scores; the choice by score plus correction inside the groups that are worth most
    (their two best choice scores); weights from the scores without the correction."""
    h = torch.eye(6, dtype=torch.float64)[:1] * 1.0  # the router's first column is the logits
    logits = torch.tensor([2.0, -1.0, 0.5, 0.4, -3.0, 3.0], dtype=torch.float64)
    w = {"router": torch.zeros(6, 6, dtype=torch.float64), "correction": torch.tensor([0.0, 0.0, 0.3, 0.3, 0.0, -2.0],
                                                                                     dtype=torch.float64)}
    w["router"][:, 0] = logits
    s = torch.sigmoid(logits)
    r = {"experts": 6, "top": 2, "scale": 2.0, "groups": {"count": 3, "keep": 1}}
    # groups (0,1), (2,3), (4,5): worth s0+s1, s2+s3+0.6, s4+s5-2 -> the middle one wins
    choice, weight = plain.route(h, w, r)
    assert sorted(choice[0].tolist()) == [2, 3]
    got = dict(zip(choice[0].tolist(), weight[0].tolist()))
    assert math.isclose(got[2], 2.0 * s[2] / (s[2] + s[3]), rel_tol=1e-12)
    # with two groups kept the best three experts by choice score among groups 0 and 1
    r["groups"]["keep"], r["top"] = 2, 3
    choice, weight = plain.route(h, w, r)
    assert choice[0].tolist() == [2, 3, 0]
    r["top"] = 2
    # choice scores may be negative: an expert outside the kept groups is never chosen for that
    w["correction"] = torch.tensor([-5.0, -6.0, -9.0, -9.5, -7.0, -7.5], dtype=torch.float64)
    r["groups"]["keep"] = 1
    choice, _ = plain.route(h, w, r)
    assert sorted(choice[0].tolist()) == [0, 1]
    # no groups: every expert may be chosen
    r.pop("groups")
    w["correction"] = torch.zeros(6, dtype=torch.float64)
    choice, weight = plain.route(h, w, r)
    assert choice[0].tolist() == [5, 0] and math.isclose(float(weight.sum()), 2.0, rel_tol=1e-12)


def test_plain_stream_copies_reduce_to_the_plain_sum():
    """With link tensors of ones and an identity, one copy is the plain residual sum; and the
    sum of several copies that never mix is what each sublayer added, once for every copy."""
    config = copy.deepcopy(CONFIG_C)
    w = _weights(config, seed=3)
    tokens = [5, 9, 2, 77, 31, 8, 8, 40]
    base = plain.forward(config, w, tokens)
    one = copy.deepcopy(config)
    one["streams"] = 1
    w1 = dict(w)
    for i, layer in enumerate(config["layers"]):
        for q in (1, 2) if layer["mlp"] else (1,):
            w1[f"l{i}.hc{q}.in"] = torch.ones(1, dtype=torch.float64)
            w1[f"l{i}.hc{q}.out"] = torch.ones(1, dtype=torch.float64)
            w1[f"l{i}.hc{q}.mix"] = torch.ones(1, 1, dtype=torch.float64)
    assert torch.allclose(plain.forward(one, w1, tokens), base, atol=1e-10)


def test_plain_differential_attention_reduces_to_one_map():
    """With the second map's weight zero (`lambda` = 0) the layer is ordinary windowed attention on
    the first map, normed head by head."""
    m = {"heads": 2, "kv_heads": 1, "dim": 4, "vdim": 6, "scale": 0.5, "diff": 0.25, "mask": {"size": 3}}
    gen = torch.Generator().manual_seed(1)
    w = {k: torch.randn(s, generator=gen, dtype=torch.float64) for k, s in
         {"q": (16, 10), "k": (8, 10), "v": (6, 10), "o": (10, 12)}.items()}
    # exp(0) - exp(log(1.25)) + 0.25 = 0
    w.update(lq1=torch.zeros(4, dtype=torch.float64), lk1=torch.zeros(4, dtype=torch.float64),
             lq2=torch.full((4,), math.log(1.25) / 4, dtype=torch.float64), lk2=torch.ones(4, dtype=torch.float64))
    assert abs(plain.differential_lambda(w, m)) < 1e-12
    h = torch.randn(7, 10, generator=gen, dtype=torch.float64)
    got = plain.differential_attention(h, w, m, 1e-6)
    q = (h @ w["q"].T).view(7, 2, 2, 4)[:, :, 0]
    k = (h @ w["k"].T).view(7, 1, 2, 4)[:, 0, 0]
    v = h @ w["v"].T
    heads = []
    for head in range(2):
        s = (q[:, head] @ k.T) * 0.5
        p = plain.masked_softmax(s[None], plain.seen_keys(7, 3))[0]
        heads.append(plain.rms(p @ v, 1e-6) * 0.75)
    assert torch.allclose(got, torch.cat(heads, dim=1) @ w["o"].T, atol=1e-12)


def test_configurations_cover_what_they_say():
    assert CONFIG_A["streams"] == 3 and "streams" not in CONFIG_C and CONFIG_D["streams"] == 1
    assert {len(c["layers"]) for c, _ in CONFIGS.values()} == {4}
    windows = [plain.window_of(l["mixer"]) for c, _ in CONFIGS.values() for l in c["layers"] if l["type"] == "attention"]
    assert 1 in windows and None in windows
    assert any(l["mlp"] is None for l in CONFIG_A["layers"]) and CONFIG_B["loop"]["stop"] == 4
