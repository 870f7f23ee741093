"""Tazunex without a GPU: configuration, registry, the schedule of layers that borrow tensors,
the checkpoint layout, caches and states as the model plans them, and the plain
implementation's own consistency."""

from __future__ import annotations

import copy
import math

import pytest
import torch

from tests.plain import tazunex as plain
from tests.tazunex_helpers import CONFIG_A, CONFIG_B, CONFIG_C, CONFIG_D, CONFIGS, random_config


def spec_of(config):
    from kvcore_amd.registry import resolve_architecture

    arch = resolve_architecture(config)
    return arch.build_spec(arch.parse_config(config))


def test_the_architecture_is_registered():
    from kvcore_amd.registry import resolve_architecture

    assert resolve_architecture(CONFIG_A).name == "Tazunex"


def test_a_layer_that_borrows_tensors_is_a_second_run_of_its_owner():
    from kvcore_amd.models.decoder import DecoderModel

    spec = spec_of(CONFIG_A)
    assert len(spec.layers) == 3  # five layers, two of them borrowed
    assert [e.layer for e in spec.resolved_schedule()] == [0, 1, 2, 0, 1]
    assert [l.prefix for l in spec.layers] == ["l0", "l1", "l2"]
    model = DecoderModel(spec, torch.float32, "cpu")
    # the attention layer runs twice (two planes of one group); the latent layer has a group of its own
    assert sorted(g.num_planes for g in model.cache_groups) == [1, 2]
    windows = sorted(g.need.window for g in model.cache_groups)
    assert windows == [10, 24]
    # a latent layer keeps one row a token for keys and one for values: 8 rotated + 24 latent
    latent = next(g.need for g in model.cache_groups if g.need.window == 10)
    assert latent.planes == ((1, 32), (1, 32))
    # every run of a memory layer has its own matrices (the normaliser is their last column) and maxima
    per_call = [len(c.state_indices) for c in model.calls]
    assert per_call == [0, 2, 0, 0, 2]
    shapes = [tuple(model.state_arrays[i].need.shape) for c in model.calls for i in c.state_indices]
    assert shapes == [(3, 24, 41), (3,), (3, 24, 41), (3,)]


def test_an_owner_may_stand_behind_the_layer_that_borrows_from_it():
    import copy

    config = copy.deepcopy(CONFIG_A)
    order = [3, 4, 0, 1, 2]  # the borrowed runs first
    layers = [copy.deepcopy(config["layers"][i]) for i in order]
    for layer in layers:
        if "weights_of" in layer:
            layer["weights_of"] = order.index(layer["weights_of"])
    config["layers"] = layers
    spec = spec_of(config)
    assert [l.prefix for l in spec.layers] == ["l2", "l3", "l4"]
    assert [e.layer for e in spec.resolved_schedule()] == [0, 1, 0, 1, 2]


def test_rotations_are_shared_by_layers_with_the_same_constants():
    spec = spec_of(CONFIG_B)
    kinds = [(p.args["rot_dim"], p.args["theta"], p.args["interleaved"]) for p in spec.positions]
    assert kinds == [(64, 500000.0, False), (32, 500000.0, True)]
    assert [l.position for l in spec.layers] == [None, 0, 1]
    spec_c = spec_of(CONFIG_C)
    # no rotation at all for the attention layer without "rot" and the latent layer of no rotated elements
    assert [l.position for l in spec_c.layers] == [None, 0, 1, None, None]


def test_checkpoint_layout_has_the_design_s_names_and_shapes():
    from kvcore_amd.weights.loader import checkpoint_layout

    layout = {k: v[0] for k, v in checkpoint_layout(spec_of(CONFIG_A)).items()}
    assert layout["embed"] == (211, 96) and not any(k.startswith("head") for k in layout)
    assert layout["final.norm"] == (96,)
    for n in ("norm1", "norm1b", "norm2", "norm2b"):
        assert layout[f"l0.{n}"] == (96,)
    assert "l2.norm2" not in layout and "l2.norm1b" in layout  # a layer without a feed-forward
    assert layout["l0.mix.q"] == (128, 96) and layout["l0.mix.k"] == (64, 96) and "l0.mix.v" not in layout
    assert layout["l0.mix.q.norm"] == (128,) and layout["l0.mix.k.norm"] == (64,) and layout["l0.mix.sink"] == (4,)
    assert layout["l0.mix.o"] == (96, 128)
    assert layout["l0.mlp.gate"] == (80, 96) and layout["l0.mlp.down"] == (96, 80)
    assert layout["l1.mix.q"] == (72, 96) and layout["l1.mix.v"] == (120, 96) and layout["l1.mix.g"] == (120, 96)
    assert layout["l1.mix.i"] == (3, 96) and layout["l1.mix.f.b"] == (3,) and layout["l1.mix.norm"] == (120,)
    assert layout["l2.mix.dq"] == (40, 96) and layout["l2.mix.dq.norm"] == (40,) and layout["l2.mix.uq"] == (72, 40)
    assert layout["l2.mix.dkv"] == (32, 96) and layout["l2.mix.dkv.norm"] == (24,)
    assert layout["l2.mix.uk"] == (48, 24) and layout["l2.mix.uv"] == (72, 24)
    assert layout["l2.mix.g"] == (3, 96) and layout["l2.mix.o"] == (96, 72)
    assert not any(k.startswith(("l3.", "l4.")) for k in layout)  # the borrowed layers have no tensors


def test_every_constant_is_read_from_the_file():
    from kvcore_amd.registry import resolve_architecture

    arch = resolve_architecture(CONFIG_B)
    typed = arch.parse_config(CONFIG_B)
    assert typed.logit_softcap == 6.0 and typed.eps == 1e-6
    att = typed.layers[1].mixer
    assert (att.window, att.rot_dims, att.rot_base, att.scale) == (48, 64, 500000.0, 0.125)
    assert typed.layers[3].weights_of == 1 and typed.layers[3].mixer is att
    lat = typed.layers[2].mixer
    assert (lat.kv_rank, lat.q_rank, lat.rot_dim, lat.window, lat.rot_base) == (96, 64, 32, 100, 500000.0)
    assert typed.layers[0].mixer.gate_cap == 2.0
    spec = arch.build_spec(typed)
    assert spec.head.args["soft_cap"] == 6.0 and spec.head.args["tied"]
    assert spec.layers[1].mixer.args["window"] == 48 and spec.layers[1].mixer.args["scale"] == 0.125
    assert spec.layers[0].mixer.args["gate_cap"] == 2.0
    no_cap = arch.parse_config(CONFIG_C)
    assert no_cap.logit_softcap == 0.0 and no_cap.layers[3].mixer.window == 0 and no_cap.layers[3].mixer.rot_dims == 0


@pytest.mark.parametrize("change,match", [
    (lambda c: c["layers"][0].__setitem__("type", "conv"), "type"),
    (lambda c: c["layers"][0]["mixer"].pop("scale"), "scale"),
    (lambda c: c["layers"][0]["mixer"].__setitem__("kv_heads", 3), "kv_heads"),
    (lambda c: c["layers"][0]["mixer"].__setitem__("vdim", 16), "vdim"),
    (lambda c: c["layers"][0]["mixer"]["rot"].__setitem__("dims", 34), "rot.dims"),
    (lambda c: c["layers"][2]["mixer"]["rot"].__setitem__("dims", 4), "rot_dim"),
    (lambda c: c["layers"][1]["mixer"].__setitem__("gate_cap", 0.0), "gate_cap"),
    (lambda c: c["layers"][0]["mlp"].__setitem__("kind", "moe"), "kind"),
    (lambda c: c["layers"][3].__setitem__("weights_of", 3), "weights_of"),
    (lambda c: c.pop("norm"), "norm"),
    (lambda c: c.__setitem__("layers", []), "layers"),
])
def test_a_wrong_configuration_is_refused_by_name(change, match):
    from kvcore_amd.config.model_config import ConfigError
    from kvcore_amd.registry import resolve_architecture

    bad = copy.deepcopy(CONFIG_A)
    change(bad)
    with pytest.raises(ConfigError, match=match):
        resolve_architecture(bad).parse_config(bad)


@pytest.mark.parametrize("seed", range(12))
def test_drawn_configurations_build(seed):
    import random

    from kvcore_amd.models.decoder import DecoderModel

    cfg = random_config(random.Random(seed))
    model = DecoderModel(spec_of(cfg), torch.float32, "cpu")
    assert len(model.calls) == len(cfg["layers"])


def random_model(config, seed):
    """Weights for the plain model straight from the layout (float64, lively)."""
    from kvcore_amd.weights.loader import checkpoint_layout

    gen = torch.Generator().manual_seed(seed)
    out = {}
    for name, (shape, *_rest) in checkpoint_layout(spec_of(config)).items():
        leaf = name.split(".")[-1]
        t = torch.randn(shape, generator=gen, dtype=torch.float64)
        if leaf.startswith("norm"):
            out[name] = 1.0 + 0.2 * t
        elif name.endswith("f.b"):
            out[name] = 3.0 + t
        elif name == "embed" or leaf in ("sink", "b"):
            out[name] = t
        else:
            out[name] = t * (0.5 if leaf in ("i", "f") else 0.1)
    return out


@pytest.mark.parametrize("name", list(CONFIGS))
def test_the_plain_model_is_causal_and_borrowed_layers_share_tensors(name):
    config = CONFIGS[name][0]
    w = random_model(config, 3)
    tokens = [(7 * i + 3) % config["vocab"] for i in range(60)]
    streams = []
    full = plain.forward(config, w, tokens, streams)
    assert len(streams) == len(config["layers"]) and full.shape == (60, config["vocab"])
    part = plain.forward(config, w, tokens[:33])
    assert torch.allclose(full[:33], part, atol=1e-9)  # nothing looks ahead
    cap = config.get("logit_softcap")
    if cap:
        assert float(full.abs().max()) < cap


def test_plain_window_sink_and_rotation():
    """The pieces the other tests lean on, against definitions written out here by hand."""
    gen = torch.Generator().manual_seed(0)
    s = torch.randn(2, 5, 5, generator=gen, dtype=torch.float64)
    sink = torch.tensor([0.3, -2.0], dtype=torch.float64)
    p = plain.window_softmax(s, 2, sink)
    for h in range(2):
        for i in range(5):
            seen = [j for j in range(5) if 0 <= i - j < 2]
            den = sum(math.exp(float(s[h, i, j])) for j in seen) + math.exp(float(sink[h]))
            for j in range(5):
                want = math.exp(float(s[h, i, j])) / den if j in seen else 0.0
                assert abs(float(p[h, i, j]) - want) < 1e-12
    assert float(p.sum(-1).max()) < 1.0  # the sink takes its share
    x = torch.randn(3, 1, 6, generator=gen, dtype=torch.float64)
    pos = torch.tensor([0, 5, 9])
    half = plain.rotate(x, pos, 4, 100.0, False)
    pair = plain.rotate(x, pos, 4, 100.0, True)
    assert torch.equal(half[0], x[0]) and torch.equal(half[..., 4:], x[..., 4:])
    a = 5 * 100.0 ** (-2.0 * 1 / 4)
    assert abs(float(half[1, 0, 1]) - (float(x[1, 0, 1]) * math.cos(a) - float(x[1, 0, 3]) * math.sin(a))) < 1e-12
    assert abs(float(pair[1, 0, 3]) - (float(x[1, 0, 3]) * math.cos(a) + float(x[1, 0, 2]) * math.sin(a))) < 1e-12
    z = torch.tensor([-3.0, 0.0, 0.5, 4.0], dtype=torch.float64)
    assert torch.allclose(plain.gelu_tanh(z), torch.nn.functional.gelu(z, approximate="tanh"), atol=1e-12)


def test_plain_matrix_memory_against_its_sum_over_earlier_tokens():
    """The recurrence with its running maximum equals the sum it stands for: with F_t the sum of
    the log forget gates up to t, o_t = sum_j exp(F_t - F_j + i_j - m_t) (k_j . q_t) v_j over the
    same normaliser, where m_t = max(F_t, max_j (F_t - F_j + i_j)) (the maximum starts at 0)."""
    gen = torch.Generator().manual_seed(5)
    H, d, dv, T, width = 2, 6, 5, 40, 16
    m = {"heads": H, "dim": d, "vdim": dv, "gate_cap": 6.0}
    w = {"q": torch.randn(H * d, width, generator=gen, dtype=torch.float64) * 0.4,
         "k": torch.randn(H * d, width, generator=gen, dtype=torch.float64) * 0.4,
         "v": torch.randn(H * dv, width, generator=gen, dtype=torch.float64) * 0.4,
         "g": torch.randn(H * dv, width, generator=gen, dtype=torch.float64) * 0.4,
         "i": torch.randn(H, width, generator=gen, dtype=torch.float64),
         "f": torch.randn(H, width, generator=gen, dtype=torch.float64),
         "i.b": torch.randn(H, generator=gen, dtype=torch.float64), "f.b": torch.randn(H, generator=gen, dtype=torch.float64) + 2,
         "norm": torch.ones(H * dv, dtype=torch.float64), "o": torch.eye(H * dv, dtype=torch.float64)}
    h = torch.randn(T, width, generator=gen, dtype=torch.float64)
    got = plain.mlstm(h, w, m, 1e-6)
    q = (h @ w["q"].T).view(T, H, d) * d ** -0.5
    k = (h @ w["k"].T).view(T, H, d)
    v = (h @ w["v"].T).view(T, H, dv)
    gi = 6.0 * torch.tanh((h @ w["i"].T + w["i.b"]) / 6.0)
    gf = torch.nn.functional.logsigmoid(6.0 * torch.tanh((h @ w["f"].T + w["f.b"]) / 6.0))
    Fc = gf.cumsum(0)
    want = torch.zeros(T, H, dv, dtype=torch.float64)
    for t in range(T):
        for hh in range(H):
            logs = torch.stack([Fc[t, hh] - Fc[j, hh] + gi[j, hh] for j in range(t + 1)])
            mt = max(float(Fc[t, hh]), float(logs.max()))
            wts = torch.exp(logs - mt)
            num = sum(wts[j] * (k[j, hh] @ q[t, hh]) * v[j, hh] for j in range(t + 1))
            nq = sum(wts[j] * (k[j, hh] @ q[t, hh]) for j in range(t + 1))
            want[t, hh] = num / (max(abs(float(nq)), math.exp(-mt)) + 1e-6)
    want = plain.rms(want, 1e-6).reshape(T, H * dv) * torch.sigmoid(h @ w["g"].T)
    assert torch.allclose(got, want, atol=1e-9)
