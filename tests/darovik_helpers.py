"""Configurations, model folders and batch helpers for the Darovik tests.

The configurations differ from each other in every size and option: layer order, widths, head
counts and grouping, key and value sizes, windows (down to one position, and none), latents,
numbers of stream copies (one, several, none at all), the loop (none, a part, the whole model,
once), experts with and without groups, layers without a feed-forward, and values that are 1 or
equal where another model's differ.
"""

from __future__ import annotations

from pathlib import Path

import torch


def _attn(heads, kv, dim, vdim, scale, window, diff):
    m = {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "scale": scale, "diff": diff}
    if window:
        m["mask"] = {"size": window}
    return m


def _latent(heads, dim, vdim, kv_rank, scale):
    return {"heads": heads, "dim": dim, "vdim": vdim, "kv_rank": kv_rank, "scale": scale}


def _ff(ff):
    return {"kind": "dense", "ff": ff}


def _moe(ff, experts, top, scale, groups=None):
    router = {"experts": experts, "top": top, "scale": scale}
    if groups:
        router["groups"] = {"count": groups[0], "keep": groups[1]}
    return {"kind": "moe", "expert": {"ff": ff}, "router": router}


# three copies of the stream, windows of 24 and 10 positions (pages of 8), the two middle layers
# run three times, experts in three groups of which two are kept, a layer without a feed-forward
CONFIG_A = {
    "architecture": "Darovik", "vocab": 211, "width": 96, "norm": {"eps": 1e-5}, "residual_mult": 0.5,
    "streams": 3, "loop": {"start": 1, "stop": 3, "times": 3},
    "layers": [
        {"type": "latent_attention", "mixer": _latent(3, 16, 24, 40, 0.25), "mlp": _ff(80)},
        {"type": "attention", "mixer": _attn(4, 2, 24, 40, 0.2, 24, 0.3), "mlp": _moe(24, 12, 3, 1.5, (3, 2))},
        {"type": "latent_attention", "mixer": _latent(5, 8, 16, 24, 0.3), "mlp": None},
        {"type": "attention", "mixer": _attn(3, 3, 16, 16, 0.25, 10, 0.6), "mlp": _ff(136)},
    ],
}

# the shapes that the matrix-core attention kernels serve in bfloat16 (pages of 16): maps of 32 and
# 64 (joint keys of 64 and 128) with values of the joint keys' size and of twice that size, a
# latent of 64 and of 128 with sixteen and four heads, a window of 48 (no multiple of the kernels'
# tiles); the whole model runs twice; four copies of the stream
CONFIG_B = {
    "architecture": "Darovik", "vocab": 320, "width": 128, "norm": {"eps": 1e-6}, "residual_mult": 0.8,
    "streams": 4, "loop": {"start": 0, "stop": 4, "times": 2},
    "layers": [
        {"type": "attention", "mixer": _attn(4, 2, 32, 64, 0.18, 48, 0.5), "mlp": _ff(192)},
        {"type": "latent_attention", "mixer": _latent(16, 32, 48, 64, 0.11), "mlp": _moe(64, 8, 2, 2.0)},
        {"type": "attention", "mixer": _attn(2, 1, 64, 256, 0.125, 100, 0.2), "mlp": _ff(64)},
        {"type": "latent_attention", "mixer": _latent(4, 32, 32, 128, 0.15), "mlp": _moe(64, 16, 4, 1.0, (4, 2))},
    ],
}

# ones and equal values: no copies of the stream at all (the plain residual sum, no link tensors),
# no loop, no multiplier, one head, one kv head, a window of one position beside a layer that sees
# everything, values of one element, a latent of one value, one expert chosen of one group, all
# experts chosen, an odd vocabulary
CONFIG_C = {
    "architecture": "Darovik", "vocab": 97, "width": 40, "norm": {"eps": 1e-4},
    "layers": [
        {"type": "attention", "mixer": _attn(1, 1, 8, 1, 1.0, 1, 0.5), "mlp": _ff(8)},
        {"type": "latent_attention", "mixer": _latent(1, 8, 1, 1, 0.5), "mlp": _moe(8, 3, 3, 1.0)},
        {"type": "attention", "mixer": _attn(2, 1, 16, 24, 0.5, 0, 0.1), "mlp": None},
        {"type": "latent_attention", "mixer": _latent(2, 4, 3, 5, 1.0), "mlp": _moe(16, 4, 1, 0.7, (4, 1))},
    ],
}

# one copy of the stream that still has its link tensors, a loop that runs once, groups of two
# experts of which one is chosen (a group worth its two best with two members) and groups of one,
# twenty query heads on one latent row, a latent of 280, maps of 40 with values of 72
CONFIG_D = {
    "architecture": "Darovik", "vocab": 256, "width": 64, "norm": {"eps": 1e-6}, "residual_mult": 1.3,
    "streams": 1, "loop": {"start": 2, "stop": 3, "times": 1},
    "layers": [
        {"type": "latent_attention", "mixer": _latent(20, 16, 8, 48, 0.15), "mlp": _moe(32, 8, 2, 2.5, (4, 3))},
        {"type": "attention", "mixer": _attn(6, 2, 40, 72, 0.15, 70, 0.4), "mlp": _moe(16, 6, 2, 1.0, (6, 3))},
        {"type": "latent_attention", "mixer": _latent(2, 24, 16, 280, 0.1), "mlp": _ff(32)},
        {"type": "attention", "mixer": _attn(3, 1, 56, 112, 0.15, 33, 0.5), "mlp": None},
    ],
}

CONFIGS = {"A": (CONFIG_A, 8), "B": (CONFIG_B, 16), "C": (CONFIG_C, 4), "D": (CONFIG_D, 16)}


def random_config(rng) -> dict:
    """A configuration drawn from ``rng`` (a ``random.Random``): two to six layers of either kind in
    any order, some without a feed-forward, with and without copies of the stream and a loop; every
    size and constant drawn anew."""
    width = rng.choice([64, 96, 128, 192, 256, 100, 72])

    def attn():
        kv = rng.choice([1, 2, 3, 4])
        g = rng.choice([1, 2, 4])
        dim = rng.choice([16, 32, 48, 64, 24, 40, 8])
        vdim = rng.choice([2 * dim, 2 * dim, 4 * dim, dim, 24, 80])
        window = 0 if rng.random() < 0.15 else rng.choice([7, 16, 33, 64, 100, 128, 50, 1])
        return _attn(kv * g, kv, dim, vdim, rng.choice([0.125, 0.2, 0.09]), window, rng.choice([0.5, 0.2, 0.8, 0.35]))

    def latent():
        return _latent(rng.choice([1, 2, 4, 6, 16, 18]), rng.choice([8, 16, 32, 64, 20]), rng.choice([8, 16, 48, 80, 1]),
                       rng.choice([8, 16, 24, 32, 48, 64, 96, 128, 20]), rng.choice([0.125, 0.2, 0.09]))

    def ff():
        r = rng.random()
        if r < 0.15:
            return None
        if r < 0.55:
            return _ff(rng.choice([24, 32, 48, 64, 96, 40, 136]))
        groups = rng.choice([None, (2, 1), (4, 2), (3, 3), (2, 2)])
        per = rng.choice([1, 2, 3, 4])
        experts = per * (groups[0] if groups else rng.choice([1, 2, 3, 5]))
        allowed = per * groups[1] if groups else experts
        return _moe(rng.choice([16, 24, 32, 64, 40]), experts, rng.randint(1, min(allowed, 4)),
                    rng.choice([1.0, 2.0, 2.5, 0.5]), groups)

    kinds = {"attention": attn, "latent_attention": latent}
    layers = []
    for _ in range(rng.randint(2, 6)):
        t = rng.choice(list(kinds))
        layers.append({"type": t, "mixer": kinds[t](), "mlp": ff()})
    out = {"architecture": "Darovik", "vocab": rng.choice([97, 256, 512, 1000]), "width": width,
           "norm": {"eps": rng.choice([1e-6, 1e-5])}, "layers": layers}
    if rng.random() < 0.8:
        out["residual_mult"] = rng.choice([0.5, 0.7, 1.0, 1.4])
    if rng.random() < 0.8:
        out["streams"] = rng.choice([1, 2, 2, 3, 4, 5, 8])
    if rng.random() < 0.7:
        start = rng.randint(0, len(layers) - 1)
        out["loop"] = {"start": start, "stop": rng.randint(start, len(layers)), "times": rng.choice([1, 2, 2, 3])}
    return out


def make_model_dir(folder: Path, config: dict, seed: int) -> Path:
    """A model folder from the product's random-weights mode, with the tensors redrawn so that
    each one matters: the sinks are of the size of the scores, the norms' gains lie around one, the
    vectors behind ``lambda`` make it differ from ``diff``, the corrections are of the size of the
    differences between the experts' scores, the links mix the copies visibly (and no copy dies
    out), the biases are felt, and the matrices are livelier than N(0, 0.02)."""
    from safetensors.torch import load_file, save_file

    from kvcore_amd.weights.loader import write_random_model

    write_random_model(folder, config, seed)
    path = folder / "model.safetensors"
    tensors = load_file(str(path))
    gen = torch.Generator().manual_seed(seed + 1)

    def noise(t, std, mean=0.0):
        return (torch.randn(t.shape, generator=gen) * std + mean).to(torch.bfloat16).to(t.dtype)

    for name, t in list(tensors.items()):
        leaf = name.split(".")[-1]
        if leaf == "sink":
            tensors[name] = noise(t, 1.0, 1.0)
        elif leaf in ("lq1", "lk1", "lq2", "lk2"):
            tensors[name] = noise(t, 0.6 * t.shape[0] ** -0.5, 0.5 * t.shape[0] ** -0.5 * (1 if leaf[-1] == "1" else -1))
        elif leaf == "correction":
            tensors[name] = noise(t, 0.3)
        elif leaf == "b":
            tensors[name] = noise(t, 0.3)
        elif ".hc" in name and leaf in ("in", "out"):
            tensors[name] = noise(t, 0.3, 0.8)
        elif ".hc" in name and leaf == "mix":
            tensors[name] = (torch.eye(t.shape[0]) * 0.7 + torch.randn(t.shape, generator=gen) * 0.25) \
                .to(torch.bfloat16).to(t.dtype)
        elif leaf == "norm" or leaf.startswith("norm"):
            tensors[name] = noise(t, 0.2, 1.0)
        elif name == "embed":
            tensors[name] = noise(t, 1.5 * t.shape[1] ** -0.5)
        elif leaf == "router":
            tensors[name] = noise(t, 0.25)
        elif t.dim() == 2:
            tensors[name] = noise(t, 0.08)
    save_file(tensors, str(path))
    return folder


def load_model_folder(folder):
    """``(config mapping, name -> float64 tensor)`` of a folder with config.json and safetensors files."""
    import json

    from safetensors.torch import load_file

    folder = Path(folder)
    config = json.loads((folder / "config.json").read_text())
    weights = {}
    for file in sorted(folder.glob("*.safetensors")):
        weights.update({k: v.to(torch.float64) for k, v in load_file(str(file)).items()})
    return config, weights


def batch_tensors(reqs, device="cuda"):
    """``reqs``: (slot, first position, number of tokens) per request, or None for a padded
    request of one padding token -> positions, token_req, q_start, slots (int32 on the device)
    and the number of tokens."""
    positions, token_req, q_start, slots = [], [], [0], []
    for r, item in enumerate(reqs):
        if item is None:
            positions.append(0)
            token_req.append(-1)
            slots.append(0)
        else:
            slot, start, n = item
            positions += list(range(start, start + n))
            token_req += [r] * n
            slots.append(slot)
        q_start.append(len(positions))

    def dev(v):
        return torch.tensor(v, dtype=torch.int32, device=device)

    return dict(positions=dev(positions), token_req=dev(token_req), q_start=dev(q_start), slots=dev(slots),
                num_reqs=len(reqs)), len(positions)
