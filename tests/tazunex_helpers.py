"""Configurations, model folders and batch helpers for the Tazunex tests.

The configurations differ from each other in every size and option: layer order, widths, head
counts and grouping, key sizes, windows (down to one position, and none), rotated widths (part
of a head, a whole head, two elements, none), latent sizes, gate caps, feed-forward widths,
layers without a feed-forward, layers that run another layer's tensors, with and without a cap
on the logits, and values that are 1 or equal where another model's differ.
"""

from __future__ import annotations

import json
from pathlib import Path

import torch


def _attn(heads, kv, dim, scale, window, rot):
    m = {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": dim, "scale": scale}
    if window:
        m["mask"] = {"size": window}
    if rot:
        m["rot"] = {"dims": rot[0], "base": rot[1]}
    return m


def _latent(heads, dim, rot_dim, vdim, kv_rank, q_rank, scale, window, base=10000.0):
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "q_rank": q_rank,
         "scale": scale}
    if window:
        m["mask"] = {"size": window}
    if rot_dim:
        m["rot"] = {"dims": rot_dim, "base": base}
    return m


def _mem(heads, dim, vdim, cap):
    return {"heads": heads, "dim": dim, "vdim": vdim, "gate_cap": cap}


def _ff(ff):
    return {"kind": "dense", "ff": ff}


_ATT_A = _attn(4, 2, 32, 0.2, 24, (16, 10000.0))
_MEM_A = _mem(3, 24, 40, 3.0)

# grouped heads of 32 with half of each rotated and windows of 24 and 10 positions (pages of 8),
# an attention layer and a memory layer that run twice, a latent layer without a feed-forward
CONFIG_A = {
    "architecture": "Tazunex", "vocab": 211, "width": 96, "norm": {"eps": 1e-5}, "logit_softcap": 4.0,
    "layers": [
        {"type": "attention", "mixer": _ATT_A, "mlp": _ff(80)},
        {"type": "mlstm", "mixer": _MEM_A, "mlp": _ff(136)},
        {"type": "latent_attention", "mixer": _latent(3, 16, 8, 24, 24, 40, 0.25, 10), "mlp": None},
        {"type": "attention", "mixer": _ATT_A, "mlp": _ff(80), "weights_of": 0},
        {"type": "mlstm", "mixer": _MEM_A, "mlp": _ff(136), "weights_of": 1},
    ],
}

# the shapes that the matrix-core attention kernels serve in bfloat16 (pages of 16): heads of 64
# rotated whole, four query heads a kv head, a window of 48 (no multiple of the kernels' tiles);
# a latent of 96 with 32 rotated elements (rows of 128, four heads), a window of 100
_ATT_B = _attn(8, 2, 64, 0.125, 48, (64, 500000.0))
CONFIG_B = {
    "architecture": "Tazunex", "vocab": 320, "width": 128, "norm": {"eps": 1e-6}, "logit_softcap": 6.0,
    "layers": [
        {"type": "mlstm", "mixer": _mem(2, 64, 64, 2.0), "mlp": _ff(64)},
        {"type": "attention", "mixer": _ATT_B, "mlp": _ff(192)},
        {"type": "latent_attention", "mixer": _latent(4, 32, 32, 48, 96, 64, 0.11, 100, 500000.0), "mlp": _ff(64)},
        {"type": "attention", "mixer": _ATT_B, "mlp": _ff(192), "weights_of": 1},
    ],
}

# ones and equal values: one head, one kv head, a window of one position (a token sees itself
# and the sink only) beside layers that see everything, two rotated elements and none, values of
# one element, a query latent of one value, no cap on the logits, an odd vocabulary
CONFIG_C = {
    "architecture": "Tazunex", "vocab": 97, "width": 40, "norm": {"eps": 1e-4},
    "layers": [
        {"type": "mlstm", "mixer": _mem(1, 8, 1, 1.0), "mlp": _ff(8)},
        {"type": "attention", "mixer": _attn(1, 1, 16, 1.0, 1, (2, 100.0)), "mlp": None},
        {"type": "latent_attention", "mixer": _latent(1, 8, 2, 1, 6, 1, 0.5, 0, 50.0), "mlp": _ff(24)},
        {"type": "attention", "mixer": _attn(2, 1, 16, 0.5, 0, None), "mlp": _ff(16)},
        {"type": "latent_attention", "mixer": _latent(2, 4, 0, 3, 5, 7, 1.0, 3), "mlp": None},
    ],
}

# wide states and many heads: 200 key channels a head (many rows a thread), 80 value channels
# (with the normaliser's column more than one tile), twenty query heads on one latent row of 64
# (more than the kernel for single tokens takes a kv head), heads of 48 rotated whole, a latent of
# 280 values (cached rows of 288: wider than the attention kernels' usual instances)
CONFIG_D = {
    "architecture": "Tazunex", "vocab": 256, "width": 64, "norm": {"eps": 1e-6}, "logit_softcap": 10.0,
    "layers": [
        {"type": "mlstm", "mixer": _mem(2, 200, 80, 5.0), "mlp": _ff(32)},
        {"type": "latent_attention", "mixer": _latent(20, 16, 16, 8, 48, 24, 0.15, 70), "mlp": _ff(32)},
        {"type": "attention", "mixer": _attn(3, 1, 48, 0.15, 100, (48, 25000.0)), "mlp": None},
        {"type": "latent_attention", "mixer": _latent(2, 24, 8, 16, 280, 32, 0.1, 40), "mlp": None},
    ],
}

CONFIGS = {"A": (CONFIG_A, 8), "B": (CONFIG_B, 16), "C": (CONFIG_C, 4), "D": (CONFIG_D, 16)}


def random_config(rng) -> dict:
    """A configuration drawn from ``rng`` (a ``random.Random``): three to eight layers of any kind in
    any order, some borrowing an earlier layer's tensors, some without a feed-forward; every size
    and constant drawn anew."""
    width = rng.choice([64, 96, 128, 192, 256, 100, 72])

    def attn():
        kv = rng.choice([1, 2, 3, 4])
        g = rng.choice([1, 2, 4])
        dim = rng.choice([16, 32, 48, 64, 64, 128, 24, 40])
        rot = None if rng.random() < 0.15 else (rng.choice([d for d in (2, 8, 16, 32, 64, dim) if d <= dim and d % 2 == 0]),
                                                 rng.choice([10000.0, 500000.0, 300.0]))
        window = 0 if rng.random() < 0.15 else rng.choice([7, 16, 33, 64, 100, 128, 50, 1])
        return _attn(kv * g, kv, dim, rng.choice([0.125, 0.2, 0.09]), window, rot)

    def latent():
        rot = rng.choice([0, 2, 8, 16, 32])
        rank = rng.choice([8, 16, 24, 32, 48, 64 - rot, 96, 128 - rot, 20])
        window = 0 if rng.random() < 0.15 else rng.choice([7, 16, 33, 64, 100, 50])
        return _latent(rng.choice([1, 2, 4, 6, 16, 18]), rng.choice([8, 16, 32, 64, 20]), rot, rng.choice([8, 16, 48, 80, 1]),
                       rank, rng.choice([8, 32, 48, 96, 5]), rng.choice([0.125, 0.2, 0.09]), window,
                       rng.choice([10000.0, 500000.0]))

    def mem():
        return _mem(rng.choice([1, 2, 3, 6]), rng.choice([8, 16, 32, 48, 64, 20]), rng.choice([16, 64, 32, 40, 128, 9]),
                    rng.choice([1.0, 2.0, 3.0, 5.0]))

    kinds = {"attention": attn, "latent_attention": latent, "mlstm": mem}
    layers = []
    for _ in range(rng.randint(3, 8)):
        own = [j for j, l in enumerate(layers) if "weights_of" not in l]
        if own and rng.random() < 0.3:
            j = rng.choice(own)
            layer = dict(layers[j])
            layer["weights_of"] = j
            layers.append(layer)
            continue
        t = rng.choice(list(kinds))
        layers.append({"type": t, "mixer": kinds[t](), "mlp": _ff(rng.choice([24, 32, 48, 64, 96, 40, 136])) if rng.random() < 0.85 else None})
    out = {"architecture": "Tazunex", "vocab": rng.choice([97, 256, 512, 1000]), "width": width,
           "norm": {"eps": rng.choice([1e-6, 1e-5])}, "layers": layers}
    if rng.random() < 0.8:
        out["logit_softcap"] = rng.choice([3.0, 5.0, 15.0])
    return out


def make_model_dir(folder: Path, config: dict, seed: int) -> Path:
    """A model folder from the product's random-weights mode, with the tensors redrawn so that
    each one matters: the sinks and gate biases spread widely, the norms' gains lie around one,
    the gate matrices are large enough for the caps to bite (and no larger: the input gate stands
    in an exponent, so a model with wild gates magnifies bfloat16's rounding beyond any fixed
    bound), the embedding gives logits of a size that the cap bends, and the matrices are
    livelier than N(0, 0.02)."""
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
            tensors[name] = noise(t, 1.5, 1.0)
        elif name.endswith("i.b"):
            tensors[name] = noise(t, 0.5)
        elif name.endswith("f.b"):
            tensors[name] = noise(t, 1.5, 3.0)
        elif name.endswith("mix.i") or name.endswith("mix.f"):
            tensors[name] = noise(t, 0.1)
        elif leaf == "norm" or leaf.startswith("norm"):
            tensors[name] = noise(t, 0.2, 1.0)
        elif name == "embed":
            tensors[name] = noise(t, 1.5 * t.shape[1] ** -0.5)
        elif t.dim() == 2:
            tensors[name] = noise(t, 0.08)
    save_file(tensors, str(path))
    return folder


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
