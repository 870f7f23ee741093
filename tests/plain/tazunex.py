"""The Tazunex decoder written out plainly in float64, one function a mechanism.

Nothing here is shared with the product: the tests compare the engine's logits with these.
A model is ``(config mapping, name -> float64 tensor)``; the config mapping is config.json's.
"""

from __future__ import annotations

import math

import torch

F = torch.float64


def rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def gelu_tanh(z: torch.Tensor) -> torch.Tensor:
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def rotate(x: torch.Tensor, positions: torch.Tensor, dims: int, base: float, interleaved: bool) -> torch.Tensor:
    """``x [T, heads, d]``: the first ``dims`` elements of every head turn by ``p * base^(-2i/dims)``;
    element i pairs with i + dims/2, or 2i with 2i+1 when ``interleaved``."""
    half = dims // 2
    freq = torch.tensor([base ** (-2.0 * i / dims) for i in range(half)], dtype=F)
    ang = positions.to(F)[:, None] * freq[None, :]
    c, s = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
    out = x.clone()
    if interleaved:
        u, v = x[..., 0:dims:2], x[..., 1:dims:2]
        out[..., 0:dims:2] = u * c - v * s
        out[..., 1:dims:2] = v * c + u * s
    else:
        u, v = x[..., :half], x[..., half:dims]
        out[..., :half] = u * c - v * s
        out[..., half:dims] = v * c + u * s
    return out


def window_of(m: dict) -> int | None:
    """The mixer's window, None where its configuration names none (every earlier token is seen)."""
    return (m.get("mask") or {}).get("size")


def window_softmax(scores: torch.Tensor, window: int | None, sink: torch.Tensor | None) -> torch.Tensor:
    """``scores [heads, T, T]`` -> weights; query i sees key j with ``0 <= i - j < window``; with
    ``sink [heads]`` the denominator also holds ``exp(sink)``."""
    T = scores.shape[-1]
    window = T + 1 if window is None else window
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    seen = (j <= i) & (i - j < window)
    scores = scores.masked_fill(~seen, -math.inf)
    top = scores.max(-1, keepdim=True).values
    if sink is not None:
        top = torch.maximum(top, sink[:, None, None])
    e = torch.exp(scores - top)
    denom = e.sum(-1, keepdim=True)
    if sink is not None:
        denom = denom + torch.exp(sink[:, None, None] - top)
    return e / denom


def sink_attention(h: torch.Tensor, w: dict, m: dict, eps: float) -> torch.Tensor:
    """Grouped-query attention whose values are the keys as projected; q and k are normed over the
    whole projection, then rotated (half layout); a window; a sink in the softmax."""
    T = h.shape[0]
    H, G, d = m["heads"], m["kv_heads"], m["dim"]
    q = h @ w["q"].T
    k = h @ w["k"].T
    v = k.view(T, G, d)
    q = (rms(q, eps) * w["q.norm"]).view(T, H, d)
    kk = (rms(k, eps) * w["k.norm"]).view(T, G, d)
    pos = torch.arange(T)
    if m.get("rot"):
        q = rotate(q, pos, m["rot"]["dims"], m["rot"]["base"], False)
        kk = rotate(kk, pos, m["rot"]["dims"], m["rot"]["base"], False)
    rep = H // G
    kh = kk.repeat_interleave(rep, dim=1)
    vh = v.repeat_interleave(rep, dim=1)
    scores = torch.einsum("ihd,jhd->hij", q, kh) * m["scale"]
    p = window_softmax(scores, window_of(m), w["sink"])
    o = torch.einsum("hij,jhd->ihd", p, vh).reshape(T, H * d)
    return o @ w["o"].T


def latent_attention(h: torch.Tensor, w: dict, m: dict, eps: float) -> torch.Tensor:
    """Queries through a normed latent; keys and values from a normed latent ``c`` plus one rotated
    key part shared by the heads (interleaved rotation); a window; a gate per head."""
    T = h.shape[0]
    H, d, r, dv, rank = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    cq = rms(h @ w["dq"].T, eps) * w["dq.norm"]
    q = (cq @ w["uq"].T).view(T, H, d + r)
    q_plain, q_rot = q[..., :d], q[..., d:]
    dkv = h @ w["dkv"].T
    c = rms(dkv[:, :rank], eps) * w["dkv.norm"]
    k_rot = dkv[:, rank:].view(T, 1, r)
    pos = torch.arange(T)
    if r:
        q_rot = rotate(q_rot, pos, r, m["rot"]["base"], True)
        k_rot = rotate(k_rot, pos, r, m["rot"]["base"], True)
    k_rot = k_rot[:, 0]
    k_plain = (c @ w["uk"].T).view(T, H, d)
    v = (c @ w["uv"].T).view(T, H, dv)
    scores = (torch.einsum("ihd,jhd->hij", q_plain, k_plain) + torch.einsum("ihd,jd->hij", q_rot, k_rot)) * m["scale"]
    p = window_softmax(scores, window_of(m), None)
    o = torch.einsum("hij,jhd->ihd", p, v)
    gate = torch.sigmoid(h @ w["g"].T)
    return (o * gate[:, :, None]).reshape(T, H * dv) @ w["o"].T


def mlstm(h: torch.Tensor, w: dict, m: dict, eps: float) -> torch.Tensor:
    """A matrix memory per head with log gates and a running maximum that starts at 0."""
    T = h.shape[0]
    H, d, dv, cap = m["heads"], m["dim"], m["vdim"], m["gate_cap"]
    q = (h @ w["q"].T).view(T, H, d) * d ** -0.5
    k = (h @ w["k"].T).view(T, H, d)
    v = (h @ w["v"].T).view(T, H, dv)
    gi = cap * torch.tanh((h @ w["i"].T + w["i.b"]) / cap)
    gf = torch.nn.functional.logsigmoid(cap * torch.tanh((h @ w["f"].T + w["f.b"]) / cap))
    S = torch.zeros(H, d, dv, dtype=F)
    n = torch.zeros(H, d, dtype=F)
    mx = torch.zeros(H, dtype=F)
    out = torch.zeros(T, H, dv, dtype=F)
    for t in range(T):
        new = torch.maximum(gf[t] + mx, gi[t])
        keep = torch.exp(gf[t] + mx - new)
        take = torch.exp(gi[t] - new)
        S = keep[:, None, None] * S + take[:, None, None] * k[t][:, :, None] * v[t][:, None, :]
        n = keep[:, None] * n + take[:, None] * k[t]
        mx = new
        num = torch.einsum("hdv,hd->hv", S, q[t])
        den = torch.maximum((n * q[t]).sum(-1).abs(), torch.exp(-mx)) + 1e-6
        out[t] = num / den[:, None]
    o = rms(out, eps).reshape(T, H * dv) * w["norm"]
    return (o * torch.sigmoid(h @ w["g"].T)) @ w["o"].T


def gated_feed_forward(h: torch.Tensor, w: dict) -> torch.Tensor:
    return (gelu_tanh(h @ w["gate"].T) * (h @ w["up"].T)) @ w["down"].T


MIXERS = {"attention": sink_attention, "latent_attention": latent_attention, "mlstm": mlstm}


def sub(weights: dict, prefix: str) -> dict:
    return {k[len(prefix):]: v for k, v in weights.items() if k.startswith(prefix)}


def forward(config: dict, weights: dict, tokens: list[int], streams: list | None = None) -> torch.Tensor:
    """Logits ``[T, vocab]`` of one sequence from position 0; ``streams`` collects the residual
    stream after every layer run."""
    eps = config["norm"]["eps"]
    x = weights["embed"][torch.tensor(tokens)]
    for i, layer in enumerate(config["layers"]):
        owner = layer.get("weights_of")
        owner = i if owner is None else owner
        while config["layers"][owner].get("weights_of") is not None:
            owner = config["layers"][owner]["weights_of"]
        own = config["layers"][owner]
        p = f"l{owner}."
        a = MIXERS[own["type"]](rms(x, eps) * weights[p + "norm1"], sub(weights, p + "mix."), own["mixer"], eps)
        x = x + rms(a, eps) * weights[p + "norm1b"]
        if own.get("mlp") is not None:
            f = gated_feed_forward(rms(x, eps) * weights[p + "norm2"], sub(weights, p + "mlp."))
            x = x + rms(f, eps) * weights[p + "norm2b"]
        if streams is not None:
            streams.append(x.clone())
    logits = (rms(x, eps) * weights["final.norm"]) @ weights["embed"].T
    cap = config.get("logit_softcap")
    if cap:
        logits = cap * torch.tanh(logits / cap)
    return logits


def load_model_folder(folder):
    """``(config mapping, name -> float64 tensor)`` of a folder with config.json and safetensors files."""
    import json
    from pathlib import Path

    from safetensors.torch import load_file

    folder = Path(folder)
    config = json.loads((folder / "config.json").read_text())
    weights = {}
    for file in sorted(folder.glob("*.safetensors")):
        weights.update({k: v.to(F) for k, v in load_file(str(file)).items()})
    return config, weights


def windowed_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float, window: int | None,
                       sink: torch.Tensor | None) -> torch.Tensor:
    """``q [T, H, d]``, ``k [T, G, d]``, ``v [T, G, dv]`` at positions 0..T-1 -> ``[T, H, dv]``."""
    rep = q.shape[1] // k.shape[1]
    kh, vh = k.repeat_interleave(rep, dim=1), v.repeat_interleave(rep, dim=1)
    p = window_softmax(torch.einsum("ihd,jhd->hij", q, kh) * scale, window, sink)
    return torch.einsum("hij,jhd->ihd", p, vh)
