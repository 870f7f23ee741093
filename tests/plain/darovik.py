"""The Darovik decoder written out plainly in float64, one function a mechanism.

Nothing here is shared with the product: the tests compare the engine's logits with these.
A model is ``(config mapping, name -> float64 tensor)``; the config mapping is config.json's.
Whole sequences, no cache: every function sees all ``T`` tokens of one request.
"""

from __future__ import annotations

import math

import torch

F = torch.float64


def rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def window_of(m: dict) -> int | None:
    """The mixer's window, None where its configuration names none (every earlier token is seen)."""
    return (m.get("mask") or {}).get("size")


def seen_keys(T: int, window: int | None) -> torch.Tensor:
    """``[T, T]`` bool: query i sees key j with ``j <= i`` and, under a window, ``i - j < window``."""
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    seen = j <= i
    if window is not None:
        seen = seen & (i - j < window)
    return seen


def masked_softmax(scores: torch.Tensor, seen: torch.Tensor, sink: torch.Tensor | None = None) -> torch.Tensor:
    """``scores [heads, T, T]`` -> weights over the seen keys; with ``sink [heads]`` the denominator
    holds ``exp(sink)`` as well, a term without a key or a value."""
    scores = scores.masked_fill(~seen, -math.inf)
    top = scores.max(-1, keepdim=True).values
    if sink is not None:
        top = torch.maximum(top, sink[:, None, None])
    e = torch.exp(scores - top)
    denom = e.sum(-1, keepdim=True)
    if sink is not None:
        denom = denom + torch.exp(sink[:, None, None] - top)
    return e / denom


def differential_lambda(w: dict, m: dict) -> float:
    return float(torch.exp((w["lq1"] * w["lk1"]).sum()) - torch.exp((w["lq2"] * w["lk2"]).sum()) + m["diff"])


def differential_attention(h: torch.Tensor, w: dict, m: dict, eps: float) -> torch.Tensor:
    """Two softmax maps a head over the same values, the second taken off the first ``lambda``
    times; the difference divided by its root mean square over the head, times ``1 - diff``."""
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ w["q"].T).view(T, H, 2, d)
    k = (h @ w["k"].T).view(T, G, 2, d)
    v = (h @ w["v"].T).view(T, G, dv)
    lam = differential_lambda(w, m)
    seen = seen_keys(T, window_of(m))
    out = torch.zeros(T, H, dv, dtype=F)
    for head in range(H):
        g = head // (H // G)
        maps = []
        for which in range(2):
            s = (q[:, head, which] @ k[:, g, which].T) * m["scale"]
            p = masked_softmax(s[None], seen)[0]
            maps.append(p @ v[:, g])
        o = maps[0] - lam * maps[1]
        out[:, head] = rms(o, eps) * (1.0 - m["diff"])
    return out.reshape(T, H * dv) @ w["o"].T


def latent_attention(h: torch.Tensor, w: dict, m: dict, eps: float) -> torch.Tensor:
    """Keys and values of every head from one normed latent a token; no positions; a sink a head."""
    T = h.shape[0]
    H, d, dv = m["heads"], m["dim"], m["vdim"]
    q = (h @ w["q"].T).view(T, H, d)
    c = rms(h @ w["dkv"].T, eps) * w["dkv.norm"]
    k = (c @ w["uk"].T).view(T, H, d)
    v = (c @ w["uv"].T).view(T, H, dv)
    s = torch.einsum("ihd,jhd->hij", q, k) * m["scale"]
    p = masked_softmax(s, seen_keys(T, window_of(m)), w["sink"])
    o = torch.einsum("hij,jhv->ihv", p, v)
    return o.reshape(T, H * dv) @ w["o"].T


def dense_ff(h: torch.Tensor, w: dict) -> torch.Tensor:
    z = torch.relu(h @ w["up"].T + w["up.b"])
    return (z * z) @ w["down"].T + w["down.b"]


def route(h: torch.Tensor, w: dict, r: dict) -> tuple[torch.Tensor, torch.Tensor]:
    """``(choice [T, top], weight [T, top])``: sigmoid scores; the choice is made on the scores
    plus the correction, inside the best groups only (a group is worth its two best choice
    scores); the weights are the plain scores of the chosen, over their sum, times the scale."""
    E, top = r["experts"], r["top"]
    s = torch.sigmoid(h @ w["router"].T)
    pick = s + w["correction"]
    groups = r.get("groups")
    if groups:
        count, keep = groups["count"], groups["keep"]
        per = E // count
        worth = pick.view(-1, count, per).topk(min(2, per), dim=-1).values.sum(-1)
        best = worth.topk(keep, dim=-1).indices
        allowed = torch.zeros(h.shape[0], count, dtype=torch.bool)
        allowed.scatter_(1, best, True)
        pick = pick.masked_fill(~allowed[:, :, None].expand(-1, -1, per).reshape(-1, E), -math.inf)
    choice = pick.topk(top, dim=-1).indices
    chosen = s.gather(1, choice)
    weight = chosen / (chosen.sum(-1, keepdim=True) + 1e-20) * r["scale"]
    return choice, weight


def expert(h: torch.Tensor, w: dict, e: int) -> torch.Tensor:
    g = h @ w[f"e{e}.gate"].T
    return (g * torch.sigmoid(g) * (h @ w[f"e{e}.up"].T)) @ w[f"e{e}.down"].T


def routed_ff(h: torch.Tensor, w: dict, mlp: dict) -> torch.Tensor:
    choice, weight = route(h, w, mlp["router"])
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for c in range(choice.shape[1]):
            out[t] += weight[t, c] * expert(h[t: t + 1], w, int(choice[t, c]))[0]
    return out


def sub(weights: dict, prefix: str) -> dict:
    return {k[len(prefix):]: v for k, v in weights.items() if k.startswith(prefix)}


def layer_order(config: dict) -> list[int]:
    n = len(config["layers"])
    loop = config.get("loop")
    if not loop:
        return list(range(n))
    start, stop, times = loop["start"], loop["stop"], loop["times"]
    return list(range(start)) + list(range(start, stop)) * times + list(range(stop, n))


def forward(config: dict, weights: dict, tokens, streams_after=None) -> torch.Tensor:
    """Logits ``[T, vocab]`` for one request.  ``streams_after``: a list that receives the stream
    (the sum of its copies) after every layer run."""
    eps, m = config["norm"]["eps"], config.get("residual_mult", 1.0)
    copies = config.get("streams")
    x0 = weights["embed"][torch.as_tensor(tokens, dtype=torch.long)]
    xs = [x0.clone() for _ in range(copies or 1)]
    for i in layer_order(config):
        layer = config["layers"][i]
        for q, kind in ((1, "mix"), (2, "mlp")):
            if kind == "mlp" and layer.get("mlp") is None:
                continue
            w = sub(weights, f"l{i}.{kind}.")
            if copies:
                hc = sub(weights, f"l{i}.hc{q}.")
                u = sum(hc["in"][s] * xs[s] for s in range(copies))
            else:
                u = xs[0]
            h = rms(u, eps) * weights[f"l{i}.norm{q}"]
            if kind == "mix":
                if layer["type"] == "attention":
                    y = differential_attention(h, w, layer["mixer"], eps)
                elif layer["type"] == "latent_attention":
                    y = latent_attention(h, w, layer["mixer"], eps)
                else:
                    raise ValueError(layer["type"])
            elif layer["mlp"]["kind"] == "dense":
                y = dense_ff(h, w)
            else:
                y = routed_ff(h, w, layer["mlp"])
            if copies:
                xs = [sum(hc["mix"][s, t] * xs[s] for s in range(copies)) + m * hc["out"][t] * y
                      for t in range(copies)]
            else:
                xs = [xs[0] + m * y]
        if streams_after is not None:
            streams_after.append(sum(xs))
    x = rms(sum(xs), eps) * weights["final.norm"]
    return x @ weights["embed"].T
