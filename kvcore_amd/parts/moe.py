"""A feed-forward of routed experts: every token runs the few experts its router chooses.

    scores = softmax(W_r h), or sigmoid(W_r h) element by element            (float32)
    choice = the `top` best experts, by score (+ a learned correction per expert, where the layer
             has one), among those of the `keep` best of `groups` equal groups of neighbouring
             experts (a group is as good as its best expert, or as the sum of its best two)
    weight = scores[choice] / (sum of them + 1e-20) * weight_scale    (the scores without the correction)
    out    = sum_c weight_c * expert_choice_c(h)  (+ shared(h), an expert that every token runs)

An expert is a gated feed-forward with a clamped activation: ``g = min(W_gate h, limit)``, ``u =
clamp(W_up h, -limit, limit)``, ``W_down (g * sigmoid(alpha g) * (u + up_shift))``; an infinite
limit, ``alpha`` 1 and ``up_shift`` 0 make it ``W_down (silu(W_gate h) * W_up h)``.  The experts' matrices are
stacked along a leading expert dimension (each expert's gate rows, then its up rows), the routing
stays on the device and every launch is sized by the step's token count alone, so a step may be
captured into a graph.  The result is float32 rows: the weighted sum is not rounded before it
joins the stream.
"""

from __future__ import annotations

import math

import torch

from kvcore_amd.ops import library as ops

from .base import FeedForward, ParamSource, ParamSpec, register_feed_forward

GLU_ALPHA = 1.702


class RoutedExperts(FeedForward):
    """``experts`` experts of ``expert_size`` hidden units, ``top`` a token; ``groups`` and
    ``keep`` as above (1 and 1: every expert may be chosen); ``shared_size`` > 0 adds the shared
    expert (``shared_limit`` its clamp).  ``limit`` None: no clamp.  ``score``: ``softmax`` or
    ``sigmoid``; ``correction``: the layer has a learned value per expert (tensor ``correction``)
    that joins the scores for the choice alone; ``group_best``: a group is worth its best 1 or 2
    choice scores; ``weight_scale`` multiplies the weights; ``up_shift`` is added to the up branch.
    ``tensor_names`` renames checkpoint tensors (keys: router, correction, expert (a pattern with
    ``{e}``), shared, gate, up, down)."""

    def __init__(self, *, hidden_size: int, experts: int, top: int, expert_size: int, limit: float | None,
                 groups: int = 1, keep: int = 1, shared_size: int = 0, shared_limit: float | None = None,
                 alpha: float = GLU_ALPHA, score: str = "softmax", correction: bool = False, group_best: int = 1,
                 weight_scale: float = 1.0, up_shift: float = 1.0,
                 tensor_names: dict[str, str] | None = None) -> None:
        if experts <= 0 or not 0 < top <= experts or expert_size <= 0:
            raise ValueError(f"{top} of {experts} experts of {expert_size} units")
        if groups <= 0 or experts % groups or not 0 < keep <= groups:
            raise ValueError(f"{experts} experts do not form {groups} equal groups of which {keep} are kept")
        if top > 64:
            raise ValueError("the routing kernel serves at most 64 choices a token")
        self.hidden_size, self.experts, self.top, self.expert_size = hidden_size, experts, top, expert_size
        if score not in ops.ROUTE_SCORES or group_best not in (1, 2):
            raise ValueError(f"router scores by {sorted(ops.ROUTE_SCORES)}, groups by their best 1 or 2; "
                             f"got {score!r} and {group_best}")
        if shared_size and (limit is None or up_shift != 1.0):
            raise ValueError("the shared expert's kernel has the clamped activation with an up branch plus one")
        limit = math.inf if limit is None else float(limit)
        self.limit, self.groups, self.keep, self.alpha = limit, groups, keep, float(alpha)
        self.score, self.has_correction, self.group_best = score, bool(correction), int(group_best)
        self.weight_scale, self.up_shift = float(weight_scale), float(up_shift)
        self.shared_size = shared_size
        self.shared_limit = float(limit if shared_limit is None else shared_limit)
        self.names = {"router": "router.weight", "correction": "correction", "expert": "experts.{e}", "shared": "shared",
                      "gate": "gate.weight", "up": "up.weight", "down": "down.weight", **(tensor_names or {})}

    def param_specs(self) -> list[ParamSpec]:
        n, H, E, I = self.names, self.hidden_size, self.experts, self.expert_size
        gate_up, down = [], []
        for e in range(E):
            prefix = n["expert"].format(e=e)
            gate_up.append(ParamSource(f"{prefix}.{n['gate']}", 2 * I * e, I))
            gate_up.append(ParamSource(f"{prefix}.{n['up']}", 2 * I * e + I, I))
            down.append(ParamSource(f"{prefix}.{n['down']}", H * e, H))
        specs = [
            ParamSpec("router.weight", (E, H), kind="vector", init="normal", sources=(ParamSource(n["router"], 0, E),)),
            ParamSpec("experts.gate_up", (2 * I * E, H), sources=tuple(gate_up)),
            ParamSpec("experts.down", (H * E, I), sources=tuple(down)),
        ]
        if self.has_correction:
            specs.append(ParamSpec("correction", (E,), kind="vector", init="normal",
                                   sources=(ParamSource(n["correction"], 0, E),)))
        if self.shared_size:
            S, sp = self.shared_size, n["shared"]
            specs.append(ParamSpec("shared.gate_up", (2 * S, H), sources=(
                ParamSource(f"{sp}.{n['gate']}", 0, S), ParamSource(f"{sp}.{n['up']}", S, S))))
            specs.append(ParamSpec("shared.down", (H, S), sources=(ParamSource(f"{sp}.{n['down']}", 0, H),)))
        return specs

    def product_weights(self) -> tuple[str, ...]:
        # the experts' stacked matrices too: steps of single tokens stream their packed twins
        shared = ("shared.gate_up", "shared.down") if self.shared_size else ()
        return ("experts.gate_up", "experts.down", *shared)

    def forward_into(self, residual, x, ctx, call, add=None):
        """``residual += add + ff(x)`` (float32 rows), the sums made in the kernel that adds up the
        experts: what a block calls that would otherwise add the result into the stream itself."""
        self.forward(x, ctx, call, into=residual, add=add)

    def forward(self, x, ctx, call, sink=None, into=None, add=None):
        p, H, E, I, top = self.params, self.hidden_size, self.experts, self.expert_size, self.top
        T = ctx.num_tokens
        pairs = T * top
        # the router reads the rows as they are and sums in float32; logits and choice in one kernel
        choice = ctx.buf(f"moe_choice:{top}", top, torch.int32)
        weight = ctx.buf(f"moe_weight:{top}", top, torch.float32)
        ops.moe_router(choice, weight, x, p["router.weight"], top=top, groups=self.groups, keep=self.keep,
                       score=self.score, correction=p.get("correction"), group_best=self.group_best,
                       weight_scale=self.weight_scale)
        cap = ctx.buffers.token_capacity
        sorted_pairs = ctx.buffers.get(f"moe_sorted:{top}", pairs, 1, torch.int32, reserve=cap * top).view(-1)
        # portions of prompts give the experts rows enough for tiles of 64, single tokens tiles of 16
        tile_rows = ops.moe_tile_rows(pairs, E, x, (H, I))
        max_tiles = ops.moe_max_tiles(pairs, E, tile_rows)
        tiles = ctx.buffers.get(f"moe_tiles:{top}:{E}", max_tiles, 3, torch.int32,
                                reserve=ops.moe_max_tiles(cap * top, E, 16))
        num_tiles = ctx.buffers.get("moe_num_tiles", 1, 1, torch.int32).view(-1)
        ops.moe_align(sorted_pairs, tiles, num_tiles, choice, E, tile_rows)
        act = ctx.buffers.get(f"moe_act:{I}", pairs, I, ctx.dtype, reserve=cap * top)
        ops.moe_gemm(act, x, p["experts.gate_up"], sorted_pairs, tiles, num_tiles, pairs=pairs, experts=E,
                     in_div=top, out_sorted=True, gated=True, limit=self.limit, alpha=self.alpha, up_shift=self.up_shift,
                     tile_rows=tile_rows)
        y = ctx.buffers.get(f"moe_y:{H}", pairs, H, torch.float32, reserve=cap * top)
        ops.moe_gemm(y, act, p["experts.down"], sorted_pairs, tiles, num_tiles, pairs=pairs, experts=E,
                     in_div=0, out_sorted=False, gated=False, tile_rows=tile_rows)
        shared = None
        if self.shared_size:
            S = self.shared_size
            gate_up = ctx.buf(f"moe_shared_gu:{2 * S}", 2 * S)
            ops.linear(gate_up, x, p["shared.gate_up"])
            sact = ctx.buf(f"moe_shared_act:{S}", S)
            ops.clamped_glu(sact, gate_up, self.shared_limit, self.alpha)
            shared = ctx.buf(f"moe_shared_out:{H}", H, torch.float32)
            ops.linear(shared, sact, p["shared.down"])
        if into is not None:
            ops.moe_combine(into, y, weight, shared, add, accumulate=True)
            return into
        out = ctx.buf("ffn_out_f32", H, torch.float32)
        ops.moe_combine(out, y, weight, shared, None)
        return out


register_feed_forward("routed_experts", RoutedExperts)
