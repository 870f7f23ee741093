"""Mixers whose memory is one float32 matrix per head and request, ``S [dim, vdim]``, updated
token by token and read with the query (linear attention and its kin).

``GatedLinearAttention``: ``q = W_q h * q_scale``, ``k = W_k h``, ``v = W_v h``; a decay per key
channel from a low-rank product, ``a = sigmoid(W_a2 (W_a1 h) + b) ^ (1 / tau)``;

    S_t = diag(a_t) S_(t-1) + k_t v_t^T,    o_t = S_t^T q_t.

``GatedDeltaRule``: q, k (``qk_heads`` heads of ``dim``, shared by ``heads / qk_heads`` value heads
each) and v pass a short causal convolution per channel and silu; q and k become unit vectors per
head (q times ``q_scale``); ``beta = sigmoid(W_b h)``, one decay per head ``g = exp(-exp(A_log)
softplus(W_a h + dt_bias))``;

    S <- g S;   u = beta (v - S^T k);   S <- S + k u^T;   o = S^T q.

Both finish alike: every head's ``o`` over its root mean square, times a gain of ``vdim`` values
shared by the heads, times ``silu(W_g h)``, then the output product.  The state (and the
convolution's last ``taps - 1`` inputs) live in float32 slot arrays; a request starts from zeros
at position 0.  Decays, gates, unit norms and the recurrence are float32; the products run in the
model dtype with float32 sums, which the recurrence reads unrounded.
"""

from __future__ import annotations

import torch

from kvcore_amd.ops import library as ops

from .base import Mixer, ParamSource, ParamSpec, StateNeed, register_mixer


def _src(name: str, rows: int) -> tuple[ParamSource, ...]:
    return (ParamSource(name, 0, rows),)


def _stacked(pairs: list[tuple[str, int]]) -> tuple[ParamSource, ...]:
    out, at = [], 0
    for name, rows in pairs:
        out.append(ParamSource(name, at, rows))
        at += rows
    return tuple(out)


class _MatrixStateMixer(Mixer):
    """What the two mixers share: the sizes, the state, the head norm with its gate, the output."""

    def _finish(self, o: torch.Tensor, gate: torch.Tensor, ctx) -> torch.Tensor:
        p = self.params
        normed = ctx.buf(f"ms_normed:{self.inner}", self.inner)
        ops.head_rmsnorm_gate(normed, o, gate, p["norm"], self.eps, self.heads, self.vdim)
        if self.float32_result:
            out = ctx.buf("mixer_out_f32", self.hidden_size, torch.float32)
        else:
            out = ctx.buf("mixer_out", self.hidden_size)
        ops.linear(out, normed, p["o.weight"])
        return out

    def check_limits(self, limits) -> None:
        if self.dim > 256:
            raise ValueError(f"{self.dim} key channels a head: the recurrence kernel serves 256")

    @staticmethod
    def _batch(ctx) -> dict:
        return dict(positions=ctx.positions, token_req=ctx.token_req, q_start=ctx.q_start,
                    slots=ctx.slots, num_reqs=ctx.num_reqs)


class GatedLinearAttention(_MatrixStateMixer):
    """``heads`` heads with keys of ``dim`` and values of ``vdim``; ``tau`` the decay's root;
    ``decay_rank`` the width of the low-rank product behind the decay.  ``tensor_names`` renames
    checkpoint tensors (keys: q, k, v, g, o, norm, a1, a2, a2_bias)."""

    def __init__(self, *, hidden_size: int, heads: int, dim: int, vdim: int, tau: float, decay_rank: int,
                 eps: float, q_scale: float | None = None, tensor_names: dict[str, str] | None = None,
                 float32_result: bool = False, position=None) -> None:
        if min(heads, dim, vdim, decay_rank) <= 0 or not tau > 0:
            raise ValueError("gated linear attention needs positive sizes and a positive tau")
        self.hidden_size, self.heads, self.dim, self.vdim = hidden_size, heads, dim, vdim
        self.tau, self.rank, self.eps = float(tau), decay_rank, eps
        self.q_scale = dim ** -0.5 if q_scale is None else float(q_scale)
        self.float32_result = float32_result
        self.qk, self.inner = heads * dim, heads * vdim
        self.names = {"q": "q.weight", "k": "k.weight", "v": "v.weight", "g": "g.weight", "o": "o.weight",
                      "norm": "norm.weight", "a1": "a1.weight", "a2": "a2.weight", "a2_bias": "a2.bias",
                      **(tensor_names or {})}

    def param_specs(self) -> list[ParamSpec]:
        n, H = self.names, self.hidden_size
        return [
            ParamSpec("in_proj.weight", (2 * self.qk + 2 * self.inner, H), sources=_stacked(
                [(n["q"], self.qk), (n["k"], self.qk), (n["v"], self.inner), (n["g"], self.inner)])),
            ParamSpec("a1.weight", (self.rank, H), sources=_src(n["a1"], self.rank)),
            ParamSpec("a2.weight", (self.qk, self.rank), sources=_src(n["a2"], self.qk)),
            ParamSpec("a2.bias", (self.qk,), kind="vector", init="normal", sources=_src(n["a2_bias"], self.qk)),
            ParamSpec("norm", (self.vdim,), kind="vector", init="gain", sources=_src(n["norm"], self.vdim)),
            ParamSpec("o.weight", (H, self.inner), sources=_src(n["o"], H)),
        ]

    def product_weights(self) -> tuple[str, ...]:
        return ("in_proj.weight", "o.weight")

    def state_needs(self) -> tuple[StateNeed, ...]:
        return (StateNeed((self.heads, ops.linear_state_rows(self.dim), self.vdim)),)

    def forward(self, x, ctx, call, sink=None):
        p, qk, inner = self.params, self.qk, self.inner
        state = ctx.states[call.state_indices[0]]
        width = 2 * qk + 2 * inner
        proj = ctx.buf(f"gla_proj:{width}", width, torch.float32)
        ops.linear(proj, x, p["in_proj.weight"])
        low = ctx.buf(f"gla_low:{self.rank}", self.rank)
        ops.linear(low, x, p["a1.weight"])
        z = ctx.buf(f"gla_z:{qk}", qk, torch.float32)
        ops.linear(z, low, p["a2.weight"])
        decay = ctx.buf(f"gla_decay:{qk}", qk, torch.float32)
        ops.sigmoid_power(decay, z, p["a2.bias"], 1.0 / self.tau)
        o = ctx.buf(f"ms_o:{inner}", inner, torch.float32)
        ops.linear_state_scan(o, proj[:, :qk], proj[:, qk:2 * qk], proj[:, 2 * qk:2 * qk + inner], decay, None,
                              state, heads=self.heads, qk_heads=self.heads, dim=self.dim, vdim=self.vdim,
                              delta_rule=False, q_scale=self.q_scale, **self._batch(ctx))
        return self._finish(o, proj[:, 2 * qk + inner:], ctx)


class GatedDeltaRule(_MatrixStateMixer):
    """``heads`` value heads of ``vdim``, ``qk_heads`` query/key heads of ``dim``, a convolution of
    ``conv`` taps (the last column of its weights is the current token's, no bias); ``unit_eps``
    the eps inside the root of the unit norm.  ``tensor_names`` renames checkpoint tensors (keys:
    q, k, v, q_conv, k_conv, v_conv, b, a, a_log, dt_bias, g, o, norm)."""

    def __init__(self, *, hidden_size: int, heads: int, qk_heads: int, dim: int, vdim: int, conv: int,
                 eps: float, unit_eps: float = 1e-6, q_scale: float | None = None,
                 tensor_names: dict[str, str] | None = None, float32_result: bool = False,
                 position=None) -> None:
        if min(heads, qk_heads, dim, vdim) <= 0 or heads % qk_heads:
            raise ValueError(f"{heads} heads are not a multiple of {qk_heads} query/key heads")
        if conv < 1:
            raise ValueError(f"a convolution needs at least one tap, got {conv}")
        self.hidden_size, self.heads, self.qk_heads, self.dim, self.vdim = hidden_size, heads, qk_heads, dim, vdim
        self.taps, self.eps, self.unit_eps = conv, eps, float(unit_eps)
        self.q_scale = dim ** -0.5 if q_scale is None else float(q_scale)
        self.float32_result = float32_result
        self.qk, self.inner = qk_heads * dim, heads * vdim
        self.conv_dim = 2 * self.qk + self.inner
        self.names = {"q": "q.weight", "k": "k.weight", "v": "v.weight", "q_conv": "q.conv.weight",
                      "k_conv": "k.conv.weight", "v_conv": "v.conv.weight", "b": "b.weight", "a": "a.weight",
                      "a_log": "A_log", "dt_bias": "dt_bias", "g": "g.weight", "o": "o.weight",
                      "norm": "norm.weight", **(tensor_names or {})}

    def param_specs(self) -> list[ParamSpec]:
        n, H, nh = self.names, self.hidden_size, self.heads
        return [
            ParamSpec("in_proj.weight", (self.conv_dim + self.inner + 2 * nh, H), sources=_stacked(
                [(n["q"], self.qk), (n["k"], self.qk), (n["v"], self.inner), (n["g"], self.inner),
                 (n["a"], nh), (n["b"], nh)])),
            ParamSpec("conv.weight", (self.conv_dim, self.taps), kind="vector", init="normal", sources=_stacked(
                [(n["q_conv"], self.qk), (n["k_conv"], self.qk), (n["v_conv"], self.inner)])),
            ParamSpec("A_log", (nh,), kind="vector", init="normal", sources=_src(n["a_log"], nh)),
            ParamSpec("dt_bias", (nh,), kind="vector", init="normal", sources=_src(n["dt_bias"], nh)),
            ParamSpec("norm", (self.vdim,), kind="vector", init="gain", sources=_src(n["norm"], self.vdim)),
            ParamSpec("o.weight", (H, self.inner), sources=_src(n["o"], H)),
        ]

    def product_weights(self) -> tuple[str, ...]:
        return ("in_proj.weight", "o.weight")

    def state_needs(self) -> tuple[StateNeed, ...]:
        # the convolution's last inputs (at least one row, so that the array exists), the matrices
        return (StateNeed((max(self.taps - 1, 1), self.conv_dim)),
                StateNeed((self.heads, ops.linear_state_rows(self.dim), self.vdim)))

    def forward(self, x, ctx, call, sink=None):
        p, qk, inner, nh = self.params, self.qk, self.inner, self.heads
        conv_state, state = (ctx.states[i] for i in call.state_indices)
        conv_state = conv_state[:, : self.taps - 1]
        batch = self._batch(ctx)
        width = self.conv_dim + inner + 2 * nh
        proj = ctx.buf(f"gdr_proj:{width}", width, torch.float32)
        ops.linear(proj, x, p["in_proj.weight"])
        qkv = ctx.buf(f"gdr_qkv:{self.conv_dim}", self.conv_dim, torch.float32)
        ops.causal_conv(qkv, proj[:, : self.conv_dim], p["conv.weight"], None, conv_state, act="silu",
                        single_tokens=ctx.max_query_len == 1, **batch)
        # q and k in one launch: the q heads come first and take their scale
        ops.unit_heads(qkv[:, :2 * qk], 2 * self.qk_heads, self.dim, self.unit_eps, 1.0,
                       first_heads=self.qk_heads, first_scale=self.q_scale)
        g = ctx.buf(f"gdr_g:{nh}", nh, torch.float32)
        beta = ctx.buf(f"gdr_beta:{nh}", nh, torch.float32)
        at = self.conv_dim + inner
        ops.decay_and_write_gates(g, beta, proj[:, at:at + nh], proj[:, at + nh:], p["A_log"], p["dt_bias"])
        o = ctx.buf(f"ms_o:{inner}", inner, torch.float32)
        ops.linear_state_scan(o, qkv[:, :qk], qkv[:, qk:2 * qk], qkv[:, 2 * qk:], g, beta, state, heads=nh,
                              qk_heads=self.qk_heads, dim=self.dim, vdim=self.vdim, delta_rule=True, **batch)
        return self._finish(o, proj[:, self.conv_dim: self.conv_dim + inner], ctx)


class MaxGatedMatrixMemory(_MatrixStateMixer):
    """The matrix memory of the xLSTM family (mLSTM): per head ``S [dim, vdim]``, a normaliser ``n
    [dim]`` and a running maximum ``m`` of the log gates, which starts at 0:

        i = cap tanh((W_i h + b_i) / cap),   f = logsigmoid(cap tanh((W_f h + b_f) / cap))
        m_t = max(f + m_(t-1), i)
        S_t = exp(f + m_(t-1) - m_t) S_(t-1) + exp(i - m_t) k v^T      (n likewise with k alone)
        o = S_t^T q / (max(|n_t . q|, exp(-m_t)) + den_eps),           q = W_q h * q_scale.

    The normaliser is one more column of the state (the values get a column of ones), so the
    recurrence is the scan of the other matrix-state mixers with two scalar gates a head.  Then
    each head's ``o`` over its root mean square, times a gain of all heads' size, times
    ``sigmoid(W_g h)``, and the output product.  ``tensor_names`` renames checkpoint tensors
    (keys: q, k, v, g, o, norm, i, f, i_bias, f_bias)."""

    def __init__(self, *, hidden_size: int, heads: int, dim: int, vdim: int, gate_cap: float, eps: float,
                 den_eps: float = 1e-6, q_scale: float | None = None, tensor_names: dict[str, str] | None = None,
                 float32_result: bool = False, position=None) -> None:
        if min(heads, dim, vdim) <= 0 or not gate_cap > 0:
            raise ValueError("a matrix memory needs positive sizes and a positive gate cap")
        self.hidden_size, self.heads, self.dim, self.vdim = hidden_size, heads, dim, vdim
        self.cap, self.eps, self.den_eps = float(gate_cap), eps, float(den_eps)
        self.q_scale = dim ** -0.5 if q_scale is None else float(q_scale)
        self.float32_result = float32_result
        self.qk, self.inner = heads * dim, heads * vdim
        self.names = {"q": "q.weight", "k": "k.weight", "v": "v.weight", "g": "g.weight", "o": "o.weight",
                      "norm": "norm.weight", "i": "i.weight", "f": "f.weight", "i_bias": "i.bias", "f_bias": "f.bias",
                      **(tensor_names or {})}

    def param_specs(self) -> list[ParamSpec]:
        n, H, nh = self.names, self.hidden_size, self.heads
        return [
            ParamSpec("in_proj.weight", (2 * self.qk + 2 * self.inner + 2 * nh, H), sources=_stacked(
                [(n["q"], self.qk), (n["k"], self.qk), (n["v"], self.inner), (n["g"], self.inner),
                 (n["i"], nh), (n["f"], nh)])),
            ParamSpec("i.bias", (nh,), kind="vector", init="normal", sources=_src(n["i_bias"], nh)),
            ParamSpec("f.bias", (nh,), kind="vector", init="normal", sources=_src(n["f_bias"], nh)),
            ParamSpec("norm", (self.inner,), kind="vector", init="gain", sources=_src(n["norm"], self.inner)),
            ParamSpec("o.weight", (H, self.inner), sources=_src(n["o"], H)),
        ]

    def product_weights(self) -> tuple[str, ...]:
        return ("in_proj.weight", "o.weight")

    @property
    def takes_slice_sink(self) -> bool:
        return self.inner % 8 == 0

    def state_needs(self) -> tuple[StateNeed, ...]:
        # the matrices with the normaliser as their last column, and the running maxima
        return (StateNeed((self.heads, ops.linear_state_rows(self.dim), self.vdim + 1)), StateNeed((self.heads,)))

    def forward(self, x, ctx, call, sink=None):
        p, qk, inner, nh = self.params, self.qk, self.inner, self.heads
        state, maxima = (ctx.states[i] for i in call.state_indices)
        batch = self._batch(ctx)
        width = 2 * qk + 2 * inner + 2 * nh
        proj = ctx.buf(f"mm_proj:{width}", width, torch.float32)
        ops.linear(proj, x, p["in_proj.weight"])
        keep = ctx.buf(f"mm_keep:{nh}", nh, torch.float32)
        take = ctx.buf(f"mm_take:{nh}", nh, torch.float32)
        m = ctx.buf(f"mm_max:{nh}", nh, torch.float32)
        at = 2 * qk + 2 * inner
        ops.max_gates(keep, take, m, proj[:, at:at + nh], proj[:, at + nh:], p["i.bias"], p["f.bias"], self.cap,
                      maxima, **batch)
        wide = nh * (self.vdim + 1)
        o = ctx.buf(f"mm_o:{wide}", wide, torch.float32)
        ops.linear_state_scan(o, proj[:, :qk], proj[:, qk:2 * qk], proj[:, 2 * qk:2 * qk + inner], keep, take, state,
                              heads=nh, qk_heads=nh, dim=self.dim, vdim=self.vdim + 1, scalar_gates=True,
                              ones_column=True, q_scale=self.q_scale, **batch)
        normed = ctx.buf(f"ms_normed:{inner}", inner)
        ops.max_gated_finish(normed, o, m, proj[:, 2 * qk + inner:2 * qk + 2 * inner], p["norm"], self.eps,
                             self.den_eps, nh, self.vdim)
        if sink is not None:
            return ops.linear(sink, normed, p["o.weight"])
        if self.float32_result:
            out = ctx.buf("mixer_out_f32", self.hidden_size, torch.float32)
        else:
            out = ctx.buf("mixer_out", self.hidden_size)
        ops.linear(out, normed, p["o.weight"])
        return out


register_mixer("gated_linear_attention", GatedLinearAttention)
register_mixer("max_gated_matrix_memory", MaxGatedMatrixMemory)
register_mixer("gated_delta_rule", GatedDeltaRule)
