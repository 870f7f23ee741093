"""Gated feed-forward: ``down(act(gate(x)) * up(x))`` with gate and up stacked; ``act`` is silu
unless the layer names another (``gelu_tanh``).

Reference: kvcore/model/models/llama3.py:25-45 (gate rows first, then up rows) and
kvcore/model/layer/activation.py:14-16.
"""

from __future__ import annotations

import torch

from kvcore_amd.ops import library as ops

from .base import FeedForward, ParamSource, ParamSpec, register_feed_forward


class SwiGLU(FeedForward):
    @property
    def takes_scaled_rows(self) -> bool:  # x only goes into the gate-up product
        return self.hidden_size % 8 == 0

    @property
    def takes_sink(self) -> bool:
        return self.intermediate_size % 8 == 0 and not self.float32_result

    @property
    def takes_slice_sink(self) -> bool:  # float32 partial sums whatever the result's type
        return self.intermediate_size % 8 == 0

    def __init__(self, *, hidden_size: int, intermediate_size: int, bias: bool = False,
                 gate_name: str = "gate_proj", up_name: str = "up_proj", down_name: str = "down_proj",
                 suffix: str = ".weight", sized_buffers: bool = False, activation: str = "silu",
                 float32_result: bool = False) -> None:
        """``gate_name``, ``up_name`` and ``down_name`` are the checkpoint's names of the three
        matrices relative to the part's prefix, ``suffix`` what follows each (biases end in
        ``.bias``).  ``sized_buffers``: name the step buffers by their width, for a model whose
        layers may differ in width (a buffer whose width changed from layer to layer would be
        allocated anew at every layer).  ``activation``: the gate's, ``silu`` or ``gelu_tanh``.
        ``float32_result``: the output rows are float32 sums, for a consumer that normalises them."""
        if activation not in ops.GATE_ACTS:
            raise ValueError(f"gate activation {activation!r} is not supported (supported: {sorted(ops.GATE_ACTS)})")
        self.activation = activation
        self.float32_result = float32_result
        self.hidden_size = hidden_size
        self.intermediate_size = intermediate_size
        self.bias = bias
        self.names = (gate_name, up_name, down_name)
        self.suffix = suffix
        self.sized_buffers = sized_buffers

    def param_specs(self) -> list[ParamSpec]:
        I, H = self.intermediate_size, self.hidden_size

        gate, up, down = self.names

        def stacked(suffix: str) -> tuple[ParamSource, ...]:
            return (ParamSource(gate + suffix, 0, I), ParamSource(up + suffix, I, I))

        specs = [
            ParamSpec("gate_up_proj.weight", (2 * I, H), sources=stacked(self.suffix)),
            ParamSpec("down_proj.weight", (H, I), sources=(ParamSource(down + self.suffix, 0, H),)),
        ]
        if self.bias:
            specs.append(ParamSpec("gate_up_proj.bias", (2 * I,), init="zeros", sources=stacked(".bias")))
            specs.append(ParamSpec("down_proj.bias", (H,), init="zeros",
                                   sources=(ParamSource(down + ".bias", 0, H),)))
        return specs

    def product_weights(self) -> tuple[str, ...]:
        return ("gate_up_proj.weight", "down_proj.weight")

    def _buf(self, name: str) -> str:
        return f"{name}:{self.intermediate_size}" if self.sized_buffers else name

    def forward(self, x, ctx, call, sink=None):
        p = self.params
        act = ctx.buf(self._buf("ffn_act"), self.intermediate_size)
        # few rows: the product and the activation are one kernel and gate_up is never stored
        ops.linear_silu_mul(act, x, p["gate_up_proj.weight"], p.get("gate_up_proj.bias"),
                            lambda: ctx.buf(self._buf("ffn_gate_up"), 2 * self.intermediate_size),
                            act=self.activation)
        if sink is not None:
            return ops.linear(sink, act, p["down_proj.weight"], p.get("down_proj.bias"))
        if self.float32_result:
            out = ctx.buf("ffn_out_f32", self.hidden_size, torch.float32)
        else:
            out = ctx.buf("ffn_out", self.hidden_size)
        ops.linear(out, act, p["down_proj.weight"], p.get("down_proj.bias"))
        return out


class DenseMLP(FeedForward):
    """A feed-forward without a gate: ``down(act(up(x) + b_up)) + b_down``; ``activation`` is one of
    ``ops.ACTIVATIONS`` (``relu_squared``: the square of relu), computed in float32 from the rows
    as stored.  ``up_name``/``down_name`` are the checkpoint's names of the two matrices relative to
    the part's prefix, ``suffix`` what follows each, ``bias_suffix`` what follows a bias."""

    @property
    def takes_slice_sink(self) -> bool:  # float32 partial sums whatever the result's type
        return self.intermediate_size % 8 == 0

    def __init__(self, *, hidden_size: int, intermediate_size: int, activation: str = "relu_squared",
                 bias: bool = False, up_name: str = "up_proj", down_name: str = "down_proj",
                 suffix: str = ".weight", bias_suffix: str = ".bias", float32_result: bool = False) -> None:
        if activation not in ops.ACTIVATIONS:
            raise ValueError(f"activation {activation!r} is not supported (supported: {sorted(ops.ACTIVATIONS)})")
        self.hidden_size, self.intermediate_size = hidden_size, intermediate_size
        self.activation, self.bias, self.float32_result = activation, bool(bias), float32_result
        self.names, self.suffix, self.bias_suffix = (up_name, down_name), suffix, bias_suffix

    def param_specs(self) -> list[ParamSpec]:
        I, H = self.intermediate_size, self.hidden_size
        up, down = self.names
        specs = [ParamSpec("up_proj.weight", (I, H), sources=(ParamSource(up + self.suffix, 0, I),)),
                 ParamSpec("down_proj.weight", (H, I), sources=(ParamSource(down + self.suffix, 0, H),))]
        if self.bias:
            # in the model's dtype, as the products' kernels take them
            specs.append(ParamSpec("up_proj.bias", (I,), init="normal",
                                   sources=(ParamSource(up + self.bias_suffix, 0, I),)))
            specs.append(ParamSpec("down_proj.bias", (H,), init="normal",
                                   sources=(ParamSource(down + self.bias_suffix, 0, H),)))
        return specs

    def product_weights(self) -> tuple[str, ...]:
        return ("up_proj.weight", "down_proj.weight")

    def forward(self, x, ctx, call, sink=None):
        p, I = self.params, self.intermediate_size
        act = ctx.buf(f"mlp_act:{I}", I)
        # few rows: the product and the activation are one kernel
        ops.linear_act(act, x, p["up_proj.weight"], p.get("up_proj.bias"), self.activation)
        if sink is not None:
            return ops.linear(sink, act, p["down_proj.weight"], p.get("down_proj.bias"))
        if self.float32_result:
            out = ctx.buf("ffn_out_f32", self.hidden_size, torch.float32)
        else:
            out = ctx.buf("ffn_out", self.hidden_size)
        ops.linear(out, act, p["down_proj.weight"], p.get("down_proj.bias"))
        return out


class NoFeedForward(FeedForward):
    """A layer that has a mixer only: the block skips the second norm and the second sum."""

    absent = True

    def forward(self, x, ctx, call, sink=None):
        raise RuntimeError("a layer without a feed-forward has nothing to run here")


register_feed_forward("swiglu", SwiGLU)
register_feed_forward("mlp", DenseMLP)
register_feed_forward("none", NoFeedForward)
