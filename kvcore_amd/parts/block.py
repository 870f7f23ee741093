"""Arrangements of norms, mixer and feed-forward around the residual stream.

Reference: kvcore/model/models/llama3.py:124-142.  The reference carries
``(hidden, residual)`` and lets each norm add the pending ``hidden`` first; this is
the same arrangement with the pending output called ``delta`` and the stream kept in
float32.
"""

from __future__ import annotations

import torch

from kvcore_amd.ops import library as ops

from .base import Block, FeedForward, Mixer, Norm, ParamSource, ParamSpec, Part, register_block


class PreNormBlock(Block):
    """``r += delta; a = mixer(norm_in(r)); r += a; out = ffn(norm_post(r))``, the last
    sum left pending for the next block's first norm.  With a feed-forward of kind ``none`` the
    block is ``r += delta; out = mixer(norm_in(r))``."""

    def __init__(self, *, mixer: Mixer, ffn: FeedForward, norms: dict[str, Norm],
                 mixer_name: str = "self_attn", ffn_name: str = "mlp",
                 input_norm: str | None = None, post_norm: str | None = None) -> None:
        """``input_norm`` and ``post_norm`` name the norm before the mixer and the norm before
        the feed-forward among ``norms`` (they are also the norms' checkpoint sub-prefixes);
        left out, they are the first and the second norm that the layer lists."""
        super().__init__(mixer=mixer, ffn=ffn, norms=norms)
        listed = list(norms)
        self.mixer_only = bool(getattr(ffn, "absent", False))
        if input_norm is None and listed:
            input_norm = listed[0]
        if post_norm is None:
            post_norm = next((n for n in listed if n != input_norm), None)
        if self.mixer_only:
            post_norm = None
            if input_norm not in norms:
                raise ValueError(f"a pre-norm block needs a norm before the mixer; given {listed}")
        missing = [n for n in (input_norm, post_norm) if n not in norms and not self.mixer_only]
        if missing or input_norm == post_norm:
            raise ValueError(f"a pre-norm block needs two norms, one before the mixer and one before the "
                             f"feed-forward; asked for {(input_norm, post_norm)}, given {listed}")
        self.norm_names = (input_norm, post_norm)
        self.mixer_name = mixer_name
        self.ffn_name = ffn_name

    def children(self) -> dict[str, Part]:
        if self.mixer_only:
            return {self.norm_names[0]: self.norms[self.norm_names[0]], self.mixer_name: self.mixer}
        return {
            self.norm_names[0]: self.norms[self.norm_names[0]],
            self.mixer_name: self.mixer,
            self.norm_names[1]: self.norms[self.norm_names[1]],
            self.ffn_name: self.ffn,
        }

    def input_gain(self, scaled: bool = True):
        """The first norm as (gain, eps) if the block before may do its work: leaving scaled
        rows for this block's mixer to finish (``scaled``), or finishing it itself."""
        gain = self.norms[self.norm_names[0]].as_gain()
        if scaled and not self.mixer.takes_scaled_rows:
            return None
        return gain

    def forward(self, delta, residual: torch.Tensor, ctx, call, next_block=None):
        # With very few rows of bfloat16 the norms fold into the products around them: the product
        # before a norm adds into the residual and keeps the sums of squares, the product after
        # it applies the scale factor.  Otherwise every norm is a kernel of its own.
        # With a few dozen rows the product before a norm leaves partial sums of slices along
        # K, and one kernel adds them into the residual and normalises.
        fold, sums = self.norm_folding(ctx, residual.shape[1])
        if isinstance(delta, ops.ScaledRows):
            x = delta  # the block before made the first norm's rows
        elif isinstance(delta, ops.NormedRows):
            x = delta.data  # the block before did the first norm
        else:
            x = ctx.buf("block_x", residual.shape[1])
            self.norms[self.norm_names[0]].forward_fused(x, residual, delta)

        if self.mixer_only:  # x + mixer(norm(x)) and nothing more; the sum stays pending
            return self.mixer.forward(x, ctx, call)
        post = self.norms[self.norm_names[1]]
        gain = None
        if self.mixer.takes_sink and ((fold and self.ffn.takes_scaled_rows) or sums):
            gain = post.as_gain()
        if gain is not None:
            x2 = self.mixer.forward(x, ctx, call, sink=self.residual_sink(ctx, residual, gain, "block_x2", fold))
            if isinstance(x2, ops.NormedRows):
                x2 = x2.data
        else:
            a = self.mixer.forward(x, ctx, call)
            x2 = ctx.buf("block_x2", residual.shape[1])
            post.forward_fused(x2, residual, a)

        gain = None
        if next_block is not None and self.ffn.takes_sink and (fold or sums):
            gain = next_block.input_gain(scaled=fold)
        if gain is not None:
            return self.ffn.forward(x2, ctx, call, sink=self.residual_sink(ctx, residual, gain, "block_x", fold))
        return self.ffn.forward(x2, ctx, call)


class ParallelResidualBlock(Block):
    """``r += delta; h = norm(r); r += mixer(h) + ffn(h)``: one norm a layer, both branches read
    its output, and both sums go straight into the float32 stream (nothing stays pending, so the
    branches may hand over float32 rows).  With a feed-forward of kind ``none`` the mixer is
    the layer."""

    def __init__(self, *, mixer: Mixer, ffn: FeedForward, norms: dict[str, Norm],
                 mixer_name: str = "mixer", ffn_name: str = "mlp", norm: str | None = None) -> None:
        super().__init__(mixer=mixer, ffn=ffn, norms=norms)
        self.norm_name = norm if norm is not None else next(iter(norms), None)
        if self.norm_name not in norms:
            raise ValueError(f"a parallel block needs its one norm; asked for {norm!r}, given {list(norms)}")
        self.mixer_only = bool(getattr(ffn, "absent", False))
        self.mixer_name, self.ffn_name = mixer_name, ffn_name

    def children(self) -> dict[str, Part]:
        out = {self.norm_name: self.norms[self.norm_name], self.mixer_name: self.mixer}
        if not self.mixer_only:
            out[self.ffn_name] = self.ffn
        return out

    def forward(self, delta, residual: torch.Tensor, ctx, call, next_block=None):
        if isinstance(delta, (ops.ScaledRows, ops.NormedRows)):
            raise RuntimeError("a parallel block takes its input from the stream, not from folded norms")
        x = ctx.buf("block_x", residual.shape[1])
        self.norms[self.norm_name].forward_fused(x, residual, delta)
        a = self.mixer.forward(x, ctx, call)
        if self.mixer_only:
            ops.residual_add(residual, a)
        elif a.dtype == torch.float32 and hasattr(self.ffn, "forward_into"):
            # a feed-forward whose last kernel can add into the stream takes the mixer's rows along
            self.ffn.forward_into(residual, x, ctx, call, add=a)
        else:
            f = self.ffn.forward(x, ctx, call)
            ops.residual_add2(residual, a, f)
        return None


class SandwichNormBlock(Block):
    """A norm before and a norm behind each sublayer: ``r += post_mixer(mixer(pre_mixer(r)));
    r += post_ffn(ffn(pre_ffn(r)))``, all four RMS norms with a gain.  Between two sublayers the
    norm of the result, the sum into the float32 stream and the next sublayer's first norm are one
    kernel (``ops.norm_add_norm``); so the block hands the next block its first norm's rows where
    that block says it takes them (``input_gain``), and takes its own from the block before.  With
    a feed-forward of kind ``none`` the layer is its first half."""

    def __init__(self, *, mixer: Mixer, ffn: FeedForward, norms: dict[str, Norm],
                 mixer_name: str = "mixer", ffn_name: str = "mlp", pre_mixer: str = "norm1",
                 post_mixer: str = "norm1b", pre_ffn: str = "norm2", post_ffn: str = "norm2b") -> None:
        super().__init__(mixer=mixer, ffn=ffn, norms=norms)
        self.mixer_only = bool(getattr(ffn, "absent", False))
        self.mixer_name, self.ffn_name = mixer_name, ffn_name
        self.norm_names = (pre_mixer, post_mixer) if self.mixer_only else (pre_mixer, post_mixer, pre_ffn, post_ffn)
        missing = [n for n in self.norm_names if n not in norms]
        if missing or len(set(self.norm_names)) != len(self.norm_names):
            raise ValueError(f"a block with norms on both sides of its sublayers needs {self.norm_names}; "
                             f"given {list(norms)}")

    def children(self) -> dict[str, Part]:
        out: dict[str, Part] = {n: self.norms[n] for n in self.norm_names}
        out[self.mixer_name] = self.mixer
        if not self.mixer_only:
            out[self.ffn_name] = self.ffn
        return out

    def input_gain(self, scaled: bool = True):
        # finished rows are welcome; rows whose norm the mixer's first product would have to
        # finish are not (the mixers of such layers read their input more than once)
        return None if scaled else self.norms[self.norm_names[0]].as_gain()

    def _gain(self, i: int):
        gain = self.norms[self.norm_names[i]].as_gain()
        if gain is None:
            raise RuntimeError(f"norm {self.norm_names[i]!r} is not an RMS norm with a gain")
        return gain

    def _join(self, result, residual, ctx, post, following, name: str):
        """``residual += post(result)``, and the rows of the norm ``following`` (a (gain, eps) or
        None) into the step buffer ``name``.  ``result`` is a tensor or the partial sums that a
        part's last product left (``ops.SlicedRows``)."""
        post_gain, post_eps = post
        if following is None:
            ops.norm_add_norm(None, residual, result, post_gain, post_eps)
            return None
        rows = ctx.buf(name, residual.shape[1])
        ops.norm_add_norm(rows, residual, result, post_gain, post_eps, following[0], following[1])
        return rows

    def _slice_sink(self, part, residual, ctx):
        """In a step of a few dozen rows a part's last product may leave partial sums of slices
        along K, which the norm behind it adds up on its way: the ``ops.SliceSink`` for that, or
        None where the step or the part does not take one."""
        H = residual.shape[1]
        if not (getattr(part, "takes_slice_sink", False) and H % 8 == 0
                and ops.rows_sinkable(ctx.num_tokens, ctx.dtype)):
            return None
        return ops.SliceSink(ctx.buffers.get("block_slices", ops.mid_slices_bound(H) * ops.MID_ROWS, H, torch.float32))

    def forward(self, delta, residual: torch.Tensor, ctx, call, next_block=None):
        if isinstance(delta, ops.ScaledRows):
            raise RuntimeError("this block takes finished rows or the stream, not rows still to be scaled")
        if isinstance(delta, ops.NormedRows):
            x = delta.data  # the block before made this block's first norm
        else:
            x = ctx.buf("block_x", residual.shape[1])
            self.norms[self.norm_names[0]].forward_fused(x, residual, delta)
        following = next_block.input_gain(scaled=False) if next_block is not None else None
        sink = self._slice_sink(self.mixer, residual, ctx)
        a = self.mixer.forward(x, ctx, call) if sink is None else self.mixer.forward(x, ctx, call, sink=sink)
        if self.mixer_only:
            rows = self._join(a, residual, ctx, self._gain(1), following, "block_x")
            return None if rows is None else ops.NormedRows(rows)
        x2 = self._join(a, residual, ctx, self._gain(1), self._gain(2), "block_x2")
        sink = self._slice_sink(self.ffn, residual, ctx)
        f = self.ffn.forward(x2, ctx, call) if sink is None else self.ffn.forward(x2, ctx, call, sink=sink)
        rows = self._join(f, residual, ctx, self._gain(3), following, "block_x")
        return None if rows is None else ops.NormedRows(rows)


class StreamLink(Part):
    """How one sublayer hangs on a residual stream of several copies: ``in [copies]`` weighs the
    copies into the sublayer's input, ``mix [copies, copies]`` (indexed [from, to]) carries the old
    copies into the new ones, ``out [copies]`` weighs the sublayer's result into each.  All float32."""

    def __init__(self, copies: int, names: tuple[str, str, str] = ("in", "mix", "out")) -> None:
        self.copies, self.names = copies, names

    def param_specs(self) -> list[ParamSpec]:
        c, (n_in, n_mix, n_out) = self.copies, self.names
        return [ParamSpec("in", (c,), kind="vector", init="gain", sources=(ParamSource(n_in, 0, c),)),
                ParamSpec("mix", (c, c), kind="vector", init="mixing", sources=(ParamSource(n_mix, 0, c),)),
                ParamSpec("out", (c,), kind="vector", init="gain", sources=(ParamSource(n_out, 0, c),))]


class HyperConnectionBlock(Block):
    """A pre-norm layer on a residual stream kept as ``copies`` rows a token, ``x_1 .. x_c``.  For
    each sublayer f (mixer, then feed-forward) with its link (in, mix, out) and its norm:

        u = sum_s in[s] x_s;   y = f(norm(u));   x_t <- sum_s mix[s, t] x_s + mult * out[t] * y

    for all t at once from the old copies.  ``learned`` False: no link tensors, in = out = 1 and mix
    the identity, which with one copy is the plain ``x <- x + mult * f(norm(x))``.  The write of one
    sublayer and the read and norm of the next are one kernel (``ops.hyper_step``), across blocks
    too: a block returns its last sublayer's result as a pending ``ops.StreamWrite``.  After the
    last block the copies are added up and normed by the model's final norm.  The norms must be RMS
    norms with a gain (``Norm.as_gain``).  With a feed-forward of kind ``none`` the layer is its
    first half."""

    def __init__(self, *, mixer: Mixer, ffn: FeedForward, norms: dict[str, Norm], copies: int = 1,
                 learned: bool = True, mult: float = 1.0, mixer_name: str = "mixer", ffn_name: str = "mlp",
                 mixer_norm: str = "norm1", ffn_norm: str = "norm2", mixer_link: str = "hc1",
                 ffn_link: str = "hc2") -> None:
        super().__init__(mixer=mixer, ffn=ffn, norms=norms)
        if not 1 <= copies <= ops.HYPER_MAX_COPIES:
            raise ValueError(f"a stream of {copies} copies (1 to {ops.HYPER_MAX_COPIES})")
        self.stream_copies, self.learned, self.mult = int(copies), bool(learned), float(mult)
        self.mixer_only = bool(getattr(ffn, "absent", False))
        self.mixer_name, self.ffn_name = mixer_name, ffn_name
        self.norm_names = (mixer_norm,) if self.mixer_only else (mixer_norm, ffn_norm)
        missing = [n for n in self.norm_names if n not in norms]
        if missing:
            raise ValueError(f"this block needs the norms {self.norm_names}; given {list(norms)}")
        self.link_names = (mixer_link, ffn_link)
        self.links = [StreamLink(self.stream_copies) for _ in self.norm_names] if self.learned else []

    def children(self) -> dict[str, Part]:
        out: dict[str, Part] = {self.norm_names[0]: self.norms[self.norm_names[0]], self.mixer_name: self.mixer}
        if not self.mixer_only:
            out[self.norm_names[1]] = self.norms[self.norm_names[1]]
            out[self.ffn_name] = self.ffn
        for name, link in zip(self.link_names, self.links):
            out[name] = link
        return out

    def _gain(self, i: int):
        gain = self.norms[self.norm_names[i]].as_gain()
        if gain is None:
            raise RuntimeError(f"norm {self.norm_names[i]!r} is not an RMS norm with a gain")
        return gain

    def _written(self, y, i: int) -> "ops.StreamWrite":
        """Sublayer i's result on its way into the copies."""
        link = self.links[i].params if self.learned else {}
        return ops.StreamWrite(y, self.stream_copies, link.get("mix"), link.get("out"), self.mult)

    def _read(self, name: str, residual, ctx, pending, i: int):
        """What is pending joins the copies; sublayer i's input, normed, into the step buffer ``name``."""
        rows = ctx.buf(name, residual.shape[1] // self.stream_copies)
        gain, eps = self._gain(i)
        in_w = self.links[i].params["in"] if self.learned else None
        ops.stream_write_read(rows, residual, self.stream_copies, pending, in_w=in_w, gain=gain, eps=eps)
        return rows

    def _slice_sink(self, part, width: int, ctx):
        """In a step of a few dozen rows a part's last product may leave partial sums of slices
        along K, which the kernel that carries the result into the copies adds up on its way:
        the ``ops.SliceSink`` for that, or None where the step or the part does not take one.
        One room serves both sublayers: a result is read before the next product is launched."""
        if not (getattr(part, "takes_slice_sink", False) and width % 8 == 0
                and ops.rows_sinkable(ctx.num_tokens, ctx.dtype)):
            return None
        return ops.SliceSink(ctx.buffers.get("block_slices", ops.mid_slices_bound(width) * ops.MID_ROWS, width,
                                             torch.float32), takes_bias=True)

    def forward(self, delta, residual: torch.Tensor, ctx, call, next_block=None):
        if delta is not None and not isinstance(delta, ops.StreamWrite):
            raise RuntimeError("this block follows blocks of its own kind")
        width = residual.shape[1] // self.stream_copies
        x = self._read("block_x", residual, ctx, delta, 0)
        sink = self._slice_sink(self.mixer, width, ctx)
        a = self.mixer.forward(x, ctx, call) if sink is None else self.mixer.forward(x, ctx, call, sink=sink)
        if self.mixer_only:
            return self._written(a, 0)
        x2 = self._read("block_x2", residual, ctx, self._written(a, 0), 1)
        sink = self._slice_sink(self.ffn, width, ctx)
        f = self.ffn.forward(x2, ctx, call) if sink is None else self.ffn.forward(x2, ctx, call, sink=sink)
        return self._written(f, 1)

    def settle(self, delta, residual: torch.Tensor, ctx) -> None:
        if delta is not None:
            ops.stream_write_read(None, residual, self.stream_copies, delta)

    def finish(self, delta, residual: torch.Tensor, ctx, final_norm: Norm, hidden: torch.Tensor) -> None:
        gain = final_norm.as_gain()
        if gain is None:
            raise RuntimeError("the final norm of a stream of several copies is an RMS norm with a gain")
        ops.stream_write_read(hidden, residual, self.stream_copies, delta, in_w=None, gain=gain[0], eps=gain[1])


register_block("prenorm", PreNormBlock)
register_block("hyper_connections", HyperConnectionBlock)
register_block("sandwich_norm", SandwichNormBlock)
register_block("parallel_residual", ParallelResidualBlock)
