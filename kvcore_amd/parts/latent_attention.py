"""Attention whose keys and values are made from one small latent vector a token.

Per token the cache keeps ``c`` (``kv_rank`` values, RMS-normed) and one rotated key part of
``rot_dim`` values that all heads share.  Head h's key is ``[W_uk[h] c | k_rot]`` and its value
``W_uv[h] c``; its query ``[q_plain[h] | q_rot[h]]`` comes through a normed latent of its own,
``q = W_uq norm(W_dq x)``.  Because ``q_plain . (W_uk c) = (W_uk^T q_plain) . c``, the scores
are those of attention with ONE key/value head over the rows ``[k_rot | c]`` and queries
``[q_rot | W_uk[h]^T q_plain[h]]``, and the values' product moves behind the softmax: ``out_h =
W_uv[h] sum_j p_j c_j``.  So this part is the paged attention of ``parts/attention.py`` with
one kv head of ``rot_dim + kv_rank`` values (the rotated part first, where the kernels rotate),
reading the same row as key and as value and keeping the last ``kv_rank`` columns of the
result.  The products with ``W_uk`` and ``W_uv`` are folded into their neighbours when the
weights arrive (``W_uk^T W_uq`` per head, ``W_o W_uv`` per head), which costs nothing per token
where the latent is about as wide as a head; a design whose latent is several heads wide would
want them as products per head instead.  A sigmoid gate per head (from the layer's input)
multiplies the head's result before the output product.

Options: ``q_rank`` None: the queries come straight from the layer's input, ``q = W_q x`` (then
``W_uk^T W_q`` per head is what the step multiplies by); ``gated`` False: no gate; ``sinks``: a
learned score per head in the softmax's denominator, as in ``parts/attention.py``; ``rot_dim`` 0:
no rotated part, positions do not enter the scores.
"""

from __future__ import annotations

import torch

from kvcore_amd.ops import library as ops

from .attention import PagedAttention
from .base import ParamSource, ParamSpec, PositionEncoding, register_mixer


class LatentAttention(PagedAttention):
    """``heads`` query heads of ``dim`` plain and ``rot_dim`` rotated elements; values of ``vdim``;
    latents of ``kv_rank`` (keys and values) and ``q_rank`` (queries; None: queries without a
    latent, from the tensor ``q``); ``eps`` of the latents' norms; ``window`` 0 sees every earlier
    token.  ``tensor_names`` renames checkpoint tensors (keys: dq, dq_norm, uq, q, dkv, dkv_norm,
    uk, uv, g, o, sink)."""

    any_head_size = True
    takes_scaled_rows = False  # the input feeds the gate as well
    takes_sink = False

    @property
    def takes_slice_sink(self) -> bool:
        return (self.heads * self.kv_rank) % 8 == 0

    def __init__(self, *, hidden_size: int, heads: int, dim: int, rot_dim: int, vdim: int, kv_rank: int,
                 q_rank: int | None, scale: float, eps: float, window: int = 0, page_size: int | None = None,
                 gated: bool = True, sinks: bool = False, tensor_names: dict[str, str] | None = None,
                 float32_result: bool = False, position: PositionEncoding | None = None) -> None:
        if min(heads, dim, vdim, kv_rank, 1 if q_rank is None else q_rank) <= 0 or rot_dim < 0 or rot_dim % 2:
            raise ValueError("latent attention needs positive sizes and an even rotated width")
        width = rot_dim + kv_rank
        if width > 512:
            raise ValueError(f"a latent of {kv_rank} with {rot_dim} rotated elements: the attention kernels "
                             f"serve rows of up to 512 values")
        super().__init__(hidden_size=hidden_size, num_heads=heads, num_kv_heads=1, head_dim=width, scale=scale,
                         window=window, page_size=page_size, float32_result=float32_result, sinks=sinks,
                         position=position)
        self.heads, self.dim, self.rot, self.vdim = heads, dim, rot_dim, vdim
        self.kv_rank, self.q_rank, self.eps, self.gated = kv_rank, q_rank, eps, bool(gated)
        self.row = width
        self.q_latent = q_rank is not None
        self.q_off = q_rank if self.q_latent else 0  # where the key/value latent starts in a row of `down`
        self.down_width = self.q_off + kv_rank + rot_dim + (heads if gated else 0)
        self.latent_names = {"dq": "dq.weight", "dq_norm": "dq_norm.weight", "uq": "uq.weight", "q": "q.weight",
                             "sink": "sinks", "dkv": "dkv.weight",
                             "dkv_norm": "dkv_norm.weight", "uk": "uk.weight", "uv": "uv.weight", "g": "g.weight",
                             "o": "o.weight", **(tensor_names or {})}

    def param_specs(self) -> list[ParamSpec]:
        n, H, nh = self.latent_names, self.hidden_size, self.heads
        down = [ParamSource(n["dkv"], self.q_off, self.kv_rank + self.rot)]
        if self.q_latent:
            down.insert(0, ParamSource(n["dq"], 0, self.q_rank))
        if self.gated:
            down.append(ParamSource(n["g"], self.q_off + self.kv_rank + self.rot, nh))

        def src(name: str, rows: int) -> tuple[ParamSource, ...]:
            return (ParamSource(n[name], 0, rows),)

        q_rows = nh * (self.dim + self.rot)
        if self.q_latent:
            queries = [ParamSpec("dq_norm", (self.q_rank,), kind="vector", init="gain", sources=src("dq_norm", self.q_rank)),
                       ParamSpec("uq.weight", (q_rows, self.q_rank), sources=src("uq", q_rows))]
        else:
            queries = [ParamSpec("uq.weight", (q_rows, H), sources=src("q", q_rows))]
        specs = [
            ParamSpec("down.weight", (self.down_width, H), sources=tuple(down)),
            *queries,
            ParamSpec("dkv_norm", (self.kv_rank,), kind="vector", init="gain", sources=src("dkv_norm", self.kv_rank)),
            ParamSpec("uk.weight", (nh * self.dim, self.kv_rank), sources=src("uk", nh * self.dim)),
            ParamSpec("uv.weight", (nh * self.vdim, self.kv_rank), sources=src("uv", nh * self.vdim)),
            ParamSpec("o.weight", (H, nh * self.vdim), sources=src("o", H)),
        ]
        if self.has_sinks:
            specs.append(ParamSpec("sinks", (nh,), kind="vector", init="normal", sources=src("sink", nh)))
        return specs

    def product_weights(self) -> tuple[str, ...]:
        return ("down.weight", "q_latent.weight", "o_latent.weight")

    def weights_loaded(self) -> None:
        """The two matrices that the steps multiply by, from the checkpoint's four: per head
        ``[W_uq rotated rows ; W_uk^T W_uq plain rows]`` (queries straight into the cache's
        layout) and ``W_o[:, head] W_uv[head]`` (the output product from the latent)."""
        p, nh, d, r, rank = self.params, self.heads, self.dim, self.rot, self.kv_rank
        f = torch.float32
        uq = p["uq.weight"].to(f).view(nh, d + r, -1)  # from the query latent, or from the layer's input
        uk = p["uk.weight"].to(f).view(nh, d, rank)
        uv = p["uv.weight"].to(f).view(nh, self.vdim, rank)
        wo = p["o.weight"].to(f).view(self.hidden_size, nh, self.vdim)
        plain = torch.matmul(uk.transpose(1, 2), uq[:, :d])           # [heads, rank, q_rank]
        q_latent = torch.cat([uq[:, d:], plain], dim=1).reshape(nh * self.row, uq.shape[2])
        o_latent = torch.einsum("xhv,hvr->xhr", wo, uv).reshape(self.hidden_size, nh * rank)
        for name, value in (("q_latent.weight", q_latent), ("o_latent.weight", o_latent)):
            old = p.get(name)
            if old is None:
                p[name] = value.to(self.runtime.dtype).contiguous()
            else:  # weights loaded again: the same storage, so nothing that holds it goes stale
                old.copy_(value)
                if hasattr(old, "kvc_packed"):
                    del old.kvc_packed

    def _project(self, x, ctx):
        p, nh, row, rank, rot = self.params, self.heads, self.row, self.kv_rank, self.rot
        if "q_latent.weight" not in p:
            self.weights_loaded()
        down = ctx.buf(f"latent_down:{self.down_width}", self.down_width)
        ops.linear(down, x, p["down.weight"])
        cq = ctx.buf(f"latent_cq:{self.q_rank}", self.q_rank) if self.q_latent else None
        qkv = ctx.buf(f"latent_qkv:{(nh + 2) * row}", (nh + 2) * row)
        # both latents' norms and the one key/value row a token (the rotated part as projected,
        # then the normed latent; the same values in the key's place and in the value's)
        ops.latent_rows(cq, qkv[:, nh * row: (nh + 1) * row], qkv[:, (nh + 1) * row:], down, p.get("dq_norm"),
                        p["dkv_norm"], self.eps, rot)
        ops.linear(qkv[:, : nh * row], cq if self.q_latent else x, p["q_latent.weight"])
        ctx.scratch[("latent_down", id(self))] = down
        return qkv

    def _output(self, attn, ctx, sink=None):
        p, nh, rank = self.params, self.heads, self.kv_rank
        down = ctx.scratch[("latent_down", id(self))]
        if self.gated:
            kept = ctx.buf(f"latent_out:{nh * rank}", nh * rank)
            ops.head_gate(kept, attn, down[:, self.down_width - nh:], heads=nh, head_stride=self.row,
                          skip=self.rot, n=rank)
        elif self.rot:
            kept = ctx.buf(f"latent_out:{nh * rank}", nh * rank)
            kept.view(-1, nh, rank).copy_(attn.view(-1, nh, self.row)[:, :, self.rot:])
        else:
            kept = attn
        if sink is not None:
            return ops.linear(sink, kept, p["o_latent.weight"])
        if self.float32_result:
            out = ctx.buf("mixer_out_f32", self.hidden_size, torch.float32)
        else:
            out = ctx.buf("mixer_out", self.hidden_size)
        ops.linear(out, kept, p["o_latent.weight"])
        return out


register_mixer("latent_attention", LatentAttention)
