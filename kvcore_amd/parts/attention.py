"""Grouped-query attention over the paged cache.

Reference: kvcore/model/models/llama3.py:48-104 (stacked qkv projection with rows in
the order q, k, v; rotation of q and k; attention; output projection) and
kvcore/model/attn_backend/torch_paged.py:70-117 (keys and values are written to their
page slots first, then every query reads keys ``0..position`` back from the cache).
"""

from __future__ import annotations

import torch

from kvcore_amd.ops import library as ops

from .base import CacheNeed, Mixer, ParamSource, ParamSpec, PositionEncoding, register_mixer


DECODE_MAX_SPLITS = 32


def decode_target_blocks() -> int:
    """Blocks a launch of the decode kernel wants: one for each compute unit."""
    return ops.compute_units()


def prefill_target_blocks() -> int:
    """Blocks a launch of the kernel for portions wants: a compute unit holds two."""
    return 2 * ops.compute_units()


def prefill_split_rows(nkv: int, g: int) -> int:
    """An upper bound on tokens x splits when ``prefill_splits`` gives more than one split."""
    rows_tokens = max(128 // g, 1)
    return 4 * prefill_target_blocks() * rows_tokens // nkv + 2 * rows_tokens


def prefill_few_tiles() -> int:
    """Up to so many small tiles (half the compute units), splits go with small tiles."""
    return ops.compute_units() // 2


PREFILL_MIN_KEYS = 256      # for steps of few tokens, whose partial results are small
PREFILL_MIN_KEYS_MOST = 1024
PREFILL_MAX_SPLITS = 32


def prefill_splits(T: int, nkv: int, g: int, max_query_len: int, max_seq_len: int, window: int,
                   num_reqs: int = 1) -> int:
    """How many blocks share the keys of one tile of query rows in the kernel for portions
    of prompts.  A compute unit holds two of its blocks, so a launch wants some 512.  The
    kernel has tiles of 64 rows (one or two a block) and of 128 (two a block, cheaper per
    key); with splits it takes the small tiles one a block for very few rows and the large
    ones otherwise (`launch_prefill` in csrc/attention_prefill.hip, which must agree with
    this on where "very few" ends).  Measured on the 8B shape: splits pay when the rows are
    few and every block still has a few hundred keys to walk, a thousand for steps of a
    thousand tokens (a row sees ``max_seq_len`` keys at most and, under the causal mask,
    about half a portion fewer on average).  Every request but one may add a ragged tile."""
    small_tokens = max(64 // g, 1)
    small_tiles = (-(-T // small_tokens) + num_reqs - 1) * nkv  # blocks of one small tile each
    keys = max_seq_len - min(T, max_query_len) // 2
    if window > 0:
        keys = min(keys, window + 2 * small_tokens)
    target = prefill_target_blocks()
    if small_tiles <= prefill_few_tiles():
        return max(1, min(-(-target // small_tiles), keys // PREFILL_MIN_KEYS, PREFILL_MAX_SPLITS))
    if small_tiles <= target:
        if small_tiles == target:
            return 1  # one small tile a block fills the chip as it is
        min_keys = min(max(T, PREFILL_MIN_KEYS), PREFILL_MIN_KEYS_MOST)
    else:
        min_keys = min(max(T // 2, PREFILL_MIN_KEYS), PREFILL_MIN_KEYS_MOST)
    rows_tokens = max(128 // g, 1)
    blocks = ((-(-T // rows_tokens)) + num_reqs) // 2 * nkv
    if blocks >= target:
        return 1
    return max(1, min(-(-target // blocks), keys // min_keys, PREFILL_MAX_SPLITS))


def decode_splits(num_tokens: int, num_kv_heads: int, max_seq_len: int, waves: int,
                  window: int = 0) -> int:
    """Into how many parts each request's key range is cut for the decode kernel, beyond the
    ``waves`` waves of a block that share a part.  One compute unit draws keys and values
    from memory far slower than the chip can deliver them, so the parts are made many
    enough to occupy every unit, as long as each wave still has a block of 16 keys."""
    keys = max_seq_len if window <= 0 else min(max_seq_len, window + 16)
    blocks = -(-keys // 16)
    by_room = -(-decode_target_blocks() // max(num_tokens * num_kv_heads, 1))
    by_length = max(1, blocks // waves)
    return max(1, min(by_room, by_length, DECODE_MAX_SPLITS))


class PagedAttention(Mixer):
    """``scale`` is a parameter (the reference fixes ``head_dim ** -0.5`` at
    llama3.py:60); ``window`` 0 attends to every earlier token; ``page_size`` asks for cache
    pages of that many tokens for this layer's group (None: the engine's block size)."""

    any_head_size = False  # a subclass whose heads need not be a multiple of 16 takes the general kernels then
    # a subclass that joins the heads' results before anything is rounded asks the attention kernels
    # for their float32 sums instead of results in the model's dtype
    float32_heads = False

    @property
    def takes_scaled_rows(self) -> bool:  # x only goes into the qkv product
        return self.hidden_size % 8 == 0

    @property
    def takes_sink(self) -> bool:  # the output product's rows are whole heads
        return self.o_size % 8 == 0 and not self.float32_result

    @property
    def takes_slice_sink(self) -> bool:  # float32 partial sums whatever the result's type
        return self.o_size % 8 == 0

    def __init__(self, *, hidden_size: int, num_heads: int, num_kv_heads: int, head_dim: int,
                 scale: float, bias: bool = False, window: int = 0, page_size: int | None = None,
                 v_head_dim: int | None = None, qk_norm_eps: float | None = None,
                 tensor_names: dict[str, str] | None = None, float32_result: bool = False,
                 qk_norm_gain: bool = True, distance_slopes: tuple[float, ...] | None = None,
                 chunk: int = 0, qk_norm_span: str = "head", values_are_keys: bool = False,
                 sinks: bool = False, sized_buffers: bool = False,
                 position: PositionEncoding | None = None) -> None:
        """``v_head_dim``: the size of a value head where it differs from ``head_dim``, the
        size of a query and key head.  ``qk_norm_eps`` (None: no such norm): every query and
        key head is divided by its root mean square, eps inside the root, and multiplied by a
        gain of ``head_dim`` values shared by all heads, before the rotation.  ``tensor_names``
        renames checkpoint tensors (keys ``q``, ``k``, ``v``, ``o``, ``q_norm``, ``k_norm``;
        values relative to the part's prefix).  ``float32_result``: the output rows are
        float32 sums, for a consumer that normalises them.  ``qk_norm_gain`` False: the norm of
        the heads has no gain (and no tensors).  ``distance_slopes``: a value per query head;
        ``slope * (i - j)`` is taken off the score of query i and key j before the softmax (no
        rotation is needed for such a layer).  ``chunk`` > 0: query i sees key j <= i only if
        both lie in the same chunk of that many positions, counted from the sequence's start.
        ``qk_norm_span`` ``"projection"``: the norm spans all query heads at once (and all key
        heads at once), with a gain of that whole size each, instead of every head alone.
        ``values_are_keys``: there is no value projection; a token's values are its keys as
        projected, before norm and rotation.  ``sinks``: a learned score per query head (tensor
        ``sink``) that joins the softmax's denominator without a key or a value, unscaled.
        ``sized_buffers``: name the step buffers by their width, for a model whose attention layers
        differ in size."""
        if qk_norm_span not in ("head", "projection"):
            raise ValueError(f"qk_norm_span is 'head' or 'projection', got {qk_norm_span!r}")
        if qk_norm_span == "projection" and (qk_norm_eps is None or not qk_norm_gain):
            raise ValueError("a norm over the whole projection needs its eps and has gains")
        if values_are_keys and v_head_dim not in (None, head_dim):
            raise ValueError("values that are the keys have the keys' size")
        if num_heads % num_kv_heads:
            raise ValueError(f"{num_heads} heads are not a multiple of {num_kv_heads} kv heads")
        v_head_dim = head_dim if v_head_dim is None else v_head_dim
        self.head_norm = qk_norm_eps is not None and qk_norm_span == "head"
        self.wide_norm = qk_norm_eps is not None and qk_norm_span == "projection"
        plain = v_head_dim == head_dim and not self.head_norm
        if plain and (head_dim % 16 or head_dim > 256):
            if qk_norm_eps is None and not values_are_keys and not self.any_head_size:
                raise ValueError(f"head size {head_dim} is not supported (multiples of 16 up to 256)")
            plain = False  # the kernel that rotates and writes heads of any size, and the general attention
        if not 0 < head_dim <= 512 or not 0 < v_head_dim <= 512:
            raise ValueError(f"head sizes {head_dim} and {v_head_dim} are not supported (1 to 512)")
        self.hidden_size = hidden_size
        self.num_heads = num_heads
        self.num_kv_heads = num_kv_heads
        self.head_dim = head_dim
        self.v_head_dim = v_head_dim
        self.qk_norm_eps = qk_norm_eps
        self.qk_norm_gain = bool(qk_norm_gain)
        self.values_are_keys = bool(values_are_keys)
        self.has_sinks = bool(sinks)
        if distance_slopes is not None and len(distance_slopes) != num_heads:
            raise ValueError(f"{len(distance_slopes)} distance slopes for {num_heads} heads")
        if chunk < 0:
            raise ValueError(f"a chunk of {chunk} positions")
        self.distance_slopes = None if distance_slopes is None else tuple(float(v) for v in distance_slopes)
        self.chunk = int(chunk)
        self.scale = scale
        self.bias = bias
        self.window = window
        self.page_size = page_size  # None: the engine's block size
        self.position = position
        self.float32_result = float32_result
        self.q_size = num_heads * head_dim
        self.kv_size = num_kv_heads * head_dim
        self.v_size = num_kv_heads * v_head_dim
        self.o_size = num_heads * v_head_dim
        self.plain = plain
        # layers that are all alike share one step buffer a role; others name theirs by width
        self.shared_buffers = plain and not sized_buffers and not self.any_head_size
        # values wider than the keys by a whole factor (up to four) are kept in that many cache
        # planes of the keys' size, so that the kernels for keys and values of one size serve them
        factor = v_head_dim // head_dim if v_head_dim % head_dim == 0 else 0
        self.v_planes = factor if 1 < factor <= 4 else 1
        self.v_plane_dim = v_head_dim // self.v_planes
        self.names = {"q": "q_proj.weight", "k": "k_proj.weight", "v": "v_proj.weight",
                      "o": "o_proj.weight", "q_norm": "q_norm.weight", "k_norm": "k_norm.weight",
                      "q_bias": "q_proj.bias", "k_bias": "k_proj.bias", "v_bias": "v_proj.bias",
                      "o_bias": "o_proj.bias", "sink": "sinks", **(tensor_names or {})}

    def param_specs(self) -> list[ParamSpec]:
        total = self.q_size + self.kv_size + self.v_size
        n = self.names

        if self.values_are_keys:  # no value projection: q and k alone
            total = self.q_size + self.kv_size

        def stacked(q: str, k: str, v: str) -> tuple[ParamSource, ...]:
            qk = (ParamSource(n[q], 0, self.q_size), ParamSource(n[k], self.q_size, self.kv_size))
            if self.values_are_keys:
                return qk
            return (*qk, ParamSource(n[v], self.q_size + self.kv_size, self.v_size))

        specs = [
            ParamSpec("qkv_proj.weight", (total, self.hidden_size), sources=stacked("q", "k", "v")),
            ParamSpec("o_proj.weight", (self.hidden_size, self.o_size),
                      sources=(ParamSource(n["o"], 0, self.hidden_size),)),
        ]
        if self.bias:
            specs.append(ParamSpec("qkv_proj.bias", (total,), init="zeros",
                                   sources=stacked("q_bias", "k_bias", "v_bias")))
            specs.append(ParamSpec("o_proj.bias", (self.hidden_size,), init="zeros",
                                   sources=(ParamSource(n["o_bias"], 0, self.hidden_size),)))
        if self.qk_norm_eps is not None and self.qk_norm_gain:
            for key, whole in (("q_norm", self.q_size), ("k_norm", self.kv_size)):
                size = whole if self.wide_norm else self.head_dim
                specs.append(ParamSpec(key, (size,), kind="vector", init="gain",
                                       sources=(ParamSource(n[key], 0, size),)))
        if self.has_sinks:
            specs.append(ParamSpec("sinks", (self.num_heads,), kind="vector", init="normal",
                                   sources=(ParamSource(n["sink"], 0, self.num_heads),)))
        return specs

    def setup(self, runtime) -> None:
        super().setup(runtime)
        self._slopes = self._unit_gain = None
        if self.distance_slopes is not None:
            self._slopes = torch.tensor(self.distance_slopes, dtype=torch.float32, device=runtime.device)
        if self.head_norm and not self.qk_norm_gain:
            self._unit_gain = torch.ones(self.head_dim, dtype=torch.float32, device=runtime.device)

    def cache_need(self) -> CacheNeed:
        values = ((self.num_kv_heads, self.v_plane_dim),) * self.v_planes
        return CacheNeed(((self.num_kv_heads, self.head_dim), *values), self.window, self.page_size)

    def check_limits(self, limits) -> None:
        """The decode kernel keeps the page ids of a split's key range in LDS; a block table
        too wide for that is refused here, when the engine is built, not in a decode step.
        So is a cache in another dtype than the model's, which the attention kernels do not
        read (a subclass that names one in its ``cache_need`` must bring kernels that do)."""
        need = self.cache_need()
        if need.dtype is not None and need.dtype != self.runtime.dtype:
            raise ValueError(
                f"{type(self).__name__} keeps its cache in {need.dtype} beside a model in "
                f"{self.runtime.dtype}: the attention kernels read keys and values in the model's dtype")
        if not self._same_sizes() or self.runtime.dtype != torch.bfloat16 or not ops.decode_attention_supported(
                self.num_heads, self.num_kv_heads, self.head_dim, limits.page_size, self.runtime.dtype):
            return
        widest = ops.decode_attention_max_table(self.num_heads, self.num_kv_heads, self.head_dim)
        if limits.max_pages_per_seq > widest:
            raise ValueError(
                f"max_model_len={limits.max_model_len} with cache pages of {limits.page_size} tokens gives a "
                f"block table of {limits.max_pages_per_seq} entries per request; the decode attention kernel "
                f"serves at most {widest} for {self.num_heads} heads of {self.head_dim} over "
                f"{self.num_kv_heads} kv heads: use a larger block_size or a smaller max_model_len")

    def product_weights(self) -> tuple[str, ...]:
        return ("qkv_proj.weight", "o_proj.weight")

    def _same_sizes(self) -> bool:
        """Keys and values of one size in every plane: what the matrix-core kernels serve."""
        return self.v_plane_dim == self.head_dim

    def forward(self, x, ctx, call, sink=None):
        return self._output(self._attention(self._project(x, ctx), ctx, call), ctx, sink)

    def _project(self, x, ctx):
        """Rows ``[q heads | k heads | v heads]`` for the step's tokens, normed over the whole
        projection where the layer says so (norms of single heads and rotation come later)."""
        p = self.params
        # step buffers are named by their width: layers of one model may differ in size
        qkv = ctx.buf(_sized("attn_qkv", self.q_size + self.kv_size + self.v_size, self.shared_buffers),
                      self.q_size + self.kv_size + self.v_size)
        if self.values_are_keys:
            ops.linear(qkv[:, : self.q_size + self.kv_size], x, p["qkv_proj.weight"], p.get("qkv_proj.bias"))
            if not self.wide_norm:  # the values are the keys as projected
                qkv[:, self.q_size + self.kv_size:].copy_(qkv[:, self.q_size: self.q_size + self.kv_size])
        else:
            ops.linear(qkv, x, p["qkv_proj.weight"], p.get("qkv_proj.bias"))
        if self.wide_norm:
            # one norm over all query heads and one over all key heads, each with a gain of its
            # whole size; the raw keys become the values on the way where the layer says so
            ops.wide_qk_norm(qkv, p["q_norm"], p["k_norm"], self.qk_norm_eps, copy_k=self.values_are_keys)
        return qkv

    def _attention(self, qkv, ctx, call):
        """Norm of the heads, rotation, the cache write and the attention itself for rows ``qkv``;
        returns ``[T, heads * value size]`` in a step buffer."""
        p = self.params
        group = ctx.groups[call.group_index]
        # K pages [kv_heads, page, d]; V pages [kv_heads, dv, page]: the keys of a page lie
        # side by side, which is how the matrix cores want the values.  Values wider than the
        # keys by a whole factor lie in that many planes of the keys' size
        k_cache = group.plane(call.cache_index, 0, self.num_kv_heads, group.page_size, self.head_dim)
        v_planes = [group.plane(call.cache_index, 1 + c, self.num_kv_heads, self.v_plane_dim, group.page_size)
                    for c in range(self.v_planes)]
        rot = self.position.rotary(ctx) if self.position is not None else None
        if rot is None:
            cos = sin = ctx.buffers.get("rope_none", ctx.num_tokens, 0, torch.float32)
            rot_dim, interleaved = 0, False
        else:
            cos, sin, rot_dim, interleaved = rot.cos, rot.sin, rot.rot_dim, rot.interleaved
        if self.float32_heads:
            attn = ctx.buf(f"attn_out_f32:{self.o_size}", self.o_size, torch.float32)
        else:
            attn = ctx.buf(_sized("attn_out", self.o_size, self.shared_buffers), self.o_size)
        # with a norm of the heads, or values of another size than the keys, one kernel norms,
        # rotates and writes the cache; the attention kernels then take q and the cache as they are
        prepared = not self.plain
        if prepared:
            kv_slot = self._kv_slots(ctx, call, group, k_cache)
            ops.qk_norm_rope_kv_write(qkv, k_cache, v_planes, cos, sin, rot_dim=rot_dim,
                                      interleaved=interleaved, kv_slot=kv_slot, nh=self.num_heads,
                                      nkv=self.num_kv_heads, d=self.head_dim, dv=self.v_head_dim,
                                      q_gain=p.get("q_norm", self._unit_gain) if self.head_norm else None,
                                      k_gain=p.get("k_norm", self._unit_gain) if self.head_norm else None,
                                      eps=self.qk_norm_eps or 0.0, write_kv=call.write_cache)
            rot_dim, interleaved = 0, False
            cos = sin = ctx.buffers.get("rope_none", ctx.num_tokens, 0, torch.float32)
        if self.v_planes == 1:
            self._attend(attn, qkv, k_cache, v_planes[0], ctx, call, group, cos, sin, rot_dim, interleaved, prepared)
        else:
            # the same scores against each plane of the values; the planes' results, each [T, heads
            # * plane size], are then laid side by side within every head
            T, m, part = ctx.num_tokens, self.v_planes, self.num_heads * self.v_plane_dim
            parts = ctx.buffers.get(f"attn_planes:{part}:{attn.dtype}", m * T, part, attn.dtype,
                                    reserve=m * ctx.buffers.token_capacity)
            for c in range(m):
                self._attend(parts[c * T: (c + 1) * T], qkv, k_cache, v_planes[c], ctx, call, group, cos, sin,
                             rot_dim, interleaved, prepared)
            attn.view(T, self.num_heads, m, self.v_plane_dim).copy_(
                parts.view(m, T, self.num_heads, self.v_plane_dim).permute(1, 2, 0, 3))
        return attn

    def _output(self, attn, ctx, sink=None):
        p = self.params
        if sink is not None:
            return ops.linear(sink, attn, p["o_proj.weight"], p.get("o_proj.bias"))
        if self.float32_result:
            out = ctx.buf("mixer_out_f32", self.hidden_size, torch.float32)
        else:
            out = ctx.buf("mixer_out", self.hidden_size)
        ops.linear(out, attn, p["o_proj.weight"], p.get("o_proj.bias"))
        return out

    def _attend(self, attn, qkv, k_cache, v_cache, ctx, call, group, cos, sin, rot_dim, interleaved, prepared):
        """The attention itself into ``attn [T, heads * plane size]`` over one plane of values,
        by the kernel that serves the step's shape.  ``prepared``: q is ready and the cache is
        written; otherwise the kernels chosen here rotate and write on their way."""
        common = dict(table=group.table, positions=ctx.positions, token_req=ctx.token_req,
                      slots=ctx.slots, nh=self.num_heads, nkv=self.num_kv_heads, d=self.head_dim,
                      scale=self.scale, window=self.window)
        x_dtype = qkv.dtype
        # a distance bias and a chunked view are options of every attention kernel
        common.update(slopes=self._slopes, chunk=self.chunk, sinks=self.params.get("sinks"))
        # a token never sees more keys than its window or its chunk holds: what the launch plans count
        reach = min((n for n in (self.window, self.chunk) if n > 0), default=0)
        if not self._same_sizes():
            ops.paged_attention(attn, qkv, k_cache, v_cache, dv=self.v_plane_dim, **common)
        elif ctx.max_query_len == 1 and ops.decode_attention_supported(
                self.num_heads, self.num_kv_heads, self.head_dim, group.page_size, x_dtype):
            # single tokens: rotation, cache write and attention in one kernel on the matrix
            # cores, a block per (token, kv head, split)
            T = ctx.num_tokens
            waves = ops.decode_attention_waves(self.num_heads, self.num_kv_heads, self.head_dim)
            nsplit = decode_splits(T, self.num_kv_heads, ctx.max_seq_len, waves, reach)
            part_o = part_ml = None
            if nsplit > 1:
                # tokens x splits is at most the blocks wanted per kv head plus the tokens: room
                # for the largest at once, since a buffer that grows drops the graphs
                most = (decode_target_blocks() // self.num_kv_heads + 1 + max(T, ctx.buffers.seq_capacity)) \
                    * self.num_heads
                part_o = ctx.buffers.get(_sized("attn_part_o", self.head_dim, self.shared_buffers),
                                         T * self.num_heads * nsplit, self.head_dim,
                                         torch.float32, reserve=most)
                part_ml = ctx.buffers.get("attn_part_ml", T * self.num_heads * nsplit, 2, torch.float32,
                                          reserve=most)
            ops.decode_attention(attn, qkv, k_cache, v_cache, nsplit=nsplit, part_o=part_o,
                                 part_ml=part_ml, cos=cos, sin=sin, rot_dim=rot_dim,
                                 interleaved=interleaved, write_kv=call.write_cache and not prepared,
                                 token_rows=ctx.token_rows, **common)
        else:
            on_matrix_cores = ctx.max_query_len > 1 and self.scale > 0 and ops.prefill_attention_supported(
                self.num_heads, self.num_kv_heads, self.head_dim, group.page_size, x_dtype)
            # the kernel for portions rotates the queries on their way in where it can, which
            # saves writing them and reading them again
            rotates = on_matrix_cores and ops.prefill_attention_rotates(rot_dim, interleaved)
            if not prepared:
                ops.rope_kv_write(qkv, k_cache, v_cache, cos, sin, rot_dim=rot_dim,
                                  interleaved=interleaved, kv_slot=self._kv_slots(ctx, call, group, k_cache),
                                  nh=self.num_heads, nkv=self.num_kv_heads, d=self.head_dim,
                                  write_kv=call.write_cache, rotate_q=not rotates)
            if on_matrix_cores:
                # portions of prompts (single tokens may ride along): tiles of query rows per
                # block, and several blocks per tile where few rows meet many keys
                T = ctx.num_tokens
                nsplit = prefill_splits(T, self.num_kv_heads, self.num_heads // self.num_kv_heads,
                                        ctx.max_query_len, ctx.max_seq_len, reach, ctx.num_reqs)
                part_o = part_ml = None
                if nsplit > 1:
                    # asked for at their largest at once: a buffer that grows drops the graphs
                    most = prefill_split_rows(self.num_kv_heads, self.num_heads // self.num_kv_heads) * self.num_heads
                    part_o = ctx.buffers.get(_sized("attn_prefill_part_o", self.head_dim, self.shared_buffers),
                                             T * self.num_heads * nsplit,
                                             self.head_dim, torch.float32, reserve=most)
                    part_ml = ctx.buffers.get("attn_prefill_part_ml", T * self.num_heads * nsplit, 2,
                                              torch.float32, reserve=most)
                ops.prefill_attention(attn, qkv, k_cache, v_cache, table=group.table,
                                      positions=ctx.positions, q_start=ctx.q_start, slots=ctx.slots,
                                      num_reqs=ctx.num_reqs, nh=self.num_heads, nkv=self.num_kv_heads,
                                      d=self.head_dim, scale=self.scale, window=self.window,
                                      slopes=self._slopes, chunk=self.chunk, sinks=self.params.get("sinks"),
                                      nsplit=nsplit, part_o=part_o, part_ml=part_ml,
                                      **(dict(cos=cos, sin=sin, rot_dim=rot_dim, interleaved=interleaved)
                                         if rotates else {}))
            else:
                ops.paged_attention(attn, qkv, k_cache, v_cache, **common)

    @staticmethod
    def _kv_slots(ctx, call, group, k_cache):
        """Where each token's key and value go: once per step and cache group."""
        slot_key = ("kv_slot", call.group_index)
        kv_slot = ctx.scratch.get(slot_key)
        if kv_slot is None:
            kv_slot = ctx.buf(f"kv_slot_{call.group_index}", 1, torch.int32).view(-1)
            ops.kv_slots(kv_slot, positions=ctx.positions, token_req=ctx.token_req,
                         slots=ctx.slots, table=group.table, page_size=group.page_size,
                         num_pages=k_cache.shape[0])
            ctx.scratch[slot_key] = kv_slot
        return kv_slot


def _sized(name: str, cols: int, plain: bool) -> str:
    """The name of a step buffer: the plain attention of a model whose layers are all alike
    keeps one buffer per role; the others name theirs by width, since a buffer whose width
    changes from layer to layer would be allocated anew at every layer."""
    return name if plain else f"{name}:{cols}"


class DifferentialAttention(PagedAttention):
    """Grouped-query attention with two softmax maps a head over the same values: ``o = a1 - lambda
    * a2``, then each head's ``o`` over its root mean square (``eps`` inside the root, no gain) times
    ``1 - diff``, then the output product.  ``lambda = exp(lq1 . lk1) - exp(lq2 . lk2) + diff`` is one
    number for the layer, from four learned vectors of ``head_dim`` values.

    The checkpoint's q and k hold, head by head, the two maps' parts ``[map 1 | map 2]``.  A kv
    head's two key parts are kept as ONE cached key of ``2 * head_dim`` values, and every query head
    becomes two heads of that size, ``[q1 | 0]`` and ``[0 | q2]``: their scores against the joint key
    are the two maps' scores, so the layer is the paged attention of this file with ``2 * heads``
    query heads over ``kv_heads`` key/value heads (a token's keys and values are stored and read
    once for both maps), followed by one small kernel that joins the maps.  The zeros are rows of
    the fused projection matrix made when the weights arrive.  ``tensor_names`` renames checkpoint
    tensors (keys ``q``, ``k``, ``v``, ``o``, ``lq1``, ``lk1``, ``lq2``, ``lk2``)."""

    any_head_size = True
    takes_sink = False  # the maps are joined between the attention and the output product's input
    # where the two maps nearly cancel (lambda near one, a short window), rounding them to bfloat16
    # first would be magnified by the head's norm: they are joined as float32 sums
    float32_heads = True

    @property
    def takes_slice_sink(self) -> bool:  # float32 partial sums whatever the result's type
        return (self.heads * self.v_head_dim) % 8 == 0

    def __init__(self, *, hidden_size: int, num_heads: int, num_kv_heads: int, head_dim: int, v_head_dim: int,
                 scale: float, diff: float, eps: float, window: int = 0, page_size: int | None = None,
                 tensor_names: dict[str, str] | None = None, float32_result: bool = False,
                 position: PositionEncoding | None = None) -> None:
        if position is not None:
            raise ValueError("differential attention rotates nothing: the zero halves of its query heads "
                             "must stay zero")
        super().__init__(hidden_size=hidden_size, num_heads=2 * num_heads, num_kv_heads=num_kv_heads,
                         head_dim=2 * head_dim, v_head_dim=v_head_dim, scale=scale, window=window,
                         page_size=page_size, float32_result=float32_result, sized_buffers=True)
        self.heads, self.map_dim, self.diff, self.eps = num_heads, head_dim, float(diff), float(eps)
        self.map_names = {"q": "q_proj.weight", "k": "k_proj.weight", "v": "v_proj.weight", "o": "o_proj.weight",
                          "lq1": "lambda_q1", "lk1": "lambda_k1", "lq2": "lambda_q2", "lk2": "lambda_k2",
                          **(tensor_names or {})}
        self.lam: float | None = None

    def param_specs(self) -> list[ParamSpec]:
        n, H, d = self.map_names, self.hidden_size, self.map_dim

        def one(name: str, key: str, shape: tuple[int, ...], **kw) -> ParamSpec:
            return ParamSpec(name, shape, sources=(ParamSource(n[key], 0, shape[0]),), **kw)

        return [
            one("q.weight", "q", (self.heads * 2 * d, H)),
            one("k.weight", "k", (self.kv_size, H)),
            one("v.weight", "v", (self.v_size, H)),
            one("o_proj.weight", "o", (H, self.heads * self.v_head_dim)),
            *[one(key, key, (d,), kind="vector") for key in ("lq1", "lk1", "lq2", "lk2")],
        ]

    def weights_loaded(self) -> None:
        """The fused projection ``[padded q heads | k | v]`` and the layer's ``lambda``."""
        p, d = self.params, self.map_dim
        q = p["q.weight"].view(self.heads, 2, d, self.hidden_size)
        padded = torch.zeros(self.heads, 2, 2, d, self.hidden_size, dtype=q.dtype, device=q.device)
        padded[:, 0, 0] = q[:, 0]  # head 2h: [q1 | 0]
        padded[:, 1, 1] = q[:, 1]  # head 2h + 1: [0 | q2]
        fused = torch.cat([padded.view(self.q_size, self.hidden_size), p["k.weight"], p["v.weight"]], dim=0)
        old = p.get("qkv_proj.weight")
        if old is None:
            p["qkv_proj.weight"] = fused.contiguous()
        else:  # weights loaded again: the same storage, so nothing that holds it goes stale
            old.copy_(fused)
            if hasattr(old, "kvc_packed"):
                del old.kvc_packed
        f = torch.float32
        lam = torch.exp((p["lq1"].to(f) * p["lk1"].to(f)).sum()) - torch.exp((p["lq2"].to(f) * p["lk2"].to(f)).sum())
        self.lam = float(lam.item()) + self.diff

    def forward(self, x, ctx, call, sink=None):
        if "qkv_proj.weight" not in self.params or self.lam is None:
            self.weights_loaded()
        maps = self._attention(self._project(x, ctx), ctx, call)  # [T, heads x (a1 | a2)]
        width = self.heads * self.v_head_dim
        joined = ctx.buf(f"attn_joined:{width}", width)
        ops.diff_heads_norm(joined, maps, heads=self.heads, dv=self.v_head_dim, lam=self.lam, eps=self.eps,
                            post=1.0 - self.diff)
        return self._output(joined, ctx, sink)


register_mixer("paged_attention", PagedAttention)
register_mixer("differential_attention", DifferentialAttention)
