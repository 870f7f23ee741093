"""Python face of the gfx950 kernel library: loads it, checks operands on the host,
launches on torch's current stream.

There is no other compute path.  If the library cannot be loaded or built, the first
use raises; nothing falls back to the CPU or to torch's operators (library matrix
products for bfloat16 excepted, which is where the reference uses a library too:
``nn.Linear`` at kvcore/model/layer/linear.py:6-11).
"""

from __future__ import annotations

import os

import ctypes
from ctypes import c_float, c_int, c_int64, c_void_p
from dataclasses import dataclass

import torch

from . import build as _build

_LIB: ctypes.CDLL | None = None
_LIB_PATH: str | None = None

DTYPE_CODE = {torch.float32: 0, torch.bfloat16: 1}


class KernelError(RuntimeError):
    """The kernel library refused its arguments or could not launch."""


def _declare(lib: ctypes.CDLL) -> None:
    P, I, L, F = c_void_p, c_int, c_int64, c_float
    sigs = {
        "kvc_embed": [P, P, P, I, I, I, I, F, P],
        "kvc_logits_finish": [P, I, I, L, P, I, F, F, P],
        "kvc_fill_pages": [P, P, I, I, I, I, L, I, ctypes.c_uint32, P],
        "kvc_fill_normal": [P, L, I, ctypes.c_uint32, ctypes.c_uint32, F, F, P],
        "kvc_add_rmsnorm": [P, P, P, P, F, I, I, I, P],
        "kvc_add_slices_rmsnorm": [P, P, P, I, P, P, F, I, I, I, P],
        "kvc_rmsnorm": [P, P, P, F, I, I, L, L, I, P],
        "kvc_residual_add": [P, P, I, I, I, P],
        "kvc_residual_add2": [P, P, I, P, I, I, I, P],
        "kvc_silu_mul": [P, P, I, I, I, P],
        "kvc_gate_mul": [P, P, I, I, I, I, P],
        "kvc_activation": [P, P, L, I, I, P],
        "kvc_hyper_step": [P, I, P, P, I, I, P, I, P, P, F, P, P, F, I, I, I, P],
        "kvc_spread_streams": [P, P, I, I, I, P],
        "kvc_diff_heads_norm": [P, P, L, I, F, F, F, I, I, I, I, P],
        "kvc_norm_add_norm": [P, I, P, P, I, P, F, P, F, I, I, I, P],
        "kvc_wide_qk_norm": [P, L, P, P, F, I, I, I, I, I, P],
        "kvc_head_gate": [P, P, L, P, L, I, I, I, I, I, I, P],
        "kvc_latent_rows": [P, L, P, P, L, P, L, P, P, F, I, I, I, I, I, P],
        "kvc_max_gates": [P, P, P, P, L, P, L, P, P, F, P, P, P, P, P, I, I, I, P],
        "kvc_max_gated_finish": [P, I, P, P, P, L, I, P, F, F, I, I, I, P],
        "kvc_gather_rows": [P, P, P, I, I, I, I, P],
        "kvc_to_float": [P, P, L, I, P],
        "kvc_rope_table": [P, P, P, P, I, I, P],
        "kvc_kv_slots": [P, P, P, P, P, I, I, I, I, P],
        "kvc_rope_kv_write": [P, P, P, P, P, I, I, P, I, I, I, I, I, I, I, I, P],
        "kvc_paged_attention": [P, P, L, P, P, P, I, P, P, P, I, I, I, I, I, I, I, F, I, P, I, P, I, I, P],
        "kvc_linear_state_scan": [P, P, L, P, L, P, L, P, L, P, L, P, P, P, P, P, I, I, I, I, I, I, F, I, P],
        "kvc_sigmoid_power": [P, P, L, P, F, I, I, P],
        "kvc_decay_and_write_gates": [P, P, P, L, P, L, P, P, I, I, P],
        "kvc_unit_heads": [P, L, I, I, I, F, F, I, F, P],
        "kvc_head_rmsnorm_gate": [P, I, P, P, L, I, P, F, I, I, I, P],
        "kvc_moe_route": [P, P, P, I, I, I, I, I, I, P, I, F, P],
        "kvc_moe_router": [P, P, P, L, I, P, I, I, I, I, I, I, I, P, I, F, P],
        "kvc_moe_max_tiles": [I, I, I],
        "kvc_moe_tile_rows": [I, I],
        "kvc_moe_align": [P, P, P, P, I, I, I, I, P],
        "kvc_moe_gemm": [P, L, I, P, L, P, I, P, P, P, I, I, I, I, I, I, I, F, F, F, I, P],
        "kvc_moe_combine": [P, P, P, I, P, I, P, I, I, I, P],
        "kvc_clamped_glu": [P, P, I, I, F, F, I, P],
        "kvc_qk_norm_rope_kv_write": [P, L, P, P, I, P, P, F, P, P, I, I, P, I, I, I, I, I, I, I, I, P],
        "kvc_add_layernorm": [P, P, P, P, P, F, I, I, I, P],
        "kvc_rms_branches_mean": [P, P, P, I, F, I, I, I, P],
        "kvc_concat2": [P, P, P, I, I, I, P],
        "kvc_add_row": [P, P, I, I, P],
        "kvc_causal_conv": [P, L, I, P, L, I, P, P, P, P, P, P, P, I, I, I, I, I, I, I, P],
        "kvc_rglru_gates": [P, P, P, P, P, P, P, P, F, I, I, I, P],
        "kvc_rglru_scan": [P, I, P, P, P, L, I, P, P, P, P, P, I, I, I, P, L, P],
        "kvc_ssm_scan": [P, P, L, P, L, I, P, P, P, P, P, P, P, P, I, I, I, I, I, P],
        "kvc_gated_group_rmsnorm": [P, I, P, P, L, I, P, F, I, I, I, P],
        "kvc_decode_attention": [P, P, P, P, L, P, P, P, I, P, P, P, P, P, P, I, I, I, I, I, I, I, I, I,
                                 F, I, P, I, P, I, I, P],
        "kvc_decode_attention_waves": [I, I, I],
        "kvc_decode_attention_max_table": [I, I, I],
        "kvc_decode_attention_supported": [I, I, I, I, I],
        "kvc_prefill_attention": [P, P, L, P, P, P, I, P, P, P, I, I, I, I, I, I, I, F, I, P, I, P, P, P, I,
                                  P, P, I, I, I, P],
        "kvc_prefill_attention_supported": [I, I, I, I, I],
        "kvc_gemm_mid_slices": [I, I],
        "kvc_gemm_mid_bf16": [P, P, P, P, P, I, I, I, L, L, I, I, I, P],
        "kvc_gemm_f32": [P, P, P, P, I, I, I, L, L, P],
        "kvc_gemm_skinny_bf16": [P, P, P, P, I, I, I, L, L, I, I, P],
        "kvc_gemm_skinny_act_bf16": [P, P, P, P, I, I, I, L, L, I, I, P],
        "kvc_gemm_skinny_silu_mul_bf16": [P, P, P, P, I, I, I, L, L, I, P],
        "kvc_pack_weight": [P, P, I, I, P],
        "kvc_gemm_skinny_blocks": [I, I, I, I],
        "kvc_gemm_skinny_fused_bf16": [P, P, P, P, I, I, I, L, L, I, P, I, I, F, P, L, P, P, I, P],
        "kvc_table_update": [P, I, I, P, I, P],
        "kvc_argmax": [P, P, I, I, L, P, P, I, P],
        "kvc_argmax_static": [P, P, I, I, L, P],
        "kvc_sample": [P, P, I, I, L, P, P, P, P, P, P, P, L, I, P],
        "kvc_sample_workspace_words": [I, I],
        "kvc_peak_read": [P, L, I, P, P],
        "kvc_peak_mfma_bf16": [P, I, I, P],
    }
    for name, argtypes in sigs.items():
        fn = getattr(lib, name)
        fn.argtypes = argtypes
        fn.restype = c_int
    lib.kvc_last_error.restype = ctypes.c_char_p
    lib.kvc_last_error.argtypes = []
    lib.kvc_version.restype = c_int
    lib.kvc_compute_units.restype = c_int
    lib.kvc_compute_units.argtypes = []
    lib.kvc_last_variant.restype = ctypes.c_char_p
    lib.kvc_last_variant.argtypes = [c_int]
    lib.kvc_argmax_static_capacity.restype = c_int
    lib.kvc_argmax_static_capacity.argtypes = []
    lib.kvc_ssm_scan_max_state.restype = c_int
    lib.kvc_ssm_scan_max_state.argtypes = []
    lib.kvc_rglru_scan_segment.restype = c_int
    lib.kvc_rglru_scan_segment.argtypes = []


def load(build_if_missing: bool = True) -> ctypes.CDLL:
    """The loaded library; built first when no matching build is found."""
    global _LIB, _LIB_PATH
    if _LIB is not None:
        return _LIB
    path = _build.find_library()
    if path is None:
        if not build_if_missing:
            raise KernelError("kvcore_amd: the gfx950 kernel library is not built")
        path = _build.build()
    try:
        lib = ctypes.CDLL(str(path))
    except OSError as exc:
        raise KernelError(f"kvcore_amd: cannot load the kernel library {path}: {exc}") from exc
    _declare(lib)
    _LIB, _LIB_PATH = lib, str(path)
    return lib


def library_path() -> str | None:
    return _LIB_PATH


def _check(code: int, name: str) -> None:
    if code != 0:
        msg = load().kvc_last_error().decode("utf-8", "replace")
        raise KernelError(f"{name} failed ({code}): {msg}")


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream() -> int:
    """The current stream's handle (asked of torch at every launch: a stream context or a
    graph capture may have changed it)."""
    if _raw_stream is not None:
        return _raw_stream(torch.cuda.current_device())
    return torch.cuda.current_stream().cuda_stream


def _dev(t: torch.Tensor, name: str, dtype: torch.dtype | None = None) -> int:
    if not t.is_cuda:
        raise KernelError(f"{name} must be a GPU tensor (this engine has no CPU path)")
    if dtype is not None and t.dtype != dtype:
        raise KernelError(f"{name} must be {dtype}, got {t.dtype}")
    if not t.is_contiguous():
        raise KernelError(f"{name} must be contiguous")
    return t.data_ptr()


def _code(t: torch.Tensor, name: str) -> int:
    try:
        return DTYPE_CODE[t.dtype]
    except KeyError:
        raise KernelError(f"{name}: unsupported dtype {t.dtype}") from None


# ------------------------------------------------------------------------ wrappers
def embed(residual: torch.Tensor, table: torch.Tensor, ids: torch.Tensor, scale: float = 1.0) -> None:
    """``residual[t] = float(table[ids[t]]) * scale``; an id outside the table gives a NaN row."""
    T, H = residual.shape
    V = table.shape[0]
    if table.shape[1] != H or ids.numel() != T:
        raise KernelError("embed: shapes do not match")
    _check(load().kvc_embed(_dev(residual, "residual", torch.float32), _dev(table, "table"),
                            _dev(ids, "ids", torch.int32), T, H, V, _code(table, "table"), float(scale),
                            _stream()), "kvc_embed")


def logits_finish(logits: torch.Tensor, bias: torch.Tensor | None = None, soft_cap: float = 0.0,
                  scale: float = 1.0) -> None:
    """In place on float32 ``logits [S, V]``: ``+ bias``, then ``soft_cap * tanh(x / soft_cap)``
    when ``soft_cap > 0``, then ``* scale`` (the order of kvcore/sample/logits_processor.py:50-54)."""
    S, V = logits.shape
    if logits.dtype != torch.float32 or not logits.is_cuda or logits.stride(1) != 1:
        raise KernelError("logits_finish: expects float32 GPU logits [S, V]")
    if bias is not None and bias.shape != (V,):
        raise KernelError("logits_finish: bias must be [V]")
    _check(load().kvc_logits_finish(logits.data_ptr(), S, V, logits.stride(0),
                                    None if bias is None else _dev(bias, "bias"),
                                    0 if bias is None else _code(bias, "bias"), float(soft_cap),
                                    float(scale), _stream()), "kvc_logits_finish")


def fill_pages(storage: torch.Tensor, pages: torch.Tensor, n: int, value: float, stride: int = 1,
               page_axis: int = -4) -> None:
    """``storage`` is cache memory whose axis ``page_axis`` counts pages, everything behind it
    being one page and everything before it planes (a cache group's ``[entries, pages, elements
    a page]`` with ``page_axis=1``; by default ``[..., pages, kv_heads, page_size, head_dim]``);
    contiguous, float32 or bfloat16.  Every element of the pages ``pages[i * stride]``,
    ``i < n`` (int32 on the device), in all planes becomes ``value`` (0 or NaN as a
    rule); the null page is skipped."""
    axis = page_axis if page_axis >= 0 else storage.dim() + page_axis
    if not 0 <= axis < storage.dim() - 1 or not storage.is_contiguous():
        raise KernelError("fill_pages: storage must be contiguous [..., pages, a page...]")
    if n > 0 and pages.numel() < (n - 1) * stride + 1:
        raise KernelError("fill_pages: page list too short")
    num_pages = storage.shape[axis]
    page_elems = 1
    for size in storage.shape[axis + 1:]:
        page_elems *= size
    outer = storage.numel() // (num_pages * page_elems)
    esize = storage.element_size()
    probe = torch.tensor([value], dtype=storage.dtype)
    bits = int(probe.view(torch.int16 if esize == 2 else torch.int32)[0]) & (0xFFFF if esize == 2 else 0xFFFFFFFF)
    if pages.dtype != torch.int32 or not pages.is_cuda:
        raise KernelError("fill_pages: pages must be int32 on the GPU")
    _check(load().kvc_fill_pages(_dev(storage, "storage"), pages.data_ptr(), stride, n, outer,
                                 num_pages, page_elems, esize, bits, _stream()), "kvc_fill_pages")


def fill_normal(out: torch.Tensor, seed_lo: int, seed_hi: int, mean: float, std: float) -> None:
    """``out`` (contiguous float32 or bfloat16 on the GPU) gets ``mean + std * z_i``, ``z_i`` the
    normal variate of (seed_lo, seed_hi, i): the same bits as ``weights/random_normal.py``."""
    _check(load().kvc_fill_normal(_dev(out, "out"), out.numel(), _code(out, "out"),
                                  seed_lo & 0xFFFFFFFF, seed_hi & 0xFFFFFFFF, float(mean), float(std),
                                  _stream()), "kvc_fill_normal")


def add_rmsnorm(out: torch.Tensor, residual: torch.Tensor, delta: torch.Tensor | None,
                weight: torch.Tensor, eps: float) -> None:
    T, H = residual.shape
    if out.shape != (T, H) or weight.shape != (H,) or (delta is not None and delta.shape != (T, H)):
        raise KernelError("add_rmsnorm: shapes do not match")
    if delta is not None and delta.dtype != out.dtype:
        raise KernelError("add_rmsnorm: delta and out must share a dtype")
    _check(load().kvc_add_rmsnorm(_dev(out, "out"), _dev(residual, "residual", torch.float32),
                                  None if delta is None else _dev(delta, "delta"),
                                  _dev(weight, "weight", torch.float32), float(eps), T, H,
                                  _code(out, "out"), _stream()), "kvc_add_rmsnorm")


def rmsnorm(out: torch.Tensor, x: torch.Tensor, weight: torch.Tensor, eps: float) -> None:
    """Rows of ``x`` (last dim contiguous, any row stride) normalised into ``out``."""
    if x.dim() != 2 or out.shape != x.shape or x.stride(1) != 1 or out.stride(1) != 1:
        raise KernelError("rmsnorm: expects 2-D tensors with a contiguous last dim")
    if x.dtype != out.dtype or not x.is_cuda or not out.is_cuda:
        raise KernelError("rmsnorm: x and out must be GPU tensors of one dtype")
    T, H = x.shape
    if weight.shape != (H,):
        raise KernelError("rmsnorm: weight shape")
    _check(load().kvc_rmsnorm(out.data_ptr(), x.data_ptr(), _dev(weight, "weight", torch.float32),
                              float(eps), T, H, x.stride(0), out.stride(0), _code(x, "x"), _stream()),
           "kvc_rmsnorm")


def residual_add(residual: torch.Tensor, delta: torch.Tensor) -> None:
    T, H = residual.shape
    if delta.shape != (T, H):
        raise KernelError("residual_add: shapes do not match")
    _check(load().kvc_residual_add(_dev(residual, "residual", torch.float32), _dev(delta, "delta"),
                                   T, H, _code(delta, "delta"), _stream()), "kvc_residual_add")


def residual_add2(residual: torch.Tensor, a: torch.Tensor, b: torch.Tensor) -> None:
    """``residual += a + b``, the two branches added to each other first."""
    T, H = residual.shape
    if a.shape != (T, H) or b.shape != (T, H):
        raise KernelError("residual_add2: shapes do not match")
    _check(load().kvc_residual_add2(_dev(residual, "residual", torch.float32), _dev(a, "a"), _code(a, "a"),
                                    _dev(b, "b"), _code(b, "b"), T, H, _stream()), "kvc_residual_add2")


GATE_ACTS = {"silu": 0, "gelu_tanh": 1}  # the activations of a gated feed-forward's gate


def _gate_act(act: str) -> int:
    try:
        return GATE_ACTS[act]
    except KeyError:
        raise KernelError(f"unknown gate activation {act!r} (known: {sorted(GATE_ACTS)})") from None


def silu_mul(out: torch.Tensor, gate_up: torch.Tensor, act: str = "silu") -> None:
    """``out = act(gate) * up`` for rows ``[gate | up]``; ``act`` is ``silu`` or ``gelu_tanh``."""
    T, I2 = gate_up.shape
    if I2 % 2 or out.shape != (T, I2 // 2) or out.dtype != gate_up.dtype:
        raise KernelError("silu_mul: shapes or dtypes do not match")
    _check(load().kvc_gate_mul(_dev(out, "out"), _dev(gate_up, "gate_up"), T, I2 // 2, _gate_act(act),
                               _code(out, "out"), _stream()), "kvc_gate_mul")


ACTIVATIONS = {"relu_squared": 0}  # activations of a feed-forward without a gate


def activation(out: torch.Tensor, x: torch.Tensor, act: str) -> None:
    """``out = act(x)`` elementwise (in place is fine); ``act``: ``relu_squared``."""
    if act not in ACTIVATIONS:
        raise KernelError(f"unknown activation {act!r} (known: {sorted(ACTIVATIONS)})")
    if out.shape != x.shape or out.dtype != x.dtype or not out.is_contiguous() or not x.is_contiguous():
        raise KernelError("activation: shapes or dtypes do not match")
    _check(load().kvc_activation(_dev(out, "out"), _dev(x, "x"), x.numel(), ACTIVATIONS[act], _code(x, "x"),
                                 _stream()), "kvc_activation")


HYPER_MAX_COPIES = 8


def hyper_step(out: torch.Tensor | None, streams: torch.Tensor, copies: int,
               y: "torch.Tensor | SlicedRows | None" = None, *,
               mix: torch.Tensor | None = None, out_w: torch.Tensor | None = None, mult: float = 1.0,
               in_w: torch.Tensor | None = None, gain: torch.Tensor | None = None, eps: float = 0.0) -> None:
    """One step of a residual stream kept as ``copies`` rows a token (``streams [T, copies * H]``
    float32).  With ``y [T, H]``: every copy at once from the old ones, ``x_t <- sum_s mix[s, t] x_s
    + mult * out_w[t] * y`` (``mix`` None: the identity, ``out_w`` None: ones).  Then, with ``out
    [T, H]``: ``u = sum_t in_w[t] x_t`` (``in_w`` None: ones) and ``out = gain * u / sqrt(mean(u^2)
    + eps)``.  One copy and no coefficients: ``x += mult * y`` and the norm.  ``y`` may be the
    :class:`SlicedRows` that a product left (their sum is the result)."""
    T = streams.shape[0]
    if copies < 1 or streams.shape[1] % copies or streams.dtype != torch.float32 or not streams.is_contiguous():
        raise KernelError("hyper_step: the stream is contiguous float32 [T, copies * H]")
    H = streams.shape[1] // copies
    slices, bias = 1, None
    if isinstance(y, SlicedRows):
        if (y.rows, y.width) != (T, H) or y.data.dtype != torch.float32 or y.data.numel() < y.count * T * H \
                or not y.data.is_contiguous():
            raise KernelError("hyper_step: the partial sums do not fit")
        if y.bias is not None and (y.bias.shape != (H,) or not y.bias.is_contiguous()):
            raise KernelError("hyper_step: the bias does not fit")
        slices, bias, y = y.count, y.bias, y.data.view(-1)[: T * H].view(T, H)
    for t, name in ((y, "y"), (out, "out")):
        if t is not None and (t.shape != (T, H) or not t.is_contiguous()):
            raise KernelError(f"hyper_step: {name} must be contiguous [T, H]")
    for t, n, name in ((mix, copies * copies, "mix"), (out_w, copies, "out_w"), (in_w, copies, "in_w"), (gain, H, "gain")):
        if t is not None and (t.numel() != n or t.dtype != torch.float32 or not t.is_contiguous()):
            raise KernelError(f"hyper_step: {name} must be float32 with {n} values")
    if out is not None and gain is None:
        raise KernelError("hyper_step: the norm needs its gain")
    _check(load().kvc_hyper_step(
        None if out is None else _dev(out, "out"), 0 if out is None else _code(out, "out"), _dev(streams, "streams"),
        None if y is None else _dev(y, "y"), 0 if y is None else _code(y, "y"), slices,
        None if bias is None else _dev(bias, "bias"), 0 if bias is None else _code(bias, "bias"),
        None if mix is None else _dev(mix, "mix"), None if out_w is None else _dev(out_w, "out_w"), float(mult),
        None if in_w is None else _dev(in_w, "in_w"), None if gain is None else _dev(gain, "gain"), float(eps),
        T, H, copies, _stream()), "kvc_hyper_step")


@dataclass
class StreamWrite:
    """A sublayer's result ``y [T, H]`` that has still to join a stream of ``copies`` rows a token:
    ``x_t <- sum_s mix[s, t] x_s + mult * out_w[t] * y`` (see :func:`hyper_step`)."""

    y: "torch.Tensor | SlicedRows"
    copies: int
    mix: torch.Tensor | None
    out_w: torch.Tensor | None
    mult: float


def stream_write_read(out: torch.Tensor | None, streams: torch.Tensor, copies: int, pending: StreamWrite | None, *,
                      in_w: torch.Tensor | None = None, gain: torch.Tensor | None = None, eps: float = 0.0) -> None:
    """The pending write (may be None) and the next read with its norm (``out`` None: no read) in
    one pass over the copies."""
    if pending is None:
        if out is not None:
            hyper_step(out, streams, copies, in_w=in_w, gain=gain, eps=eps)
        return
    if pending.copies != copies:
        raise KernelError("stream_write_read: the pending result was made for another number of copies")
    hyper_step(out, streams, copies, pending.y, mix=pending.mix, out_w=pending.out_w, mult=pending.mult,
               in_w=in_w, gain=gain, eps=eps)


def spread_streams(streams: torch.Tensor, rows: torch.Tensor, copies: int) -> None:
    """``streams[t, c, :] = rows[t, :]`` for every copy ``c``: all copies start as the same row."""
    T, H = rows.shape
    if streams.shape != (T, copies * H) or streams.dtype != torch.float32 or rows.dtype != torch.float32 \
            or not streams.is_contiguous() or not rows.is_contiguous():
        raise KernelError("spread_streams: float32 [T, copies * H] from float32 [T, H]")
    _check(load().kvc_spread_streams(_dev(streams, "streams"), _dev(rows, "rows"), T, H, copies, _stream()),
           "kvc_spread_streams")


def diff_heads_norm(out: torch.Tensor, attn: torch.Tensor, *, heads: int, dv: int, lam: float, eps: float,
                    post: float) -> None:
    """Rows of ``attn`` hold ``heads`` pairs of results ``[a1 | a2]`` of ``dv`` values each; ``out[t,
    h] = (a1 - lam * a2) / sqrt(mean((a1 - lam * a2)^2) + eps) * post`` over the head's ``dv`` values.
    ``attn`` has the dtype of ``out`` or is float32 (results that were never rounded)."""
    T = out.shape[0]
    if out.shape != (T, heads * dv) or not out.is_contiguous() or attn.shape[0] < T or attn.stride(1) != 1 \
            or attn.shape[1] < 2 * heads * dv or attn.dtype not in (out.dtype, torch.float32):
        raise KernelError("diff_heads_norm: shapes do not match")
    _check(load().kvc_diff_heads_norm(_dev(out, "out"), attn.data_ptr(), attn.stride(0), _code(attn, "attn"),
                                      float(lam), float(eps), float(post), T, heads, dv, _code(out, "out"),
                                      _stream()), "kvc_diff_heads_norm")


def gather_rows(out: torch.Tensor, src: torch.Tensor, rows: torch.Tensor) -> None:
    S, H = out.shape
    if src.shape[1] != H or rows.numel() != S:
        raise KernelError("gather_rows: shapes do not match")
    _check(load().kvc_gather_rows(_dev(out, "out"), _dev(src, "src"), _dev(rows, "rows", torch.int32),
                                  S, H, _code(src, "src"), _code(out, "out"), _stream()),
           "kvc_gather_rows")


def to_float(out: torch.Tensor, src: torch.Tensor) -> None:
    if out.numel() != src.numel():
        raise KernelError("to_float: sizes do not match")
    _check(load().kvc_to_float(_dev(out, "out", torch.float32), _dev(src, "src"), src.numel(),
                               _code(src, "src"), _stream()), "kvc_to_float")


def rope_table(cos: torch.Tensor, sin: torch.Tensor, positions: torch.Tensor,
               inv_freq: torch.Tensor) -> None:
    T, half = cos.shape
    if sin.shape != (T, half) or positions.numel() < T or inv_freq.numel() != half:
        raise KernelError("rope_table: shapes do not match")
    _check(load().kvc_rope_table(_dev(cos, "cos", torch.float32), _dev(sin, "sin", torch.float32),
                                 _dev(positions, "positions", torch.int32),
                                 _dev(inv_freq, "inv_freq", torch.float32), T, half, _stream()),
           "kvc_rope_table")


def kv_slots(out: torch.Tensor, *, positions: torch.Tensor, token_req: torch.Tensor,
             slots: torch.Tensor, table: torch.Tensor, page_size: int, num_pages: int) -> None:
    """``out[t]`` = cache slot of token ``t`` (page * page_size + offset), -1 without a page,
    -2 for a padding token.  Reference: kvcore/kv/block_table.py:215-227 computes the same
    mapping per layer in Python."""
    T = out.numel()
    if positions.numel() < T or token_req.numel() < T:
        raise KernelError("kv_slots: per-token arrays too short")
    _check(load().kvc_kv_slots(_dev(out, "out", torch.int32), _dev(positions, "positions", torch.int32),
                               _dev(token_req, "token_req", torch.int32),
                               _dev(slots, "slots", torch.int32), _dev(table, "table", torch.int32),
                               table.shape[1], T, page_size, num_pages, _stream()), "kvc_kv_slots")


def rope_kv_write(qkv: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                  cos: torch.Tensor, sin: torch.Tensor, *, rot_dim: int, interleaved: bool,
                  kv_slot: torch.Tensor, nh: int, nkv: int, d: int, write_kv: bool = True,
                  rotate_q: bool = True) -> None:
    """``k_cache`` is ``[pages, nkv, page_size, d]``, ``v_cache`` ``[pages, nkv, d, page_size]``,
    both of the dtype of ``qkv``; ``kv_slot`` comes from ``kv_slots``.  Without ``rotate_q``
    the query heads are left as they are, for an attention kernel that rotates them itself."""
    T = qkv.shape[0]
    if qkv.shape != (T, (nh + 2 * nkv) * d):
        raise KernelError(f"rope_kv_write: qkv shape {tuple(qkv.shape)} does not fit heads")
    num_pages, page_size = _check_cache(k_cache, v_cache, nkv, d, "rope_kv_write")
    if k_cache.dtype != qkv.dtype or v_cache.dtype != qkv.dtype:
        raise KernelError("rope_kv_write: cache dtype differs from qkv")
    if cos.shape[0] < T or cos.shape[1] != rot_dim // 2 or sin.shape != cos.shape:
        raise KernelError("rope_kv_write: rotary tables do not fit")
    if kv_slot.numel() < T:
        raise KernelError("rope_kv_write: kv_slot too short")
    _check(load().kvc_rope_kv_write(
        _dev(qkv, "qkv"), _dev(k_cache, "k_cache"), _dev(v_cache, "v_cache"),
        _dev(cos, "cos", torch.float32), _dev(sin, "sin", torch.float32), rot_dim, int(interleaved),
        _dev(kv_slot, "kv_slot", torch.int32), T, nh, nkv, d, page_size, int(write_kv),
        int(rotate_q), _code(qkv, "qkv"), _stream()), "kvc_rope_kv_write")


def paged_attention(out: torch.Tensor, q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                    *, table: torch.Tensor, positions: torch.Tensor, token_req: torch.Tensor,
                    slots: torch.Tensor, nh: int, nkv: int, d: int, scale: float,
                    window: int = 0, dv: int | None = None, slopes: torch.Tensor | None = None,
                    chunk: int = 0, sinks: torch.Tensor | None = None) -> None:
    """``q`` is a ``[T, >= nh*d]`` view whose rows hold the query heads first.  ``dv``: the size
    of a value head where it differs from a key head's ``d`` (``out`` is ``[T, nh*dv]``).
    ``slopes`` (float32 ``[nh]``): ``slopes[h] * distance`` is taken off every score of head h;
    ``chunk``: a token sees only the keys of its own chunk of that many positions.  ``sinks``
    (float32 ``[nh]``): ``exp(sinks[h])`` joins the softmax's denominator of head h.  ``out`` has
    the queries' dtype, or is float32 beside bfloat16 queries: the weighted sums unrounded (the two
    matrix-core kernels take such an ``out`` too)."""
    if slopes is not None and (slopes.shape != (nh,) or slopes.dtype != torch.float32):
        raise KernelError("paged_attention: slopes must be float32 [nh]")
    T = out.shape[0]
    dv = d if dv is None else dv
    if out.shape != (T, nh * dv) or not out.is_contiguous():
        raise KernelError("paged_attention: out must be contiguous [T, nh*dv]")
    if q.shape[0] != T or q.stride(1) != 1 or q.shape[1] < nh * d or out.dtype not in (q.dtype, torch.float32):
        raise KernelError("paged_attention: q does not fit")
    num_pages, page_size = _check_cache(k_cache, v_cache, nkv, d, "paged_attention", dv)
    if k_cache.dtype != q.dtype:
        raise KernelError("paged_attention: cache dtype differs from the queries'")
    if positions.numel() < T or token_req.numel() < T:
        raise KernelError("paged_attention: per-token arrays too short")
    _check(load().kvc_paged_attention(
        out.data_ptr(), q.data_ptr(), q.stride(0), _dev(k_cache, "k_cache"), _dev(v_cache, "v_cache"),
        _dev(table, "table", torch.int32), table.shape[1],
        _dev(positions, "positions", torch.int32), _dev(token_req, "token_req", torch.int32),
        _dev(slots, "slots", torch.int32), T, nh, nkv, d, dv, page_size, num_pages, float(scale),
        int(window), None if slopes is None else _dev(slopes, "slopes"), int(chunk), _sinks(sinks, nh),
        int(out.dtype == torch.float32 and q.dtype != torch.float32), _code(q, "q"), _stream()), "kvc_paged_attention")


def qk_norm_rope_kv_write(qkv: torch.Tensor, k_cache: torch.Tensor,
                          v_cache: "torch.Tensor | list[torch.Tensor]",
                          cos: torch.Tensor, sin: torch.Tensor, *, rot_dim: int, interleaved: bool,
                          kv_slot: torch.Tensor, nh: int, nkv: int, d: int, dv: int,
                          q_gain: torch.Tensor | None = None, k_gain: torch.Tensor | None = None,
                          eps: float = 0.0, write_kv: bool = True) -> None:
    """Rows of ``qkv`` are ``[nh heads of d | nkv heads of d | nkv heads of dv]``.  With gains
    (float32 ``[d]``, shared by all heads) every q and k head is first divided by its root mean
    square (``eps`` inside the root) and multiplied by the gain; then the first ``rot_dim``
    elements are rotated; q and k are rewritten in place, k and v stored at ``kv_slot``
    (``k_cache [pages, nkv, page_size, d]``, ``v_cache [pages, nkv, dv, page_size]``, or a list of
    up to four planes ``[pages, nkv, dv / n, page_size]`` that each hold a slice of every value
    head)."""
    T = qkv.shape[0]
    if qkv.dim() != 2 or qkv.stride(1) != 1 or qkv.shape[1] < (nh + nkv) * d + nkv * dv:
        raise KernelError(f"qk_norm_rope_kv_write: qkv shape {tuple(qkv.shape)} does not fit the heads")
    planes = list(v_cache) if isinstance(v_cache, (list, tuple)) else [v_cache]
    if not 1 <= len(planes) <= 4 or dv % len(planes):
        raise KernelError("qk_norm_rope_kv_write: one to four value planes that divide the value size")
    for plane in planes:
        _check_cache(k_cache, plane, nkv, d, "qk_norm_rope_kv_write", dv // len(planes))
        if plane.dtype != qkv.dtype:
            raise KernelError("qk_norm_rope_kv_write: cache dtype differs from qkv")
    page_size = k_cache.shape[2]
    if k_cache.dtype != qkv.dtype:
        raise KernelError("qk_norm_rope_kv_write: cache dtype differs from qkv")
    if rot_dim and (cos.shape[0] < T or cos.shape[1] != rot_dim // 2 or sin.shape != cos.shape):
        raise KernelError("qk_norm_rope_kv_write: rotary tables do not fit")
    if kv_slot.numel() < T:
        raise KernelError("qk_norm_rope_kv_write: kv_slot too short")
    for g in (q_gain, k_gain):
        if g is not None and (g.shape != (d,) or g.dtype != torch.float32):
            raise KernelError("qk_norm_rope_kv_write: a gain must be float32 [d]")
    pointers = (c_void_p * len(planes))(*[_dev(plane, "v_cache") for plane in planes])
    _check(load().kvc_qk_norm_rope_kv_write(
        qkv.data_ptr(), qkv.stride(0), _dev(k_cache, "k_cache"), pointers, len(planes),
        None if q_gain is None else _dev(q_gain, "q_gain"), None if k_gain is None else _dev(k_gain, "k_gain"),
        float(eps), _dev(cos, "cos", torch.float32), _dev(sin, "sin", torch.float32), int(rot_dim),
        int(bool(interleaved)), _dev(kv_slot, "kv_slot", torch.int32), T, nh, nkv, d, dv, page_size,
        int(write_kv), _code(qkv, "qkv"), _stream()), "kvc_qk_norm_rope_kv_write")


def _slopes(slopes: torch.Tensor | None, nh: int) -> int | None:
    """Pointer to the distance slopes (float32, a value per query head) of the attention kernels."""
    if slopes is None:
        return None
    if slopes.shape != (nh,):
        raise KernelError("attention: a distance slope per query head")
    return _dev(slopes, "slopes", torch.float32)


def _sinks(sinks: torch.Tensor | None, nh: int) -> int | None:
    """Pointer to the softmax sinks (float32, a value per query head) of the attention kernels."""
    if sinks is None:
        return None
    if sinks.shape != (nh,):
        raise KernelError("attention: a sink per query head")
    return _dev(sinks, "sinks", torch.float32)


def decode_attention_supported(nh: int, nkv: int, d: int, page_size: int, dtype: torch.dtype) -> bool:
    return bool(load().kvc_decode_attention_supported(nh, nkv, d, page_size, DTYPE_CODE.get(dtype, -1)))


KERNEL_FAMILIES = {"prefill_attention": 0, "rope_kv_write": 1, "decode_attention": 2}


def last_variant(family: str) -> str:
    """Which variant of a kernel family this thread's last launch took (see the C header): for
    tests that must know which code ran."""
    return load().kvc_last_variant(KERNEL_FAMILIES[family]).decode()


def measure_peaks(device: str | torch.device = "cuda:0") -> dict[str, float]:
    """What this chip gives a kernel that does nothing but read (bytes a second: 16-byte loads
    over 1 GiB pieces of a 3 GiB buffer, so that no cache serves them, two blocks a compute
    unit) and nothing but multiply on the matrix cores (bfloat16 flops a second, operands in
    registers, four waves a SIMD).  Some 0.1 s.  The data sheet says 8 TB/s and 2.5 PFLOP/s."""
    lib = load()
    device = torch.device(device)
    cus = compute_units()
    piece = 1 << 30
    buf = torch.empty(3 * piece, dtype=torch.uint8, device=device)
    buf.fill_(1)
    sink = torch.zeros(4, dtype=torch.int32, device=device)
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)

    def read(i: int) -> None:
        _check(lib.kvc_peak_read(buf.data_ptr() + (i % 3) * piece, piece, 2 * cus, sink.data_ptr(), _stream()),
               "kvc_peak_read")

    for i in range(3):
        read(i)
    start.record()
    for i in range(12):
        read(i)
    end.record()
    end.synchronize()
    read_rate = 12 * piece / (start.elapsed_time(end) * 1e-3)
    del buf
    blocks, rounds = 4 * cus, 8000
    out = torch.empty(blocks * 256, dtype=torch.float32, device=device)
    for _ in range(2):
        _check(lib.kvc_peak_mfma_bf16(out.data_ptr(), blocks, 200, _stream()), "kvc_peak_mfma_bf16")
    flops = blocks * 4 * rounds * 4 * 2.0 * 32 * 32 * 16
    best = 0.0
    for _ in range(4):  # the clock takes a few milliseconds to rise: the fastest run is the peak
        start.record()
        _check(lib.kvc_peak_mfma_bf16(out.data_ptr(), blocks, rounds, _stream()), "kvc_peak_mfma_bf16")
        end.record()
        end.synchronize()
        best = max(best, flops / (start.elapsed_time(end) * 1e-3))
    return {"read_bytes_per_s": read_rate, "mfma_bf16_flops_per_s": best}


_COMPUTE_UNITS: int | None = None


def compute_units() -> int:
    """Compute units of the current GPU, which launch plans count their blocks against (256, an
    MI355X's, where no GPU is visible: plans are also worked out on a host without one)."""
    global _COMPUTE_UNITS
    if _COMPUTE_UNITS is None:
        _COMPUTE_UNITS = int(load().kvc_compute_units()) if torch.cuda.is_available() else 256
    return _COMPUTE_UNITS


def decode_attention_max_table(nh: int, nkv: int, d: int) -> int:
    """The widest block table (entries per request) that :func:`decode_attention` serves."""
    return int(load().kvc_decode_attention_max_table(nh, nkv, d))


def decode_attention_waves(nh: int, nkv: int, d: int) -> int:
    """How many waves of a block share its range of keys in :func:`decode_attention`."""
    return int(load().kvc_decode_attention_waves(nh, nkv, d))


def decode_attention(out: torch.Tensor, qkv: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                     *, table: torch.Tensor, positions: torch.Tensor, token_req: torch.Tensor,
                     slots: torch.Tensor, nh: int, nkv: int, d: int, scale: float, window: int = 0,
                     nsplit: int = 1, part_o: torch.Tensor | None = None,
                     part_ml: torch.Tensor | None = None, cos: torch.Tensor | None = None,
                     sin: torch.Tensor | None = None, rot_dim: int = 0, interleaved: bool = False,
                     write_kv: bool = False, token_rows: torch.Tensor | None = None,
                     slopes: torch.Tensor | None = None, chunk: int = 0,
                     sinks: torch.Tensor | None = None) -> None:
    """bfloat16 attention of single tokens on the matrix cores (see the C header), with the
    rotation of each token's query and key and the write of its key and value into the cache
    (``write_kv``) in the same kernel; ``qkv`` is not changed.  With ``rot_dim = 0`` and
    ``write_kv = False`` it is the attention alone over queries as they are.  ``token_rows``
    (``slots[token_req]``, -1 for padding) may be given to save the kernel a lookup.  ``part_o`` and
    ``part_ml`` are float32 workspaces of at least ``T*nh*nsplit*d`` and ``T*nh*nsplit*2``
    elements when ``nsplit > 1``."""
    T = out.shape[0]
    if out.shape != (T, nh * d) or not out.is_contiguous() or out.dtype not in (torch.bfloat16, torch.float32):
        raise KernelError("decode_attention: out must be contiguous bfloat16 (or float32) [T, nh*d]")
    need = (nh + 2 * nkv) * d if write_kv else nh * d
    if qkv.shape[0] != T or qkv.stride(1) != 1 or qkv.shape[1] < need or qkv.dtype != torch.bfloat16:
        raise KernelError("decode_attention: qkv does not fit")
    num_pages, page_size = _check_cache(k_cache, v_cache, nkv, d, "decode_attention")
    if k_cache.dtype != qkv.dtype:
        raise KernelError("decode_attention: cache dtype differs from the queries'")
    if positions.numel() < T or token_req.numel() < T:
        raise KernelError("decode_attention: per-token arrays too short")
    c = s_ = None
    if rot_dim:
        if cos is None or sin is None or cos.shape[0] < T or cos.shape[1] != rot_dim // 2 \
                or sin.shape != cos.shape or not cos.is_contiguous() or not sin.is_contiguous():
            raise KernelError("decode_attention: cos and sin must be contiguous [>= T, rot_dim/2]")
        c, s_ = _dev(cos, "cos", torch.float32), _dev(sin, "sin", torch.float32)
    po = pm = None
    if nsplit > 1:
        if part_o is None or part_ml is None or part_o.numel() < T * nh * nsplit * d \
                or part_ml.numel() < T * nh * nsplit * 2:
            raise KernelError("decode_attention: workspace missing or too small")
        po, pm = _dev(part_o, "part_o", torch.float32), _dev(part_ml, "part_ml", torch.float32)
    _check(load().kvc_decode_attention(
        out.data_ptr(), po, pm, qkv.data_ptr(), qkv.stride(0), _dev(k_cache, "k_cache"),
        _dev(v_cache, "v_cache"), _dev(table, "table", torch.int32), table.shape[1],
        _dev(positions, "positions", torch.int32), _dev(token_req, "token_req", torch.int32),
        _dev(slots, "slots", torch.int32),
        None if token_rows is None else _dev(token_rows, "token_rows", torch.int32),
        c, s_, int(rot_dim), int(bool(interleaved)),
        int(bool(write_kv)), T, nh, nkv, d, page_size, num_pages, float(scale),
        int(window), _slopes(slopes, nh), int(chunk), _sinks(sinks, nh), int(nsplit),
        int(out.dtype == torch.float32), _stream()),
        "kvc_decode_attention")


def prefill_attention_supported(nh: int, nkv: int, d: int, page_size: int, dtype: torch.dtype) -> bool:
    return bool(load().kvc_prefill_attention_supported(nh, nkv, d, page_size, DTYPE_CODE.get(dtype, -1)))


def prefill_attention(out: torch.Tensor, q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                      *, table: torch.Tensor, positions: torch.Tensor, q_start: torch.Tensor,
                      slots: torch.Tensor, num_reqs: int, nh: int, nkv: int, d: int, scale: float,
                      window: int = 0, nsplit: int = 1, part_o: torch.Tensor | None = None,
                      part_ml: torch.Tensor | None = None, cos: torch.Tensor | None = None,
                      sin: torch.Tensor | None = None, rot_dim: int = 0, interleaved: bool = False,
                      slopes: torch.Tensor | None = None, chunk: int = 0,
                      sinks: torch.Tensor | None = None) -> None:
    """bfloat16 attention of portions of prompts on the matrix cores (see the C header).
    ``nsplit > 1`` deals every tile's keys to that many blocks; ``part_o`` (float32,
    ``T*nh*nsplit*d`` values) and ``part_ml`` (``T*nh*nsplit*2``) are then the workspace.
    With ``cos`` and ``sin`` (``[T, rot_dim / 2]`` float32) the queries come unrotated and
    the kernel rotates them (``prefill_attention_rotates`` says for which shapes)."""
    T = out.shape[0]
    if out.shape != (T, nh * d) or not out.is_contiguous() or out.dtype not in (torch.bfloat16, torch.float32):
        raise KernelError("prefill_attention: out must be contiguous bfloat16 (or float32) [T, nh*d]")
    if q.shape[0] != T or q.stride(1) != 1 or q.shape[1] < nh * d or q.dtype != torch.bfloat16:
        raise KernelError("prefill_attention: q does not fit")
    num_pages, page_size = _check_cache(k_cache, v_cache, nkv, d, "prefill_attention")
    if k_cache.dtype != q.dtype:
        raise KernelError("prefill_attention: cache dtype differs from the queries'")
    if positions.numel() < T or q_start.numel() < num_reqs + 1 or slots.numel() < num_reqs:
        raise KernelError("prefill_attention: index arrays too short")
    po = pml = None
    if nsplit > 1:
        if part_o is None or part_ml is None or part_o.numel() < T * nh * nsplit * d or \
                part_ml.numel() < T * nh * nsplit * 2:
            raise KernelError("prefill_attention: the workspace for splits is missing or too small")
        po, pml = _dev(part_o, "part_o", torch.float32), _dev(part_ml, "part_ml", torch.float32)
    cs = sn = None
    if cos is not None:
        if sin is None or cos.shape[0] < T or cos.shape[1] != rot_dim // 2 or sin.shape != cos.shape \
                or not prefill_attention_rotates(rot_dim, interleaved):
            raise KernelError("prefill_attention: rotary tables do not fit")
        cs, sn = _dev(cos, "cos", torch.float32), _dev(sin, "sin", torch.float32)
    _check(load().kvc_prefill_attention(
        out.data_ptr(), q.data_ptr(), q.stride(0), _dev(k_cache, "k_cache"), _dev(v_cache, "v_cache"),
        _dev(table, "table", torch.int32), table.shape[1], _dev(positions, "positions", torch.int32),
        _dev(q_start, "q_start", torch.int32), _dev(slots, "slots", torch.int32), T, num_reqs,
        nh, nkv, d, page_size, num_pages, float(scale), int(window), _slopes(slopes, nh), int(chunk),
        _sinks(sinks, nh), po, pml, int(nsplit), cs, sn, int(rot_dim) if cs is not None else 0, int(interleaved),
        int(out.dtype == torch.float32), _stream()),
        "kvc_prefill_attention")


def prefill_attention_rotates(rot_dim: int, interleaved: bool) -> bool:
    """Whether ``prefill_attention`` can rotate the queries itself: a lane of the kernel
    must hold both elements of every rotary pair."""
    return rot_dim > 0 and rot_dim % (32 if interleaved else 64) == 0


def _check_cache(k_cache: torch.Tensor, v_cache: torch.Tensor, nkv: int, d: int, who: str,
                 dv: int | None = None) -> tuple[int, int]:
    """K pages are ``[pages, nkv, page_size, d]``, V pages ``[pages, nkv, dv, page_size]``
    (``dv`` None: values as wide as keys)."""
    dv = d if dv is None else dv
    if k_cache.dim() != 4 or v_cache.dim() != 4:
        raise KernelError(f"{who}: cache planes must be 4-D")
    num_pages, ckv, page_size, cd = k_cache.shape
    if (ckv, cd) != (nkv, d) or tuple(v_cache.shape) != (num_pages, nkv, dv, page_size):
        raise KernelError(f"{who}: cache shapes {tuple(k_cache.shape)} / {tuple(v_cache.shape)} do not fit "
                          f"{nkv} kv heads of {d} and {dv}")
    if k_cache.dtype != v_cache.dtype:
        raise KernelError(f"{who}: K and V planes differ in dtype")
    return num_pages, page_size


def gemm_f32(out: torch.Tensor, a: torch.Tensor, w: torch.Tensor, bias: torch.Tensor | None) -> None:
    M, K = a.shape
    N = w.shape[0]
    if w.shape != (N, K) or out.shape != (M, N) or a.stride(1) != 1 or out.stride(1) != 1:
        raise KernelError("gemm_f32: shapes do not match")
    for t, name in ((a, "a"), (out, "out")):
        if t.dtype != torch.float32 or not t.is_cuda:
            raise KernelError(f"gemm_f32: {name} must be a float32 GPU tensor")
    _check(load().kvc_gemm_f32(out.data_ptr(), a.data_ptr(), _dev(w, "w", torch.float32),
                               None if bias is None else _dev(bias, "bias", torch.float32),
                               M, N, K, a.stride(0), out.stride(0), _stream()), "kvc_gemm_f32")


SKINNY_MAX_ROWS = 64
SKINNY_PREFERRED_ROWS = 16


def can_pack_weight(w: torch.Tensor) -> bool:
    return (w.dim() == 2 and w.dtype == torch.bfloat16 and w.is_cuda and w.is_contiguous()
            and w.shape[0] % 16 == 0 and w.shape[1] % 64 == 0)


def pack_weight(w: torch.Tensor) -> torch.Tensor:
    """A copy of the bfloat16 matrix ``w [N, K]`` in tiles of 16 rows x 32 columns, each 1 KB in
    one piece, the tiles of 16 rows one after the other along K: the order in which the
    weight-streaming products for few rows read a matrix, so that a load of theirs is one
    contiguous kilobyte instead of 64 bytes from each of 16 rows (some 8% more bandwidth on
    this chip).  The copy is kept as ``w.kvc_packed``; the products find it there and give
    the same bits with it as without."""
    if not can_pack_weight(w):
        raise KernelError("pack_weight: a contiguous bfloat16 GPU matrix of a multiple of 16 rows "
                          "and a multiple of 64 columns")
    packed = torch.empty_like(w)
    _check(load().kvc_pack_weight(packed.data_ptr(), w.data_ptr(), w.shape[0], w.shape[1], _stream()),
           "kvc_pack_weight")
    w.kvc_packed = packed
    return packed


def _streamed(w: torch.Tensor, rows: int | None = None) -> tuple[int, int]:
    """(pointer, packed flag) of the matrix a weight-streaming product should read: the packed
    twin of ``w`` where there is one (``rows``: the product's own row count, a multiple of 16
    for a packed matrix, which the gated product's half must be too)."""
    packed = getattr(w, "kvc_packed", None)
    if packed is not None and (rows is None or rows % 16 == 0):
        return packed.data_ptr(), 1
    return _dev(w, "w"), 0


def gemm_skinny_bf16(out: torch.Tensor, a: torch.Tensor, w: torch.Tensor,
                     bias: torch.Tensor | None = None) -> None:
    """``out = a @ w.T (+ bias)`` for up to 64 rows of bfloat16; ``out`` is bfloat16 or
    float32 (the sums are float32 either way)."""
    M, K = a.shape
    N = w.shape[0]
    if w.shape != (N, K) or out.shape != (M, N) or a.stride(1) != 1 or out.stride(1) != 1:
        raise KernelError("gemm_skinny_bf16: shapes do not match")
    if a.dtype != torch.bfloat16 or w.dtype != torch.bfloat16 or not a.is_cuda or not out.is_cuda:
        raise KernelError("gemm_skinny_bf16: operands must be bfloat16 GPU tensors")
    if bias is not None and (bias.dtype != torch.bfloat16 or bias.shape != (N,)):
        raise KernelError("gemm_skinny_bf16: bias must be bfloat16 [N]")
    w_ptr, packed = _streamed(w)
    _check(load().kvc_gemm_skinny_bf16(out.data_ptr(), a.data_ptr(), w_ptr,
                                       None if bias is None else _dev(bias, "bias"), M, N, K,
                                       a.stride(0), out.stride(0), _code(out, "out"), packed, _stream()),
           "kvc_gemm_skinny_bf16")


@dataclass
class ScaledRows:
    """Activation rows ``[T, H]`` that carry an RMS norm still to be finished: ``data`` holds
    ``residual * gain`` in bfloat16, ``ss_parts`` ``[T, parts]`` float32 partial sums of the
    residual's squares.  ``linear`` and ``linear_silu_mul`` take it in place of ``x`` and
    multiply row ``t``'s sums by ``rsqrt(sum(ss_parts[t]) / width + eps)``, which equals
    the product of the normalised row.  Made by ``linear`` into a :class:`ResidualSink`."""

    data: torch.Tensor
    ss_parts: torch.Tensor
    width: int
    eps: float

    @property
    def shape(self) -> torch.Size:
        return self.data.shape

    @property
    def dtype(self) -> torch.dtype:
        return self.data.dtype


@dataclass
class ResidualSink:
    """Where a product's result may go instead of a plain tensor: added into the float32
    ``residual`` rows, with ``out`` receiving ``bfloat16(residual * gain)`` and ``ss_parts``
    (room for ``[T, parts]`` float32) the new rows' partial sums of squares: the next norm,
    done but for the scale factor that the consuming product applies."""

    residual: torch.Tensor
    gain: torch.Tensor
    eps: float
    out: torch.Tensor
    ss_parts: torch.Tensor | None
    # for steps of 17 to 192 rows: float32 room for the partial sums of a product cut along K
    # (``mid_slices_bound(N) * T * N`` values); the sink then finishes the norm itself and
    # ``out`` receives the normalised rows
    slices: torch.Tensor | None = None


@dataclass
class NormedRows:
    """Rows that a :class:`ResidualSink` has already added into the residual and normalised:
    what ``linear`` returns for a sink that carries a workspace (steps of 17 to 192 rows)."""

    data: torch.Tensor


@dataclass
class SliceSink:
    """Where the last product of a part goes when the block behind it norms the result before
    it joins the stream (steps of 17 to 192 rows): ``slices`` is float32 room for the partial
    sums of a product cut along K (``mid_slices_bound(N) * T * N`` values).  ``linear`` leaves
    them there and returns :class:`SlicedRows`; ``norm_add_norm`` sums them on its way.
    ``takes_bias``: the consumer adds a product's bias itself (``SlicedRows.bias``), so a product
    with a bias may be cut along K as well."""

    slices: torch.Tensor
    takes_bias: bool = False


@dataclass
class SlicedRows:
    """``count`` partial sums ``[count, T, N]`` float32 at the start of ``data``'s storage: rows
    of a product that the consumer adds up (one slice is the product itself).  ``bias``: the
    product's bias ``[N]``, still to be added to the sum (only for a sink that ``takes_bias``)."""

    data: torch.Tensor
    count: int
    rows: int
    width: int
    bias: torch.Tensor | None = None


# The most rows the kernel that shares its rows through LDS takes (twelve tiles of 16 a wave).
# Measured on the 8B shape against the vendor's products with a norm kernel between them, a
# whole decode step: 72 rows 5.93 against 6.66 ms, 96 rows 6.53 against 7.72, 128 rows 7.57
# against 8.63, 160 rows 9.37 against 9.79, 192 rows 10.12 against 11.35; with sixteen tiles a
# wave 256 rows took 12.86 against 11.11, so the vendor's product has them.
MID_ROWS = 192
# Which products gain beyond 64 rows, one by one against the vendor's (us at 96 / 128 / 192 rows,
# packed weights): the narrow ones that are cut along K do (4096 x 14336: 33 / 45 / 64 against
# 64 / 76 / 104; 4096 x 4096: 13 / 15 / 21 against 23 / 25 / 34; 8192 x 28672: 109 / 136 / 209
# against 123 / 201 / 232); the gated one up to 128 rows (28672 x 4096: 54 / 67 / 83 against 53 /
# 54 / 61 and an activation kernel of 8 to 12; in a whole step of 128 rows 7.64 against 7.74 ms,
# of 192 rows 10.19 against 9.96); the head does not (128256 x 4096: 224 / 256 / 324 against
# 226 / 233 / 254; no difference in a whole step).  Matrices without a packed copy are read row by row, which
# the vendor's product does better from 65 rows on (a step of the 70B shape at 96 requests:
# 40.8 ms against 43.6) and up to 32 (24 requests: 30.4 against 32.7 ms, 32: 31.2 against 32.8;
# 48: 39.2 against 36.3, 64: the same).
MID_ROWS_UNPACKED = 64
MID_ROWS_UNPACKED_FROM = 33
MID_ROWS_GATED = 128
MID_ROWS_WIDE = 64


# Up to here the few-row kernel with the norms folded in is the fastest.  Measured at 16 rows
# against the kernels that share their rows through LDS: the 8B shape 4.13 against 4.45 ms a
# step, the 70B shape 30.4 against 32.6, the 1B shape 1.13 against 1.11.
FOLD_ROWS = 16


def mid_rows_ok(num_rows: int, packed: bool, most: int) -> bool:
    """Whether a product of ``num_rows`` rows by a matrix with or without a packed copy runs in
    the kernel that shares its rows through LDS (``most``: the kind of product's own limit)."""
    if packed:
        return FOLD_ROWS < num_rows <= most
    return MID_ROWS_UNPACKED_FROM <= num_rows <= min(most, MID_ROWS_UNPACKED)


def rows_fusable(num_rows: int, dtype: torch.dtype) -> bool:
    """Whether a step of ``num_rows`` tokens hands its norms to the products around them: up
    to 16 rows of bfloat16."""
    return dtype == torch.bfloat16 and 0 < num_rows <= FOLD_ROWS


def rows_sinkable(num_rows: int, dtype: torch.dtype) -> bool:
    """Whether a step of ``num_rows`` tokens sends the products before its norms into a
    :class:`ResidualSink` that finishes the norm itself: 17 to 192 rows."""
    return dtype == torch.bfloat16 and FOLD_ROWS < num_rows <= MID_ROWS


def skinny_blocks(N: int, K: int, gated: bool = False, packed: bool = False) -> int:
    """How many blocks of columns the weight-streaming kernel cuts ``N`` outputs into."""
    return int(load().kvc_gemm_skinny_blocks(N, K, int(gated), int(packed)))


def _fused_skinny(out: torch.Tensor | ResidualSink, x: torch.Tensor | ScaledRows, w: torch.Tensor,
                  bias: torch.Tensor | None, gated: bool, act: str = "silu") -> ScaledRows | None:
    """The weight-streaming product with a norm on either side folded in (see the C header);
    ``act`` is the gate's activation of the gated form."""
    data = x.data if isinstance(x, ScaledRows) else x
    M, K = data.shape
    N = w.shape[0] // 2 if gated else w.shape[0]
    if data.dtype != torch.bfloat16 or w.dtype != torch.bfloat16 or w.shape[1] != K:
        raise KernelError("fused product: operands must be bfloat16 of matching width")
    if not _skinny_operands_ok(data, w):
        raise KernelError("fused product: at most 64 rows, K a multiple of 8, 16-byte aligned operands")
    if bias is not None and (bias.dtype != torch.bfloat16 or bias.numel() != w.shape[0]):
        raise KernelError("fused product: bias must be bfloat16, one per weight row")
    in_ss = in_parts = in_width = 0
    in_eps = 0.0
    if isinstance(x, ScaledRows):
        in_parts = x.ss_parts.shape[1]
        if x.ss_parts.shape[0] < M or x.ss_parts.dtype != torch.float32 or not x.ss_parts.is_contiguous():
            raise KernelError("fused product: ss_parts must be contiguous float32 [>= T, parts]")
        in_ss, in_width, in_eps = x.ss_parts.data_ptr(), x.width, x.eps
    result = None
    if isinstance(out, ResidualSink):
        parts = skinny_blocks(N, K, packed=bool(_streamed(w, N)[1]))
        if out.residual.shape != (M, N) or out.residual.dtype != torch.float32 or out.residual.stride(1) != 1:
            raise KernelError("fused product: the residual must be float32 [T, N]")
        if out.gain.shape != (N,) or out.gain.dtype != torch.float32:
            raise KernelError("fused product: the gain must be float32 [N]")
        if out.out.shape != (M, N) or out.out.dtype != torch.bfloat16 or out.out.stride(1) != 1:
            raise KernelError("fused product: the sink's rows must be bfloat16 [T, N]")
        if out.ss_parts.numel() < M * parts or out.ss_parts.dtype != torch.float32 \
                or not out.ss_parts.is_contiguous():
            raise KernelError("fused product: the sink's ss_parts is too small")
        ss_view = out.ss_parts.view(-1)[: M * parts].view(M, parts)
        c_ptr, ldc = out.out.data_ptr(), out.out.stride(0)
        residual, ldr, gain, out_ss = (out.residual.data_ptr(), out.residual.stride(0),
                                       out.gain.data_ptr(), ss_view.data_ptr())
        result = ScaledRows(out.out, ss_view, N, out.eps)
    else:
        if out.shape != (M, N) or out.dtype != torch.bfloat16 or out.stride(1) != 1:
            raise KernelError("fused product: out must be bfloat16 [T, N]")
        c_ptr, ldc = out.data_ptr(), out.stride(0)
        residual = gain = out_ss = None
        ldr = 0
    if M:
        w_ptr, packed = _streamed(w, N)
        _check(load().kvc_gemm_skinny_fused_bf16(
            c_ptr, data.data_ptr(), w_ptr, None if bias is None else _dev(bias, "bias"), M, N, K,
            data.stride(0), ldc, (1 + _gate_act(act)) if gated else 0, in_ss or None, in_parts, in_width, float(in_eps),
            residual, ldr, gain, out_ss, packed, _stream()), "kvc_gemm_skinny_fused_bf16")
    return result


def skinny_operands_ok(x: torch.Tensor, w: torch.Tensor) -> bool:
    """Whether the weight-streaming product for few rows takes these operands."""
    return (x.shape[0] <= SKINNY_MAX_ROWS and x.shape[1] % 8 == 0 and x.stride(0) % 8 == 0
            and x.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0)


_skinny_operands_ok = skinny_operands_ok


def mid_slices_bound(N: int) -> int:
    """The most slices along K that ``gemm_mid`` cuts a weight with ``N`` rows into: blocks
    enough for 256 compute units, a block owning 64 weight rows, or 128 from 16,384 rows on
    (``plan_mid`` in csrc/gemm_mid.hip)."""
    rows_a_block = 128 if N >= 16384 else 64
    return min(64, -(-256 // -(-N // rows_a_block)))


def mid_slices(N: int, K: int) -> int:
    """Slices along K that ``gemm_mid`` cuts an [N, K] weight into when it may (see mode 2)."""
    return int(load().kvc_gemm_mid_slices(N, K))


def mid_operands_ok(x: torch.Tensor, w: torch.Tensor) -> bool:
    """Whether ``gemm_mid`` takes these operands (K a multiple of 512, aligned rows)."""
    return (x.shape[1] % 512 == 0 and x.stride(1) == 1 and x.stride(0) % 8 == 0 and w.is_contiguous()
            and x.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0)


def gemm_mid(out: torch.Tensor | None, x: torch.Tensor, w: torch.Tensor, bias: torch.Tensor | None = None,
             *, mode: int = 0, partial: torch.Tensor | None = None) -> None:
    """The weight-streaming product for up to 192 rows of bfloat16 whose waves share the rows
    through LDS, the faster one from 9 rows on (see the C header for the
    modes: 0 plain, 1 ``silu(gate) * up``, 2 partial sums of slices along K only, 3 plain
    with slices and a kernel that sums them, 4 ``gelu_tanh(gate) * up``)."""
    M, K = x.shape
    N = w.shape[0] // 2 if mode in (1, 4) else w.shape[0]
    if w.shape[1] != K or x.dtype != torch.bfloat16 or w.dtype != torch.bfloat16 or not x.is_cuda:
        raise KernelError("gemm_mid: operands must be bfloat16 GPU tensors with matching K")
    if not mid_operands_ok(x, w):
        raise KernelError("gemm_mid: K must be a multiple of 512 and the operands aligned")
    if bias is not None and (bias.dtype != torch.bfloat16 or bias.numel() != w.shape[0]):
        raise KernelError("gemm_mid: bias must be bfloat16, one value per weight row")
    out_ptr, ldc, code = None, N, 1
    if mode != 2:
        if out is None or out.shape != (M, N) or out.stride(1) != 1 or not out.is_cuda:
            raise KernelError("gemm_mid: out does not fit")
        out_ptr, ldc, code = out.data_ptr(), out.stride(0), _code(out, "out")
    part_ptr = None
    if partial is not None:
        if partial.dtype != torch.float32 or partial.numel() < mid_slices(N, K) * M * N:
            raise KernelError("gemm_mid: the buffer for partial sums is too small")
        part_ptr = _dev(partial, "partial", torch.float32)
    w_ptr, packed = _streamed(w, N)
    _check(load().kvc_gemm_mid_bf16(out_ptr, part_ptr, x.data_ptr(), w_ptr,
                                    None if bias is None else _dev(bias, "bias"), M, N, K, x.stride(0),
                                    ldc, code, mode, packed, _stream()), "kvc_gemm_mid_bf16")


def add_slices_rmsnorm(out: torch.Tensor, residual: torch.Tensor, partial: torch.Tensor, slices: int,
                       bias: torch.Tensor | None, weight: torch.Tensor, eps: float) -> None:
    """``residual += sum_s partial[s] (+ bias)``; ``out = rmsnorm(residual) * weight`` (see the
    C header); ``partial`` holds ``[slices, T, H]`` float32."""
    T, H = residual.shape
    if out.shape != (T, H) or not out.is_contiguous() or not residual.is_contiguous():
        raise KernelError("add_slices_rmsnorm: out and residual must be contiguous [T, H]")
    if partial.dtype != torch.float32 or partial.numel() < slices * T * H:
        raise KernelError("add_slices_rmsnorm: the partial sums do not fit")
    _check(load().kvc_add_slices_rmsnorm(
        _dev(out, "out"), _dev(residual, "residual", torch.float32), _dev(partial, "partial"), slices,
        None if bias is None else _dev(bias, "bias", torch.bfloat16), _dev(weight, "weight", torch.float32),
        float(eps), T, H, _code(out, "out"), _stream()), "kvc_add_slices_rmsnorm")


def _sink_mid(sink: ResidualSink, x: torch.Tensor, w: torch.Tensor, bias: torch.Tensor | None) -> NormedRows:
    """A product of 17 to 192 rows into a sink: partial sums of slices along K, then one kernel
    that adds them into the residual and normalises.  Shapes the weight-streaming kernel does
    not take run the vendor product into the same workspace first."""
    M, K = x.shape
    N = w.shape[0]
    if sink.slices is None or sink.slices.dtype != torch.float32:
        raise KernelError("linear: this sink needs its float32 workspace")
    if sink.residual.shape != (M, N) or sink.residual.dtype != torch.float32 or not sink.residual.is_contiguous():
        raise KernelError("linear: the sink's residual must be contiguous float32 [T, N]")
    if sink.out.shape != (M, N) or not sink.out.is_contiguous():
        raise KernelError("linear: the sink's rows must be contiguous [T, N]")
    # measured: the vendor product is as fast or faster once the output is wide and K is not
    # long (8192 x 8192), and slower for narrow outputs and long K (8192 x 28672: 139 against
    # 107 us at 64 rows; 4096 x 4096: 19 against 12)
    ours = (N < 8192 or K > 8192) and mid_rows_ok(M, bool(_streamed(w, N)[1]), MID_ROWS)
    if ours and x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and mid_operands_ok(x, w) and N % 8 == 0:
        slices = mid_slices(N, K)
        if sink.slices.numel() < slices * M * N:
            raise KernelError("linear: the sink's workspace is too small")
        gemm_mid(None, x, w, mode=2, partial=sink.slices)
        add_slices_rmsnorm(sink.out, sink.residual, sink.slices, slices, bias, sink.gain, sink.eps)
    else:
        if sink.slices.numel() * 2 < M * N:
            raise KernelError("linear: the sink's workspace is too small")
        tmp = sink.slices.view(-1).view(x.dtype)[: M * N].view(M, N)
        linear(tmp, x, w, bias)
        add_rmsnorm(sink.out, sink.residual, tmp, sink.gain, sink.eps)
    return NormedRows(sink.out)


def _slices_mid(sink: SliceSink, x: torch.Tensor, w: torch.Tensor, bias: torch.Tensor | None) -> SlicedRows:
    """A product of 17 to 192 rows whose float32 sums a norm consumes: partial sums of slices
    along K where the weight-streaming kernel takes the shape (as ``_sink_mid`` decides), else
    the unrounded product itself as the one slice."""
    M, K = x.shape
    N = w.shape[0]
    if sink.slices.dtype != torch.float32 or not sink.slices.is_contiguous():
        raise KernelError("linear: the room for partial sums must be contiguous float32")
    ours = (N < 8192 or K > 8192) and mid_rows_ok(M, bool(_streamed(w, N)[1]), MID_ROWS) \
        and (bias is None or (sink.takes_bias and bias.shape == (N,) and bias.is_contiguous()))
    if ours and x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and mid_operands_ok(x, w) and N % 8 == 0:
        slices = mid_slices(N, K)
        if sink.slices.numel() < slices * M * N:
            raise KernelError("linear: the room for partial sums is too small")
        gemm_mid(None, x, w, mode=2, partial=sink.slices)
        return SlicedRows(sink.slices, slices, M, N, bias)
    if sink.slices.numel() < M * N:
        raise KernelError("linear: the room for partial sums is too small")
    linear(sink.slices.view(-1)[: M * N].view(M, N), x, w, bias)
    return SlicedRows(sink.slices, 1, M, N)


def linear_silu_mul(out: torch.Tensor, x: torch.Tensor | ScaledRows, w: torch.Tensor,
                    bias: torch.Tensor | None, scratch, act: str = "silu") -> None:
    """``out = act(x @ wg.T) * (x @ wu.T)`` with ``wg`` the first half of ``w``'s rows and
    ``wu`` the second (biases likewise); ``act`` is ``silu`` or ``gelu_tanh``.  Few rows of
    bfloat16 run as one weight-streaming kernel; otherwise ``scratch()`` gives the ``[M, 2I]``
    buffer for the two-kernel form."""
    if isinstance(x, ScaledRows):
        _fused_skinny(out, x, w, bias, gated=True, act=act)
        return
    M, K = x.shape
    I = w.shape[0] // 2
    if w.shape != (2 * I, K) or out.shape != (M, I):
        raise KernelError("linear_silu_mul: shapes do not match")
    if (x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and out.dtype == torch.bfloat16
            and x.is_cuda and _skinny_operands_ok(x, w)
            and M <= FOLD_ROWS):
        if M == 0:
            return
        if bias is not None and (bias.dtype != torch.bfloat16 or bias.shape != (2 * I,)):
            raise KernelError("linear_silu_mul: bias must be bfloat16 [2I]")
        if act != "silu":
            _fused_skinny(out, x, w, bias, gated=True, act=act)
            return
        w_ptr, packed = _streamed(w, I)
        _check(load().kvc_gemm_skinny_silu_mul_bf16(
            out.data_ptr(), x.data_ptr(), w_ptr, None if bias is None else _dev(bias, "bias"),
            M, I, K, x.stride(0), out.stride(0), packed, _stream()), "kvc_gemm_skinny_silu_mul_bf16")
        return
    if (x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and out.dtype == torch.bfloat16
            and x.is_cuda and mid_operands_ok(x, w) and out.stride(1) == 1
            and mid_rows_ok(M, bool(_streamed(w, I)[1]), MID_ROWS_GATED)):
        # 17 to 128 rows: the waves of a block share the rows through LDS
        gemm_mid(out, x, w, bias, mode=4 if _gate_act(act) == 1 else 1)
        return
    gate_up = scratch()
    linear(gate_up, x, w, bias)
    silu_mul(out, gate_up, act)


def linear(out: torch.Tensor | ResidualSink, x: torch.Tensor | ScaledRows, w: torch.Tensor,
           bias: torch.Tensor | None = None) -> ScaledRows | None:
    """``out = x @ w.T (+ bias)``.  float32 runs the library's own true-float32 kernel.
    bfloat16 with few rows runs the weight-streaming matrix-core kernel; more rows run the
    vendor matrix product through torch.  All sum in float32, and a float32 ``out`` receives
    the sums unrounded on either path.  With a :class:`ScaledRows` for ``x`` or a :class:`ResidualSink` for ``out``
    (few rows of bfloat16 only) the norm before or after the product is folded into it; a
    sink returns the :class:`ScaledRows` it made, or, in a step of 17 to 192 rows, where it
    finishes the norm itself, :class:`NormedRows`."""
    if isinstance(out, SliceSink):
        if isinstance(x, ScaledRows):
            raise KernelError("linear: a product that leaves partial sums takes plain rows")
        return _slices_mid(out, x, w, bias)
    if isinstance(out, ResidualSink) and out.slices is not None:
        if isinstance(x, ScaledRows):
            raise KernelError("linear: a sink that finishes the norm itself takes plain rows")
        return _sink_mid(out, x, w, bias)
    if isinstance(x, ScaledRows) or isinstance(out, ResidualSink):
        return _fused_skinny(out, x, w, bias, gated=False)
    if x.dtype == torch.float32:
        gemm_f32(out, x, w, bias)
        return
    if x.dtype != torch.bfloat16 or w.dtype != torch.bfloat16 or not x.is_cuda:
        raise KernelError(f"linear: unsupported operands {x.dtype}/{w.dtype} on {x.device}")
    if x.shape[0] == 0:
        return
    M, K = x.shape
    N = w.shape[0]
    kernel = choose_product(M, N, K, few_rows_ok=_skinny_operands_ok(x, w),
                            shared_rows_ok=mid_operands_ok(x, w) and out.stride(1) == 1)
    if kernel == "few rows":
        gemm_skinny_bf16(out, x, w, bias)
        return
    if kernel == "shared rows":
        gemm_mid(out, x, w, bias, mode=0)
        return
    if out.dtype == torch.float32:
        # the vendor product with float32 sums stored as they are (no rounding to bfloat16)
        if out.stride(1) != 1 or not out.is_contiguous():
            raise KernelError("linear: a float32 result of bfloat16 operands must be contiguous")
        torch.mm(x, w.t(), out_dtype=torch.float32, out=out)
        if bias is not None:
            out.add_(bias)  # promoted to float32 on the way, no copy of the bias
        return
    if out.dtype != torch.bfloat16:
        raise KernelError(f"linear: unsupported result type {out.dtype}")
    if bias is None:
        torch.mm(x, w.t(), out=out)
    else:
        torch.addmm(bias, x, w.t(), out=out)


def linear_act(out: torch.Tensor, x: torch.Tensor, w: torch.Tensor, bias: torch.Tensor | None, act: str) -> None:
    """``out = act(x @ w.T (+ bias))`` with ``act`` one of :data:`ACTIVATIONS`, the product rounded
    to the model's dtype before the activation.  Few rows of bfloat16 take the weight-streaming
    kernel with the activation on its way out; every other shape the product and the activation
    kernel one after the other, which gives the same bits."""
    if act not in ACTIVATIONS:
        raise KernelError(f"unknown activation {act!r} (known: {sorted(ACTIVATIONS)})")
    M, K = x.shape
    N = w.shape[0]
    if (x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and out.dtype == torch.bfloat16 and x.is_cuda
            and M > 0 and out.shape == (M, N) and out.stride(1) == 1
            and choose_product(M, N, K, few_rows_ok=_skinny_operands_ok(x, w), shared_rows_ok=False) == "few rows"
            and (bias is None or (bias.dtype == torch.bfloat16 and bias.shape == (N,)))):
        w_ptr, packed = _streamed(w)
        _check(load().kvc_gemm_skinny_act_bf16(out.data_ptr(), x.data_ptr(), w_ptr,
                                               None if bias is None else _dev(bias, "bias"), M, N, K, x.stride(0),
                                               out.stride(0), ACTIVATIONS[act], packed, _stream()),
               "kvc_gemm_skinny_act_bf16")
        return
    linear(out, x, w, bias)
    activation(out, out, act)


def choose_product(M: int, N: int, K: int, *, few_rows_ok: bool = True, shared_rows_ok: bool = True) -> str:
    """Which kernel multiplies ``M`` rows of bfloat16 by an ``[N, K]`` matrix when nothing is
    folded into the product: ``"few rows"`` (``gemm_skinny_bf16``: every wave streams its own
    weight rows), ``"shared rows"`` (``gemm_mid``: the waves of a block share the rows through
    LDS) or ``"vendor"`` (the vendor's product through torch).  The one place where row counts
    and matrix sizes decide this; parts do not.  Measured on an MI355X with N x K from 4096 x
    4096 to 128256 x 4096 and 8192 x 28672: the few-row kernel wins up to 8 rows everywhere,
    up to 12 rows unless K is very long, up to 16 rows unless the output is as wide as a
    vocabulary, and up to 32 rows for small matrices; from 17 to 64 rows the shared-row
    kernel wins for outputs as wide as a vocabulary (215 against 231 us at 64 rows of 128256
    x 4096) and the vendor's product is as fast or faster otherwise, as it is beyond 64 rows.
    The flags say whether the operands' alignment and strides allow each kernel."""
    if few_rows_ok and M <= SKINNY_MAX_ROWS and (
            M <= 8 or (M <= 12 and K <= 8192) or (M <= SKINNY_PREFERRED_ROWS and K <= 8192 and N < 65536)
            or (M <= 32 and K <= 4096 and N <= 4096)):
        return "few rows"
    if shared_rows_ok and SKINNY_PREFERRED_ROWS < M <= MID_ROWS_WIDE and N >= 65536:
        return "shared rows"
    return "vendor"


def add_layernorm(out: torch.Tensor, residual: torch.Tensor, delta: torch.Tensor | None,
                  weight: torch.Tensor, bias: torch.Tensor | None, eps: float) -> None:
    """``residual += delta`` (float32, in place); ``out = (residual - mean) / sqrt(var + eps) *
    weight + bias`` with the variance as the mean of the squared deviations."""
    T, H = residual.shape
    if out.shape != (T, H) or weight.shape != (H,) or (delta is not None and delta.shape != (T, H)) \
            or (bias is not None and bias.shape != (H,)):
        raise KernelError("add_layernorm: shapes do not match")
    if delta is not None and delta.dtype != out.dtype:
        raise KernelError("add_layernorm: delta and out must share a dtype")
    _check(load().kvc_add_layernorm(_dev(out, "out"), _dev(residual, "residual", torch.float32),
                                    None if delta is None else _dev(delta, "delta"),
                                    _dev(weight, "weight", torch.float32),
                                    None if bias is None else _dev(bias, "bias", torch.float32),
                                    float(eps), T, H, _code(out, "out"), _stream()), "kvc_add_layernorm")


def rms_branches_mean(out: torch.Tensor, branches: list[tuple[torch.Tensor, torch.Tensor]], eps: float) -> None:
    """``out = mean_b(gain_b * x_b / rms(x_b))`` over up to four ``(x_b [T, H] float32, gain_b [H]
    float32)``, every branch divided by its own root mean square (``eps`` inside the root)."""
    T, H = out.shape
    n = len(branches)
    if not 1 <= n <= 4 or not out.is_contiguous():
        raise KernelError("rms_branches_mean: one to four branches, a contiguous result")
    xs = (c_void_p * n)()
    gs = (c_void_p * n)()
    for b, (x, g) in enumerate(branches):
        if x.shape != (T, H) or g.shape != (H,):
            raise KernelError("rms_branches_mean: shapes do not match")
        xs[b], gs[b] = _dev(x, "x", torch.float32), _dev(g, "gain", torch.float32)
    _check(load().kvc_rms_branches_mean(_dev(out, "out"), xs, gs, n, float(eps), T, H, _code(out, "out"),
                                        _stream()), "kvc_rms_branches_mean")


def concat2(out: torch.Tensor, a: torch.Tensor, b: torch.Tensor) -> None:
    """``out [T, 2H] = [a | b]`` from float32 ``a, b [T, H]``, rounded to ``out``'s dtype."""
    T, H = a.shape
    if b.shape != (T, H) or out.shape != (T, 2 * H):
        raise KernelError("concat2: shapes do not match")
    _check(load().kvc_concat2(_dev(out, "out"), _dev(a, "a", torch.float32), _dev(b, "b", torch.float32),
                              T, H, _code(out, "out"), _stream()), "kvc_concat2")


def add_row(x: torch.Tensor, v: torch.Tensor) -> None:
    """``x[t, :] += v`` on float32 rows."""
    T, H = x.shape
    if v.shape != (H,):
        raise KernelError("add_row: shapes do not match")
    _check(load().kvc_add_row(_dev(x, "x", torch.float32), _dev(v, "v", torch.float32), T, H, _stream()),
           "kvc_add_row")


def _rows(t: torch.Tensor, name: str, cols: int) -> tuple[int, int, int]:
    """(pointer, row stride, dtype code) of rows that may be columns of a wider tensor."""
    if t.dim() != 2 or t.stride(1) != 1 or t.shape[1] != cols or not t.is_cuda:
        raise KernelError(f"{name}: expects GPU rows of {cols} contiguous elements, got {tuple(t.shape)}")
    return t.data_ptr(), t.stride(0), _code(t, name)


def causal_conv(out: torch.Tensor, x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor | None,
                state: torch.Tensor, *, positions: torch.Tensor, token_req: torch.Tensor,
                q_start: torch.Tensor, slots: torch.Tensor, num_reqs: int, act: str = "none",
                update_state: bool = True, single_tokens: bool = False) -> None:
    """Causal convolution per channel over each request's tokens (see the C header): ``x [T, C]``
    (a column view is fine), ``weight [C, K]`` float32 with the last column the current token's,
    ``state [slots, K-1, C]`` float32 (read, and with ``update_state`` rewritten).
    ``single_tokens``: every request brings exactly one token, which lets one kernel do both."""
    T, C = x.shape
    K = weight.shape[1]
    if weight.shape != (C, K) or (bias is not None and bias.shape != (C,)):
        raise KernelError("causal_conv: weight or bias does not fit")
    if state.dim() != 3 or tuple(state.shape[1:]) != (K - 1, C) or state.dtype != torch.float32:
        raise KernelError("causal_conv: state must be float32 [slots, K-1, C]")
    if out.shape[0] != T or positions.numel() < T or token_req.numel() < T or q_start.numel() < num_reqs + 1:
        raise KernelError("causal_conv: index arrays or out too short")
    o_ptr, o_stride, o_code = _rows(out, "out", C)
    x_ptr, x_stride, x_code = _rows(x, "x", C)
    _check(load().kvc_causal_conv(
        o_ptr, o_stride, o_code, x_ptr, x_stride, x_code, _dev(weight, "weight", torch.float32),
        None if bias is None else _dev(bias, "bias", torch.float32), _dev(state, "state"),
        _dev(positions, "positions", torch.int32), _dev(token_req, "token_req", torch.int32),
        _dev(q_start, "q_start", torch.int32), _dev(slots, "slots", torch.int32), T, num_reqs, C, K,
        {"none": 0, "silu": 1}[act], int(update_state), int(bool(single_tokens)), _stream()), "kvc_causal_conv")


def rglru_gates(a_out: torch.Tensor, drive: torch.Tensor, u: torch.Tensor, wa: torch.Tensor,
                wi: torch.Tensor, ba: torch.Tensor, bi: torch.Tensor, lam: torch.Tensor,
                c_decay: float) -> None:
    """Decay ``a = exp(-c_decay * sigmoid(wa u + ba) * softplus(lam))`` and driven input
    ``sqrt(1 - a^2) * sigmoid(wi u + bi) * u`` of the gated linear recurrent unit, the gate
    matrices block-diagonal ``[blocks, W/blocks, W/blocks]``; everything float32."""
    T, W = u.shape
    nb = wa.shape[0]
    if W % nb or wa.shape != (nb, W // nb, W // nb) or wi.shape != wa.shape:
        raise KernelError("rglru_gates: gate matrices do not fit")
    if a_out.shape != (T, W) or drive.shape != (T, W) or ba.numel() != W or bi.numel() != W or lam.numel() != W:
        raise KernelError("rglru_gates: shapes do not match")
    f = torch.float32
    _check(load().kvc_rglru_gates(_dev(a_out, "a_out", f), _dev(drive, "drive", f), _dev(u, "u", f),
                                  _dev(wa, "wa", f), _dev(wi, "wi", f), _dev(ba, "ba", f), _dev(bi, "bi", f),
                                  _dev(lam, "lam", f), float(c_decay), T, W, nb, _stream()), "kvc_rglru_gates")


def rglru_scan_workspace_floats(num_reqs: int, width: int, max_query_len: int) -> int:
    """float32 values of workspace with which ``rglru_scan`` works on the segments of long
    portions side by side (0: the portions are too short to gain from it)."""
    seg = int(load().kvc_rglru_scan_segment())
    segs = -(-max_query_len // seg)
    return 0 if segs <= 1 else num_reqs * (segs + 1) * 2 * width


def rglru_scan(out: torch.Tensor, a: torch.Tensor, drive: torch.Tensor, y: torch.Tensor,
               state: torch.Tensor, *, positions: torch.Tensor, token_req: torch.Tensor,
               q_start: torch.Tensor, slots: torch.Tensor, num_reqs: int, max_query_len: int = 0,
               workspace: torch.Tensor | None = None) -> None:
    """``S_t = a_t S_(t-1) + drive_t`` per channel along each request, ``out[t] = S_t *
    gelu_tanh(y[t])``; ``state [slots, W]`` float32 is read (a request at position 0 starts
    from zero) and rewritten.  With ``max_query_len`` (a bound on a request's tokens in this
    step) and a float32 ``workspace`` of ``rglru_scan_workspace_floats`` values, long portions
    are scanned in segments side by side."""
    T, W = a.shape
    if drive.shape != (T, W) or out.shape != (T, W) or not out.is_contiguous() or state.shape[1:] != (W,):
        raise KernelError("rglru_scan: shapes do not match")
    y_ptr, y_stride, y_code = _rows(y, "y", W)
    _check(load().kvc_rglru_scan(
        _dev(out, "out"), _code(out, "out"), _dev(a, "a", torch.float32), _dev(drive, "drive", torch.float32),
        y_ptr, y_stride, y_code, _dev(state, "state", torch.float32),
        _dev(positions, "positions", torch.int32), _dev(token_req, "token_req", torch.int32),
        _dev(q_start, "q_start", torch.int32), _dev(slots, "slots", torch.int32), num_reqs, W,
        int(max_query_len), None if workspace is None else _dev(workspace, "workspace", torch.float32),
        0 if workspace is None else workspace.numel(), _stream()), "kvc_rglru_scan")


def ssm_scan_max_state() -> int:
    return int(load().kvc_ssm_scan_max_state())


def ssm_scan(y: torch.Tensor, xbc: torch.Tensor, dt_raw: torch.Tensor, dt_bias: torch.Tensor,
             a_log: torch.Tensor, d_skip: torch.Tensor, state: torch.Tensor, *, positions: torch.Tensor,
             token_req: torch.Tensor, q_start: torch.Tensor, slots: torch.Tensor, num_reqs: int,
             heads: int, head_dim: int, state_size: int, groups: int) -> None:
    """The state-space recurrence with a scalar decay per head (see the C header): ``xbc [T, heads
    * head_dim + 2 * groups * state_size]`` float32 (x, B, C after their convolution), ``dt_raw
    [T, heads]`` (a column view is fine), ``state [slots, heads, state_size, head_dim]`` float32,
    ``y [T, heads * head_dim]`` float32."""
    T = xbc.shape[0]
    inner = heads * head_dim
    if y.shape != (T, inner) or not y.is_contiguous() or y.dtype != torch.float32:
        raise KernelError("ssm_scan: y must be contiguous float32 [T, heads * head_dim]")
    if tuple(state.shape[1:]) != (heads, state_size, head_dim) or state.dtype != torch.float32:
        raise KernelError("ssm_scan: state must be float32 [slots, heads, state_size, head_dim]")
    if dt_bias.numel() != heads or a_log.numel() != heads or d_skip.numel() != heads:
        raise KernelError("ssm_scan: a value per head for dt_bias, a_log and d_skip")
    x_ptr, x_stride, x_code = _rows(xbc, "xbc", inner + 2 * groups * state_size)
    if x_code != 0:
        raise KernelError("ssm_scan: xbc must be float32")
    d_ptr, d_stride, d_code = _rows(dt_raw, "dt_raw", heads)
    f = torch.float32
    _check(load().kvc_ssm_scan(
        y.data_ptr(), x_ptr, x_stride, d_ptr, d_stride, d_code, _dev(dt_bias, "dt_bias", f),
        _dev(a_log, "a_log", f), _dev(d_skip, "d_skip", f), _dev(state, "state"),
        _dev(positions, "positions", torch.int32), _dev(token_req, "token_req", torch.int32),
        _dev(q_start, "q_start", torch.int32), _dev(slots, "slots", torch.int32), num_reqs, heads,
        head_dim, state_size, groups, _stream()), "kvc_ssm_scan")


def gated_group_rmsnorm(out: torch.Tensor, y: torch.Tensor, z: torch.Tensor, gain: torch.Tensor,
                        eps: float, groups: int) -> None:
    """``out = gain * v / rms_part(v)`` with ``v = y * silu(z)``: the gate first, then the norm
    in ``groups`` equal parts of the width.  ``y`` float32, ``z`` a column view of any dtype."""
    T, width = y.shape
    if out.shape != (T, width) or not out.is_contiguous() or not y.is_contiguous() or gain.shape != (width,):
        raise KernelError("gated_group_rmsnorm: shapes do not match")
    z_ptr, z_stride, z_code = _rows(z, "z", width)
    _check(load().kvc_gated_group_rmsnorm(
        _dev(out, "out"), _code(out, "out"), _dev(y, "y", torch.float32), z_ptr, z_stride, z_code,
        _dev(gain, "gain", torch.float32), float(eps), T, width, groups, _stream()),
        "kvc_gated_group_rmsnorm")


def _f32_rows(t: torch.Tensor, name: str, cols: int) -> tuple[int, int]:
    ptr, stride, code = _rows(t, name, cols)
    if code != 0:
        raise KernelError(f"{name} must be float32")
    return ptr, stride


def linear_state_rows(dim: int) -> int:
    """Rows of a head's state as ``linear_state_scan`` keeps it: ``dim`` rounded up to a multiple of 4
    (the kernel lays the rows out in fours)."""
    return -(-dim // 4) * 4


def linear_state_scan(out: torch.Tensor, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor,
                      decay: torch.Tensor, beta: torch.Tensor | None, state: torch.Tensor, *,
                      positions: torch.Tensor, token_req: torch.Tensor, q_start: torch.Tensor,
                      slots: torch.Tensor, num_reqs: int, heads: int, qk_heads: int, dim: int,
                      vdim: int, delta_rule: bool = False, q_scale: float = 1.0,
                      scalar_gates: bool = False, ones_column: bool = False) -> None:
    """The recurrence of a matrix state per head (see the C header): ``q, k [T, qk_heads * dim]``,
    ``v [T, heads * vdim]``, all float32 rows (column views are fine); ``decay [T, heads * dim]``
    (a factor per key channel) or, with ``delta_rule``, ``decay`` and ``beta [T, heads]``; with
    ``scalar_gates`` the rule is ``S <- decay S + beta k v^T`` with the same two ``[T, heads]``;
    with ``ones_column`` ``v`` is ``[T, heads * (vdim - 1)]`` and the last of a head's ``vdim``
    columns takes a one for every token (a normaliser beside the matrix);
    ``state [slots, heads, linear_state_rows(dim), vdim]`` float32, in an order of the kernel's own;
    ``out [T, heads * vdim]`` float32.  ``q_scale``
    multiplies every q on its way in."""
    T = out.shape[0]
    if out.shape != (T, heads * vdim) or not out.is_contiguous() or out.dtype != torch.float32:
        raise KernelError("linear_state_scan: out must be contiguous float32 [T, heads * vdim]")
    if tuple(state.shape[1:]) != (heads, linear_state_rows(dim), vdim) or state.dtype != torch.float32 \
            or not state.is_contiguous():
        raise KernelError("linear_state_scan: state must be float32 [slots, heads, linear_state_rows(dim), vdim]")
    if min(q.shape[0], k.shape[0], v.shape[0], decay.shape[0]) < T or positions.numel() < T \
            or token_req.numel() < T or q_start.numel() < num_reqs + 1:
        raise KernelError("linear_state_scan: rows or index arrays too short")
    qp, qs = _f32_rows(q, "q", qk_heads * dim)
    kp, ks = _f32_rows(k, "k", qk_heads * dim)
    vp, vs = _f32_rows(v, "v", heads * (vdim - 1 if ones_column else vdim))
    if delta_rule and scalar_gates:
        raise KernelError("linear_state_scan: one rule at a time")
    per_head = delta_rule or scalar_gates
    dp, ds = _f32_rows(decay, "decay", heads if per_head else heads * dim)
    bp, bs = (0, 0)
    if per_head:
        if beta is None or beta.shape[0] < T:
            raise KernelError("linear_state_scan: this rule needs beta")
        bp, bs = _f32_rows(beta, "beta", heads)
    _check(load().kvc_linear_state_scan(
        out.data_ptr(), qp, qs, kp, ks, vp, vs, dp, ds, bp or None, bs, _dev(state, "state"),
        _dev(positions, "positions", torch.int32), _dev(token_req, "token_req", torch.int32),
        _dev(q_start, "q_start", torch.int32), _dev(slots, "slots", torch.int32), num_reqs, heads,
        qk_heads, dim, vdim, 2 if scalar_gates else int(bool(delta_rule)), float(q_scale), int(bool(ones_column)),
        _stream()),
        "kvc_linear_state_scan")


def sigmoid_power(out: torch.Tensor, z: torch.Tensor, bias: torch.Tensor | None, inv_tau: float) -> None:
    """``out = sigmoid(z + bias) ** inv_tau`` in float32 (through the logarithm)."""
    T, W = out.shape
    if not out.is_contiguous() or out.dtype != torch.float32 or z.shape[0] < T or (bias is not None and bias.shape != (W,)):
        raise KernelError("sigmoid_power: shapes do not match")
    zp, zs = _f32_rows(z, "z", W)
    _check(load().kvc_sigmoid_power(out.data_ptr(), zp, zs, None if bias is None else _dev(bias, "bias", torch.float32),
                                    float(inv_tau), T, W, _stream()), "kvc_sigmoid_power")


def decay_and_write_gates(g: torch.Tensor, beta: torch.Tensor, a_raw: torch.Tensor, b_raw: torch.Tensor,
                          a_log: torch.Tensor, dt_bias: torch.Tensor) -> None:
    """``g = exp(-exp(a_log) * softplus(a_raw + dt_bias))``, ``beta = sigmoid(b_raw)``, float32 ``[T, heads]``."""
    T, nh = g.shape
    if beta.shape != (T, nh) or a_log.shape != (nh,) or dt_bias.shape != (nh,) or a_raw.shape[0] < T or b_raw.shape[0] < T:
        raise KernelError("decay_and_write_gates: shapes do not match")
    ap, as_ = _f32_rows(a_raw, "a_raw", nh)
    bp, bs = _f32_rows(b_raw, "b_raw", nh)
    f = torch.float32
    _check(load().kvc_decay_and_write_gates(_dev(g, "g", f), _dev(beta, "beta", f), ap, as_, bp, bs,
                                            _dev(a_log, "a_log", f), _dev(dt_bias, "dt_bias", f), T, nh, _stream()),
           "kvc_decay_and_write_gates")


def unit_heads(x: torch.Tensor, heads: int, dim: int, eps: float, scale: float = 1.0, first_heads: int = 0,
               first_scale: float = 1.0) -> None:
    """Every head of ``dim`` values of the float32 rows ``x [T, heads * dim]`` (a column view is
    fine) over its Euclidean length (``eps`` inside the root), times ``scale`` (the first
    ``first_heads`` heads times ``first_scale`` instead), in place."""
    xp, xs = _f32_rows(x, "x", heads * dim)
    _check(load().kvc_unit_heads(xp, xs, x.shape[0], heads, dim, float(eps), float(scale), int(first_heads),
                                 float(first_scale), _stream()), "kvc_unit_heads")


def head_rmsnorm_gate(out: torch.Tensor, o: torch.Tensor, gate: torch.Tensor, gain: torch.Tensor, eps: float,
                      heads: int, vdim: int) -> None:
    """``out = o / rms_head(o) * gain * silu(gate)``: every head of ``vdim`` values of the float32
    ``o [T, heads * vdim]`` over its root mean square, times ``gain [vdim]`` (shared by the heads),
    times the gate (rows of any dtype, a column view is fine)."""
    T = o.shape[0]
    if o.shape != (T, heads * vdim) or out.shape != o.shape or not out.is_contiguous() or not o.is_contiguous() \
            or gain.shape != (vdim,):
        raise KernelError("head_rmsnorm_gate: shapes do not match")
    gp, gs, gc = _rows(gate, "gate", heads * vdim)
    _check(load().kvc_head_rmsnorm_gate(_dev(out, "out"), _code(out, "out"), _dev(o, "o", torch.float32), gp, gs, gc,
                                        _dev(gain, "gain", torch.float32), float(eps), T, heads, vdim, _stream()),
           "kvc_head_rmsnorm_gate")


def max_gates(keep: torch.Tensor, take: torch.Tensor, m_out: torch.Tensor, i_raw: torch.Tensor,
              f_raw: torch.Tensor, i_bias: torch.Tensor, f_bias: torch.Tensor, cap: float,
              m_state: torch.Tensor, *, positions: torch.Tensor, token_req: torch.Tensor,
              q_start: torch.Tensor, slots: torch.Tensor, num_reqs: int) -> None:
    """The gates of a matrix memory with log gates and a running maximum, per request in token
    order (see the C header): ``keep, take, m_out [T, heads]`` float32 from the raw gate rows
    ``i_raw, f_raw`` (float32, column views are fine); ``m_state [slots, heads]`` float32."""
    T, nh = keep.shape
    f = torch.float32
    if take.shape != (T, nh) or m_out.shape != (T, nh) or i_bias.shape != (nh,) or f_bias.shape != (nh,) \
            or m_state.dim() != 2 or m_state.shape[1] != nh or not m_state.is_contiguous() \
            or i_raw.shape[0] < T or f_raw.shape[0] < T or q_start.numel() < num_reqs + 1:
        raise KernelError("max_gates: shapes do not match")
    for t in (keep, take, m_out):
        if not t.is_contiguous():
            raise KernelError("max_gates: the results must be contiguous")
    ip, is_ = _f32_rows(i_raw, "i_raw", nh)
    fp, fs = _f32_rows(f_raw, "f_raw", nh)
    _check(load().kvc_max_gates(
        _dev(keep, "keep", f), _dev(take, "take", f), _dev(m_out, "m_out", f), ip, is_, fp, fs,
        _dev(i_bias, "i_bias", f), _dev(f_bias, "f_bias", f), float(cap), _dev(m_state, "m_state", f),
        _dev(positions, "positions", torch.int32), _dev(token_req, "token_req", torch.int32),
        _dev(q_start, "q_start", torch.int32), _dev(slots, "slots", torch.int32), T, num_reqs, nh, _stream()),
        "kvc_max_gates")


def max_gated_finish(out: torch.Tensor, o: torch.Tensor, m: torch.Tensor, gate: torch.Tensor,
                     gain: torch.Tensor, eps: float, den_eps: float, heads: int, vdim: int) -> None:
    """``y = o[..., :vdim] / (max(|o[..., vdim]|, exp(-m)) + den_eps)``; ``out = y / rms_head(y) *
    gain * sigmoid(gate)``: ``o [T, heads * (vdim + 1)]`` float32 (the last column of a head is
    the normaliser's product with the query), ``m [T, heads]``, ``gain [heads * vdim]``, the gate
    rows of any dtype (a column view is fine)."""
    T = o.shape[0]
    if o.shape != (T, heads * (vdim + 1)) or out.shape != (T, heads * vdim) or not out.is_contiguous() \
            or not o.is_contiguous() or gain.shape != (heads * vdim,) or m.shape != (T, heads) or not m.is_contiguous():
        raise KernelError("max_gated_finish: shapes do not match")
    gp, gs, gc = _rows(gate, "gate", heads * vdim)
    _check(load().kvc_max_gated_finish(
        _dev(out, "out"), _code(out, "out"), _dev(o, "o", torch.float32), _dev(m, "m", torch.float32), gp, gs, gc,
        _dev(gain, "gain", torch.float32), float(eps), float(den_eps), T, heads, vdim, _stream()),
        "kvc_max_gated_finish")


def norm_add_norm(out: torch.Tensor | None, residual: torch.Tensor, delta: "torch.Tensor | SlicedRows",
                  post_gain: torch.Tensor, eps: float, next_gain: torch.Tensor | None = None,
                  next_eps: float | None = None) -> None:
    """``residual += post_gain * delta / rms(delta)``, then, given ``out``, ``out = next_gain *
    residual / rms(residual)``: the norm behind a sublayer, the sum into the float32 stream and the
    norm before the next sublayer in one pass (both roots hold their eps).  ``delta`` is float32
    or bfloat16, or the :class:`SlicedRows` that a product left (their sum is the result)."""
    T, H = residual.shape
    slices = 1
    if isinstance(delta, SlicedRows):
        if delta.bias is not None:
            raise KernelError("norm_add_norm: partial sums whose bias is still to be added")
        if (delta.rows, delta.width) != (T, H) or delta.data.dtype != torch.float32 \
                or delta.data.numel() < delta.count * T * H or not delta.data.is_contiguous():
            raise KernelError("norm_add_norm: the partial sums do not fit")
        slices, delta = delta.count, delta.data
    elif delta.shape != (T, H) or not delta.is_contiguous():
        raise KernelError("norm_add_norm: shapes do not match")
    if not residual.is_contiguous() or post_gain.shape != (H,):
        raise KernelError("norm_add_norm: shapes do not match")
    if out is not None and (out.shape != (T, H) or not out.is_contiguous() or next_gain is None
                            or next_gain.shape != (H,)):
        raise KernelError("norm_add_norm: the second norm's rows or gain do not fit")
    _check(load().kvc_norm_add_norm(
        None if out is None else _dev(out, "out"), 0 if out is None else _code(out, "out"),
        _dev(residual, "residual", torch.float32), _dev(delta, "delta"), _code(delta, "delta"),
        _dev(post_gain, "post_gain", torch.float32), float(eps),
        None if out is None else _dev(next_gain, "next_gain", torch.float32),
        float(eps if next_eps is None else next_eps), T, H, slices, _stream()), "kvc_norm_add_norm")


def wide_qk_norm(qkv: torch.Tensor, q_gain: torch.Tensor, k_gain: torch.Tensor, eps: float, *,
                 copy_k: bool = False) -> None:
    """Rows of ``qkv`` start with all query heads (as many values as ``q_gain`` has) and all key
    heads (``k_gain``): each of the two runs is divided by its root mean square as a whole and
    multiplied by its gain, in place.  With ``copy_k`` the keys as they were are first copied
    behind themselves (where a layer's values are its keys as projected)."""
    nq, nk = q_gain.numel(), k_gain.numel()
    if qkv.dim() != 2 or qkv.stride(1) != 1 or qkv.shape[1] < nq + nk * (2 if copy_k else 1):
        raise KernelError("wide_qk_norm: rows too short")
    _check(load().kvc_wide_qk_norm(qkv.data_ptr(), qkv.stride(0), _dev(q_gain, "q_gain", torch.float32),
                                   _dev(k_gain, "k_gain", torch.float32), float(eps), qkv.shape[0], nq, nk,
                                   int(bool(copy_k)), _code(qkv, "qkv"), _stream()), "kvc_wide_qk_norm")


def latent_rows(cq: torch.Tensor | None, key: torch.Tensor, value: torch.Tensor, down: torch.Tensor,
                q_gain: torch.Tensor | None, kv_gain: torch.Tensor, eps: float, rot: int) -> None:
    """From rows ``down = [query latent | key/value latent | rot rotated key elements | ...]``: the
    query latent normed with ``q_gain`` into ``cq``; ``[rotated elements as they are | key/value
    latent normed with kv_gain]`` into ``key`` and into ``value`` (column views of one buffer with
    equal row strides are fine).  All of one dtype; the norms are float32."""
    T = down.shape[0]
    q_rank, rank = (0 if q_gain is None else q_gain.numel()), kv_gain.numel()
    if (cq is None) != (q_gain is None):
        raise KernelError("latent_rows: a query latent has rows and a gain, or neither")
    for t, cols in ((cq, q_rank), (key, rank + rot), (value, rank + rot)):
        if t is None:
            continue
        if t.dim() != 2 or t.shape != (T, cols) or t.stride(1) != 1 or t.dtype != down.dtype:
            raise KernelError("latent_rows: results do not fit")
    if down.stride(1) != 1 or down.shape[1] < q_rank + rank + rot or key.stride(0) != value.stride(0):
        raise KernelError("latent_rows: rows too short, or keys and values with different strides")
    _check(load().kvc_latent_rows(None if cq is None else cq.data_ptr(), 0 if cq is None else cq.stride(0),
                                  key.data_ptr(), value.data_ptr(), key.stride(0), down.data_ptr(), down.stride(0),
                                  None if q_gain is None else _dev(q_gain, "q_gain", torch.float32),
                                  _dev(kv_gain, "kv_gain", torch.float32), float(eps), T, q_rank, rank, int(rot),
                                  _code(down, "down"), _stream()), "kvc_latent_rows")


def head_gate(out: torch.Tensor, x: torch.Tensor, gate: torch.Tensor, *, heads: int, head_stride: int,
              skip: int, n: int) -> None:
    """``out[t, h, :n] = x[t, h, skip : skip + n] * sigmoid(gate[t, h])``: ``x`` rows of ``heads`` heads of
    ``head_stride`` values, ``gate`` rows of ``heads`` values (column views are fine),
    ``out [T, heads * n]``, all of one dtype."""
    T = out.shape[0]
    if out.shape != (T, heads * n) or not out.is_contiguous() or out.dtype != x.dtype or x.stride(1) != 1 \
            or x.shape[0] < T or x.shape[1] < heads * head_stride or gate.shape[0] < T:
        raise KernelError("head_gate: shapes do not match")
    gp, gs, gc = _rows(gate, "gate", heads)
    if gc != _code(x, "x"):
        raise KernelError("head_gate: the gate has another dtype than the rows")
    _check(load().kvc_head_gate(out.data_ptr(), x.data_ptr(), x.stride(0), gp, gs, T, heads, head_stride, skip, n,
                                _code(out, "out"), _stream()), "kvc_head_gate")


ROUTE_SCORES = {"softmax": 0, "sigmoid": 1}  # how a router's logits become scores


def _route_rule(E: int, score: str, correction: torch.Tensor | None, group_best: int,
                weight_scale: float) -> tuple[int, int | None, int, float]:
    if score not in ROUTE_SCORES:
        raise KernelError(f"unknown router score {score!r} (known: {sorted(ROUTE_SCORES)})")
    if correction is not None and (correction.shape != (E,) or correction.dtype != torch.float32):
        raise KernelError("moe routing: the correction is float32 [experts]")
    if group_best not in (1, 2):
        raise KernelError("moe routing: a group is worth its best choice score or the sum of its best two")
    return (ROUTE_SCORES[score], None if correction is None else _dev(correction, "correction"), int(group_best),
            float(weight_scale))


def moe_route(choice: torch.Tensor, weight: torch.Tensor, logits: torch.Tensor, *, top: int, groups: int = 1,
              keep: int = 1, score: str = "softmax", correction: torch.Tensor | None = None, group_best: int = 1,
              weight_scale: float = 1.0) -> None:
    """The router's choice from float32 ``logits [T, E]``: ``choice`` (int32) and ``weight``
    (float32), both ``[T, top]``.  ``score``: ``softmax`` over the experts or a ``sigmoid`` of each
    logit; ``correction`` (float32 ``[E]``) joins the scores for the choice alone; a group is worth
    its ``group_best`` (1 or 2) best choice scores; the weights (the chosen experts' plain scores
    over their sum) are multiplied by ``weight_scale``."""
    T, E = logits.shape
    if choice.shape != (T, top) or weight.shape != (T, top):
        raise KernelError("moe_route: shapes do not match")
    _check(load().kvc_moe_route(_dev(choice, "choice", torch.int32), _dev(weight, "weight", torch.float32),
                                _dev(logits, "logits", torch.float32), T, E, top, groups, keep,
                                *_route_rule(E, score, correction, group_best, weight_scale), _stream()),
           "kvc_moe_route")


def moe_router(choice: torch.Tensor, weight: torch.Tensor, x: torch.Tensor, router: torch.Tensor, *, top: int,
               groups: int = 1, keep: int = 1, score: str = "softmax", correction: torch.Tensor | None = None,
               group_best: int = 1, weight_scale: float = 1.0) -> None:
    """``moe_route`` of the logits ``x @ router.T`` (float32 sums in one fixed order; ``x [T, H]`` of
    either dtype, ``router [E, H]`` float32) without storing the logits."""
    T, H = x.shape
    E = router.shape[0]
    if router.shape != (E, H) or choice.shape != (T, top) or weight.shape != (T, top) or x.stride(1) != 1:
        raise KernelError("moe_router: shapes do not match")
    _check(load().kvc_moe_router(_dev(choice, "choice", torch.int32), _dev(weight, "weight", torch.float32),
                                 x.data_ptr(), x.stride(0), _code(x, "x"), _dev(router, "router", torch.float32),
                                 T, H, E, top, groups, keep,
                                 *_route_rule(E, score, correction, group_best, weight_scale), _stream()),
           "kvc_moe_router")


def moe_tile_rows(pairs: int, experts: int, x: torch.Tensor | None = None, k_sizes: tuple[int, ...] = ()) -> int:
    """Rows a tile of the experts' products holds for a step of this size: 64 where the experts
    have that many rows on average and the operands allow (bfloat16, every K a multiple of 32), else 16."""
    rows = int(load().kvc_moe_tile_rows(pairs, experts))
    if rows > 16 and (x is None or x.dtype != torch.bfloat16 or any(k % 32 for k in k_sizes)):
        return 16
    return rows


def moe_max_tiles(pairs: int, experts: int, tile_rows: int = 16) -> int:
    return int(load().kvc_moe_max_tiles(pairs, experts, tile_rows))


def moe_align(sorted_pairs: torch.Tensor, tiles: torch.Tensor, num_tiles: torch.Tensor, choice: torch.Tensor,
              experts: int, tile_rows: int = 16) -> None:
    """(token, choice) pairs sorted by expert, and the list of row tiles (``tiles [>= max_tiles, 3]``)
    of up to ``tile_rows`` rows."""
    pairs = choice.numel()
    if sorted_pairs.numel() < pairs or tiles.dim() != 2 or tiles.shape[1] != 3 or num_tiles.numel() < 1:
        raise KernelError("moe_align: buffers too small")
    _check(load().kvc_moe_align(_dev(sorted_pairs, "sorted", torch.int32), _dev(tiles, "tiles", torch.int32),
                                _dev(num_tiles, "num_tiles", torch.int32), _dev(choice, "choice", torch.int32),
                                pairs, experts, tiles.shape[0], tile_rows, _stream()), "kvc_moe_align")


def moe_gemm(out: torch.Tensor, x: torch.Tensor, w: torch.Tensor, sorted_pairs: torch.Tensor, tiles: torch.Tensor,
             num_tiles: torch.Tensor, *, pairs: int, experts: int, in_div: int, out_sorted: bool, gated: bool,
             limit: float = 0.0, alpha: float = 0.0, up_shift: float = 1.0, tile_rows: int = 16) -> None:
    """Every expert's product over its own rows.  ``w`` is ``[experts * N, K]`` (``experts * 2N``
    rows when ``gated``: each expert's gate rows, then its up rows); ``out [pairs, N]``.  The gated
    form stores ``min(g, limit) * sigmoid(alpha * g) * (clamp(u, -limit, limit) + up_shift)``."""
    N = out.shape[1]
    K = x.shape[1]
    rows = experts * N * (2 if gated else 1)
    if w.shape != (rows, K) or out.shape[0] < pairs or x.dtype != w.dtype or out.stride(1) != 1 or x.stride(1) != 1:
        raise KernelError("moe_gemm: shapes do not match")
    max_tiles = min(tiles.shape[0], moe_max_tiles(pairs, experts, tile_rows))
    # the bfloat16 kernels read the packed twin of the experts' matrix where the model keeps one
    w_ptr, packed = (_streamed(w, N) if N % 16 == 0 and K % 64 == 0 else (_dev(w, "w"), 0))
    _check(load().kvc_moe_gemm(out.data_ptr(), out.stride(0), _code(out, "out"), x.data_ptr(), x.stride(0),
                               w_ptr, _code(x, "x"), _dev(sorted_pairs, "sorted", torch.int32),
                               _dev(tiles, "tiles", torch.int32), _dev(num_tiles, "num_tiles", torch.int32),
                               max_tiles, tile_rows, N, K, int(in_div), int(bool(out_sorted)), int(bool(gated)),
                               float(limit), float(alpha), float(up_shift), packed, _stream()), "kvc_moe_gemm")


def moe_combine(out: torch.Tensor, y: torch.Tensor, weight: torch.Tensor, add0: torch.Tensor | None = None,
                add1: torch.Tensor | None = None, accumulate: bool = False) -> None:
    """``out[t] = sum_c weight[t, c] * y[t * top + c] (+ add0[t]) (+ add1[t])``, float32; ``add0``
    of either dtype, ``add1`` float32.  ``accumulate``: the sum is added into ``out``."""
    T, H = out.shape
    top = weight.shape[1] if weight.dim() == 2 else 0
    if out.dtype != torch.float32 or (top and (y.shape[0] < T * top or y.shape[1] != H)):
        raise KernelError("moe_combine: shapes do not match")
    for a in (add0, add1):
        if a is not None and a.shape != (T, H):
            raise KernelError("moe_combine: an added row set does not fit")
    _check(load().kvc_moe_combine(_dev(out, "out"), _dev(y, "y", torch.float32), _dev(weight, "weight", torch.float32),
                                  top, None if add0 is None else _dev(add0, "add0"),
                                  0 if add0 is None else _code(add0, "add0"),
                                  None if add1 is None else _dev(add1, "add1", torch.float32), T, H,
                                  int(bool(accumulate)), _stream()), "kvc_moe_combine")


def clamped_glu(out: torch.Tensor, gate_up: torch.Tensor, limit: float, alpha: float) -> None:
    """``out = g * sigmoid(alpha * g) * (u + 1)`` with ``g = min(gate, limit)``, ``u = clamp(up,
    -limit, limit)`` from ``gate_up [T, 2I]`` (gate columns first)."""
    T, I = out.shape
    if gate_up.shape != (T, 2 * I) or gate_up.dtype != out.dtype:
        raise KernelError("clamped_glu: shapes do not match")
    _check(load().kvc_clamped_glu(_dev(out, "out"), _dev(gate_up, "gate_up"), T, I, float(limit), float(alpha),
                                  _code(out, "out"), _stream()), "kvc_clamped_glu")


def table_update(table: torch.Tensor, triples: torch.Tensor, n: int) -> None:
    if triples.numel() < 3 * n:
        raise KernelError("table_update: triples too short")
    _check(load().kvc_table_update(_dev(table, "table", torch.int32), table.shape[1], table.shape[0],
                                   _dev(triples, "triples", torch.int32), n, _stream()),
           "kvc_table_update")


def argmax(out: torch.Tensor, logits: torch.Tensor, part_val: torch.Tensor | None = None,
           part_idx: torch.Tensor | None = None) -> None:
    """``part_val`` (float32) and ``part_idx`` (int32) of equal length are an optional
    workspace that lets several blocks search one long row."""
    S, V = logits.shape
    if out.numel() < S or logits.stride(1) != 1 or logits.dtype != torch.float32 or not logits.is_cuda:
        raise KernelError("argmax: expects float32 GPU logits [S, V] and S outputs")
    pv = pi = None
    cap = 0
    if part_val is not None and part_idx is not None:
        pv, pi = _dev(part_val, "part_val", torch.float32), _dev(part_idx, "part_idx", torch.int32)
        cap = min(part_val.numel(), part_idx.numel())
    _check(load().kvc_argmax(_dev(out, "out", torch.int32), logits.data_ptr(), S, V,
                             logits.stride(0), pv, pi, cap, _stream()), "kvc_argmax")


def sample_workspace_words(S: int, V: int) -> int:
    """64-bit words of workspace with which ``sample`` deals each row to several blocks
    (0 for rows too short to gain from it)."""
    return int(load().kvc_sample_workspace_words(S, V))


def sample(out: torch.Tensor, logits: torch.Tensor, *, temperature: torch.Tensor,
           top_k: torch.Tensor, top_p: torch.Tensor, seed_lo: torch.Tensor, seed_hi: torch.Tensor,
           index: torch.Tensor, workspace: torch.Tensor | None = None, filters: int = 3) -> None:
    """``workspace``: int64, ``sample_workspace_words(S, V)`` values or more, lets several
    blocks work on a row (the same draws, sooner); ``filters`` says which of top-k (1) and
    top-p (2) some row uses."""
    S, V = logits.shape
    if logits.stride(1) != 1 or logits.dtype != torch.float32 or not logits.is_cuda:
        raise KernelError("sample: expects float32 GPU logits [S, V]")
    for t, name in ((out, "out"), (temperature, "temperature"), (top_k, "top_k"), (top_p, "top_p"),
                    (seed_lo, "seed_lo"), (seed_hi, "seed_hi"), (index, "index")):
        if t.numel() < S or t.element_size() != 4:
            raise KernelError(f"sample: {name} must hold {S} 32-bit values")
    _check(load().kvc_sample(_dev(out, "out", torch.int32), logits.data_ptr(), S, V, logits.stride(0),
                             _dev(temperature, "temperature", torch.float32),
                             _dev(top_k, "top_k", torch.int32), _dev(top_p, "top_p", torch.float32),
                             _dev(seed_lo, "seed_lo"), _dev(seed_hi, "seed_hi"), _dev(index, "index"),
                             None if workspace is None else _dev(workspace, "workspace", torch.int64),
                             0 if workspace is None else workspace.numel(), int(filters),
                             _stream()), "kvc_sample")
