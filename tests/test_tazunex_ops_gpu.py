"""Every mechanism of the Tazunex decoder alone: the kernel against the plain function of
``tests/plain/tazunex.py``, at sizes of the tests' own, whole and in steps, beside other
requests and padding, from slots that hold another request's leftovers, with inputs made so
that a far token, a window's edge, a sink or a lost state shows."""

from __future__ import annotations

import pytest
import torch

from tests.plain import tazunex as plain
from tests.tazunex_helpers import batch_tensors

pytestmark = pytest.mark.gpu

DEV = "cuda"
F64 = torch.float64


def gpu(t, dtype=torch.float32):
    return t.to(device=DEV, dtype=dtype).contiguous()


def rel(got, want):
    return float((got.double().cpu() - want).pow(2).mean().sqrt() / (want.pow(2).mean().sqrt() + 1e-30))


# ------------------------------------------------------------------------- the norms
@pytest.mark.parametrize("H", [96, 40, 100, 7, 4096, 16392])
@pytest.mark.parametrize("delta_dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
def test_norm_behind_a_sublayer_sum_and_next_norm(H, delta_dtype):
    from kvcore_amd.ops import library as ops

    gen = torch.Generator().manual_seed(H)
    T, eps = 37, 1e-5
    r = torch.randn(T, H, generator=gen, dtype=F64)
    d = (torch.randn(T, H, generator=gen, dtype=F64) * 3).to(delta_dtype).double()
    g1, g2 = 1 + 0.3 * torch.randn(H, generator=gen, dtype=F64), 1 + 0.3 * torch.randn(H, generator=gen, dtype=F64)
    want_r = r + plain.rms(d, eps) * g1
    want_x = plain.rms(want_r, 2 * eps) * g2
    for out_dtype in (torch.float32, torch.bfloat16):
        res, out = gpu(r), torch.full((T, H), float("nan"), dtype=out_dtype, device=DEV)
        ops.norm_add_norm(out, res, gpu(d, delta_dtype), gpu(g1), eps, gpu(g2), 2 * eps)
        assert rel(res, want_r) < 1e-6
        assert rel(out, want_x) < (1e-6 if out_dtype == torch.float32 else 4e-3)
    res = gpu(r)
    ops.norm_add_norm(None, res, gpu(d, delta_dtype), gpu(g1), eps)
    assert rel(res, want_r) < 1e-6


@pytest.mark.parametrize("H,slices", [(96, 3), (100, 2), (2048, 4)])
def test_norm_behind_a_sublayer_adds_up_partial_sums(H, slices):
    """The result of the sublayer as partial sums of slices, as a product cut along K leaves them."""
    from kvcore_amd.ops import library as ops

    gen = torch.Generator().manual_seed(H + slices)
    T, eps = 29, 1e-5
    r = torch.randn(T, H, generator=gen, dtype=F64)
    parts = torch.randn(slices, T, H, generator=gen, dtype=F64).float().double()
    g1, g2 = 1 + 0.3 * torch.randn(H, generator=gen, dtype=F64), 1 + 0.3 * torch.randn(H, generator=gen, dtype=F64)
    want_r = r + plain.rms(parts.sum(0), eps) * g1
    want_x = plain.rms(want_r, eps) * g2
    room = torch.full((slices * T * H + 64,), float("nan"), device=DEV)
    room[: slices * T * H] = gpu(parts).view(-1)
    res, out = gpu(r), torch.full((T, H), float("nan"), dtype=torch.bfloat16, device=DEV)
    ops.norm_add_norm(out, res, ops.SlicedRows(room, slices, T, H), gpu(g1), eps, gpu(g2), eps)
    assert rel(res, want_r) < 1e-6 and rel(out, want_x) < 4e-3


@pytest.mark.parametrize("M,N,K,packed", [(40, 1024, 2048, True), (64, 512, 4096, True), (40, 1024, 2048, False),
                                          (23, 96, 80, False), (100, 2048, 8192, True), (33, 192, 512, False),
                                          (64, 256, 1024, True), (17, 200, 512, False), (192, 72, 1536, True),
                                          (50, 8, 512, False), (37, 320, 512, True), (150, 104, 1024, False)])
def test_a_product_that_leaves_partial_sums_for_the_norm_behind_it(M, N, K, packed):
    """``linear`` into a ``SliceSink`` and the norm that adds the slices up, against the plain
    product and norm on the same rounded operands: shapes that the weight-streaming kernel cuts
    along K, and shapes it does not take (then the one slice is the product itself)."""
    from kvcore_amd.ops import library as ops

    gen = torch.Generator().manual_seed(M + N)
    x = torch.randn(M, K, generator=gen).to(torch.bfloat16)
    w = (torch.randn(N, K, generator=gen) * K ** -0.5).to(torch.bfloat16)
    r = torch.randn(M, N, generator=gen, dtype=F64)
    g1 = 1 + 0.3 * torch.randn(N, generator=gen, dtype=F64)
    eps = 1e-6
    want_r = r + plain.rms(x.double() @ w.double().T, eps) * g1
    wd = gpu(w, torch.bfloat16)
    if packed and ops.can_pack_weight(wd):
        ops.pack_weight(wd)
    room = torch.full((ops.mid_slices_bound(N) * ops.MID_ROWS * N,), float("nan"), device=DEV)
    got = ops.linear(ops.SliceSink(room), gpu(x, torch.bfloat16), wd)
    assert isinstance(got, ops.SlicedRows) and (got.rows, got.width) == (M, N)
    if packed and K % 512 == 0 and ops.can_pack_weight(wd):
        assert got.count == ops.mid_slices(N, K)
    res = gpu(r)
    ops.norm_add_norm(None, res, got, gpu(g1), eps)
    assert rel(res, want_r) < 1e-5


@pytest.mark.parametrize("nq,nk,extra", [(128, 64, 0), (16, 16, 5), (3, 1, 0), (4096, 1024, 8)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
def test_norm_over_a_whole_projection(nq, nk, extra, dtype):
    """All query heads share one root mean square and all key heads another (not a head each),
    the gains have the projections' whole size, and the keys as they were land behind."""
    from kvcore_amd.ops import library as ops

    gen = torch.Generator().manual_seed(nq)
    T, eps = 21, 1e-4
    rows = (torch.randn(T, nq + 2 * nk + extra, generator=gen, dtype=F64) * 2).to(dtype).double()
    rows[:, :nq // 2] *= 5  # the heads differ in size, so a norm per head would show
    gq, gk = 1 + 0.3 * torch.randn(nq, generator=gen, dtype=F64), 1 + 0.3 * torch.randn(nk, generator=gen, dtype=F64)
    x = gpu(rows, dtype)
    ops.wide_qk_norm(x, gpu(gq), gpu(gk), eps, copy_k=True)
    tol = 1e-6 if dtype == torch.float32 else 4e-3
    assert rel(x[:, :nq], plain.rms(rows[:, :nq], eps) * gq) < tol
    assert rel(x[:, nq:nq + nk], plain.rms(rows[:, nq:nq + nk], eps) * gk) < tol
    assert torch.equal(x[:, nq + nk:nq + 2 * nk].double().cpu(), rows[:, nq:nq + nk])
    assert torch.equal(x[:, nq + 2 * nk:].double().cpu(), rows[:, nq + 2 * nk:])
    y = gpu(rows, dtype)
    ops.wide_qk_norm(y, gpu(gq), gpu(gk), eps)
    assert torch.equal(y[:, nq + nk:].double().cpu(), rows[:, nq + nk:])  # nothing copied unasked


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
def test_gate_per_head_on_a_run_of_columns(dtype):
    from kvcore_amd.ops import library as ops

    gen = torch.Generator().manual_seed(2)
    T, heads, stride, skip, n = 19, 5, 14, 4, 9
    x = torch.randn(T, heads * stride + 3, generator=gen, dtype=F64).to(dtype).double()
    g = (torch.randn(T, heads + 2, generator=gen, dtype=F64) * 2).to(dtype).double()
    out = torch.empty(T, heads * n, dtype=dtype, device=DEV)
    ops.head_gate(out, gpu(x, dtype), gpu(g, dtype)[:, 2:], heads=heads, head_stride=stride, skip=skip, n=n)
    want = x[:, :heads * stride].view(T, heads, stride)[:, :, skip:skip + n] * torch.sigmoid(g[:, 2:])[:, :, None]
    assert rel(out, want.reshape(T, -1)) < (1e-6 if dtype == torch.float32 else 4e-3)


@pytest.mark.parametrize("q_rank,rank,rot,extra", [(40, 24, 8, 3), (1, 6, 2, 1), (7, 5, 0, 2), (1024, 96, 32, 16)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
def test_latent_norms_and_the_cached_row(q_rank, rank, rot, extra, dtype):
    """The query latent and the key/value latent each over its own root mean square; the cached
    row is the rotated part as projected (not normed), then the normed latent, twice."""
    from kvcore_amd.ops import library as ops

    gen = torch.Generator().manual_seed(q_rank + rank)
    T, eps, heads = 13, 1e-5, 3
    down = (torch.randn(T, q_rank + rank + rot + extra, generator=gen, dtype=F64) * 2).to(dtype).double()
    down[:, q_rank:q_rank + rank] *= 4  # the two latents differ in size, so one norm over both would show
    gq, gc = 1 + 0.3 * torch.randn(q_rank, generator=gen, dtype=F64), 1 + 0.3 * torch.randn(rank, generator=gen, dtype=F64)
    row = rot + rank
    cq = torch.full((T, q_rank), float("nan"), dtype=dtype, device=DEV)
    qkv = torch.full((T, (heads + 2) * row), float("nan"), dtype=dtype, device=DEV)
    ops.latent_rows(cq, qkv[:, heads * row:(heads + 1) * row], qkv[:, (heads + 1) * row:], gpu(down, dtype), gpu(gq),
                    gpu(gc), eps, rot)
    tol = 1e-6 if dtype == torch.float32 else 4e-3
    assert rel(cq, plain.rms(down[:, :q_rank], eps) * gq) < tol
    want = torch.cat([down[:, q_rank + rank:q_rank + rank + rot], plain.rms(down[:, q_rank:q_rank + rank], eps) * gc], dim=1)
    assert rel(qkv[:, heads * row:(heads + 1) * row], want) < tol
    assert torch.equal(qkv[:, heads * row:(heads + 1) * row], qkv[:, (heads + 1) * row:])
    assert torch.isnan(qkv[:, :heads * row]).all()  # the queries' place is left alone


# ------------------------------------------------------------------ the gated feed-forward
@pytest.mark.parametrize("dtype,M,H,I", [(torch.float32, 9, 40, 24), (torch.bfloat16, 1, 64, 48), (torch.bfloat16, 16, 128, 136),
                                         (torch.bfloat16, 40, 512, 256), (torch.bfloat16, 150, 1024, 128),
                                         (torch.bfloat16, 300, 96, 80), (torch.bfloat16, 5, 100, 20)])
def test_feed_forward_gate_in_the_tanh_form_of_gelu(dtype, M, H, I):
    """Through every kernel that may serve the gate-up product (few rows, rows shared through LDS,
    the vendor's product with a kernel for the gate), and not silu."""
    from kvcore_amd.ops import library as ops

    gen = torch.Generator().manual_seed(M + I)
    x = torch.randn(M, H, generator=gen, dtype=F64).to(dtype).double()
    w = (torch.randn(2 * I, H, generator=gen, dtype=F64) * 0.2).to(dtype).double()
    gate, up = x @ w[:I].T, x @ w[I:].T
    if dtype == torch.bfloat16:
        gate, up = gate.to(dtype).double(), up.to(dtype).double()
    want = plain.gelu_tanh(gate) * up
    out = torch.empty(M, I, dtype=dtype, device=DEV)
    ops.linear_silu_mul(out, gpu(x, dtype), gpu(w, dtype), None,
                        lambda: torch.empty(M, 2 * I, dtype=dtype, device=DEV), act="gelu_tanh")
    assert rel(out, want) < (2e-6 if dtype == torch.float32 else 6e-3)
    assert rel(out, torch.nn.functional.silu(gate) * up) > 1e-2
    packed = torch.cat([gate, up], dim=1)
    plainly = torch.empty(M, I, dtype=dtype, device=DEV)
    ops.silu_mul(plainly, gpu(packed, dtype), "gelu_tanh")
    assert rel(plainly, want) < (2e-6 if dtype == torch.float32 else 4e-3)
    with pytest.raises(ops.KernelError):
        ops.silu_mul(plainly, gpu(packed, dtype), "relu")


# ------------------------------------------------------------------ the matrix memory
def memory_weights(H, d, dv, cap, gen, f_bias=2.0):
    """A mixer whose projections pick columns of its input, so that the plain function takes q, k,
    v, the gate and the raw gates as given."""
    qk, inner = H * d, H * dv
    width = 2 * qk + 2 * inner + 2 * H
    eye = torch.eye(width, dtype=F64)
    at = [0, qk, 2 * qk, 2 * qk + inner, 2 * qk + 2 * inner, 2 * qk + 2 * inner + H, width]
    w = {n: eye[at[i]:at[i + 1]] for i, n in enumerate(("q", "k", "v", "g", "i", "f"))}
    w["i.b"] = torch.randn(H, generator=gen, dtype=F64)
    w["f.b"] = torch.randn(H, generator=gen, dtype=F64) + f_bias
    w["norm"] = 1 + 0.2 * torch.randn(inner, generator=gen, dtype=F64)
    w["o"] = torch.eye(inner, dtype=F64)
    return w, {"heads": H, "dim": d, "vdim": dv, "gate_cap": cap}, width


def run_memory(h, w, m, state, maxima, reqs, eps):
    """The kernels in the order the mixer launches them, on rows ``h`` of the whole batch."""
    from kvcore_amd.ops import library as ops

    H, d, dv = m["heads"], m["dim"], m["vdim"]
    qk, inner = H * d, H * dv
    batch, T = batch_tensors(reqs)
    proj = gpu(h)
    keep, take, mx = (torch.full((T, H), float("nan"), device=DEV) for _ in range(3))
    at = 2 * qk + 2 * inner
    ops.max_gates(keep, take, mx, proj[:, at:at + H], proj[:, at + H:], gpu(w["i.b"]), gpu(w["f.b"]), m["gate_cap"],
                  maxima, **batch)
    o = torch.full((T, H * (dv + 1)), float("nan"), device=DEV)
    ops.linear_state_scan(o, proj[:, :qk], proj[:, qk:2 * qk], proj[:, 2 * qk:2 * qk + inner], keep, take, state,
                          heads=H, qk_heads=H, dim=d, vdim=dv + 1, scalar_gates=True, ones_column=True,
                          q_scale=d ** -0.5, **batch)
    out = torch.full((T, inner), float("nan"), device=DEV)
    ops.max_gated_finish(out, o, mx, proj[:, 2 * qk + inner:at], gpu(w["norm"]), eps, 1e-6, H, dv)
    return out


def new_memory(slots, H, d, dv):
    from kvcore_amd.ops import library as ops

    return (torch.full((slots, H, ops.linear_state_rows(d), dv + 1), float("nan"), device=DEV),
            torch.full((slots, H), float("nan"), device=DEV))


@pytest.mark.parametrize("H,d,dv,cap", [(3, 24, 40, 15.0), (1, 8, 1, 1.0), (2, 200, 80, 20.0), (4, 64, 64, 8.0),
                                        (2, 64, 127, 12.0), (6, 20, 16, 3.0)])
def test_matrix_memory_whole_in_steps_and_beside_others(H, d, dv, cap):
    gen = torch.Generator().manual_seed(H * d + dv)
    w, m, width = memory_weights(H, d, dv, cap, gen)
    eps = 1e-5
    seqs = [torch.randn(n, width, generator=gen, dtype=F64) for n in (70, 33, 5)]
    for s in seqs:
        s[:, -2 * H:] *= 4  # raw gates large enough for the cap to bite
    want = [plain.mlstm(s, w, m, eps) for s in seqs]
    state, maxima = new_memory(5, H, d, dv)
    # whole, three requests side by side with a padded one between them
    got = run_memory(torch.cat([seqs[0], torch.zeros(1, width, dtype=F64), seqs[1], seqs[2]]), w, m, state, maxima,
                     [(3, 0, 70), None, (0, 0, 33), (4, 0, 5)], eps)
    assert rel(got[:70], want[0]) < 2e-5 and rel(got[71:104], want[1]) < 2e-5 and rel(got[104:], want[2]) < 2e-5
    assert torch.equal(got[70], torch.zeros_like(got[70])) or torch.isfinite(got[70]).all()
    # in steps: portions of 2, 1, 30, 16 and single tokens, the other request beside them from
    # another slot; slot 1 held NaN before
    state, maxima = new_memory(5, H, d, dv)
    cuts_a, cuts_b = [2, 1, 30, 16, 1, 1, 19], [1, 16, 2, 1, 1, 12, 0]
    at_a = at_b = 0
    for na, nb in zip(cuts_a, cuts_b):
        rows = [seqs[0][at_a:at_a + na]] + ([seqs[1][at_b:at_b + nb]] if nb else [])
        reqs = [(1, at_a, na)] + ([(2, at_b, nb)] if nb else [])
        got = run_memory(torch.cat(rows), w, m, state, maxima, reqs, eps)
        assert rel(got[:na], want[0][at_a:at_a + na]) < 2e-5, (at_a, na)
        if nb:
            assert rel(got[na:], want[1][at_b:at_b + nb]) < 2e-5, (at_b, nb)
        at_a, at_b = at_a + na, at_b + nb
    assert at_a == 70 and at_b == 33
    # the slot is taken over by a new request: it starts from nothing, whatever the slot holds
    got = run_memory(seqs[2], w, m, state, maxima, [(1, 0, 5)], eps)
    assert rel(got, want[2]) < 2e-5


def test_the_running_maximum_starts_at_zero_and_the_floor_of_the_denominator_counts():
    """Input gates far below zero: with a maximum that started at minus infinity the first token's
    weight would be one; here exp(i) stays tiny and the denominator is exp(-m) = 1."""
    gen = torch.Generator().manual_seed(1)
    H, d, dv = 2, 8, 6
    w, m, width = memory_weights(H, d, dv, 30.0, gen)
    w["i.b"] = torch.full((H,), -12.0, dtype=F64)
    h = torch.randn(4, width, generator=gen, dtype=F64)
    h[:, -2 * H:] = 0.0
    w_flat = dict(w, norm=torch.ones(H * dv, dtype=F64))
    want = plain.mlstm(h, w_flat, m, 1e-6)
    state, maxima = new_memory(2, H, d, dv)
    got = run_memory(h, w_flat, m, state, maxima, [(1, 0, 4)], 1e-6)
    assert rel(got, want) < 2e-5
    assert float(maxima[1].abs().max()) < 1.0  # near log(sigmoid) sums, not near -12


def test_a_token_written_six_hundred_tokens_ago_is_still_read():
    """Forget gates of almost one: the first token's value, written with a large input gate,
    dominates what a query that matches its key reads 600 tokens later, in one portion, in
    portions, and token by token."""
    gen = torch.Generator().manual_seed(4)
    H, d, dv, T = 2, 16, 12, 640
    w, m, width = memory_weights(H, d, dv, 25.0, gen, f_bias=20.0)
    w["i.b"] = torch.zeros(H, dtype=F64)
    qk, inner = H * d, H * dv
    h = torch.randn(T, width, generator=gen, dtype=F64) * 0.3
    h[:, -2 * H:-H] = -6.0  # small input gates
    h[:, -H:] = 0.0
    h[0, -2 * H:-H] = 8.0   # but the first token's
    h[0, qk:2 * qk] = 0.0
    h[0, qk] = 3.0          # its key: the first channel of head 0
    h[1:, qk] = 0.0
    h[T - 1, :qk] = 0.0
    h[T - 1, 0] = 5.0       # the last query asks for exactly that channel
    want = plain.mlstm(h, w, m, 1e-6)
    lone = h.clone()
    lone[0, 2 * qk:2 * qk + inner] = 0.0
    assert rel(plain.mlstm(lone, w, m, 1e-6)[T - 1, :dv], want[T - 1, :dv]) > 0.3  # the far token matters
    for cuts in ([T], [100, 2, 300, 237, 1], [600] + [1] * 40):
        state, maxima = new_memory(2, H, d, dv)
        at, rows = 0, []
        for n in cuts:
            rows.append(run_memory(h[at:at + n], w, m, state, maxima, [(1, at, n)], 1e-6))
            at += n
        assert rel(torch.cat(rows), want) < 5e-5, cuts


# ------------------------------------------------------------------------ attention
def paged(q, k, v, page, *, scale, window, sink, dtype, positions=None, kernel="general", nsplit=1):
    """Attention of ``q [T, H, d]`` (tokens at ``positions``, default 0..T-1) over keys and values
    ``k, v [S, G, d / dv]`` laid into pages in a shuffled order, through the general kernel, or
    (bfloat16) the matrix-core kernel for portions (``"portion"``) or for single tokens
    (``"single"``, one launch a token); ``nsplit`` parts of the key range."""
    from kvcore_amd.ops import library as ops

    S, G, d = k.shape
    dv = v.shape[2]
    T, H, _ = q.shape
    n_pages = -(-S // page)
    order = torch.randperm(n_pages, generator=torch.Generator().manual_seed(1))
    k_cache = torch.full((n_pages + 1, G, page, d), float("nan"), dtype=dtype, device=DEV)
    v_cache = torch.full((n_pages + 1, G, dv, page), float("nan"), dtype=dtype, device=DEV)
    table = torch.zeros((2, n_pages), dtype=torch.int32, device=DEV)
    for p in range(n_pages):
        pid = int(order[p]) + 1
        table[1, p] = pid
        n = min(page, S - p * page)
        k_cache[pid, :, :n] = gpu(k[p * page:p * page + n].transpose(0, 1), dtype)
        v_cache[pid, :, :, :n] = gpu(v[p * page:p * page + n].permute(1, 2, 0), dtype)
        k_cache[pid, :, n:] = 0  # the rest of the last page: beyond every query, never seen
        v_cache[pid, :, :, n:] = 0
    pos = list(range(T)) if positions is None else positions
    out = torch.empty(T, H * dv, dtype=dtype, device=DEV)
    sinks = None if sink is None else gpu(sink)
    ints = dict(dtype=torch.int32, device=DEV)
    part_o = part_ml = None
    if nsplit > 1:
        part_o = torch.full((T * H * nsplit, d), float("nan"), device=DEV)
        part_ml = torch.full((T * H * nsplit, 2), float("nan"), device=DEV)
    if kernel == "portion":
        assert ops.prefill_attention_supported(H, G, d, page, dtype) and dv == d
        ops.prefill_attention(out, gpu(q.reshape(T, -1), dtype), k_cache, v_cache, table=table,
                              positions=torch.tensor(pos, **ints), q_start=torch.tensor([0, T], **ints),
                              slots=torch.tensor([1], **ints), num_reqs=1, nh=H, nkv=G, d=d, scale=scale,
                              window=window, sinks=sinks, nsplit=nsplit, part_o=part_o, part_ml=part_ml)
        assert ops.last_variant("prefill_attention").startswith("prefill_attention_kernel")
    elif kernel == "single":
        assert ops.decode_attention_supported(H, G, d, page, dtype) and dv == d
        for i in range(T):
            ops.decode_attention(out[i:i + 1], gpu(q[i:i + 1].reshape(1, -1), dtype), k_cache, v_cache, table=table,
                                 positions=torch.tensor(pos[i:i + 1], **ints), token_req=torch.zeros(1, **ints),
                                 slots=torch.tensor([1], **ints), nh=H, nkv=G, d=d, scale=scale, window=window,
                                 sinks=sinks, nsplit=nsplit, part_o=part_o, part_ml=part_ml)
    else:
        ops.paged_attention(out, gpu(q.reshape(T, -1), dtype), k_cache, v_cache, table=table,
                            positions=torch.tensor(pos, **ints), token_req=torch.zeros(T, **ints),
                            slots=torch.tensor([1], **ints), nh=H, nkv=G, d=d, dv=dv, scale=scale, window=window,
                            sinks=sinks)
    return out.double().cpu().view(T, H, dv)


@pytest.mark.parametrize("H,G,d,dv,window,page", [(4, 2, 32, 32, 24, 8), (6, 6, 16, 16, 10, 16), (1, 1, 16, 16, 1, 4),
                                                   (2, 1, 16, 16, 0, 4), (3, 1, 48, 48, 100, 16), (20, 1, 64, 64, 70, 16),
                                                   (3, 1, 30, 30, 33, 8)])
def test_windowed_attention_with_a_sink(H, G, d, dv, window, page):
    gen = torch.Generator().manual_seed(H * 100 + window)
    T = 131
    q = torch.randn(T, H, d, generator=gen, dtype=F64)
    k = torch.randn(T, G, d, generator=gen, dtype=F64)
    v = torch.randn(T, G, dv, generator=gen, dtype=F64)
    sink = torch.randn(H, generator=gen, dtype=F64) * 2 + 1
    want = plain.windowed_attention(q, k, v, 0.3, window or None, sink)
    got = paged(q, k, v, page, scale=0.3, window=window, sink=sink, dtype=torch.float32)
    assert rel(got, want) < 2e-6
    # the sink matters, and it is not scaled: without it, or scaled like a score, the result differs
    assert rel(paged(q, k, v, page, scale=0.3, window=window, sink=None, dtype=torch.float32), want) > 1e-2
    assert rel(paged(q, k, v, page, scale=0.3, window=window, sink=sink * 0.3, dtype=torch.float32), want) > 1e-3
    if d % 16 == 0:
        got = paged(q, k, v, page, scale=0.3, window=window, sink=sink, dtype=torch.bfloat16)
        qb, kb, vb = (t.to(torch.bfloat16).double() for t in (q, k, v))
        assert rel(got, plain.windowed_attention(qb, kb, vb, 0.3, window or None, sink)) < 1e-2


@pytest.mark.parametrize("single", [False, True], ids=["portion", "single"])
def test_a_key_that_stands_out_at_a_window_s_edges_and_far_back(single):
    """One key is made to outscore all others (and the sink) for every query.  A query sees it iff
    it lies among the last ``window`` positions up to the query's own: just inside the window,
    just outside, a page's first and last slot, hundreds of tokens back in a long window.  The
    queries come as a portion of a prompt or as single tokens."""
    H, G, d, page = 2, 1, 16, 16
    for window, T, marked, query in ((64, 200, 64, 127), (64, 200, 63, 127), (64, 200, 128, 128), (64, 200, 127, 191),
                                     (64, 200, 128, 191), (400, 420, 0, 399), (400, 420, 0, 400), (400, 420, 15, 414),
                                     (400, 420, 16, 415), (400, 420, 16, 416), (0, 420, 3, 419), (48, 200, 95, 143),
                                     (48, 200, 96, 143), (48, 200, 96, 144), (1, 50, 30, 30), (1, 50, 29, 30)):
        gen = torch.Generator().manual_seed(marked + query)
        k = torch.randn(T, G, d, generator=gen, dtype=F64) * 0.3
        k[:, 0, 0] = 0.0
        k[marked, 0] = 0.0
        k[marked, 0, 0] = 1.0
        v = torch.randn(T, G, d, generator=gen, dtype=F64)
        q = torch.randn(T, H, d, generator=gen, dtype=F64) * 0.3
        q[:, :, 0] = 40.0
        sink = torch.tensor([2.0, -1.0], dtype=F64)
        visible = marked <= query and (window == 0 or query - marked < window)
        want = plain.windowed_attention(q, k, v, 1.0, window or None, sink)
        assert torch.allclose(want[query, 1], v[marked, 0], atol=1e-3) == visible
        lo = max(query - 2, 0)
        qs = q[query:query + 1] if single else q[lo:query + 1]
        pos = [query] if single else list(range(lo, query + 1))
        got = paged(qs, k, v, page, scale=1.0, window=window, sink=sink, dtype=torch.float32, positions=pos)
        assert rel(got[-1], want[query]) < 1e-5, (window, marked, query)
        assert torch.allclose(got[-1, 1], v[marked, 0], atol=1e-3) == visible, (window, marked, query)


def test_a_sink_that_outweighs_every_key():
    """A large sink takes nearly all of the weight: the result shrinks towards zero by exactly the
    plain function's factor, in every kernel."""
    gen = torch.Generator().manual_seed(8)
    T, H, G, d = 80, 4, 2, 64
    q = torch.randn(T, H, d, generator=gen, dtype=F64).to(torch.bfloat16).double()
    k = torch.randn(T, G, d, generator=gen, dtype=F64).to(torch.bfloat16).double()
    v = torch.randn(T, G, d, generator=gen, dtype=F64).to(torch.bfloat16).double()
    sink = torch.tensor([30.0, 9.0, -40.0, 0.0], dtype=F64)
    want = plain.windowed_attention(q, k, v, 0.2, 20, sink)
    assert float(want[:, 0].abs().max()) < 1e-3
    assert rel(paged(q, k, v, 16, scale=0.2, window=20, sink=sink, dtype=torch.float32), want) < 2e-6
    assert rel(paged(q, k, v, 16, scale=0.2, window=20, sink=sink, dtype=torch.bfloat16, kernel="portion"), want) < 1e-2
    rows = [0, 1, 19, 20, 21, 79]
    got = paged(q[rows], k, v, 16, scale=0.2, window=20, sink=sink, dtype=torch.bfloat16, kernel="single", positions=rows)
    assert rel(got, want[rows]) < 1e-2


@pytest.mark.parametrize("kernel,nsplit", [("portion", 1), ("portion", 3), ("single", 1), ("single", 4)])
@pytest.mark.parametrize("H,G,d,window", [(8, 2, 64, 48), (4, 4, 128, 0), (4, 1, 128, 100), (16, 2, 64, 1), (6, 1, 96, 150)])
def test_matrix_core_kernels_with_windows_and_sinks(kernel, nsplit, H, G, d, window):
    """The bfloat16 kernels for portions and for single tokens against the plain function on the
    same rounded values: every position of a prompt of 300 tokens (windows that are no multiple of
    the kernels' tiles of 16 and 64 keys, a window of one position, none), with the key range in one
    part and in several (the sink counts once, whatever the number of parts), then the key that
    stands out at a window's edges."""
    from kvcore_amd.ops import library as ops

    if kernel == "portion" and not ops.prefill_attention_supported(H, G, d, 16, torch.bfloat16):
        pytest.skip("the kernel for portions serves heads of 64 and 128")
    gen = torch.Generator().manual_seed(H + d + window)
    T, page = 300, 16
    q = torch.randn(T, H, d, generator=gen, dtype=F64).to(torch.bfloat16).double()
    k = torch.randn(T, G, d, generator=gen, dtype=F64).to(torch.bfloat16).double()
    v = torch.randn(T, G, d, generator=gen, dtype=F64).to(torch.bfloat16).double()
    sink = torch.randn(H, generator=gen, dtype=F64) * 2 + 1
    scale = 0.5 * d ** -0.5
    want = plain.windowed_attention(q, k, v, scale, window or None, sink)
    rows = list(range(T)) if kernel == "portion" else [0, 1, 15, 16, 47, 48, 95, 96, 143, 144, 199, 200, 255, 256, 299]
    got = paged(q[rows] if kernel == "single" else q, k, v, page, scale=scale, window=window, sink=sink,
                dtype=torch.bfloat16, positions=rows, kernel=kernel, nsplit=nsplit)
    assert rel(got, want[rows]) < 1e-2
    no_sink = paged(q[rows] if kernel == "single" else q, k, v, page, scale=scale, window=window, sink=None,
                    dtype=torch.bfloat16, positions=rows, kernel=kernel, nsplit=nsplit)
    assert rel(no_sink, want[rows]) > 2e-2
    for size, marked, query in ((48, 95, 143), (48, 96, 143), (48, 96, 144), (48, 48, 95), (200, 0, 199), (200, 0, 200),
                                (200, 16, 215), (200, 16, 216), (0, 3, 299)):
        k2 = torch.randn(T, G, d, generator=gen, dtype=F64) * 0.3
        k2[:, :, 0] = 0.0
        k2[marked] = 0.0
        k2[marked, :, 0] = 1.0
        q2 = torch.randn(T, H, d, generator=gen, dtype=F64) * 0.3
        q2[:, :, 0] = 40.0
        q2, k2 = q2.to(torch.bfloat16).double(), k2.to(torch.bfloat16).double()
        visible = marked <= query and (size == 0 or query - marked < size)
        rows = [query - 2, query - 1, query] if kernel == "portion" else [query]
        got = paged(q2[rows], k2, v, page, scale=1.0, window=size, sink=sink, dtype=torch.bfloat16, positions=rows,
                    kernel=kernel, nsplit=nsplit)
        assert torch.allclose(got[-1, H - 1], v[marked, G - 1], atol=2e-2) == visible, (size, marked, query)
