"""Every mechanism of the Darovik decoder alone: the kernel or part against the plain function of
``tests/plain/darovik.py``, at sizes of the tests' own, with inputs made so that a far token, a
window's edge, a sink, a negative choice score or a copy of the stream that is left out shows."""

from __future__ import annotations

import math

import pytest
import torch

from tests.plain import darovik as plain

pytestmark = pytest.mark.gpu

DEV = "cuda"
F64 = torch.float64


def gpu(t, dtype=torch.float32):
    return t.to(device=DEV, dtype=dtype).contiguous()


def rel(got, want):
    return float((got.double().cpu() - want).pow(2).mean().sqrt() / (want.pow(2).mean().sqrt() + 1e-30))


# ---------------------------------------------------------- the stream of several copies
@pytest.mark.parametrize("copies", [1, 2, 3, 4, 5, 8])
@pytest.mark.parametrize("H", [96, 40, 7, 1030, 4096])
def test_a_sublayer_s_result_joins_the_copies_and_the_next_input_is_normed(copies, H):
    from kvcore_amd.ops import library as ops

    gen = torch.Generator().manual_seed(copies * 100 + H)
    T, eps, mult = 19, 1e-5, 0.7
    x = torch.randn(T, copies, H, generator=gen, dtype=F64)
    mix = torch.eye(copies, dtype=F64) * 0.6 + 0.3 * torch.randn(copies, copies, generator=gen, dtype=F64)
    w_in, w_out = (0.8 + 0.4 * torch.randn(copies, generator=gen, dtype=F64) for _ in range(2))
    gain = 1 + 0.3 * torch.randn(H, generator=gen, dtype=F64)
    for y_dtype in (torch.float32, torch.bfloat16):
        y = (torch.randn(T, H, generator=gen, dtype=F64) * 2).to(y_dtype).double()
        new = torch.einsum("st,ksh->kth", mix, x) + mult * w_out[None, :, None] * y[:, None, :]
        u = torch.einsum("t,kth->kh", w_in, new)
        want = plain.rms(u, eps) * gain
        for out_dtype in (torch.float32, torch.bfloat16):
            streams = gpu(x.reshape(T, copies * H))
            out = torch.full((T, H), float("nan"), dtype=out_dtype, device=DEV)
            ops.hyper_step(out, streams, copies, gpu(y, y_dtype), mix=gpu(mix), out_w=gpu(w_out), mult=mult,
                           in_w=gpu(w_in), gain=gpu(gain), eps=eps)
            assert rel(streams.view(T, copies, H), new) < 1e-6
            assert rel(out, want) < (2e-6 if out_dtype == torch.float32 else 4e-3)
        # the write alone, and the read alone of what it left
        streams = gpu(x.reshape(T, copies * H))
        ops.hyper_step(None, streams, copies, gpu(y, y_dtype), mix=gpu(mix), out_w=gpu(w_out), mult=mult)
        assert rel(streams.view(T, copies, H), new) < 1e-6
        out = torch.full((T, H), float("nan"), device=DEV)
        before = streams.clone()
        ops.hyper_step(out, streams, copies, in_w=gpu(w_in), gain=gpu(gain), eps=eps)
        assert torch.equal(before, streams) and rel(out, want) < 2e-6
    # no coefficients: the identity carries every copy, the result joins each, the input is their sum
    streams = gpu(x.reshape(T, copies * H))
    out = torch.full((T, H), float("nan"), device=DEV)
    ops.hyper_step(out, streams, copies, gpu(y), mult=mult, gain=gpu(gain), eps=eps)
    new = x + mult * y[:, None, :]
    assert rel(streams.view(T, copies, H), new) < 1e-6 and rel(out, plain.rms(new.sum(1), eps) * gain) < 2e-6


@pytest.mark.parametrize("copies,H,slices", [(2, 96, 3), (4, 2048, 4), (1, 100, 2), (3, 5000, 2)])
def test_a_result_left_as_partial_sums_is_added_up_on_its_way_into_the_copies(copies, H, slices):
    """The sublayer's result as partial sums of slices, as a product cut along K leaves them."""
    from kvcore_amd.ops import library as ops

    gen = torch.Generator().manual_seed(H + slices)
    T, eps, mult = 29, 1e-5, 1.3
    x = torch.randn(T, copies, H, generator=gen, dtype=F64)
    parts = torch.randn(slices, T, H, generator=gen, dtype=F64).float().double()
    mix = torch.eye(copies, dtype=F64) * 0.6 + 0.3 * torch.randn(copies, copies, generator=gen, dtype=F64)
    w_in, w_out = (0.8 + 0.4 * torch.randn(copies, generator=gen, dtype=F64) for _ in range(2))
    gain = 1 + 0.3 * torch.randn(H, generator=gen, dtype=F64)
    room = torch.full((slices * T * H + 64,), float("nan"), device=DEV)
    room[: slices * T * H] = gpu(parts).view(-1)
    # without a bias, and with the product's bias still to be added (in either dtype)
    for bias_dtype in (None, torch.float32, torch.bfloat16):
        bias = None if bias_dtype is None else torch.randn(H, generator=gen, dtype=F64).to(bias_dtype).double()
        y = parts.sum(0) + (0 if bias is None else bias)
        new = torch.einsum("st,ksh->kth", mix, x) + mult * w_out[None, :, None] * y[:, None, :]
        want = plain.rms(torch.einsum("t,kth->kh", w_in, new), eps) * gain
        streams = gpu(x.reshape(T, copies * H))
        out = torch.full((T, H), float("nan"), dtype=torch.bfloat16, device=DEV)
        rows = ops.SlicedRows(room, slices, T, H, None if bias is None else gpu(bias, bias_dtype))
        ops.stream_write_read(out, streams, copies, ops.StreamWrite(rows, copies, gpu(mix), gpu(w_out), mult),
                              in_w=gpu(w_in), gain=gpu(gain), eps=eps)
        assert rel(streams.view(T, copies, H), new) < 1e-6 and rel(out, want) < 4e-3


@pytest.mark.parametrize("M,N,K,packed", [(40, 1024, 2048, True), (64, 512, 4096, True), (23, 96, 80, False),
                                          (100, 2048, 8192, True), (33, 192, 512, False)])
def test_a_product_with_a_bias_that_leaves_partial_sums_for_the_stream(M, N, K, packed):
    """``linear`` into a ``SliceSink`` that takes the bias along, and the stream kernel that adds the
    slices and the bias up, against the plain product on the same rounded operands: shapes that the
    weight-streaming kernel cuts along K, and shapes it does not take."""
    from kvcore_amd.ops import library as ops

    gen = torch.Generator().manual_seed(M + N)
    a = torch.randn(M, K, generator=gen).to(torch.bfloat16)
    w = (torch.randn(N, K, generator=gen) * K ** -0.5).to(torch.bfloat16)
    b = torch.randn(N, generator=gen).to(torch.bfloat16)
    x = torch.randn(M, 2, N, generator=gen, dtype=F64)
    wd = gpu(w, torch.bfloat16)
    if packed and ops.can_pack_weight(wd):
        ops.pack_weight(wd)
    room = torch.full((ops.mid_slices_bound(N) * ops.MID_ROWS * N,), float("nan"), device=DEV)
    got = ops.linear(ops.SliceSink(room, takes_bias=True), gpu(a, torch.bfloat16), wd, gpu(b, torch.bfloat16))
    assert isinstance(got, ops.SlicedRows) and (got.rows, got.width) == (M, N)
    if packed and K % 512 == 0 and ops.can_pack_weight(wd):
        assert got.count == ops.mid_slices(N, K) and got.bias is not None
    streams = gpu(x.reshape(M, 2 * N))
    ops.stream_write_read(None, streams, 2, ops.StreamWrite(got, 2, None, None, 0.5))
    want = x + 0.5 * (a.double() @ w.double().T + b.double())[:, None, :]
    assert rel(streams.view(M, 2, N), want) < 1e-5
    # a sink that does not take the bias gets it added by the product, as one slice
    got = ops.linear(ops.SliceSink(room), gpu(a, torch.bfloat16), wd, gpu(b, torch.bfloat16))
    assert got.bias is None and got.count == 1


def test_every_copy_starts_as_the_embedding_s_row():
    from kvcore_amd.ops import library as ops

    rows = torch.randn(13, 50, dtype=F64)
    streams = torch.full((13, 150), float("nan"), device=DEV)
    ops.spread_streams(streams, gpu(rows), 3)
    assert torch.equal(streams.view(13, 3, 50).double().cpu(), rows.float().double()[:, None, :].expand(13, 3, 50))
    with pytest.raises(ops.KernelError):
        ops.hyper_step(None, streams, 4, gpu(rows))  # 150 columns are no four copies


# ----------------------------------------------------------------- joining the two maps
@pytest.mark.parametrize("heads,dv", [(4, 40), (1, 1), (3, 96), (2, 300), (6, 64)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
def test_the_second_map_is_taken_off_and_the_head_normed(heads, dv, dtype):
    from kvcore_amd.ops import library as ops

    gen = torch.Generator().manual_seed(heads + dv)
    T, lam, eps, diff = 23, 0.37, 1e-5, 0.3
    maps = (torch.randn(T, heads, 2, dv, generator=gen, dtype=F64) * 2).to(dtype).double()
    extra = 5  # the rows may be wider than the maps
    rows = torch.cat([maps.reshape(T, -1), torch.randn(T, extra, generator=gen, dtype=F64)], dim=1)
    want = plain.rms(maps[:, :, 0] - lam * maps[:, :, 1], eps) * (1 - diff)
    out = torch.full((T, heads * dv), float("nan"), dtype=dtype, device=DEV)
    ops.diff_heads_norm(out, gpu(rows, dtype)[:, : 2 * heads * dv], heads=heads, dv=dv, lam=lam, eps=eps, post=1 - diff)
    assert rel(out.view(T, heads, dv), want) < (2e-6 if dtype == torch.float32 else 4e-3)
    # maps that were never rounded (float32) beside a result in the model's dtype: two maps that
    # nearly cancel keep their difference
    near = torch.randn(T, heads, 1, dv, generator=gen, dtype=F64).expand(T, heads, 2, dv).clone()
    near[:, :, 1] = near[:, :, 0] / lam * (1 + 1e-3 * torch.randn(T, heads, dv, generator=gen, dtype=F64))
    near = near.float().double()
    want = plain.rms(near[:, :, 0] - lam * near[:, :, 1], eps) * (1 - diff)
    out = torch.full((T, heads * dv), float("nan"), dtype=dtype, device=DEV)
    ops.diff_heads_norm(out, gpu(near.reshape(T, -1)), heads=heads, dv=dv, lam=lam, eps=eps, post=1 - diff)
    assert rel(out.view(T, heads, dv), want) < (2e-3 if dtype == torch.float32 else 6e-3)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
def test_the_square_of_relu(dtype):
    from kvcore_amd.ops import library as ops

    for shape in ((37, 80), (5, 13), (1, 1)):
        x = (torch.randn(shape, dtype=F64) * 3).to(dtype).double()
        out = gpu(x, dtype)
        ops.activation(out, out, "relu_squared")
        assert rel(out, torch.relu(x) ** 2) < (1e-7 if dtype == torch.float32 else 4e-3)
    with pytest.raises(ops.KernelError):
        ops.activation(out, out, "relu")


@pytest.mark.parametrize("M,N,K,packed", [(1, 384, 256, False), (8, 1024, 512, True), (13, 200, 96, False),
                                          (40, 512, 256, False), (300, 384, 256, False)])
def test_product_bias_and_activation_in_one_kernel_give_the_bits_of_the_three_steps(M, N, K, packed):
    """Few rows take the weight-streaming product with the activation on its way out; it must equal
    the product stored in bfloat16 and the activation kernel applied to it, bit for bit, and both
    the plain ``relu(x W^T + b)^2``."""
    from kvcore_amd.ops import library as ops

    gen = torch.Generator().manual_seed(M + N)
    x = torch.randn(M, K, generator=gen).to(torch.bfloat16)
    w = (torch.randn(N, K, generator=gen) * K ** -0.5).to(torch.bfloat16)
    b = (torch.randn(N, generator=gen) * 0.3).to(torch.bfloat16)
    wd = gpu(w, torch.bfloat16)
    if packed and ops.can_pack_weight(wd):
        ops.pack_weight(wd)
    fused = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device=DEV)
    ops.linear_act(fused, gpu(x, torch.bfloat16), wd, gpu(b, torch.bfloat16), "relu_squared")
    steps = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device=DEV)
    ops.linear(steps, gpu(x, torch.bfloat16), wd, gpu(b, torch.bfloat16))
    ops.activation(steps, steps, "relu_squared")
    assert torch.equal(fused, steps)
    want = torch.relu(x.double() @ w.double().T + b.double()) ** 2
    assert rel(fused, want) < 8e-3
    f32 = torch.full((M, N), float("nan"), device=DEV)
    ops.linear_act(f32, gpu(x.float()), gpu(w.float()), gpu(b.float()), "relu_squared")
    assert rel(f32, want) < 2e-6


# ------------------------------------------------------------------------- the router
def plain_route(logits, correction, top, groups, keep, scale):
    E = logits.shape[1]
    w = {"router": torch.eye(E, dtype=F64), "correction": correction}
    r = {"experts": E, "top": top, "scale": scale}
    if groups:
        r["groups"] = {"count": groups, "keep": keep}
    return plain.route(logits, w, r)


def route_margin(logits, correction, top, groups, keep) -> torch.Tensor:
    """Per token, how far the choice is from turning: the smallest gap between choice scores."""
    pick = torch.sigmoid(logits) + correction
    gaps = (pick[:, :, None] - pick[:, None, :]).abs() + torch.eye(pick.shape[1], dtype=F64)[None] * 9
    return gaps.flatten(1).min(1).values


@pytest.mark.parametrize("E,top,groups,keep", [(12, 3, 3, 2), (16, 3, 2, 1), (8, 2, 0, 0), (6, 2, 6, 3), (4, 1, 4, 1),
                                               (3, 3, 0, 0), (70, 6, 10, 3), (8, 4, 4, 2)])
def test_routing_with_sigmoid_scores_a_correction_and_groups_worth_their_best_two(E, top, groups, keep):
    from kvcore_amd.ops import library as ops

    gen = torch.Generator().manual_seed(E * 7 + top)
    T = 90
    logits = (torch.randn(T, E, generator=gen, dtype=F64) * 2).float().double()
    # corrections large enough to make choice scores negative and to overturn the plain scores
    correction = (torch.randn(E, generator=gen, dtype=F64) * 0.8 - 0.5).float().double()
    choice = torch.empty(T, top, dtype=torch.int32, device=DEV)
    weight = torch.empty(T, top, dtype=torch.float32, device=DEV)
    ops.moe_route(choice, weight, gpu(logits), top=top, groups=groups or 1, keep=keep or 1, score="sigmoid",
                  correction=gpu(correction), group_best=2, weight_scale=2.5)
    want_e, want_w = plain_route(logits, correction, top, groups, keep, 2.5)
    sure = route_margin(logits, correction, top, groups, keep) > 1e-5
    assert int(sure.sum()) > T * 0.8
    live = min(top, (keep * (E // groups)) if groups else E)
    for t in range(T):
        if not sure[t]:
            continue
        assert choice[t, :live].tolist() == want_e[t, :live].tolist(), t
        assert torch.allclose(weight[t, :live].double().cpu(), want_w[t, :live], atol=2e-6), t
    assert (torch.sigmoid(logits) + correction).min() < 0  # negative choice scores did occur


def test_experts_outside_the_kept_groups_are_never_chosen_for_negative_scores():
    """All choice scores negative: the experts of the groups that are not kept count as minus
    infinity, not as zero, which would beat every allowed expert."""
    from kvcore_amd.ops import library as ops

    logits = torch.tensor([[0.0, 0.1, -0.2, 0.3, 0.2, -0.1]], dtype=F64)
    correction = torch.tensor([-5.0, -6.0, -9.0, -9.5, -7.0, -7.5], dtype=F64)
    choice = torch.empty(1, 2, dtype=torch.int32, device=DEV)
    weight = torch.empty(1, 2, dtype=torch.float32, device=DEV)
    ops.moe_route(choice, weight, gpu(logits), top=2, groups=3, keep=1, score="sigmoid", correction=gpu(correction),
                  group_best=2)
    assert choice[0].tolist() == [0, 1]
    s = torch.sigmoid(logits[0])
    assert math.isclose(float(weight[0, 0]), float(s[0] / (s[0] + s[1])), rel_tol=1e-6)
    assert math.isclose(float(weight.sum()), 1.0, rel_tol=1e-6)
    # a group with one strong expert against a group with two good ones: worth its best one the
    # first wins, worth its best two the second
    logits = torch.tensor([[3.0, -3.0, 0.5, 0.5]], dtype=F64)
    one = torch.empty(1, 1, dtype=torch.int32, device=DEV)
    w1 = torch.empty(1, 1, dtype=torch.float32, device=DEV)
    ops.moe_route(one, w1, gpu(logits), top=1, groups=2, keep=1, score="sigmoid", group_best=1)
    assert one.tolist() == [[0]]
    ops.moe_route(one, w1, gpu(logits), top=1, groups=2, keep=1, score="sigmoid", group_best=2, weight_scale=3.0)
    assert one.tolist() == [[2]] and math.isclose(float(w1), 3.0, rel_tol=1e-6)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("E,top,groups,keep,H,I,T", [(12, 3, 3, 2, 96, 24, 75), (8, 2, 0, 0, 128, 64, 300),
                                                    (3, 3, 0, 0, 40, 8, 1), (4, 1, 4, 1, 40, 16, 2),
                                                    (16, 3, 4, 1, 192, 48, 1100), (5, 2, 0, 0, 36, 20, 19)])
def test_the_feed_forward_of_routed_experts_with_silu(dtype, E, top, groups, keep, H, I, T):
    """The part itself on rows of its own: routing, the arrangement by expert, both products with
    ``silu(gate) * up`` between them (no clamp, nothing added to the up branch) and the weighted
    sum, against the plain function token by token."""
    from kvcore_amd.engine.context import StepBuffers, StepContext
    from kvcore_amd.parts.base import Runtime
    from kvcore_amd.parts.moe import RoutedExperts

    gen = torch.Generator().manual_seed(E + T)
    w = {"router": torch.randn(E, H, generator=gen, dtype=F64) * 0.5,
         "correction": torch.randn(E, generator=gen, dtype=F64) * 0.3}
    for e in range(E):
        w[f"e{e}.gate"] = torch.randn(I, H, generator=gen, dtype=F64) * 0.3
        w[f"e{e}.up"] = torch.randn(I, H, generator=gen, dtype=F64) * 0.3
        w[f"e{e}.down"] = torch.randn(H, I, generator=gen, dtype=F64) * 0.3
    w = {k: (v.float().double() if k in ("router", "correction") else v.to(dtype).double()) for k, v in w.items()}
    part = RoutedExperts(hidden_size=H, experts=E, top=top, expert_size=I, limit=None, alpha=1.0, up_shift=0.0,
                         groups=groups or 1, keep=keep or 1, score="sigmoid", correction=True, group_best=2,
                         weight_scale=1.5,
                         tensor_names={"router": "router", "correction": "correction", "expert": "e{e}",
                                       "gate": "gate", "up": "up", "down": "down"})
    part.setup(Runtime(dtype=dtype, device=torch.device(DEV)))
    params = {}
    for ps in part.param_specs():
        t = torch.empty(ps.shape, dtype=torch.float32 if ps.kind == "vector" else dtype, device=DEV)
        for src in ps.resolved_sources():
            t[src.row:src.row + src.rows] = gpu(w[src.name], t.dtype)
        params[ps.name] = t
    part.bind(params)
    x = torch.randn(T, H, generator=gen, dtype=F64).to(dtype).double()
    mlp = {"kind": "moe", "expert": {"ff": I}, "router": {"experts": E, "top": top, "scale": 1.5}}
    if groups:
        mlp["router"]["groups"] = {"count": groups, "keep": keep}
    want = plain.routed_ff(x, w, mlp)
    sure = route_margin(x @ w["router"].T, w["correction"], top, groups, keep) > 1e-4
    buffers = StepBuffers(torch.device(DEV), token_capacity=T)
    none = torch.zeros(1, dtype=torch.int32, device=DEV)
    ctx = StepContext(num_tokens=T, num_reqs=1, token_ids=none, positions=none, token_req=none, q_start=none,
                      seq_lens=none, slots=none, groups=[], states=[], buffers=buffers, dtype=dtype,
                      device=torch.device(DEV))
    out = part.forward(gpu(x, dtype), ctx, None)
    assert out.dtype == torch.float32 and out.shape == (T, H)
    assert int(sure.sum()) >= T * 0.9
    assert rel(out[sure.to(DEV)], want[sure]) < (3e-6 if dtype == torch.float32 else 8e-3)


# ------------------------------------------------------------ the mixers, through a model
def one_layer_model(tmp_path, mixer_type, mixer, *, width, vocab, seed, special, probe, boost):
    """A folder with one layer and no feed-forward whose query of token ``probe`` and key of token
    ``special`` are made to match: wherever ``special`` is visible from ``probe``, it outweighs
    all other keys together (a score ``boost`` above theirs), and its value is large, so a window
    or a cache that is one token off moves the logits by their own size."""
    import json

    from safetensors.torch import save_file

    gen = torch.Generator().manual_seed(seed)
    config = {"architecture": "Darovik", "vocab": vocab, "width": width, "norm": {"eps": 1e-5},
              "layers": [{"type": mixer_type, "mixer": mixer, "mlp": None}]}
    from kvcore_amd.registry import resolve_architecture
    from kvcore_amd.weights.loader import checkpoint_layout

    arch = resolve_architecture(config)
    layout = checkpoint_layout(arch.build_spec(arch.parse_config(config)))
    w = {}
    for name, (shape, _, _) in layout.items():
        leaf = name.split(".")[-1]
        if leaf.startswith("norm"):
            w[name] = torch.ones(shape)
        elif name == "embed":
            w[name] = torch.randn(shape, generator=gen)
        elif leaf in ("lq1", "lk1", "lq2", "lk2"):
            w[name] = torch.randn(shape, generator=gen) * 0.3
        elif leaf == "sink":
            w[name] = torch.randn(shape, generator=gen)
        elif leaf == "o":  # the mixer's result outweighs the embedding's row in the stream
            w[name] = torch.randn(shape, generator=gen) * (8.0 * shape[-1] ** -0.5)
        else:
            w[name] = torch.randn(shape, generator=gen) * (0.3 * shape[-1] ** -0.5)
    # the directions of the two tokens after the layer's norm (its gain is one)
    e = w["embed"].double()
    hs, hp = (plain.rms(e[t], 1e-5) for t in (special, probe))
    # make every head's (first map's) query of `probe` and key of `special` the same long vector:
    # add rank-one terms to the projections that fire on those two rows only as far as the rows differ
    if mixer_type == "attention":
        H, G, d = mixer["heads"], mixer["kv_heads"], mixer["dim"]
        amp = math.sqrt(boost / (mixer["scale"] * d))
        q = w["l0.mix.q"].double().view(H, 2, d, width)
        k = w["l0.mix.k"].double().view(G, 2, d, width)
        q[:, 0] += amp * hp[None, None, :] / (hp @ hp)
        k[:, 0] += amp * hs[None, None, :] / (hs @ hs)
        w["l0.mix.q"], w["l0.mix.k"] = q.reshape(-1, width).float(), k.reshape(-1, width).float()
        w["l0.mix.v"] = (w["l0.mix.v"].double() + 2.0 * torch.ones(w["l0.mix.v"].shape[0], 1, dtype=F64) * hs[None, :] / (hs @ hs)).float()
    else:
        H, d, rank = mixer["heads"], mixer["dim"], mixer["kv_rank"]
        amp = math.sqrt(boost / (mixer["scale"] * d))
        q = w["l0.mix.q"].double().view(H, d, width)
        q += amp * hp[None, None, :] / (hp @ hp)
        w["l0.mix.q"] = q.reshape(-1, width).float()
        # the latent of `special` gets one large component, which uk spreads over every head's key
        dkv = w["l0.mix.dkv"].double()
        dkv[0] += 6.0 * hs / (hs @ hs)
        w["l0.mix.dkv"] = dkv.float()
        uk = w["l0.mix.uk"].double()
        uk[:, 0] += amp / 2.0
        w["l0.mix.uk"] = uk.float()
        w["l0.mix.dkv.norm"] = torch.ones(rank)
    w = {k: v.to(torch.bfloat16).contiguous() for k, v in w.items()}
    tmp_path.mkdir(parents=True, exist_ok=True)
    (tmp_path / "config.json").write_text(json.dumps(config))
    save_file(w, str(tmp_path / "model.safetensors"))
    return config, {k: v.double() for k, v in w.items()}


def run_cuts(folder, config, weights, tokens, want_at, dtype, page, cuts):
    """The logits at ``want_at`` under each way of cutting ``tokens`` (a list of portion sizes)
    against the plain model's; returns the plain rows."""
    from kvcore_amd.engine.replay import TraceSession
    from tests.test_cuts_gpu import collect

    want = plain.forward(config, weights, tokens)
    for cut in cuts:
        assert sum(cut) == len(tokens)
        s = TraceSession(str(folder), dtype, max_tokens=len(tokens) + 64, block_size=page, poison_cache=True,
                         max_num_seqs=2)
        steps, at = [], 0
        for n in cut:
            asked = [p - at for p in want_at if at <= p < at + n]
            steps.append({"step": len(steps), "entries": [{"id": "a", "tokens": tokens[at: at + n], "want": asked}],
                          "end": ["a"] if at + n == len(tokens) else []})
            at += n
        got = collect(s, steps)
        assert sorted(p for _, p in got) == sorted(want_at)
        limit = 2e-4 if dtype == torch.float32 else 6e-2
        for (_, pos), row in got.items():
            d = row - want[pos]
            err = float((d - d.mean()).pow(2).mean().sqrt() / (want[pos] - want[pos].mean()).pow(2).mean().sqrt())
            assert err < limit, f"cut {cut[:6]}..., position {pos}: {err:.3e}"
    return want


def spread(a, b) -> float:
    d = a - b
    return float((d - d.mean()).pow(2).mean().sqrt() / (a - a.mean()).pow(2).mean().sqrt())


@pytest.mark.parametrize("dtype,dim,vdim,page", [(torch.float32, 24, 40, 8), (torch.bfloat16, 24, 40, 8),
                                                  (torch.bfloat16, 32, 64, 16), (torch.bfloat16, 64, 128, 16),
                                                  (torch.bfloat16, 32, 128, 16), (torch.float32, 20, 7, 4)],
                         ids=["f32", "bf16", "bf16-64", "bf16-128", "bf16-planes", "f32-odd"])
def test_a_key_that_stands_out_just_inside_and_just_outside_the_window(tmp_path, dtype, dim, vdim, page):
    """Two maps a head with a window of 37: the token whose key the probe's query matches lies 36
    positions back (seen) and 37 back (not seen), at a page's border and in its middle; in a whole
    prompt, in portions cut at the edge, and with the probe decoded alone.  The plain model's logits
    at the two places differ by their own size, so a window one token off could not pass."""
    window = 37
    mixer = {"heads": 4, "kv_heads": 2, "dim": dim, "vdim": vdim, "scale": dim ** -0.5, "diff": 0.4,
             "mask": {"size": window}}
    vocab, special, probe = 60, 58, 59
    config, weights = one_layer_model(tmp_path / "m", "attention", mixer, width=64, vocab=vocab, seed=dim + vdim,
                                      special=special, probe=probe, boost=14.0)
    gen = torch.Generator().manual_seed(1)
    for at in (16, 21):  # the special token at a page's first place and inside a page
        tokens = torch.randint(0, 57, (at + window + 12,), generator=gen).tolist()
        tokens[at] = special
        inside, outside = at + window - 1, at + window
        tokens[inside] = tokens[outside] = probe
        n = len(tokens)
        cuts = [[n], [inside, 1, 1, n - outside - 1], [at + 1, window - 3, 2, 2, n - outside - 2],
                [inside - 1] + [1] * (n - inside + 1), [2] * (n // 2) + [1] * (n % 2)]
        want = run_cuts(tmp_path / "m", config, weights, tokens, [at, inside, outside, n - 1], dtype, page, cuts)
        assert spread(want[inside], want[outside]) > 0.15


@pytest.mark.parametrize("dtype,heads,rank,page", [(torch.float32, 3, 40, 8), (torch.bfloat16, 3, 40, 8),
                                                   (torch.bfloat16, 16, 64, 16), (torch.bfloat16, 4, 128, 16),
                                                   (torch.float32, 2, 20, 4)],
                         ids=["f32", "bf16", "bf16-64", "bf16-128", "f32-odd"])
def test_a_key_far_back_and_a_sink_that_outweighs_it(tmp_path, dtype, heads, rank, page):
    """Latent attention sees every earlier token: the token whose key the probe's query matches lies
    600 positions back, among hundreds of others, in a prompt and for a probe decoded alone; without
    it the logits differ by their own size.  With sinks far above every score the layer's output
    all but vanishes, and the engine follows."""
    mixer = {"heads": heads, "dim": 16, "vdim": 24, "kv_rank": rank, "scale": 0.25}
    vocab, special, probe = 60, 58, 59
    config, weights = one_layer_model(tmp_path / "m", "latent_attention", mixer, width=64, vocab=vocab,
                                      seed=heads + rank, special=special, probe=probe, boost=16.0)
    gen = torch.Generator().manual_seed(2)
    tokens = torch.randint(0, 57, (640,), generator=gen).tolist()
    tokens[17] = special
    tokens[617] = tokens[639] = probe
    cuts = [[640], [600, 17, 1, 22], [617] + [1] * 23, [250, 250, 100, 2, 2, 36]]
    want = run_cuts(tmp_path / "m", config, weights, tokens, [17, 616, 617, 639], dtype, page, cuts)
    without = list(tokens)
    without[17] = 3
    assert spread(want[617], plain.forward(config, weights, without)[617]) > 0.2
    # a sink that outweighs every key
    import json

    from safetensors.torch import load_file, save_file

    folder = tmp_path / "sunk"
    folder.mkdir()
    (folder / "config.json").write_text(json.dumps(config))
    t = load_file(str(tmp_path / "m" / "model.safetensors"))
    t["l0.mix.sink"] = torch.full_like(t["l0.mix.sink"], 300.0)
    save_file(t, str(folder / "model.safetensors"))
    sunk = {k: v.double() for k, v in t.items()}
    short = tokens[:80]
    short[70] = probe
    got = run_cuts(folder, config, sunk, short, [0, 70, 79], dtype, page, [[80], [70, 1, 9]])
    assert spread(got[70], plain.forward(config, weights, short)[70]) > 0.3
