"""The Darovik decoder in the engine against the plain implementation, under every way of cutting
the work: whole prompts, prompts then single tokens, portions down to two tokens, unequal requests
side by side, pages and slots that are given back and used again, long decoding, and greedy
generation through the engine's own entry point and scheduler."""

from __future__ import annotations

import copy

import pytest
import torch

from tests.darovik_helpers import CONFIGS, load_model_folder, make_model_dir
from tests.helpers import random_tokens
from tests.plain import darovik as plain
from tests.test_cuts_gpu import collect

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.bfloat16]


@pytest.fixture(scope="module")
def models(tmp_path_factory):
    out = {}
    for name, (config, page) in CONFIGS.items():
        folder = make_model_dir(tmp_path_factory.mktemp(f"darovik_{name}"), config, seed=31 + len(out))
        cfg, weights = load_model_folder(folder)
        out[name] = (folder, cfg, weights, page)
    return out


_oracle: dict = {}


def oracle(name, cfg, weights, tokens):
    key = (name, tuple(tokens))
    if key not in _oracle:
        _oracle[key] = plain.forward(cfg, weights, tokens)
    return _oracle[key]


_floors: dict = {}


def floors_for(name, cfg, weights, seqs, want, dtype):
    """``rounding_floor`` for every request of ``seqs``, in bfloat16 (float32 keeps the fixed limit)."""
    if dtype == torch.float32:
        return None
    out = {}
    for k, tokens in seqs.items():
        key = (name, tuple(tokens))
        if key not in _floors:
            _floors[key] = rounding_floor(cfg, weights, tokens, want[k], dtype)
        out[k] = _floors[key]
    return out


def session_for(folder, dtype, page, max_tokens, **kw):
    from kvcore_amd.engine.replay import TraceSession

    return TraceSession(str(folder), dtype, max_tokens=max_tokens, block_size=page, poison_cache=True, **kw)


def row_error(row, ref) -> float:
    d = row - ref
    d = d - d.mean()
    return float(d.pow(2).mean().sqrt() / (ref - ref.mean()).pow(2).mean().sqrt())


def rounding_floor(cfg, weights, tokens, want, dtype) -> list[float]:
    """How far the plain model's own logits move, position by position, when every weight is moved
    by a random relative amount of the size of ``dtype``'s rounding: what rounding alone may do to
    this model at this place.  A drawn model can be touchy (two maps that nearly cancel before
    their norm, two experts that score alike), and then no fixed bound separates rounding from a
    fault; a multiple of this does."""
    size = 2.0 ** -24 if dtype == torch.float32 else 2.0 ** -9
    gen = torch.Generator().manual_seed(99)
    moved = {k: v * (1 + size * torch.randn(v.shape, generator=gen, dtype=v.dtype)) for k, v in weights.items()}
    other = plain.forward(cfg, moved, tokens)
    return [row_error(other[i], want[i]) for i in range(len(tokens))]


def compare(got, expect_by_id, dtype, floors=None, excused=0):
    """Logit rows against the plain model's: the difference with its mean taken off, root mean
    square over the vocabulary, relative to the root mean square of the row itself.  float32
    differs by the order of its sums only, and every position must agree: that pins the routing
    itself.  bfloat16 rounds activations to 8 bits at a dozen places a layer (measured: 0.01 of a
    row's size at eight layer runs, about what rounding the weights does to the plain model), and
    where two experts' choice scores lie within that rounding the router turns and the token's row
    moves by a tenth of its size; so in bfloat16 one position in ten (``excused`` says so) may lie
    anywhere, the others within the limit, and half of all within the fixed limit.  With
    ``floors`` (see ``rounding_floor``) a position's limit is at least five times what rounding
    alone does there."""
    base = 2e-4 if dtype == torch.float32 else 8e-2
    assert got, "nothing was compared"
    worst, within, far = 0.0, 0, []
    for (rid, pos), row in sorted(got.items()):
        ref = expect_by_id[rid][pos]
        assert torch.isfinite(row).all(), f"non-finite logits at {rid}:{pos}"
        err = row_error(row, ref)
        within += err <= base
        limit = base if floors is None else max(base, 5 * floors[rid][pos])
        if err <= limit:
            worst = max(worst, err)
        else:
            far.append(f"{rid}:{pos} differs by {err:.3e} of its size (limit {limit})")
    allowed = max(excused, len(got) // 10) if dtype == torch.bfloat16 else 0
    assert len(far) <= allowed, (len(far), len(got), far[:5])
    assert 2 * within >= len(got), f"only {within} of {len(got)} positions lie within {base}"
    return worst


def test_the_test_weights_make_every_mechanism_count(models):
    """What the other tests rest on: without the sinks, with a window one position off, with
    another `lambda`, without the corrections, with groups worth their best one, with another
    multiplier or with the copies' links undone, the plain model's logits move by far more than
    the limits of the comparisons."""
    folder, cfg, weights, page = models["A"]
    tokens = random_tokens(60, cfg["vocab"], 5)
    base = plain.forward(cfg, weights, tokens)

    def moved(cfg2, w2):
        other = plain.forward(cfg2, w2, tokens)
        return float((other - base).pow(2).mean().sqrt() / base.pow(2).mean().sqrt())

    no_sink = {k: (v - 30.0 if k.endswith("sink") else v) for k, v in weights.items()}
    assert moved(cfg, no_sink) > 1e-2
    for layer in (1, 3):
        for step in (1, -1):
            off = copy.deepcopy(cfg)
            off["layers"][layer]["mixer"]["mask"]["size"] += step
            assert moved(off, weights) > 1e-3
    off = copy.deepcopy(cfg)
    off["layers"][1]["mixer"]["diff"] = 0.5
    assert moved(off, weights) > 1e-2
    assert moved(cfg, {k: (v * 0 if k.endswith("lq1") else v) for k, v in weights.items()}) > 1e-3
    assert moved(cfg, {k: (v * 0 if k.endswith("correction") else v) for k, v in weights.items()}) > 1e-2
    off = copy.deepcopy(cfg)
    off["layers"][1]["mlp"]["router"]["scale"] = 1.0
    assert moved(off, weights) > 1e-2
    off = copy.deepcopy(cfg)
    off["residual_mult"] = 1.0
    assert moved(off, weights) > 1e-2
    assert moved(cfg, {k: (v.T.contiguous() if k.endswith("hc1.mix") else v) for k, v in weights.items()}) > 1e-2
    assert moved(cfg, {k: (v * 0 + 1 if k.endswith("hc2.in") else v) for k, v in weights.items()}) > 1e-2
    assert moved(cfg, {k: (v * 0 if k.endswith(".b") else v) for k, v in weights.items()}) > 1e-2
    off = copy.deepcopy(cfg)
    off["loop"]["times"] = 2
    assert moved(off, weights) > 1e-2


@pytest.mark.parametrize("dtype", DTYPES, ids=["f32", "bf16"])
@pytest.mark.parametrize("name", list(CONFIGS))
def test_whole_prompts_then_single_tokens_then_portions(models, name, dtype):
    folder, cfg, weights, page = models[name]
    V = cfg["vocab"]
    tokens = random_tokens(75, V, 5)
    want = {"a": oracle(name, cfg, weights, tokens)}
    floors = floors_for(name, cfg, weights, {"a": tokens}, want, dtype)
    s = session_for(folder, dtype, page, 256)
    # whole
    got = collect(s, [{"step": 0, "entries": [{"id": "a", "tokens": tokens, "want": list(range(75))}], "end": ["a"]}])
    compare(got, want, dtype, floors, excused=2)
    # a prompt, then token by token (the slot and the pages of the first run are used again)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": tokens[:40], "want": [0, 39]}], "end": []}]
    for i in range(40, 75):
        steps.append({"step": i, "entries": [{"id": "a", "tokens": tokens[i: i + 1], "want": [0]}],
                      "end": ["a"] if i == 74 else []})
    compare(collect(s, steps), want, dtype, floors, excused=1)
    # token by token from the very first token
    steps = [{"step": i, "entries": [{"id": "a", "tokens": tokens[i: i + 1], "want": [0]}],
              "end": ["a"] if i == 29 else []} for i in range(30)]
    compare(collect(s, steps), want, dtype, floors, excused=1)
    # portions of every size down to two tokens and one, cut inside pages and windows
    steps, at = [], 0
    for n in (2, 3, 2, 1, 9, 2, 17, 1, 1, 2, 30, 5):
        steps.append({"step": len(steps), "entries": [{"id": "a", "tokens": tokens[at: at + n],
                                                       "want": list(range(n))}],
                      "end": ["a"] if at + n == 75 else []})
        at += n
    assert at == 75
    compare(collect(s, steps), want, dtype, floors, excused=2)


@pytest.mark.parametrize("dtype", DTYPES, ids=["f32", "bf16"])
@pytest.mark.parametrize("name", list(CONFIGS))
def test_unequal_requests_side_by_side_with_slots_used_again(models, name, dtype):
    """Up to three live requests in two slots' worth of pages more than one needs: portions of
    some beside single tokens of others, requests that pause, end and are followed by new ones
    in the same slots and pages (the cache is poisoned when pages are given back)."""
    folder, cfg, weights, page = models[name]
    V = cfg["vocab"]
    seqs = {"a": random_tokens(61, V, 1), "b": random_tokens(33, V, 2), "c": random_tokens(9, V, 3),
            "d": random_tokens(47, V, 4), "e": random_tokens(2, V, 5), "f": random_tokens(1, V, 6)}
    want = {k: oracle(name, cfg, weights, v) for k, v in seqs.items()}
    s = session_for(folder, dtype, page, 192, max_num_seqs=3)
    at = {k: 0 for k in seqs}

    def entry(k, n):
        lo = at[k]
        n = min(n, len(seqs[k]) - lo)
        at[k] += n
        return {"id": k, "tokens": seqs[k][lo: lo + n], "want": list(range(n))}

    plan = [
        [("a", 20), ("b", 2)], [("a", 1), ("b", 13), ("c", 9)], [("a", 7), ("b", 1)],
        [("b", 1), ("d", 2), ("a", 1)], [("d", 30), ("a", 1), ("b", 1)], [("a", 31)],
        [("b", 15), ("d", 1)], [("d", 14), ("e", 2)], [("f", 1)],
    ]
    steps = []
    for i, group in enumerate(plan):
        entries = [entry(k, n) for k, n in group]
        ended = [k for k, _ in group if at[k] == len(seqs[k])]
        steps.append({"step": i, "entries": entries, "end": ended})
    assert all(at[k] == len(v) for k, v in seqs.items())
    compare(collect(s, steps), want, dtype, floors_for(name, cfg, weights, seqs, want, dtype), excused=3)


@pytest.mark.parametrize("dtype", DTYPES, ids=["f32", "bf16"])
def test_long_decoding_through_graphs(models, dtype):
    """Three hundred single tokens after a short prompt, two requests side by side (the steps of
    single tokens are captured into a graph and replayed), one of them starting later; the
    windows of 48 and 100 positions pass over decoded tokens, and their pages come back."""
    folder, cfg, weights, page = models["B"]
    V = cfg["vocab"]
    seqs = {"a": random_tokens(330, V, 7), "b": random_tokens(290, V, 8)}
    want = {k: oracle("B", cfg, weights, v) for k, v in seqs.items()}
    s = session_for(folder, dtype, page, 704)
    assert s.model.graph_safe()
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": seqs["a"][:30], "want": [29]}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": seqs["a"][30:31], "want": [0]},
                                     {"id": "b", "tokens": seqs["b"][:10], "want": [9]}], "end": []}]
    for i in range(280):
        steps.append({"step": 2 + i, "entries": [{"id": "a", "tokens": seqs["a"][31 + i: 32 + i], "want": [0]},
                                                 {"id": "b", "tokens": seqs["b"][10 + i: 11 + i], "want": [0]}],
                      "end": []})
    got = collect(s, steps)
    assert s.runner.graph_replays > 200
    compare(got, want, dtype, floors_for("B", cfg, weights, seqs, want, dtype), excused=6)


@pytest.mark.parametrize("dtype", DTYPES, ids=["f32", "bf16"])
@pytest.mark.parametrize("name", ["A", "B", "D"])
def test_the_stream_after_every_layer_run(models, name, dtype):
    """The float32 stream itself (the sum of its copies), layer run by layer run, against the plain
    model's: a step of one whole prompt with a hook on the blocks; what a block leaves pending for
    the next block's read is settled into a copy of the stream first."""
    folder, cfg, weights, page = models[name]
    tokens = random_tokens(40, cfg["vocab"], 21)
    layers: list = []
    plain.forward(cfg, weights, tokens, layers)
    s = session_for(folder, dtype, page, 64)
    seen = []
    copies = s.model.stream_copies
    assert copies == (cfg.get("streams") or 1)
    for block in s.model.blocks:
        inner = block.forward

        def hooked(delta, residual, ctx, call, next_block=None, inner=inner, block=block):
            out = inner(delta, residual, ctx, call, next_block=next_block)
            settled = residual[: ctx.num_tokens].clone()
            block.settle(out, settled, ctx)
            seen.append(settled.view(ctx.num_tokens, copies, -1).sum(1).double().cpu())
            return out

        block.forward = hooked
    s.run_step({"step": 0, "entries": [{"id": "a", "tokens": tokens, "want": [39]}], "end": ["a"]})
    assert len(seen) == len(plain.layer_order(cfg))
    # token by token; in bfloat16 a router may turn for a token where two experts score alike
    limit = 1e-4 if dtype == torch.float32 else 5e-2
    for i, got in enumerate(seen):
        per = (got - layers[i]).pow(2).mean(1).sqrt() / layers[i].pow(2).mean(1).sqrt()
        above = int((per >= limit).sum())
        assert above <= (0 if dtype == torch.float32 else 4), f"layer run {i}: {above} tokens, worst {float(per.max()):.3e}"
        assert float(per.median()) < limit / 2, f"layer run {i}: median {float(per.median()):.3e}"


@pytest.mark.parametrize("seed", [0, 1, 2, 3, 4, 5, 6, 7, 8, 9])
def test_configurations_drawn_at_random(tmp_path, seed):
    """Models whose every size, constant and layer order is drawn from a seed (widths that 8 does
    not divide, maps of 8 to 64 with values of any size, windows of 1 to 128 positions and none,
    latents of 8 to 128, one to eight copies of the stream or none, loops, experts in groups), in
    float32 and in bfloat16: two requests side by side, portions, then single tokens."""
    import random

    from tests.darovik_helpers import random_config

    cfg = random_config(random.Random(seed))
    folder = make_model_dir(tmp_path / "drawn", cfg, seed=seed)
    c, w = load_model_folder(folder)
    seqs = {"a": random_tokens(150, cfg["vocab"], seed + 1), "b": random_tokens(70, cfg["vocab"], seed + 2)}
    want = {k: plain.forward(c, w, v) for k, v in seqs.items()}
    for dtype in DTYPES:
        floors = {k: rounding_floor(c, w, v, want[k], dtype) for k, v in seqs.items()}
        s = session_for(folder, dtype, 16, 320, max_num_seqs=4)
        at = {"a": 0, "b": 0}
        steps = []
        for who, count in [("a", 37), ("b", 2), ("a", 50), ("b", 33)] + [("ab", 1)] * 30 + [("a", 33), ("b", 5)]:
            entries = []
            for k in who:
                lo, hi = at[k], min(at[k] + count, len(seqs[k]))
                if hi > lo:
                    entries.append({"id": k, "tokens": seqs[k][lo:hi], "want": list(range(hi - lo))})
                    at[k] = hi
            if entries:
                steps.append({"step": len(steps), "entries": entries, "end": [k for k in who if at[k] == len(seqs[k])]})
        got = collect(s, steps)
        assert len(got) == 220
        compare(got, want, dtype, floors, excused=10)


def test_the_attention_layers_run_the_kernels_they_are_meant_to(models):
    """In bfloat16 the two-map attention with joint keys of 64 and of 128, and the latent attention
    with rows of 64 and 128, take the matrix-core kernels (portions and single tokens); values of
    twice the joint key's size run them once a plane."""
    from kvcore_amd.ops import library as ops

    folder, cfg, weights, page = models["B"]
    m = cfg["layers"][0]["mixer"]
    assert ops.prefill_attention_supported(2 * m["heads"], m["kv_heads"], 2 * m["dim"], page, torch.bfloat16)
    assert ops.decode_attention_supported(2 * m["heads"], m["kv_heads"], 2 * m["dim"], page, torch.bfloat16)
    lat = cfg["layers"][3]["mixer"]
    assert ops.prefill_attention_supported(lat["heads"], 1, lat["kv_rank"], page, torch.bfloat16)
    s = session_for(folder, torch.bfloat16, page, 128)
    names = []
    real_prefill, real_decode, real_general = ops.prefill_attention, ops.decode_attention, ops.paged_attention
    try:
        ops.prefill_attention = lambda *a, **k: (names.append("portion"), real_prefill(*a, **k))[1]
        ops.decode_attention = lambda *a, **k: (names.append("single"), real_decode(*a, **k))[1]
        ops.paged_attention = lambda *a, **k: (names.append("general"), real_general(*a, **k))[1]
        tokens = random_tokens(71, cfg["vocab"], 9)
        s.run_step({"step": 0, "entries": [{"id": "a", "tokens": tokens[:70], "want": [69]}], "end": []})
        # four layers, the third with two planes of values, and the whole model twice
        assert names == ["portion"] * 10
        del names[:]
        s.run_step({"step": 1, "entries": [{"id": "a", "tokens": tokens[70:], "want": [0]}], "end": ["a"]})
        assert names == ["single"] * 10
    finally:
        ops.prefill_attention, ops.decode_attention, ops.paged_attention = real_prefill, real_decode, real_general


@pytest.mark.parametrize("dtype", DTYPES, ids=["f32", "bf16"])
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_greedy_generation_through_the_engine(models, name, dtype):
    """``LLMEngine.generate`` with the scheduler cutting prompts into portions of 16 tokens:
    every generated token is the plain model's greedy choice given the tokens before it (a
    choice is skipped where the plain model's two best logits lie closer than rounding
    can tell apart)."""
    from kvcore_amd import CacheConfig, KVCoreConfig, ModelConfig, SamplingParams, SchedulerConfig
    from kvcore_amd.engine.llm_engine import GenerationRequest, LLMEngine

    folder, cfg, weights, page = models[name]
    V = cfg["vocab"]
    config = KVCoreConfig(
        model_config=ModelConfig(model=str(folder), dtype="float32" if dtype == torch.float32 else "bfloat16",
                                 max_model_len=128),
        cache_config=CacheConfig(block_size=page, num_gpu_blocks=40 if page >= 8 else 80),
        scheduler_config=SchedulerConfig(max_num_seqs=3, max_num_scheduled_tokens=24,
                                         long_prefill_token_threshold=16))
    engine = LLMEngine(config)
    prompts = {"r0": random_tokens(37, V, 11), "r1": random_tokens(5, V, 12), "r2": random_tokens(50, V, 13),
               "r3": random_tokens(18, V, 14), "r4": random_tokens(1, V, 15)}
    params = SamplingParams(max_tokens=12, temperature=0.0)
    outs = engine.generate([GenerationRequest(k, params, prompt_token_ids=tuple(v)) for k, v in prompts.items()])
    by_id = {o.request_id: list(o.output_token_ids) for o in outs}
    assert set(by_id) == set(prompts)
    margin = 1e-4 if dtype == torch.float32 else 5e-2
    checked = wrong = 0
    for rid, prompt in prompts.items():
        gen = by_id[rid]
        assert len(gen) == 12
        logits = plain.forward(cfg, weights, prompt + gen)
        for i, tok in enumerate(gen):
            row = logits[len(prompt) + i - 1]
            top = torch.topk(row, 2).values
            if float(top[0] - top[1]) < margin * float(row.std()):
                continue
            wrong += int(torch.argmax(row)) != tok
            checked += 1
    assert checked > 40
    assert wrong == 0 if dtype == torch.float32 else wrong <= 1, f"{wrong} of {checked} tokens differ"


def test_command_lines(models, tmp_path):
    """``bin/kvcore_offline_batch`` generates with a Darovik folder, and ``bin/trace_run`` replays
    steps on it and writes logits that match the plain model's."""
    import json
    import subprocess
    import sys
    from pathlib import Path

    import numpy as np

    repo = Path(__file__).resolve().parent.parent
    folder, cfg, weights, page = models["A"]
    cmd = [sys.executable, str(repo / "bin" / "kvcore_offline_batch"), "--model", str(folder),
           "--dtype", "float32", "--prompt-lens", "7,16", "--max-tokens", "5", "--seed", "3",
           "--max-num-seqs", "4", "--max-num-scheduled-tokens", "32", "--num-gpu-blocks", "32",
           "--block-size", str(page), "--max-model-len", "128",
           "--ignore-eos", "--log-level", "WARNING", "--no-log-file"]
    proc = subprocess.run(cmd, capture_output=True, text=True, timeout=240)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert proc.stdout.count("finish_reason=length") == 2

    tokens = random_tokens(21, cfg["vocab"], 17)
    steps = [{"step": 0, "entries": [{"id": "x", "tokens": tokens[:13], "want": [0, 12]}], "end": []},
             {"step": 1, "entries": [{"id": "x", "tokens": tokens[13:15], "want": []}], "end": []},
             {"step": 2, "entries": [{"id": "x", "tokens": tokens[15:], "want": [5]}], "end": ["x"]}]
    out_dir = tmp_path / "logits"
    cmd = [str(repo / "bin" / "trace_run"), "--model", str(folder), "--dtype", "float32", "--out", str(out_dir),
           "--max-tokens", "64", "--block-size", str(page)]
    proc = subprocess.run(cmd, input="\n".join(json.dumps(s) for s in steps) + "\n", capture_output=True,
                          text=True, timeout=240)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert [l for l in proc.stdout.splitlines() if l.startswith("done")] == ["done 0", "done 1", "done 2"]
    assert not (out_dir / "1.f32").exists()
    want = oracle("A", cfg, weights, tokens)
    first = np.fromfile(out_dir / "0.f32", dtype="<f4").reshape(2, -1)
    last = np.fromfile(out_dir / "2.f32", dtype="<f4").reshape(1, -1)
    got = {("x", 0): torch.from_numpy(first[0]).double(), ("x", 12): torch.from_numpy(first[1]).double(),
           ("x", 20): torch.from_numpy(last[0]).double()}
    compare(got, {"x": want}, torch.float32)
