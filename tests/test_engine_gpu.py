"""Generation through the entry points against the plain implementation; batching, portions, preemption, sampling."""

from __future__ import annotations

import json
import subprocess
import sys
from pathlib import Path

import pytest
import torch

import plain_llama as pl
from tiny import BF16_ULP, TINY, random_tokens

pytestmark = pytest.mark.gpu
ROOT = Path(__file__).resolve().parent.parent
NEW = {"A": 16, "B": 24}


def prompts_of(name):
    vocab = TINY[name]["cfg"]["vocab_size"]
    return [random_tokens(n, vocab, 7 * n + 1) for n in TINY[name]["prompts"]]


_PLAIN, _MODELS = {}, {}


def plain_greedy(folder, name, dtype):
    if (name, dtype) not in _PLAIN:
        cfg, w = pl.read_config(folder), pl.read_weights(folder, dtype)
        _PLAIN[name, dtype] = [pl.greedy_continuation(w, cfg, p, NEW[name], dtype) for p in prompts_of(name)]
    return _PLAIN[name, dtype]


def model_of(folder, name, dtype):
    from nanospec_amd import load_model

    if (name, dtype) not in _MODELS:
        _MODELS[name, dtype] = load_model(folder, dtype=dtype)
    return _MODELS[name, dtype]


def assert_tokens(ours, ref_tokens, ref_logits, strict, what):
    """Token for token; when not strict a difference is accepted only where the plain implementation's logit for our
    token is within 8 bf16 ulps of its best at that step (reference: tests/conftest.py:42-55)."""
    for k, (a, b) in enumerate(zip(ours, ref_tokens)):
        if a == b:
            continue
        assert not strict, f"{what}: differs at step {k}: {ours} vs {ref_tokens}"
        row = ref_logits[k].float()
        gap = float(row.max() - row[a])
        assert gap <= 8 * BF16_ULP * float(row.abs().max()), f"{what}: differs at step {k} with a clear gap {gap}"
        return
    assert len(ours) == len(ref_tokens), what


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("name", ["A", "B"])
def test_greedy_generation_matches_plain(tiny_folders, name, dtype):
    """Engine.generate with continuous batching, a token budget and portions, graphs on."""
    from nanospec_amd import Engine, EngineConfig, SamplingParams

    ref = plain_greedy(tiny_folders[name], name, dtype)
    model = model_of(tiny_folders[name], name, dtype)
    eng = Engine(model, EngineConfig(num_blocks=128, block_size=TINY[name]["page"], max_admit=2, max_step_tokens=48, prefill_chunk=32,
                                     record_logits=True))
    reqs = [eng.add(p, SamplingParams(max_tokens=NEW[name])) for p in prompts_of(name)]
    while eng.sched.has_work:
        eng.step()
        eng.cache.check()
    for i, (r, (toks, logits)) in enumerate(zip(reqs, ref)):
        assert_tokens(r.out_tokens, toks, logits, dtype == torch.float32, f"{name} prompt {i}")
        if r.out_tokens == toks:
            ours = torch.stack(r.step_logits)
            tol = 1e-4 if dtype == torch.float32 else 8 * BF16_ULP
            err = ((ours - logits).abs().amax(-1) / logits.abs().amax(-1)).max()
            assert err <= tol, f"{name} prompt {i}: step logits off by {err:.2e} of the row's largest"
    assert eng.cache.num_free() == eng.usable_blocks


@pytest.mark.parametrize("name", ["A", "B"])
def test_generate_entry_point_and_command_line(tiny_folders, name):
    from nanospec_amd import SamplingParams, generate

    ref = plain_greedy(tiny_folders[name], name, torch.float32)
    outs = generate(str(tiny_folders[name]), prompts_of(name), SamplingParams(max_tokens=NEW[name]), dtype="float32",
                    block_size=TINY[name]["page"])
    assert outs == [r[0] for r in ref]
    args = [sys.executable, "-m", "nanospec_amd", "--model", str(tiny_folders[name]), "--dtype", "float32", "--max-tokens", str(NEW[name]),
            "--block-size", str(TINY[name]["page"]), "--logprobs"]
    for p in prompts_of(name)[:2]:
        args += ["--prompt-ids", ",".join(map(str, p))]
    proc = subprocess.run(args, capture_output=True, text=True, cwd=ROOT, timeout=600)
    assert proc.returncode == 0, proc.stderr[-2000:]
    rows = [json.loads(l) for l in proc.stdout.strip().split("\n")]
    assert [r["output_ids"] for r in rows] == [r[0] for r in ref[:2]]
    lp = torch.log_softmax(ref[0][1][0], -1)[ref[0][0][0]]
    assert abs(rows[0]["logprobs"][0] - float(lp)) < 1e-4


def run_engine(model, prompts, params, **cfg):
    from nanospec_amd import Engine, EngineConfig

    eng = Engine(model, EngineConfig(**cfg))
    reqs = [eng.add(p, s) for p, s in zip(prompts, params)]
    order = []
    while eng.sched.has_work:
        order += [r.id for r in eng.step()]
        eng.cache.check()
    assert eng.cache.num_free() == eng.usable_blocks
    return reqs, order, eng


def test_batched_equals_one_by_one_and_lengths_differ(tiny_folders):
    """reference tests/test_batching.py:50-74: whatever the admission rate, every request's output equals its own run
    alone; different max_tokens make requests finish out of order; the pool is returned."""
    from nanospec_amd import SamplingParams

    name = "B"
    model = model_of(tiny_folders[name], name, torch.float32)
    prompts = prompts_of(name) * 2
    params = [SamplingParams(max_tokens=(i % 5) * 5 + 2) for i in range(len(prompts))]
    alone = []
    for p, s in zip(prompts, params):
        r, _, _ = run_engine(model, [p], [s], num_blocks=64, block_size=8, cuda_graphs=False)
        alone.append(r[0].out_tokens)
    for max_admit in (1, 4, 32):
        reqs, order, _ = run_engine(model, prompts, params, num_blocks=160, block_size=8, max_admit=max_admit)
        assert [r.out_tokens for r in reqs] == alone, f"max_admit={max_admit}"
        assert all(len(r.out_tokens) == s.max_tokens for r, s in zip(reqs, params))
        assert order != sorted(order)


def test_portions_and_whole_prompts_agree_and_small_pool_waits(tiny_folders):
    """A token budget, portions and a pool for about two requests: admission throttles, nothing raises
    (reference tests/test_batch_scale.py:41-57), and the tokens are those of unconstrained runs."""
    from nanospec_amd import SamplingParams

    name = "A"
    model = model_of(tiny_folders[name], name, torch.float32)
    prompts = prompts_of(name) * 3
    params = [SamplingParams(max_tokens=10)] * len(prompts)
    free, _, _ = run_engine(model, prompts, params, num_blocks=256, block_size=4)
    tight, _, eng = run_engine(model, prompts, params, num_blocks=2 * -(-(33 + 10) // 4) + 2, block_size=4, max_step_tokens=12, prefill_chunk=7)
    assert [r.out_tokens for r in tight] == [r.out_tokens for r in free]
    assert eng.steps > 30


def test_preemption_gives_the_same_tokens(tiny_folders):
    from nanospec_amd import SamplingParams

    name = "B"
    model = model_of(tiny_folders[name], name, torch.float32)
    prompts = [p[:20] for p in prompts_of(name)[2:]] * 2
    params = [SamplingParams(max_tokens=30)] * len(prompts)
    calm, _, _ = run_engine(model, prompts, params, num_blocks=128, block_size=8)
    rough, _, eng = run_engine(model, prompts, params, num_blocks=17, block_size=8, on_exhaustion="preempt", prefill_chunk=16)
    assert eng.sched.preempted_total > 0, "the pool was meant to run out"
    assert [r.out_tokens for r in rough] == [r.out_tokens for r in calm]


@pytest.mark.parametrize("policy,graphs,lookahead", [("preempt", True, True), ("reserve", True, True), ("preempt", False, False)])
def test_requests_arriving_over_time_in_a_pool_that_is_too_small(tiny_folders, policy, graphs, lookahead):
    """Thirty requests of random lengths arrive a few per step into a pool that holds a handful of them: whatever is
    preempted, recomputed, looked ahead or replayed from a graph, every request's tokens are the plain implementation's,
    and no page is lost."""
    import random

    from nanospec_amd import Engine, EngineConfig, SamplingParams

    rnd = random.Random(4)
    folder = tiny_folders["A"]
    cfg, w = pl.read_config(folder), pl.read_weights(folder, torch.float32)
    eng = Engine(model_of(folder, "A", torch.float32),
                 EngineConfig(num_blocks=40, block_size=4, max_admit=5, max_running=12, max_step_tokens=48, prefill_chunk=20,
                              on_exhaustion=policy, cuda_graphs=graphs, lookahead=lookahead))
    todo = [(random_tokens(rnd.randint(1, 50), 256, 1000 + i), rnd.randint(1, 20)) for i in range(30)]
    arriving, live, steps = iter(todo), [], 0
    while len(live) < len(todo) or eng.has_work:
        for _ in range(rnd.randint(0, 2)):
            nxt = next(arriving, None)
            if nxt is not None:
                live.append(eng.add(nxt[0], SamplingParams(max_tokens=nxt[1])))
        if eng.has_work:
            eng.step()
            steps += 1
            if steps % 20 == 0:
                eng.cache.check()
    eng.cache.check()
    assert eng.cache.num_free(0) == 40 - (1 if graphs else 0)  # all but the page of the captured graphs' pad rows
    if policy == "preempt":
        assert sum(r.preemptions for r in live) > 0
    for r, (prompt, n_new) in zip(live, todo):
        assert r.out_tokens == pl.greedy_continuation(w, cfg, prompt, n_new, torch.float32)[0], (prompt, r.preemptions)


def test_temperature_sampling_is_seeded_and_batch_independent(tiny_folders):
    """Per-request generators (reference sched/scheduler.py:64): the same seed gives the same tokens alone or in a batch,
    and every one of a request's 24 tokens is the plain implementation's inverse-CDF draw from the plain logits of the
    sequence so far with the request's own next uniform number: the same token, or one no more than rounding away in
    the cumulative distribution."""
    from nanospec_amd import SamplingParams

    name = "B"
    model = model_of(tiny_folders[name], name, torch.float32)
    prompts = prompts_of(name)
    params = [SamplingParams(max_tokens=24, temperature=0.8, seed=2 + i) for i in range(len(prompts))]
    batch, _, _ = run_engine(model, prompts, params, num_blocks=160, block_size=8)
    again, _, _ = run_engine(model, prompts, params, num_blocks=160, block_size=8, max_admit=1, cuda_graphs=False)
    assert [r.out_tokens for r in batch] == [r.out_tokens for r in again]
    other, _, _ = run_engine(model, prompts[:1], [SamplingParams(max_tokens=24, temperature=0.8, seed=99)], num_blocks=64, block_size=8)
    assert other[0].out_tokens != batch[0].out_tokens
    cfg, w = pl.read_config(tiny_folders[name]), pl.read_weights(tiny_folders[name], torch.float32)
    exact = 0
    for p, s, r in zip(prompts, params, batch):
        assert len(r.out_tokens) == 24
        gen = torch.Generator().manual_seed(s.seed)
        rows = pl.logits_of_sequence(w, cfg, p + r.out_tokens[:-1])[len(p) - 1 :]  # the logits each token was drawn from
        for k, got in enumerate(r.out_tokens):
            u = float(torch.rand(1, generator=gen))
            lp = pl.processed_logprobs(rows[k], 0.8, 0, 1.0)
            want = pl.draw_token(lp, u)
            cdf = torch.cumsum(torch.exp(lp.double()), 0)
            assert lp[got] > -30 and abs(float(cdf[got]) - float(cdf[want])) < 1e-4, (p[:3], k, got, want)
            exact += got == want
    assert exact >= 0.95 * 24 * len(prompts)  # a draw that lands within rounding of a boundary is rare


def test_profile_records_the_phases_of_every_step(tiny_folders):
    """EngineConfig(profile=True) (reference engine/engine.py:83-95): event timings per phase in Engine.prof, one entry per
    step for the forward pass and one per sampling pass; the tokens are those of an unprofiled run."""
    from nanospec_amd import SamplingParams

    name = "A"
    model = model_of(tiny_folders[name], name, torch.float32)
    prompts = prompts_of(name)
    params = [SamplingParams(max_tokens=6)] * len(prompts)
    base, _, _ = run_engine(model, prompts, params, num_blocks=96, block_size=4)
    reqs, _, eng = run_engine(model, prompts, params, num_blocks=96, block_size=4, profile=True)
    assert [r.out_tokens for r in reqs] == [r.out_tokens for r in base]
    assert set(eng.prof) == {"forward", "sample"}
    assert len(eng.prof["forward"]) == eng.steps and 0 < len(eng.prof["sample"]) <= eng.steps
    assert all(t > 0 for t in eng.prof["forward"]) and all(t >= 0 for t in eng.prof["sample"])


def test_top_k_top_p_and_logprobs_through_the_engine(tiny_folders):
    from nanospec_amd import SamplingParams

    name = "A"
    model = model_of(tiny_folders[name], name, torch.float32)
    cfg, w = pl.read_config(tiny_folders[name]), pl.read_weights(tiny_folders[name], torch.float32)
    p = prompts_of(name)[1]
    reqs, _, _ = run_engine(model, [p] * 6, [SamplingParams(max_tokens=1, temperature=1.0, top_k=3, seed=i, logprobs=True) for i in range(6)],
                            num_blocks=64, block_size=4)
    row = pl.logits_of_sequence(w, cfg, p)[-1]
    top3 = set(row.topk(3).indices.tolist())
    lp3 = pl.processed_logprobs(row, 1.0, 3, 1.0)
    for r in reqs:
        t = r.out_tokens[0]
        assert t in top3
        assert abs(r.logprobs[0].sample_logprob - float(lp3[t])) < 1e-4
        assert abs(r.logprobs[0].logprob - float(torch.log_softmax(row, -1)[t])) < 1e-4


def test_eos_stops_and_is_kept(tiny_folders, tmp_path):
    """The stopping token is kept in the output and nothing follows it (reference engine/engine.py:155-163)."""
    import shutil

    from nanospec_amd import SamplingParams, generate

    ref = plain_greedy(tiny_folders["A"], "A", torch.float32)
    toks = ref[1][0]
    stop = toks[5]
    folder = tmp_path / "A_eos"
    shutil.copytree(tiny_folders["A"], folder)
    (folder / "generation_config.json").write_text(json.dumps({"eos_token_id": [stop, 999999]}))
    out = generate(str(folder), [prompts_of("A")[1]], SamplingParams(max_tokens=16), dtype="float32", block_size=4)[0]
    first = toks.index(stop)
    assert out == toks[: first + 1]


def test_lookahead_changes_nothing_but_the_timing(tiny_folders, tmp_path):
    """Decode steps enqueued ahead of their turn take their input ids from the GPU; tokens, stops on end-of-sequence
    (found one step late, the extra step dropped) and the state of the pool must be those of step-by-step running."""
    import shutil

    from nanospec_amd import SamplingParams, load_model

    folder = tmp_path / "B_eos"
    shutil.copytree(tiny_folders["B"], folder)
    ref = plain_greedy(tiny_folders["B"], "B", torch.float32)
    stops = sorted({ref[1][0][7], ref[3][0][11]})
    (folder / "generation_config.json").write_text(json.dumps({"eos_token_id": stops}))
    model = load_model(folder, dtype="float32")
    prompts = prompts_of("B")
    params = [SamplingParams(max_tokens=NEW["B"] - 3 * i, temperature=0.0 if i % 2 else 0.9, seed=i) for i in range(len(prompts))]
    outs = {}
    for ahead in (False, True):
        reqs, _, eng = run_engine(model, prompts, params, num_blocks=96, block_size=8, lookahead=ahead)
        outs[ahead] = [r.out_tokens for r in reqs]
        assert all(len(r.out_tokens) <= p.max_tokens for r, p in zip(reqs, params))
    assert outs[True] == outs[False]
    assert any(o[-1] in stops and len(o) < p.max_tokens for o, p in zip(outs[True], params)), "no request stopped on an end token"


@pytest.mark.parametrize("n_requests,bucket", [(40, 48), (150, 176), (250, 256)])
def test_many_requests_decode_through_one_graph(tiny_folders, n_requests, bucket):
    """More rows than the reference's largest captured batch (64) through the engine: admission of all of them at once,
    decoding in the captured step of that many rows with pad rows, against the plain implementation's greedy tokens
    (a token may differ only where the plain logits of the two are within rounding of each other)."""
    from nanospec_amd import SamplingParams

    name = "B"
    folder = tiny_folders[name]
    model = model_of(folder, name, torch.bfloat16)
    cfg, w = pl.read_config(folder), pl.read_weights(folder, torch.bfloat16)
    vocab = TINY[name]["cfg"]["vocab_size"]
    prompts = [random_tokens(3 + i % 11, vocab, 900 + i) for i in range(n_requests)]
    new = 5
    reqs, _, eng = run_engine(model, prompts, [SamplingParams(max_tokens=new)] * n_requests, num_blocks=900, block_size=8,
                              max_admit=n_requests, max_running=n_requests)
    assert (bucket, 0) in eng.runner._graphs, f"the {n_requests} rows did not replay the graph of {bucket}"
    for i, (p, r) in enumerate(zip(prompts, reqs)):
        assert len(r.out_tokens) == new
        rows = pl.logits_of_sequence(w, cfg, p + r.out_tokens[:-1], torch.bfloat16)[len(p) - 1 :]
        for k, tok in enumerate(r.out_tokens):
            gap = float(rows[k].max() - rows[k][tok])
            assert gap <= 8 * BF16_ULP * float(rows[k].abs().max()), f"request {i} token {k}: not the plain implementation's choice"


def test_engine_on_a_callers_side_stream(tiny_folders):
    """The engine works on its runner's stream whatever stream the caller is on, hands the caller's stream back, and
    its tokens are those of a run from the default stream."""
    from nanospec_amd import SamplingParams

    name = "A"
    model = model_of(tiny_folders[name], name, torch.float32)
    prompts = prompts_of(name)
    params = [SamplingParams(max_tokens=NEW[name])] * len(prompts)
    base, _, _ = run_engine(model, prompts, params, num_blocks=96, block_size=8)
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        busy = torch.randn(1 << 20, device="cuda").cumsum(0)  # work of the caller's own, still under way
        reqs, _, eng = run_engine(model, prompts, params, num_blocks=96, block_size=8)
        assert torch.cuda.current_stream() == side
    assert eng.runner.stream not in (side, torch.cuda.default_stream())
    assert [r.out_tokens for r in reqs] == [r.out_tokens for r in base]
    del busy


def test_refuses_what_it_cannot_run(tiny_folders):
    from nanospec_amd import Engine, EngineConfig, SamplingParams
    from nanospec_amd.cache import PoolExhausted

    model = model_of(tiny_folders["A"], "A", torch.float32)
    eng = Engine(model, EngineConfig(num_blocks=8, block_size=4))
    with pytest.raises(ValueError):
        eng.add([1, 2, 256])  # a token id outside the vocabulary
    with pytest.raises(PoolExhausted):
        eng.add(list(range(30)), SamplingParams(max_tokens=10))  # never fits 7 usable pages
    with pytest.raises(ValueError):
        eng2 = Engine(model, EngineConfig(num_blocks=64, block_size=4))
        eng2.generate([list(range(120))], SamplingParams(max_tokens=20))  # runs past the model's 128 positions
