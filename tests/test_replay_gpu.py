"""The engine's step function against the plain implementation, in 32-bit and in bfloat16, for the same requests
cut into steps in four ways.  The logits at a position must not depend on the cut, the batch or the pages."""

from __future__ import annotations

import json
import os
import subprocess
import sys
from pathlib import Path

import pytest
import torch

import plain_llama as pl
import traces
from tiny import TINY, random_tokens, ulps_of_row_max

pytestmark = pytest.mark.gpu
ROOT = Path(__file__).resolve().parent.parent

LENGTHS = {"A": (5, 17, 33, 64, 97, 128), "B": (1, 9, 40, 100, 130, 255)}


def sequences(name):
    vocab = TINY[name]["cfg"]["vocab_size"]
    return {f"r{i}": random_tokens(n, vocab, 100 * i + n) for i, n in enumerate(LENGTHS[name])}


_PLAIN = {}


def plain_logits(folder, name, dtype):
    key = (name, dtype)
    if key not in _PLAIN:
        cfg, w = pl.read_config(folder), pl.read_weights(folder, dtype)
        _PLAIN[key] = {rid: pl.logits_of_sequence(w, cfg, toks, dtype) for rid, toks in sequences(name).items()}
    return _PLAIN[key]


_MODELS = {}


def engine_model(folder, name, dtype):
    from nanospec_amd.loader import load_model

    key = (name, dtype)
    if key not in _MODELS:
        _MODELS[key] = load_model(folder, dtype=dtype)
    return _MODELS[key]


def check(ours: torch.Tensor, ref: torch.Tensor, dtype, what: str):
    assert ours.shape == ref.shape, (what, ours.shape, ref.shape)
    assert torch.isfinite(ours).all(), what
    if dtype == torch.float32:
        err = ((ours - ref).abs().amax(-1) / ref.abs().amax(-1)).max().item()
        assert err <= 1e-4, f"{what}: {err:.2e} of the row's largest logit"
    else:
        u = ulps_of_row_max(ours, ref)
        assert u.max() <= 8, f"{what}: {u.max():.2f} bf16 ulps of the row's largest logit (median {u.median():.2f})"


def churn(manager, rounds=200, seed=0):
    """Random reservations and releases before a run (reference: tests/test_correctness.py:25-50), so that the free list
    is in no order and every request's pages lie scattered over the pool."""
    import random

    rng = random.Random(seed)
    held = []
    for i in range(rounds):
        if held and (rng.random() < 0.5 or manager.slots.num_free == 0 or manager.num_free(0) < 8):
            manager.release(held.pop(rng.randrange(len(held))))
        else:
            rid = f"churn{i}"
            manager.admit(rid)
            n = rng.randint(1, 7 * manager.page_size)
            manager.reserve(rid, n)
            manager.commit(rid, n)
            held.append(rid)
    rng.shuffle(held)
    for rid in held:
        manager.release(rid)
    manager.check()


def replay(model, steps, where, ref, dtype, max_tokens, page, graphs=True, link_norms=True, churned=False):
    from nanospec_amd.engine.replay import Replayer

    rep = Replayer(model, max_tokens, page_size=page, use_graphs=graphs)
    rep.runner.link_norms = link_norms
    if churned:
        churn(rep.manager)
        rep.scattered = 0
    holders: dict = {}  # (group, page) -> the requests that have held it
    real_reserve = rep.manager.reserve

    def reserve(req_id, n):
        real_reserve(req_id, n)
        for g, table in enumerate(rep.manager.get(req_id).tables):
            for page in table:
                if page is not None and page >= 0:
                    holders.setdefault((g, page), set()).add(req_id)

    rep.manager.reserve = reserve
    for step, w in zip(steps, where):
        out = rep.step(step["entries"], step["end"])
        if rep.runner.last_used_graph and any(len(e["tokens"]) > 1 for e in step["entries"]):
            rep.mixed_graph_steps = getattr(rep, "mixed_graph_steps", 0) + 1
        if churned:
            for e in step["entries"]:
                if e["id"] in rep.manager:
                    table = rep.manager.get(e["id"]).tables[0]
                    rep.scattered += sum(1 for a, b in zip(table, table[1:]) if a is not None and b is not None and abs(b - a) != 1)
        if not w:
            assert out is None
            continue
        want = torch.stack([ref[rid][p] for rid, p in w])
        check(out, want, dtype, f"step {step['step']} {[(e['id'], len(e['tokens'])) for e in step['entries']]}")
    rep.manager.check()
    live = [r for r in rep.manager.live if r != "__pad__"]
    assert not live
    rep.regranted = sum(1 for who in holders.values() if len(who) > 1)  # pages that two requests held in turn
    return rep


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("name", ["A", "B"])
@pytest.mark.parametrize("schedule", ["whole", "tail", "portions", "mixed", "mixed11", "mixed23"])
def test_schedules_match_plain(tiny_folders, name, dtype, schedule):
    folder, page = tiny_folders[name], TINY[name]["page"]
    seqs = sequences(name)
    ref = plain_logits(folder, name, dtype)
    model = engine_model(folder, name, dtype)
    if schedule == "whole":
        steps, where = traces.whole(seqs)
        max_tokens = 256
    elif schedule == "tail":
        steps, where = traces.tail_decoded(seqs)
        max_tokens = 256
    elif schedule == "portions":
        steps, where = traces.portions(seqs, seed=3)
        max_tokens = 256
    else:
        # seed 11 holds a decode-only step (a replayed graph, whose pad rows live in a state slot that a finished
        # request held before) between two portions of a request that sits that step out
        steps, where, peak = traces.mixed(seqs, seed=int(schedule[5:] or 5))
        max_tokens = peak  # so few pages that finished requests' pages are handed out again
    rep = replay(model, steps, where, ref, dtype, max_tokens, page)
    if schedule.startswith("mixed"):
        assert rep.regranted > 0, "no page was handed to a second request: the trace does not test the reuse of pages"


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("name", ["A", "B"])
def test_mixed_schedule_on_a_churned_pool(tiny_folders, name, dtype):
    """reference tests/test_correctness.py:25-50: two hundred random reservations and releases come first, so the pages a
    request gets are neither consecutive nor in rising order; the mixed schedule on so few pages that they are used again."""
    folder, page = tiny_folders[name], TINY[name]["page"]
    seqs = sequences(name)
    steps, where, peak = traces.mixed(seqs, seed=23)
    rep = replay(engine_model(folder, name, dtype), steps, where, plain_logits(folder, name, dtype), dtype, peak, page, churned=True)
    assert rep.scattered > 20, "the block tables were meant to be scattered"


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("name", ["A", "B"])
def test_long_decoding_from_the_first_token(tiny_folders, name, dtype):
    """Two requests decoded one token at a time from position 0 to the model's last position: the first tokens of a
    sequence (one key, then two, ...), every page edge on the way, and errors that would build up over many steps."""
    folder, page = tiny_folders[name], TINY[name]["page"]
    seqs = {k: v for k, v in list(sequences(name).items())[-2:]}
    ref = plain_logits(folder, name, dtype)
    model = engine_model(folder, name, dtype)
    longest = max(len(t) for t in seqs.values())
    steps, where = [], []
    for p in range(longest):
        live = [r for r, t in seqs.items() if p < len(t)]
        steps.append({"step": p, "entries": [{"id": r, "tokens": [seqs[r][p]], "want": [0]} for r in live],
                      "end": [r for r in live if p == len(seqs[r]) - 1]})
        where.append([(r, p) for r in live])
    replay(model, steps, where, ref, dtype, 512, page)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("name", ["A", "B"])
def test_mixed_steps_replay_captured_steps_of_fixed_shapes(tiny_folders, name, dtype):
    """Steps of a few prompt portions beside decode rows replay captured steps whose shapes are padded (pad rows, pad
    tokens, tiles without tokens, wanted places nobody reads); the same trace without graphs gives the same logits, and
    both are the plain implementation's.  Few logits are wanted per step here, as in generation: a captured step has room
    for one per row and one per portion."""
    folder, page = tiny_folders[name], TINY[name]["page"]
    seqs = sequences(name)
    ref = plain_logits(folder, name, dtype)
    model = engine_model(folder, name, dtype)
    steps, where, peak = traces.mixed(seqs, seed=11)
    thin_steps, thin_where = [], []
    for step, w in zip(steps, where):  # keep the last wanted place of every entry only
        entries, at, kept = [], 0, []
        for e in step["entries"]:
            n = len(e["want"])
            entries.append(dict(e, want=e["want"][-1:]))
            kept += w[at + n - 1 : at + n]
            at += n
        thin_steps.append(dict(step, entries=entries))
        thin_where.append(kept)
    rep = replay(model, thin_steps, thin_where, ref, dtype, peak, page, graphs=True)
    assert getattr(rep, "mixed_graph_steps", 0) >= 10, "the mixed steps were meant to replay captured steps"
    assert any(chunk for _, chunk in rep.runner._graphs)
    replay(model, thin_steps, thin_where, ref, dtype, peak, page, graphs=False)


def test_captured_steps_are_dropped_and_captured_again(tiny_folders, monkeypatch):
    """Room for three captured steps only, and block tables that start two pages wide: steps are captured, dropped (the one
    unused for longest first) and captured again, and captured again wider whenever a request outgrows them; the logits
    stay the plain implementation's throughout."""
    from nanospec_amd.engine import runner as runner_mod

    name = "A"
    folder, page = tiny_folders[name], TINY[name]["page"]
    seqs = sequences(name)
    ref = plain_logits(folder, name, torch.bfloat16)
    model = engine_model(folder, name, torch.bfloat16)
    monkeypatch.setattr(runner_mod, "MAX_GRAPHS", 3)
    monkeypatch.setattr(runner_mod.ModelRunner, "GRAPH_MIN_WIDTH", 2)
    captures = []
    real = runner_mod.ModelRunner._capture

    def counted(self, shape, width):
        captures.append((shape, width))
        return real(self, shape, width)

    monkeypatch.setattr(runner_mod.ModelRunner, "_capture", counted)
    steps, where, peak = traces.mixed(seqs, seed=11)
    thin = [dict(st, entries=[dict(e, want=e["want"][-1:]) for e in st["entries"]]) for st in steps]
    thin_where = []
    for st, w in zip(steps, where):
        at, kept = 0, []
        for e in st["entries"]:
            kept += w[at + len(e["want"]) - 1 : at + len(e["want"])]
            at += len(e["want"])
        thin_where.append(kept)
    rep = replay(model, thin, thin_where, ref, torch.bfloat16, peak, page, graphs=True)
    assert len(rep.runner._graphs) <= 3
    shapes = [s for s, _ in captures]
    assert len(set(shapes)) > 3 and len(shapes) > len(set(shapes)), "shapes were meant to be dropped and captured again"
    widths = [w for _, w in captures]
    assert max(widths) >= 4 * min(widths) and min(widths) < 16, "block tables were meant to start narrow and grow"
    # the captured steps share their intermediates' memory: all of them together hold less than twice what the largest needs
    arenas = {id(g.arena): g.arena for g in rep.runner._graphs.values()}
    assert len(arenas) < len(rep.runner._graphs)
    assert rep.runner.graph_arena_bytes < 2 * max(a.capacity for a in arenas.values()) + 1


@pytest.mark.parametrize("name", ["A", "B"])
def test_graph_and_eager_decode_agree(tiny_folders, name):
    folder, page = tiny_folders[name], TINY[name]["page"]
    seqs = sequences(name)
    ref = plain_logits(folder, name, torch.bfloat16)
    model = engine_model(folder, name, torch.bfloat16)
    steps, where = traces.tail_decoded(seqs)
    a = replay(model, steps, where, ref, torch.bfloat16, 256, page, graphs=True)
    assert a.runner._graphs, "decode steps did not replay a graph"
    replay(model, steps, where, ref, torch.bfloat16, 256, page, graphs=False)


# requests that decode together -> the captured step they must replay: every bucket of the runner
BUCKET_CASES = [(1, 1), (2, 2), (3, 4), (7, 8), (12, 16), (20, 32), (40, 48), (60, 64), (70, 96), (100, 128), (150, 176), (200, 208),
                (230, 240), (250, 256)]


def test_bucket_cases_cover_every_bucket():
    from nanospec_amd.engine.runner import GRAPH_BUCKETS

    assert [b for _, b in BUCKET_CASES] == list(GRAPH_BUCKETS)


@pytest.mark.parametrize("n_requests,bucket", BUCKET_CASES)
def test_every_graph_bucket_against_plain(tiny_folders, n_requests, bucket):
    """reference tests/test_graphs.py:43-72, for every bucket: so many requests decode together that the step replays the
    captured graph of that many rows (pad rows included), and every row's logits are the plain implementation's.  Above
    128 rows the step runs other code (the library's products, the sum in the product, norms of their own)."""
    from nanospec_amd.engine.replay import Replayer

    name = "B"
    folder, page = tiny_folders[name], TINY[name]["page"]
    vocab = TINY[name]["cfg"]["vocab_size"]
    cfg, w = pl.read_config(folder), pl.read_weights(folder, torch.bfloat16)
    model = engine_model(folder, name, torch.bfloat16)
    decoded = 3
    seqs = {f"q{i}": random_tokens(2 + (5 * i) % 17 + decoded, vocab, 4000 + i) for i in range(n_requests)}
    ref = {r: pl.logits_of_sequence(w, cfg, t, torch.bfloat16) for r, t in seqs.items()}
    rep = Replayer(model, sum(-(-len(t) // page) * page for t in seqs.values()) + page, page_size=page, max_live=n_requests)
    ids = list(seqs)
    for at in range(0, n_requests, 24):  # the prompts, two dozen requests to a step, nothing wanted
        rep.step([{"id": r, "tokens": seqs[r][:-decoded], "want": []} for r in ids[at : at + 24]], [])
    for d in range(decoded, 0, -1):
        entries = [{"id": r, "tokens": [seqs[r][-d]], "want": [0]} for r in ids]
        out = rep.step(entries, ids if d == 1 else [])
        assert rep.runner.last_used_graph and (bucket, 0) in rep.runner._graphs
        want = torch.stack([ref[r][len(seqs[r]) - d] for r in ids])
        check(out, want, torch.bfloat16, f"{n_requests} requests, {d} tokens before their end")
    rep.manager.check()


def test_graph_step_in_which_only_some_rows_want_logits(tiny_folders):
    """A decode-only step replays the captured graph, which computes every row's logits; what comes back is the rows that
    were asked for, in the order of the entries."""
    from nanospec_amd.engine.replay import Replayer

    name = "A"
    folder, page = tiny_folders[name], TINY[name]["page"]
    seqs = sequences(name)
    ids = list(seqs)[1:5]
    for dtype in (torch.float32, torch.bfloat16):
        ref = plain_logits(folder, name, dtype)
        rep = Replayer(engine_model(folder, name, dtype), 512, page_size=page)
        rep.step([{"id": r, "tokens": seqs[r][:9], "want": []} for r in ids], [])
        for p, wanting in ((9, [0, 2]), (10, [1, 2, 3]), (11, [3]), (12, [0, 1, 2, 3])):
            out = rep.step([{"id": r, "tokens": [seqs[r][p]], "want": [0] if i in wanting else []} for i, r in enumerate(ids)], [])
            assert rep.runner.last_used_graph
            check(out, torch.stack([ref[ids[i]][p] for i in wanting]), dtype, f"position {p}, rows {wanting}")


@pytest.mark.parametrize("name", ["A", "B"])
@pytest.mark.parametrize("schedule", ["tail", "mixed"])
def test_norms_as_kernels_of_their_own(tiny_folders, name, schedule):
    """Steps of at most 16 tokens let the products around a norm do its work; here every norm runs as its own kernel,
    and the steps in which the two ways differ are counted."""
    from nanospec_amd.kernels import ops

    folder, page = tiny_folders[name], TINY[name]["page"]
    seqs = sequences(name)
    ref = plain_logits(folder, name, torch.bfloat16)
    model = engine_model(folder, name, torch.bfloat16)
    if schedule == "tail":
        steps, where = traces.tail_decoded(seqs)
        max_tokens = 256
    else:
        steps, where, max_tokens = traces.mixed(seqs, seed=5)
    calls = {"linked": 0}
    real = ops.linear_resid_norm

    def counted(*a, **k):
        calls["linked"] += 1
        return real(*a, **k)

    ops.linear_resid_norm = counted
    try:
        replay(model, steps, where, ref, torch.bfloat16, max_tokens, page, graphs=False, link_norms=False)
        assert calls["linked"] == 0
        replay(model, steps, where, ref, torch.bfloat16, max_tokens, page, graphs=False, link_norms=True)
        assert calls["linked"] > 0, "no step took the linked path"
    finally:
        ops.linear_resid_norm = real


@pytest.mark.parametrize("name", ["A", "B"])
@pytest.mark.parametrize("schedule", ["portions", "mixed"])
def test_prompt_portions_with_their_keys_cut_into_ranges(tiny_folders, name, schedule, monkeypatch):
    """A short portion late in a long prompt has its keys cut into ranges that workgroups of their own walk.  The tiny
    models' prompts are too short for that by the engine's own rule, so the rule's threshold is lowered to one block."""
    from nanospec_amd.kernels import ops
    from nanospec_amd.parts import attention

    monkeypatch.setattr(attention, "PORTION_RANGE_BLOCKS", 1)
    folder, page = tiny_folders[name], TINY[name]["page"]
    seqs = sequences(name)
    ref = plain_logits(folder, name, torch.bfloat16)
    model = engine_model(folder, name, torch.bfloat16)
    if schedule == "portions":
        steps, where = traces.portions(seqs, seed=3)
        max_tokens = 256
    else:
        steps, where, max_tokens = traces.mixed(seqs, seed=23)
    cut = []
    real = ops.attention_mfma

    def counted(*a, **k):
        if k.get("qt") == 2 and k.get("splits", 1) > 1:
            cut.append(k["splits"])
        return real(*a, **k)

    monkeypatch.setattr(ops, "attention_mfma", counted)
    replay(model, steps, where, ref, torch.bfloat16, max_tokens, page, graphs=False)
    assert cut and max(cut) >= 3, "no portion had its keys cut into ranges"


@pytest.mark.parametrize("name", ["A", "B"])
def test_one_weight_layout_only(tiny_folders, name):
    """Without the plain layout (models that fill the memory) steps of many tokens run in slices through the streaming
    kernels: same logits."""
    from nanospec_amd.loader import load_model

    folder, page = tiny_folders[name], TINY[name]["page"]
    seqs = sequences(name)
    ref = plain_logits(folder, name, torch.bfloat16)
    model = load_model(folder, dtype=torch.bfloat16, layouts="tiled")
    assert model.layers[0].ffn.down.plain is None and model.layers[0].ffn.gate_up.stacked is None
    both = load_model(folder, dtype=torch.bfloat16, layouts="both")  # a second model in the process keeps its own choice
    assert both.layers[0].ffn.down.plain is not None and model.layers[0].mixer.wo.plain is None
    for make in (traces.whole, traces.tail_decoded):
        steps, where = make(seqs)
        replay(model, steps, where, ref, torch.bfloat16, 256, page)


def test_trace_run_program(tiny_folders, tmp_path):
    """bin/trace_run as a user calls it: JSON lines in, <step>.f32 out, 'done <step>' after every step."""
    name = "B"
    folder = tiny_folders[name]
    seqs = sequences(name)
    steps, where, peak = traces.mixed(seqs, seed=11)
    for dtype_name, dtype in (("float32", torch.float32), ("bfloat16", torch.bfloat16)):
        ref = plain_logits(folder, name, dtype)
        out_dir = tmp_path / dtype_name
        proc = subprocess.run([sys.executable, str(ROOT / "bin" / "trace_run"), "--model", str(folder), "--dtype", dtype_name,
                               "--out", str(out_dir), "--max-tokens", str(peak)],
                              input="\n".join(json.dumps(s) for s in steps) + "\n", capture_output=True, text=True, timeout=600)
        assert proc.returncode == 0, proc.stderr[-2000:]
        assert [l for l in proc.stdout.split("\n") if l.startswith("done")] == [f"done {s['step']}" for s in steps]
        vocab = TINY[name]["cfg"]["vocab_size"]
        for step, w in zip(steps, where):
            path = out_dir / f"{step['step']}.f32"
            if not w:
                assert not path.exists()
                continue
            got = torch.from_file(str(path), size=len(w) * vocab, dtype=torch.float32).view(len(w), vocab)
            check(got, torch.stack([ref[rid][p] for rid, p in w]), dtype, f"trace_run step {step['step']}")


# ------------------------------------------------------------------------------------------------ a real shape


@pytest.fixture(scope="module")
def llama_1b_slice(tmp_path_factory):
    """Two layers of the Llama-3.2-1B shape (width 2048, 32 heads over 8 key/value heads of 64, feed-forward 8192,
    vocabulary 128256, tied head, llama3 scaling with factor 32), random weights."""
    from nanospec_amd.config import LlamaConfig
    from nanospec_amd.weights import write_model_folder

    cfg = dict(architectures=["LlamaForCausalLM"], model_type="llama", vocab_size=128256, hidden_size=2048, intermediate_size=8192,
               num_hidden_layers=2, num_attention_heads=32, num_key_value_heads=8, head_dim=64, rms_norm_eps=1e-5, rope_theta=500000.0,
               max_position_embeddings=131072, tie_word_embeddings=True,
               rope_scaling=dict(rope_type="llama3", factor=32.0, low_freq_factor=1.0, high_freq_factor=4.0,
                                 original_max_position_embeddings=8192))
    return write_model_folder(tmp_path_factory.mktemp("llama1b") / "m", LlamaConfig.from_hf(cfg), seed=3, dtype=torch.bfloat16)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
def test_real_shape_slice_matches_plain(llama_1b_slice, dtype, request):
    """The kernels at the sizes of a real model (head size 64, a vocabulary of 128256, width 2048): one request whole with
    its last tokens decoded, one in portions, mixed in one batch, at positions where the llama3 scaling matters."""
    from nanospec_amd.engine.replay import Replayer
    from nanospec_amd.loader import load_model

    folder = llama_1b_slice
    cfg, w = pl.read_config(folder), pl.read_weights(folder, dtype)
    seqs = {"a": random_tokens(150, 128256, 1), "b": random_tokens(83, 128256, 2)}
    ref = {r: pl.logits_of_sequence(w, cfg, t, dtype) for r, t in seqs.items()}
    model = load_model(folder, dtype=dtype)
    rep = Replayer(model, 384, page_size=16)
    from nanospec_amd.kernels import ops

    seen = {"unadded": 0, "linked": 0}
    real_wide, real_link = ops.linear_wide, ops.linear_resid_norm

    def wide(*a, **k):
        out = real_wide(*a, **k)
        seen["unadded"] += isinstance(out, ops.PartialSums)
        return out

    def linked(*a, **k):
        seen["linked"] += 1
        return real_link(*a, **k)

    ops.linear_wide, ops.linear_resid_norm = wide, linked
    request.addfinalizer(lambda: (setattr(ops, "linear_wide", real_wide), setattr(ops, "linear_resid_norm", real_link)))

    def step(entries, end=()):
        out = rep.step([{"id": r, "tokens": seqs[r][s:e], "want": list(wants)} for r, s, e, wants in entries], list(end))
        want = torch.cat([ref[r][s:e][list(wants)] for r, s, e, wants in entries])
        check(out, want, dtype, str([(r, s, e) for r, s, e, _ in entries]))

    step([("a", 0, 130, [0, 64, 129])])
    step([("a", 130, 131, [0]), ("b", 0, 37, [36])])
    step([("a", 131, 132, [0]), ("b", 37, 39, [0, 1])])
    for p in range(132, 150):
        q = 39 + (p - 132) * 2
        step([("a", p, p + 1, [0]), ("b", q, q + 2, [0, 1])], end=["a"] if p == 149 else [])
    step([("b", 75, 83, list(range(8)))], end=["b"])
    rep.manager.check()
    if dtype == torch.bfloat16:
        # the step of 38 tokens handed unadded ranges to the norms, the steps of up to 16 tokens linked norms and products
        assert seen["unadded"] > 0 and seen["linked"] > 0, seen
    else:
        assert seen == {"unadded": 0, "linked": 0}


def plain_logits_at(folder, dtype, toks, places) -> dict:
    """The plain implementation's logits of one sequence at a few places (the head is applied there only)."""
    cfg, w = pl.read_config(folder), pl.read_weights(folder, dtype)
    w = {k: (v if v.dim() == 1 else v.float()) for k, v in w.items()}  # the stored values, converted once
    x = w["model.embed_tokens.weight"][torch.tensor(toks)].to(dtype)
    cos, sin = pl.rotation_tables(torch.arange(len(toks)), pl.inverse_frequencies(cfg["head_dim"], cfg["theta"], cfg["scaling"]))
    for i in range(cfg["layers"]):
        x = pl.decoder_layer(x, w, f"model.layers.{i}.", cfg, cos, sin)
    head = w["lm_head.weight"] if "lm_head.weight" in w else w["model.embed_tokens.weight"]
    ref = pl.rms_norm(x[places], w["model.norm.weight"], cfg["eps"]).float() @ head.T
    return {p: ref[i] for i, p in enumerate(places)}


@pytest.mark.parametrize("slice_k", [8192, 2048])
def test_many_rows_with_one_weight_layout(llama_1b_slice, monkeypatch, slice_k):
    """A model that keeps the re-laid matrices only.  A prompt portion of 1,100 tokens, launched kernel by kernel: every
    matrix is written out in plain rows for the library's product (o's and down's add into the residual stream; with
    slices of 2,048 the down-projection's inner size of 8,192 goes in four slices summed in 32-bit).  A portion of 800
    tokens, a captured step: no plain copies, every product in blocks through the many-row kernel.  Then 100 tokens and
    single ones."""
    from nanospec_amd.engine.replay import Replayer
    from nanospec_amd.kernels import ops
    from nanospec_amd.loader import load_model
    from nanospec_amd.parts import linear

    monkeypatch.setattr(linear, "PLAIN_SLICE_K", slice_k)

    folder, dtype = llama_1b_slice, torch.bfloat16
    toks = random_tokens(2010, 128256, 5)
    places = [0, 1, 511, 767, 1099, 1100, 1500, 1899, 1900, 1999, 2000, 2003, 2009]
    at = plain_logits_at(folder, dtype, toks, places)
    model = load_model(folder, dtype=dtype, layouts="tiled")
    calls = {"untile": 0, "rows": 0}
    real_untile, real_rows = ops.untile, ops.linear_rows
    monkeypatch.setattr(ops, "untile", lambda *a, **k: (calls.__setitem__("untile", calls["untile"] + 1), real_untile(*a, **k))[1])
    monkeypatch.setattr(ops, "linear_rows", lambda *a, **k: (calls.__setitem__("rows", calls["rows"] + 1), real_rows(*a, **k))[1])
    rep = Replayer(model, 2048, page_size=16)

    def step(s, e):
        wants = [p - s for p in places if s <= p < e]
        out = rep.step([{"id": "a", "tokens": toks[s:e], "want": wants}], [])
        if wants:
            check(out, torch.stack([at[s + i] for i in wants]), dtype, f"tokens {s}:{e}")

    step(0, 1100)
    assert not rep.runner.last_used_graph
    # per layer: q/k/v, o, gate, up, and down whole or in four slices; the last layer's down-projection, which no norm of
    # the layer loop follows, is not summed in 32-bit slices: with the short slices it stays with the many-row kernel
    copies, blocks = (2 * 5, 0) if slice_k == 8192 else (8 + 4, 1)
    assert calls == {"untile": copies, "rows": blocks}, calls
    step(1100, 1900)
    assert rep.runner.last_used_graph
    # (the step ran twice: once before its capture and once while captured; a replay's kernels do not pass through here)
    assert calls["untile"] == copies and calls["rows"] == blocks + 2 * 2 * 4, calls  # q/k/v, o, gate/up, down: all in blocks
    step(1900, 2000)
    for p in range(2000, 2010):
        step(p, p + 1)
    rep.manager.check()


def test_long_inner_sizes_never_reach_the_library_in_one_piece(llama_1b_slice, monkeypatch):
    """Both layouts kept, and the longest inner size that the library takes in one piece set below the down-projection's
    (8,192 here).  A portion of 1,100 tokens launched kernel by kernel: the down-projection goes to the library in slices
    summed in 32-bit; the last layer's, which does not end in the stream, through the many-row kernel.  A captured step of
    800 tokens: the many-row kernel both times.  Every other product stays with the library, and none of the library's
    products runs over more than the bound."""
    from nanospec_amd.engine.replay import Replayer
    from nanospec_amd.kernels import ops
    from nanospec_amd.loader import load_model
    from nanospec_amd.parts import linear

    monkeypatch.setattr(linear, "LIBRARY_MAX_K", 4096)
    monkeypatch.setattr(linear, "PLAIN_SLICE_K", 4096)
    folder, dtype = llama_1b_slice, torch.bfloat16
    toks = random_tokens(2010, 128256, 6)
    places = [0, 700, 1099, 1100, 1899, 1900, 2000, 2009]
    at = plain_logits_at(folder, dtype, toks, places)
    model = load_model(folder, dtype=dtype, layouts="both")
    seen = {"library": [], "rows": []}
    real_lib, real_rows = linear.library_product, ops.linear_rows
    monkeypatch.setattr(linear, "library_product", lambda x, w_t, **k: (seen["library"].append((x.shape[1], k.get("into") is not None and k["into"].dtype == torch.float32)), real_lib(x, w_t, **k))[1])
    monkeypatch.setattr(ops, "linear_rows", lambda x, w, **k: (seen["rows"].append(w.k), real_rows(x, w, **k))[1])
    rep = Replayer(model, 2048, page_size=16)

    def step(s, e):
        wants = [p - s for p in places if s <= p < e]
        out = rep.step([{"id": "a", "tokens": toks[s:e], "want": wants}], [])
        if wants:
            check(out, torch.stack([at[s + i] for i in wants]), dtype, f"tokens {s}:{e}")

    step(0, 1100)
    assert not rep.runner.last_used_graph
    # q/k/v, o and gate/up of both layers in one piece; the first layer's down-projection in two slices into a 32-bit sum
    assert sorted(seen["library"]) == [(2048, False)] * 6 + [(4096, True)] * 2, seen
    assert seen["rows"] == [8192], seen
    seen["library"].clear(), seen["rows"].clear()
    step(1100, 1900)
    assert rep.runner.last_used_graph
    # (the step ran twice: once before its capture and once while captured)
    assert sorted(seen["library"]) == [(2048, False)] * 12 and seen["rows"] == [8192] * 4, seen
    step(1900, 2000)
    for p in range(2000, 2010):
        step(p, p + 1)
    assert max(k for k, _ in seen["library"]) <= 4096
    rep.manager.check()
    with pytest.raises(ops.KernelRefused):
        x = torch.zeros((256, 8192), dtype=dtype, device="cuda")
        real_lib(x, torch.zeros((8192, 64), dtype=dtype, device="cuda"))


@pytest.fixture(scope="module")
def llama_8b_slice(tmp_path_factory):
    """Two layers of the Llama-3.1-8B shape (width 4096, 32 heads over 8 key/value heads of 128, feed-forward 14336,
    vocabulary 128256, a head of its own, llama3 scaling with factor 8), random weights: the sizes that the benchmark runs."""
    from nanospec_amd.config import LlamaConfig
    from nanospec_amd.weights import write_model_folder

    cfg = dict(architectures=["LlamaForCausalLM"], model_type="llama", vocab_size=128256, hidden_size=4096, intermediate_size=14336,
               num_hidden_layers=2, num_attention_heads=32, num_key_value_heads=8, head_dim=128, rms_norm_eps=1e-5, rope_theta=500000.0,
               max_position_embeddings=131072, tie_word_embeddings=False,
               rope_scaling=dict(rope_type="llama3", factor=8.0, low_freq_factor=1.0, high_freq_factor=4.0,
                                 original_max_position_embeddings=8192))
    return write_model_folder(tmp_path_factory.mktemp("llama8b") / "m", LlamaConfig.from_hf(cfg), seed=4, dtype=torch.bfloat16)


def test_a_captured_step_of_512_rows_replayed_over_and_over(llama_8b_slice):
    """The benchmark's layer sizes in the step that serving repeats most often: 32 decode rows beside a prompt portion of 480
    tokens, 512 rows through the library's products inside a captured graph.  The same captured step is replayed six
    times with new tokens, longer contexts and other work on the GPU in between, and every replay is compared with the
    same step launched kernel by kernel in a second cache (a captured library call that keeps state between replays,
    or a node that is not replayed, would show from the second replay on)."""
    from nanospec_amd.engine.replay import Replayer
    from nanospec_amd.loader import load_model

    model = load_model(llama_8b_slice, dtype=torch.bfloat16)
    vocab = pl.read_config(llama_8b_slice)["vocab"]
    graphs = Replayer(model, 8192, page_size=16, use_graphs=True, max_live=40)
    eager = Replayer(model, 8192, page_size=16, use_graphs=False, max_live=40)
    rows = {f"d{i}": random_tokens(8 + 7, vocab, 900 + i) for i in range(32)}
    prompt = random_tokens(6 * 480, vocab, 77)

    def both(entries):
        a, b = graphs.step(entries, []), eager.step(entries, [])
        torch.cuda.synchronize()
        return a, b

    both([{"id": r, "tokens": t[:8], "want": []} for r, t in rows.items()])
    for k in range(6):
        entries = [{"id": r, "tokens": t[8 + k : 9 + k], "want": [0]} for r, t in rows.items()]
        entries.append({"id": "p", "tokens": prompt[480 * k : 480 * (k + 1)], "want": [0, 479]})
        a, b = both(entries)
        assert graphs.runner.last_used_graph and not eager.runner.last_used_graph
        check(a, b, torch.bfloat16, f"replay {k}")
        # other work on the GPU between the replays, of the program's own kind: a decode-only step of the same requests'
        # cache would change it, so a product of the library on unrelated data
        junk = torch.randn(300, 4096, dtype=torch.bfloat16, device="cuda")
        (junk @ junk.t()).sum().item()
    assert (32, 480) in graphs.runner._graphs  # one captured step served all six


def test_a_captured_decode_step_of_208_rows_replayed_over_and_over(llama_8b_slice):
    """The benchmark's layer sizes with 200 live requests: decode steps of more than 128 rows run their products through the
    library inside a captured graph (few rows, inner sizes of 4,096 and 14,336: shapes for which a library may cut the
    inner size and keep partial results in a workspace of its own).  Five replays with new tokens, each compared with the
    same step launched kernel by kernel in a second cache."""
    from nanospec_amd.engine.replay import Replayer
    from nanospec_amd.loader import load_model

    model = load_model(llama_8b_slice, dtype=torch.bfloat16)
    vocab = pl.read_config(llama_8b_slice)["vocab"]
    graphs = Replayer(model, 200 * 64, page_size=16, use_graphs=True, max_live=200)
    eager = Replayer(model, 200 * 64, page_size=16, use_graphs=False, max_live=200)
    rows = {f"d{i}": random_tokens(3 + i % 5 + 5, vocab, 300 + i) for i in range(200)}
    for at in range(0, 200, 50):  # prompts, fifty requests a step
        entries = [{"id": r, "tokens": t[:-5], "want": []} for r, t in list(rows.items())[at : at + 50]]
        graphs.step(entries, []), eager.step(entries, [])
    for k in range(5):
        entries = [{"id": r, "tokens": [t[len(t) - 5 + k]], "want": [0]} for r, t in rows.items()]
        a, b = graphs.step(entries, []), eager.step(entries, [])
        torch.cuda.synchronize()
        assert graphs.runner.last_used_graph and not eager.runner.last_used_graph
        check(a, b, torch.bfloat16, f"replay {k}")
        junk = torch.randn(300, 4096, dtype=torch.bfloat16, device="cuda")
        (junk @ junk.t()).sum().item()
    assert (208, 0) in graphs.runner._graphs


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
def test_benchmark_shape_slice_matches_plain(llama_8b_slice, dtype):
    """The layer sizes of the benchmark end to end: a portion of 280 tokens, a mixed step, decoding with 8 live requests
    (captured step; norms folded into the products), prompts of 56 more requests, decoding with 64 live requests (the
    17-to-64-row kernels, unadded ranges into the norms, the library's q/k/v product), and a step of 63 decode rows beside
    a new prompt."""
    from nanospec_amd.engine.replay import Replayer
    from nanospec_amd.loader import load_model

    folder = llama_8b_slice
    cfg = pl.read_config(folder)
    w = pl.read_weights(folder, dtype)
    # matrices as 32-bit tensors that hold the stored (bfloat16-rounded) values: the plain functions convert a matrix at
    # every use, which at these sizes would take most of the test's time; vectors (norm weights) keep the dtype, which
    # decides how the norm rounds
    w = {k: (v if v.dim() == 1 else v.float()) for k, v in w.items()}
    vocab = cfg["vocab"]
    lengths = {"r0": 305, **{f"r{i}": 6 + i % 7 + 5 for i in range(1, 8)}, **{f"r{i}": 4 + i % 9 + 3 for i in range(8, 64)}, "r64": 40}
    seqs = {r: random_tokens(n, vocab, 7000 + i) for i, (r, n) in enumerate(lengths.items())}
    inv = pl.inverse_frequencies(cfg["head_dim"], cfg["theta"], cfg["scaling"])
    hidden = {}
    for r, toks in seqs.items():  # the stream after the last layer, every position
        x = w["model.embed_tokens.weight"][torch.tensor(toks)].to(dtype)
        cos, sin = pl.rotation_tables(torch.arange(len(toks)), inv)
        for i in range(cfg["layers"]):
            x = pl.decoder_layer(x, w, f"model.layers.{i}.", cfg, cos, sin)
        hidden[r] = x

    def plain_rows(places):
        x = torch.stack([hidden[r][p] for r, p in places])
        return pl.rms_norm(x, w["model.norm.weight"], cfg["eps"]).float() @ w["lm_head.weight"].T

    model = load_model(folder, dtype=dtype)
    rep = Replayer(model, 305 + 64 * 64 + 64, page_size=16, max_live=65)
    at = {r: 0 for r in seqs}

    def step(parts, graph=None):
        """parts: (request, tokens it brings, places among them whose logits are compared)"""
        entries, places = [], []
        for r, n, wants in parts:
            entries.append({"id": r, "tokens": seqs[r][at[r] : at[r] + n], "want": list(wants)})
            places += [(r, at[r] + i) for i in wants]
            at[r] += n
        out = rep.step(entries, [])
        if graph is not None:
            assert rep.runner.last_used_graph and (graph, 0) in rep.runner._graphs
        if places:
            check(out, plain_rows(places), dtype, str([(r, n) for r, n, _ in parts][:4]))
        else:
            assert out is None

    first8 = [f"r{i}" for i in range(8)]
    step([("r0", 280, [0, 255, 279])])
    step([("r0", 20, [19])] + [(r, lengths[r] - 5, [lengths[r] - 6]) for r in first8[1:]])
    for _ in range(2):
        step([(r, 1, [0]) for r in first8], graph=8)
    rest = [f"r{i}" for i in range(8, 64)]
    step([(r, lengths[r] - 3, []) for r in rest[:28]])
    step([(r, lengths[r] - 3, [lengths[r] - 4]) for r in rest[28:]])
    for _ in range(2):
        step([(r, 1, [0]) for r in first8 + rest], graph=64)
    step([(r, 1, [0]) for r in first8[1:] + rest] + [("r64", 40, [0, 39])])
    assert all(at[r] == lengths[r] for r in lengths if r != "r0") and at["r0"] == 304
    rep.manager.check()


class PlainRows:
    """The plain implementation's logits at chosen (request, position) places of many sequences: every sequence runs
    whole through the plain layers once (matrices held as 32-bit tensors of the stored values, converted once), the last
    norm and the head only at the places asked for."""

    _stored: dict = {}  # folder -> its tensors in 32-bit (the stored values; shared by the runs in both precisions)

    def __init__(self, folder, dtype, seqs: dict) -> None:
        self.cfg = cfg = pl.read_config(folder)
        if str(folder) not in self._stored:
            self._stored.clear()  # one model's worth of memory at a time
            self._stored[str(folder)] = pl.read_weights(folder, torch.float32)
        # vectors (norm weights) in the run's precision, which decides how the norm rounds
        self.w = w = {k: (v.to(dtype) if v.dim() == 1 else v) for k, v in self._stored[str(folder)].items()}
        inv = pl.inverse_frequencies(cfg["head_dim"], cfg["theta"], cfg["scaling"])
        self.hidden = {}
        for r, toks in seqs.items():
            x = w["model.embed_tokens.weight"][torch.tensor(toks)].to(dtype)
            cos, sin = pl.rotation_tables(torch.arange(len(toks)), inv)
            for i in range(cfg["layers"]):
                x = pl.decoder_layer(x, w, f"model.layers.{i}.", cfg, cos, sin)
            self.hidden[r] = x

    def __call__(self, places) -> torch.Tensor:
        x = torch.stack([self.hidden[r][p] for r, p in places])
        return pl.rms_norm(x, self.w["model.norm.weight"], self.cfg["eps"]).float() @ self.w["lm_head.weight"].float().T


class Stepper:
    """Feeds sequences through a Replayer in the steps a test names and compares the wanted logits with ``PlainRows``."""

    def __init__(self, rep, seqs, plain, dtype) -> None:
        self.rep, self.seqs, self.plain, self.dtype = rep, seqs, plain, dtype
        self.at = {r: 0 for r in seqs}

    def __call__(self, parts, end=(), graph=None):
        """parts: (request, tokens it brings, places among them whose logits are compared); ``graph``: the (rows, tokens)
        of the captured step that must have run, or False for a step launched kernel by kernel."""
        entries, places = [], []
        for r, n, wants in parts:
            entries.append({"id": r, "tokens": self.seqs[r][self.at[r] : self.at[r] + n], "want": list(wants)})
            places += [(r, self.at[r] + i) for i in wants]
            self.at[r] += n
        out = self.rep.step(entries, list(end))
        if graph is False:
            assert not self.rep.runner.last_used_graph
        elif graph is not None:
            assert self.rep.runner.last_used_graph and graph in self.rep.runner._graphs, (graph, list(self.rep.runner._graphs))
        if places:
            check(out, self.plain(places), self.dtype, str([(r, n) for r, n, _ in parts][:4]))
        else:
            assert out is None


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
def test_benchmark_shape_steps_of_many_rows_match_plain(llama_8b_slice, dtype):
    """Steps of more than 128 rows at the benchmark's layer sizes, where other code runs than below (the library's
    products, sums into the stream by the library, norms of their own), against the plain implementation: decoding with
    200 live requests (the captured step of 208 rows) and a captured step of 32 decode rows beside a prompt portion of
    480 tokens, replayed with new tokens."""
    from nanospec_amd.engine.replay import Replayer
    from nanospec_amd.loader import load_model

    folder = llama_8b_slice
    vocab = pl.read_config(folder)["vocab"]
    lengths = {**{f"d{i}": 3 + i % 6 + 4 for i in range(200)}, "p": 2 * 480 + 3}
    seqs = {r: random_tokens(n, vocab, 8100 + i) for i, (r, n) in enumerate(lengths.items())}
    plain = PlainRows(folder, dtype, seqs)
    model = load_model(folder, dtype=dtype)
    rep = Replayer(model, 201 * 64 + 1024, page_size=16, max_live=201)
    step = Stepper(rep, seqs, plain, dtype)
    rows = [f"d{i}" for i in range(200)]
    for at in range(0, 200, 50):  # the prompts, fifty requests a step
        step([(r, lengths[r] - 4, [lengths[r] - 5] if r in ("d0", "d57", "d199") else []) for r in rows[at : at + 50]])
    every = [0] if dtype == torch.bfloat16 else []
    shown = {"d0", "d1", "d57", "d128", "d129", "d199"}  # (the 32-bit head over 200 rows takes its time: a few rows there)
    for _ in range(2):
        step([(r, 1, [0] if (every or r in shown) else []) for r in rows], graph=(208, 0))
    # 32 decode rows beside 480 prompt tokens: 512 rows in one captured step, twice
    for k in range(2):
        step([(r, 1, [0]) for r in rows[:32]] + [("p", 480, [0, 479])], graph=(32, 480), end=rows if k else ())
    step([("p", 3, [0, 1, 2])], end=["p"])
    rep.manager.check()


# ------------------------------------------------------------------------------------------------ the target model, whole


@pytest.fixture(scope="module")
def llama_1b_full(tmp_path_factory):
    """The Llama-3.2-1B shape at its full depth: 16 layers of width 2048, 32 heads over 8 key/value heads of 64,
    feed-forward 8192, vocabulary 128256, the head tied to the embedding, llama3 scaling with factor 32; random weights."""
    from nanospec_amd.config import LlamaConfig
    from nanospec_amd.weights import write_model_folder

    cfg = dict(architectures=["LlamaForCausalLM"], model_type="llama", vocab_size=128256, hidden_size=2048, intermediate_size=8192,
               num_hidden_layers=16, num_attention_heads=32, num_key_value_heads=8, head_dim=64, rms_norm_eps=1e-5, rope_theta=500000.0,
               max_position_embeddings=131072, tie_word_embeddings=True,
               rope_scaling=dict(rope_type="llama3", factor=32.0, low_freq_factor=1.0, high_freq_factor=4.0,
                                 original_max_position_embeddings=8192))
    return write_model_folder(tmp_path_factory.mktemp("llama1b_full") / "m", LlamaConfig.from_hf(cfg), seed=16, dtype=torch.bfloat16)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
def test_llama_1b_at_full_depth_matches_plain(llama_1b_full, dtype):
    """reference tests/test_correctness.py:68-80, at the depth of the model itself: sixteen layers of rounding on top of
    each other, the tied head of 128,256 rows after them.  One request whole; one with its last 32 tokens decoded one by
    one (captured steps); a third joins as a portion beside a decoded token, goes on with two tokens beside the next, and
    decodes beside it."""
    from nanospec_amd.engine.replay import Replayer
    from nanospec_amd.loader import load_model

    folder = llama_1b_full
    seqs = {"a": random_tokens(100, 128256, 41), "b": random_tokens(100, 128256, 42), "c": random_tokens(45, 128256, 43)}
    plain = PlainRows(folder, dtype, seqs)
    model = load_model(folder, dtype=dtype)
    assert len(model.layers) == 16 and model.spec.tie_head
    rep = Replayer(model, 4 * 128, page_size=16)
    step = Stepper(rep, seqs, plain, dtype)
    step([("a", 100, [0, 1, 31, 63, 64, 98, 99])], end=["a"], graph=False)
    step([("b", 68, [0, 67])])
    for p in range(68, 100):
        if p == 80:
            step([("b", 1, [0]), ("c", 37, [0, 36])])
        elif p == 81:
            step([("b", 1, [0]), ("c", 2, [0, 1])])
        elif p < 88:
            step([("b", 1, [0])] + ([("c", 1, [0])] if p > 81 else []))
        else:
            step([("b", 1, [0])], graph=(1, 0), end=["b"] if p == 99 else [])
    assert step.at == {"a": 100, "b": 100, "c": 45}
    rep.runner.release("c")
    rep.manager.check()


# ------------------------------------------------------------------------------------------------ the largest layer sizes


@pytest.fixture(scope="module")
def llama_70b_layer(tmp_path_factory):
    """Two layers of the Llama-3.1-70B shape (width 8192, 64 heads over 8 key/value heads of 128, feed-forward 28672,
    llama3 scaling with factor 8) with a vocabulary of 512, so that the plain implementation's head costs nothing.  (Two,
    because a layer's last product is handed to the next layer's norm in other forms than to the norm before the head.)"""
    from nanospec_amd.config import LlamaConfig
    from nanospec_amd.weights import write_model_folder

    cfg = dict(architectures=["LlamaForCausalLM"], model_type="llama", vocab_size=512, hidden_size=8192, intermediate_size=28672,
               num_hidden_layers=2, num_attention_heads=64, num_key_value_heads=8, head_dim=128, rms_norm_eps=1e-5, rope_theta=500000.0,
               max_position_embeddings=131072, tie_word_embeddings=False,
               rope_scaling=dict(rope_type="llama3", factor=8.0, low_freq_factor=1.0, high_freq_factor=4.0,
                                 original_max_position_embeddings=8192))
    return write_model_folder(tmp_path_factory.mktemp("llama70b") / "m", LlamaConfig.from_hf(cfg), seed=70, dtype=torch.bfloat16)


_PLAIN_70B = {}


@pytest.mark.parametrize("layouts", ["tiled", "both"])
def test_the_largest_layer_sizes_match_plain(llama_70b_layer, layouts, monkeypatch):
    """reference tests/test_backends.py:25-71 runs its kernels at the real head shape; here a whole layer at the largest
    shape the benchmark names, with only the re-laid matrices kept and with both layouts: a step of 1,100 tokens launched
    kernel by kernel (the library over plain copies or plain rows; the down-projection's inner size of 28,672 in four
    slices summed in 32-bit), a captured step of 800 tokens (the many-row kernel for what the library is kept from),
    decoding with 8 and with 64 live requests, and 63 decode rows beside a new prompt."""
    from nanospec_amd.engine.replay import Replayer
    from nanospec_amd.kernels import ops
    from nanospec_amd.loader import load_model
    from nanospec_amd.parts import linear

    folder, dtype = llama_70b_layer, torch.bfloat16
    lengths = {"p": 1903, **{f"r{i}": 4 + i % 7 + 5 for i in range(64)}, "q": 40}
    seqs = {r: random_tokens(n, 512, 7700 + i) for i, (r, n) in enumerate(lengths.items())}
    if "plain" not in _PLAIN_70B:
        _PLAIN_70B["plain"] = PlainRows(folder, dtype, seqs)
    plain = _PLAIN_70B["plain"]
    model = load_model(folder, dtype=dtype, layouts=layouts)
    seen = {"library": [], "rows": 0, "untile": 0}
    real_lib, real_rows, real_untile = linear.library_product, ops.linear_rows, ops.untile
    monkeypatch.setattr(linear, "library_product", lambda x, w_t, **k: (seen["library"].append(x.shape[1]), real_lib(x, w_t, **k))[1])
    monkeypatch.setattr(ops, "linear_rows", lambda *a, **k: (seen.__setitem__("rows", seen["rows"] + 1), real_rows(*a, **k))[1])
    monkeypatch.setattr(ops, "untile", lambda *a, **k: (seen.__setitem__("untile", seen["untile"] + 1), real_untile(*a, **k))[1])
    rep = Replayer(model, 2048 + 66 * 64, page_size=16, max_live=66)
    step = Stepper(rep, seqs, plain, dtype)
    step([("p", 1100, [0, 1, 640, 1099])], graph=False)
    # q/k/v, o, gate/up of both layers in one piece each and the first layer's down-projection in four slices of 7,168,
    # whichever layouts are kept; the last layer's, which does not end in the stream, through the many-row kernel
    assert sorted(seen["library"]) == [7168] * 4 + [8192] * 6, seen
    assert seen["rows"] == 1 and seen["untile"] == (12 if layouts == "tiled" else 0), seen
    seen["library"].clear()
    seen["rows"] = 0
    step([("p", 800, [0, 799])], graph=(0, 832))
    # (the step ran twice, before and during its capture) the down-projection through the many-row kernel; with only the
    # re-laid matrices every product, with both layouts the other three through the library
    if layouts == "tiled":
        assert seen["library"] == [] and seen["rows"] == 2 * 2 * 4, seen
    else:
        assert sorted(seen["library"]) == [8192] * 12 and seen["rows"] == 2 * 2, seen
    step([("p", 3, [0, 1, 2])], end=["p"])
    first8 = [f"r{i}" for i in range(8)]
    step([(r, lengths[r] - 5, [lengths[r] - 6]) for r in first8])
    for _ in range(2):
        step([(r, 1, [0]) for r in first8], graph=(8, 0))
    rest = [f"r{i}" for i in range(8, 64)]
    step([(r, lengths[r] - 3, [lengths[r] - 4]) for r in rest])
    for _ in range(2):
        step([(r, 1, [0]) for r in first8 + rest], graph=(64, 0))
    step([(r, 1, [0]) for r in first8[1:] + rest] + [("q", 40, [0, 39])])
    assert max(seen["library"], default=0) <= linear.LIBRARY_MAX_K
    rep.manager.check()
