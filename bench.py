"""Decode and prefill throughput of the Llama-3.1-8B shape with random weights on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

Prints ONE JSON line.  ``value`` is decoded tokens per second at batch 8 through the whole engine (scheduler,
step function, captured graphs, sampling).  The benchmark decodes from context 2,048 to 4,096; a step's time grows
linearly with the context, so K timed steps (after W untimed ones) are taken as a window centred on context 3,072,
the mean of 2,048..4,096, and stand for the whole run; with K >= 2,048 the whole run is timed (prompts of 2,048
random token ids, then 2,048 decode steps).  ``metric`` and ``config`` name the contexts that were timed.  ``points``
holds the same at batch 1 and 64 (windows of at most 256 steps), one request with a prompt of 128 tokens and 256 new tokens
timed as a whole (``decode_b1_ctx128``: the workload of the one figure that the reference publishes), and the new tokens per second of 32 requests served by
continuous batching at the Llama-3.2-1B shape (prompts of 16 to 1,024 tokens in portions of 512, 128 new tokens each);
``points_roofline_frac`` holds their fractions of the memory roofline (for the serving run: of what memory and matrix units
need together).  ``prefill`` is one step of 2,048 prompt tokens of one request; ``roofline`` is the bytes a decode
step must read (every weight once, the cache of the live requests) over its time, against 8 TB/s.
"""

from __future__ import annotations

import argparse
import json
import sys
import time

HBM_GBPS = 8000.0
PEAK_FLOPS = {"bf16": 2.5e15, "fp32": 157.3e12}

SHAPES = {}
SHAPES["8b"] = SHAPE_8B = dict(vocab_size=128256, hidden_size=4096, intermediate_size=14336, num_hidden_layers=32, num_attention_heads=32,
                num_key_value_heads=8, head_dim=128, rms_norm_eps=1e-5, rope_theta=500000.0, max_position_embeddings=131072,
                rope_scaling=dict(factor=8.0, low_freq_factor=1.0, high_freq_factor=4.0, original_max_position_embeddings=8192),
                tie_word_embeddings=False)
SHAPES["1b"] = dict(SHAPE_8B, hidden_size=2048, intermediate_size=8192, num_hidden_layers=16, head_dim=64, tie_word_embeddings=True,
                    rope_scaling=dict(SHAPE_8B["rope_scaling"], factor=32.0))
SHAPES["70b"] = dict(SHAPE_8B, hidden_size=8192, intermediate_size=28672, num_hidden_layers=80, num_attention_heads=64)
SHAPE_NAMES = {"8b": "Llama-3.1-8B shape", "1b": "Llama-3.2-1B shape", "70b": "Llama-3.1-70B shape"}


def weight_bytes(c, esize: int) -> int:
    """Bytes of every weight a decode step reads once: the layers, the last norm and the head (an embedding row per
    token is negligible and left out)."""
    per_layer = ((c.num_attention_heads + 2 * c.num_key_value_heads) * c.head_dim * c.hidden_size
                 + c.hidden_size * c.num_attention_heads * c.head_dim + 3 * c.intermediate_size * c.hidden_size + 2 * c.hidden_size)
    return (c.num_hidden_layers * per_layer + c.hidden_size + c.vocab_size * c.hidden_size) * esize


def kv_bytes_per_token(c, esize: int) -> int:
    return c.num_hidden_layers * 2 * c.num_key_value_heads * c.head_dim * esize


def prefill_flops(c, n: int, rows_with_logits: int) -> float:
    per_layer = ((c.num_attention_heads + 2 * c.num_key_value_heads) * c.head_dim * c.hidden_size
                 + c.hidden_size * c.num_attention_heads * c.head_dim + 3 * c.intermediate_size * c.hidden_size)
    linear = 2.0 * n * c.num_hidden_layers * per_layer + 2.0 * rows_with_logits * c.vocab_size * c.hidden_size
    attention = c.num_hidden_layers * 4.0 * c.num_attention_heads * c.head_dim * (n * (n + 1) / 2)
    return linear + attention


def decode_run(model, cfg, batch: int, prompt_len: int, first_ctx: int, steps: int, warmup: int, block_size: int, seed: int):
    """-> (seconds for ``steps`` decode steps, mean context of the first timed step and one past that of the last)."""
    import torch

    from nanospec_amd import Engine, EngineConfig, SamplingParams

    # Prompts are taken in portions beside the decoding of the requests that are through theirs, so the first request is a
    # few tokens ahead of the last when the clock starts.  No request ends before the clock stops: the engine enqueues
    # each step one ahead of the one it waits for, so the step enqueued in the last warm-up call has run before the
    # clock starts and the last timed call enqueues one more, and the clock covers the GPU's work of exactly ``steps`` steps.
    # (a prompt takes one step per 2,048 tokens, and one more when the decode rows of the step leave it less than that)
    ahead = batch * (-(-first_ctx // 2048) + 1) + 2
    total = first_ctx + ahead + warmup + steps + 2
    blocks = batch * -(-(total + 1) // block_size) + 2
    eng = Engine(model, EngineConfig(num_blocks=blocks, block_size=block_size, max_admit=batch, max_running=batch,
                                     max_step_tokens=2048, prefill_chunk=2048, max_seq_len=total + block_size))
    g = torch.Generator().manual_seed(seed)
    # a prompt of ``first_ctx`` tokens puts the first decode step at that context
    prompts = torch.randint(0, cfg.vocab_size, (batch, first_ctx), generator=g).tolist()
    reqs = [eng.add(p, SamplingParams(max_tokens=total - first_ctx)) for p in prompts]
    while any(r.computed < first_ctx for r in reqs):
        eng.step()  # prefill in portions of at most 2,048 tokens
    for _ in range(warmup):
        eng.step()
    eng.runner.synchronize()
    torch.cuda.synchronize()
    had = [len(r.out_tokens) for r in reqs]
    ctx0 = sum(r.computed for r in reqs) / batch + 1  # keys that the first timed step of the GPU attends to, on average
    t0 = time.perf_counter()
    for _ in range(steps):
        eng.step()
    eng.runner.synchronize()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    assert all(len(r.out_tokens) == n + steps for r, n in zip(reqs, had)), "a decode step did not produce one token per request"
    assert all(r.computed == len(r.prompt_ids) + n + steps for r, n in zip(reqs, had)), "the step enqueued ahead is missing"
    assert eng.runner.last_used_graph, "decode steps did not replay a captured graph"
    del eng
    torch.cuda.empty_cache()
    return dt, ctx0, ctx0 + steps


def prefill_run(model, cfg, n_tokens: int, block_size: int, reps: int = 3, portion: int = 0):
    """Seconds for a prompt of ``n_tokens``, whole or in portions of ``portion`` tokens (the best of ``reps`` passes)."""
    import torch

    from nanospec_amd.engine.replay import Replayer

    rep = Replayer(model, n_tokens + 64, page_size=block_size, use_graphs=False)
    toks = torch.randint(0, cfg.vocab_size, (n_tokens,), generator=torch.Generator().manual_seed(7)).tolist()
    portion = portion or n_tokens
    best = None
    for i in range(reps + 1):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for s in range(0, n_tokens, portion):
            last = s + portion >= n_tokens
            rep.step([{"id": f"p{i}", "tokens": toks[s : s + portion], "want": [min(portion, n_tokens - s) - 1] if last else []}],
                     [f"p{i}"] if last else [])
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        if i and (best is None or dt < best):
            best = dt  # the first pass warms the library's kernel selection
    del rep
    torch.cuda.empty_cache()
    return best


def short_run(model, cfg, prompt_len: int, new_tokens: int, block_size: int, reps: int = 2):
    """One request at a time, a short prompt and ``new_tokens`` greedy tokens, timed from ``add`` to the last token with the
    prompt's step included (the reference's own workload and clock: bench/run.py:162-172, batch 1, 256 new tokens after a
    short chat prompt).  -> seconds of the best pass; the first pass captures the graphs and is not timed."""
    import torch

    from nanospec_amd import Engine, EngineConfig, SamplingParams

    total = prompt_len + new_tokens + 2
    eng = Engine(model, EngineConfig(num_blocks=-(-total // block_size) + 4, block_size=block_size, max_admit=1, max_running=1,
                                     max_step_tokens=2048, prefill_chunk=2048, max_seq_len=total + block_size))
    g = torch.Generator().manual_seed(11)
    best = None
    for i in range(reps + 1):
        prompt = torch.randint(0, cfg.vocab_size, (prompt_len,), generator=g).tolist()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        req = eng.add(prompt, SamplingParams(max_tokens=new_tokens))
        while eng.has_work:
            eng.step()
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        assert len(req.out_tokens) == new_tokens
        if i and (best is None or dt < best):
            best = dt
    del eng
    torch.cuda.empty_cache()
    return best


def serve_run(model, cfg, n_requests: int, new_tokens: int, chunk: int, block_size: int, seed: int = 0, reps: int = 2):
    """Continuous batching with chunked prefill: ``n_requests`` arrive at once with prompts of 16 to 1,024 uniform-random
    token ids and generate ``new_tokens`` each; a step holds at most ``chunk`` tokens: one for every request that is
    through its prompt, the rest portions of prompts.  -> (seconds of the best pass, steps, prompt lengths, new tokens)."""
    import torch

    from nanospec_amd import Engine, EngineConfig, SamplingParams

    g = torch.Generator().manual_seed(seed)
    lens = torch.randint(16, 1025, (n_requests,), generator=g).tolist()
    prompts = [torch.randint(0, cfg.vocab_size, (n,), generator=g).tolist() for n in lens]
    per_request = -(-(1024 + new_tokens + 1) // block_size)
    best = None
    # One engine for all passes, as a server is one engine for all its requests: the first pass captures the steps' graphs
    # (the reference captures its graphs before it serves), the later ones are timed.
    eng = Engine(model, EngineConfig(num_blocks=n_requests * per_request + 2, block_size=block_size, max_admit=n_requests,
                                     max_running=n_requests, max_step_tokens=chunk, prefill_chunk=chunk,
                                     max_seq_len=1024 + new_tokens + block_size))
    for i in range(reps + 1):
        reqs = [eng.add(p, SamplingParams(max_tokens=new_tokens)) for p in prompts]
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        steps = 0
        while eng.has_work:
            eng.step()
            steps += 1
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        assert all(len(r.out_tokens) == new_tokens for r in reqs)
        if i and (best is None or dt < best[0]):
            best = (dt, steps, lens, n_requests * new_tokens)
    del eng
    torch.cuda.empty_cache()
    return best


def serve_ideal_seconds(cfg, esize: int, lens, new_tokens: int, steps: int, dtype: str) -> float:
    """What the serve workload needs at the least: every step reads the weights once, every decoded token the keys and
    values of its context, both at the memory's peak rate; and the arithmetic of the prompts at the matrix units' peak."""
    nbytes = steps * weight_bytes(cfg, esize)
    nbytes += sum((n + t) * kv_bytes_per_token(cfg, esize) for n in lens for t in range(new_tokens))
    flops = sum(prefill_flops(cfg, n, 1) for n in lens)
    return nbytes / (HBM_GBPS * 1e9) + flops / PEAK_FLOPS[dtype]


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=2048)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--layers", type=int, default=None, help="fewer layers than the shape has (both numbers are reported)")
    ap.add_argument("--dtype", default="bf16", choices=["bf16", "fp32"])
    ap.add_argument("--no-points", action="store_true")
    ap.add_argument("--ctx", type=int, default=2048, help="context of the first timed decode step (the benchmark's is 2,048)")
    ap.add_argument("--prefill-tokens", type=int, default=2048, help="length of the prompt of the prefill figure (the benchmark's is 2,048)")
    ap.add_argument("--prefill-portion", type=int, default=0, help="take that prompt in portions of this many tokens (0: whole)")
    ap.add_argument("--serve", type=int, default=0, metavar="REQUESTS",
                    help="instead of the benchmark: continuous batching of this many requests (prompts of 16 to 1,024 tokens, 128 new "
                         "tokens each, prompts in portions of 512)")
    ap.add_argument("--shape", default="8b", choices=sorted(SHAPES), help="the benchmark's shape is 8b; the others are for profiles")
    a = ap.parse_args()
    if a.gpus != 1:
        print("bench.py measures one GPU; this engine has no multi-GPU path (--gpus must be 1)")
        return 2

    import torch

    from nanospec_amd import LlamaConfig
    from nanospec_amd.loader import random_model

    shape = dict(SHAPES[a.shape])
    full_layers = shape["num_hidden_layers"]
    if a.layers:
        shape["num_hidden_layers"] = a.layers
    cfg = LlamaConfig.from_hf(dict(model_type="llama", **{k: v for k, v in shape.items() if k != "rope_scaling"},
                                   rope_scaling=dict(rope_type="llama3", **shape["rope_scaling"])))
    dtype = torch.bfloat16 if a.dtype == "bf16" else torch.float32
    esize = 2 if a.dtype == "bf16" else 4
    model = random_model(cfg, seed=0, dtype=dtype, on_device=True)
    block, prompt = 16, 2048
    if a.serve:
        dt, n_steps, lens, n_new = serve_run(model, cfg, a.serve, 128, 512, block)
        n_prompt = sum(lens)
        frac = serve_ideal_seconds(cfg, esize, lens, 128, n_steps, a.dtype) / dt
        print(json.dumps({"metric": f"continuous batching with chunked prefill of 512 ({SHAPE_NAMES[a.shape]}, {a.dtype}): new tok/s",
                          "value": round(n_new / dt, 1), "unit": "tok/s", "n_gpus": 1, "steps": n_steps, "seconds": round(dt, 4),
                          "all_tokens_per_s": round((n_prompt + n_new) / dt, 1), "higher_is_better": True, "dtype": a.dtype,
                          "roofline": {"bound": "hbm + matrix units", "frac": round(frac, 4),
                                       "what": "seconds that the weights of every step, the keys and values of every decoded token (at 8 TB/s) "
                                               "and the prompts' arithmetic (at the matrix units' peak) need at the least, over the seconds measured"},
                          "data": "synthetic: random weights N(0,0.02), uniform random token ids",
                          "config": {"model": SHAPE_NAMES[a.shape], "requests": a.serve, "prompt_tokens": n_prompt, "new_tokens": n_new,
                                     "prompt_len": "uniform 16..1024", "prefill_chunk": 512, "page_size": block}}), flush=True)
        return 0
    steps = a.steps
    whole_run = a.ctx == 2048 and steps >= 2048
    if a.ctx == 2048 and not whole_run:
        # a window of the run from 2,048 to 4,096, centred on its mean context (the requests are batch / 2 tokens into
        # their decoding, on average, when the last is through its prompt)
        first_ctx = 3072 - steps // 2 - a.warmup - 1 - a.batch
        window = f"{steps} steps centred on context 3072, the mean of the run from 2048 to 4096"
    else:
        first_ctx = a.ctx
        window = "the whole run" if whole_run else f"{steps} steps from context {a.ctx}"
    dt, ctx0, ctx1 = decode_run(model, cfg, a.batch, prompt, first_ctx, steps, a.warmup, block, seed=1)
    ms = 1000 * dt / steps
    value = a.batch * steps / dt
    mean_ctx = (ctx0 + ctx1 - 1) / 2
    step_bytes = weight_bytes(cfg, esize) + a.batch * mean_ctx * kv_bytes_per_token(cfg, esize)
    achieved = step_bytes / (dt / steps) / 1e9

    p_tokens = a.prefill_tokens
    p_dt = prefill_run(model, cfg, p_tokens, block, portion=a.prefill_portion)
    p_frac = prefill_flops(cfg, p_tokens, 1) / p_dt / PEAK_FLOPS[a.dtype]

    points, points_frac = {}, {}
    if not a.no_points:
        k = min(steps, 256)
        for b in (1, 64):
            lead = b  # the requests are b / 2 tokens into their decoding, on average, when the last is through its prompt
            d, c0, c1 = decode_run(model, cfg, b, prompt, 3072 - k // 2 - a.warmup - 1 - lead, k, a.warmup, block, seed=2 + b)
            points[f"decode_b{b}"] = round(b * k / d, 1)
            nbytes = weight_bytes(cfg, esize) + b * (c0 + c1 - 1) / 2 * kv_bytes_per_token(cfg, esize)
            points_frac[f"decode_b{b}"] = round(nbytes / (d / k) / 1e9 / HBM_GBPS, 4)

        # the reference's own published workload (README.md:72-76: 137 tok/s on an H100): one request, a short prompt, 256 new
        # tokens, the clock around the whole request
        d = short_run(model, cfg, 128, 256, block)
        points["decode_b1_ctx128"] = round(256 / d, 1)
        nbytes = weight_bytes(cfg, esize) + (128 + 128) * kv_bytes_per_token(cfg, esize)
        points_frac["decode_b1_ctx128"] = round(nbytes / (d / 256) / 1e9 / HBM_GBPS, 4)

    if not a.no_points and a.shape == "8b" and not a.layers:
        # the serving workload beside the headline: 32 requests through the Llama-3.2-1B shape, continuous batching with
        # prompts in portions of 512
        del model
        torch.cuda.empty_cache()
        small = dict(SHAPES["1b"])
        cfg1 = LlamaConfig.from_hf(dict(model_type="llama", **{k: v for k, v in small.items() if k != "rope_scaling"},
                                        rope_scaling=dict(rope_type="llama3", **small["rope_scaling"])))
        model1 = random_model(cfg1, seed=0, dtype=dtype, on_device=True)
        s_dt, s_steps, s_lens, s_new = serve_run(model1, cfg1, 32, 128, 512, block)
        points["serve_1b_32req_new_tok_s"] = round(s_new / s_dt, 1)
        points_frac["serve_1b_32req_new_tok_s"] = round(serve_ideal_seconds(cfg1, esize, s_lens, 128, s_steps, a.dtype) / s_dt, 4)
        del model1

    line = {
        "metric": f"decode tok/s at bs {a.batch}, ctx {ctx0:.0f}->{ctx1 - 1:.0f} ({SHAPE_NAMES[a.shape]}, {a.dtype}); prefill tok/s @{p_tokens} tok",
        "value": round(value, 1), "unit": "tok/s", "n_gpus": 1, "steps": steps, "warmup": a.warmup,
        "ms_per_step": round(ms, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": a.dtype, "data": "synthetic: random weights N(0,0.02), uniform random token ids",
        "config": {"model": SHAPE_NAMES[a.shape], "layers": shape["num_hidden_layers"], "layers_of_shape": full_layers,
                   "hidden": cfg.hidden_size, "heads": cfg.num_attention_heads, "kv_heads": cfg.num_key_value_heads,
                   "head_dim": cfg.head_dim, "intermediate": cfg.intermediate_size, "vocab": cfg.vocab_size,
                   "global_batch": a.batch, "seq_len": int(round(ctx1 - 1)), "prompt_len": first_ctx, "ctx_first_step": round(ctx0, 1),
                   "ctx_last_step": round(ctx1 - 1, 1), "timed": window, "page_size": block, "parallelism": "single GPU", "graphs": True},
        "prefill": {"value": round(p_tokens / p_dt, 1), "tokens": p_tokens, "ms": round(1000 * p_dt, 3), "frac": round(p_frac, 4)},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_GBPS, "unit": "GB/s",
                     "frac": round(achieved / HBM_GBPS, 4)},
        "points": points, "points_roofline_frac": points_frac,
    }
    print(json.dumps(line), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
