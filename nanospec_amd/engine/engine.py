"""The engine: requests in, tokens out, by continuous batching over the step function.

Names and meanings follow the reference (engine/engine.py): ``EngineConfig`` with ``num_blocks``,
``block_size``, ``max_admit``, ``max_running``, ``cuda_graphs``, ``record_logits``, ``profile``,
``head_chunk``; ``Engine.add`` / ``step`` / ``generate``; ``eng.sched.has_work``.  Token ids in, token
ids out; there is no tokenizer (reference: engine/engine.py:141-153).
"""

from __future__ import annotations

from dataclasses import dataclass

import torch

from ..cache.manager import CacheManager
from ..cache.storage import CacheStorage, plan_groups
from ..sampling.params import SamplingParams, TokenInfo
from ..sampling.sampler import sample_rows
from .runner import ModelRunner, StepEntry
from .scheduler import Request, Scheduler, Work


@dataclass(frozen=True)
class EngineConfig:
    num_blocks: int  # pages in the cache pool (of every group of layers)
    block_size: int = 16  # tokens per page
    max_admit: int = 32  # admissions per step
    max_running: int | None = None  # concurrent requests; None = whatever the pool holds (at most 256)
    cuda_graphs: bool = True  # decode steps replay a captured HIP graph (the reference's name for the option)
    record_logits: bool = False  # keep each request's per-step next-token logits on the CPU (tests)
    profile: bool = False  # per-phase event timings in Engine.prof
    head_chunk: int = 256  # rows per head + sampling pass
    max_step_tokens: int | None = None  # token budget of a step; None = whole prompts, as the reference
    prefill_chunk: int | None = None  # longest portion of one prompt in a step
    on_exhaustion: str = "reserve"  # "reserve" | "preempt": see engine/scheduler.py
    max_seq_len: int | None = None  # longest request (sizes the block tables); None = the whole pool


class Engine:
    def __init__(self, model, config: EngineConfig) -> None:
        self.model, self.config = model, config
        self.device, self.dtype = model.device, model.dtype
        if self.device.type != "cuda":
            raise RuntimeError("the engine runs on a GPU only; there is no CPU path")
        specs, _needs, _ = plan_groups(model.cache_needs)
        max_running = config.max_running if config.max_running is not None else 256
        num_slots = max_running + 1  # one for the pad rows of captured graphs
        self.cache = CacheManager(specs, config.num_blocks, config.block_size, num_slots)
        self.storage = CacheStorage(model, [config.num_blocks] * len(specs), config.block_size, num_slots, self.dtype, self.device)
        width = config.num_blocks if config.max_seq_len is None else -(-config.max_seq_len // config.block_size)
        self.runner = ModelRunner(model, self.cache, self.storage, max_running, width, use_graphs=config.cuda_graphs)
        self.sched = Scheduler(self.cache, config.max_admit, config.max_running, config.max_step_tokens, config.prefill_chunk,
                               config.on_exhaustion)
        self.sched.on_admit = self.runner.admit
        self.sched.on_release = self.runner.release
        self.usable_blocks = config.num_blocks
        if self.runner.use_graphs:
            self.runner._ensure_pad()  # one page is held for pad rows for good (reference: engine/engine.py:101-102)
            self.usable_blocks -= 1
        self.eos = set(model.spec.eos_token_ids)
        self._next_id = 0
        self.prof: dict[str, list[float]] = {}
        self._events: list[tuple[str, torch.cuda.Event]] = []
        self.steps = 0

    # ------------------------------------------------------------------ profiling (reference: engine/engine.py:83-95)

    def _mark(self, name: str) -> None:
        if self.config.profile:
            e = torch.cuda.Event(enable_timing=True)
            e.record(self.runner.stream)
            self._events.append((name, e))

    def _flush_prof(self) -> None:
        if not self._events:
            return
        self.runner.synchronize()
        for (_, ea), (b, eb) in zip(self._events, self._events[1:]):
            self.prof.setdefault(b, []).append(ea.elapsed_time(eb))
        self._events.clear()

    # ------------------------------------------------------------------ requests

    def add(self, prompt_ids: list[int], params: SamplingParams = SamplingParams()) -> Request:
        vocab = self.model.spec.vocab_size
        if any(not 0 <= int(t) < vocab for t in prompt_ids):
            raise ValueError(f"prompt holds a token id outside [0, {vocab})")
        req = Request(self._next_id, [int(t) for t in prompt_ids], params)
        self._next_id += 1
        self.sched.add(req)
        return req

    def generate(self, prompts: list[list[int]], params: SamplingParams | list[SamplingParams] = SamplingParams()) -> list[list[int]]:
        per = params if isinstance(params, (list, tuple)) else [params] * len(prompts)
        reqs = [self.add(p, s) for p, s in zip(prompts, per)]
        while self.sched.has_work:
            self.step()
        return [r.out_tokens for r in reqs]

    # ------------------------------------------------------------------ one step

    def step(self) -> list[Request]:
        """Admit, run one batch, sample, emit.  -> the requests that finished in this step."""
        work = self.sched.next_batch()
        if not work:
            return []
        self.steps += 1
        self._mark("start")
        entries = [StepEntry(w.req.id, [w.req.token(i) for i in range(w.start, w.start + w.n)], [w.n - 1] if w.samples else [])
                   for w in work]
        logits = self.runner.step(entries)
        self._mark("forward")
        for w in work:
            w.req.computed += w.n
        sampling = [w for w in work if w.samples]
        finished: list[Request] = []
        if sampling:
            infos: list[TokenInfo] = []
            with torch.cuda.stream(self.runner.stream):
                for s in range(0, len(sampling), self.config.head_chunk):
                    chunk = sampling[s : s + self.config.head_chunk]
                    # one uniform per request and step from its own generator (reference: engine/engine.py:283)
                    u = [float(torch.rand(1, generator=w.req.gen)) for w in chunk]
                    rows = logits[s : s + len(chunk)]
                    infos.extend(sample_rows(rows, [w.req.params for w in chunk], u))
                    if self.config.record_logits:
                        cpu = rows.cpu()
                        for i, w in enumerate(chunk):
                            w.req.step_logits.append(cpu[i].clone())
            self._mark("sample")
            for w, info in zip(sampling, infos):
                req = w.req
                req.out_tokens.append(info.token)
                if req.params.logprobs:
                    req.logprobs.append(info)
                # the stopping token is kept; the last token is never fed back (reference: engine/engine.py:155-163)
                if info.token in self.eos or len(req.out_tokens) >= req.params.max_tokens:
                    self.sched.finish(req)
                    finished.append(req)
        self._flush_prof()
        return finished
