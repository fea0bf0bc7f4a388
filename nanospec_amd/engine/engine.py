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
from ..sampling.sampler import SampleStage, launch_sample
from .runner import ModelRunner, StepEntry
from .scheduler import Request, Scheduler, Work


@dataclass(frozen=True)
class EngineConfig:
    num_blocks: int  # pages in the cache pool (of every group of layers)
    block_size: int = 16  # tokens per page
    max_admit: int = 32  # admissions per step
    max_running: int | None = None  # concurrent requests; None = whatever the pool holds (at most 256)
    cuda_graphs: bool = True  # steps replay captured HIP graphs where they can (the reference's name for the option)
    record_logits: bool = False  # keep each request's per-step next-token logits on the CPU (tests)
    profile: bool = False  # per-phase event timings in Engine.prof
    head_chunk: int = 256  # rows per head + sampling pass
    max_step_tokens: int | None = None  # token budget of a step; None = whole prompts, as the reference
    prefill_chunk: int | None = None  # longest portion of one prompt in a step
    on_exhaustion: str = "reserve"  # "reserve" | "preempt": see engine/scheduler.py
    max_seq_len: int | None = None  # longest request that is accepted; None = what the model's positions and the pool allow
    lookahead: bool = True  # enqueue the next decode step before waiting for this one's tokens


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
        # the longest request: what the caller says and the model's positions allow (the pool bounds it too; the scheduler
        # refuses what can never fit it).  Block tables are only ever as wide as the live requests need: the runner's
        # captured steps grow with them.
        limits = [n for n in (model.max_positions, config.max_seq_len) if n is not None]
        self.max_seq_len = min(limits) if limits else None
        width = config.num_blocks if self.max_seq_len is None else min(config.num_blocks, -(-self.max_seq_len // config.block_size))
        self.runner = ModelRunner(model, self.cache, self.storage, max_running, width, use_graphs=config.cuda_graphs)
        self.sched = Scheduler(self.cache, config.max_admit, config.max_running, config.max_step_tokens, config.prefill_chunk,
                               config.on_exhaustion)
        self.sched.on_admit = self.runner.admit
        self.sched.on_release = self.runner.release
        self.sched.decode_rows_cost = self.runner.rows_cost
        self.usable_blocks = config.num_blocks
        if self.runner.use_graphs:
            self.runner._ensure_pad()  # one page is held for pad rows for good (reference: engine/engine.py:101-102)
            self.usable_blocks -= 1
        self.eos = set(model.spec.eos_token_ids)
        self._next_id = 0
        self.prof: dict[str, list[float]] = {}
        self._events: list[tuple[str, torch.cuda.Event]] = []
        self.steps = 0
        self._ahead: dict | None = None  # a decode step that was enqueued ahead of its turn
        self._stage = SampleStage(config.head_chunk)

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
        if self.max_seq_len is not None and len(prompt_ids) + params.max_tokens - 1 > self.max_seq_len:
            # (the last sampled token is never fed back, so a request holds at most prompt + max_tokens - 1 positions)
            raise ValueError(f"a prompt of {len(prompt_ids)} tokens with max_tokens={params.max_tokens} runs past the "
                             f"{self.max_seq_len} positions that the model and the engine's settings allow")
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

    @property
    def has_work(self) -> bool:
        return self.sched.has_work

    def step(self) -> list[Request]:
        """Admit, run one batch, sample, emit.  -> the requests that finished in this step.

        With ``lookahead`` (the default) a decode-only step whose requests go on is followed at once by the launch of
        the next step, whose input ids are taken on the GPU from this step's samples; only then does the host wait for
        this step's tokens.  The host's work between two steps is hidden behind the GPU's.  A request that turns out to
        have stopped on an end-of-sequence token has then already been given one more step, whose result is dropped."""
        with torch.cuda.stream(self.runner.stream):  # the whole step lives on the runner's stream: no waits between streams
            launched, self._ahead = self._ahead, None
            if launched is None:
                work = self.sched.next_batch()
                if not work:
                    return []
                launched = self._launch(work, None)
            if self._may_look_ahead(launched):
                try:
                    self._ahead = self._launch_ahead(launched)
                except Exception:
                    self._harvest(launched)  # this step's tokens are not lost to a failure of the next one's launch
                    raise
            return self._harvest(launched)

    def _launch(self, work: list[Work], token_src) -> dict:
        """Enqueue one step and its sampling.  ``token_src``: the launched step whose samples are this step's input ids."""
        self.steps += 1
        self._mark("start")
        device_tokens = None
        if token_src is None:
            entries = [StepEntry(w.req.id, [w.req.token(i) for i in range(w.start, w.start + w.n)], [w.n - 1] if w.samples else [])
                       for w in work]
        else:
            row_of = {id(w.req): i for i, w in enumerate(token_src["sampling"])}
            entries = [StepEntry(w.req.id, [0], [0]) for w in work]
            device_tokens = (token_src["sampled"][0][0], [(j, row_of[id(w.req)]) for j, w in enumerate(work)])  # row 0: the tokens
        samples = [w.samples for w in work] if token_src is None else [True] * len(work)
        sampling = [w for w, smp in zip(work, samples) if smp]
        # one uniform per request and step from its own generator (reference: engine/engine.py:283)
        uniforms = [float(torch.rand(1, generator=w.req.gen)) for w in sampling]
        # one per wanted place; with ``profile`` sampling stays a phase of its own, so that its time can be told apart
        in_graph = ([w.req.params for w in sampling], uniforms) if sampling and not self.config.profile else None
        logits = self.runner.step(entries, device_tokens, sampling=in_graph)
        self._mark("forward")
        for w in work:
            w.req.computed += w.n
        sampled, staged, kept = [], [], []
        if sampling and self.runner.last_sampled is not None:  # the captured step sampled as well
            buf, n = self.runner.last_sampled
            with torch.cuda.stream(self.runner.stream):
                sampled.append(buf)
                staged.append(self._stage.stage(buf, n))
                if self.config.record_logits:
                    kept.append(logits.cpu())
        elif sampling:
            with torch.cuda.stream(self.runner.stream):
                for s in range(0, len(sampling), self.config.head_chunk):
                    chunk = sampling[s : s + self.config.head_chunk]
                    u = uniforms[s : s + len(chunk)]
                    rows = logits[s : s + len(chunk)]
                    sampled.append(launch_sample(rows, [w.req.params for w in chunk], u, self._stage))
                    staged.append(self._stage.stage(sampled[-1]))
                    if self.config.record_logits:
                        kept.append(rows.cpu())
            self._mark("sample")
        return {"work": work, "sampling": sampling, "sampled": sampled, "staged": staged, "logits": kept,
                "graph": self.runner.last_used_graph}

    def _harvest(self, launched: dict) -> list[Request]:
        """Wait for a launched step's tokens, emit them, finish what is finished."""
        finished: list[Request] = []
        infos: list[TokenInfo] = []
        for chunk in launched["staged"]:  # waits for this step's samples only, not for a step enqueued after it
            infos.extend(self._stage.read(chunk))
        row = 0
        for w, info in zip(launched["sampling"], infos):
            req = w.req
            if req.state == "done":  # stopped on an end-of-sequence token while this step was already under way
                row += 1
                continue
            if launched["logits"]:
                cpu = launched["logits"][row // self.config.head_chunk]
                req.step_logits.append(cpu[row % self.config.head_chunk].clone())
            row += 1
            req.out_tokens.append(info.token)
            if req.params.logprobs:
                req.logprobs.append(info)
            # the stopping token is kept; the last token is never fed back (reference: engine/engine.py:155-163)
            if info.token in self.eos or len(req.out_tokens) >= req.params.max_tokens:
                self.sched.finish(req)
                finished.append(req)
        self._flush_prof()
        return finished

    def _may_look_ahead(self, launched: dict) -> bool:
        c = self.config
        if not c.lookahead or c.record_logits or c.profile or not launched["graph"] or self.sched.waiting:
            return False
        work = launched["work"]
        if len(work) != len(self.sched.running) or len(launched["sampling"]) != len(work):
            return False
        if c.max_step_tokens is not None and len(work) > c.max_step_tokens:
            return False
        # whoever reaches max_tokens with the token now being sampled stops; the others go on (unless that token ends them)
        return any(len(w.req.out_tokens) + 1 < w.req.params.max_tokens for w in work)

    def _launch_ahead(self, launched: dict) -> dict | None:
        from ..cache.pages import PoolExhausted

        work = [Work(w.req, w.req.computed, 1) for w in launched["work"] if len(w.req.out_tokens) + 1 < w.req.params.max_tokens]
        need = [0] * len(self.cache.groups)
        for w in work:
            for g, n in enumerate(self.cache.pages_missing(w.req.id, 1)):
                need[g] += n
        if any(n > self.cache.num_free(g) for g, n in enumerate(need)):
            return None  # let the scheduler decide who is preempted
        try:
            return self._launch(work, launched)
        except PoolExhausted:
            return None
