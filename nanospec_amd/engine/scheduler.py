"""Which requests run in a step, and with how many tokens.  No tensors (bar each request's generator).

Reference: sched/scheduler.py.  Kept from it: FIFO admission without overtaking, ``max_admit`` per step,
``max_running`` live requests, and the rule that a request is admitted only if the pool can hold every
live request at its longest (:84-86,102-120), so that decoding never runs out of pages.  Added: a token
budget per step and prompts cut into portions under it, and a second policy for what happens when
pages run out.

A request's tokens are ``prompt + output``; ``computed`` of them are in the cache.  Every step a running
request brings its next tokens: exactly one when it is decoding, a portion when (part of) its prompt is
still to be computed.  It samples in the step that consumes its last known token.

Token budget (``max_step_tokens``): decoding requests come first with one token each.  The engine pads them to the
rows of a captured step, and ``decode_rows_cost`` says to how many: where the padded rows fit the budget they are what
is charged, so that prompts get what the padding leaves and a step of decode rows and its padding stays within the
budget; where they do not fit, the rows are charged as what they are (the padding then goes beyond the budget rather
than requests that would fit being left out).  What is left is given to unfinished prompts in admission order, at most
``prefill_chunk`` tokens per request and step.  The budget bounds the tokens that requests bring; the engine may pad a
step of prompt portions beside decode rows by up to 63 rows more to reach a captured shape.
When the budget does not even cover the decoding requests, those that have waited longest since their
last step go first (so that all of them advance in turn), and an eighth of the budget (at least one
token) is kept for the oldest unfinished prompt, so that it advances too.

Pages running out, by ``on_exhaustion``:
  "reserve"  (default, the reference's way): cannot happen; admission waits until the worst case fits.
  "preempt"  admission only needs the pages of the first portion.  When a step's tokens do not fit,
             the most recently admitted running requests are preempted until they do: their pages are
             freed and they go back to the HEAD of the queue to be recomputed from prompt + output
             (reference: Scheduler.restart, sched/scheduler.py:128-134).  A request that does not fit
             even alone raises ``PoolExhausted``.
"""

from __future__ import annotations

from collections import deque
from dataclasses import dataclass, field

import torch

from ..cache.manager import CacheManager
from ..cache.pages import PoolExhausted
from ..sampling.params import SamplingParams, TokenInfo


@dataclass
class Request:
    id: int
    prompt_ids: list[int]
    params: SamplingParams
    out_tokens: list[int] = field(default_factory=list)
    state: str = "waiting"  # waiting | running | done
    computed: int = 0  # tokens of prompt + output whose keys and values are in the cache
    gen: torch.Generator = None  # the request's own CPU generator (reference: sched/scheduler.py:64)
    logprobs: list[TokenInfo] = field(default_factory=list)  # only with params.logprobs
    step_logits: list = field(default_factory=list)  # only with EngineConfig.record_logits
    preemptions: int = 0
    served_at: int = -1  # the scheduler's ticket for this request's last step: smaller = longer ago

    def __post_init__(self) -> None:
        if not self.prompt_ids:
            raise ValueError("a request needs at least one prompt token")
        self.gen = torch.Generator()
        if self.params.seed is not None:
            self.gen.manual_seed(self.params.seed)
        else:
            self.gen.seed()

    @property
    def seq_len(self) -> int:
        return len(self.prompt_ids) + len(self.out_tokens)

    def token(self, i: int) -> int:
        n = len(self.prompt_ids)
        return self.prompt_ids[i] if i < n else self.out_tokens[i - n]

    @property
    def max_len(self) -> int:
        """The length the pool must be able to hold for this request: prompt + max_tokens, as the
        reference counts it (sched/scheduler.py:99-100)."""
        return len(self.prompt_ids) + self.params.max_tokens


@dataclass
class Work:
    """What one request brings to a step: tokens [start, start + n) of its sequence."""

    req: Request
    start: int
    n: int

    @property
    def samples(self) -> bool:
        return self.start + self.n == self.req.seq_len


class Scheduler:
    def __init__(self, cache: CacheManager, max_admit: int = 32, max_running: int | None = None,
                 max_step_tokens: int | None = None, prefill_chunk: int | None = None, on_exhaustion: str = "reserve") -> None:
        if on_exhaustion not in ("reserve", "preempt"):
            raise ValueError(f"on_exhaustion is 'reserve' or 'preempt', not {on_exhaustion!r}")
        self.cache = cache
        self.max_admit, self.max_running = max_admit, max_running
        self.max_step_tokens, self.prefill_chunk = max_step_tokens, prefill_chunk
        self.on_exhaustion = on_exhaustion
        self.waiting: deque[Request] = deque()
        self.running: list[Request] = []
        self.preempted_total = 0
        self.batches = 0  # tickets given so far (one per request and step)
        # hooks the engine sets so that device state follows admission and release
        self.on_admit = cache.admit
        self.on_release = cache.release
        # what so many rows of one token take of a step's token budget: the engine pads them to the size of a captured
        # step, and a step padded beyond the budget would cost more than the budget was meant to allow
        self.decode_rows_cost = lambda n: n

    @property
    def has_work(self) -> bool:
        return bool(self.waiting or self.running)

    def add(self, req: Request) -> None:
        assert req.state == "waiting"
        worst = self.cache.worst_case_pages(req.max_len)
        for g, need in enumerate(worst):
            if need > self._capacity(g):
                raise PoolExhausted(f"request {req.id} can need {need} pages of group {self.cache.groups[g].name!r}; "
                                    f"the pool has {self._capacity(g)}")
        self.waiting.append(req)

    def _capacity(self, g: int) -> int:
        ours = {r.id for r in self.running}
        held_by_others = sum(self.cache.get(rid).held[g] for rid in self.cache.live if rid not in ours)
        return self.cache.pools[g].num_pages - held_by_others

    # ------------------------------------------------------------------ admission

    def _held(self, req: Request) -> list[int]:
        return self.cache.get(req.id).held

    def _admit(self) -> list[Request]:
        groups = range(len(self.cache.groups))
        if self.on_exhaustion == "reserve":
            headroom = [self.cache.num_free(g) for g in groups]
            for r in self.running:
                worst, held = self.cache.worst_case_pages(r.max_len), self._held(r)
                for g in groups:
                    headroom[g] -= max(0, worst[g] - held[g])
        else:
            headroom = [self.cache.num_free(g) for g in groups]
        admitted: list[Request] = []
        while self.waiting and len(admitted) < self.max_admit and len(self.running) != self.max_running:
            req = self.waiting[0]
            if self.cache.slots.num_free == 0:
                break
            if self.on_exhaustion == "reserve":
                need = self.cache.worst_case_pages(req.max_len)
            else:
                first = req.seq_len if self.prefill_chunk is None else min(req.seq_len, self.prefill_chunk)
                need = self.cache.worst_case_pages(first)
            if any(need[g] > headroom[g] for g in groups):
                break  # strictly first come first served: nobody overtakes the head of the queue
            for g in groups:
                headroom[g] -= need[g]
            self.waiting.popleft()
            self.on_admit(req.id)
            req.state, req.computed = "running", 0
            self.running.append(req)
            admitted.append(req)
        return admitted

    # ------------------------------------------------------------------ one step

    def next_batch(self) -> list[Work]:
        """Admit, then say what every running request brings to this step.  Under "preempt" requests may be
        sent back to the queue so that what remains fits the pages."""
        self._admit()
        while True:
            work = self._compose()
            short = self._pages_short(work)
            if not short:
                # tickets in the order of the last ones: who was served earliest then is earliest again (a round robin)
                for w in sorted(work, key=lambda w: w.req.served_at):
                    self.batches += 1
                    w.req.served_at = self.batches
                return work
            if self.on_exhaustion != "preempt":
                raise PoolExhausted("pages ran out although admission reserves the worst case")
            if len(self.running) <= 1:
                raise PoolExhausted(f"request {self.running[0].id} does not fit the pool even alone")
            self.preempt(self.running[-1])

    def _compose(self) -> list[Work]:
        budget = self.max_step_tokens
        work: list[Work] = []
        decoding = [r for r in self.running if r.seq_len - r.computed == 1]
        filling = [r for r in self.running if r.seq_len - r.computed > 1]

        def cost(n: int, room: int) -> int:
            """What ``n`` rows of one token take of ``room`` tokens: with their padding if that fits, else as they are."""
            padded = self.decode_rows_cost(n)
            return padded if padded <= room else n

        if budget is not None and len(decoding) + (1 if filling else 0) > budget:
            # not every decoding request fits: the longest-waiting first, and a share for the oldest unfinished prompt
            share = max(1, budget // 8) if filling and budget > 1 else 0
            decoding = sorted(decoding, key=lambda r: r.served_at)[: max(0, budget - share)]
        for r in decoding:
            work.append(Work(r, r.computed, 1))
        if budget is not None:
            budget -= cost(len(decoding), budget - (1 if filling else 0))
        for r in filling:
            n = r.seq_len - r.computed
            if self.prefill_chunk is not None:
                n = min(n, self.prefill_chunk)
            if budget is not None:
                n = min(n, budget)
            if n <= 0:
                break
            work.append(Work(r, r.computed, n))
            if budget is not None:
                budget -= n
        order = {id(r): i for i, r in enumerate(self.running)}
        work.sort(key=lambda w: order[id(w.req)])
        return work

    def _pages_short(self, work: list[Work]) -> bool:
        need = [0] * len(self.cache.groups)
        for w in work:
            for g, n in enumerate(self.cache.pages_missing(w.req.id, w.n)):
                need[g] += n
        return any(n > self.cache.num_free(g) for g, n in enumerate(need))

    # ------------------------------------------------------------------ ends

    def finish(self, req: Request) -> None:
        self.running.remove(req)
        self.on_release(req.id)
        req.state = "done"

    def preempt(self, req: Request) -> None:
        """Free the request's pages and put it back at the head of the queue; prompt + output are
        recomputed when it is admitted again.  Emitted tokens are kept."""
        self.running.remove(req)
        self.on_release(req.id)
        req.state, req.computed = "waiting", 0
        req.preemptions += 1
        self.preempted_total += 1
        self.waiting.appendleft(req)
