"""The step function: a batch of (request, its next tokens) -> logits at the wanted places.

``ModelRunner.step`` runs only the tokens it is given, as one batch, from the cache that earlier steps
left: portions of prompts beside single decoded tokens, cut anywhere.  It reserves pages for the new
tokens, builds the batch, runs the model and commits the new lengths.  Steps of one token per request,
and steps of a few prompt portions of moderate length beside such rows, replay a captured HIP graph of
a fixed shape when the model allows it; every other step is launched kernel by kernel.

Reference: engine/engine.py:200-252 (rows per request, one forward, hidden states at the last rows)
and model/llama.py:269-286 (logits only at the rows asked for).  Unlike the reference, prompts and
decode rows share ONE forward, and a prompt may come in portions.
"""

from __future__ import annotations

from dataclasses import dataclass, field

import numpy as np
import torch

from ..cache.manager import CacheManager
from ..cache.storage import CacheStorage
from ..kernels import ops
from .arena import Arena
from .context import BatchLayout, StepContext, fill_batch

# reference: engine/graphs.py:22 (powers of two up to 64).  48 and 96 besides: the products' cost goes by 16 rows at a time
# between 17 and 128 rows, so 40 requests padded to 64 rows pay for a quarter more than padded to 48.  Above 128 rows
# the library's products take the steps; 176, 208 and 240 are row counts at which its choice of kernels was measured to
# be good for all four shapes of a layer (160, 192 and 256 are not: q/k/v takes 40 us at 256 rows and 27 at 240).
GRAPH_BUCKETS = (1, 2, 4, 8, 16, 32, 48, 64, 96, 128, 176, 208, 240, 256)
PAD_REQUEST = "__pad__"


@dataclass
class StepEntry:
    req_id: object
    tokens: list[int]
    want: list[int] = field(default_factory=list)  # places among ``tokens`` whose logits are wanted


# Steps that hold prompt portions beside decode rows are captured too, in fixed shapes: so many rows of one token each (a
# bucket, or none), so many tokens of prompt portions (padded so that the step's rows are a multiple of MIXED_TOKEN_STEP) of at
# most MIXED_PORTIONS requests.  Launching such a step kernel by kernel costs the host about 0.1 ms a layer, more than the kernels of a small
# model take.  Longer steps run eagerly: there the GPU's work hides the host's.
MIXED_PORTIONS = 4
MIXED_TOKEN_STEP = 64
MIXED_MAX_TOKENS = 1024
MAX_GRAPHS = 96  # captured steps kept; the one not used for longest goes first.  What a captured step holds for itself is
#                   small (its batch buffer on both sides and its samples); the intermediates of all of them lie in one
#                   shared arena, see ``ModelRunner._arena_for``


class _StepGraph:
    """One captured step of a fixed shape: ``rows`` requests that bring one token each and up to ``portions`` requests
    that bring ``chunk`` tokens together; a static batch buffer, fixed addresses in the arena that all captured steps share
    (they replay one after another on one stream), logits and samples for ``rows + portions`` wanted places.  What a step does not fill is padding: pad rows and pad tokens belong to the
    runner's pad request (position 0 of a page nobody reads), tiles without tokens, wanted rows that nobody reads."""

    def __init__(self, runner: "ModelRunner", rows: int, chunk: int, width: int) -> None:
        self.rows, self.chunk, self.width = rows, chunk, width  # width: pages per request that its block tables can name
        self.portions = MIXED_PORTIONS if chunk else 0
        n_groups = len(runner.manager.groups)
        self.n_reqs = rows + self.portions + (1 if chunk else 0)  # the last one owns the pad tokens
        self.n_want = rows + self.portions
        plans = [(p, p.shape_captured(rows, chunk, self.portions)) for p in runner.plans]
        self.layout = BatchLayout(rows + chunk, self.n_reqs, self.n_want, n_groups, width, n_patch=rows, n_sample=self.n_want, plans=plans)
        dev = runner.device
        self.dev_buf = torch.zeros(self.layout.total, dtype=torch.int32, device=dev)
        self.host = torch.zeros(self.layout.total, dtype=torch.int32).pin_memory()
        self.host_np = self.host.numpy()
        self.arena: Arena | None = None  # the captured steps' shared arena, given at capture
        self.logits: torch.Tensor | None = None
        self.sampled = torch.zeros((3, self.n_want), dtype=torch.int32, device=dev)  # what the captured sampling kernel writes
        self.graph = None
        self.used = 0

    def sample_options(self):
        """Views of the batch buffer: (temperature, top_p, uniform) float32 and top_k int32, one per wanted place."""
        off, n = self.layout.fields["sample_opts"]
        opts = self.dev_buf[off : off + n].view(4, self.n_want)
        f = opts[:3].view(torch.float32)
        return f[0], f[1], f[2], opts[3]

    def context(self, runner, arena) -> StepContext:
        return StepContext(self.layout, self.dev_buf, arena, link_norms=runner.link_norms, max_position=0,
                           max_kv_len=self.width * runner.page_size, captured=True, pad_slot=runner.manager.get(PAD_REQUEST).slot)


class ModelRunner:
    def __init__(self, model, manager: CacheManager, storage: CacheStorage, max_requests: int, table_width: int,
                 use_graphs: bool = True) -> None:
        self.model, self.manager, self.storage = model, manager, storage
        self.device, self.dtype = model.device, model.dtype
        self.page_size = manager.page_size
        self.table_width = table_width  # the most pages that a request's block table can name
        self.max_requests = max_requests
        self.stream = torch.cuda.Stream(device=self.device)
        # whatever the caller's stream still has to do to the weights and the cache (copies, the pools' zero fill) comes
        # before the first step on this one
        self.stream.wait_stream(torch.cuda.current_stream(self.device))
        self.arena = Arena(self.device)
        self._kv_layers = sum(1 for need in model.cache_needs if need is not None and hasattr(need, "kv_heads"))
        self.plans = model.batch_plans() if hasattr(model, "batch_plans") else []  # what the parts want of every batch
        self.link_norms = True  # see StepContext; set False before the first step to run every norm as a kernel of its own
        n_groups = len(manager.groups)
        # host mirror of every live request's block tables, one row per state slot
        self._tables = [np.full((manager.slots.num_slots, table_width), -1, dtype=np.int32) for _ in range(n_groups)]
        self._mirrored = [[0] * manager.slots.num_slots for _ in range(n_groups)]
        self._released = [[0] * manager.slots.num_slots for _ in range(n_groups)]
        self._host = torch.zeros(1 << 14, dtype=torch.int32).pin_memory()
        self._dev = torch.zeros(1 << 14, dtype=torch.int32, device=self.device)
        self.use_graphs = bool(use_graphs and model.graph_safe)
        # captured steps by (rows of one token, tokens of prompt portions); recaptured wider when a request outgrows one
        self._graphs: dict[tuple[int, int], _StepGraph] = {}
        self._graph_uses = 0
        self._graph_arena: Arena | None = None  # the newest (largest) arena of the captured steps
        self._pad_ready = False
        self._staged: torch.cuda.Event | None = None
        self.last_used_graph = False
        self.last_sampled = None

    # ------------------------------------------------------------------ requests

    def admit(self, req_id) -> None:
        rc = self.manager.admit(req_id)
        for g in range(len(self._tables)):
            self._mirrored[g][rc.slot] = 0
            self._released[g][rc.slot] = 0
        if self.storage.states:
            with torch.cuda.stream(self.stream):
                self.storage.reset_slot(rc.slot)

    def release(self, req_id) -> None:
        self.manager.release(req_id)

    def _mirror(self, rc) -> None:
        for g, table in enumerate(rc.tables):
            if len(table) > self.table_width:
                raise ValueError(f"request {rc.req_id!r} needs {len(table)} pages; block tables hold {self.table_width}")
            row = self._tables[g][rc.slot]
            have = self._mirrored[g][rc.slot]
            if len(table) > have:
                row[have : len(table)] = table[have:]
                self._mirrored[g][rc.slot] = len(table)
            first = rc.first_kept[g]
            if first > self._released[g][rc.slot]:
                row[self._released[g][rc.slot] : first] = -1
                self._released[g][rc.slot] = first

    # ------------------------------------------------------------------ the step

    def step(self, entries: list[StepEntry], device_tokens=None, sampling=None) -> torch.Tensor | None:
        """Run one batch.  -> float32 logits [number of wanted places, vocab] in the order of the entries
        and of their ``want`` lists, or None if nothing is wanted.  Nothing here waits for the GPU.

        ``device_tokens`` = (int32 tensor on the GPU, [(entry index, row of the tensor), ...]): the first token id of
        those entries is taken from the tensor when the step runs (the id in ``tokens`` is a placeholder), so that a
        step can be enqueued before the step that samples its input has finished.

        ``sampling`` = ([SamplingParams per wanted place], [uniform number per wanted place]): if the step replays a
        captured graph the graph samples too, and ``last_sampled`` is then (int32 [3, places of the graph] on the GPU,
        places that count); otherwise ``last_sampled`` is None and the caller samples from the returned logits."""
        self.last_sampled = None
        if not entries:
            return None
        vocab = self.model.spec.vocab_size
        mgr = self.manager
        seen = set()
        for e in entries:
            if e.req_id in seen:
                raise ValueError(f"request {e.req_id!r} appears twice in one step")
            seen.add(e.req_id)
            if not e.tokens:
                raise ValueError(f"request {e.req_id!r} brings no tokens")
            if min(e.tokens) < 0 or max(e.tokens) >= vocab:
                raise ValueError(f"request {e.req_id!r} has a token id outside [0, {vocab})")
            if any(not 0 <= w < len(e.tokens) for w in e.want):
                raise ValueError(f"request {e.req_id!r} wants logits at a place it brings no token for")
        # pages for everything first: running out leaves every request as it was
        self._reserve_all(entries)
        rcs = [mgr.get(e.req_id) for e in entries]
        lens = [len(e.tokens) for e in entries]
        starts = [rc.length for rc in rcs]
        for rc in rcs:
            self._mirror(rc)
        n_want = sum(len(e.want) for e in entries)
        # A caller that works on another stream is ordered against this one on both sides.  A caller already on the
        # runner's stream (the engine) needs neither wait, and a wait between streams before every replay of a captured
        # step was measured to slow the replay itself by several per cent.
        caller = torch.cuda.current_stream(self.device)
        foreign = caller != self.stream
        if foreign:
            self.stream.wait_stream(caller)  # whatever the caller still reads of the last step's results
        if self._staged is not None:
            self._staged.synchronize()  # the last batch has left the pinned staging buffers
        with torch.cuda.stream(self.stream):
            shape = self._graph_shape(lens, n_want) if self.use_graphs else None
            if shape is not None:
                logits = self._step_graph(shape, entries, rcs, starts, lens, n_want, device_tokens, sampling)
                self.last_used_graph = True
            else:
                logits = self._step_eager(entries, rcs, starts, lens, n_want, device_tokens)
                self.last_used_graph = False
        if foreign:
            caller.wait_stream(self.stream)  # the caller's stream sees the logits
        for e, rc in zip(entries, rcs):
            mgr.commit(e.req_id, len(e.tokens))
        return logits

    def _reserve_all(self, entries) -> None:
        mgr = self.manager
        need = [0] * len(mgr.groups)
        for e in entries:
            for g, n in enumerate(mgr.pages_missing(e.req_id, len(e.tokens))):
                need[g] += n
        for g, n in enumerate(need):
            if n > mgr.num_free(g):
                from ..cache.pages import PoolExhausted

                raise PoolExhausted(f"the step needs {n} more pages in group {mgr.groups[g].name!r}, {mgr.num_free(g)} free")
        for e in entries:
            mgr.reserve(e.req_id, len(e.tokens))

    @staticmethod
    def _put_patch(host, layout, dst_rows, src_rows) -> None:
        off, size = layout.fields["patch_dst"]
        host[off : off + len(dst_rows)] = dst_rows
        off, size = layout.fields["patch_src"]
        host[off : off + len(src_rows)] = src_rows

    @staticmethod
    def _apply_patch(dev, layout, src, n) -> None:
        f = layout.fields
        ids = dev[f["token_ids"][0] : f["token_ids"][0] + f["token_ids"][1]]
        ops.scatter_i32(ids, dev[f["patch_dst"][0] : f["patch_dst"][0] + n], src, dev[f["patch_src"][0] : f["patch_src"][0] + n])

    def _step_eager(self, entries, rcs, starts, lens, n_want, device_tokens=None):
        n_tokens = sum(lens)
        max_kv = max(s + n for s, n in zip(starts, lens))
        self.model.check_positions(max_kv - 1)
        width = max(1, -(-max_kv // self.page_size))
        n_patch = len(device_tokens[1]) if device_tokens else 0
        layout = BatchLayout(n_tokens, len(entries), n_want, len(self._tables), width, n_patch, plans=[(p, p.shape(lens)) for p in self.plans])
        if layout.total > self._host.numel():
            size = 1 << (layout.total - 1).bit_length()
            self._host = torch.zeros(size, dtype=torch.int32).pin_memory()
            self._dev = torch.zeros(size, dtype=torch.int32, device=self.device)
        slots = [rc.slot for rc in rcs]
        token_ids = [t for e in entries for t in e.tokens]
        want_rows, base = [], 0
        for e, n in zip(entries, lens):
            want_rows.extend(base + w for w in e.want)
            base += n
        tables = [t[slots, :width] for t in self._tables]
        fill_batch(self._host.numpy(), layout, token_ids, starts, lens, slots, want_rows, tables, self._kv_layers)
        if n_patch:
            first_row = np.concatenate(([0], np.cumsum(lens)[:-1]))
            self._put_patch(self._host.numpy(), layout, [int(first_row[e]) for e, _ in device_tokens[1]], [r for _, r in device_tokens[1]])
        self._dev[: layout.total].copy_(self._host[: layout.total], non_blocking=True)
        self._staged = torch.cuda.Event()
        self._staged.record(self.stream)
        if n_patch:
            self._apply_patch(self._dev, layout, device_tokens[0], n_patch)
        self.arena.reset()
        chunk_kv = max((s + n for s, n in zip(starts, lens) if n != 1), default=0)
        ctx = StepContext(layout, self._dev, self.arena, max_position=max_kv - 1, max_kv_len=max_kv, link_norms=self.link_norms,
                          max_chunk_kv=chunk_kv)
        resid, delta = self.model.forward_hidden(ctx, self.storage.views)
        if not n_want:
            return None
        return self.model.logits(ctx, resid, delta, ctx.want_rows)

    # ------------------------------------------------------------------ graphs

    def _bucket(self, n: int) -> int | None:
        return next((b for b in GRAPH_BUCKETS if b >= n), None)

    def _graph_shape(self, lens, n_want: int) -> tuple[int, int] | None:
        """(rows of one token, tokens of prompt portions) of the captured step that takes this batch, or None if it runs
        eagerly: nothing wanted, more rows than the largest bucket, more or longer portions than a captured step holds.  The
        rows of a step that holds portions are padded to a multiple of ``MIXED_TOKEN_STEP``, up to 63 rows more than the
        requests bring (the scheduler's token budget counts what they bring)."""
        if not n_want:
            return None
        singles = sum(1 for n in lens if n == 1)
        rows = self._bucket(singles) if singles else 0
        if rows is None:
            return None
        if singles == len(lens):
            return (rows, 0) if n_want <= rows else None
        tokens = sum(lens) - singles
        if len(lens) - singles > MIXED_PORTIONS or tokens > MIXED_MAX_TOKENS or n_want > rows + MIXED_PORTIONS:
            return None
        # the step's rows, not the portions' tokens, are rounded up: a budget of 512 tokens then gives steps of 512 rows,
        # which the library's products take a fifth faster than 528 to 640 rows
        return rows, -(-(rows + tokens) // MIXED_TOKEN_STEP) * MIXED_TOKEN_STEP - rows

    def rows_cost(self, n: int) -> int:
        """Rows of a step that ``n`` requests with one token each take (they are padded to a bucket in a captured step)."""
        if not self.use_graphs or n == 0:
            return n
        return self._bucket(n) or n

    def _ensure_pad(self) -> None:
        if not self._pad_ready:
            self.admit(PAD_REQUEST)  # through admit(): the slot's mirrored block table starts empty
            self.manager.reserve(PAD_REQUEST, 1)
            self._mirror(self.manager.get(PAD_REQUEST))
            self._pad_ready = True

    def _fill_graph(self, g: _StepGraph, entries, rcs, starts, lens, device_tokens=None, sampling=None) -> int:
        """Real rows first, then pad rows that read and write the reserved pad page at position 0
        (reference: engine/graphs.py:115-167); then the prompt portions and the pad tokens.  -> wanted places filled."""
        pad = self.manager.get(PAD_REQUEST)
        single = [i for i, n in enumerate(lens) if n == 1]
        multi = [i for i, n in enumerate(lens) if n != 1]
        n_pad_rows, n_pad_portions = g.rows - len(single), g.portions - len(multi)
        slots = [rcs[i].slot for i in single] + [pad.slot] * n_pad_rows + [rcs[i].slot for i in multi]
        token_ids = [entries[i].tokens[0] for i in single] + [0] * n_pad_rows
        st = [starts[i] for i in single] + [0] * n_pad_rows + [starts[i] for i in multi]
        ln = [1] * g.rows + [lens[i] for i in multi]
        first_row = {i: r for r, i in enumerate(single)}
        at = g.rows
        for i in multi:
            first_row[i] = at
            token_ids += entries[i].tokens
            at += lens[i]
        tail = None
        if g.chunk:
            tail = g.rows + g.chunk - at
            slots += [pad.slot] * (n_pad_portions + 1)
            st += [0] * (n_pad_portions + 1)
            ln += [0] * n_pad_portions + [tail]
            token_ids += [0] * tail
        want_rows = [first_row[i] + w for i, e in enumerate(entries) for w in e.want]
        tables = [t[slots, : g.width] for t in self._tables]
        fill_batch(g.host_np, g.layout, token_ids, st, ln, slots, want_rows, tables, self._kv_layers, pad_tail=tail)
        if device_tokens:
            self._put_patch(g.host_np, g.layout, [first_row[e] for e, _ in device_tokens[1]], [r for _, r in device_tokens[1]])
        off, n = g.layout.fields["sample_opts"]
        opts = g.host_np[off : off + n].reshape(4, g.n_want)
        opts[:] = 0  # places that nobody reads: temperature 0
        if sampling is not None:
            params, uniforms = sampling
            k = len(params)
            f = opts[:3].view(np.float32)
            f[0, :k] = [p.temperature for p in params]
            f[1, :k] = [p.top_p for p in params]
            f[2, :k] = uniforms
            opts[3, :k] = [p.top_k for p in params]
        else:
            opts[:3].view(np.float32)[1] = 1.0
        g.dev_buf.copy_(g.host, non_blocking=True)
        self._staged = torch.cuda.Event()
        self._staged.record(self.stream)
        if device_tokens:
            self._apply_patch(g.dev_buf, g.layout, device_tokens[0], len(device_tokens[1]))
        return len(want_rows)

    GRAPH_MIN_WIDTH = 16  # pages per request that the narrowest captured step's block tables hold

    def _graph_for(self, shape: tuple[int, int], pages: int) -> _StepGraph:
        """The captured step of this shape, its block tables wide enough for ``pages`` pages per request.  Tables are as
        wide as the longest request has needed so far, rounded up to a power of two (every replay fills and copies
        requests x width ints), so a shape is captured again, twice as wide, when a request outgrows it."""
        g = self._graphs.get(shape)
        if g is None or g.width < pages:
            width = max(self.GRAPH_MIN_WIDTH, 1 << (pages - 1).bit_length())
            width = min(width, self.table_width)
            if g is not None or len(self._graphs) >= MAX_GRAPHS:
                self.stream.synchronize()  # a graph that is dropped may still be running
                self._graphs.pop(shape, None)
                if len(self._graphs) >= MAX_GRAPHS:
                    del self._graphs[min(self._graphs, key=lambda k: self._graphs[k].used)]
            g = self._capture(shape, width)
        self._graph_uses += 1
        g.used = self._graph_uses
        return g

    def _arena_for(self, nbytes: int) -> Arena:
        """The arena that a step captured now takes its intermediates from.  Captured steps replay one after another on
        the runner's stream, so all of them share one arena as large as the largest of them needs; a step that needs more
        than the arena has gets a new one, of the next power of two, which the steps captured later share.  Steps
        captured earlier keep the arena they were captured with until they are dropped, so all arenas together are less
        than twice the largest plus what dropped steps have not given back yet: the intermediates of one step, not of
        ``MAX_GRAPHS``."""
        have = self._graph_arena
        if have is None or have.capacity < nbytes:
            have = self._graph_arena = Arena(self.device, nbytes=1 << max(20, (nbytes - 1).bit_length()), fixed=True)
        return have

    @property
    def graph_arena_bytes(self) -> int:
        """Bytes of intermediates that the captured steps hold together (each shared arena counted once)."""
        arenas = {id(g.arena): g.arena for g in self._graphs.values() if g.arena is not None}
        if self._graph_arena is not None:
            arenas[id(self._graph_arena)] = self._graph_arena
        return sum(a.capacity for a in arenas.values())

    def _capture(self, shape: tuple[int, int], width: int) -> _StepGraph:
        self._ensure_pad()
        g = _StepGraph(self, shape[0], shape[1], width)
        self._fill_graph(g, [], [], [], [])

        def run(ctx):
            ctx.arena.reset()
            resid, delta = self.model.forward_hidden(ctx, self.storage.views)
            logits = self.model.logits(ctx, resid, delta, ctx.want_rows)
            temp, top_p, uni, top_k = g.sample_options()
            ops.sample(logits, temp, uni, top_k=top_k, top_p=top_p, out=g.sampled)
            return logits

        # a run outside the capture, in an arena that grows: it loads the libraries and measures what the step needs
        probe = Arena(self.device)
        run(g.context(self, probe))
        self.stream.synchronize()
        g.arena = self._arena_for(probe.high_water)
        del probe
        ctx = g.context(self, g.arena)
        graph = ops.Graph(self.stream)
        with graph:
            g.logits = run(ctx)
        g.graph = graph
        self._graphs[shape] = g
        return g

    def _step_graph(self, shape, entries, rcs, starts, lens, n_want, device_tokens=None, sampling=None):
        self._ensure_pad()
        max_kv = max(s + n for s, n in zip(starts, lens))
        pages = -(-max_kv // self.page_size)
        if pages > self.table_width:
            raise ValueError(f"a request needs {pages} pages; block tables hold {self.table_width}")
        self.model.check_positions(max_kv - 1)
        g = self._graph_for(shape, pages)
        if sampling is not None and len(sampling[0]) != n_want:
            sampling = None  # the caller samples from the logits
        self._fill_graph(g, entries, rcs, starts, lens, device_tokens, sampling)
        g.graph.launch()
        if sampling is not None:
            self.last_sampled = (g.sampled, n_want)
        return g.logits[:n_want]

    def synchronize(self) -> None:
        self.stream.synchronize()
