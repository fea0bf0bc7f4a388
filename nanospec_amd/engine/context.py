"""One step's batch as the parts see it: flat token arrays, per-request arrays, block tables per cache
group and whatever plans the model's parts ask for (a mixer that works tile by tile, as the attention kernels
do, asks for the batch's requests as lists of tiles), all views of ONE int32 buffer that is filled on the host
and copied to the device in one piece.

Layout of the batch (reference: kv/cache.py:42-61,125-157 builds the same facts as qo_indptr /
kv_indptr / kv_indices / kv_last_page_len / positions / slots):
    token_ids[N] positions[N] token_req[N]        per token; token_req = index of its request in the batch
    qo_indptr[B+1] kv_lens[B] state_slots[B]      per request; kv_lens counts the keys after this step
    want_rows[R]                                  token rows whose logits are wanted
    patch_dst[P] patch_src[P]                     token rows whose ids come from a device tensor of the step before
    sample_opts[4, S]                             temperature, top_p, uniform number (float bits) and top_k of the rows that a
                                                  captured step samples itself
    plans                                         one region per batch plan of the model's parts (see ``BatchFacts``)
    block_table[g][B, P]                          page of positions [i*page, (i+1)*page), -1 if released
Slots are not materialised: the kernels compute page and offset from the position and the block table.

A batch plan is how a part gets a per-step description of the batch of its own onto the device, in the same copy: an
object with
    key                                  a name; parts that return plans of one key share one region
    shape(lens) -> shape                 what a batch of these token counts per request needs (any object)
    shape_captured(rows, tokens, portions) -> shape
                                         the most that a captured step needs: ``rows`` requests of one token, then up to
                                         ``portions`` requests that bring ``tokens`` tokens together
    ints(shape) -> int                   the size of the region, in 32-bit words
    fill(out, shape, facts)              write the region (a numpy int32 view) from the ``BatchFacts``
A part offers its plans as ``batch_plans() -> [plan, ...]`` and finds them at ``ctx.plans[key] = (device view, shape)``.
"""

from __future__ import annotations

from dataclasses import dataclass

import numpy as np
import torch


@dataclass
class BatchFacts:
    """What a batch plan is filled from (numpy int32 arrays per request unless said otherwise)."""

    n_tokens: int
    n_reqs: int
    lens: np.ndarray  # tokens each request brings
    starts: np.ndarray  # position of its first token
    indptr: np.ndarray  # [n_reqs + 1]: row of its first token
    kv: np.ndarray  # keys after this step (starts + lens)
    covered: int  # the first so many requests are to be described; in a batch of fixed shape the last one is a stand-in
    #               that owns the padding tokens behind the prompt portions, which no plan covers
    kv_layers: int  # run-order entries that keep keys and values in pages


def _pad4(n: int) -> int:
    return -(-n // 4) * 4


class BatchLayout:
    """Offsets of the fields inside the int32 buffer for given sizes."""

    def __init__(self, n_tokens: int, n_reqs: int, n_want: int, n_groups: int, table_width: int, n_patch: int = 0,
                 n_sample: int = 0, plans=()) -> None:
        """``plans``: (batch plan, its shape for this batch) pairs."""
        self.N, self.B, self.R, self.G, self.P = n_tokens, n_reqs, n_want, n_groups, table_width
        off = 0
        self.fields = {}
        self.plans = {plan.key: (plan, shape) for plan, shape in plans}
        for name, size in (("token_ids", n_tokens), ("positions", n_tokens), ("token_req", n_tokens), ("qo_indptr", n_reqs + 1),
                           ("kv_lens", n_reqs), ("state_slots", n_reqs), ("want_rows", n_want),
                           ("patch_dst", n_patch), ("patch_src", n_patch), ("sample_opts", 4 * n_sample),
                           *((key, plan.ints(shape)) for key, (plan, shape) in self.plans.items())):
            if name in self.fields:
                raise ValueError(f"two fields of the batch are called {name!r}")
            self.fields[name] = (off, size)
            off += _pad4(max(size, 1))
        self.table_off = []
        for _ in range(n_groups):
            self.table_off.append(off)
            off += _pad4(max(n_reqs * table_width, 1))
        self.total = off


class StepContext:
    """Device views of one step's batch plus the arena; handed to every part."""

    def __init__(self, layout: BatchLayout, dev_buf: torch.Tensor, arena, max_position: int, max_kv_len: int, captured: bool = False,
                 link_norms: bool = True, max_chunk_kv: int | None = None, pad_slot: int | None = None) -> None:
        self.layout, self.arena = layout, arena
        # A captured step has a fixed shape; what a batch does not fill is padding: rows that belong to a stand-in request
        # whose state slot is ``pad_slot`` (None in steps without padding).  A padding row's input may be anything (no
        # mixer tile covers the padding behind the prompt portions, so what earlier kernels left in the arena flows
        # through it, infinities and NaNs included) and nobody reads its output: a part must keep rows independent of
        # each other, or tell padding by ``state_slots[token_req[row]] == pad_slot`` on the device.
        self.pad_slot = pad_slot
        # the most keys that a request bringing a prompt portion has after this step (at most max_kv_len)
        self.max_chunk_kv = max_kv_len if max_chunk_kv is None else max_chunk_kv
        # blocks may let the products around an RMS norm do the norm's work (see parts.block.PreNormBlock.forward)
        self.link_norms = link_norms
        self.n_tokens, self.n_reqs = layout.N, layout.B
        self.max_position, self.max_kv_len = max_position, max_kv_len
        # the step is being captured for replays with other lengths (up to max_kv_len keys): a part's choices may depend
        # on the counts of the batch but not on this step's lengths
        self.captured = captured
        f = layout.fields

        def view(name):
            off, size = f[name]
            return dev_buf[off : off + size]

        self.token_ids, self.positions, self.token_req = view("token_ids"), view("positions"), view("token_req")
        self.qo_indptr, self.kv_lens, self.state_slots = view("qo_indptr"), view("kv_lens"), view("state_slots")
        self.want_rows = view("want_rows")
        # what the parts' batch plans wrote, by key: (device view of the plan's region, its shape for this batch)
        self.plans = {key: (view(key), shape) for key, (_, shape) in layout.plans.items()}
        self.block_tables = [dev_buf[o : o + layout.B * layout.P].view(layout.B, layout.P) for o in layout.table_off]


def fill_batch(host: np.ndarray, layout: BatchLayout, token_ids, starts, lens, slots, want_rows, tables: list[np.ndarray],
               kv_layers: int = 1, pad_tail: int | None = None) -> None:
    """Write one batch into ``host`` (int32, at least layout.total long).  ``starts``/``lens``: first
    position and token count per request; ``tables[g]``: int32 [B, P] block tables; ``kv_layers``: how many layers keep
    keys and values in pages.

    ``pad_tail`` (batches of a fixed shape, for captured steps): the last request of the batch is a stand-in that owns
    the last ``pad_tail`` token rows; they are all at position 0 (of a page nobody reads) and no plan covers them.  The
    plans' regions may then be larger than the batch needs (a plan fills the rest with entries that describe nothing), and
    ``want_rows`` is filled up with row 0."""
    f = layout.fields
    B = layout.B
    lens_a = np.asarray(lens, dtype=np.int32)
    starts_a = np.asarray(starts, dtype=np.int32)
    indptr = np.zeros(B + 1, dtype=np.int32)
    np.cumsum(lens_a, out=indptr[1:])

    def put(name, arr):
        off, size = f[name]
        host[off : off + size] = arr

    put("token_ids", np.asarray(token_ids, dtype=np.int32))
    req_of = np.repeat(np.arange(B, dtype=np.int32), lens_a)
    put("token_req", req_of)
    positions = np.arange(layout.N, dtype=np.int32) - indptr[req_of] + starts_a[req_of]
    tiled = B if pad_tail is None else B - 1  # requests that the plans cover
    if pad_tail:
        positions[layout.N - pad_tail :] = 0
    put("positions", positions)
    put("qo_indptr", indptr)
    put("kv_lens", starts_a + lens_a)
    put("state_slots", np.asarray(slots, dtype=np.int32))
    if layout.R:
        off, size = f["want_rows"]
        host[off : off + len(want_rows)] = np.asarray(want_rows, dtype=np.int32)
        host[off + len(want_rows) : off + size] = 0
    if layout.plans:
        facts = BatchFacts(layout.N, B, lens_a, starts_a, indptr, starts_a + lens_a, tiled, kv_layers)
        for key, (plan, shape) in layout.plans.items():
            off, size = f[key]
            plan.fill(host[off : off + size], shape, facts)
    for g, off in enumerate(layout.table_off):
        host[off : off + B * layout.P] = tables[g].reshape(-1)
