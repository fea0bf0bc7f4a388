"""One step's batch as the parts see it: flat token arrays, per-request arrays, block tables per cache
group and the batch's requests as lists of tiles (for mixers that work tile by tile, as the attention
kernels do), all views of ONE int32 buffer that is filled on the host and copied to the device in one piece.

Layout of the batch (reference: kv/cache.py:42-61,125-157 builds the same facts as qo_indptr /
kv_indptr / kv_indices / kv_last_page_len / positions / slots):
    token_ids[N] positions[N] token_req[N]        per token; token_req = index of its request in the batch
    qo_indptr[B+1] kv_lens[B] state_slots[B]      per request; kv_lens counts the keys after this step
    want_rows[R]                                  token rows whose logits are wanted
    patch_dst[P] patch_src[P]                     token rows whose ids come from a device tensor of the step before
    sample_opts[4, S]                             temperature, top_p, uniform number (float bits) and top_k of the rows that a
                                                  captured step samples itself
    chunk tiles [Tc, 8]                           requests with more than one token, 32 tokens per tile; a tile is
    decode tiles [Td, 8]                          (request, first token, first row, tokens, keys, 0, 0, 0); decode
                                                  tiles are the requests with exactly one token
    block_table[g][B, P]                          page of positions [i*page, (i+1)*page), -1 if released
Slots are not materialised: the kernels compute page and offset from the position and the block table.
"""

from __future__ import annotations

import numpy as np
import torch

CHUNK_TILE = 32  # tokens per tile of a prompt portion in the batch's tile lists
TILE_INTS = 8  # a tile descriptor: request, first token, row of the request's first token, tokens, keys, 0, 0, 0


def _pad4(n: int) -> int:
    return -(-n // 4) * 4


class BatchLayout:
    """Offsets of the fields inside the int32 buffer for given sizes."""

    def __init__(self, n_tokens: int, n_reqs: int, n_want: int, n_chunk_tiles: int, n_decode_tiles: int, n_groups: int,
                 table_width: int, n_patch: int = 0, n_sample: int = 0) -> None:
        self.N, self.B, self.R, self.Tc, self.Td, self.G, self.P = n_tokens, n_reqs, n_want, n_chunk_tiles, n_decode_tiles, n_groups, table_width
        off = 0
        self.fields = {}
        for name, size in (("token_ids", n_tokens), ("positions", n_tokens), ("token_req", n_tokens), ("qo_indptr", n_reqs + 1),
                           ("kv_lens", n_reqs), ("state_slots", n_reqs), ("want_rows", n_want),
                           ("ctiles", TILE_INTS * n_chunk_tiles), ("dtiles", TILE_INTS * n_decode_tiles),
                           ("patch_dst", n_patch), ("patch_src", n_patch), ("sample_opts", 4 * n_sample)):
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
                 link_norms: bool = True, max_chunk_kv: int | None = None) -> None:
        self.layout, self.arena = layout, arena
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
        # The requests of the batch as tiles, for mixers that work tile by tile: those that bring more than one token cut
        # into tiles of CHUNK_TILE tokens, and those that bring exactly one (int32 [tiles, TILE_INTS] each, see above)
        self.chunk_tiles = view("ctiles").view(-1, TILE_INTS)
        self.decode_tiles = view("dtiles").view(-1, TILE_INTS)
        self.n_chunk_tiles, self.n_decode_tiles = layout.Tc, layout.Td
        self.chunk_tiles_tokens = CHUNK_TILE
        self.block_tables = [dev_buf[o : o + layout.B * layout.P].view(layout.B, layout.P) for o in layout.table_off]


def fill_batch(host: np.ndarray, layout: BatchLayout, token_ids, starts, lens, slots, want_rows, tables: list[np.ndarray],
               kv_layers: int = 1, pad_tail: int | None = None) -> None:
    """Write one batch into ``host`` (int32, at least layout.total long).  ``starts``/``lens``: first
    position and token count per request; ``tables[g]``: int32 [B, P] block tables; ``kv_layers``: how many layers keep
    keys and values in pages.

    ``pad_tail`` (batches of a fixed shape, for captured steps): the last request of the batch is a stand-in that owns
    the last ``pad_tail`` token rows; they are all at position 0 (of a page nobody reads) and no tile covers them.  The
    layout's tile lists may then be longer than the batch needs: the rest of the prompt-portion tiles hold no tokens, and
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
    tiled = B if pad_tail is None else B - 1  # requests that the tile lists cover
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
    kv = starts_a + lens_a
    if layout.Td:
        req = np.nonzero(lens_a[:tiled] == 1)[0].astype(np.int32)
        d = np.zeros((len(req), TILE_INTS), dtype=np.int32)
        d[:, 0], d[:, 2], d[:, 3], d[:, 4] = req, indptr[req], 1, kv[req]
        # keys the decode rows read in this step over all layers: what would have to stay cached until the next step, by
        # which the attention kernel chooses its loads
        d[:, 5] = min(int(kv[req].sum()) * kv_layers, 2**31 - 1)
        put("dtiles", d.reshape(-1))
    if layout.Tc:
        rows = [(b, t0, indptr[b], n, kv[b], 0, 0, 0) for b, n in enumerate(lens[:tiled]) if n != 1 for t0 in range(0, n, CHUNK_TILE)]
        rows += [(B - 1, 0, 0, 0, 0, 0, 0, 0)] * (layout.Tc - len(rows))  # tiles without tokens
        put("ctiles", np.asarray(rows, dtype=np.int32).reshape(-1))
    for g, off in enumerate(layout.table_off):
        host[off : off + B * layout.P] = tables[g].reshape(-1)


def count_tiles(lens) -> tuple[int, int]:
    tc = sum(-(-n // CHUNK_TILE) for n in lens if n != 1)
    td = sum(1 for n in lens if n == 1)
    return tc, td
