"""Grouped-query soft-max attention over the paged cache (reference: model/llama.py:161-184 and
model/attention.py).

Per step: one product for q, k and v together (the three checkpoint matrices are stacked at load
time), rotation of q and k fused with the write of k and v into the pages, attention of every token
over its request's pages, output projection.  float32 runs the plain attention kernel; bfloat16 runs
the matrix-core kernel: prompt portions as tiles of 16 tokens of one head, decode rows as tiles of
all heads of a group with the keys cut into ranges that are joined afterwards.
"""

from __future__ import annotations

from dataclasses import dataclass

import numpy as np
import torch

from ..kernels import ops
from . import registry
from .linear import LinearWeight
from .needs import PagedNeed

# How the matrix-core attention kernel is launched, from the counts of a step's batch and the size of the GPU
PORTION_RANGE_BLOCKS = 16  # the fewest 32-key blocks that a range of a prompt portion's keys is worth a workgroup of its own
PORTION_SINGLE_SET_BLOCKS = 128  # 32-key blocks of the longest row from which a workgroup is one set of waves instead of two
DECODE_WAVES_PER_UNIT = 4  # decode rows' keys are cut into ranges until about this many waves per compute unit are at work
LONG_ROW_KEYS = 8192  # rows that may reach this many keys get up to 32 ranges instead of 16
QKV_JOIN_MAX_RANGES = 4  # 17 to 128 rows: the kernel that joins the ranges of the q/k/v product, rotates and writes the cache reads
#                          every range, so more of them cost it what they gain the product


class TilePlan:
    """The batch as the matrix-core attention kernel walks it (a batch plan, see ``engine.context``): the requests that
    bring more than one token cut into tiles of ``TOKENS`` tokens, then the requests that bring exactly one, a tile each.
    A tile is ``ops.TILE_INTS`` ints: request, first token of the tile among the request's tokens of this step, row of the
    request's first token, tokens of the request in this step, keys after this step, and for one-token tiles the keys that
    all of them read in this step over all layers (by which the kernel chooses its loads: what cannot stay cached until
    the next step is read past the caches).  shape = (portion tiles, one-token tiles); a region of a fixed shape may hold
    more portion tiles than the batch needs: the rest bring no tokens and the kernel skips them."""

    key = "attention.tiles"
    TOKENS = 32

    def shape(self, lens) -> tuple[int, int]:
        return sum(-(-n // self.TOKENS) for n in lens if n != 1), sum(1 for n in lens if n == 1)

    def shape_captured(self, rows: int, tokens: int, portions: int) -> tuple[int, int]:
        # every portion may end in a tile that is not full
        return (-(-tokens // self.TOKENS) + portions if tokens else 0), rows

    def ints(self, shape) -> int:
        return ops.TILE_INTS * (shape[0] + shape[1])

    def fill(self, out: np.ndarray, shape, facts) -> None:
        tc, td = shape
        lens, indptr, kv, n = facts.lens, facts.indptr, facts.kv, facts.covered
        if tc:
            rows = [(b, t0, indptr[b], lens[b], kv[b], 0, 0, 0) for b in range(n) if lens[b] != 1 for t0 in range(0, lens[b], self.TOKENS)]
            rows += [(facts.n_reqs - 1, 0, 0, 0, 0, 0, 0, 0)] * (tc - len(rows))  # tiles without tokens
            out[: ops.TILE_INTS * tc] = np.asarray(rows, dtype=np.int32).reshape(-1)
        if td:
            req = np.nonzero(lens[:n] == 1)[0].astype(np.int32)
            d = np.zeros((td, ops.TILE_INTS), dtype=np.int32)
            k = len(req)
            d[:k, 0], d[:k, 2], d[:k, 3], d[:k, 4] = req, indptr[req], 1, kv[req]
            d[:k, 5] = min(int(kv[req].sum()) * facts.kv_layers, 2**31 - 1)
            out[ops.TILE_INTS * tc : ops.TILE_INTS * (tc + td)] = d.reshape(-1)

    @staticmethod
    def views(ctx):
        """-> (portion tiles, one-token tiles) as int32 [tiles, TILE_INTS] device views."""
        region, (tc, td) = ctx.plans[TilePlan.key]
        cut = ops.TILE_INTS * tc
        return region[:cut].view(tc, ops.TILE_INTS), region[cut : cut + ops.TILE_INTS * td].view(td, ops.TILE_INTS)


TILES = TilePlan()


@dataclass
class LaunchPlan:
    tiles: torch.Tensor  # int32 [n_tiles, 8]
    hp: int
    splits: int
    workspace: tuple | None
    qt: int = 1
    coop: bool = False


def launch_plans(ctx, group: int, kv_heads: int, head_dim: int) -> list[LaunchPlan]:
    """How the matrix-core attention kernel is launched for a mixer with ``group`` query heads per key/value head, over
    the tile lists of the batch: prompt portions as 32-token tiles of one head, their keys cut into ranges when there
    are too few tiles to fill the GPU and many keys (a short portion late in a long prompt); decode rows with all heads
    of a group in one tile and the keys cut into ranges so that the launch fills the GPU."""
    plans = []  # made afresh per call: the workspace lives in the caller's arena scope
    units = ops.compute_units(ctx.token_ids.device)
    chunk_tiles, decode_tiles = TilePlan.views(ctx)
    n_chunk_tiles, n_decode_tiles = chunk_tiles.shape[0], decode_tiles.shape[0]
    if n_chunk_tiles:
        tokens = TilePlan.TOKENS
        wgs = n_chunk_tiles * kv_heads * -(-group // 4)
        blocks = -(-ctx.max_chunk_kv // 32)
        # fewer workgroups than compute units (one fits a unit): cut the keys into ranges
        splits = max(1, min(16, units // wgs, blocks // PORTION_RANGE_BLOCKS))
        ws = None
        if splits > 1:
            cols = n_chunk_tiles * tokens * kv_heads * group
            ws = (ctx.arena.take((cols * splits * head_dim,), torch.float32), ctx.arena.take((cols * splits * 2,), torch.float32))
        # many workgroups with long rows of keys: one set of four waves per workgroup, two workgroups to a compute unit,
        # each with a barrier of its own (4 to 8% faster from 4,096 keys on; slower for short rows)
        single = splits == 1 and wgs >= 2 * units and blocks >= PORTION_SINGLE_SET_BLOCKS
        plans.append(LaunchPlan(chunk_tiles, 1, splits, ws, qt=tokens // 16, coop=single))
    if n_decode_tiles:
        hp = 1
        while hp < min(group, 16):
            hp *= 2
        # decode is bound by the latency of each wave's chain of loads: the four waves of a workgroup share a tile, and
        # the keys are cut into ranges until about a thousand waves are at work
        # (up to 32 ranges where requests may reach 8,192 keys and the tiles are few, a single request say: at 131,072
        # keys 86 against 132 us a layer; the kernel leaves the ranges beyond the sixteenth empty for shorter rows,
        # and where no request can be that long they are not launched: they would cost a captured step 1%)
        items = n_decode_tiles * kv_heads * -(-group // hp)
        splits = max(1, min(32 if ctx.max_kv_len >= LONG_ROW_KEYS else 16, DECODE_WAVES_PER_UNIT * units // (4 * items)))
        # never ranges of fewer than 256 keys (in a captured step: of what its block tables can hold): short rows are
        # short chains already, and a single range needs no kernel to join it
        splits = max(1, min(splits, -(-ctx.max_kv_len // 256)))
        ws = None
        if splits > 1:
            cols = n_decode_tiles * (16 // hp) * kv_heads * group
            ws = (ctx.arena.take((cols * splits * head_dim,), torch.float32), ctx.arena.take((cols * splits * 2,), torch.float32))
        plans.append(LaunchPlan(decode_tiles, hp, splits, ws, coop=True))
    return plans


class Attention:
    graph_safe = True
    ends_in_residual = True  # forward takes residual=IntoResidual
    takes_layouts = True  # load takes which copies of its matrices to keep

    def __init__(self, spec, prefix: str) -> None:
        if spec.heads % spec.kv_heads:
            raise ValueError(f"{spec.heads} heads are not a multiple of {spec.kv_heads} key/value heads")
        self.spec, self.prefix = spec, prefix
        self.position = registry.build("position", spec.position, prefix)
        if self.position.rotary_dim > spec.head_dim:
            raise ValueError("the rotary part of a head cannot be wider than the head")
        self.wqkv: LinearWeight | None = None
        self.wo: LinearWeight | None = None

    @property
    def _names(self):
        p = self.prefix
        return p + "q_proj.weight", p + "k_proj.weight", p + "v_proj.weight", p + "o_proj.weight"

    def wanted(self) -> dict:
        s = self.spec
        q, k, v, o = self._names
        return {
            q: ((s.heads * s.head_dim, s.hidden), "linear"),
            k: ((s.kv_heads * s.head_dim, s.hidden), "linear"),
            v: ((s.kv_heads * s.head_dim, s.hidden), "linear"),
            o: ((s.hidden, s.heads * s.head_dim), "linear"),
            **self.position.wanted(),
        }

    def load(self, get, dtype, device, layouts: str = "both") -> None:
        s = self.spec
        plain = layouts == "both"
        q, k, v, o = self._names
        rows = (s.heads + 2 * s.kv_heads) * s.head_dim
        wqkv = torch.empty((rows, s.hidden), dtype=dtype, device=device)
        at = 0
        for name in (q, k, v):
            t = get(name)
            wqkv[at : at + t.shape[0]].copy_(t)
            at += t.shape[0]
        self.position.load(get, dtype, device)
        # how the position encoding pairs channels and scales cosine and sine (the kernels' ``RopeForm``)
        self._form = dict(interleaved=bool(getattr(self.position, "interleaved", False)), factor=float(getattr(self.position, "factor", 1.0)))
        # for few rows the stacked matrix is streamed by a kernel that rotates and writes the cache in its epilogue; it
        # wants the rows tiled in an order of its own
        rot = self.position.rotary_dim
        self.wqkv_rope = None
        if dtype == torch.bfloat16 and s.hidden % 8 == 0 and s.head_dim % 16 == 0 and rot % 16 == 0:
            self.wqkv_rope = ops.TiledWeight(wqkv, ops.qkv_rope_row_order(s.heads, s.kv_heads, s.head_dim, rot, self._form["interleaved"]))
        # (without the plain layout the stacked matrix is also kept tiled in its own row order, for more than 16 rows)
        self.wqkv = LinearWeight(wqkv, keep_plain=plain, tiled=self.wqkv_rope is None or not plain)
        self.wo = LinearWeight(get(o).to(device=device, dtype=dtype).contiguous(), keep_plain=plain)

    def cache_need(self):
        return PagedNeed(self.spec.kv_heads, self.spec.head_dim, self.spec.window)

    def batch_plans(self) -> list:
        """What this mixer asks the batch builder to put on the device each step (``engine.context``)."""
        return [TILES]

    def max_positions(self) -> int | None:
        return self.position.max_positions

    def links_norms(self, rows: int) -> bool:
        """Whether, for this many rows, ``forward`` takes a ``PreNormed`` input and an ``IntoResidual`` ending."""
        first = self.wqkv_rope is not None or self.wqkv.links_norms(rows)
        return rows <= 16 and first and self.wo.links_norms(rows)

    def forward(self, ctx, x, cache, owns_cache: bool = True, out: torch.Tensor | None = None, residual=None):
        s = self.spec
        n = x.shape[0]
        pos = self.position
        if pos.max_positions is not None and ctx.max_position >= pos.max_positions:
            raise ValueError(f"position {ctx.max_position} is beyond the model's {pos.max_positions} positions")
        qkv = ctx.arena.take((n, self.wqkv.n), x.dtype)
        table = ctx.block_tables[cache.group]
        if self.wqkv_rope is not None and n <= 16 and ops.tiled_takes(x.x if isinstance(x, ops.PreNormed) else x, s.hidden):
            ops.linear_qkv_rope(x, self.wqkv_rope, qkv, ctx.positions, ctx.token_req, table, pos.inv_freq, cache.k, cache.v,
                                s.heads, s.kv_heads, s.head_dim, pos.rotary_dim, write_kv=owns_cache, **self._form)
        elif (self.wqkv_rope is not None and n <= ops.WIDE_TALL_ROWS and not isinstance(x, ops.PreNormed) and ops.tiled_takes(x[:1], s.hidden)
              and ops.wide_plan(self.wqkv_rope.n, s.hidden, n)[0] > 1):
            # 17 to 128 rows: the product streams the same tiled matrix with K cut into ranges, and the kernel that adds the
            # ranges rotates and writes the cache in the same pass (the library's product and a rotation kernel otherwise)
            ksplit, nt = ops.wide_plan(self.wqkv_rope.n, s.hidden, n)
            ksplit = min(ksplit, QKV_JOIN_MAX_RANGES)
            ws = ctx.arena.take((ksplit * n * self.wqkv_rope.n,), torch.float32)
            part = ops.linear_wide(x, self.wqkv_rope, workspace=ws, ksplit=ksplit, nt=nt, defer=True)
            ops.rope_kv_from_partial(part, qkv, ctx.positions, ctx.token_req, table, pos.inv_freq, cache.k, cache.v, s.heads, s.kv_heads,
                                     s.head_dim, pos.rotary_dim, write_kv=owns_cache, **self._form)
        else:
            self.wqkv(x, out=qkv, arena=ctx.arena, plain_copy=not ctx.captured)
            ops.rope_kv_write(qkv, ctx.positions, ctx.token_req, table, pos.inv_freq, cache.k, cache.v, s.heads, s.kv_heads,
                              s.head_dim, pos.rotary_dim, write_kv=owns_cache, **self._form)
        att = ctx.arena.take((n, s.heads * s.head_dim), x.dtype)
        page = cache.k.shape[2]
        if ops.mfma_attention_takes(x.dtype, s.head_dim, page):
            group = s.heads // s.kv_heads
            for plan in launch_plans(ctx, group, s.kv_heads, s.head_dim):
                ops.attention_mfma(qkv, att, cache.k, cache.v, plan.tiles, table, s.heads, s.kv_heads, s.head_dim,
                                   s.softmax_scale, window=s.window, hp=plan.hp, splits=plan.splits, workspace=plan.workspace,
                                   qt=plan.qt, coop=plan.coop)
        else:
            ops.attention_generic(qkv, att, cache.k, cache.v, ctx.token_req, ctx.positions, table, s.heads, s.kv_heads,
                                  s.head_dim, s.softmax_scale, window=s.window)
        if residual is not None:
            return self.wo.into_residual(att, residual, arena=ctx.arena, plain_copy=not ctx.captured)
        return self.wo(att, out=out, arena=ctx.arena, plain_copy=not ctx.captured)


registry.register("mixer", "attention", Attention)
