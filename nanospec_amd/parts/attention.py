"""Grouped-query soft-max attention over the paged cache (reference: model/llama.py:161-184 and
model/attention.py).

Per step: one product for q, k and v together (the three checkpoint matrices are stacked at load
time), rotation of q and k fused with the write of k and v into the pages, attention of every token
over its request's pages, output projection.  float32 runs the plain attention kernel; bfloat16 runs
the matrix-core kernel: prompt portions as tiles of 16 tokens of one head, decode rows as tiles of
all heads of a group with the keys cut into ranges that are joined afterwards.
"""

from __future__ import annotations

import torch

from ..kernels import ops
from . import registry
from .linear import Layouts, LinearWeight
from .needs import PagedNeed


class Attention:
    graph_safe = True
    ends_in_residual = True  # forward takes residual=IntoResidual

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

    def load(self, get, dtype, device) -> None:
        s = self.spec
        q, k, v, o = self._names
        rows = (s.heads + 2 * s.kv_heads) * s.head_dim
        wqkv = torch.empty((rows, s.hidden), dtype=dtype, device=device)
        at = 0
        for name in (q, k, v):
            t = get(name)
            wqkv[at : at + t.shape[0]].copy_(t)
            at += t.shape[0]
        self.position.load(get, dtype, device)
        # for few rows the stacked matrix is streamed by a kernel that rotates and writes the cache in its epilogue; it
        # wants the rows tiled in an order of its own
        rot = self.position.rotary_dim
        self.wqkv_rope = None
        if dtype == torch.bfloat16 and s.hidden % 8 == 0 and s.head_dim % 16 == 0 and rot % 16 == 0:
            self.wqkv_rope = ops.TiledWeight(wqkv, ops.qkv_rope_row_order(s.heads, s.kv_heads, s.head_dim, rot))
        # (without the plain layout the stacked matrix is also kept tiled in its own row order, for more than 16 rows)
        self.wqkv = LinearWeight(wqkv, tiled=self.wqkv_rope is None or not Layouts.keep_plain)
        self.wo = LinearWeight(get(o).to(device=device, dtype=dtype).contiguous())

    def cache_need(self):
        return PagedNeed(self.spec.kv_heads, self.spec.head_dim, self.spec.window)

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
                                s.heads, s.kv_heads, s.head_dim, pos.rotary_dim, write_kv=owns_cache)
        else:
            self.wqkv(x, out=qkv, arena=ctx.arena)
            ops.rope_kv_write(qkv, ctx.positions, ctx.token_req, table, pos.inv_freq, cache.k, cache.v, s.heads, s.kv_heads,
                              s.head_dim, pos.rotary_dim, write_kv=owns_cache)
        att = ctx.arena.take((n, s.heads * s.head_dim), x.dtype)
        page = cache.k.shape[2]
        if ops.mfma_attention_takes(x.dtype, s.head_dim, page):
            group = s.heads // s.kv_heads
            for plan in ctx.attention_plans(group, s.kv_heads, s.head_dim):
                ops.attention_mfma(qkv, att, cache.k, cache.v, plan.tiles, table, s.heads, s.kv_heads, s.head_dim,
                                   s.softmax_scale, window=s.window, hp=plan.hp, splits=plan.splits, workspace=plan.workspace,
                                   qt=plan.qt, coop=plan.coop)
        else:
            ops.attention_generic(qkv, att, cache.k, cache.v, ctx.token_req, ctx.positions, table, s.heads, s.kv_heads,
                                  s.head_dim, s.softmax_scale, window=s.window)
        if residual is not None:
            return self.wo.into_residual(att, residual, arena=ctx.arena)
        return self.wo(att, out=out, arena=ctx.arena)


registry.register("mixer", "attention", Attention)
