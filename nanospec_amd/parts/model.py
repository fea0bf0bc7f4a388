"""A model built from a ``ModelSpec``: embedding, the layers in their run order, the last norm and
the output head (reference: model/llama.py:211-286).  Nothing here knows an architecture's name."""

from __future__ import annotations

import math
import sys

import torch

from ..kernels import ops
from ..weights import source as wsource
from . import registry
from .linear import LAYOUTS, LinearWeight
from .needs import PagedNeed, StateNeed


def _build_layers(spec):
    return [registry.build("block", layer, None) for layer in spec.layers]


def wanted_tensors(spec, layers=None) -> dict:
    """Every tensor the model reads from a checkpoint: name -> (shape, role)."""
    layers = layers if layers is not None else _build_layers(spec)
    out = {spec.embed_name: ((spec.vocab_size, spec.hidden), "embedding")}
    for layer in layers:
        out.update(layer.wanted())
    out.update(registry.build("norm", spec.final_norm, spec.final_norm_name).wanted())
    out[spec.head_name] = ((spec.vocab_size, spec.hidden), "linear")
    return out


class DecoderModel:
    def __init__(self, spec, config=None) -> None:
        self.spec, self.config = spec, config
        self.layers = _build_layers(spec)
        self.final_norm = registry.build("norm", spec.final_norm, spec.final_norm_name)
        self.embed: torch.Tensor | None = None
        self.head: LinearWeight | None = None
        self.dtype = self.device = None
        self._max_positions = "?"  # not asked yet
        # what every entry of the run order keeps in the cache
        self.cache_needs = [self.layers[c.layer].cache_need() if c.cache_from is None else None for c in spec.run_order]

    @property
    def graph_safe(self) -> bool:
        return all(layer.graph_safe for layer in self.layers)

    def batch_plans(self) -> list:
        """The batch plans of all layers' parts, one per key (``engine.context``)."""
        plans = {}
        for layer in self.layers:
            for plan in getattr(layer, "batch_plans", list)():
                plans.setdefault(plan.key, plan)
        return list(plans.values())

    def wanted(self) -> dict:
        return wanted_tensors(self.spec, self.layers)

    def load(self, source, dtype: torch.dtype, device, layouts: str = "auto") -> "DecoderModel":
        """Check the source against what the model wants (one error that lists everything wrong), then read
        each tensor once.  A head that is absent is the embedding table if the configuration ties them
        (reference: model/loader.py:62-70).  ``layouts``: "both" keeps every bfloat16 matrix in two layouts
        (``parts.linear.LAYOUTS``), "tiled" only in the re-laid one, "auto" chooses by the memory that is free."""
        spec = self.spec
        full = self.wanted()
        wanted = {k: v[0] for k, v in full.items()}
        wsource.check(source, wanted, optional={spec.head_name} if spec.tie_head else frozenset())
        self.dtype, self.device = dtype, torch.device(device)
        if layouts != "auto" and layouts not in LAYOUTS:
            raise ValueError(f"layouts={layouts!r}: use 'auto', 'both' or 'tiled'")
        if layouts == "auto":
            size = torch.finfo(dtype).bits // 8
            linear = sum(size * math.prod(shape) for name, (shape, role) in full.items() if role == "linear" and name != spec.head_name)
            free = torch.cuda.mem_get_info(self.device)[0]
            layouts = "both" if 2.2 * linear + size * 2 * spec.vocab_size * spec.hidden < 0.8 * free else "tiled"
            if layouts == "tiled" and dtype == torch.bfloat16:
                print(f"[nanospec_amd] {linear / 2**30:.0f} GiB of matrices, {free / 2**30:.0f} GiB free: keeping one layout; "
                      "steps of many tokens copy matrices into plain rows first and are slower", file=sys.stderr, flush=True)
        self.layouts = layouts
        get = source.get
        self.embed = get(spec.embed_name).to(device=device, dtype=dtype).contiguous()
        if spec.head_name in source.names():
            self.head = LinearWeight(get(spec.head_name).to(device=device, dtype=dtype).contiguous(), keep_plain=False)
        else:
            self.head = LinearWeight(self.embed, keep_plain=False)  # the embedding table is the head
        for layer in self.layers:
            if getattr(layer, "takes_layouts", False):
                layer.load(get, dtype, device, layouts)
            else:
                layer.load(get, dtype, device)
        self.final_norm.load(get, dtype, device)
        # whoever runs the model works on a stream of their own: everything that loading enqueued (copies, re-laying of
        # matrices, random draws) is finished before anyone can read it
        torch.cuda.synchronize(self.device)
        return self

    # ------------------------------------------------------------------ positions

    @property
    def max_positions(self) -> int | None:
        """The positions the model's parts can encode; None if nothing bounds them."""
        if self._max_positions == "?":
            limits = [layer.max_positions() for layer in self.layers if hasattr(layer, "max_positions")]
            limits = [n for n in limits if n is not None]
            self._max_positions = min(limits) if limits else None
        return self._max_positions

    def check_positions(self, last_position: int) -> None:
        limit = self.max_positions
        if limit is not None and last_position >= limit:
            raise ValueError(f"position {last_position} is beyond the model's {limit} positions")

    # ------------------------------------------------------------------ one pass over the given tokens

    def forward_hidden(self, ctx, caches) -> tuple[torch.Tensor, torch.Tensor]:
        """Run the tokens of ``ctx`` through every entry of the run order.  -> (resid, delta): the stream
        before the last sum.  ``caches[i]`` is the cache view of run-order entry i (its own or the one
        it reads)."""
        n = ctx.n_tokens
        resid = ctx.arena.take((n, self.spec.hidden), self.dtype)
        delta = ctx.arena.take((n, self.spec.hidden), self.dtype)
        ops.embed(self.embed, ctx.token_ids, out=resid, scale=self.spec.embed_scale)
        pending = None
        order = self.spec.run_order
        # buffers for what one block hands to the next (see PreNormBlock.forward)
        sums = ctx.arena.take((n, -(-self.spec.hidden // 16)), torch.float32)
        carry = ctx.arena.take((16 * n * self.spec.hidden,), torch.float32) if 16 < n <= ops.WIDE_TALL_ROWS and self.dtype == torch.bfloat16 else None
        for i, call in enumerate(order):
            layer = self.layers[call.layer]
            if getattr(layer, "links_blocks", False) and i + 1 < len(order):
                # the norm that reads this block's result is the next block's first
                nxt = getattr(self.layers[order[i + 1].layer], "entry_norm", None)
                out = layer.forward(ctx, resid, pending, caches[i], call.cache_from is None, delta, next_norm=nxt, next_sums=sums,
                                    next_carry=carry)
            else:
                if isinstance(pending, (ops.PreNormed, ops.Added)):
                    pending = None  # resid is whole already; a block that does not know the hand-over starts from it
                elif isinstance(pending, ops.PartialSums):
                    pending = ops.reduce_partial(pending, out=delta)
                out = layer.forward(ctx, resid, pending, caches[i], call.cache_from is None, delta)
            pending = out if out is not None else delta
        return resid, pending

    def logits(self, ctx, resid, delta, rows: torch.Tensor) -> torch.Tensor:
        """32-bit logits [len(rows), vocab] at the given token rows: last sum, last norm and head only there
        (reference: model/llama.py:284-286, engine/engine.py:382)."""
        n = rows.numel()
        h = self.final_norm.forward(ctx, resid=resid, x=delta, rows=rows, out=ctx.arena.take((n, self.spec.hidden), self.dtype))
        out = self.head(h, out=ctx.arena.take((n, self.spec.vocab_size), torch.float32), out_f32=True, arena=ctx.arena)
        if self.spec.logit_scale != 1.0 or self.spec.logit_softcap:
            ops.logit_transform(out, self.spec.logit_scale, self.spec.logit_softcap)
        return out
