"""The pre-norm residual block (reference: model/llama.py:198-208):
    x = x + mixer(norm1(x));  x = x + feed_forward(norm2(x)).

The stream is carried as ``resid`` plus a ``delta`` that has not been added yet, so that every sum is
done inside the norm kernel that follows it (the reference's fused form, model/llama.py:240-254)."""

from __future__ import annotations

import torch

from ..kernels import ops
from . import registry
from .linear import IntoResidual

class PreNormBlock:
    def __init__(self, spec, prefix: str | None = None) -> None:
        p = spec.prefix if prefix is None else prefix
        self.spec = spec
        under = lambda given, part: p + (given if given is not None else part.kind + ".")
        self.mixer_norm = registry.build("norm", spec.mixer_norm, p + spec.mixer_norm_name)
        self.mixer = registry.build("mixer", spec.mixer, under(spec.mixer_prefix, spec.mixer))
        self.ffn_norm = registry.build("norm", spec.ffn_norm, p + spec.ffn_norm_name)
        self.ffn = registry.build("ffn", spec.ffn, under(spec.ffn_prefix, spec.ffn))
        self.parts = (self.mixer_norm, self.mixer, self.ffn_norm, self.ffn)

    @property
    def graph_safe(self) -> bool:
        return all(getattr(p, "graph_safe", False) for p in self.parts)

    def wanted(self) -> dict:
        out = {}
        for p in self.parts:
            out.update(p.wanted())
        return out

    def load(self, get, dtype, device, layouts: str = "both") -> None:
        for p in self.parts:
            if getattr(p, "takes_layouts", False):
                p.load(get, dtype, device, layouts)
            else:
                p.load(get, dtype, device)

    takes_layouts = True

    def cache_need(self):
        return self.mixer.cache_need()

    def batch_plans(self) -> list:
        return [plan for p in self.parts for plan in getattr(p, "batch_plans", list)()]

    def max_positions(self) -> int | None:
        """The positions the block's parts can encode; None if nothing bounds them."""
        limits = [p.max_positions() for p in self.parts if hasattr(p, "max_positions")]
        limits = [n for n in limits if n is not None]
        return min(limits) if limits else None

    @property
    def entry_norm(self):
        """The norm that reads what the block before this one left (for blocks that ``links_blocks``)."""
        return self.mixer_norm

    links_blocks = True  # forward takes next_norm, next_sums and next_carry

    def forward(self, ctx, resid, delta, cache, owns_cache, delta_out, next_norm=None, next_sums=None, next_carry=None):
        """``delta``: what the block before left to be added: a tensor (None at the start), a ``PartialSums``, a
        ``PreNormed``, in which case ``resid`` is already whole and the first norm's input comes ready for a product that
        ``links_norms``, or an ``Added`` (``resid`` is whole, nothing else comes with it).  ``next_norm``: the norm that will read this block's result (the next block's first one), if it
        ``links_products``; ``next_sums`` (float32 [tokens, ceil(width / 16)]) and ``next_carry`` (float32, 16 * tokens *
        width, or None): buffers that live as long as the step.
        -> None, with the block's not yet added output in ``delta_out``; or that output in one of the forms of
        ``IntoResidual`` (a tensor is then ``delta_out``)."""
        n = resid.shape[0]
        mark = ctx.arena.mark()
        link = getattr(ctx, "link_norms", False) and resid.dtype == torch.bfloat16
        takes = lambda part: link and getattr(part, "links_norms", lambda rows: False)(n)  # a PreNormed input
        ends = lambda part: link and getattr(part, "ends_in_residual", False)
        lp = lambda norm: link and norm is not None and getattr(norm, "links_products", False) and norm.weight.dtype == resid.dtype
        buf = lambda: ctx.arena.take(resid.shape, resid.dtype)

        # first norm and mixer
        whole = (ops.PreNormed, ops.Added)  # forms in which resid already holds the sum
        if isinstance(delta, whole):
            h = delta if isinstance(delta, ops.PreNormed) and takes(self.mixer) else self.mixer_norm.forward(ctx, resid=resid, out=buf())
        else:
            h = self.mixer_norm.forward(ctx, resid=resid, x=delta, write_resid=delta is not None, out=buf())
        if ends(self.mixer) and lp(self.ffn_norm):
            a = self.mixer.forward(ctx, h, cache, owns_cache, residual=IntoResidual(resid, self.ffn_norm.weight, self.ffn_norm.spec.eps))
        else:
            a = self.mixer.forward(ctx, h, cache, owns_cache, out=buf())

        # second norm and feed-forward
        if isinstance(a, whole):
            h2 = a if isinstance(a, ops.PreNormed) and takes(self.ffn) else self.ffn_norm.forward(ctx, resid=resid, out=buf())
        else:
            h2 = self.ffn_norm.forward(ctx, resid=resid, x=a, write_resid=True, out=buf())
        if ends(self.ffn) and lp(next_norm) and next_sums is not None:
            # what the next block reads must outlive this block's scratch
            out = self.ffn.forward(ctx, h2, residual=IntoResidual(resid, next_norm.weight, next_norm.spec.eps, delta_out, next_sums,
                                                                 next_carry, outlives=True))
            ctx.arena.release(mark)
            return out
        self.ffn.forward(ctx, h2, out=delta_out)
        ctx.arena.release(mark)
        return None


registry.register("block", "prenorm", PreNormBlock)
