"""The dense SwiGLU feed-forward: down(silu(gate(x)) * up(x)), no bias (reference: model/llama.py:187-195).
Gate and up matrices are stacked at load time so that one pass over the input serves both."""

from __future__ import annotations

import torch

from . import registry
from .linear import GatedWeights, LinearWeight


class SwiGLU:
    graph_safe = True
    ends_in_residual = True  # forward takes residual=IntoResidual
    takes_layouts = True  # load takes which copies of its matrices to keep

    def __init__(self, spec, prefix: str) -> None:
        self.spec, self.prefix = spec, prefix
        self.gate_up: GatedWeights | None = None
        self.down: LinearWeight | None = None

    def wanted(self) -> dict:
        s, p = self.spec, self.prefix
        return {
            p + "gate_proj.weight": ((s.intermediate, s.hidden), "linear"),
            p + "up_proj.weight": ((s.intermediate, s.hidden), "linear"),
            p + "down_proj.weight": ((s.hidden, s.intermediate), "linear"),
        }

    def load(self, get, dtype, device, layouts: str = "both") -> None:
        s, p = self.spec, self.prefix
        plain = layouts == "both"
        self.gate_up = GatedWeights(get(p + "gate_proj.weight").to(device=device, dtype=dtype),
                                    get(p + "up_proj.weight").to(device=device, dtype=dtype), keep_plain=plain)
        self.down = LinearWeight(get(p + "down_proj.weight").to(device=device, dtype=dtype).contiguous(), keep_plain=plain)

    def links_norms(self, rows: int) -> bool:
        """Whether, for this many rows, ``forward`` takes a ``PreNormed`` input and an ``IntoResidual`` ending."""
        return self.gate_up.links_norms(rows) and self.down.links_norms(rows)

    def forward(self, ctx, x, out: torch.Tensor | None = None, residual=None):
        act = self.gate_up(ctx, x, out=ctx.arena.take((x.shape[0], self.spec.intermediate), x.dtype))
        if residual is not None:
            return self.down.into_residual(act, residual, arena=ctx.arena, plain_copy=not ctx.captured)
        return self.down(act, out=out, arena=ctx.arena, plain_copy=not ctx.captured)


registry.register("ffn", "swiglu", SwiGLU)
