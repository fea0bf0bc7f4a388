"""The dense SwiGLU feed-forward: down(silu(gate(x)) * up(x)), no bias (reference: model/llama.py:187-195).
Gate and up matrices are stacked at load time so that one pass over the input serves both."""

from __future__ import annotations

import torch

from ..kernels import ops
from . import registry
from .linear import linear, swiglu_up


class SwiGLU:
    graph_safe = True

    def __init__(self, spec, prefix: str) -> None:
        self.spec, self.prefix = spec, prefix
        self.gate_up: torch.Tensor | None = None
        self.down: torch.Tensor | None = None

    def wanted(self) -> dict:
        s, p = self.spec, self.prefix
        return {
            p + "gate_proj.weight": ((s.intermediate, s.hidden), "linear"),
            p + "up_proj.weight": ((s.intermediate, s.hidden), "linear"),
            p + "down_proj.weight": ((s.hidden, s.intermediate), "linear"),
        }

    def load(self, get, dtype, device) -> None:
        s, p = self.spec, self.prefix
        self.gate_up = torch.empty((2 * s.intermediate, s.hidden), dtype=dtype, device=device)
        self.gate_up[: s.intermediate].copy_(get(p + "gate_proj.weight"))
        self.gate_up[s.intermediate :].copy_(get(p + "up_proj.weight"))
        self.down = get(p + "down_proj.weight").to(device=device, dtype=dtype).contiguous()

    def forward(self, ctx, x: torch.Tensor, out: torch.Tensor | None = None) -> torch.Tensor:
        n, inter = x.shape[0], self.spec.intermediate
        act = ctx.arena.take((n, inter), x.dtype)
        fused = x.dtype == torch.bfloat16 and n <= ops.SKINNY_MAX_ROWS and ops.skinny_takes(x, self.gate_up)
        scratch = None if fused else ctx.arena.take((n, 2 * inter), x.dtype)
        swiglu_up(x, self.gate_up, out=act, scratch=scratch)
        return linear(act, self.down, out=out)


registry.register("ffn", "swiglu", SwiGLU)
