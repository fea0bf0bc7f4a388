"""RMS norm (reference: model/llama.py:86-95), with the residual sum of the surrounding block fused in."""

from __future__ import annotations

import torch

from ..kernels import ops
from .registry import register


class RMSNorm:
    graph_safe = True
    # y = weight * r / rms(r): linear in 1/rms(r), so a product that follows can apply that factor to its sums and a
    # product that precedes can gather the sum of squares (``parts.linear.IntoResidual``)
    links_products = True

    def __init__(self, spec, name: str) -> None:
        self.spec, self.name = spec, name
        self.weight: torch.Tensor | None = None

    def wanted(self) -> dict:
        return {self.name: ((self.spec.dim,), "norm")}

    def load(self, get, dtype, device) -> None:
        self.weight = get(self.name).to(device=device, dtype=dtype).contiguous()

    def forward(self, ctx, resid=None, x=None, rows=None, write_resid=False, out=None) -> torch.Tensor:
        return ops.rmsnorm(self.weight, self.spec.eps, resid=resid, x=x, rows=rows, write_resid=write_resid, out=out)


register("norm", "rmsnorm", RMSNorm)
