"""Logits -> tokens for a batch of rows with their own options, on the GPU, with one transfer back.

One uniform number per row comes from the request's own CPU generator, so a request's tokens do not
depend on what else is in the batch (reference: sched/scheduler.py:64,74-76, engine/engine.py:283);
the draw itself is ``kernels.ops.sample``.
"""

from __future__ import annotations

import torch

from ..kernels import ops
from .params import SamplingParams, TokenInfo


def sample_rows(logits: torch.Tensor, params: list[SamplingParams], uniforms: list[float]) -> list[TokenInfo]:
    """logits float32 [rows, vocab] on the GPU -> one TokenInfo per row.  Synchronises once."""
    dev = logits.device
    rows = logits.shape[0]
    if rows != len(params) or rows != len(uniforms):
        raise ValueError("one set of sampling options and one uniform number per row are wanted")
    host = torch.tensor([[p.temperature, p.top_p, u] for p, u in zip(params, uniforms)], dtype=torch.float32).t().contiguous()
    f = host.to(dev, non_blocking=True)
    filtered = any(p.top_k > 0 or p.top_p < 1.0 for p in params)
    top_k = torch.tensor([p.top_k for p in params], dtype=torch.int32).to(dev) if filtered else None
    tok, lp, slp = ops.sample(logits, f[0], f[2], top_k=top_k, top_p=f[1] if filtered else None)
    packed = torch.stack([tok.to(torch.float32), lp, slp]).tolist()  # the step's one synchronisation
    return [TokenInfo(int(packed[0][i]), packed[1][i], packed[2][i]) for i in range(rows)]
