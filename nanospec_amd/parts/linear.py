"""x @ W^T for the parts, choosing the kernel by precision and row count.

float32: always the plain tiled kernel with 32-bit fused multiply-adds in a fixed order (the true
32-bit path; no matrix-core mode of reduced precision is ever used).
bfloat16: up to 64 rows the hand-written matrix-core kernel that streams W once; beyond that the
platform's GEMM library, as the reference's nn.Linear does (model/llama.py:168-171), except for
32-bit results (logits), which run through the streaming kernel in slices of 64 rows.
"""

from __future__ import annotations

import torch

from ..kernels import ops


def linear(x: torch.Tensor, w: torch.Tensor, out: torch.Tensor | None = None, out_f32: bool = False) -> torch.Tensor:
    if x.dtype == torch.float32:
        return ops.linear_generic(x, w, out=out, out_f32=out_f32)
    if not ops.skinny_takes(x[:1], w):
        if x.shape[0] > ops.SKINNY_MAX_ROWS and not out_f32 and w.shape[1] % 8 == 0:
            return _library(x, w, out)
        return ops.linear_generic(x, w, out=out, out_f32=out_f32)
    m = x.shape[0]
    if m <= ops.SKINNY_MAX_ROWS:
        return ops.linear_skinny(x, w, out=out, out_f32=out_f32)
    if not out_f32:
        return _library(x, w, out)
    if out is None:
        out = torch.empty((m, w.shape[0]), dtype=torch.float32, device=x.device)
    for s in range(0, m, ops.SKINNY_MAX_ROWS):
        e = min(m, s + ops.SKINNY_MAX_ROWS)
        ops.linear_skinny(x[s:e], w, out=out[s:e], out_f32=True)
    return out


def _library(x: torch.Tensor, w: torch.Tensor, out: torch.Tensor | None) -> torch.Tensor:
    if out is None:
        return torch.matmul(x, w.t())
    return torch.matmul(x, w.t(), out=out)


def swiglu_up(x: torch.Tensor, gate_up: torch.Tensor, out: torch.Tensor | None = None, scratch=None) -> torch.Tensor:
    """silu(x @ Wg^T) * (x @ Wu^T) for gate_up = [Wg; Wu] of shape [2 I, H]."""
    inter = gate_up.shape[0] // 2
    if x.dtype == torch.bfloat16 and x.shape[0] <= ops.SKINNY_MAX_ROWS and ops.skinny_takes(x, gate_up):
        return ops.linear_skinny(x, gate_up[:inter], w2=gate_up[inter:], out=out)
    gu = linear(x, gate_up, out=scratch)
    return ops.silu_mul(gu, out=out)
