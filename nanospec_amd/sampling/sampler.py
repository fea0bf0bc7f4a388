"""Logits -> tokens for a batch of rows with their own options, on the GPU, with one transfer back.

One uniform number per row comes from the request's own CPU generator, so a request's tokens do not
depend on what else is in the batch (reference: sched/scheduler.py:64,74-76, engine/engine.py:283);
the draw itself is ``kernels.ops.sample``.
"""

from __future__ import annotations

import torch

from ..kernels import ops
from .params import SamplingParams, TokenInfo


def launch_sample(logits: torch.Tensor, params: list[SamplingParams], uniforms: list[float], stage: "SampleStage | None" = None):
    """logits float32 [rows, vocab] on the GPU -> int32 [3, rows] on the GPU (tokens, bits of the raw log-probability,
    bits of the processed log-probability; see ``kernels.ops.sample``).  Waits for nothing: with a ``stage`` the options travel through pinned memory (a copy from ordinary host
    memory would wait for everything enqueued before it)."""
    dev = logits.device
    rows = logits.shape[0]
    if rows != len(params) or rows != len(uniforms):
        raise ValueError("one set of sampling options and one uniform number per row are wanted")
    # (contiguous buffers only: a copy between host and GPU of a strided view goes through a temporary and waits)
    host = stage.options(rows) if stage is not None else torch.empty((4, rows), dtype=torch.int32)
    fl = host[:3].view(torch.float32)
    fl[0] = torch.tensor([p.temperature for p in params], dtype=torch.float32)
    fl[1] = torch.tensor([p.top_p for p in params], dtype=torch.float32)
    fl[2] = torch.tensor(uniforms, dtype=torch.float32)
    host[3] = torch.tensor([p.top_k for p in params], dtype=torch.int32)
    d = torch.empty((4, rows), dtype=torch.int32, device=dev)
    d.copy_(host, non_blocking=True)
    if stage is not None:
        stage.sent(host)
    f = d[:3].view(torch.float32)
    filtered = any(p.top_k > 0 or p.top_p < 1.0 for p in params)
    return ops.sample(logits, f[0], f[2], top_k=d[3] if filtered else None, top_p=f[1] if filtered else None)


class SampleStage:
    """Pinned host buffers that sampled rows are copied into as soon as they exist, each copy followed by an event, so
    that reading one step's tokens waits for that step only and not for whatever was enqueued after it.  A buffer is
    taken by ``stage`` and given back by ``read``."""

    def __init__(self, rows: int) -> None:
        self.rows = rows
        self.free: list[torch.Tensor] = []
        self._options: list[tuple[torch.Tensor, torch.cuda.Event | None]] = []  # pinned [4, rows] int32 and their copies' events

    def options(self, rows: int) -> torch.Tensor:
        """A pinned buffer for the options of ``rows`` rows whose last copy to the GPU has finished."""
        if rows <= self.rows:
            for i, (buf, ev) in enumerate(self._options):
                if ev is None or ev.query():
                    del self._options[i]
                    return buf[: 4 * rows].view(4, rows)
        return torch.empty(4 * max(rows, self.rows), dtype=torch.int32).pin_memory()[: 4 * rows].view(4, rows)

    def sent(self, view: torch.Tensor) -> None:
        ev = torch.cuda.Event()
        ev.record(torch.cuda.current_stream())
        base = view._base if view._base is not None else view
        if base.numel() == 4 * self.rows:
            self._options.append((base, ev))

    def stage(self, sampled: torch.Tensor, rows: int | None = None):
        """``sampled``: int32 [3, width] on the GPU, contiguous; the first ``rows`` of each line count."""
        width = sampled.shape[1]
        host = self.free.pop() if self.free else torch.empty(3 * max(self.rows, width), dtype=torch.int32).pin_memory()
        host[: 3 * width].copy_(sampled.view(-1), non_blocking=True)
        done = torch.cuda.Event()
        done.record(torch.cuda.current_stream(sampled.device))
        return host, (width, width if rows is None else rows), done

    def read(self, staged) -> list[TokenInfo]:
        """The step's one wait for the GPU (reference: the single ``.tolist()`` of engine/engine.py:403)."""
        host, (width, n), done = staged
        done.synchronize()
        tok = host[:n].tolist()
        lp = host[width : 3 * width].view(torch.float32).tolist()
        if host.numel() == 3 * self.rows:
            self.free.append(host)
        return [TokenInfo(tok[i], lp[i], lp[width + i]) for i in range(n)]


def read_sample(sampled: torch.Tensor) -> list[TokenInfo]:
    n = sampled.shape[1]
    host = sampled.cpu()
    tok, lp, slp = host[0].tolist(), host[1].view(torch.float32).tolist(), host[2].view(torch.float32).tolist()
    return [TokenInfo(tok[i], lp[i], slp[i]) for i in range(n)]


def sample_rows(logits: torch.Tensor, params: list[SamplingParams], uniforms: list[float]) -> list[TokenInfo]:
    """logits float32 [rows, vocab] on the GPU -> one TokenInfo per row.  Synchronises once."""
    return read_sample(launch_sample(logits, params, uniforms))
