"""Trace replay: given token ids go through the model step by step; the logits at the wanted places
are written out.  Nothing is sampled and nothing is scheduled: the trace says what every step holds.

This drives the same model, step function, cache manager and kernels that generation uses.
Closest patterns in the reference: tests/decode.py:12-39 and tests/test_graphs.py:43-72.
"""

from __future__ import annotations

import json
import sys
from pathlib import Path

import torch

from ..cache.manager import CacheManager
from ..cache.storage import CacheStorage, plan_groups
from .runner import ModelRunner, StepEntry

MAX_LIVE = 4  # requests a trace keeps alive at a time; one more slot serves the pad rows of graphs


class Replayer:
    def __init__(self, model, max_tokens: int, page_size: int = 16, use_graphs: bool = True, max_live: int = MAX_LIVE) -> None:
        self.model = model
        specs, _, _ = plan_groups(model.cache_needs)
        # room for ``max_tokens`` tokens of live requests, each rounded up to whole pages, plus the pad page
        pages = -(-max_tokens // page_size) + 1
        slots = max_live + 4
        self.manager = CacheManager(specs, pages, page_size, slots)
        self.storage = CacheStorage(model, [pages] * len(specs), page_size, slots, model.dtype, model.device)
        self.runner = ModelRunner(model, self.manager, self.storage, slots, pages, use_graphs=use_graphs)

    def step(self, entries: list[dict], end: list) -> torch.Tensor | None:
        with torch.cuda.stream(self.runner.stream):  # as the engine: everything on the runner's stream
            batch = []
            for e in entries:
                if e["id"] not in self.manager:
                    self.runner.admit(e["id"])
                batch.append(StepEntry(e["id"], [int(t) for t in e["tokens"]], [int(w) for w in e.get("want", [])]))
            logits = self.runner.step(batch)
            out = logits.cpu() if logits is not None else None  # copied before anything is given back
            for rid in end:
                if rid in self.manager:
                    self.runner.release(rid)
        return out


def run(model, max_tokens: int, out_dir, lines=None, page_size: int = 16, use_graphs: bool = True, log=sys.stdout) -> None:
    """Read one JSON object per line ({"step", "entries", "end"}), run it, write ``<step>.f32`` (little-endian
    float32 [wanted, vocab]) when something is wanted, print ``done <step>`` and flush."""
    out_dir = Path(out_dir)
    out_dir.mkdir(parents=True, exist_ok=True)
    rep = Replayer(model, max_tokens, page_size, use_graphs)
    for line in (lines if lines is not None else sys.stdin):
        line = line.strip()
        if not line:
            continue
        rec = json.loads(line)
        logits = rep.step(rec.get("entries", []), rec.get("end", []))
        if logits is not None:
            logits.contiguous().numpy().astype("<f4", copy=False).tofile(out_dir / f"{rec['step']}.f32")
        print(f"done {rec['step']}", file=log, flush=True)
