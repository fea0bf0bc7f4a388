"""Schedules for trace replay: the same token sequences cut into steps in different ways.

A trace is a list of steps ``{"step": i, "entries": [{"id", "tokens", "want"}], "end": [ids]}``.  Every builder
also returns, per step, which (request, position) each wanted row is, so that the logits can be compared
with the plain implementation's whole-sequence logits.
"""

from __future__ import annotations

import random


def whole(seqs: dict[str, list[int]]):
    """Each request alone and whole, every position wanted."""
    steps, where = [], []
    for i, (rid, toks) in enumerate(seqs.items()):
        steps.append({"step": i, "entries": [{"id": rid, "tokens": toks, "want": list(range(len(toks)))}], "end": [rid]})
        where.append([(rid, p) for p in range(len(toks))])
    return steps, where


def tail_decoded(seqs: dict[str, list[int]], tail: int = 32):
    """Most of a request in one step, the last ``tail`` tokens one by one."""
    steps, where = [], []
    for rid, toks in seqs.items():
        head = max(1, len(toks) - tail)
        steps.append({"step": len(steps), "entries": [{"id": rid, "tokens": toks[:head], "want": [head - 1]}], "end": []})
        where.append([(rid, head - 1)])
        for p in range(head, len(toks)):
            steps.append({"step": len(steps), "entries": [{"id": rid, "tokens": [toks[p]], "want": [0]}],
                          "end": [rid] if p == len(toks) - 1 else []})
            where.append([(rid, p)])
        if head == len(toks):
            steps[-1]["end"] = [rid]
    return steps, where


def portions(seqs: dict[str, list[int]], seed: int = 0, sizes=(2, 3, 5, 7, 16, 17, 31, 2, 40)):
    """Portions of changing size, down to two tokens; every position wanted."""
    rng = random.Random(seed)
    steps, where = [], []
    for rid, toks in seqs.items():
        at = 0
        while at < len(toks):
            n = min(rng.choice(sizes), len(toks) - at)
            last = at + n == len(toks)
            steps.append({"step": len(steps), "entries": [{"id": rid, "tokens": toks[at : at + n], "want": list(range(n))}],
                          "end": [rid] if last else []})
            where.append([(rid, p) for p in range(at, at + n)])
            at += n
    return steps, where


def mixed(seqs: dict[str, list[int]], seed: int = 0, max_live: int = 4, decode_tail: int = 12):
    """Up to ``max_live`` requests live: portions of some beside decoded tokens of others; a request sometimes sits
    a step out; finished requests give their pages back and later ones get them.  -> (steps, where, peak tokens held
    when each request's count is rounded up to a multiple of 64)."""
    rng = random.Random(seed)
    queue = list(seqs.items())
    live: dict[str, int] = {}  # id -> tokens done
    steps, where, peak = [], [], 0
    while queue or live:
        while queue and len(live) < max_live and (not live or rng.random() < 0.6):
            rid, _ = queue.pop(0)
            live[rid] = 0
        entries, w, ended = [], [], []
        for rid in list(live):
            toks, at = seqs[rid], live[rid]
            if len(live) > 1 and rng.random() < 0.2:
                continue  # sits this step out
            left = len(toks) - at
            if left <= decode_tail:
                n = 1
            else:
                n = min(rng.choice((2, 3, 6, 11, 19, 30)), left - decode_tail)
            want = list(range(n)) if rng.random() < 0.7 else [n - 1]
            entries.append({"id": rid, "tokens": toks[at : at + n], "want": want})
            w.extend((rid, at + i) for i in want)
            live[rid] = at + n
            if live[rid] == len(toks):
                ended.append(rid)
        peak = max(peak, sum(-(-max(n, 1) // 64) * 64 for n in live.values()))
        if entries:
            steps.append({"step": len(steps), "entries": entries, "end": ended})
            where.append(w)
        for rid in ended:
            del live[rid]
    return steps, where, peak
