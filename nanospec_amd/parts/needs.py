"""What a mixer asks of the cache manager."""

from __future__ import annotations

from dataclasses import dataclass

import torch


@dataclass(frozen=True)
class PagedNeed:
    """Keys and values per token, in pages.  Mixers with equal needs share a group of pages."""

    kv_heads: int
    head_dim: int
    window: int = 0  # 0 = every earlier token stays

    @property
    def group_name(self) -> str:
        return f"kv{self.kv_heads}x{self.head_dim}" + (f"w{self.window}" if self.window else "")


@dataclass(frozen=True)
class StateNeed:
    """State of fixed size per request, kept in the request's slot; zeroed when a request is admitted."""

    shape: tuple[int, ...]
    dtype: torch.dtype = torch.float32
