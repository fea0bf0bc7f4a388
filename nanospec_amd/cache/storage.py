"""The memory behind the cache manager: pages of keys and values per group of layers, and state slots.

A run-order entry of the model with a ``PagedNeed`` gets one layer of its group's page tensors:
    K [entries, pages, kv_heads, page, head_dim]       (the reference keeps [pages, page, kv_heads, head_dim],
                                                        kv/cache.py:16-19; here a head's part of a page is contiguous)
    V [entries, pages, kv_heads, head_dim, page]       (transposed per page for the attention kernels)
Both start as zeros: slots that are masked out are still read (reference: kv/cache.py:18).  A page id
means the same page in every entry of its group.  An entry with a ``StateNeed`` gets a tensor
[slots, *shape]; an entry that reads another entry's cache gets that entry's view.
"""

from __future__ import annotations

from dataclasses import dataclass

import torch

from ..parts.needs import PagedNeed, StateNeed
from .manager import GroupSpec


@dataclass
class PagedView:
    group: int
    k: torch.Tensor
    v: torch.Tensor


@dataclass
class StateView:
    state: torch.Tensor  # [slots, *shape]


def plan_groups(cache_needs: list) -> tuple[list[GroupSpec], list[PagedNeed], list[int | None]]:
    """Run-order entries with equal paged needs share a group.  -> (group specs for the manager, the need
    of each group, group index of each entry or None)."""
    needs: list[PagedNeed] = []
    of_entry: list[int | None] = []
    for need in cache_needs:
        if isinstance(need, PagedNeed):
            if need not in needs:
                needs.append(need)
            of_entry.append(needs.index(need))
        else:
            of_entry.append(None)
    specs = [GroupSpec(n.group_name, n.window) for n in needs]
    return specs, needs, of_entry


class CacheStorage:
    def __init__(self, model, num_pages: list[int], page_size: int, num_slots: int, dtype, device) -> None:
        self.group_specs, needs, of_entry = plan_groups(model.cache_needs)
        self.page_size = page_size
        counts = [sum(1 for g in of_entry if g == i) for i in range(len(needs))]
        self.k = [torch.zeros((counts[i], num_pages[i], n.kv_heads, page_size, n.head_dim), dtype=dtype, device=device)
                  for i, n in enumerate(needs)]
        self.v = [torch.zeros((counts[i], num_pages[i], n.kv_heads, n.head_dim, page_size), dtype=dtype, device=device)
                  for i, n in enumerate(needs)]
        self.states: list[torch.Tensor] = []
        self.views: list = []
        taken = [0] * len(needs)
        for i, (need, call) in enumerate(zip(model.cache_needs, model.spec.run_order)):
            if call.cache_from is not None:
                self.views.append(self.views[call.cache_from])
            elif isinstance(need, PagedNeed):
                g = of_entry[i]
                self.views.append(PagedView(g, self.k[g][taken[g]], self.v[g][taken[g]]))
                taken[g] += 1
            elif isinstance(need, StateNeed):
                t = torch.zeros((num_slots, *need.shape), dtype=need.dtype, device=device)
                self.states.append(t)
                self.views.append(StateView(t))
            else:
                self.views.append(None)

    def reset_slot(self, slot: int) -> None:
        """A newly admitted request starts from zero state."""
        for t in self.states:
            t[slot].zero_()

    def bytes_per_token(self) -> int:
        return sum(k[:, 0, :, 0].numel() * 2 * k.element_size() for k in self.k)
