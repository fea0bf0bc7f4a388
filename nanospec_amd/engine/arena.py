"""A bump allocator for the intermediates of one step.

Every buffer a part needs between kernels comes from here, so a step allocates nothing from the
framework's general allocator once the arena has grown to its working size, and a captured graph
owns an arena of fixed size whose addresses never change.  ``mark``/``release`` let a layer hand its
buffers back for the next layer.
"""

from __future__ import annotations

import math

import torch

_ALIGN = 256
_ESIZE: dict = {}  # bytes per element of the types asked for so far


class Arena:
    def __init__(self, device, nbytes: int = 0, fixed: bool = False) -> None:
        self.device, self.fixed = device, fixed
        self._chunks: list[torch.Tensor] = []
        self._typed: dict = {}  # (chunk, dtype) -> the chunk seen as that type
        self._cur, self._off = -1, 0
        self.high_water = 0  # the most bytes that were in use at once since the arena was made (tails of chunks that a buffer
        #                      did not fit into count as used: one chunk of this size holds the same sequence of buffers)
        if nbytes:
            self._chunks.append(torch.empty(nbytes, dtype=torch.uint8, device=device))
            self._cur = 0

    def take(self, shape, dtype) -> torch.Tensor:
        shape = tuple(int(s) for s in shape)
        esize = _ESIZE.get(dtype) or _ESIZE.setdefault(dtype, torch.empty(0, dtype=dtype).element_size())
        count = math.prod(shape)
        nbytes = max(1, count) * esize
        need = -(-nbytes // _ALIGN) * _ALIGN
        while self._cur < 0 or self._off + need > self._chunks[self._cur].numel():
            if self._cur + 1 < len(self._chunks):
                self._cur, self._off = self._cur + 1, 0
                continue
            if self.fixed:
                raise RuntimeError(f"a fixed arena of {sum(c.numel() for c in self._chunks)} bytes is exhausted")
            size = max(need, 2 * sum(c.numel() for c in self._chunks), 1 << 20)
            self._chunks.append(torch.empty(size, dtype=torch.uint8, device=self.device))
            self._cur, self._off = len(self._chunks) - 1, 0
        # a view of the chunk in the wanted type is kept, so a buffer costs one slice and one reshape (offsets are
        # multiples of 256 bytes, hence of every element size)
        typed = self._typed.get((self._cur, dtype))
        if typed is None:
            chunk = self._chunks[self._cur]
            typed = self._typed[self._cur, dtype] = chunk[: chunk.numel() // esize * esize].view(dtype)
        first = self._off // esize
        out = typed[first : first + count].view(shape)
        self._off += need
        used = self._off + sum(c.numel() for c in self._chunks[: self._cur])
        if used > self.high_water:
            self.high_water = used
        return out

    @property
    def capacity(self) -> int:
        return sum(c.numel() for c in self._chunks)

    def mark(self) -> tuple[int, int]:
        return self._cur, self._off

    def release(self, mark: tuple[int, int]) -> None:
        self._cur, self._off = mark

    def reset(self) -> None:
        """Start of a step.  Several chunks mean the arena grew during the last step: merge them."""
        if len(self._chunks) > 1 and not self.fixed:
            total = sum(c.numel() for c in self._chunks)
            self._chunks = [torch.empty(total, dtype=torch.uint8, device=self.device)]
            self._typed.clear()
        self._cur, self._off = (0, 0) if self._chunks else (-1, 0)
