"""Where tensors come from: a folder of safetensors files, or a dictionary in memory.

A source answers ``names()``, ``shape(name)`` and ``get(name)`` so that a model can be checked
against the header alone (names and shapes) before a single byte of data is read, and so that
each tensor is materialised once, straight where its part wants it.

Stored precisions are kept: bfloat16 stays bfloat16, a tensor stored in 32-bit stays 32-bit,
16-bit IEEE halves become bfloat16's neighbour only when a part asks for another dtype, integer
tables come out as int32.  Reference for the file handling: model/loader.py:56-60 (every
``*.safetensors`` of the folder in sorted order, the index json is not consulted).
"""

from __future__ import annotations

from pathlib import Path

import torch


class WeightError(Exception):
    """Raised once per load with everything that is wrong: missing and unexpected tensor names
    and tensors of the wrong shape."""

    def __init__(self, where: str, missing=(), unexpected=(), wrong_shape=()) -> None:
        self.missing, self.unexpected, self.wrong_shape = list(missing), list(unexpected), list(wrong_shape)
        lines = [f"weights of {where} do not fit the model:"]
        if self.missing:
            lines.append(f"  missing tensors ({len(self.missing)}): " + ", ".join(self.missing))
        if self.unexpected:
            lines.append(f"  unexpected tensors ({len(self.unexpected)}): " + ", ".join(self.unexpected))
        for name, have, want in self.wrong_shape:
            lines.append(f"  wrong shape: {name} is {list(have)}, the model wants {list(want)}")
        super().__init__("\n".join(lines))


def _normalise(t: torch.Tensor) -> torch.Tensor:
    if t.dtype in (torch.int64, torch.int16, torch.int8, torch.uint8, torch.bool):
        return t.to(torch.int32)
    if t.dtype == torch.float64:
        return t.to(torch.float32)
    return t


class DictSource:
    def __init__(self, tensors: dict[str, torch.Tensor], where: str = "<memory>") -> None:
        self._t, self.where = tensors, where

    def names(self) -> list[str]:
        return list(self._t)

    def shape(self, name: str) -> tuple[int, ...]:
        return tuple(self._t[name].shape)

    def get(self, name: str) -> torch.Tensor:
        return _normalise(self._t[name])


class SafetensorsSource:
    """Every ``*.safetensors`` file of a folder; tensors are read lazily, memory-mapped."""

    def __init__(self, folder) -> None:
        from safetensors import safe_open

        self.where = str(folder)
        files = sorted(Path(folder).glob("*.safetensors"))
        if not files:
            raise FileNotFoundError(f"{folder} holds no *.safetensors file")
        self._files = [safe_open(str(f), framework="pt", device="cpu") for f in files]
        self._of: dict[str, object] = {}
        for f in self._files:
            for name in f.keys():
                self._of[name] = f

    def names(self) -> list[str]:
        return list(self._of)

    def shape(self, name: str) -> tuple[int, ...]:
        return tuple(self._of[name].get_slice(name).get_shape())

    def get(self, name: str) -> torch.Tensor:
        return _normalise(self._of[name].get_tensor(name))


def check(source, wanted: dict[str, tuple[int, ...]], optional: set[str] = frozenset()) -> None:
    """Compare a source's header with the tensors a model wants; raise one WeightError that lists
    everything wrong.  ``optional`` names may be absent (a tied output head)."""
    have = set(source.names())
    missing = sorted(n for n in wanted if n not in have and n not in optional)
    unexpected = sorted(have - set(wanted))
    wrong = [(n, source.shape(n), wanted[n]) for n in sorted(have & set(wanted)) if tuple(source.shape(n)) != tuple(wanted[n])]
    if missing or unexpected or wrong:
        raise WeightError(source.where, missing, unexpected, wrong)
