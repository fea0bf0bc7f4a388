"""Seeded random weights for any model spec, and a writer of whole model folders.

The law: linear matrices and embedding tables are N(0, 0.02); norm weights are 1 + N(0, 0.02).
Tensors are drawn in the sorted order of their names from one ``torch.Generator`` seeded with
``seed``, in 32-bit, then cast, so that a folder written here and the tensors made in memory from
the same (spec, seed) are identical.
"""

from __future__ import annotations

import json
from pathlib import Path

import torch

STD = 0.02


def random_tensors(wanted: dict[str, tuple[tuple[int, ...], str]], seed: int, dtype=torch.float32, device="cpu",
                   skip: set[str] = frozenset()) -> dict[str, torch.Tensor]:
    """``wanted``: name -> (shape, role), role in {"linear", "embedding", "norm"}; see
    ``parts.model.wanted_tensors``.  On the CPU the draw is reproducible across machines; with
    another ``device`` the same law is drawn there (large models for measurement)."""
    gen = torch.Generator(device=device)
    gen.manual_seed(seed)
    out = {}
    for name in sorted(wanted):
        if name in skip:
            continue
        shape, role = wanted[name]
        t = torch.empty(shape, dtype=torch.float32 if device == "cpu" else dtype, device=device)
        t.normal_(0.0, STD, generator=gen)
        if role == "norm":
            t += 1.0
        out[name] = t.to(dtype)
    return out


def write_model_folder(folder, config, seed: int, dtype=torch.float32) -> Path:
    """config.json + model.safetensors of a randomly initialised model.  ``config`` is a typed
    configuration with ``to_hf()`` and ``model_spec()``.  A tied head is left out of the file, as
    checkpoints with tied embeddings do."""
    from safetensors.torch import save_file

    from ..parts.model import wanted_tensors

    folder = Path(folder)
    folder.mkdir(parents=True, exist_ok=True)
    spec = config.model_spec()
    wanted = wanted_tensors(spec)
    skip = {spec.head_name} if spec.tie_head else set()
    tensors = random_tensors(wanted, seed, dtype, skip=skip)
    (folder / "config.json").write_text(json.dumps(config.to_hf(), indent=1))
    save_file({k: v.contiguous() for k, v in tensors.items()}, str(folder / "model.safetensors"))
    return folder
