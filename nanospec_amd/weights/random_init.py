"""Seeded random weights for any model spec, and a writer of whole model folders.

The law of a tensor is what its part says in ``wanted()``: name -> (shape, role).  A role is a name in ``LAWS``
(linear matrices and embedding tables are N(0, 0.02); norm weights are 1 + N(0, 0.02); "zeros" and "ones" for
biases and gains that start neutral), or a function ``(shape, generator) -> float32 tensor`` on the generator's
device, for a part whose tensors want a law of their own (a decay, a convolution).
Tensors are drawn in the sorted order of their names from one ``torch.Generator`` seeded with
``seed``, in 32-bit, then cast, so that a folder written here and the tensors made in memory from
the same (spec, seed) are identical.
"""

from __future__ import annotations

import json
from pathlib import Path

import torch

STD = 0.02
LAWS = {"linear": (0.0, STD), "embedding": (0.0, STD), "norm": (1.0, STD), "zeros": (0.0, 0.0), "ones": (1.0, 0.0)}  # role -> (mean, std)


def draw(shape, role, gen: torch.Generator, dtype=torch.float32, draw_dtype=torch.float32) -> torch.Tensor:
    """One tensor of the given role's law, on the generator's device: drawn in ``draw_dtype``, returned in ``dtype``."""
    if callable(role):
        t = role(tuple(shape), gen)
        if tuple(t.shape) != tuple(shape):
            raise ValueError(f"an initial law returned shape {tuple(t.shape)} for a tensor of shape {tuple(shape)}")
        return t.to(dtype)
    if role not in LAWS:
        raise ValueError(f"unknown role {role!r} of a tensor; roles are {sorted(LAWS)} or a function (shape, generator) -> tensor")
    mean, std = LAWS[role]
    t = torch.empty(shape, dtype=draw_dtype, device=gen.device)
    if std:
        t.normal_(0.0, std, generator=gen)
        if mean:
            t += mean
    else:
        t.fill_(mean)
    return t.to(dtype)


def random_tensors(wanted: dict[str, tuple[tuple[int, ...], str]], seed: int, dtype=torch.float32, device="cpu",
                   skip: set[str] = frozenset()) -> dict[str, torch.Tensor]:
    """``wanted``: name -> (shape, role), see ``LAWS`` and ``parts.model.wanted_tensors``.  On the CPU the draw is reproducible across machines; with
    another ``device`` the same law is drawn there (large models for measurement)."""
    gen = torch.Generator(device=device)
    gen.manual_seed(seed)
    out = {}
    for name in sorted(wanted):
        if name in skip:
            continue
        shape, role = wanted[name]
        out[name] = draw(shape, role, gen, dtype, torch.float32 if device == "cpu" else dtype)
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
