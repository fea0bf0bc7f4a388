"""One registry from an architecture's name (config.json ``architectures[0]``) to its model.

An entry is a function ``(config.json dict, generation_config.json dict or None) -> (typed
configuration, ModelSpec)``.  Everything downstream (weights, parts, cache, engine) works from the
``ModelSpec`` alone, so another architecture is one typed configuration, its ``model_spec()`` and
one ``register_architecture`` call, made by the architecture's own module when it is imported (``config/llama.py``
does so; nothing here names an architecture).
"""

from __future__ import annotations

import json
from pathlib import Path
from typing import Callable

from .spec import ModelSpec  # noqa: F401  (what an entry returns)

_ARCHITECTURES: dict[str, Callable] = {}
_MODEL_TYPES: dict[str, str] = {}  # config.json model_type -> architecture, for files without `architectures`


def register_architecture(name: str, build: Callable, model_type: str | None = None) -> None:
    _ARCHITECTURES[name] = build
    if model_type is not None:
        _MODEL_TYPES[model_type] = name


def architectures() -> list[str]:
    return sorted(_ARCHITECTURES)


def resolve(cfg: dict, generation_cfg: dict | None = None):
    """config.json -> (typed configuration, ModelSpec) of the architecture it names."""
    names = cfg.get("architectures") or []
    name = names[0] if names else _MODEL_TYPES.get(cfg.get("model_type"))
    if name not in _ARCHITECTURES:
        raise ValueError(
            f"unknown architecture {name!r} (architectures={names!r}, model_type={cfg.get('model_type')!r}); "
            f"registered: {architectures()}"
        )
    return _ARCHITECTURES[name](cfg, generation_cfg)


def load_config(folder):
    """A model folder's config.json (+ generation_config.json if present) -> (configuration, ModelSpec).
    Reference: model/loader.py:33-38."""
    folder = Path(folder)
    path = folder / "config.json"
    if not path.is_file():
        raise FileNotFoundError(f"{folder} holds no config.json")
    cfg = json.loads(path.read_text())
    gen_path = folder / "generation_config.json"
    gen = json.loads(gen_path.read_text()) if gen_path.is_file() else None
    return resolve(cfg, gen)
