"""A model folder (config.json + *.safetensors) -> a model on the GPU, ready for the engine.

Reference: model/loader.py:41-83 (``load_model(model, device="cuda", dtype=torch.bfloat16)``).  The
architecture is chosen by config.json through the registry, never by the caller.
"""

from __future__ import annotations

from pathlib import Path

import torch

from .config import load_config
from .parts import DecoderModel
from .weights import DictSource, SafetensorsSource, random_tensors
from .weights.random_init import draw

_DTYPES = {"bfloat16": torch.bfloat16, "bf16": torch.bfloat16, "float32": torch.float32, "fp32": torch.float32, "f32": torch.float32}


def as_dtype(dtype) -> torch.dtype:
    if isinstance(dtype, torch.dtype):
        if dtype not in (torch.bfloat16, torch.float32):
            raise ValueError(f"the engine computes in bfloat16 or float32, not {dtype}")
        return dtype
    if dtype not in _DTYPES:
        raise ValueError(f"unknown dtype {dtype!r}; use 'bfloat16' or 'float32'")
    return _DTYPES[dtype]


def _require_gpu(device) -> torch.device:
    device = torch.device(device)
    if device.type != "cuda" or not torch.cuda.is_available():
        raise RuntimeError("nanospec_amd runs on an AMD GPU (torch device 'cuda') only; no GPU is visible")
    return device


def load_model(model, device="cuda", dtype=torch.bfloat16, layouts: str = "auto") -> DecoderModel:
    """``model``: a folder with config.json and safetensors files.  ``layouts``: see ``DecoderModel.load``."""
    folder = Path(model)
    if not folder.is_dir():
        raise FileNotFoundError(f"{model} is not a model folder (no network access is attempted)")
    config, spec = load_config(folder)
    device = _require_gpu(device)
    return DecoderModel(spec, config).load(SafetensorsSource(folder), as_dtype(dtype), device, layouts)


def random_model(config, seed: int = 0, device="cuda", dtype=torch.bfloat16, on_device: bool = False,
                 layouts: str = "auto") -> DecoderModel:
    """A model with seeded random weights, without a folder.  ``on_device`` draws the numbers on the GPU
    (large models; the numbers then differ from the CPU draw of the same seed, the law does not)."""
    device = _require_gpu(device)
    dtype = as_dtype(dtype)
    spec = config.model_spec()
    net = DecoderModel(spec, config)
    skip = {spec.head_name} if spec.tie_head else set()
    if not on_device:
        return net.load(DictSource(random_tensors(net.wanted(), seed, dtype, skip=skip), "<random>"), dtype, device, layouts)

    class _Lazy:
        """Draws each tensor on the device when it is asked for, so that no second copy is ever held."""

        where = "<random on device>"

        def __init__(self, wanted):
            self.wanted = {k: v for k, v in wanted.items() if k not in skip}
            self.gen = torch.Generator(device=device)
            self.gen.manual_seed(seed)

        def names(self):
            return list(self.wanted)

        def shape(self, name):
            return tuple(self.wanted[name][0])

        def get(self, name):
            shape, role = self.wanted[name]
            return draw(shape, role, self.gen, dtype, dtype)

    return net.load(_Lazy(net.wanted()), dtype, device, layouts)
