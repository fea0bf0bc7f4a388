"""Rotary position encoding: the inverse frequencies, with the llama3 scaling of long wavelengths.

Only the frequencies and the form of the rotation live here (which elements make a pair, a factor on cosine and
sine); the rotation itself is fused into the kernels that write keys and values to the cache (``kernels.ops.rope_kv_write``
and the q/k/v products' epilogues, all through the one device function of ``csrc/rope.h``), which form
angle = position * inv_freq and its cosine and sine in 32-bit.  Reference: model/llama.py:98-118 (frequencies),
:133-136 (angles), :150-158 (pairing of element j with j + d/2).

A position encoding of another kind that the attention part can apply is an object with ``inv_freq`` (float32 on the
device, rotary_dim / 2 values), ``rotary_dim``, ``max_positions`` and optionally ``interleaved`` and ``factor``.
"""

from __future__ import annotations

import math

import torch

from .registry import register


def inverse_frequencies(rotary_dim: int, theta: float, scaling) -> torch.Tensor:
    """float32 [rotary_dim / 2], computed on the CPU as the reference does (model/llama.py:100-102)."""
    exponent = torch.arange(0, rotary_dim, 2, dtype=torch.int64, device="cpu").to(torch.float32) / rotary_dim
    inv = 1.0 / (theta ** exponent)
    if scaling is None:
        return inv
    factor, low, high, original = scaling
    wavelen = 2 * math.pi / inv
    long_wave, short_wave = original / low, original / high
    scaled = torch.where(wavelen > long_wave, inv / factor, inv)
    t = (original / wavelen - low) / (high - low)
    between = (wavelen >= short_wave) & (wavelen <= long_wave)
    return torch.where(between, (1 - t) * scaled / factor + t * scaled, scaled)


class Rope:
    graph_safe = True

    def __init__(self, spec, prefix: str = "") -> None:
        if spec.rotary_dim % 2:
            raise ValueError(f"rotary_dim={spec.rotary_dim} must be even")
        self.spec = spec
        self.rotary_dim = spec.rotary_dim
        self.max_positions = spec.max_positions
        self.interleaved, self.factor = bool(spec.interleaved), float(spec.cos_sin_factor)
        self.inv_freq: torch.Tensor | None = None

    def wanted(self) -> dict:
        return {}

    def load(self, get, dtype, device) -> None:
        self.inv_freq = inverse_frequencies(self.spec.rotary_dim, self.spec.theta, self.spec.scaling).to(device)


class NoPosition:
    """Keys and queries are left as they are."""

    graph_safe = True
    rotary_dim = 0
    max_positions = None
    interleaved, factor = False, 1.0

    def __init__(self, spec, prefix: str = "") -> None:
        self.inv_freq = None

    def wanted(self) -> dict:
        return {}

    def load(self, get, dtype, device) -> None:
        self.inv_freq = torch.zeros(1, dtype=torch.float32, device=device)


register("position", "rope", Rope)
register("position", "none", NoPosition)
