"""Which class implements which kind of part.

A role ("norm", "position", "mixer", "ffn", "block") and a spec's ``kind`` name a class.  A new part is
registered once with ``register(role, kind, cls)``, from anywhere (a test registers toy parts), and is
then built wherever a spec of that kind appears in a ``ModelSpec``.

What each role must offer (``ctx`` is the engine's ``StepContext``, tensors are [tokens, width]):

  every part   __init__(spec, prefix)             prefix: tensor-name prefix of its weights
               wanted() -> {name: (shape, role)}   tensors it reads from the checkpoint; role says how random weights
                                                  are drawn: "linear" | "embedding" | "norm" | "zeros" | "ones", or a
                                                  function (shape, generator) -> tensor (weights/random_init.py)
               load(get, dtype, device)           get(name) returns the stored tensor (CPU)
               graph_safe: bool                   True if forward only launches kernels on the current
                                                  stream into buffers taken from ctx.arena
  norm         forward(ctx, resid=None, x=None, rows=None, write_resid=False, out=None)
                                                  normalise resid + x (the sum optionally stored back)
  position     an object the mixer that owns it knows how to use (rope: ``inv_freq`` on the device, ``rotary_dim``,
               ``max_positions``: an int or None)
  mixer        cache_need() -> PagedNeed | StateNeed | None
               forward(ctx, x, cache, owns_cache, out=None) -> [tokens, hidden]
  ffn          forward(ctx, x, out=None) -> [tokens, hidden]
  block        __init__(spec, None): the spec carries the layer's tensor-name prefix and its parts' names
               cache_need(); forward(ctx, resid, delta, cache, owns_cache, delta_out) -> None
                                                  resid is updated in place; the not yet added output of
                                                  the block's last part is left in delta_out

Rows of a step may be padding (captured steps have fixed shapes): their inputs are arbitrary bits, NaNs included, and their
outputs are never read.  A part keeps rows independent of each other (as every product, norm and per-token mixer does), or
tells padding rows on the device by ``ctx.state_slots[ctx.token_req[row]] == ctx.pad_slot`` (``pad_slot`` is None in steps
without padding).

Optional:
  mixer, block max_positions() -> int | None      the positions it can encode (the engine refuses requests beyond the
                                                  smallest limit of a model's layers)
  any part     takes_layouts = True: load(get, dtype, device, layouts) with layouts "both" | "tiled"
                                                  (which copies of a bfloat16 matrix to keep, ``parts.linear.LAYOUTS``)

Optional, for parts whose products can do the work of the RMS norms around them (``parts.linear.IntoResidual``):
  norm         links_products = True, weight, spec.eps
  mixer, ffn   ends_in_residual = True: forward(..., residual=IntoResidual) -> PreNormed | PartialSums | Added | tensor;
               links_norms(rows) -> bool: x may be a PreNormed
  block        links_blocks = True; entry_norm (the norm that reads the block's input);
               forward(..., next_norm=None, next_sums=None, next_carry=None) -> None or one of those three
"""

from __future__ import annotations

_PARTS: dict[tuple[str, str], type] = {}
ROLES = ("norm", "position", "mixer", "ffn", "block")


def register(role: str, kind: str, cls: type) -> None:
    if role not in ROLES:
        raise ValueError(f"unknown role {role!r}; roles are {ROLES}")
    _PARTS[(role, kind)] = cls


def build(role: str, spec, prefix: str):
    kind = getattr(spec, "kind", None)
    if (role, kind) not in _PARTS:
        known = sorted(k for r, k in _PARTS if r == role)
        raise ValueError(f"no {role} of kind {kind!r} is registered (known: {known})")
    return _PARTS[(role, kind)](spec, prefix)


def registered(role: str) -> list[str]:
    return sorted(k for r, k in _PARTS if r == role)
