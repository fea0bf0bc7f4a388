"""The one-call Python entry point."""

from __future__ import annotations

from .sampling import SamplingParams


def generate(model, prompts: list[list[int]], params: SamplingParams | list[SamplingParams] = SamplingParams(), dtype="bfloat16",
             num_blocks: int | None = None, block_size: int = 16, **engine_options) -> list[list[int]]:
    """Token ids in, token ids out.  ``model`` is a model folder or a loaded model.  The cache pool is
    sized for all requests at their longest unless ``num_blocks`` is given."""
    from .engine import Engine, EngineConfig
    from .loader import load_model

    if isinstance(model, (str, bytes)) or hasattr(model, "__fspath__"):
        model = load_model(model, dtype=dtype)
    per = params if isinstance(params, (list, tuple)) else [params] * len(prompts)
    if num_blocks is None:
        num_blocks = sum(-(-(len(p) + s.max_tokens) // block_size) for p, s in zip(prompts, per)) + 1
    engine = Engine(model, EngineConfig(num_blocks=num_blocks, block_size=block_size, **engine_options))
    return engine.generate(prompts, list(per))
