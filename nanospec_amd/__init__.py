"""nanospec_amd: a small inference engine for AMD MI355X (gfx950), written for it from the start.

    from nanospec_amd import load_model, Engine, EngineConfig, SamplingParams
    model = load_model("/path/to/model_folder", dtype="bfloat16")
    engine = Engine(model, EngineConfig(num_blocks=4096))
    outputs = engine.generate([[1, 2, 3]], SamplingParams(max_tokens=16))
"""

from .config import LlamaConfig, load_config, register_architecture
from .sampling import SamplingParams, TokenInfo

__all__ = ["LlamaConfig", "load_config", "register_architecture", "SamplingParams", "TokenInfo", "load_model", "random_model",
           "Engine", "EngineConfig", "generate"]


def __getattr__(name):
    # the GPU-side modules load torch and the kernel bindings; they are imported on first use
    if name in ("load_model", "random_model"):
        from . import loader

        return getattr(loader, name)
    if name in ("Engine", "EngineConfig"):
        from . import engine

        return getattr(engine, name)
    if name == "generate":
        from .api import generate

        return generate
    raise AttributeError(name)
