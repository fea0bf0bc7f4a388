from .registry import architectures, load_config, register_architecture, resolve
from .llama import LlamaConfig  # (importing an architecture's module registers it)
from .spec import (AttentionSpec, LayerCall, ModelSpec, NoPositionSpec, PreNormBlockSpec, RMSNormSpec, RopeSpec,
                   SwiGLUSpec)

__all__ = [
    "LlamaConfig", "architectures", "load_config", "register_architecture", "resolve", "AttentionSpec", "LayerCall",
    "ModelSpec", "NoPositionSpec", "PreNormBlockSpec", "RMSNormSpec", "RopeSpec", "SwiGLUSpec",
]
