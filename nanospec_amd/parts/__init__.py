from . import attention, block, norm, rope, swiglu  # noqa: F401  (each registers its parts)
from .model import DecoderModel, wanted_tensors
from .needs import PagedNeed, StateNeed
from .registry import build, register, registered

__all__ = ["DecoderModel", "wanted_tensors", "PagedNeed", "StateNeed", "build", "register", "registered"]
