from .params import SamplingParams, TokenInfo

__all__ = ["SamplingParams", "TokenInfo"]
