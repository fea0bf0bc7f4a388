from .random_init import random_tensors, write_model_folder
from .source import DictSource, SafetensorsSource, WeightError, check

__all__ = ["DictSource", "SafetensorsSource", "WeightError", "check", "random_tensors", "write_model_folder"]
