from .base import CacheBinding, Runtime, TensorInfo
from .registry import build_part, part_class, register_part, unregister_part
from . import norm, rope, attention, mlp, block  # registers the built-in parts
from .model import DecoderModel, cache_plan, expected_tensors
