from .base import RunInfo, build_part, register_part
from . import norm, rotary, attention, feed_forward, block   # registers the built-in kinds
from .model import DecoderModel, expected_tensors

__all__ = ["RunInfo", "build_part", "register_part", "DecoderModel", "expected_tensors"]
