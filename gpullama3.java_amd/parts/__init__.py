from .base import RunInfo, build_part, register_part
from . import (norm, rotary, attention, delta, mingru, time_mix, retention, state_space, side_by_side, latent_attention, feed_forward,
               routed, block)   # registers the built-in kinds
from .model import DecoderModel, expected_tensors

__all__ = ["RunInfo", "build_part", "register_part", "DecoderModel", "expected_tensors"]
