from .base import (FeedForward, FixedState, Mixer, Norm, PagedKV, Part, Position, part_class,
                   register_ffn, register_mixer, register_norm, register_position)
from . import norm, position, mlp, attention   # registers the built-in parts
from .assemble import generated_tensors, layer_tensors, model_tensors
from .block import Block
from .linear import Linear
