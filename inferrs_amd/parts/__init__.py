from .base import (BlockBase, Embedding, FeedForward, FixedState, Head, Mixer, Norm, PagedKV, Part, Position,
                   block_class, part_class, register_block, register_embedding, register_ffn, register_head,
                   register_mixer, register_norm, register_position)
from . import norm, position, mlp, attention, io, block   # registers the built-in parts
from .assemble import generated_tensors, layer_tensors, model_tensors
from .block import Block
from .linear import Linear
