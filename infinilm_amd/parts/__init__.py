from . import attention, block, ends, mlp, norm, rotary  # noqa: F401  (register the built-in kinds)
from .base import (BuildContext, FeedForward, Mixer, Norm, Param, Part, PositionEncoding, ResidualStream)
from .block import build_block
from .ends import Embedding, OutputHead
from .registry import (register_arrangement, register_embedding, register_feed_forward, register_head, register_mixer,
                       register_norm, register_position_encoding)
from .rotary import register_rope_scaling

__all__ = ["BuildContext", "Embedding", "OutputHead", "register_embedding", "register_head", "FeedForward", "Mixer", "Norm", "Param", "Part", "PositionEncoding", "ResidualStream",
           "build_block", "register_arrangement", "register_feed_forward", "register_mixer", "register_norm",
           "register_position_encoding", "register_rope_scaling"]
