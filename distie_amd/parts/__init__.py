from . import (attention, block, conv_attention, embedding, feed_forward, latent_attention, linear_attention, norm,  # noqa: F401  (registration)
               parallel, position, recurrent, state_space)
from .attention import PagedKV
from .base import (PAGE, Block, Borrowed, CacheNeeds, Embedding, FeedForward, FixedState, Head, Mixer, Norm, PagedTensors, ParamSpec, Part,
                   PositionEncoding, ResidualStream, StepContext, TensorDecl, build_part, register_part)

__all__ = ["PAGE", "Block", "Borrowed", "CacheNeeds", "Embedding", "FeedForward", "FixedState", "Head", "Mixer", "Norm", "PagedKV", "PagedTensors",
           "ParamSpec", "Part", "PositionEncoding", "ResidualStream", "StepContext", "TensorDecl", "build_part",
           "register_part"]
