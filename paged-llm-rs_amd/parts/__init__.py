from .registry import (BLOCKS, FEED_FORWARDS, MIXERS, NORMS, POSITIONS, register_block, register_embed_transform,
                       register_feed_forward, register_logit_transform, register_mixer, register_norm,
                       register_position)
from .linear import Linear
from .model import DecoderModel, LayerContext, build_model, declare_parameters, load_model

__all__ = ["BLOCKS", "FEED_FORWARDS", "MIXERS", "NORMS", "POSITIONS", "register_block", "register_feed_forward",
           "register_mixer", "register_norm", "register_position", "register_embed_transform",
           "register_logit_transform", "Linear", "DecoderModel", "LayerContext", "build_model",
           "declare_parameters", "load_model"]
