from .registry import (BLOCKS, FEED_FORWARDS, MIXERS, NORMS, register_block, register_feed_forward,
                       register_mixer, register_norm)
from .linear import Linear
from .model import DecoderModel, LayerContext, build_model, declare_parameters, load_model

__all__ = ["BLOCKS", "FEED_FORWARDS", "MIXERS", "NORMS", "register_block", "register_feed_forward",
           "register_mixer", "register_norm", "Linear", "DecoderModel", "LayerContext", "build_model",
           "declare_parameters", "load_model"]
