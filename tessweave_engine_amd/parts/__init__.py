from .base import (Block, FeedForward, GroupStep, HeadHook, LayerRun, Mixer, Norm, Part, PositionEncoding,
                   StepContext, Workspace, fold_pending)
from .linear import Linear
from .norms import RMSNorm
from .positions import NoPositionEncoding, RotaryEmbedding
from .attention import GroupedQueryAttention
from .feedforward import SwiGLU
from .blocks import PreNormBlock
from .embedding import OutputHead, TokenEmbedding
from .model import DecoderModel, walk

__all__ = ["Block", "FeedForward", "GroupStep", "HeadHook", "LayerRun", "Mixer", "Norm", "Part", "PositionEncoding",
           "StepContext", "Workspace", "fold_pending", "Linear", "RMSNorm", "NoPositionEncoding", "RotaryEmbedding",
           "GroupedQueryAttention", "SwiGLU", "PreNormBlock", "OutputHead", "TokenEmbedding",
           "DecoderModel", "walk"]
