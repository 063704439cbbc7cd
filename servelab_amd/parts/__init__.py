from .base import (Block, Embedding, FeedForward, Mixer, Norm, PagedKVSpec, ParamSpec, Part,
                   PositionEncoding, RotaryLayout, RotaryTables, Runtime, StateSpec, prefixed)
from .norm import LayerNorm, NormedDelta, PostRMSNorm, RMSNorm
from .position import NoPosition, RotaryPosition
from .attention import PagedAttention, ProjectionNormAttention, ShortConvAttention
from .feedforward import GatedMLP, PlainMLP
from .routed import RoutedExperts
from .recurrent import GatedDeltaRule, GatedLinearAttention, MatrixLSTM, SideBySide, StateSpaceMixer
from .block import ParallelBlock, PostNormBlock, PreNormBlock, SandwichBlock, StreamReentry
from .embedding import OutputHead, TokenEmbedding
from .model import DecoderModel, LayerCall, ModelSpec, build_model_spec
