from .base import (Block, FeedForward, GroupStep, HeadHook, LayerRun, Mixer, Norm, Part, PositionEncoding,
                   StepContext, Workspace, fold_pending)
from .linear import JoinedLinear, Linear
from .norms import RMSNorm
from .positions import NoPositionEncoding, RotaryEmbedding
from .attention import GroupedQueryAttention
from .feedforward import GatedFeedForward, PlainFeedForward, ReluSquaredFeedForward, SwiGLU
from .blocks import DepthMixedBlock, ParallelBlock, PostNormBlock, PreNormBlock, ResultNormBlock
from .embedding import HashedPairEmbedding, OutputHead, PositionedEmbedding, TokenEmbedding
from .convolution import CausalConv
from .parallel import GatedLinearRecurrence, MixedHeadAttention, MixerBranch, ParallelMixer
from .side_input import SideTable, TokenSideInput
from .latent import LatentAttention
from .retention import Retention
from .delta import GatedDeltaRule
from .experts import RoutedExperts
from .mlstm import MatrixLSTM
from .windowed import ConvolvedWindowAttention
from .model import DecoderModel, walk

__all__ = ["Block", "FeedForward", "GroupStep", "HeadHook", "LayerRun", "Mixer", "Norm", "Part", "PositionEncoding",
           "StepContext", "Workspace", "fold_pending", "Linear", "RMSNorm", "NoPositionEncoding", "RotaryEmbedding",
           "GroupedQueryAttention", "SwiGLU", "PreNormBlock", "OutputHead", "TokenEmbedding",
           "JoinedLinear", "GatedFeedForward", "DepthMixedBlock", "PositionedEmbedding", "CausalConv",
           "GatedLinearRecurrence", "MixedHeadAttention", "MixerBranch", "ParallelMixer", "SideTable", "TokenSideInput",
           "HashedPairEmbedding", "LatentAttention", "PostNormBlock", "ReluSquaredFeedForward", "Retention",
           "GatedDeltaRule", "ParallelBlock", "RoutedExperts",
           "ConvolvedWindowAttention", "MatrixLSTM", "PlainFeedForward", "ResultNormBlock",
           "DecoderModel", "walk"]
