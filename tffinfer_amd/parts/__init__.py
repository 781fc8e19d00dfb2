"""Parts layers are put together from; importing the package registers the
built-in ones."""
from .base import (BLOCKS, FEED_FORWARDS, MIXERS, NORMS, POSITION_ENCODINGS, Block, FeedForward,
                   KVCacheSpec, Mixer, Norm, Part, PositionEncoding, StateSpec, WeightSpec,
                   register_block, register_feed_forward, register_mixer, register_norm,
                   register_position_encoding)
from . import attention, block, embedding, gated_delta, latent_attention, mixed_attention, mlp, norm, position, wkv  # noqa: F401  (registration)
from .attention import DifferentialAttention, GatedGQAttention, GQAttention
from .block import OutputNormBlock, ParallelBlock, PostNormBlock, PreNormBlock
from .gated_delta import GatedDeltaMixer, MixerPair
from .latent_attention import LatentAttention
from .embedding import Embedding, OutputHead
from .mlp import GeluMLP, NoFeedForward, RoutedExperts, SwiGLU, TableExperts
from .mixed_attention import MixedHeadAttention
from .norm import DynamicTanh, GroupRMSNorm, RMSNorm
from .wkv import WKVMixer
from .position import NoPosition, RotaryEmbedding, ScaledRotaryEmbedding
