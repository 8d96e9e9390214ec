"""Parts a model is assembled from, and their registration under kind names."""
from .. import registry
from .attention import Attention
from .base import (Block, FeedForward, Gated, KVNeed, Mixer, Norm, Part, PartSpec, PositionEncoding, StateNeed,
                   TensorSpec)
from .block import PreNormBlock
from .channel_delta import ChannelDelta
from .clamped_glu import ClampedGLU
from .dense_xielu import DenseXielu
from .embedding import Embedding, LMHead
from .gated_residual import GatedPreNormBlock, GatedPreNormMixerBlock, ResidualGate
from .gelu_glu import GeluGLU
from .gla import GatedLinearAttention
from .hgrn2 import HGRN2
from .latent_attention import LatentAttention
from .lightning import LightningAttention
from .mixer_pair import MixerPair
from .norm_layer import LayerNorm
from .norm_rms import RMSNorm
from .parallel import (CausalConvInput, LayerScale, ParallelBlock, ParallelMixerBlock, ScaledParallelBlock,
                       ScaledParallelMixerBlock, TokenSide)
from .rope import RotaryEncoding
from .routed_experts import GroupedRoutedExperts, RoutedExperts
from .sink_attention import SinkAttention
from .streams import HyperBlock, HyperConnection, HyperMixerBlock
from .swiglu import SwiGLU

registry.register_part("mixer", "attention", Attention)
registry.register_part("feed_forward", "swiglu", SwiGLU)
registry.register_part("norm", "rmsnorm", RMSNorm)
registry.register_part("position", "rope", RotaryEncoding)
registry.register_part("block", "pre_norm", PreNormBlock)
registry.register_part("embedding", "table", Embedding)
registry.register_part("head", "linear", LMHead)
registry.register_part("mixer", "latent_attention", LatentAttention)
registry.register_part("mixer", "hgrn2", HGRN2)
registry.register_part("mixer", "channel_delta", ChannelDelta)
registry.register_part("feed_forward", "dense_xielu", DenseXielu)
registry.register_part("norm", "layernorm", LayerNorm)
registry.register_part("connection", "hyper", HyperConnection)
registry.register_part("block", "hyper", HyperBlock)
registry.register_part("block", "hyper_mixer_only", HyperMixerBlock)
registry.register_part("mixer", "gla", GatedLinearAttention)
registry.register_part("mixer", "sink_attention", SinkAttention)
registry.register_part("feed_forward", "clamped_glu", ClampedGLU)
registry.register_part("feed_forward", "routed_experts", RoutedExperts)
registry.register_part("connection", "causal_conv", CausalConvInput)
registry.register_part("connection", "token_side", TokenSide)
registry.register_part("block", "parallel", ParallelBlock)
registry.register_part("block", "parallel_mixer_only", ParallelMixerBlock)
registry.register_part("mixer", "lightning_attention", LightningAttention)
registry.register_part("mixer", "mixer_pair", MixerPair)
registry.register_part("feed_forward", "grouped_experts", GroupedRoutedExperts)
registry.register_part("connection", "layer_scale", LayerScale)
registry.register_part("block", "parallel_scaled", ScaledParallelBlock)
registry.register_part("block", "parallel_scaled_mixer_only", ScaledParallelMixerBlock)
registry.register_part("connection", "residual_gate", ResidualGate)
registry.register_part("block", "pre_norm_gated", GatedPreNormBlock)
registry.register_part("block", "pre_norm_gated_mixer_only", GatedPreNormMixerBlock)
registry.register_part("feed_forward", "gelu_glu", GeluGLU)
