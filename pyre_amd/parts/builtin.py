"""Registers the parts that ship with the framework."""

from pyre_amd.parts.attention import Attention
from pyre_amd.parts.base import register_part
from pyre_amd.parts.block import ParallelBlock, PostNormBlock, PreNormBlock, SandwichBlock
from pyre_amd.parts.branch import ParallelMixer
from pyre_amd.parts.capped_attention import CappedAttention
from pyre_amd.parts.delta_rule import GatedDeltaRule
from pyre_amd.parts.embedding import BigramEmbedding, LMHead, TokenEmbedding
from pyre_amd.parts.feedforward import ClippedGLU, GeluGLU, ReluSquaredMLP, SwiGLU
from pyre_amd.parts.latent_attention import LatentAttention
from pyre_amd.parts.linear_attention import GatedLinearAttention, Retention
from pyre_amd.parts.moe import GroupedSoftmaxMoE, SigmoidMoE, SoftmaxTopKMoE
from pyre_amd.parts.norm import LayerNorm, RMSNorm, TanhNorm
from pyre_amd.parts.rotary import NoPosition, RotaryEncoding
from pyre_amd.parts.sink_attention import SinkAttention
from pyre_amd.parts.tied_attention import TiedAttention
from pyre_amd.parts.token_side import TokenSide
from pyre_amd.parts.window_attention import WindowAttention

register_part("mixer", "attention", Attention)
register_part("feed_forward", "swiglu", SwiGLU)
register_part("norm", "rmsnorm", RMSNorm)
register_part("position", "rotary", RotaryEncoding)
register_part("position", "none", NoPosition)
register_part("block", "pre_norm", PreNormBlock)
register_part("embedding", "embedding", TokenEmbedding)
register_part("head", "lm_head", LMHead)
register_part("mixer", "capped_attention", CappedAttention)
register_part("mixer", "gated_linear_attention", GatedLinearAttention)
register_part("mixer", "parallel", ParallelMixer)
register_part("feed_forward", "clipped_glu", ClippedGLU)
register_part("norm", "layernorm", LayerNorm)
register_part("block", "sandwich", SandwichBlock)
register_part("mixer", "tied_attention", TiedAttention)
register_part("mixer", "latent_attention", LatentAttention)
register_part("feed_forward", "gelu_glu", GeluGLU)
register_part("feed_forward", "sigmoid_moe", SigmoidMoE)
register_part("norm", "tanh_norm", TanhNorm)
register_part("block", "parallel_block", ParallelBlock)
register_part("embedding", "bigram_embedding", BigramEmbedding)
register_part("block", "post_norm", PostNormBlock)
register_part("mixer", "sink_attention", SinkAttention)
register_part("mixer", "retention", Retention)
register_part("feed_forward", "relu2_mlp", ReluSquaredMLP)
register_part("feed_forward", "grouped_softmax_moe", GroupedSoftmaxMoE)
register_part("mixer", "window_attention", WindowAttention)
register_part("mixer", "gated_delta_rule", GatedDeltaRule)
register_part("feed_forward", "softmax_topk_moe", SoftmaxTopKMoE)
register_part("token_input", "token_side", TokenSide)
