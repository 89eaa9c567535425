"""MI355X-native Pairformer pair stack: drop-in modules for Protenix's
TriangleMultiplication*, TriangleAttention, LayerNorm, Transition,
AttentionPairBias, PairformerBlock and PairformerStack, backed by hand-written
gfx950 kernels in libprotenix_amd.so (C ABI: include/protenix_amd.h)."""

from .graph import Graphed
from .layer_norm import FusedLayerNorm, LayerNorm
from .pairformer import PairformerBlock, PairformerStack
from .primitives import Linear, LinearNoBias, Transition
from .transformer import AttentionPairBias
from .tri_attention import TriAttentionFunction, tri_attention, tri_attention_forward
from .triangular import (
    TriangleAttention,
    TriangleAttentionEndingNode,
    TriangleAttentionStartingNode,
    TriangleMultiplicationIncoming,
    TriangleMultiplicationOutgoing,
    TriangleMultiplicativeUpdate,
    kernel_triangular_mult,
    triangle_multiplicative_update,
)

__all__ = [
    "Graphed",
    "AttentionPairBias", "FusedLayerNorm", "LayerNorm", "Linear", "LinearNoBias",
    "PairformerBlock", "PairformerStack", "Transition", "TriangleAttention",
    "TriangleAttentionEndingNode", "TriangleAttentionStartingNode",
    "TriangleMultiplicationIncoming", "TriangleMultiplicationOutgoing",
    "TriangleMultiplicativeUpdate", "kernel_triangular_mult", "triangle_multiplicative_update",
    "TriAttentionFunction", "tri_attention", "tri_attention_forward",
]
