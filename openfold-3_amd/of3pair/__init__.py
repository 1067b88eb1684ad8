"""of3pair: MI355X-native kernels for the OpenFold3 Pairformer pair stack (triangle
multiplicative updates, triangle attention and the pair transition) behind the reference's layer-module API."""
from .layers import (AttentionPairBias, FusedTriangleMultiplicationIncoming, FusedTriangleMultiplicationOutgoing,
                     FusedTriangleMultiplicativeUpdate, PairBiasProjection, SwiGLUTransition, TriangleAttention, TriangleAttentionEndingNode, TriangleAttentionStartingNode,
                     TriangleMultiplicationIncoming, TriangleMultiplicationOutgoing,
                     TriangleMultiplicativeUpdate)
from .pair_stack import PairBlock, PairStack
from .pairformer import PairFormerBlock, PairFormerStack
from .template import TemplateEmbedderCore, TemplatePairBlock, TemplatePairStack
from . import checkpoint

__all__ = [
    "TriangleMultiplicativeUpdate", "TriangleMultiplicationOutgoing", "TriangleMultiplicationIncoming",
    "FusedTriangleMultiplicativeUpdate", "FusedTriangleMultiplicationOutgoing", "FusedTriangleMultiplicationIncoming",
    "TriangleAttention", "TriangleAttentionStartingNode", "TriangleAttentionEndingNode", "SwiGLUTransition", "PairBiasProjection", "AttentionPairBias",
    "PairStack", "PairBlock", "PairFormerBlock", "PairFormerStack", "TemplatePairBlock", "TemplatePairStack", "TemplateEmbedderCore", "checkpoint",
]
