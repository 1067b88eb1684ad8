"""of3pair: MI355X-native kernels for the OpenFold3 Pairformer pair stack (triangle
multiplicative updates and triangle attention) behind the reference's layer-module API."""
from .layers import (TriangleAttention, TriangleAttentionEndingNode, TriangleAttentionStartingNode,
                     TriangleMultiplicationIncoming, TriangleMultiplicationOutgoing,
                     TriangleMultiplicativeUpdate)
from .pair_stack import PairStack

__all__ = [
    "TriangleMultiplicativeUpdate", "TriangleMultiplicationOutgoing", "TriangleMultiplicationIncoming",
    "TriangleAttention", "TriangleAttentionStartingNode", "TriangleAttentionEndingNode", "PairStack",
]
