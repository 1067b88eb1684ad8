"""The pair-stack half of the reference's PairBlock: sequencing of the four modules with
their residual adds, as in openfold3/core/model/latent/base_blocks.py:307-406, and the
per-template variant of template_module.py:148-166 (templates are independent pair
representations, so they are folded into the batch instead of looped over).

Unlike the reference, no physical transpose of z is made around the ending-node attention
(base_blocks.py:380-404): the kernels walk the transposed view through strides.  The
residual adds are fused into each module's output kernel.
"""
from __future__ import annotations

import torch
import torch.nn as nn

from . import functional as F3
from ._guard import forward_only
from .layers import (FusedTriangleMultiplicationIncoming, FusedTriangleMultiplicationOutgoing, SwiGLUTransition,
                     TriangleAttention, TriangleMultiplicationIncoming, TriangleMultiplicationOutgoing)


class PairStack(nn.Module):
    """tri_mul_out -> tri_mul_in -> tri_att_start -> tri_att_end, each followed by its
    residual add (dropout is the identity in eval mode, dropout.py:57-58).  Sub-module names
    match PairBlock's, so `pair_stack.<name>.<param>` checkpoint keys load unchanged.  The
    pair transition that follows in PairBlock.forward (base_blocks.py:470-478) is added by the
    PairBlock subclass below."""

    def __init__(self, c_z: int, c_hidden_mul: int, c_hidden_pair_att: int, no_heads_pair: int,
                 inf: float = 1e9, linear_init_params=None, fuse_projection_weights: bool = False):
        super().__init__()
        ta = None if linear_init_params is None else linear_init_params["tri_att"]
        if fuse_projection_weights:  # base_blocks.py:260-266
            tm = None if linear_init_params is None else linear_init_params["fused_tri_mul"]
            self.tri_mul_out = FusedTriangleMultiplicationOutgoing(c_z, c_hidden_mul, linear_init_params=tm)
            self.tri_mul_in = FusedTriangleMultiplicationIncoming(c_z, c_hidden_mul, linear_init_params=tm)
        else:
            tm = None if linear_init_params is None else linear_init_params["tri_mul"]
            self.tri_mul_out = TriangleMultiplicationOutgoing(c_z, c_hidden_mul, linear_init_params=tm)
            self.tri_mul_in = TriangleMultiplicationIncoming(c_z, c_hidden_mul, linear_init_params=tm)
        self.tri_att_start = TriangleAttention(c_z, c_hidden_pair_att, no_heads_pair, inf=inf,
                                               linear_init_params=ta)
        # like the reference, a *starting* module that is handed the transposed tensor
        self.tri_att_end = TriangleAttention(c_z, c_hidden_pair_att, no_heads_pair, inf=inf,
                                             linear_init_params=ta)

    @staticmethod
    def _mul(module, z, mask, inplace):
        return F3.triangle_multiplicative_update(z, mask, *module._weights(), outgoing=module._outgoing,
                                                 add_residual=True, inplace=inplace)

    @staticmethod
    def _att(module, z, mask, inplace):
        return F3.triangle_attention(
            z, mask, module.layer_norm.weight, module.layer_norm.bias, module.linear_z.weight,
            module.mha.linear_q.weight, module.mha.linear_k.weight, module.mha.linear_v.weight,
            module.mha.linear_g.weight, module.mha.linear_o.weight,
            no_heads=module.no_heads, inf=module.inf, add_residual=True, inplace=inplace)

    @forward_only
    def tri_mul_out_in(self, z, pair_mask, inplace_safe: bool = False, use_cueq_triangle_kernels: bool = False):
        """base_blocks.py:307-351.  Without inplace_safe the caller's tensor is left intact:
        the first z + update lands in a new tensor, which the second module then overwrites."""
        z = self._mul(self.tri_mul_out, z, pair_mask, inplace=inplace_safe)
        return self._mul(self.tri_mul_in, z, pair_mask, inplace=True)

    @forward_only
    def tri_att_start_end(self, z, pair_mask, _attn_chunk_size=None, use_deepspeed_evo_attention=False,
                          use_cueq_triangle_kernels=False, use_lma=False, inplace_safe: bool = False):
        """base_blocks.py:353-406; the ending node is the starting-node module run on the
        transposed view of z and of the mask."""
        z = self._att(self.tri_att_start, z, pair_mask, inplace=inplace_safe)
        zt = z.transpose(-2, -3)
        mt = pair_mask.transpose(-1, -2) if pair_mask is not None else None
        zt = self._att(self.tri_att_end, zt, mt, inplace=True)
        return zt.transpose(-2, -3)

    @forward_only
    def forward(self, z, pair_mask, chunk_size=None, use_deepspeed_evo_attention=False,
                use_cueq_triangle_kernels=False, use_lma=False, inplace_safe: bool = False,
                _attn_chunk_size=None):
        """z [*, N, N, C_z], pair_mask [*, N, N] -> z after the four residual updates.
        Leading dimensions (batch, templates) are independent and processed together.  With
        inplace_safe the input tensor is overwritten; otherwise it is left intact."""
        z = self.tri_mul_out_in(z, pair_mask, inplace_safe=inplace_safe)
        # z is now a tensor this module owns (or the caller allowed overwriting)
        return self.tri_att_start_end(z, pair_mask, inplace_safe=True)


class PairBlock(PairStack):
    """The reference's PairBlock (base_blocks.py:218-480): the four triangle updates, then
    z + pair_transition(z, mask).  Same constructor arguments and sub-module names
    (tri_mul_out, tri_mul_in, tri_att_start, tri_att_end, pair_transition).  Only what the
    AF3 configuration uses is implemented: the SwiGLU transition; fuse_projection_weights selects the
    fused-projection triangle multiplications (bias-free, as the reference's table initialises them);
    pair_dropout is accepted for signature parity (inference: identity)."""

    def __init__(self, c_z: int, c_hidden_mul: int, c_hidden_pair_att: int, no_heads_pair: int,
                 transition_type: str = "swiglu", transition_n: int = 4, pair_dropout: float = 0.0,
                 fuse_projection_weights: bool = False, inf: float = 1e9, linear_init_params=None):
        if transition_type != "swiglu":
            raise ValueError("Transition type %s is not available (the kernels implement 'swiglu')" % transition_type)
        super().__init__(c_z, c_hidden_mul, c_hidden_pair_att, no_heads_pair, inf=inf,
                         linear_init_params=linear_init_params, fuse_projection_weights=fuse_projection_weights)
        pt = None
        if linear_init_params is not None and "pair_transition" in linear_init_params:
            pt = linear_init_params["pair_transition"]
            pt = pt["swiglu"] if "swiglu" in pt else pt
        self.pair_transition = SwiGLUTransition(c_z, transition_n, linear_init_params=pt)
        self.pair_dropout = pair_dropout

    @forward_only
    def forward(self, z, pair_mask, chunk_size=None, use_deepspeed_evo_attention=False,
                use_cueq_triangle_kernels=False, use_lma=False, inplace_safe: bool = False,
                _mask_trans: bool = True, _attn_chunk_size=None):
        """base_blocks.py:408-480.  _mask_trans=False runs the transition unmasked
        (base_blocks.py:445-448)."""
        z = super().forward(z, pair_mask, inplace_safe=inplace_safe)
        # z is owned by this call (or may be overwritten): the transition updates it in place
        return self.pair_transition(z, mask=pair_mask if _mask_trans else None, _add_residual=True, _inplace=True)
