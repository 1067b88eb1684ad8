"""The Pairformer trunk on the kernels of this package: the reference's PairFormerBlock and
PairFormerStack (openfold3/core/model/latent/pairformer.py:36-215, :217-470, AF3 Algorithm 17)
with the same constructor arguments, sub-module names and forward signatures, so that
`config.architecture.pairformer` constructs the stack and the `pairformer_stack.*` keys of a
checkpoint load unchanged.  Inference only, bf16.
"""
from __future__ import annotations

import torch
import torch.nn as nn

from ._guard import forward_only
from .layers import AttentionPairBias, SwiGLUTransition
from .pair_stack import PairBlock


def _sub(params, key):
    if params is None:
        return None
    return params.get(key) if hasattr(params, "get") else params[key]


class PairFormerBlock(nn.Module):
    """pairformer.py:36-215: z = pair_stack(z); s += attn_pair_bias(s, z); s += single_transition(s)."""

    def __init__(self, c_s: int, c_z: int, c_hidden_pair_bias: int, no_heads_pair_bias: int, c_hidden_mul: int,
                 c_hidden_pair_att: int, no_heads_pair: int, transition_type: str = "swiglu", transition_n: int = 4,
                 pair_dropout: float = 0.0, fuse_projection_weights: bool = False, inf: float = 1e9,
                 linear_init_params=None):
        super().__init__()
        self.pair_stack = PairBlock(c_z=c_z, c_hidden_mul=c_hidden_mul, c_hidden_pair_att=c_hidden_pair_att,
                                    no_heads_pair=no_heads_pair, transition_type=transition_type,
                                    transition_n=transition_n, pair_dropout=pair_dropout,
                                    fuse_projection_weights=fuse_projection_weights, inf=inf,
                                    linear_init_params=_sub(linear_init_params, "pair_block"))
        self.attn_pair_bias = AttentionPairBias(c_q=c_s, c_k=c_s, c_v=c_s, c_s=c_s, c_z=c_z,
                                                c_hidden=c_hidden_pair_bias, no_heads=no_heads_pair_bias,
                                                use_ada_layer_norm=False, gating=True, inf=inf,
                                                linear_init_params=_sub(linear_init_params, "att_pair_bias"))
        tr = _sub(linear_init_params, "transition")
        if tr is not None and "swiglu" in tr and "linear_out" not in tr:
            tr = tr["swiglu"]
        self.single_transition = SwiGLUTransition(c_in=c_s, n=transition_n, linear_init_params=tr)

    @forward_only
    def forward(self, s, z, single_mask, pair_mask, chunk_size=None, use_deepspeed_evo_attention=False,
                use_cueq_triangle_kernels=False, use_lma=False, inplace_safe: bool = False, _mask_trans: bool = True,
                _attn_chunk_size=None):
        """s [*, N, C_s], z [*, N, N, C_z], single_mask [*, N], pair_mask [*, N, N] -> (s, z).
        With inplace_safe both inputs are overwritten; otherwise they are left intact."""
        z = self.pair_stack(z, pair_mask, inplace_safe=inplace_safe, _mask_trans=_mask_trans)
        s = self.attn_pair_bias(a=s, z=z, s=None, mask=single_mask, _add_residual=True, _inplace=inplace_safe)
        # s is now a tensor this call owns (or may be overwritten)
        s = self.single_transition(s, mask=single_mask if _mask_trans else None, _add_residual=True, _inplace=True)
        return s, z


class PairFormerStack(nn.Module):
    """pairformer.py:217-470: `no_blocks` PairFormerBlocks under `blocks.<i>`.  blocks_per_ckpt,
    use_reentrant, clear_cache_between_blocks and tune_chunk_size are accepted for signature
    parity (inference only; nothing here needs chunking or cache clearing)."""

    def __init__(self, c_s: int, c_z: int, c_hidden_pair_bias: int, no_heads_pair_bias: int, c_hidden_mul: int,
                 c_hidden_pair_att: int, no_heads_pair: int, no_blocks: int, transition_type: str = "swiglu",
                 transition_n: int = 4, pair_dropout: float = 0.0, fuse_projection_weights: bool = False,
                 blocks_per_ckpt=None, inf: float = 1e9, linear_init_params=None, use_reentrant=None,
                 clear_cache_between_blocks: bool = False, tune_chunk_size: bool = False, **kwargs):
        super().__init__()
        self.blocks_per_ckpt = blocks_per_ckpt
        self.use_reentrant = use_reentrant
        self.clear_cache_between_blocks = clear_cache_between_blocks
        self.tune_chunk_size = tune_chunk_size
        self.blocks = nn.ModuleList([
            PairFormerBlock(c_s, c_z, c_hidden_pair_bias, no_heads_pair_bias, c_hidden_mul, c_hidden_pair_att,
                            no_heads_pair, transition_type, transition_n, pair_dropout, fuse_projection_weights, inf,
                            linear_init_params)
            for _ in range(no_blocks)
        ])

    @forward_only
    def forward(self, s, z, single_mask, pair_mask, chunk_size=None, use_deepspeed_evo_attention=False,
                use_cueq_triangle_kernels=False, use_lma=False, inplace_safe: bool = False, _mask_trans: bool = True):
        """s [*, N, C_s], z [*, N, N, C_z], single_mask [*, N], pair_mask [*, N, N] -> (s, z)
        (pairformer.py:398-470)."""
        for i, blk in enumerate(self.blocks):
            # after the first block both tensors belong to this call
            s, z = blk(s, z, single_mask, pair_mask, inplace_safe=inplace_safe or i > 0, _mask_trans=_mask_trans)
        return s, z
