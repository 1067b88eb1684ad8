"""Template branch built on the pair-stack kernels: the reference's TemplatePairBlock,
TemplatePairStack and the part of TemplateEmbedderAllAtom that follows the feature embedding
(openfold3/core/model/latent/template_module.py:37-198, :200-378, :381-467).

The reference loops over the templates one by one (template_module.py:148-193); templates are
independent pair representations, so here they are folded into the batch and every kernel is
launched once for all of them.  The stack's closing LayerNorm, the mean over the templates, the
ReLU and linear_t run as one fused kernel in the embedder.
"""
from __future__ import annotations

import torch
import torch.nn as nn

from . import functional as F3
from ._guard import forward_only
from .layers import _init_linear, _init_name
from .pair_stack import PairBlock


class TemplatePairBlock(PairBlock):
    """template_module.py:37-198: a PairBlock over [*, N_templ, N, N, C_t], with the triangle
    multiplications before or after the triangle attention (tri_mul_first)."""

    def __init__(self, c_t: int, c_hidden_tri_att: int, c_hidden_tri_mul: int, no_heads: int,
                 transition_type: str = "swiglu", pair_transition_n: int = 2, dropout_rate: float = 0.0,
                 tri_mul_first: bool = True, fuse_projection_weights: bool = False, inf: float = 1e9,
                 linear_init_params=None):
        super().__init__(c_z=c_t, c_hidden_mul=c_hidden_tri_mul, c_hidden_pair_att=c_hidden_tri_att,
                         no_heads_pair=no_heads, transition_type=transition_type, transition_n=pair_transition_n,
                         pair_dropout=dropout_rate, fuse_projection_weights=fuse_projection_weights, inf=inf,
                         linear_init_params=linear_init_params)
        self.tri_mul_first = tri_mul_first

    @forward_only
    def forward(self, z, mask, chunk_size=None, use_deepspeed_evo_attention=False, use_cueq_triangle_kernels=False,
                use_lma=False, inplace_safe: bool = False, _mask_trans: bool = True, _attn_chunk_size=None):
        """z [*, N_templ, N, N, C_t], mask [*, N_templ, N, N] -> updated z.  Without inplace_safe
        the input is left intact."""
        if self.tri_mul_first:
            z = self.tri_mul_out_in(z, mask, inplace_safe=inplace_safe)
            z = self.tri_att_start_end(z, mask, inplace_safe=True)
        else:
            z = self.tri_att_start_end(z, mask, inplace_safe=inplace_safe)
            z = self.tri_mul_out_in(z, mask, inplace_safe=True)
        return self.pair_transition(z, mask=mask if _mask_trans else None, _add_residual=True, _inplace=True)


class TemplatePairStack(nn.Module):
    """template_module.py:200-378: `no_blocks` TemplatePairBlocks and a closing LayerNorm, under
    the reference's sub-module names (blocks.<i>.*, layer_norm.*).  blocks_per_ckpt,
    use_reentrant and tune_chunk_size are accepted for signature parity (inference only; no
    chunking is needed, the kernels hold no N^3 intermediate)."""

    def __init__(self, c_t: int, c_hidden_tri_att: int, c_hidden_tri_mul: int, no_blocks: int, no_heads: int,
                 transition_type: str = "swiglu", pair_transition_n: int = 2, dropout_rate: float = 0.0,
                 tri_mul_first: bool = True, fuse_projection_weights: bool = False, blocks_per_ckpt=None,
                 inf: float = 1e9, linear_init_params=None, use_reentrant=None, tune_chunk_size: bool = False,
                 **kwargs):
        super().__init__()
        self.blocks_per_ckpt = blocks_per_ckpt
        self.use_reentrant = use_reentrant
        self.tune_chunk_size = tune_chunk_size
        self.blocks = nn.ModuleList([
            TemplatePairBlock(c_t, c_hidden_tri_att, c_hidden_tri_mul, no_heads, transition_type, pair_transition_n,
                              dropout_rate, tri_mul_first, fuse_projection_weights, inf, linear_init_params)
            for _ in range(no_blocks)
        ])
        self.layer_norm = nn.LayerNorm(c_t, eps=1e-5)

    @staticmethod
    def _expand_mask(t, mask):
        if mask is not None and mask.shape[-3] == 1 and t.shape[-4] != 1:  # template_module.py:326-329
            shape = list(mask.shape)
            shape[-3] = t.shape[-4]
            mask = mask.expand(*shape)
        return mask

    @forward_only
    def run_blocks(self, t, mask, inplace_safe: bool = False, _mask_trans: bool = True):
        """The blocks without the closing LayerNorm (the embedder fuses it into its tail)."""
        mask = self._expand_mask(t, mask)
        for i, blk in enumerate(self.blocks):
            # after the first block the tensor belongs to this call
            t = blk(t, mask, inplace_safe=inplace_safe or i > 0, _mask_trans=_mask_trans)
        return t

    @forward_only
    def forward(self, t, mask, chunk_size=None, use_deepspeed_evo_attention=False, use_cueq_triangle_kernels=False,
                use_lma=False, inplace_safe: bool = False, _mask_trans: bool = True):
        """t [*, N_templ, N, N, C_t], mask [*, N_templ, N, N] or [*, 1, N, N] -> LayerNorm of the
        blocks' output, same shape."""
        t = self.run_blocks(t, mask, inplace_safe=inplace_safe, _mask_trans=_mask_trans)
        return F3.layer_norm(t, self.layer_norm.weight, self.layer_norm.bias)


class TemplateEmbedderCore(nn.Module):
    """TemplateEmbedderAllAtom (template_module.py:381-467) from the template pair embedding
    onwards: template_pair_stack and linear_t under the reference's names, so the matching keys
    of a `template_embedder.` state dict load unchanged (strict=False skips the feature
    embedder's).  The feature embedding itself (template_pair_embedder, distogram and frame
    features) is outside this package: forward takes its output."""

    def __init__(self, c_t: int, c_z: int, template_pair_stack: dict, linear_init_params=None):
        super().__init__()
        self.template_pair_stack = TemplatePairStack(**template_pair_stack)
        self.linear_t = nn.Linear(c_t, c_z, bias=False)
        _init_linear(self.linear_t, _init_name(linear_init_params, "linear_t", "default"))

    @forward_only
    def forward(self, template_embeds, pair_mask, chunk_size=None, _mask_trans: bool = True,
                use_deepspeed_evo_attention=False, use_cueq_triangle_kernels=False, use_lma=False,
                inplace_safe: bool = False):
        """template_embeds [*, N_templ, N, N, C_t] (what template_pair_embedder returns),
        pair_mask [*, N, N] -> [*, N, N, C_z] (template_module.py:447-467)."""
        mask = pair_mask[..., None, :, :].to(dtype=torch.float32)
        stack = self.template_pair_stack
        t = stack.run_blocks(template_embeds, mask, inplace_safe=inplace_safe, _mask_trans=_mask_trans)
        return F3.template_tail(t, stack.layer_norm.weight, stack.layer_norm.bias, self.linear_t.weight)
