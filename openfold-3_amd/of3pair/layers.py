"""Drop-in counterparts of the reference's pair-stack layer modules.

Constructor arguments, parameter names (state-dict keys) and forward signatures follow
  openfold3/core/model/layers/triangular_multiplicative_update.py:119-152, :421-429, :506-519
  openfold3/core/model/layers/triangular_attention.py:31-69, :102-111, :171-179
  openfold3/core/model/layers/transition.py:225-255, :90-110 (SwiGLUTransition)
so that a PairBlock (openfold3/core/model/latent/base_blocks.py:268-288) can hold these
modules instead and load the same checkpoints.  The arithmetic runs in libof3pair (HIP);
there is one implementation, so the reference's kernel-selection and chunking keyword
arguments are accepted and ignored.  Forward only: gradients are not recorded.
"""
from __future__ import annotations

import math
from functools import partialmethod

import torch
import torch.nn as nn

from . import functional as F3
from ._guard import forward_only


def _truncated_normal_(weight: torch.Tensor, scale: float = 1.0):
    """LeCun fan-in truncated normal (cut at two standard deviations), the reference's
    "default" Linear initialiser (initialization.py:48-63).  Drawn with torch's generator;
    the reference draws the same distribution from scipy on numpy's global generator, so the
    sample streams differ while the distribution does not."""
    fan_in = weight.shape[1]
    # standard deviation of a unit normal truncated to [-2, 2]
    trunc_std = 0.87962566103423978
    std = math.sqrt(scale / max(1, fan_in)) / trunc_std
    with torch.no_grad():
        nn.init.trunc_normal_(weight, mean=0.0, std=std, a=-2.0 * std, b=2.0 * std)


def _init_linear(lin: nn.Linear, how: str):
    if how == "default":
        _truncated_normal_(lin.weight)
    elif how in ("relu", "he_normal"):  # He initialisation, truncated normal (initialization.py:66-67)
        _truncated_normal_(lin.weight, scale=2.0)
    elif how in ("final", "gating"):
        with torch.no_grad():
            lin.weight.zero_()
    else:
        raise ValueError("Invalid init string.")


# Initialiser table of the AF3 pair stack (default_linear_init_config.py:110-119, :45-53,
# :78-83): every Linear is bias-free; gates and output projections start at zero.
TRI_MUL_INIT = {
    "linear_a_p": "default", "linear_a_g": "final", "linear_b_p": "default", "linear_b_g": "final",
    "linear_g": "final", "linear_z": "final",
}
TRI_ATT_INIT = {
    "linear_z": "default",
    "mha": {"linear_q": "default", "linear_k": "default", "linear_v": "default", "linear_g": "gating",
            "linear_o": "final"},
}


# the fused-projection form (default_linear_init_config.py:122-129): bias-free as well
FUSED_TRI_MUL_INIT = {"linear_ab_p": "default", "linear_ab_g": "gating", "linear_g": "gating", "linear_z": "final"}


# default_linear_init_config.py:29-34, :157-162
SWIGLU_TRANSITION_INIT = {"swiglu": {"linear_a": "relu", "linear_b": "relu"}, "linear_out": "final"}


def _init_name(spec, key, default):
    """Accepts the table above or a reference-style mapping {"bias": False, "init": "..."}."""
    if spec is None:
        return default
    v = spec[key] if not hasattr(spec, "get") else spec.get(key, default)
    if isinstance(v, str):
        return v
    if v.get("bias", False):
        raise ValueError("the pair-stack kernels implement the bias-free Linears of the AF3 tables")
    return v.get("init", default)


class TriangleMultiplicativeUpdate(nn.Module):
    """AF3 Algorithms 12 and 13 (tmu.py:119-503)."""

    def __init__(self, c_z, c_hidden, _outgoing=True, linear_init_params=None):
        super().__init__()
        self.c_z = c_z
        self.c_hidden = c_hidden
        self._outgoing = _outgoing
        self.linear_g = nn.Linear(c_z, c_z, bias=False)
        self.linear_z = nn.Linear(c_hidden, c_z, bias=False)
        self.layer_norm_in = nn.LayerNorm(c_z, eps=1e-5)
        self.layer_norm_out = nn.LayerNorm(c_hidden, eps=1e-5)
        self.linear_a_p = nn.Linear(c_z, c_hidden, bias=False)
        self.linear_a_g = nn.Linear(c_z, c_hidden, bias=False)
        self.linear_b_p = nn.Linear(c_z, c_hidden, bias=False)
        self.linear_b_g = nn.Linear(c_z, c_hidden, bias=False)
        for name, default in TRI_MUL_INIT.items():
            _init_linear(getattr(self, name), _init_name(linear_init_params, name, default))

    def _weights(self):
        """The ten tensors of F3.triangle_multiplicative_update, in its order."""
        return (self.layer_norm_in.weight, self.layer_norm_in.bias, self.layer_norm_out.weight, self.layer_norm_out.bias,
                self.linear_a_p.weight, self.linear_a_g.weight, self.linear_b_p.weight, self.linear_b_g.weight,
                self.linear_g.weight, self.linear_z.weight)

    @forward_only
    def forward(self, z, mask=None, inplace_safe=False, use_cueq_triangle_kernels=False,
                _add_with_inplace=False, _inplace_chunk_size=256):
        """z [*, N, N, C_z], mask [*, N, N] -> [*, N, N, C_z].

        Returns the update; with inplace_safe the result overwrites z and, if
        _add_with_inplace is also set, is z + update (tmu.py:473-480, :399-405).  The
        kernel-selection flag and the chunk size are accepted for signature compatibility."""
        return F3.triangle_multiplicative_update(
            z, mask,
            self.layer_norm_in.weight, self.layer_norm_in.bias,
            self.layer_norm_out.weight, self.layer_norm_out.bias,
            self.linear_a_p.weight, self.linear_a_g.weight, self.linear_b_p.weight, self.linear_b_g.weight,
            self.linear_g.weight, self.linear_z.weight,
            outgoing=self._outgoing,
            add_residual=bool(inplace_safe and _add_with_inplace),
            inplace=bool(inplace_safe),
        )


class TriangleMultiplicationOutgoing(TriangleMultiplicativeUpdate):
    """AF3 Algorithm 12."""

    __init__ = partialmethod(TriangleMultiplicativeUpdate.__init__, _outgoing=True)


class TriangleMultiplicationIncoming(TriangleMultiplicativeUpdate):
    """AF3 Algorithm 13."""

    __init__ = partialmethod(TriangleMultiplicativeUpdate.__init__, _outgoing=False)


class FusedTriangleMultiplicativeUpdate(nn.Module):
    """The fused-projection form of the triangle multiplication (tmu.py:522-666): linear_ab_p and
    linear_ab_g hold the a and b projections stacked, [2 * c_hidden, c_z], rows 0 .. c_hidden - 1 being a
    (tmu.py:578-580, :646-647).  Same arithmetic as the un-fused module, so the same kernels run it: the
    two halves of each stacked weight are handed over as the a and b matrices (contiguous row slices, no
    copy).  State-dict keys: layer_norm_in, layer_norm_out, linear_ab_p, linear_ab_g, linear_g, linear_z.
    Bias-free Linears only, as in the reference's own initialiser table for this module."""

    def __init__(self, c_z, c_hidden, _outgoing=True, linear_init_params=None):
        super().__init__()
        self.c_z = c_z
        self.c_hidden = c_hidden
        self._outgoing = _outgoing
        self.linear_g = nn.Linear(c_z, c_z, bias=False)
        self.linear_z = nn.Linear(c_hidden, c_z, bias=False)
        self.layer_norm_in = nn.LayerNorm(c_z, eps=1e-5)
        self.layer_norm_out = nn.LayerNorm(c_hidden, eps=1e-5)
        self.linear_ab_p = nn.Linear(c_z, 2 * c_hidden, bias=False)
        self.linear_ab_g = nn.Linear(c_z, 2 * c_hidden, bias=False)
        for name, default in FUSED_TRI_MUL_INIT.items():
            _init_linear(getattr(self, name), _init_name(linear_init_params, name, default))

    def _weights(self):
        """The ten tensors of F3.triangle_multiplicative_update, in its order."""
        ch = self.c_hidden
        p, g = self.linear_ab_p.weight, self.linear_ab_g.weight
        return (self.layer_norm_in.weight, self.layer_norm_in.bias, self.layer_norm_out.weight, self.layer_norm_out.bias,
                p[:ch], g[:ch], p[ch:], g[ch:], self.linear_g.weight, self.linear_z.weight)

    @forward_only
    def forward(self, z, mask=None, inplace_safe=False, use_cueq_triangle_kernels=False,
                _add_with_inplace=False, _inplace_chunk_size=256):
        """z [*, N, N, C_z], mask [*, N, N] -> [*, N, N, C_z]; the in-place contract of tmu.py:620-628."""
        if use_cueq_triangle_kernels:  # tmu.py:612-618
            raise NotImplementedError("CUEQ triangle multiplicative update kernel not supported for "
                                      "FusedTriangleMultiplicativeUpdate.")
        return F3.triangle_multiplicative_update(
            z, mask, *self._weights(), outgoing=self._outgoing,
            add_residual=bool(inplace_safe and _add_with_inplace), inplace=bool(inplace_safe))


class FusedTriangleMultiplicationOutgoing(FusedTriangleMultiplicativeUpdate):
    __init__ = partialmethod(FusedTriangleMultiplicativeUpdate.__init__, _outgoing=True)


class FusedTriangleMultiplicationIncoming(FusedTriangleMultiplicativeUpdate):
    __init__ = partialmethod(FusedTriangleMultiplicativeUpdate.__init__, _outgoing=False)


class _GatedAttentionParams(nn.Module):
    """Holds the parameters of the reference's Attention module (attention.py:206-263) under
    the same names; the computation itself is fused into the triangle-attention kernels."""

    def __init__(self, c_in, c_hidden, no_heads, init):
        super().__init__()
        hc = c_hidden * no_heads
        self.c_hidden = c_hidden
        self.no_heads = no_heads
        self.linear_q = nn.Linear(c_in, hc, bias=False)
        self.linear_k = nn.Linear(c_in, hc, bias=False)
        self.linear_v = nn.Linear(c_in, hc, bias=False)
        self.linear_o = nn.Linear(hc, c_in, bias=False)
        self.linear_g = nn.Linear(c_in, hc, bias=False)
        for name, default in TRI_ATT_INIT["mha"].items():
            _init_linear(getattr(self, name), _init_name(init, name, default))


class TriangleAttention(nn.Module):
    """AF3 Algorithms 14 and 15 (tri_att.py:31-167).  c_hidden is the per-head width, as
    the reference's Attention treats it (attention.py:240-242)."""

    def __init__(self, c_in, c_hidden, no_heads, starting=True, inf=1e9, linear_init_params=None):
        super().__init__()
        self.c_in = c_in
        self.c_hidden = c_hidden
        self.no_heads = no_heads
        self.starting = starting
        self.inf = inf
        self.layer_norm = nn.LayerNorm(c_in, eps=1e-5)
        self.linear_z = nn.Linear(c_in, no_heads, bias=False)
        _init_linear(self.linear_z, _init_name(linear_init_params, "linear_z", TRI_ATT_INIT["linear_z"]))
        mha_init = None
        if linear_init_params is not None:
            mha_init = linear_init_params["mha"] if "mha" in linear_init_params else None
        self.mha = _GatedAttentionParams(c_in, c_hidden, no_heads, mha_init)

    @forward_only
    def forward(self, x, mask=None, chunk_size=None, use_deepspeed_evo_attention=False,
                use_cueq_triangle_kernels=False, use_lma=False, inplace_safe=False,
                _add_residual=False):
        """x [*, I, J, C_in], mask [*, I, J] -> [*, I, J, C_in] (the update).

        The back-end flags and chunk_size of the reference are accepted and ignored: the
        flash kernel never materialises the logits, so there is nothing to chunk.
        _add_residual (not in the reference) returns x + update from the output kernel; the
        pair-stack runner uses it to fuse the caller's add of base_blocks.py:364-378."""
        if not self.starting:
            x = x.transpose(-2, -3)
            mask = mask.transpose(-1, -2) if mask is not None else None
        out = F3.triangle_attention(
            x, mask,
            self.layer_norm.weight, self.layer_norm.bias, self.linear_z.weight,
            self.mha.linear_q.weight, self.mha.linear_k.weight, self.mha.linear_v.weight,
            self.mha.linear_g.weight, self.mha.linear_o.weight,
            no_heads=self.no_heads, inf=self.inf, add_residual=bool(_add_residual), inplace=False,
        )
        if not self.starting:
            out = out.transpose(-2, -3)
        return out


TriangleAttentionStartingNode = TriangleAttention


class TriangleAttentionEndingNode(TriangleAttention):
    """AF3 Algorithm 15."""

    __init__ = partialmethod(TriangleAttention.__init__, starting=False)


class _SwiGLUParams(nn.Module):
    """Parameter holder with the names of the reference's SwiGLU (activations.py:33-55)."""

    def __init__(self, c_in, c_out, init):
        super().__init__()
        self.c_in = c_in
        self.c_out = c_out
        self.linear_a = nn.Linear(c_in, c_out, bias=False)
        self.linear_b = nn.Linear(c_in, c_out, bias=False)
        for name, default in SWIGLU_TRANSITION_INIT["swiglu"].items():
            _init_linear(getattr(self, name), _init_name(init, name, default))


class SwiGLUTransition(nn.Module):
    """AF3 Algorithm 11 as the pair stack uses it (transition.py:225-271): LayerNorm, SwiGLU,
    linear_out, mask.  State-dict keys: layer_norm.{weight,bias}, swiglu.linear_{a,b}.weight,
    linear_out.weight.  Pair tensors x [*, N, N, C_in] with mask [*, N, N] (C_in 64 or 128), or the
    single representation x [*, N, 384] with mask [*, N]."""

    def __init__(self, c_in, n, linear_init_params=None):
        super().__init__()
        self.c_in = c_in
        self.n = n
        self.layer_norm = nn.LayerNorm(c_in, eps=1e-5)
        sw = None
        if linear_init_params is not None:
            sw = linear_init_params["swiglu"] if "swiglu" in linear_init_params else None
        self.swiglu = _SwiGLUParams(c_in, n * c_in, sw)
        self.linear_out = nn.Linear(n * c_in, c_in, bias=False)
        _init_linear(self.linear_out, _init_name(linear_init_params, "linear_out", SWIGLU_TRANSITION_INIT["linear_out"]))

    @forward_only
    def forward(self, x, mask=None, chunk_size=None, ckpt_chunk_size=None, _add_residual=False, _inplace=False):
        """x [*, N, N, C_in], mask [*, N, N] or None (all ones, transition.py:106-107) -> the
        update.  chunk_size / ckpt_chunk_size of the reference are accepted and ignored: the
        hidden activations never leave the registers, so there is nothing to chunk.
        _add_residual / _inplace (not in the reference) return x + update from the kernel and
        overwrite x; the pair-stack runner uses them for the add of base_blocks.py:470-478."""
        return F3.swiglu_transition(
            x, mask, self.layer_norm.weight, self.layer_norm.bias, self.swiglu.linear_a.weight,
            self.swiglu.linear_b.weight, self.linear_out.weight, add_residual=bool(_add_residual),
            inplace=bool(_inplace))


class PairBiasProjection(nn.Module):
    """The pair-bias half of the reference's AttentionPairBias (attention_pair_bias.py:106-107,
    :151-161): layer_norm_z and linear_z under the same parameter names, so the matching slice
    of an AttentionPairBias state dict loads unchanged.  forward(z) returns the [*, H, N, N]
    bias that _prep_bias appends to its list."""

    def __init__(self, c_z, no_heads, create_offset=True, linear_init="default"):
        super().__init__()
        self.c_z = c_z
        self.no_heads = no_heads
        self.layer_norm_z = nn.LayerNorm(c_z, eps=1e-5, bias=create_offset)
        self.linear_z = nn.Linear(c_z, no_heads, bias=False)
        _init_linear(self.linear_z, linear_init)

    @forward_only
    def forward(self, z):
        return F3.pair_bias(z, self.layer_norm_z.weight, self.layer_norm_z.bias, self.linear_z.weight)


class _PairBiasAttentionParams(nn.Module):
    """Parameter holder with the names of the reference's Attention inside AttentionPairBias
    (attention.py:236-258 with default_linear_init_config.py:56-64: linear_q carries a bias)."""

    def __init__(self, c_q, c_hidden, no_heads, init):
        super().__init__()
        hc = c_hidden * no_heads
        self.linear_q = nn.Linear(c_q, hc, bias=True)
        self.linear_k = nn.Linear(c_q, hc, bias=False)
        self.linear_v = nn.Linear(c_q, hc, bias=False)
        self.linear_o = nn.Linear(hc, c_q, bias=False)
        self.linear_g = nn.Linear(c_q, hc, bias=False)
        for name, default in (("linear_q", "default"), ("linear_k", "default"), ("linear_v", "default"),
                              ("linear_g", "gating"), ("linear_o", "final")):
            spec = None if init is None else (init.get(name) if hasattr(init, "get") else init[name])
            how = default if spec is None else (spec if isinstance(spec, str) else spec.get("init", default))
            _init_linear(getattr(self, name), how)
        with torch.no_grad():
            self.linear_q.bias.zero_()


class AttentionPairBias(nn.Module):
    """The trunk's AttentionPairBias (attention_pair_bias.py:33-244, AF3 Algorithm 24 without
    AdaLN): same constructor arguments, parameter names (layer_norm_a, layer_norm_z, linear_z,
    mha.linear_q/k/v/g/o) and forward signature.  use_ada_layer_norm (the diffusion variant) and
    ungated attention are not implemented."""

    def __init__(self, c_q, c_k, c_v, c_s, c_z, c_hidden, no_heads, use_ada_layer_norm=False, gating=True, inf=1e9,
                 linear_init_params=None):
        super().__init__()
        if use_ada_layer_norm or not gating:
            raise ValueError("only the trunk variant (LayerNorm, gated) is implemented")
        if not (c_q == c_k == c_v):
            raise ValueError("self-attention over one representation: c_q = c_k = c_v")
        self.c_q, self.c_s, self.c_z, self.inf, self.no_heads = c_q, c_s, c_z, inf, no_heads
        self.use_ada_layer_norm = False
        offset = True
        mha_init = None
        if linear_init_params is not None:
            lz = linear_init_params.get("layer_norm_z") if hasattr(linear_init_params, "get") else None
            if lz is not None:
                offset = bool(lz.get("create_offset", True))
            mha_init = linear_init_params.get("mha") if hasattr(linear_init_params, "get") else None
        self.layer_norm_a = nn.LayerNorm(c_q, eps=1e-5)
        self.layer_norm_z = nn.LayerNorm(c_z, eps=1e-5, bias=offset)
        self.linear_z = nn.Linear(c_z, no_heads, bias=False)
        _init_linear(self.linear_z, _init_name(linear_init_params, "linear_z", "default"))
        self.mha = _PairBiasAttentionParams(c_q, c_hidden, no_heads, mha_init)

    @forward_only
    def forward(self, a, z, s=None, mask=None, use_deepspeed_evo_attention=False, use_cueq_triangle_kernels=False,
                use_lma=False, use_high_precision_attention=False, _add_residual: bool = False,
                _inplace: bool = False):
        """a [*, N, C_q], z [*, N, N, C_z], mask [*, N] -> the update [*, N, C_q]
        (a + update with _add_residual, written into a with _inplace)."""
        m = self.mha
        return F3.attention_pair_bias(
            a, z, mask, self.layer_norm_a.weight, self.layer_norm_a.bias, self.layer_norm_z.weight,
            self.layer_norm_z.bias, self.linear_z.weight, m.linear_q.weight, m.linear_q.bias, m.linear_k.weight,
            m.linear_v.weight, m.linear_g.weight, m.linear_o.weight, no_heads=self.no_heads, inf=self.inf,
            add_residual=_add_residual, inplace=_inplace)
