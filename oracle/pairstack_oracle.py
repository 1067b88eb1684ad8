"""CPU oracle for the OpenFold3 pair-stack hot path.  TEST INFRASTRUCTURE ONLY.

This file restates, in plain fp32 PyTorch on the CPU, the arithmetic of the
reference's stock (no alternative kernel) path through

  * TriangleMultiplicativeUpdate.forward
      openfold3/core/model/layers/triangular_multiplicative_update.py:482-503
    with _combine_projections (same file, :71-97),
  * TriangleAttention.forward
      openfold3/core/model/layers/triangular_attention.py:102-167
    with Attention._prep_qkv / _attention / _wrap_up
      openfold3/core/model/primitives/attention.py:265-302, :94-135,
  * PairBlock.tri_mul_out_in / tri_att_start_end
      openfold3/core/model/latent/base_blocks.py:307-406,
  * TemplatePairBlock.forward (per-template loop, tri_mul_first=True), TemplatePairStack.forward
    with its final LayerNorm, and the mean / ReLU / linear_t tail of TemplateEmbedderAllAtom
      openfold3/core/model/latent/template_module.py:148-193, :302-378, :462-465,
  * AttentionPairBias.forward of the trunk (single representation, pair bias from z)
      openfold3/core/model/layers/attention_pair_bias.py:121-244.

It may be imported by tests/, by __graft_entry__.smoke() and by the
cpu_baseline leg of bench.py, as the checker or the timed CPU baseline.
The shipped package never imports it.

The library routines it calls (F.layer_norm, F.linear, torch.einsum,
torch.softmax, torch.sigmoid) are the very routines the reference calls at
normalization.py:70-84, linear.py:127-138, tmu.py:95, attention.py:86-133 and
tmu.py:69.  The reference holds no golden vectors for this path; every
function here is pinned by tests/test_oracle_pinning.py against
oracle/brute_force.py (float64 explicit loops written from the index
formulas), against torch's scaled_dot_product_attention, and against the
algebraic invariants of the path.

Parameters travel as a flat ``dict[str, Tensor]`` keyed exactly like the
reference modules' state dicts (``layer_norm_in.weight``, ``linear_a_p.weight``,
``mha.linear_q.weight`` ...), so a drop-in module's ``state_dict()`` can be
handed to the oracle unchanged.
"""

from __future__ import annotations

import math

import torch
import torch.nn.functional as F

LN_EPS = 1e-5  # normalization.py:36 (eps default)
INF = 1e9  # triangular_attention.py:38


# --------------------------------------------------------------------------
# primitives
# --------------------------------------------------------------------------
def layer_norm(x, weight, bias, eps: float = LN_EPS):
    """normalization.py:59-86: F.layer_norm over the last dim, affine."""
    return F.layer_norm(x, (x.shape[-1],), weight.to(x.dtype), bias.to(x.dtype), eps)


def linear(x, weight):
    """linear.py:115-138 for a bias-free Linear: x @ W^T, W is [out, in]."""
    return F.linear(x, weight.to(x.dtype))


# --------------------------------------------------------------------------
# triangle multiplicative update
# --------------------------------------------------------------------------
def trimul_contract(a, b, outgoing: bool):
    """tmu.py:71-97.  a, b: [*, N, N, C] -> [*, N, N, C].

    Follows the reference literally: permute to channel-major, one matrix
    product per channel, permute back.
    """
    nd = a.dim()
    lead = list(range(nd - 3))

    def perm(t, inds):
        return t.permute(lead + [nd - 3 + i for i in inds])

    if outgoing:
        a = perm(a, (2, 0, 1))
        b = perm(b, (2, 1, 0))
    else:
        a = perm(a, (2, 1, 0))
        b = perm(b, (2, 0, 1))
    p = torch.einsum("...ij,...jk->...ik", a, b)
    return perm(p, (1, 2, 0))


def trimul_update(z, mask, p, outgoing: bool):
    """tmu.py:482-503.  Returns the update only (the caller adds it to z)."""
    if mask is None:
        mask = z.new_ones(z.shape[:-1])
    m = mask.to(z.dtype).unsqueeze(-1)
    zn = layer_norm(z, p["layer_norm_in.weight"], p["layer_norm_in.bias"])
    a = m
    a = a * torch.sigmoid(linear(zn, p["linear_a_g.weight"]))
    a = a * linear(zn, p["linear_a_p.weight"])
    b = m
    b = b * torch.sigmoid(linear(zn, p["linear_b_g.weight"]))
    b = b * linear(zn, p["linear_b_p.weight"])
    x = trimul_contract(a, b, outgoing)
    del a, b
    x = layer_norm(x, p["layer_norm_out.weight"], p["layer_norm_out.bias"])
    x = linear(x, p["linear_z.weight"])
    g = torch.sigmoid(linear(zn, p["linear_g.weight"]))
    return x * g


def fused_trimul_update(z, mask, p, outgoing: bool):
    """FusedTriangleMultiplicativeUpdate.forward, tmu.py:637-660 (bias-free Linears, as
    default_linear_init_config.py:122-129 creates them): the a and b projections come stacked out of
    linear_ab_p / linear_ab_g, [2 * c_hidden, c_z], and are cut apart after gating and masking."""
    if mask is None:
        mask = z.new_ones(z.shape[:-1])
    m = mask.to(z.dtype).unsqueeze(-1)
    c_hidden = p["linear_ab_p.weight"].shape[0] // 2
    zn = layer_norm(z, p["layer_norm_in.weight"], p["layer_norm_in.bias"])
    ab = m
    ab = ab * torch.sigmoid(linear(zn, p["linear_ab_g.weight"]))
    ab = ab * linear(zn, p["linear_ab_p.weight"])
    a = ab[..., :c_hidden]
    b = ab[..., c_hidden:]
    x = trimul_contract(a, b, outgoing)
    x = layer_norm(x, p["layer_norm_out.weight"], p["layer_norm_out.bias"])
    x = linear(x, p["linear_z.weight"])
    g = torch.sigmoid(linear(zn, p["linear_g.weight"]))
    return x * g


def fuse_trimul_params(p):
    """The un-fused parameter set of make_trimul_params under the fused module's names: a on top of b."""
    q = {k: v for k, v in p.items() if not k.startswith(("linear_a_", "linear_b_"))}
    q["linear_ab_p.weight"] = torch.cat([p["linear_a_p.weight"], p["linear_b_p.weight"]], dim=0)
    q["linear_ab_g.weight"] = torch.cat([p["linear_a_g.weight"], p["linear_b_g.weight"]], dim=0)
    return q


# --------------------------------------------------------------------------
# triangle attention
# --------------------------------------------------------------------------
def attention_core(q, k, v, biases):
    """attention.py:94-135.  q,k,v: [*, H, Q/K, c]; q already scaled."""
    s = torch.einsum("...qc,...kc->...qk", q, k)
    for bias in biases:
        s = s + bias
    s = torch.softmax(s, dim=-1)
    return torch.einsum("...qk,...kc->...qc", s.to(v.dtype), v)


def triattn_update(x, mask, p, no_heads: int, starting: bool = True, inf: float = INF,
                   row_chunk: int | None = None):
    """tri_att.py:102-167 + Attention.forward default branch (attention.py:366-413).

    x: [*, I, J, C]; mask: [*, I, J].  Returns the update only.
    ``row_chunk`` bounds the materialised logits by processing that many rows
    of I at a time; it changes no value (rows are independent).
    """
    if mask is None:
        mask = x.new_ones(x.shape[:-1])
    if not starting:
        x = x.transpose(-2, -3)
        mask = mask.transpose(-1, -2)
    xn = layer_norm(x, p["layer_norm.weight"], p["layer_norm.bias"])
    mask_bias = (inf * (mask.to(x.dtype) - 1))[..., :, None, None, :]  # [*, I, 1, 1, J]
    tb = linear(xn, p["linear_z.weight"])  # [*, I, J, H]
    nd = tb.dim()
    tb = tb.permute(list(range(nd - 3)) + [nd - 1, nd - 3, nd - 2])  # [*, H, I, J]
    tb = tb.unsqueeze(-4)  # [*, 1, H, I, J]

    H = no_heads
    n_rows = xn.shape[-3]
    step = n_rows if row_chunk is None else row_chunk
    outs = []
    for r0 in range(0, n_rows, step):
        xr = xn[..., r0:r0 + step, :, :]
        q = linear(xr, p["mha.linear_q.weight"])
        k = linear(xr, p["mha.linear_k.weight"])
        v = linear(xr, p["mha.linear_v.weight"])
        c = q.shape[-1] // H
        q = q.view(q.shape[:-1] + (H, c)).transpose(-2, -3)  # [*, I, H, J, c]
        k = k.view(k.shape[:-1] + (H, c)).transpose(-2, -3)
        v = v.view(v.shape[:-1] + (H, c)).transpose(-2, -3)
        q = q / math.sqrt(c)  # attention.py:283-284
        o = attention_core(q, k, v, [mask_bias[..., r0:r0 + step, :, :, :], tb])
        o = o.transpose(-2, -3)  # [*, I, J, H, c]
        g = torch.sigmoid(linear(xr, p["mha.linear_g.weight"]))
        g = g.view(g.shape[:-1] + (H, c))
        o = (o * g).reshape(o.shape[:-2] + (H * c,))
        outs.append(linear(o, p["mha.linear_o.weight"]))
    out = outs[0] if len(outs) == 1 else torch.cat(outs, dim=-3)
    if not starting:
        out = out.transpose(-2, -3)
    return out


# --------------------------------------------------------------------------
# pair transition (the step that follows the pair stack in every PairBlock)
# --------------------------------------------------------------------------
def transition_update(x, mask, p):
    """SwiGLUTransition.forward (transition.py:96-128, :261-271) with SwiGLU of
    activations.py:60-61: LayerNorm, silu(x Wa^T) * (x Wb^T), linear_out, times mask.
    x: [*, C]; mask: x.shape[:-1] or None (ones, transition.py:113-114).  Returns the update
    only; the caller adds it to z (base_blocks.py:470-478).  Parameter names as in the
    reference: layer_norm.{weight,bias}, swiglu.linear_a.weight, swiglu.linear_b.weight [n*C, C],
    linear_out.weight [C, n*C]."""
    if mask is None:
        mask = x.new_ones(x.shape[:-1])
    xn = layer_norm(x, p["layer_norm.weight"], p["layer_norm.bias"])
    a = linear(xn, p["swiglu.linear_a.weight"])
    b = linear(xn, p["swiglu.linear_b.weight"])
    h = torch.nn.functional.silu(a) * b
    return linear(h, p["linear_out.weight"]) * mask.to(x.dtype).unsqueeze(-1)


def pair_block(z, pair_mask, p, no_heads: int, row_chunk: int | None = None, mask_trans: bool = True):
    """PairBlock.forward in eval mode (base_blocks.py:408-480): the pair stack, then
    z + pair_transition(z, mask = pair_mask if _mask_trans else None).  ``p`` also holds the
    transition under the prefix pair_transition."""
    z = pair_stack_block(z, pair_mask, p, no_heads, row_chunk=row_chunk)
    return z + transition_update(z, pair_mask if mask_trans else None, _sub(p, "pair_transition."))


def pair_bias(z, p):
    """AttentionPairBias._prep_bias, pair part (attention_pair_bias.py:151-161): layer_norm_z,
    linear_z (no bias), permute_final_dims(z, [2, 0, 1]).  z [*, N, N, C] -> [*, H, N, N].
    Parameters: layer_norm_z.weight, layer_norm_z.bias (optional: LayerNorm without offset),
    linear_z.weight [H, C]."""
    bias = p.get("layer_norm_z.bias")
    if bias is None:
        bias = torch.zeros_like(p["layer_norm_z.weight"])
    zn = layer_norm(z, p["layer_norm_z.weight"], bias)
    out = linear(zn, p["linear_z.weight"])
    return out.movedim(-1, -3)


def attention_pair_bias(a, z, mask, p, no_heads: int, inf: float = INF):
    """AttentionPairBias.forward of the trunk (no AdaLN; attention_pair_bias.py:189-244) with
    Attention._prep_qkv / _attention / _wrap_up (attention.py:265-302, :94-135).

    a: [*, N, C_s]; z: [*, N, N, C_z]; mask: [*, N] or None.  Returns the update [*, N, C_s]
    (the caller adds it to s, pairformer.py:189-201).  Parameters under the reference's names:
    layer_norm_a.*, layer_norm_z.*, linear_z.weight, mha.linear_q.weight / .bias,
    mha.linear_k.weight, mha.linear_v.weight, mha.linear_g.weight, mha.linear_o.weight.
    """
    if mask is None:
        mask = a.new_ones(a.shape[:-1])
    an = layer_norm(a, p["layer_norm_a.weight"], p["layer_norm_a.bias"])
    mask_bias = (inf * (mask.to(a.dtype) - 1))[..., None, None, :]   # [*, 1, 1, N]
    zb = pair_bias(z, p)                                              # [*, H, N, N]
    c = p["mha.linear_q.weight"].shape[0] // no_heads

    def heads(t):  # [*, N, H*c] -> [*, H, N, c]
        return t.view(*t.shape[:-1], no_heads, c).transpose(-2, -3)

    q = heads(linear(an, p["mha.linear_q.weight"]) + p["mha.linear_q.bias"]) / math.sqrt(c)
    k = heads(linear(an, p["mha.linear_k.weight"]))
    v = heads(linear(an, p["mha.linear_v.weight"]))
    o = attention_core(q, k, v, [mask_bias, zb])                      # [*, H, N, c]
    o = o.transpose(-2, -3)                                           # [*, N, H, c]
    g = torch.sigmoid(linear(an, p["mha.linear_g.weight"]))
    o = o.reshape(*o.shape[:-2], no_heads * c) * g
    return linear(o, p["mha.linear_o.weight"])


def pairformer_block(s, z, single_mask, pair_mask, p, no_heads_pair: int, no_heads_pair_bias: int,
                     row_chunk: int | None = None, mask_trans: bool = True):
    """PairFormerBlock.forward (pairformer.py:124-215): z = pair_stack(z); s = s +
    attn_pair_bias(s, z, mask = single_mask); s = s + single_transition(s, mask = single_mask if
    _mask_trans).  ``p`` holds the three sub-modules under pair_stack. / attn_pair_bias. /
    single_transition.  Returns (s, z)."""
    z = pair_block(z, pair_mask, _sub(p, "pair_stack."), no_heads_pair, row_chunk=row_chunk, mask_trans=mask_trans)
    s = s + attention_pair_bias(s, z, single_mask, _sub(p, "attn_pair_bias."), no_heads_pair_bias)
    s = s + transition_update(s, single_mask if mask_trans else None, _sub(p, "single_transition."))
    return s, z


def make_pairformer_block_params(seed: int, c_s: int, c_z: int, c_hidden_mul: int, c_head_pair: int,
                                 no_heads_pair: int, c_head_bias: int, no_heads_bias: int, n: int):
    gen = torch.Generator().manual_seed(seed + 1000)
    p = {"pair_stack." + k: v for k, v in make_block_params(seed, c_z, c_hidden_mul, c_head_pair, no_heads_pair).items()}
    p.update({"pair_stack.pair_transition." + k: v for k, v in make_transition_params(gen, c_z, n).items()})
    p.update({"attn_pair_bias." + k: v
              for k, v in make_attention_pair_bias_params(gen, c_s, c_z, c_head_bias, no_heads_bias).items()})
    p.update({"single_transition." + k: v for k, v in make_transition_params(gen, c_s, n).items()})
    return p


def make_attention_pair_bias_params(gen, c_s: int, c_z: int, c_head: int, no_heads: int):
    hc = c_head * no_heads

    def lin(o, i):
        return torch.randn(o, i, generator=gen) / math.sqrt(i)

    p = {
        "layer_norm_a.weight": 1.0 + 0.1 * torch.randn(c_s, generator=gen),
        "layer_norm_a.bias": 0.1 * torch.randn(c_s, generator=gen),
        "mha.linear_q.weight": lin(hc, c_s),
        "mha.linear_q.bias": 0.1 * torch.randn(hc, generator=gen),
        "mha.linear_k.weight": lin(hc, c_s),
        "mha.linear_v.weight": lin(hc, c_s),
        "mha.linear_g.weight": lin(hc, c_s),
        "mha.linear_o.weight": lin(c_s, hc),
    }
    p.update(make_pair_bias_params(gen, c_z, no_heads))
    return p


def make_pair_bias_params(gen, c_z: int, no_heads: int, offset: bool = True):
    p = {
        "layer_norm_z.weight": 1.0 + 0.1 * torch.randn(c_z, generator=gen),
        "linear_z.weight": torch.randn(no_heads, c_z, generator=gen) / math.sqrt(c_z),
    }
    if offset:
        p["layer_norm_z.bias"] = 0.1 * torch.randn(c_z, generator=gen)
    return p


def make_transition_params(gen, c_in: int, n: int):
    def lin(o, i):
        return torch.randn(o, i, generator=gen) / math.sqrt(i)

    return {
        "layer_norm.weight": 1.0 + 0.1 * torch.randn(c_in, generator=gen),
        "layer_norm.bias": 0.1 * torch.randn(c_in, generator=gen),
        "swiglu.linear_a.weight": lin(n * c_in, c_in),
        "swiglu.linear_b.weight": lin(n * c_in, c_in),
        "linear_out.weight": lin(c_in, n * c_in),
    }


# --------------------------------------------------------------------------
# the same two updates restricted to a few output positions (for sizes at which
# the full fp32 evaluation does not finish in seconds); 3-D inputs only
# --------------------------------------------------------------------------
def trimul_update_at(z, mask, p, outgoing: bool, rows, cols):
    """trimul_update(z, mask, p, outgoing)[rows][:, cols] for z [N, N, C], computed from the
    2*(len(rows)+len(cols)) rows/columns of z the result depends on (tmu.py:77-82:
    outgoing x[i,j] contracts row i of a with row j of b, incoming column i with column j)."""
    rows = torch.as_tensor(rows)
    cols = torch.as_tensor(cols)
    if mask is None:
        mask = z.new_ones(z.shape[:-1])

    def gated(zs, ms, which):
        zn = layer_norm(zs, p["layer_norm_in.weight"], p["layer_norm_in.bias"])
        t = ms.to(z.dtype).unsqueeze(-1)
        t = t * torch.sigmoid(linear(zn, p["linear_%s_g.weight" % which]))
        return t * linear(zn, p["linear_%s_p.weight" % which])

    if outgoing:
        a = gated(z[rows], mask[rows], "a")                                  # [R, N(k), C]
        b = gated(z[cols], mask[cols], "b")                                  # [S, N(k), C]
    else:
        a = gated(z[:, rows].transpose(0, 1), mask[:, rows].transpose(0, 1), "a")   # a[k, i] -> [R, N(k), C]
        b = gated(z[:, cols].transpose(0, 1), mask[:, cols].transpose(0, 1), "b")
    x = torch.einsum("ikc,jkc->ijc", a, b)
    x = layer_norm(x, p["layer_norm_out.weight"], p["layer_norm_out.bias"])
    x = linear(x, p["linear_z.weight"])
    zn = layer_norm(z[rows][:, cols], p["layer_norm_in.weight"], p["layer_norm_in.bias"])
    return x * torch.sigmoid(linear(zn, p["linear_g.weight"]))


def triattn_update_rows(x, mask, p, no_heads: int, rows, starting: bool = True, inf: float = INF):
    """Rows ``rows`` of the module frame of triattn_update(x, mask, p, no_heads, starting) for
    x [N, N, C]: result[r] = update[rows[r], :, :] (starting) or update[:, rows[r], :]
    (ending).  Needs the triangle bias of the whole tensor but q, k, v of those rows only."""
    rows = torch.as_tensor(rows)
    if mask is None:
        mask = x.new_ones(x.shape[:-1])
    if not starting:
        x = x.transpose(0, 1)
        mask = mask.transpose(0, 1)
    H = no_heads
    tb = torch.empty(H, x.shape[0], x.shape[1], dtype=x.dtype)
    for r0 in range(0, x.shape[0], 256):  # linear_z(LayerNorm(x)) in slabs, [I, J, H] -> [H, I, J]
        xn = layer_norm(x[r0:r0 + 256], p["layer_norm.weight"], p["layer_norm.bias"])
        tb[:, r0:r0 + 256] = linear(xn, p["linear_z.weight"]).permute(2, 0, 1)
    xr = layer_norm(x[rows], p["layer_norm.weight"], p["layer_norm.bias"])   # [R, J, C]
    mask_bias = (inf * (mask[rows].to(x.dtype) - 1))[:, None, None, :]        # [R, 1, 1, J]
    q = linear(xr, p["mha.linear_q.weight"])
    k = linear(xr, p["mha.linear_k.weight"])
    v = linear(xr, p["mha.linear_v.weight"])
    c = q.shape[-1] // H
    q = q.view(q.shape[:-1] + (H, c)).transpose(-2, -3) / math.sqrt(c)
    k = k.view(k.shape[:-1] + (H, c)).transpose(-2, -3)
    v = v.view(v.shape[:-1] + (H, c)).transpose(-2, -3)
    o = attention_core(q, k, v, [mask_bias, tb.unsqueeze(0)]).transpose(-2, -3)  # [R, J, H, c]
    g = torch.sigmoid(linear(xr, p["mha.linear_g.weight"]))
    o = (o * g.view(g.shape[:-1] + (H, c))).reshape(o.shape[:-2] + (H * c,))
    return linear(o, p["mha.linear_o.weight"])


# --------------------------------------------------------------------------
# block sequencing
# --------------------------------------------------------------------------
def _sub(p, prefix):
    n = len(prefix)
    return {k[n:]: v for k, v in p.items() if k.startswith(prefix)}


def pair_stack_block(z, pair_mask, p, no_heads: int, row_chunk: int | None = None):
    """base_blocks.py:322-351 then :364-406 in eval mode (dropout = identity,
    dropout.py:57-58), out of place.  The pair transition (:470-478) is not
    part of this path.  ``p`` holds the four sub-modules under the reference's
    prefixes tri_mul_out. / tri_mul_in. / tri_att_start. / tri_att_end.
    """
    z = z + trimul_update(z, pair_mask, _sub(p, "tri_mul_out."), outgoing=True)
    z = z + trimul_update(z, pair_mask, _sub(p, "tri_mul_in."), outgoing=False)
    z = z + triattn_update(z, pair_mask, _sub(p, "tri_att_start."), no_heads,
                           starting=True, row_chunk=row_chunk)
    # the reference builds tri_att_end as a *starting* module and transposes
    # around the call (base_blocks.py:282-288, :380-404)
    zt = z.transpose(-2, -3)
    zt = zt + triattn_update(zt, pair_mask.transpose(-1, -2), _sub(p, "tri_att_end."),
                             no_heads, starting=True, row_chunk=row_chunk)
    return zt.transpose(-2, -3)


def template_pair_stack(t, mask, blocks, no_heads: int, row_chunk: int | None = None):
    """template_module.py:148-166 with tri_mul_first=True, for every block of
    ``blocks`` in turn: each template is an independent pair representation.
    t: [*, T, N, N, C]; mask: [*, T, N, N].  Pair transition and the final
    LayerNorm of the stack are outside this path.
    """
    outs = []
    for ti in range(t.shape[-4]):
        zt = t[..., ti, :, :, :]
        mt = mask[..., ti, :, :]
        for p in blocks:
            zt = pair_stack_block(zt, mt, p, no_heads, row_chunk=row_chunk)
        outs.append(zt.unsqueeze(-4))
    return torch.cat(outs, dim=-4)


def template_stack(t, mask, blocks, ln_weight, ln_bias, no_heads: int, row_chunk: int | None = None,
                   mask_trans: bool = True):
    """TemplatePairStack.forward (template_module.py:302-378): every template runs through every
    TemplatePairBlock (tri_mul_first=True: pair stack, then t + pair_transition(t),
    template_module.py:148-193), then the stack's LayerNorm.  t: [*, T, N, N, C]; mask: [*, T, N, N]
    or [*, 1, N, N] (expanded over the templates, template_module.py:326-329).  ``blocks`` holds one
    parameter dict per block with the PairBlock prefixes (tri_mul_out. ... pair_transition.).
    """
    if mask.shape[-3] == 1:
        mask = mask.expand(*mask.shape[:-3], t.shape[-4], *mask.shape[-2:])
    outs = []
    for ti in range(t.shape[-4]):
        zt = t[..., ti, :, :, :]
        mt = mask[..., ti, :, :]
        for p in blocks:
            zt = pair_block(zt, mt, p, no_heads, row_chunk=row_chunk, mask_trans=mask_trans)
        outs.append(zt.unsqueeze(-4))
    return layer_norm(torch.cat(outs, dim=-4), ln_weight, ln_bias)


def template_tail(t, linear_t_weight):
    """Tail of TemplateEmbedderAllAtom.forward (template_module.py:462-465): mean over the
    templates, ReLU, bias-free linear_t.  t: [*, T, N, N, C_t] (the stack's output) ->
    [*, N, N, C_z]."""
    u = torch.sum(t, dim=-4) / t.shape[-4]
    return linear(torch.relu(u), linear_t_weight)


def make_template_tail_params(gen, c_t: int, c_z: int):
    return {
        "template_pair_stack.layer_norm.weight": 1 + 0.1 * torch.randn(c_t, generator=gen),
        "template_pair_stack.layer_norm.bias": 0.1 * torch.randn(c_t, generator=gen),
        "linear_t.weight": torch.randn(c_z, c_t, generator=gen) / math.sqrt(c_t),
    }


# --------------------------------------------------------------------------
# seeded synthetic parameters / inputs (shared by tests, smoke and bench)
# --------------------------------------------------------------------------
def make_trimul_params(gen, c_z: int, c_hidden: int):
    def lin(o, i):
        return torch.randn(o, i, generator=gen) / math.sqrt(i)

    return {
        "layer_norm_in.weight": 1 + 0.1 * torch.randn(c_z, generator=gen),
        "layer_norm_in.bias": 0.1 * torch.randn(c_z, generator=gen),
        "layer_norm_out.weight": 1 + 0.1 * torch.randn(c_hidden, generator=gen),
        "layer_norm_out.bias": 0.1 * torch.randn(c_hidden, generator=gen),
        "linear_a_p.weight": lin(c_hidden, c_z),
        "linear_a_g.weight": lin(c_hidden, c_z),
        "linear_b_p.weight": lin(c_hidden, c_z),
        "linear_b_g.weight": lin(c_hidden, c_z),
        "linear_g.weight": lin(c_z, c_z),
        "linear_z.weight": lin(c_z, c_hidden),
    }


def make_triattn_params(gen, c_in: int, c_head: int, no_heads: int):
    def lin(o, i):
        return torch.randn(o, i, generator=gen) / math.sqrt(i)

    hc = c_head * no_heads
    return {
        "layer_norm.weight": 1 + 0.1 * torch.randn(c_in, generator=gen),
        "layer_norm.bias": 0.1 * torch.randn(c_in, generator=gen),
        "linear_z.weight": lin(no_heads, c_in),
        "mha.linear_q.weight": lin(hc, c_in),
        "mha.linear_k.weight": lin(hc, c_in),
        "mha.linear_v.weight": lin(hc, c_in),
        "mha.linear_g.weight": lin(hc, c_in),
        "mha.linear_o.weight": lin(c_in, hc),
    }


def make_block_params(seed: int, c_z: int, c_hidden_mul: int, c_head: int, no_heads: int):
    """Every hot-path Linear ~ N(0, 1/fan_in) (the reference's tests override
    the zero 'final'/'gating' inits the same way, tests/test_kernels.py:381-385);
    LayerNorm weight 1+0.1N, bias 0.1N so the affine terms are exercised."""
    gen = torch.Generator(device="cpu").manual_seed(seed)
    p = {}
    for name, outgoing in (("tri_mul_out.", True), ("tri_mul_in.", False)):
        for k, v in make_trimul_params(gen, c_z, c_hidden_mul).items():
            p[name + k] = v
    for name in ("tri_att_start.", "tri_att_end."):
        for k, v in make_triattn_params(gen, c_z, c_head, no_heads).items():
            p[name + k] = v
    return p


def make_pair_input(seed: int, batch_shape, n: int, c_z: int):
    gen = torch.Generator(device="cpu").manual_seed(seed)
    return torch.randn(*batch_shape, n, n, c_z, generator=gen)


def tail_padding_mask(batch_shape, n: int, n_pad):
    """pair_mask = outer(token_mask, token_mask) with the last n_pad tokens
    zeroed.  n_pad may be an int or a tensor shaped like batch_shape."""
    pad = torch.as_tensor(n_pad).expand(tuple(batch_shape)) if len(batch_shape) else torch.as_tensor(n_pad)
    idx = torch.arange(n)
    tok = (idx < (n - pad)[..., None]).to(torch.float32)
    return tok[..., :, None] * tok[..., None, :]


def round_bf16(t):
    return t.to(torch.bfloat16).to(torch.float32)
