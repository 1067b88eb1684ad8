"""Pins oracle/pairstack_oracle.py without the reference's code: float64 brute force on tiny
inputs, library routines (scaled_dot_product_attention), and algebraic invariants of the
path.  The reference holds no golden vectors for these modules (its own tests assert shapes
only), so these checks are what fixes the oracle."""
import math

import numpy as np
import pytest
import torch

from oracle import brute_force as bf
from oracle import pairstack_oracle as orc

FP32_TOL = 1e-4  # max-abs bound stated for fp32 in the build's north star


def _tiny(seed, n=6, c=8, ch=8, hd=4, heads=2):
    gen = torch.Generator().manual_seed(seed)
    z = torch.randn(n, n, c, generator=gen)
    mask = (torch.rand(n, n, generator=gen) > 0.3).float()
    mask[0, :] = 1.0
    tm = orc.make_trimul_params(gen, c, ch)
    ta = orc.make_triattn_params(gen, c, hd, heads)
    return z, mask, tm, ta, heads


@pytest.mark.parametrize("outgoing", [True, False])
@pytest.mark.parametrize("seed", [0, 1])
def test_trimul_matches_bruteforce(outgoing, seed):
    z, mask, tm, _, _ = _tiny(seed)
    got = orc.trimul_update(z, mask, tm, outgoing).double().numpy()
    want = bf.trimul_update(z, mask, tm, outgoing)
    assert np.abs(got - want).max() < FP32_TOL


@pytest.mark.parametrize("outgoing", [True, False])
def test_fused_trimul_matches_bruteforce(outgoing):
    """The fused-projection restatement (stacked a/b weights, cut after gating) against the float64 loops
    run on the two halves of the stacked weights; a swap of the halves (b on top) must lie far outside."""
    z, mask, tm, _, _ = _tiny(2)
    fused = orc.fuse_trimul_params(tm)
    assert fused["linear_ab_p.weight"].shape == (2 * tm["linear_a_p.weight"].shape[0], z.shape[-1])
    got = orc.fused_trimul_update(z, mask, fused, outgoing).double().numpy()
    want = bf.trimul_update(z, mask, tm, outgoing)
    assert np.abs(got - want).max() < FP32_TOL
    swapped = dict(tm, **{"linear_a_p.weight": tm["linear_b_p.weight"], "linear_b_p.weight": tm["linear_a_p.weight"],
                          "linear_a_g.weight": tm["linear_b_g.weight"], "linear_b_g.weight": tm["linear_a_g.weight"]})
    assert np.abs(bf.trimul_update(z, mask, swapped, outgoing) - want).max() > 1e-2


def test_trimul_outgoing_differs_from_incoming():
    # guards against the brute force and the oracle both ignoring the direction flag
    z, mask, tm, _, _ = _tiny(3)
    a = orc.trimul_update(z, mask, tm, True)
    b = orc.trimul_update(z, mask, tm, False)
    assert (a - b).abs().max() > 1e-2


@pytest.mark.parametrize("starting", [True, False])
@pytest.mark.parametrize("seed", [0, 1])
def test_triattn_matches_bruteforce(starting, seed):
    z, mask, _, ta, heads = _tiny(seed)
    got = orc.triattn_update(z, mask, ta, heads, starting=starting).double().numpy()
    want = bf.triattn_update(z, mask, ta, heads, starting=starting)
    assert np.abs(got - want).max() < FP32_TOL


def test_triattn_fully_masked_row_is_uniform_average():
    """A fully masked query row gives a uniform softmax over ALL keys (masked ones included):
    fl32(s - 1e9) == -1e9 for |s| < 32.  Output must equal gate * mean_k(v) projected."""
    z, mask, _, ta, heads = _tiny(5)
    mask[2, :] = 0.0
    got = orc.triattn_update(z, mask, ta, heads)
    want = bf.triattn_update(z, mask, ta, heads)
    assert np.abs(got.double().numpy() - want).max() < FP32_TOL
    xn = orc.layer_norm(z, ta["layer_norm.weight"], ta["layer_norm.bias"])
    v = orc.linear(xn[2], ta["mha.linear_v.weight"]).mean(0, keepdim=True)  # mean over keys
    g = torch.sigmoid(orc.linear(xn[2], ta["mha.linear_g.weight"]))
    manual = orc.linear(v * g, ta["mha.linear_o.weight"])
    assert (got[2] - manual).abs().max() < FP32_TOL


def test_triattn_partially_masked_key_has_zero_weight():
    z, mask, _, ta, heads = _tiny(6)
    mask[:] = 1.0
    mask[1, 3] = 0.0
    base = orc.triattn_update(z, mask, ta, heads)
    # changing what sits at a masked key of row 1 must not change row 1's own
    # attention values except through the (q, gate) of that very position: check the
    # other positions j != 3 of row 1, whose only dependence on z[1,3] is as a key
    # and as the source of the triangle-bias column k=3 of row q... both masked out for row 1
    z2 = z.clone()
    z2[1, 3] += 5.0
    pert = orc.triattn_update(z2, mask, ta, heads)
    keep = [j for j in range(z.shape[0]) if j != 3]
    assert (base[1, keep] - pert[1, keep]).abs().max() < 1e-6


def test_attention_core_is_sdpa():
    gen = torch.Generator().manual_seed(7)
    q = torch.randn(3, 2, 10, 8, generator=gen)
    k = torch.randn(3, 2, 10, 8, generator=gen)
    v = torch.randn(3, 2, 10, 8, generator=gen)
    b1 = -1e9 * (torch.rand(3, 1, 1, 10, generator=gen) > 0.7).float()
    b2 = torch.randn(1, 2, 10, 10, generator=gen)
    got = orc.attention_core(q / math.sqrt(8), k, v, [b1, b2])
    want = torch.nn.functional.scaled_dot_product_attention(q, k, v, attn_mask=b1 + b2, scale=1 / math.sqrt(8))
    assert (got - want).abs().max() < 1e-5


def test_contract_spellings_agree():
    gen = torch.Generator().manual_seed(8)
    a = torch.randn(2, 5, 5, 3, generator=gen)
    b = torch.randn(2, 5, 5, 3, generator=gen)
    assert torch.equal(orc.trimul_contract(a, b, True), torch.einsum("bikc,bjkc->bijc", a, b))
    assert torch.equal(orc.trimul_contract(a, b, False), torch.einsum("bkic,bkjc->bijc", a, b))


def test_trimul_symmetric_input_out_equals_in():
    z, mask, tm, _, _ = _tiny(9)
    z = z + z.transpose(0, 1)
    mask = mask * mask.t()
    o = orc.trimul_update(z, mask, tm, True)
    i = orc.trimul_update(z, mask, tm, False)
    assert (o - i).abs().max() < 1e-4


def test_trimul_zero_mask_closed_form():
    z, mask, tm, _, _ = _tiny(10)
    got = orc.trimul_update(z, torch.zeros_like(mask), tm, True)
    zn = orc.layer_norm(z, tm["layer_norm_in.weight"], tm["layer_norm_in.bias"])
    want = (tm["linear_z.weight"] @ tm["layer_norm_out.bias"]) * torch.sigmoid(orc.linear(zn, tm["linear_g.weight"]))
    assert (got - want).abs().max() < 1e-5


def test_zero_final_weights_give_zero_update():
    z, mask, tm, ta, heads = _tiny(11)
    tm = dict(tm)
    tm["linear_z.weight"] = torch.zeros_like(tm["linear_z.weight"])
    assert orc.trimul_update(z, mask, tm, True).abs().max() == 0
    ta = dict(ta)
    ta["mha.linear_o.weight"] = torch.zeros_like(ta["mha.linear_o.weight"])
    assert orc.triattn_update(z, mask, ta, heads).abs().max() == 0


def test_ending_node_is_start_on_transpose():
    z, mask, _, ta, heads = _tiny(12)
    end = orc.triattn_update(z, mask, ta, heads, starting=False)
    via = orc.triattn_update(z.transpose(0, 1), mask.t(), ta, heads, starting=True).transpose(0, 1)
    assert torch.equal(end, via)


def test_row_chunking_changes_nothing():
    z, mask, _, ta, heads = _tiny(13)
    a = orc.triattn_update(z, mask, ta, heads)
    b = orc.triattn_update(z, mask, ta, heads, row_chunk=4)
    assert (a - b).abs().max() < 1e-6


def test_block_sequence_matches_bruteforce():
    n, c, hd, heads = 5, 8, 4, 2
    p = orc.make_block_params(3, c, 8, hd, heads)
    z = orc.make_pair_input(4, (), n, c)
    mask = orc.tail_padding_mask((), n, 1)
    got = orc.pair_stack_block(z[None], mask[None], p, heads)[0].double().numpy()
    w = z.double().numpy()
    w = w + bf.trimul_update(w, mask, orc._sub(p, "tri_mul_out."), True)
    w = w + bf.trimul_update(w, mask, orc._sub(p, "tri_mul_in."), False)
    w = w + bf.triattn_update(w, mask, orc._sub(p, "tri_att_start."), heads, starting=True)
    w = w + bf.triattn_update(w, mask, orc._sub(p, "tri_att_end."), heads, starting=False)
    assert np.abs(got - w).max() < 5e-4


def test_template_stack_is_per_template_blocks():
    n, c, hd, heads = 4, 8, 4, 2
    blocks = [orc.make_block_params(s, c, 8, hd, heads) for s in (1, 2)]
    t = orc.make_pair_input(5, (1, 3), n, c)
    mask = orc.tail_padding_mask((1, 3), n, torch.tensor([[0, 1, 2]]))
    got = orc.template_pair_stack(t, mask, blocks, heads)
    for ti in range(3):
        zt = t[:, ti]
        for p in blocks:
            zt = orc.pair_stack_block(zt, mask[:, ti], p, heads)
        assert torch.equal(got[:, ti], zt)


# ---- the position-restricted forms used at sizes the full oracle cannot reach -----------------
@pytest.mark.parametrize("outgoing", [True, False])
def test_trimul_update_at_equals_full(outgoing):
    gen = torch.Generator().manual_seed(21)
    n, c = 12, 16
    z = torch.randn(n, n, c, generator=gen)
    mask = (torch.rand(n, n, generator=gen) > 0.2).float()
    p = orc.make_trimul_params(gen, c, c)
    rows, cols = [0, 5, 11], [2, 3, 7, 10]
    full = orc.trimul_update(z, mask, p, outgoing)
    part = orc.trimul_update_at(z, mask, p, outgoing, rows, cols)
    assert (part - full[rows][:, cols]).abs().max() < 1e-5


@pytest.mark.parametrize("starting", [True, False])
def test_triattn_update_rows_equals_full(starting):
    gen = torch.Generator().manual_seed(22)
    n, c, heads, d = 12, 16, 2, 4
    x = torch.randn(n, n, c, generator=gen)
    mask = (torch.rand(n, n, generator=gen) > 0.2).float()
    mask[4, :] = 0.0
    mask[:, 6] = 0.0
    p = orc.make_triattn_params(gen, c, d, heads)
    rows = [0, 4, 6, 11]
    full = orc.triattn_update(x, mask, p, heads, starting=starting)
    part = orc.triattn_update_rows(x, mask, p, heads, rows, starting=starting)
    want = full[rows] if starting else full[:, rows].transpose(0, 1)
    assert (part - want).abs().max() < 1e-5


# ---- pair transition ---------------------------------------------------------------------------
def test_transition_matches_bruteforce():
    gen = torch.Generator().manual_seed(31)
    n, c, mult = 5, 8, 4
    x = torch.randn(n, n, c, generator=gen)
    mask = (torch.rand(n, n, generator=gen) > 0.3).float()
    p = orc.make_transition_params(gen, c, mult)
    got = orc.transition_update(x, mask, p).double().numpy()
    assert np.abs(got - bf.transition_update(x, mask, p)).max() < FP32_TOL
    got = orc.transition_update(x, None, p).double().numpy()
    assert np.abs(got - bf.transition_update(x, None, p)).max() < FP32_TOL


def test_transition_invariants():
    gen = torch.Generator().manual_seed(32)
    c, mult = 16, 2
    x = torch.randn(3, 7, 7, c, generator=gen)
    mask = (torch.rand(3, 7, 7, generator=gen) > 0.5).float()
    p = orc.make_transition_params(gen, c, mult)
    out = orc.transition_update(x, mask, p)
    assert out.shape == x.shape
    assert (out[mask == 0] == 0).all()                      # masked positions give exactly 0
    q = dict(p)
    q["linear_out.weight"] = torch.zeros_like(p["linear_out.weight"])   # the shipped "final" init
    assert orc.transition_update(x, mask, q).abs().max() == 0
    q = dict(p)
    q["swiglu.linear_a.weight"] = torch.zeros_like(p["swiglu.linear_a.weight"])  # silu(0) = 0
    assert orc.transition_update(x, mask, q).abs().max() == 0
    # position-wise: permuting positions permutes the result
    perm = torch.randperm(7, generator=gen)
    assert torch.allclose(orc.transition_update(x[:, perm], mask[:, perm], p), out[:, perm], atol=1e-6)
    # swiglu against the library's own gated form: silu(a) * b == a * sigmoid(a) * b
    xn = orc.layer_norm(x, p["layer_norm.weight"], p["layer_norm.bias"])
    a = orc.linear(xn, p["swiglu.linear_a.weight"])
    b = orc.linear(xn, p["swiglu.linear_b.weight"])
    want = orc.linear(a * torch.sigmoid(a) * b, p["linear_out.weight"]) * mask.unsqueeze(-1)
    assert torch.allclose(out, want, atol=1e-6)


# ---- pair-bias projection ----------------------------------------------------------------------
def test_pair_bias_matches_bruteforce_and_library_routines():
    gen = torch.Generator().manual_seed(41)
    n, c, h = 6, 16, 5
    z = torch.randn(n, n, c, generator=gen)
    for offset in (True, False):
        p = orc.make_pair_bias_params(gen, c, h, offset=offset)
        got = orc.pair_bias(z, p)
        assert got.shape == (h, n, n)
        assert np.abs(got.double().numpy() - bf.pair_bias(z, p)).max() < FP32_TOL
        zn = torch.nn.functional.layer_norm(z, (c,), p["layer_norm_z.weight"], p.get("layer_norm_z.bias"), 1e-5)
        want = torch.nn.functional.linear(zn, p["linear_z.weight"]).permute(2, 0, 1)
        assert (got - want).abs().max() < FP32_TOL


def test_pair_bias_invariants():
    gen = torch.Generator().manual_seed(42)
    c, h = 32, 4
    z = torch.randn(2, 9, 9, c, generator=gen)
    p = orc.make_pair_bias_params(gen, c, h)
    out = orc.pair_bias(z, p)
    assert out.shape == (2, h, 9, 9)
    # LayerNorm makes the result invariant to a per-position shift and positive scale of z
    assert (orc.pair_bias(3.0 * z + 5.0, p) - out).abs().max() < 1e-4
    # head h of the output only depends on row h of the weight; a transposed input gives the transposed bias
    q = dict(p)
    q["linear_z.weight"] = p["linear_z.weight"].clone()
    q["linear_z.weight"][1] = 0
    o2 = orc.pair_bias(z, q)
    assert o2[:, 1].abs().max() == 0 and torch.equal(o2[:, 0], out[:, 0])
    assert torch.equal(orc.pair_bias(z.transpose(-2, -3), p), out.transpose(-1, -2))


def test_template_tail_matches_bruteforce_and_library_routines():
    gen = torch.Generator().manual_seed(51)
    nt, n, c_t, c_z = 3, 5, 16, 24
    t = torch.randn(nt, n, n, c_t, generator=gen)
    p = orc.make_template_tail_params(gen, c_t, c_z)
    g, b, w = p["template_pair_stack.layer_norm.weight"], p["template_pair_stack.layer_norm.bias"], p["linear_t.weight"]
    got = orc.template_tail(orc.layer_norm(t, g, b), w)
    assert got.shape == (n, n, c_z)
    assert np.abs(got.double().numpy() - bf.template_tail(t, g, b, w)).max() < FP32_TOL
    tn = torch.nn.functional.layer_norm(t, (c_t,), g, b, 1e-5)
    want = torch.nn.functional.linear(torch.relu(tn.mean(dim=0)), w)
    assert (got - want).abs().max() < FP32_TOL
    # a template whose normalised features are all negative contributes nothing after the ReLU
    # only through the mean: one template alone equals relu(LN) @ W^T
    one = orc.template_tail(orc.layer_norm(t[:1], g, b), w)
    assert (one - torch.nn.functional.linear(torch.relu(tn[0]), w)).abs().max() < FP32_TOL
    # permuting the templates changes nothing (a mean), up to summation order
    assert (orc.template_tail(orc.layer_norm(t.flip(0), g, b), w) - got).abs().max() < 1e-5


def test_template_stack_is_blocks_then_layer_norm():
    """template_stack = per-template PairBlocks (already pinned) followed by LayerNorm; a mask
    given once ([1, N, N]) is the same mask for every template."""
    gen = torch.Generator().manual_seed(52)
    nt, n, c = 2, 7, 16
    blocks = []
    for seed in (3, 4):
        p = orc.make_block_params(seed, c, c, 4, 4)
        p.update({"pair_transition." + k: v for k, v in orc.make_transition_params(gen, c, 2).items()})
        blocks.append(p)
    t = orc.make_pair_input(53, (nt,), n, c)
    mask = orc.tail_padding_mask((nt,), n, torch.tensor([0, 2]))
    g = 1 + 0.1 * torch.randn(c, generator=gen)
    b = 0.1 * torch.randn(c, generator=gen)
    got = orc.template_stack(t, mask, blocks, g, b, 4)
    for ti in range(nt):
        z = t[ti]
        for p in blocks:
            z = orc.pair_block(z, mask[ti], p, 4)
        want = torch.nn.functional.layer_norm(z, (c,), g, b, 1e-5)
        assert (got[ti] - want).abs().max() < FP32_TOL
    shared = orc.tail_padding_mask((1,), n, 2)
    a = orc.template_stack(t, shared, blocks, g, b, 4)
    bb = orc.template_stack(t, shared.expand(nt, n, n), blocks, g, b, 4)
    assert torch.equal(a, bb)


def test_attention_pair_bias_matches_bruteforce_and_sdpa():
    gen = torch.Generator().manual_seed(61)
    n, cs, cz, c, h = 7, 24, 16, 6, 4
    p = orc.make_attention_pair_bias_params(gen, cs, cz, c, h)
    a = torch.randn(n, cs, generator=gen)
    z = torch.randn(n, n, cz, generator=gen)
    mask = torch.tensor([1, 1, 0, 1, 1, 1, 0.0])
    got = orc.attention_pair_bias(a, z, mask, p, h)
    assert got.shape == (n, cs)
    assert np.abs(got.double().numpy() - bf.attention_pair_bias(a, z, mask, p, h)).max() < FP32_TOL
    assert np.abs(orc.attention_pair_bias(a, z, None, p, h).double().numpy()
                  - bf.attention_pair_bias(a, z, None, p, h)).max() < FP32_TOL
    # the same through torch's scaled_dot_product_attention (its own 1/sqrt(c) scaling)
    F = torch.nn.functional
    an = F.layer_norm(a, (cs,), p["layer_norm_a.weight"], p["layer_norm_a.bias"], 1e-5)
    heads = lambda t: t.view(n, h, c).transpose(0, 1)  # noqa: E731
    q = heads(F.linear(an, p["mha.linear_q.weight"], p["mha.linear_q.bias"]))
    k, v = heads(F.linear(an, p["mha.linear_k.weight"])), heads(F.linear(an, p["mha.linear_v.weight"]))
    bias = orc.pair_bias(z, p) + (1e9 * (mask - 1))[None, None, :]
    o = F.scaled_dot_product_attention(q, k, v, attn_mask=bias).transpose(0, 1).reshape(n, h * c)
    want = F.linear(o * torch.sigmoid(F.linear(an, p["mha.linear_g.weight"])), p["mha.linear_o.weight"])
    assert (got - want).abs().max() < FP32_TOL


def test_attention_pair_bias_invariants():
    gen = torch.Generator().manual_seed(62)
    n, cs, cz, c, h = 9, 32, 16, 8, 4
    p = orc.make_attention_pair_bias_params(gen, cs, cz, c, h)
    a = torch.randn(2, n, cs, generator=gen)
    z = torch.randn(2, n, n, cz, generator=gen)
    mask = torch.ones(2, n)
    mask[1, -3:] = 0
    out = orc.attention_pair_bias(a, z, mask, p, h)
    # a masked key does not influence any query: changing its features changes nothing but its own row
    a2 = a.clone()
    a2[1, -1] += 3.0
    out2 = orc.attention_pair_bias(a2, z, mask, p, h)
    assert (out2[1, :-1] - out[1, :-1]).abs().max() < 1e-5 and (out2[0] - out[0]).abs().max() == 0
    # a bias constant along the keys cancels in the softmax: adding a per-query shift to z's projection
    q = dict(p)
    q["mha.linear_o.weight"] = torch.zeros_like(p["mha.linear_o.weight"])
    assert orc.attention_pair_bias(a, z, mask, q, h).abs().max() == 0
    # batch elements are independent
    assert (orc.attention_pair_bias(a[:1], z[:1], mask[:1], p, h) - out[:1]).abs().max() < 1e-6
    # a fully masked sequence degenerates to the uniform average of v (all logits shifted alike)
    m0 = torch.zeros(1, n)
    o0 = orc.attention_pair_bias(a[:1], torch.zeros(1, n, n, cz), m0, p, h)
    o1 = orc.attention_pair_bias(a[:1], torch.zeros(1, n, n, cz), torch.ones(1, n), p, h)
    assert torch.isfinite(o0).all() and o0.shape == o1.shape


def _brute_pair_block(z, mask, p, heads, mask_trans=True):
    """PairBlock (base_blocks.py:408-480) as a float64 composition of the brute-force pieces."""
    w = z.double().numpy()
    w = w + bf.trimul_update(w, mask, orc._sub(p, "tri_mul_out."), True)
    w = w + bf.trimul_update(w, mask, orc._sub(p, "tri_mul_in."), False)
    w = w + bf.triattn_update(w, mask, orc._sub(p, "tri_att_start."), heads, starting=True)
    w = w + bf.triattn_update(w, mask, orc._sub(p, "tri_att_end."), heads, starting=False)
    return w + bf.transition_update(w, mask if mask_trans else None, orc._sub(p, "pair_transition."))


@pytest.mark.parametrize("mask_trans", [True, False])
def test_pair_block_matches_bruteforce_composition(mask_trans):
    """orc.pair_block = the four triangle updates, then z + transition(z, mask or None): the order
    of the modules, the residual adds and the _mask_trans switch against an independent float64
    composition."""
    n, c, hd, heads = 5, 8, 4, 2
    p = orc.make_block_params(7, c, 8, hd, heads)
    gen = torch.Generator().manual_seed(71)
    p.update({"pair_transition." + k: v for k, v in orc.make_transition_params(gen, c, 2).items()})
    z = orc.make_pair_input(8, (), n, c)
    mask = orc.tail_padding_mask((), n, 1)
    got = orc.pair_block(z, mask, p, heads, mask_trans=mask_trans).double().numpy()
    want = _brute_pair_block(z, mask, p, heads, mask_trans)
    assert np.abs(got - want).max() < 5e-4
    # the switch matters on this input (masked positions keep the transition's update without it)
    other = _brute_pair_block(z, mask, p, heads, not mask_trans)
    assert np.abs(want - other).max() > 1e-2


@pytest.mark.parametrize("mask_trans", [True, False])
def test_pairformer_block_matches_bruteforce_composition(mask_trans):
    """orc.pairformer_block (pairformer.py:176-213): z through the PairBlock first, then
    s += attn_pair_bias(s, z_new, single_mask), s += single_transition(s, single_mask or None).
    A composition that fed the old z into the attention, dropped a residual or swapped the two
    single-representation updates differs by far more than the bound."""
    n, cs, cz, hd, heads, cb, hb = 5, 12, 8, 4, 2, 3, 4
    p = orc.make_pairformer_block_params(5, cs, cz, 8, hd, heads, cb, hb, 2)
    gen = torch.Generator().manual_seed(72)
    s = torch.randn(n, cs, generator=gen)
    z = orc.make_pair_input(9, (), n, cz)
    single_mask = torch.tensor([1, 1, 1, 0, 1.0])
    pair_mask = single_mask[:, None] * single_mask[None, :]
    s_got, z_got = orc.pairformer_block(s, z, single_mask, pair_mask, p, heads, hb, mask_trans=mask_trans)
    zw = _brute_pair_block(z, pair_mask, orc._sub(p, "pair_stack."), heads, mask_trans)
    sw = s.double().numpy()
    sw = sw + bf.attention_pair_bias(sw, zw, single_mask, orc._sub(p, "attn_pair_bias."), hb)
    sw = sw + bf.transition_update(sw, single_mask if mask_trans else None, orc._sub(p, "single_transition."))
    assert np.abs(z_got.double().numpy() - zw).max() < 5e-4
    assert np.abs(s_got.double().numpy() - sw).max() < 5e-4
    # the attention must see the updated z: with the input z the result moves visibly
    s_old = s.double().numpy() + bf.attention_pair_bias(s.double().numpy(), z.double().numpy(), single_mask,
                                                        orc._sub(p, "attn_pair_bias."), hb)
    s_new = s.double().numpy() + bf.attention_pair_bias(s.double().numpy(), zw, single_mask,
                                                        orc._sub(p, "attn_pair_bias."), hb)
    assert np.abs(s_old - s_new).max() > 1e-3
