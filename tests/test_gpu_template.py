"""Parity of the template branch (TemplatePairStack / TemplateEmbedderCore modules -> C ABI ->
HIP) with the CPU oracle on the same seeded inputs and weights.

bf16: max-norm 2e-2 and rms 5e-3 relative to the oracle's output, and at most 1.5x the rms error
of the oracle's own operations executed in bfloat16 where that floor is computed.  fp32: max-abs
1e-4."""
import pytest
import torch

from gpu_util import lib, report, stream, record_parity  # noqa: F401
from oracle import pairstack_oracle as orc

import of3pair
from of3pair import _lib as L
from of3pair import functional as F3

pytestmark = pytest.mark.gpu
DEV = "cuda"
REL = 2e-2

STACK_CFG = dict(c_t=64, c_hidden_tri_att=16, c_hidden_tri_mul=64, no_blocks=2, no_heads=4,
                 transition_type="swiglu", pair_transition_n=2, dropout_rate=0.25, tri_mul_first=True,
                 fuse_projection_weights=False, blocks_per_ckpt=None, inf=1e9, use_reentrant=False,
                 tune_chunk_size=False)


def _check(name, got, want, rms_rel=5e-3, bf16_ref=None):
    got = got.float().cpu()
    want = want.float()
    record_parity(name, got, want, bf16_ref, "max|err| <= 2e-2 max|want|, rms_rel <= %.1e%s" % (
        rms_rel, ", floor <= 1.5" if bf16_ref is not None else ""))
    rms = float(want.pow(2).mean().sqrt())
    report(name, got, want, atol=REL * float(want.abs().max()), rtol=0.0)
    erms = float((got - want).pow(2).mean().sqrt())
    assert erms <= rms_rel * rms, "%s: rms error %.3g vs rms %.3g" % (name, erms, rms)
    if bf16_ref is not None:
        floor = float((bf16_ref.float() - want).pow(2).mean().sqrt())
        assert erms <= 1.5 * floor, "%s: rms error %.3g above the bf16 reference path's %.3g" % (name, erms, floor)


def _tail_bf16_reference(t, p):
    """The oracle's operations with every tensor in bfloat16, as the reference's bf16 path runs them."""
    b = {k: v.to(torch.bfloat16) for k, v in p.items()}
    tn = orc.layer_norm(t.to(torch.bfloat16), b["template_pair_stack.layer_norm.weight"],
                        b["template_pair_stack.layer_norm.bias"])
    return orc.template_tail(tn, b["linear_t.weight"])


# positions P = N*N cover: one partial wave (N=3), ragged last tile (N=21: 441 = 256 + 185),
# more tiles than work-groups fit at once per batch element (N=96 with a batch of 2)
@pytest.mark.parametrize("n,nt,batch", [(3, 1, ()), (21, 4, ()), (40, 2, (2,)), (96, 3, (2,)), (64, 4, (1, 2))])
def test_template_tail_bf16(n, nt, batch):
    lib()
    gen = torch.Generator().manual_seed(700 + n)
    p = {k: orc.round_bf16(v) for k, v in orc.make_template_tail_params(gen, 64, 128).items()}
    t = orc.round_bf16(2.0 * torch.randn(*batch, nt, n, n, 64, generator=gen) + 0.3)
    g, b, w = p["template_pair_stack.layer_norm.weight"], p["template_pair_stack.layer_norm.bias"], p["linear_t.weight"]
    print("template tail", n, nt, batch, flush=True)
    tg = t.to(DEV).to(torch.bfloat16)
    got = F3.template_tail(tg, g.to(DEV), b.to(DEV), w.to(DEV))
    assert got.shape == (*batch, n, n, 128) and got.dtype == torch.bfloat16
    want = orc.template_tail(orc.layer_norm(t, g, b), w)
    _check("template tail", got, want, bf16_ref=_tail_bf16_reference(t, p))
    # the two-step form (closing LayerNorm as its own kernel, then the tail without it)
    tn = F3.layer_norm(tg, g.to(DEV), b.to(DEV))
    _check("stack layer norm", tn, orc.layer_norm(t, g, b), rms_rel=4e-3)
    got2 = F3.template_tail(tn, None, None, w.to(DEV), apply_layer_norm=False)
    assert torch.equal(got2, got), "fused and two-step tails must round alike"
    assert torch.equal(tg.float().cpu(), t), "the input must not be touched"


def test_layer_norm_c128_and_odd_row_counts():
    lib()
    gen = torch.Generator().manual_seed(71)
    for c, rows in ((128, 1), (128, 1000), (64, 7), (64, 4099)):
        x = orc.round_bf16(3.0 * torch.randn(rows, c, generator=gen) - 1.0)
        g = orc.round_bf16(1 + 0.1 * torch.randn(c, generator=gen))
        b = orc.round_bf16(0.1 * torch.randn(c, generator=gen))
        got = F3.layer_norm(x.to(DEV).to(torch.bfloat16), g.to(DEV), b.to(DEV))
        _check("layer norm %dx%d" % (rows, c), got, orc.layer_norm(x, g, b), rms_rel=4e-3)


@pytest.mark.parametrize("n,nt,c_t,c_z", [(9, 3, 64, 128), (17, 2, 48, 40)])
def test_template_tail_fp32(n, nt, c_t, c_z):
    lib()
    gen = torch.Generator().manual_seed(720 + n)
    p = orc.make_template_tail_params(gen, c_t, c_z)
    t = 2.0 * torch.randn(2, nt, n, n, c_t, generator=gen) + 0.3
    g, b, w = p["template_pair_stack.layer_norm.weight"], p["template_pair_stack.layer_norm.bias"], p["linear_t.weight"]
    got = F3.template_tail(t.to(DEV), g.to(DEV), b.to(DEV), w.to(DEV))
    want = orc.template_tail(orc.layer_norm(t, g, b), w)
    report("template tail fp32", got.cpu(), want, atol=1e-4, rtol=0.0)
    tn = F3.layer_norm(t.to(DEV), g.to(DEV), b.to(DEV))
    report("layer norm fp32", tn.cpu(), orc.layer_norm(t, g, b), atol=1e-4, rtol=0.0)
    got2 = F3.template_tail(tn, None, None, w.to(DEV), apply_layer_norm=False)
    report("template tail fp32, two steps", got2.cpu(), want, atol=1e-4, rtol=0.0)


def _stack_params(gen, n_blocks, c=64):
    blocks = []
    for seed in range(n_blocks):
        p = {k: orc.round_bf16(v) for k, v in orc.make_block_params(30 + seed, c, c, 16, 4).items()}
        p.update({"pair_transition." + k: orc.round_bf16(v) for k, v in orc.make_transition_params(gen, c, 2).items()})
        blocks.append(p)
    return blocks


def _load_stack(stack, blocks, tail):
    sd = {}
    for i, p in enumerate(blocks):
        sd.update({"blocks.%d.%s" % (i, k): v for k, v in p.items()})
    sd["layer_norm.weight"] = tail["template_pair_stack.layer_norm.weight"]
    sd["layer_norm.bias"] = tail["template_pair_stack.layer_norm.bias"]
    stack.load_state_dict(sd, strict=True)


@pytest.mark.parametrize("mask_trans", [True, False])
def test_template_pair_stack_module(mask_trans):
    """TemplatePairStack.forward: 2 blocks over 3 templates (each with its own padded tail), then
    the closing LayerNorm; the input is left intact without inplace_safe."""
    lib()
    n, nt = 72, 3
    gen = torch.Generator().manual_seed(73)
    blocks = _stack_params(gen, 2)
    tail = {k: orc.round_bf16(v) for k, v in orc.make_template_tail_params(gen, 64, 128).items()}
    t = orc.round_bf16(orc.make_pair_input(74, (nt,), n, 64))
    mask = orc.tail_padding_mask((nt,), n, torch.tensor([0, 5, 17]))
    stack = of3pair.TemplatePairStack(**STACK_CFG)
    _load_stack(stack, blocks, tail)
    stack = stack.to(DEV).to(torch.bfloat16).eval()
    tg = t.to(DEV).to(torch.bfloat16)
    print("template pair stack", mask_trans, flush=True)
    got = stack(tg, mask.to(DEV), chunk_size=4, _mask_trans=mask_trans)
    want = orc.template_stack(t, mask, blocks, tail["template_pair_stack.layer_norm.weight"],
                              tail["template_pair_stack.layer_norm.bias"], 4, mask_trans=mask_trans)
    _check("template pair stack", got, want, rms_rel=1.5e-2)
    assert torch.equal(tg.float().cpu(), t)
    got2 = stack(tg.clone(), mask.to(DEV), inplace_safe=True, _mask_trans=mask_trans)
    assert torch.equal(got2, got)


def test_template_embedder_core_with_shared_mask():
    """TemplateEmbedderCore.forward = template_module.py:447-467 after the feature embedding: one
    pair mask for all templates, stack, mean, ReLU, linear_t; a batch dimension in front."""
    lib()
    n, nt = 48, 4
    gen = torch.Generator().manual_seed(75)
    blocks = _stack_params(gen, 2)
    tail = {k: orc.round_bf16(v) for k, v in orc.make_template_tail_params(gen, 64, 128).items()}
    emb = orc.round_bf16(orc.make_pair_input(76, (2, nt), n, 64))
    pair_mask = orc.tail_padding_mask((2,), n, torch.tensor([0, 7]))
    core = of3pair.TemplateEmbedderCore(64, 128, STACK_CFG)
    _load_stack(core.template_pair_stack, blocks, tail)
    core.linear_t.weight.data.copy_(tail["linear_t.weight"])
    core = core.to(DEV).to(torch.bfloat16).eval()
    got = core(emb.to(DEV).to(torch.bfloat16), pair_mask.to(DEV))
    assert got.shape == (2, n, n, 128)
    tn = orc.template_stack(emb, pair_mask[:, None], blocks, tail["template_pair_stack.layer_norm.weight"],
                            tail["template_pair_stack.layer_norm.bias"], 4)
    want = orc.template_tail(tn, tail["linear_t.weight"])
    _check("template embedder core", got, want, rms_rel=1.5e-2)


def test_template_tail_full_size_rows():
    """Template shape of the benchmark configurations (4 templates, N = 384, c_t = 64 -> c_z = 128): the tail is
    position-wise, so the oracle evaluates sampled rows of the same input; every output is finite."""
    lib()
    n, nt = 384, 4
    gen = torch.Generator().manual_seed(77)
    p = {k: orc.round_bf16(v) for k, v in orc.make_template_tail_params(gen, 64, 128).items()}
    g, b, w = p["template_pair_stack.layer_norm.weight"], p["template_pair_stack.layer_norm.bias"], p["linear_t.weight"]
    gg = torch.Generator(device=DEV).manual_seed(78)
    tg = (2.0 * torch.randn(nt, n, n, 64, device=DEV, generator=gg)).to(torch.bfloat16)
    got = F3.template_tail(tg, g.to(DEV), b.to(DEV), w.to(DEV))
    assert torch.isfinite(got).all()
    rows = [0, 191, 383]
    t_rows = tg[:, rows].float().cpu()
    want = orc.template_tail(orc.layer_norm(t_rows, g, b), w)
    _check("template tail rows at N=384", got[rows], want)


def test_template_tail_rejects_unsupported():
    lib()
    t = torch.zeros(2, 8, 8, 320, device=DEV, dtype=torch.bfloat16)  # c_t = 320: beyond the fp32 kernels too
    with pytest.raises(ValueError):
        F3.template_tail(t, torch.ones(320, device=DEV), torch.zeros(320, device=DEV), torch.zeros(128, 320, device=DEV))
    with pytest.raises(ValueError):
        F3.layer_norm(torch.zeros(4, 320, device=DEV, dtype=torch.bfloat16), torch.ones(320, device=DEV),
                      torch.zeros(320, device=DEV))


def test_template_tail_and_layer_norm_bf16_widths_outside_the_bf16_kernels():
    """c_t = 32 -> c_z = 96 and a LayerNorm over 96 channels in bf16: the fp32 kernels on widened activations,
    rounded to bf16 once."""
    lib()
    gen = torch.Generator().manual_seed(79)
    p = {k: orc.round_bf16(v) for k, v in orc.make_template_tail_params(gen, 32, 96).items()}
    g, b, w = p["template_pair_stack.layer_norm.weight"], p["template_pair_stack.layer_norm.bias"], p["linear_t.weight"]
    t = orc.round_bf16(torch.randn(3, 17, 17, 32, generator=gen))
    got = F3.template_tail(t.to(DEV).to(torch.bfloat16), g.to(DEV), b.to(DEV), w.to(DEV))
    assert got.dtype == torch.bfloat16 and tuple(got.shape) == (17, 17, 96)
    _check("template tail, bf16 through fp32", got, orc.template_tail(orc.layer_norm(t, g, b), w))
    gen = torch.Generator().manual_seed(80)
    x = orc.round_bf16(2.0 * torch.randn(11, 96, generator=gen) + 0.5)
    gw, gb = orc.round_bf16(1 + 0.1 * torch.randn(96, generator=gen)), orc.round_bf16(0.1 * torch.randn(96, generator=gen))
    got = F3.layer_norm(x.to(DEV).to(torch.bfloat16), gw.to(DEV), gb.to(DEV))
    assert got.dtype == torch.bfloat16
    _check("layer norm, bf16 through fp32", got, orc.layer_norm(x, gw, gb))
