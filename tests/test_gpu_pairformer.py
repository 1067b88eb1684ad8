"""Parity of the single-representation transition and of whole PairFormerBlocks / a PairFormerStack
(modules -> C ABI -> HIP) with the CPU oracle on the same seeded inputs and weights.  bf16:
max-norm 2e-2 relative to the oracle's output plus an rms bound per case."""
import pytest
import torch

from gpu_util import lib, report, record_parity  # noqa: F401
from oracle import pairstack_oracle as orc

import of3pair
from of3pair import functional as F3

pytestmark = pytest.mark.gpu
DEV = "cuda"
REL = 2e-2
CFG = dict(c_s=384, c_z=128, c_hidden_pair_bias=24, no_heads_pair_bias=16, c_hidden_mul=128, c_hidden_pair_att=32,
           no_heads_pair=4, transition_type="swiglu", transition_n=4, pair_dropout=0.25,
           fuse_projection_weights=False, inf=1e9)


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


def _round(p):
    return {k: orc.round_bf16(v) for k, v in p.items()}


# rows cover: one partial tile (5), ragged last tile (100), a batch of sequences (2 x 70), n = 2
@pytest.mark.parametrize("shape,n_mult,masked", [((5,), 4, False), ((100,), 4, True), ((2, 70), 4, True), ((64,), 2, True)])
def test_single_transition(shape, n_mult, masked):
    lib()
    gen = torch.Generator().manual_seed(900 + shape[-1])
    p = _round(orc.make_transition_params(gen, 384, n_mult))
    x = orc.round_bf16(1.5 * torch.randn(*shape, 384, generator=gen) + 0.1)
    mask = (torch.rand(*shape, generator=gen) > 0.25).float() if masked else None
    m = of3pair.SwiGLUTransition(384, n_mult)
    m.load_state_dict(p, strict=True)
    m = m.to(DEV).to(torch.bfloat16).eval()
    print("single transition", shape, n_mult, masked, flush=True)
    xg = x.to(DEV).to(torch.bfloat16)
    got = m(xg, mask=None if mask is None else mask.to(DEV))
    want = orc.transition_update(x, mask, p)
    floor = orc.transition_update(x.to(torch.bfloat16), None if mask is None else mask.to(torch.bfloat16),
                                  {k: v.to(torch.bfloat16) for k, v in p.items()})
    _check("single transition update", got, want, bf16_ref=floor)
    assert torch.equal(xg.float().cpu(), x)
    if mask is not None:
        masked_out = got.float().cpu()[mask == 0]
        assert masked_out.numel() == 0 or float(masked_out.abs().max()) == 0.0
    res = m(xg, mask=None if mask is None else mask.to(DEV), _add_residual=True, _inplace=True)
    assert res.data_ptr() == xg.data_ptr()
    _check("single transition x+update", res, x + want, rms_rel=4e-3)


def test_single_transition_in_place_on_a_strided_view():
    """_inplace on a tensor that is not contiguous: the kernel runs on a contiguous copy and the
    result is copied back, so the caller's storage holds x + update afterwards."""
    lib()
    gen = torch.Generator().manual_seed(911)
    p = _round(orc.make_transition_params(gen, 384, 2))
    wide = orc.round_bf16(torch.randn(37, 2, 384, generator=gen))
    m = of3pair.SwiGLUTransition(384, 2)
    m.load_state_dict(p, strict=True)
    m = m.to(DEV).to(torch.bfloat16).eval()
    wg = wide.to(DEV).to(torch.bfloat16)
    view = wg[:, 1]                       # rows with a stride of 2 * 384
    assert not view.is_contiguous()
    res = m(view, mask=None, _add_residual=True, _inplace=True)
    assert res.data_ptr() == view.data_ptr()
    want = wide[:, 1] + orc.transition_update(wide[:, 1], None, p)
    _check("strided in-place single transition", wg[:, 1], want, rms_rel=4e-3)
    assert torch.equal(wg[:, 0].float().cpu(), wide[:, 0]), "the other rows of the storage are untouched"


@pytest.mark.parametrize("shape,n_mult,c", [((50,), 4, 384), ((2, 19), 2, 384), ((23,), 3, 90), ((9,), 5, 62)])
def test_single_transition_fp32(shape, n_mult, c):
    """Widths that are no multiples of 4 take the kernels' scalar weight reads, hidden widths that are
    no multiples of 64 their zero padding."""
    lib()
    gen = torch.Generator().manual_seed(940 + shape[-1])
    p = orc.make_transition_params(gen, c, n_mult)
    x = 1.5 * torch.randn(*shape, c, generator=gen) + 0.1
    mask = (torch.rand(*shape, generator=gen) > 0.25).float()
    m = of3pair.SwiGLUTransition(c, n_mult)
    m.load_state_dict(p, strict=True)
    m = m.to(DEV).eval()
    got = m(x.to(DEV), mask=mask.to(DEV))
    want = orc.transition_update(x, mask, p)
    report("single transition fp32", got.cpu(), want, atol=1e-4, rtol=0.0)
    res = m(x.to(DEV), mask=None, _add_residual=True)
    report("single transition fp32 x+update", res.cpu(), x + orc.transition_update(x, None, p), atol=1e-4, rtol=0.0)


def test_pairformer_block_fp32():
    """The whole block in fp32: max-abs 1e-4."""
    lib()
    n = 40
    p = orc.make_pairformer_block_params(21, 384, 128, 128, 32, 4, 24, 16, 4)
    gen = torch.Generator().manual_seed(97)
    s = torch.randn(n, 384, generator=gen)
    z = orc.make_pair_input(98, (), n, 128)
    single_mask = torch.ones(n)
    single_mask[-6:] = 0
    pair_mask = single_mask[:, None] * single_mask[None, :]
    blk = of3pair.PairFormerBlock(**CFG)
    blk.load_state_dict(p, strict=True)
    blk = blk.to(DEV).eval()
    s_got, z_got = blk(s.to(DEV), z.to(DEV), single_mask.to(DEV), pair_mask.to(DEV))
    s_want, z_want = orc.pairformer_block(s, z, single_mask, pair_mask, p, 4, 16)
    for name, got, want in (("z", z_got, z_want), ("s", s_got, s_want)):
        rec = record_parity("pairformer block fp32 " + name, got, want, None, "fp32: max|err| <= 1e-4")
        assert rec["max_abs_err"] <= 1e-4, rec


def test_pairformer_stack_reference_unit_test_shape():
    """The reference's own unit test of the stack (test_pairformer.py:24-75), here with the values checked:
    fp32, batch 2, n_res = 22, c_s = 384, c_z = 128, pair-bias attention 3 heads of 12 (36 channels, not c_s),
    hidden width 19 in the triangle multiplication, 7 heads of 14 in the triangle attention, transition
    n = 2, two blocks, integer 0/1 masks, chunk_size = 4."""
    lib()
    n, cs, cz = 22, 384, 128
    blocks = [orc.make_pairformer_block_params(70 + i, cs, cz, 19, 14, 7, 12, 3, 2) for i in range(2)]
    gen = torch.Generator().manual_seed(99)
    s = torch.rand(2, n, cs, generator=gen)
    z = torch.rand(2, n, n, cz, generator=gen)
    single_mask = torch.randint(0, 2, (2, n), generator=gen)
    pair_mask = torch.randint(0, 2, (2, n, n), generator=gen)
    stack = of3pair.PairFormerStack(c_s=cs, c_z=cz, c_hidden_pair_bias=12, no_heads_pair_bias=3, c_hidden_mul=19,
                                    c_hidden_pair_att=14, no_heads_pair=7, no_blocks=2, transition_type="swiglu",
                                    transition_n=2, pair_dropout=0.25, fuse_projection_weights=False,
                                    blocks_per_ckpt=None, inf=1e9)
    sd = {}
    for i, p in enumerate(blocks):
        sd.update({"blocks.%d.%s" % (i, k): v for k, v in p.items()})
    stack.load_state_dict(sd, strict=True)
    stack = stack.to(DEV).eval()
    s_got, z_got = stack(s.to(DEV), z.to(DEV), single_mask=single_mask.to(DEV), pair_mask=pair_mask.to(DEV), chunk_size=4)
    assert s_got.shape == s.shape and z_got.shape == z.shape
    s_want, z_want = s, z
    for p in blocks:
        s_want, z_want = orc.pairformer_block(s_want, z_want, single_mask.float(), pair_mask.float(), p, 7, 3)
    for name, got, want in (("z", z_got, z_want), ("s", s_got, s_want)):
        rec = record_parity("pairformer stack, reference unit-test shape, fp32 " + name, got, want, None,
                            "fp32: max|err| <= 1e-4")
        assert rec["max_abs_err"] <= 1e-4, rec


def test_pairformer_block_bf16_widths_outside_the_bf16_kernels():
    """The same odd widths in bf16: every module of the block falls back to the fp32 kernels on widened
    activations and rounds its result to bf16 once (pair modules, pair bias, attention over s, transitions)."""
    lib()
    n, cs, cz = 22, 384, 128
    p = _round(orc.make_pairformer_block_params(72, cs, cz, 19, 14, 7, 12, 3, 2))
    gen = torch.Generator().manual_seed(100)
    s = orc.round_bf16(torch.rand(2, n, cs, generator=gen))
    z = orc.round_bf16(torch.rand(2, n, n, cz, generator=gen))
    single_mask = torch.randint(0, 2, (2, n), generator=gen).float()
    pair_mask = torch.randint(0, 2, (2, n, n), generator=gen).float()
    blk = of3pair.PairFormerBlock(c_s=cs, c_z=cz, c_hidden_pair_bias=12, no_heads_pair_bias=3, c_hidden_mul=19,
                                  c_hidden_pair_att=14, no_heads_pair=7, transition_type="swiglu", transition_n=2,
                                  pair_dropout=0.25, fuse_projection_weights=False, inf=1e9)
    blk.load_state_dict(p, strict=True)
    blk = blk.to(DEV).to(torch.bfloat16).eval()
    sg, zg = s.to(DEV).to(torch.bfloat16), z.to(DEV).to(torch.bfloat16)
    s_got, z_got = blk(sg, zg, single_mask.to(DEV), pair_mask.to(DEV))
    assert s_got.dtype == torch.bfloat16 and z_got.dtype == torch.bfloat16
    s_want, z_want = orc.pairformer_block(s, z, single_mask, pair_mask, p, 7, 3)
    _check("pairformer block, odd widths in bf16, z", z_got, z_want, rms_rel=1e-2)
    _check("pairformer block, odd widths in bf16, s", s_got, s_want, rms_rel=1e-2)
    s2, z2 = blk(sg.clone(), zg.clone(), single_mask.to(DEV), pair_mask.to(DEV), inplace_safe=True)
    assert torch.equal(s2, s_got) and torch.equal(z2, z_got)


@pytest.mark.parametrize("mask_trans", [True, False])
def test_pairformer_block(mask_trans):
    """One PairFormerBlock of the AF3 trunk shape at N = 72 with a padded tail: (s, z) against the
    oracle; inputs intact without inplace_safe, identical results with it."""
    lib()
    n = 72
    p = _round(orc.make_pairformer_block_params(3, 384, 128, 128, 32, 4, 24, 16, 4))
    gen = torch.Generator().manual_seed(91)
    s = orc.round_bf16(torch.randn(n, 384, generator=gen))
    z = orc.round_bf16(orc.make_pair_input(92, (), n, 128))
    single_mask = torch.ones(n)
    single_mask[-9:] = 0
    pair_mask = single_mask[:, None] * single_mask[None, :]
    blk = of3pair.PairFormerBlock(**CFG)
    blk.load_state_dict(p, strict=True)
    blk = blk.to(DEV).to(torch.bfloat16).eval()
    sg, zg = s.to(DEV).to(torch.bfloat16), z.to(DEV).to(torch.bfloat16)
    print("pairformer block", mask_trans, flush=True)
    s_got, z_got = blk(sg, zg, single_mask.to(DEV), pair_mask.to(DEV), chunk_size=4, _mask_trans=mask_trans)
    s_want, z_want = orc.pairformer_block(s, z, single_mask, pair_mask, p, 4, 16, mask_trans=mask_trans)
    _check("pairformer block z", z_got, z_want, rms_rel=1e-2)
    _check("pairformer block s", s_got, s_want, rms_rel=1e-2)
    assert torch.equal(sg.float().cpu(), s) and torch.equal(zg.float().cpu(), z)
    s2, z2 = blk(sg.clone(), zg.clone(), single_mask.to(DEV), pair_mask.to(DEV), inplace_safe=True,
                 _mask_trans=mask_trans)
    assert torch.equal(s2, s_got) and torch.equal(z2, z_got)


def test_pairformer_stack_two_blocks_with_batch():
    """PairFormerStack(**config) with 2 blocks over a batch of 2: block i loads `blocks.<i>.*`."""
    lib()
    n = 48
    blocks = [_round(orc.make_pairformer_block_params(5 + i, 384, 128, 128, 32, 4, 24, 16, 4)) for i in range(2)]
    gen = torch.Generator().manual_seed(93)
    s = orc.round_bf16(torch.randn(2, n, 384, generator=gen))
    z = orc.round_bf16(orc.make_pair_input(94, (2,), n, 128))
    single_mask = torch.ones(2, n)
    single_mask[1, -7:] = 0
    pair_mask = single_mask[:, :, None] * single_mask[:, None, :]
    stack = of3pair.PairFormerStack(no_blocks=2, blocks_per_ckpt=None, use_reentrant=False,
                                    clear_cache_between_blocks=False, tune_chunk_size=False, **CFG)
    sd = {}
    for i, p in enumerate(blocks):
        sd.update({"blocks.%d.%s" % (i, k): v for k, v in p.items()})
    stack.load_state_dict(sd, strict=True)
    stack = stack.to(DEV).to(torch.bfloat16).eval()
    s_got, z_got = stack(s.to(DEV).to(torch.bfloat16), z.to(DEV).to(torch.bfloat16), single_mask.to(DEV),
                         pair_mask.to(DEV))
    s_want, z_want = s, z
    for p in blocks:
        s_want, z_want = orc.pairformer_block(s_want, z_want, single_mask, pair_mask, p, 4, 16)
    _check("pairformer stack z", z_got, z_want, rms_rel=1.5e-2)
    _check("pairformer stack s", s_got, s_want, rms_rel=1.5e-2)


def test_pairformer_block_in_a_hip_graph_replays_like_eager():
    """A whole PairFormerBlock (about thirty kernel launches) captured once its one-time set-up has
    run; replays with eager work and synchronisations in between must reproduce the eager result
    bit for bit, also for a new input copied into the static buffers."""
    lib()
    n = 64
    p = _round(orc.make_pairformer_block_params(11, 384, 128, 128, 32, 4, 24, 16, 4))
    blk = of3pair.PairFormerBlock(**CFG)
    blk.load_state_dict(p, strict=True)
    blk = blk.to(DEV).to(torch.bfloat16).eval()
    gen = torch.Generator().manual_seed(95)
    s0 = orc.round_bf16(torch.randn(n, 384, generator=gen)).to(DEV).to(torch.bfloat16)
    z0 = orc.round_bf16(orc.make_pair_input(96, (), n, 128)).to(DEV).to(torch.bfloat16)
    single_mask = torch.ones(n, device=DEV)
    single_mask[-5:] = 0
    pair_mask = single_mask[:, None] * single_mask[None, :]
    s_eager, z_eager = blk(s0, z0, single_mask, pair_mask)  # also the warm-up: workspaces exist now
    torch.cuda.synchronize()
    s_static, z_static = s0.clone(), z0.clone()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        s_out, z_out = blk(s_static, z_static, single_mask, pair_mask)
    for rep in range(3):
        s_static.copy_(s0)
        z_static.copy_(z0)
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(s_out, s_eager) and torch.equal(z_out, z_eager), "replay %d differs" % rep
        other_s, other_z = blk(s0 * 0.5, z0 * 0.5, single_mask, pair_mask)  # eager work on the same workspaces
        assert torch.isfinite(other_s).all() and torch.isfinite(other_z).all()
        torch.cuda.synchronize()
    s1 = orc.round_bf16(torch.randn(n, 384, generator=gen)).to(DEV).to(torch.bfloat16)
    s_static.copy_(s1)
    z_static.copy_(z0)
    graph.replay()
    torch.cuda.synchronize()
    s_want, z_want = blk(s1, z0, single_mask, pair_mask)
    assert torch.equal(s_out, s_want) and torch.equal(z_out, z_want)
