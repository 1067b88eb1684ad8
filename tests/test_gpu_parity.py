"""Parity of the HIP path (drop-in modules -> C ABI -> kernels) with the CPU oracle on the
same seeded inputs and weights.

bf16 bound (north star: "2e-2 relative in bf16").  Inputs and weights are rounded to bf16
once and the oracle computes in fp32 from those rounded values.  Three checks per tensor:
  1. max-norm relative error:  max|got - want| <= 2e-2 * max|want|;
  2. rms error:                rms(got - want) <= 5e-3 * rms(want) for a single module
                               (1e-2 to 1.5e-2 after a whole block or two);
  3. noise floor (module tests): the rms error is at most 1.5x that of the reference's own
     bf16 path, i.e. the oracle's very operations executed in bfloat16 on the CPU, which
     rounds after every op (LayerNorm, each Linear, sigmoid, products, softmax ...).
An elementwise |err| <= 2e-2*|want| bound is not used: the reference's bf16 path itself
misses it at hundreds of near-zero elements per million, so it cannot separate a correct
kernel from a wrong one.  Indexing mistakes show up as O(1) errors in all three checks."""
import math

import pytest
import torch

from gpu_util import lib, report, record_parity  # noqa: F401  (lib() makes sure the library is built)
from oracle import pairstack_oracle as orc

import of3pair

pytestmark = pytest.mark.gpu
DEV = "cuda"
REL = 2e-2


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


def _bf16_params(p):
    return {k: v.to(torch.bfloat16) for k, v in p.items()}


def _round_params(p):
    return {k: orc.round_bf16(v) for k, v in p.items()}


def _load(module, params):
    module.load_state_dict(params, strict=True)
    return module.to(DEV).to(torch.bfloat16).eval()


@pytest.mark.parametrize("outgoing", [True, False])
@pytest.mark.parametrize("c,n,batch", [(128, 64, ()), (128, 100, (2,)), (64, 96, (1, 3))])
def test_trimul_module(outgoing, c, n, batch):
    lib()
    gen = torch.Generator().manual_seed(100 + n)
    p = _round_params(orc.make_trimul_params(gen, c, c))
    z = orc.round_bf16(orc.make_pair_input(1, batch, n, c))
    mask = (torch.rand(*batch, n, n, generator=gen) > 0.2).float()
    cls = of3pair.TriangleMultiplicationOutgoing if outgoing else of3pair.TriangleMultiplicationIncoming
    m = _load(cls(c, c), p)
    print("trimul module", outgoing, c, n, batch, flush=True)
    zg = z.to(DEV).to(torch.bfloat16)
    got = m(zg, mask=mask.to(DEV))
    want = orc.trimul_update(z, mask, p, outgoing)
    floor = orc.trimul_update(z.to(torch.bfloat16), mask.to(torch.bfloat16), _bf16_params(p), outgoing)
    _check("trimul update", got, want, bf16_ref=floor)
    assert torch.equal(zg.float().cpu(), z), "out-of-place call must not touch z"
    # the reference's inference contract: inplace_safe + _add_with_inplace returns z + update in z
    res = m(zg, mask=mask.to(DEV), inplace_safe=True, _add_with_inplace=True)
    assert res.data_ptr() == zg.data_ptr()
    _check("trimul z+update", res, z + want, rms_rel=4e-3)


def test_trimul_no_mask_is_all_ones():
    lib()
    gen = torch.Generator().manual_seed(5)
    p = _round_params(orc.make_trimul_params(gen, 128, 128))
    z = orc.round_bf16(orc.make_pair_input(2, (), 40, 128))
    m = _load(of3pair.TriangleMultiplicationOutgoing(128, 128), p)
    got = m(z.to(DEV).to(torch.bfloat16))
    _check("trimul maskless", got, orc.trimul_update(z, None, p, True))


@pytest.mark.parametrize("starting", [True, False])
@pytest.mark.parametrize("c,d,n,batch", [(128, 32, 64, ()), (128, 32, 100, (2,)), (64, 16, 96, (1, 3))])
def test_triattn_module(starting, c, d, n, batch):
    lib()
    gen = torch.Generator().manual_seed(200 + n)
    p = _round_params(orc.make_triattn_params(gen, c, d, 4))
    z = orc.round_bf16(orc.make_pair_input(3, batch, n, c))
    mask = (torch.rand(*batch, n, n, generator=gen) > 0.2).float()
    mask[..., 5, :] = 0  # one fully masked row
    mask[..., :, 7] = 0  # and one fully masked column (a fully masked row for the ending node)
    m = _load(of3pair.TriangleAttention(c, d, 4, starting=starting), p)
    print("triattn module", starting, c, d, n, batch, flush=True)
    got = m(z.to(DEV).to(torch.bfloat16), mask=mask.to(DEV), chunk_size=4, use_lma=True)
    want = orc.triattn_update(z, mask, p, 4, starting=starting)
    floor = orc.triattn_update(z.to(torch.bfloat16), mask.to(torch.bfloat16), _bf16_params(p), 4, starting=starting)
    # rms bound 6e-3: the bf16 reference path itself sits at about 7.5e-3 on these inputs
    _check("triattn update", got, want, rms_rel=6e-3, bf16_ref=floor)


def test_triattn_transposed_view_input():
    """PairBlock hands the ending-node module a transposed, non-contiguous view."""
    lib()
    gen = torch.Generator().manual_seed(9)
    p = _round_params(orc.make_triattn_params(gen, 128, 32, 4))
    z = orc.round_bf16(orc.make_pair_input(4, (1,), 72, 128))
    mask = orc.tail_padding_mask((1,), 72, 9)
    m = _load(of3pair.TriangleAttention(128, 32, 4), p)
    zg = z.to(DEV).to(torch.bfloat16)
    got = m(zg.transpose(-2, -3), mask=mask.to(DEV).transpose(-1, -2))
    want = orc.triattn_update(z.transpose(-2, -3), mask.transpose(-1, -2), p, 4)
    _check("triattn on transposed view", got, want)


def _pair_stack(c, ch, d, seed):
    p = _round_params(orc.make_block_params(seed, c, ch, d, 4))
    return _load(of3pair.PairStack(c, ch, d, 4), p), p


def test_block_config2_n384_padded():
    """benchmark configuration 2: N=384, c_z=128, last 10% of the tokens padded."""
    lib()
    n = 384
    m, p = _pair_stack(128, 128, 32, seed=0)
    z = orc.round_bf16(orc.make_pair_input(1, (1,), n, 128))
    mask = orc.tail_padding_mask((1,), n, n - math.ceil(0.9 * n))
    print("block config 2", flush=True)
    zg = z.to(DEV).to(torch.bfloat16)
    got = m(zg, mask.to(DEV))
    assert torch.equal(zg.float().cpu(), z), "inplace_safe=False must leave the input intact"
    want = orc.pair_stack_block(z, mask, p, 4, row_chunk=64)
    _check("block n=384", got, want, rms_rel=1e-2)


def test_block_config3_n768():
    """benchmark configuration 3 (headline shape): N=768, all-ones mask; in place."""
    lib()
    n = 768
    m, p = _pair_stack(128, 128, 32, seed=0)
    z = orc.round_bf16(orc.make_pair_input(1, (1,), n, 128))
    mask = torch.ones(1, n, n)
    print("block config 3", flush=True)
    zg = z.to(DEV).to(torch.bfloat16)
    got = m(zg, mask.to(DEV), inplace_safe=True)
    want = orc.pair_stack_block(z, mask, p, 4, row_chunk=32)
    _check("block n=768", got, want, rms_rel=1e-2)


def test_template_stack_config4():
    """benchmark configuration 4: 2 blocks, 4 templates, N=512, c_t=64, 4 heads x 16, each template
    with its own padded tail (0-20% of the tokens)."""
    lib()
    n, t = 512, 4
    gen = torch.Generator().manual_seed(2)
    blocks = [_pair_stack(64, 64, 16, seed=s) for s in (10, 11)]
    z = orc.round_bf16(orc.make_pair_input(1, (1, t), n, 64))
    pad = torch.randint(0, 103, (1, t), generator=gen)
    mask = orc.tail_padding_mask((1, t), n, pad)
    print("template config 4 pads", pad.tolist(), flush=True)
    zg = z.to(DEV).to(torch.bfloat16)
    mg = mask.to(DEV)
    for m, _ in blocks:
        zg = m(zg, mg, inplace_safe=True)
    want = orc.template_pair_stack(z, mask, [p for _, p in blocks], 4, row_chunk=64)
    _check("template stack", zg, want, rms_rel=1.5e-2)


def test_config5_n2048_modules_at_sampled_positions():
    """benchmark configuration 5 shape: N=2048, c_z=128, the last 256 tokens padded.  A full fp32
    pass on the CPU is out of reach (16 TFLOP per block), so every module's GPU output is
    compared with the oracle at sampled rows / fibres that include the first and last valid
    and padded tokens (oracle/pairstack_oracle.py: trimul_update_at, triattn_update_rows)."""
    lib()
    n, c, heads, d = 2048, 128, 4, 32
    p = _round_params(orc.make_block_params(5, c, c, d, heads))
    stack = _load(of3pair.PairStack(c, c, d, heads), p)
    z = orc.round_bf16(orc.make_pair_input(6, (), n, c))            # [N, N, C] fp32 on the host
    mask = orc.tail_padding_mask((), n, 256)
    zg = z.to(DEV).to(torch.bfloat16)[None]
    mg = mask.to(DEV)[None]
    rows = [0, 1, 1023, 1791, 1792, 2047]
    cols = [0, 511, 1790, 1791, 1792, 2046, 2047]
    print("config 5: trimul", flush=True)
    for name, mod, outgoing in (("tri_mul_out", stack.tri_mul_out, True), ("tri_mul_in", stack.tri_mul_in, False)):
        got = mod(zg, mask=mg)[0][rows][:, cols].float().cpu()
        want = orc.trimul_update_at(z, mask, orc._sub(p, name + "."), outgoing, rows, cols)
        _check("cfg5 " + name, got, want, rms_rel=6e-3)
    print("config 5: triangle attention", flush=True)
    got = stack.tri_att_start(zg, mask=mg)[0][rows].float().cpu()
    want = orc.triattn_update_rows(z, mask, orc._sub(p, "tri_att_start."), heads, rows, starting=True)
    _check("cfg5 tri_att_start", got, want, rms_rel=6e-3)
    # the ending node as the block calls it: a starting module on the transposed view
    got = stack.tri_att_end(zg.transpose(-2, -3), mask=mg.transpose(-1, -2))[0][rows].float().cpu()
    want = orc.triattn_update_rows(z.transpose(0, 1), mask.transpose(0, 1), orc._sub(p, "tri_att_end."), heads, rows,
                                   starting=True)
    _check("cfg5 tri_att_end", got, want, rms_rel=6e-3)


@pytest.mark.parametrize("n,pad", [(1000, 0), (929, 37)])
def test_ragged_large_n_modules_at_sampled_positions(n, pad):
    """Token counts far from the multiples of 128 (ragged tiles in every pass, contraction tiles that hang
    over the edge of the plane, a last key tile with few keys), at a size the CPU oracle only reaches at
    sampled rows / fibres: first and last rows, the rows around the last whole 128-wide piece and around the
    padded tail."""
    lib()
    c, heads, d = 128, 4, 32
    p = _round_params(orc.make_block_params(31, c, c, d, heads))
    stack = _load(of3pair.PairStack(c, c, d, heads), p)
    z = orc.round_bf16(orc.make_pair_input(32, (), n, c))
    mask = orc.tail_padding_mask((), n, pad)
    zg = z.to(DEV).to(torch.bfloat16)[None]
    mg = mask.to(DEV)[None]
    last_full = 128 * (n // 128)
    rows = sorted({0, 1, last_full - 1, last_full, n - pad - 1, n - 2, n - 1})
    cols = sorted({0, 511, last_full - 1, last_full, last_full + 1, n - pad - 1, n - 1})
    print("ragged n", n, "pad", pad, "rows", rows, flush=True)
    for name, mod, outgoing in (("tri_mul_out", stack.tri_mul_out, True), ("tri_mul_in", stack.tri_mul_in, False)):
        got = mod(zg, mask=mg)[0][rows][:, cols].float().cpu()
        want = orc.trimul_update_at(z, mask, orc._sub(p, name + "."), outgoing, rows, cols)
        _check("n=%d %s" % (n, name), got, want, rms_rel=6e-3)
    got = stack.tri_att_start(zg, mask=mg)[0][rows].float().cpu()
    want = orc.triattn_update_rows(z, mask, orc._sub(p, "tri_att_start."), heads, rows, starting=True)
    _check("n=%d tri_att_start" % n, got, want, rms_rel=6e-3)
    got = stack.tri_att_end(zg.transpose(-2, -3), mask=mg.transpose(-1, -2))[0][rows].float().cpu()
    want = orc.triattn_update_rows(z.transpose(0, 1), mask.transpose(0, 1), orc._sub(p, "tri_att_end."), heads, rows,
                                   starting=True)
    _check("n=%d tri_att_end" % n, got, want, rms_rel=6e-3)


def test_n4096_modules_at_sampled_positions():
    """Twice the token count of the largest benchmark configuration (a 4.3 GB pair tensor, 64-bit offsets in
    every intermediate): each module against the oracle at sampled rows / fibres, then one block in place."""
    lib()
    n, pad, c, heads, d = 4096, 100, 128, 4, 32
    p = _round_params(orc.make_block_params(5, c, c, d, heads))
    stack = _load(of3pair.PairStack(c, c, d, heads), p)
    z = orc.round_bf16(orc.make_pair_input(6, (), n, c))
    mask = orc.tail_padding_mask((), n, pad)
    zg = z.to(DEV).to(torch.bfloat16)[None]
    mg = mask.to(DEV)[None]
    rows = [0, 1, n // 2 - 1, n - pad - 1, n - 1]
    cols = [0, 511, n // 2, n - pad - 1, n - 2, n - 1]
    print("n = 4096: trimul", flush=True)
    for name, mod, outgoing in (("tri_mul_out", stack.tri_mul_out, True), ("tri_mul_in", stack.tri_mul_in, False)):
        got = mod(zg, mask=mg)[0][rows][:, cols].float().cpu()
        want = orc.trimul_update_at(z, mask, orc._sub(p, name + "."), outgoing, rows, cols)
        _check("n=4096 " + name, got, want, rms_rel=6e-3)
    print("n = 4096: triangle attention", flush=True)
    got = stack.tri_att_start(zg, mask=mg)[0][rows].float().cpu()
    want = orc.triattn_update_rows(z, mask, orc._sub(p, "tri_att_start."), heads, rows, starting=True)
    _check("n=4096 tri_att_start", got, want, rms_rel=6e-3)
    got = stack.tri_att_end(zg.transpose(-2, -3), mask=mg.transpose(-1, -2))[0][rows].float().cpu()
    want = orc.triattn_update_rows(z.transpose(0, 1), mask.transpose(0, 1), orc._sub(p, "tri_att_end."), heads, rows,
                                   starting=True)
    _check("n=4096 tri_att_end", got, want, rms_rel=6e-3)
    del got, want, z
    res = stack(zg, mg, inplace_safe=True)
    assert res.data_ptr() == zg.data_ptr() and torch.isfinite(res.float()).all()
    del res, zg
    of3pair.functional.release_workspaces()
    torch.cuda.empty_cache()


def test_config5_four_blocks_run_in_place():
    """Config 5 end to end: 4 stacked blocks at N=2048 in place (1 GiB pair tensor).  Checked
    through size-independent properties: finite output, bitwise identical on a second run,
    and the first block identical to the out-of-place call."""
    lib()
    n, c, heads, d = 2048, 128, 4, 32
    blocks = [_pair_stack(c, c, d, seed=s)[0] for s in (20, 21, 22, 23)]
    z = orc.round_bf16(orc.make_pair_input(7, (1,), n, c)).to(torch.bfloat16)
    mask = orc.tail_padding_mask((1,), n, 256).to(DEV)
    print("config 5: four blocks", flush=True)
    outs = []
    for rep in range(2):
        zg = z.to(DEV)
        first = blocks[0](zg, mask) if rep == 0 else None
        for m in blocks:
            zg = m(zg, mask, inplace_safe=True)
            if first is not None:
                assert torch.equal(first, zg), "in-place and out-of-place block differ"
                first = None
        torch.cuda.synchronize()
        assert torch.isfinite(zg.float()).all()
        outs.append(zg.cpu())
        del zg
    assert torch.equal(outs[0], outs[1]), "two runs of the same stack differ bitwise"


@pytest.mark.gpu
@pytest.mark.parametrize("outgoing", [True, False])
def test_fused_trimul_module(outgoing):
    """FusedTriangleMultiplicativeUpdate (tmu.py:522-666, bias-free) against the oracle's restatement of
    its forward, and bit for bit against the un-fused module holding the two halves of the stacked
    weights (the same kernels on the same numbers); in place with the residual as well."""
    lib()
    c, n = 128, 150
    gen = torch.Generator().manual_seed(88)
    p = {k: orc.round_bf16(v) for k, v in orc.make_trimul_params(gen, c, c).items()}
    fp = orc.fuse_trimul_params(p)
    z = orc.round_bf16(orc.make_pair_input(89, (2,), n, c))
    mask = orc.tail_padding_mask((2,), n, torch.tensor([13, 0]))
    cls = of3pair.FusedTriangleMultiplicationOutgoing if outgoing else of3pair.FusedTriangleMultiplicationIncoming
    ucls = of3pair.TriangleMultiplicationOutgoing if outgoing else of3pair.TriangleMultiplicationIncoming
    m, u = _load(cls(c, c), fp), _load(ucls(c, c), p)
    zg = z.to(DEV).to(torch.bfloat16)
    got = m(zg, mask=mask.to(DEV))
    assert torch.equal(got, u(zg, mask=mask.to(DEV)))
    want = orc.fused_trimul_update(z, mask, fp, outgoing)
    _check("fused trimul update", got, want, rms_rel=5e-3)
    res = m(zg, mask=mask.to(DEV), inplace_safe=True, _add_with_inplace=True)
    assert res.data_ptr() == zg.data_ptr()
    _check("fused trimul in place", res, z + want, rms_rel=5e-3)


def test_config5_four_blocks_against_the_fp32_path():
    """Config 5's composed output: the four stacked bf16 blocks at N=2048 against the same four blocks on
    the library's fp32 path (three-term bf16 operands, fp32 accumulation; pinned against the oracle within
    1e-4 by test_gpu_fp32.py at the sizes the CPU reaches).  A composed fp32 pass on the CPU is about
    65 TFLOP, so the fp32 kernels stand in for it here.  Every block rounds the pair tensor to bf16 four
    times (one residual write per module), so the bounds are per stack, not the per-module 2e-2: the
    error may grow with the square root of the number of modules at most."""
    lib()
    n, c, heads, d = 2048, 128, 4, 32
    seeds = (20, 21, 22, 23)
    params = [_round_params(orc.make_block_params(s, c, c, d, heads)) for s in seeds]
    z = orc.round_bf16(orc.make_pair_input(7, (1,), n, c))
    mask = orc.tail_padding_mask((1,), n, 256).to(DEV)
    print("config 5: four blocks, bf16 against fp32", flush=True)
    zb = z.to(DEV).to(torch.bfloat16)
    for p in params:
        zb = _load(of3pair.PairStack(c, c, d, heads), p)(zb, mask, inplace_safe=True)
    got = zb.float().cpu()
    del zb
    zf = z.to(DEV)
    for p in params:
        m = of3pair.PairStack(c, c, d, heads)
        m.load_state_dict(p, strict=True)
        zf = m.to(DEV).float().eval()(zf, mask, inplace_safe=True)
    want = zf.cpu()
    del zf
    of3pair.functional.release_workspaces()
    valid = slice(0, n - 256)
    g, w = got[0, valid, valid], want[0, valid, valid]
    err = (g - w)
    rms, erms = float(w.pow(2).mean().sqrt()), float(err.pow(2).mean().sqrt())
    emax, wmax = float(err.abs().max()), float(w.abs().max())
    print("cfg5 composed: rms %.4g err rms %.4g (%.3g rel) max err %.4g of max %.4g (%.3g rel)"
          % (rms, erms, erms / rms, emax, wmax, emax / wmax), flush=True)
    record_parity("cfg5 four blocks bf16 vs fp32 path", g, w, None, "rms_rel <= 1e-2, max|err| <= 2e-2 max|want|")
    assert erms <= 1e-2 * rms
    assert emax <= 2e-2 * wmax
