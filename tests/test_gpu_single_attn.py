"""Parity of the trunk's AttentionPairBias (module -> C ABI -> HIP) with the CPU oracle on the
same seeded inputs and weights.  bf16: max-norm 2e-2 and rms 8e-3 relative to the oracle's
output, at most 1.5x the rms error of the oracle's own operations executed in bfloat16."""
import pytest
import torch

from gpu_util import lib, report, record_parity  # noqa: F401
from oracle import pairstack_oracle as orc

import of3pair

pytestmark = pytest.mark.gpu
DEV = "cuda"
REL = 2e-2
C_S, C_Z, HEADS, C_HEAD = 384, 128, 16, 24


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


def _setup(seed, n, batch, c_z=C_Z):
    gen = torch.Generator().manual_seed(seed)
    p = {k: orc.round_bf16(v) for k, v in orc.make_attention_pair_bias_params(gen, C_S, c_z, C_HEAD, HEADS).items()}
    a = orc.round_bf16(torch.randn(*batch, n, C_S, generator=gen) * 1.5 + 0.2)
    z = orc.round_bf16(orc.make_pair_input(seed + 1, batch, n, c_z))
    m = of3pair.AttentionPairBias(C_S, C_S, C_S, C_S, c_z, C_HEAD, HEADS)
    m.load_state_dict(p, strict=True)
    return p, a, z, m.to(DEV).to(torch.bfloat16).eval()


# N covers: one partial tile (5), a ragged last key tile with N % 8 != 0 (45: scalar bias path),
# N % 8 == 0 but N % 32 != 0 (72), several query tiles per work-group (160), batch dimensions
@pytest.mark.parametrize("n,batch,masked", [(5, (), False), (45, (), True), (72, (2,), True), (160, (), True),
                                            (64, (1, 2), False)])
def test_attention_pair_bias_module(n, batch, masked):
    lib()
    p, a, z, m = _setup(800 + n, n, batch)
    mask = None
    if masked:
        mask = torch.ones(*batch, n)
        mask[..., n - max(1, n // 7):] = 0
    print("attention pair bias", n, batch, masked, flush=True)
    ag, zg = a.to(DEV).to(torch.bfloat16), z.to(DEV).to(torch.bfloat16)
    got = m(ag, zg, mask=None if mask is None else mask.to(DEV))
    want = orc.attention_pair_bias(a, z, mask, p, HEADS)
    pb = {k: v.to(torch.bfloat16) for k, v in p.items()}
    floor = orc.attention_pair_bias(a.to(torch.bfloat16), z.to(torch.bfloat16),
                                    None if mask is None else mask.to(torch.bfloat16), pb, HEADS)
    _check("attention pair bias update", got, want, rms_rel=8e-3, bf16_ref=floor)
    assert torch.equal(ag.float().cpu(), a), "the input must not be touched"
    # s + update, in place (pairformer.py:189-201 with inplace_safe)
    res = m(ag, zg, mask=None if mask is None else mask.to(DEV), _add_residual=True, _inplace=True)
    assert res.data_ptr() == ag.data_ptr()
    _check("attention pair bias s+update", res, a + want, rms_rel=4e-3)


def test_attention_pair_bias_fully_masked_and_template_width():
    """All keys masked: the -1e9 bias is common to every logit and cancels in the softmax, as in
    the reference; c_z = 64 exercises the other pair-bias kernel."""
    lib()
    n = 40
    p, a, z, m = _setup(31, n, (), c_z=64)
    mask = torch.zeros(n)
    got = m(a.to(DEV).to(torch.bfloat16), z.to(DEV).to(torch.bfloat16), mask=mask.to(DEV))
    want = orc.attention_pair_bias(a, z, mask, p, HEADS)
    assert torch.isfinite(got).all()
    _check("attention pair bias, all masked", got, want, rms_rel=8e-3)


def test_attention_pair_bias_n768_rows():
    """Trunk size (N = 768): queries are independent given k, v and the bias, so the oracle
    evaluates the whole module once on the CPU (2 GFLOP) and all rows are compared."""
    lib()
    n = 768
    p, a, z, m = _setup(33, n, ())
    got = m(a.to(DEV).to(torch.bfloat16), z.to(DEV).to(torch.bfloat16))
    want = orc.attention_pair_bias(a, z, None, p, HEADS)
    _check("attention pair bias N=768", got, want, rms_rel=8e-3)


def test_attention_pair_bias_deterministic():
    lib()
    p, a, z, m = _setup(35, 96, ())
    ag, zg = a.to(DEV).to(torch.bfloat16), z.to(DEV).to(torch.bfloat16)
    assert torch.equal(m(ag, zg), m(ag, zg))


def test_attention_pair_bias_rejects_unsupported():
    lib()
    with pytest.raises(ValueError):
        of3pair.AttentionPairBias(384, 384, 384, 384, 128, 24, 16, use_ada_layer_norm=True)
    m2 = of3pair.AttentionPairBias(768, 768, 768, 768, C_Z, 48, 16).to(DEV).eval()  # c_s beyond the fp32 kernels
    with pytest.raises(ValueError):
        m2(torch.zeros(8, 768, device=DEV), torch.zeros(8, 8, C_Z, device=DEV))
    with pytest.raises(ValueError):  # ... in bf16 too: there is no fp32 kernel to fall back to
        m2.to(torch.bfloat16)(torch.zeros(8, 768, device=DEV, dtype=torch.bfloat16),
                              torch.zeros(8, 8, C_Z, device=DEV, dtype=torch.bfloat16))


def test_attention_pair_bias_bf16_width_outside_the_bf16_kernels():
    """c_s = 128 with 4 heads of 32 in bf16: not a shape of the bf16 kernels; served by the fp32 kernels on
    widened activations, rounded to bf16 once."""
    lib()
    n, c_s, c_head, heads = 29, 128, 32, 4
    gen = torch.Generator().manual_seed(870)
    p = {k: orc.round_bf16(v) for k, v in orc.make_attention_pair_bias_params(gen, c_s, 64, c_head, heads).items()}
    a = orc.round_bf16(torch.randn(n, c_s, generator=gen))
    z = orc.round_bf16(orc.make_pair_input(871, (), n, 64))
    mask = torch.ones(n)
    mask[-4:] = 0
    m = of3pair.AttentionPairBias(c_s, c_s, c_s, c_s, 64, c_head, heads)
    m.load_state_dict(p, strict=True)
    m = m.to(DEV).to(torch.bfloat16).eval()
    got = m(a.to(DEV).to(torch.bfloat16), z.to(DEV).to(torch.bfloat16), mask=mask.to(DEV))
    assert got.dtype == torch.bfloat16
    want = orc.attention_pair_bias(a, z, mask, p, heads)
    report("attention pair bias, bf16 through fp32", got.float().cpu(), want, atol=2e-2 * float(want.abs().max()), rtol=0.0)
    ag = a.to(DEV).to(torch.bfloat16)
    res = m(ag, z.to(DEV).to(torch.bfloat16), mask=mask.to(DEV), _add_residual=True, _inplace=True)
    assert res.data_ptr() == ag.data_ptr()
    report("attention pair bias, bf16 through fp32, a+update", res.float().cpu(), a + want,
           atol=2e-2 * float((a + want).abs().max()), rtol=0.0)


@pytest.mark.parametrize("n,batch,c_s,c_head,heads,masked", [(37, (), 384, 24, 16, True), (130, (2,), 96, 12, 8, True),
                                                             (16, (), 256, 64, 4, False), (21, (), 90, 10, 9, True),
                                                             (11, (3,), 70, 7, 10, False)])
def test_attention_pair_bias_fp32(n, batch, c_s, c_head, heads, masked):
    """fp32 (the reference's default inference precision): max-abs 1e-4 against the oracle."""
    lib()
    gen = torch.Generator().manual_seed(850 + n)
    p = orc.make_attention_pair_bias_params(gen, c_s, 64, c_head, heads)
    a = torch.randn(*batch, n, c_s, generator=gen)
    z = orc.make_pair_input(851 + n, batch, n, 64)
    mask = None
    if masked:
        mask = torch.ones(*batch, n)
        mask[..., n - 5:] = 0
    m = of3pair.AttentionPairBias(c_s, c_s, c_s, c_s, 64, c_head, heads)
    m.load_state_dict(p, strict=True)
    m = m.to(DEV).eval()
    got = m(a.to(DEV), z.to(DEV), mask=None if mask is None else mask.to(DEV))
    want = orc.attention_pair_bias(a, z, mask, p, heads)
    report("attention pair bias fp32", got.cpu(), want, atol=1e-4, rtol=0.0)
    ag = a.to(DEV)
    res = m(ag, z.to(DEV), mask=None if mask is None else mask.to(DEV), _add_residual=True, _inplace=True)
    assert res.data_ptr() == ag.data_ptr()
    report("attention pair bias fp32 a+update", res.cpu(), a + want, atol=1e-4, rtol=0.0)
