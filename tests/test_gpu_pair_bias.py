"""Parity of the pair-bias projection (PairBiasProjection module -> C ABI -> HIP) with the CPU
oracle on the same seeded inputs and weights.  bf16: max-norm 2e-2, rms 5e-3, at most 1.5x
the rms error of the oracle's own operations executed in bfloat16.  fp32: max-abs 1e-4."""
import pytest
import torch

from gpu_util import lib, report, record_parity  # noqa: F401
from oracle import pairstack_oracle as orc

import of3pair
from of3pair import functional as F3

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _check(name, got, want, rms_rel=5e-3, bf16_ref=None):
    got = got.float().cpu()
    want = want.float()
    record_parity(name, got, want, bf16_ref, "max|err| <= 2e-2 max|want|, rms_rel <= %.1e%s" % (
        rms_rel, ", floor <= 1.5" if bf16_ref is not None else ""))
    report(name, got, want, atol=2e-2 * float(want.abs().max()), rtol=0.0)
    erms = float((got - want).pow(2).mean().sqrt())
    assert erms <= rms_rel * float(want.pow(2).mean().sqrt()), "%s: rms error %.3g" % (name, erms)
    if bf16_ref is not None:
        floor = float((bf16_ref.float() - want).pow(2).mean().sqrt())
        assert erms <= 1.5 * floor, "%s: rms error %.3g above the bf16 reference path's %.3g" % (name, erms, floor)


def _module(c, h, p, dtype):
    m = of3pair.PairBiasProjection(c, h, create_offset="layer_norm_z.bias" in p)
    m.load_state_dict(p, strict=True)
    return m.to(DEV).to(dtype).eval()


# N: partial wave, odd (scalar stores), one tile, ragged second tile; H: 16 (pairformer), 4, 32, 3
@pytest.mark.parametrize("c,h,n,batch,offset", [
    (128, 16, 5, (), True), (128, 16, 99, (2,), True), (128, 16, 256, (), False), (128, 4, 300, (), True),
    (64, 32, 72, (1, 2), True), (64, 3, 40, (), False), (128, 16, 384, (), True),
])
def test_pair_bias_module(c, h, n, batch, offset):
    lib()
    gen = torch.Generator().manual_seed(700 + n + h)
    p = {k: orc.round_bf16(v) for k, v in orc.make_pair_bias_params(gen, c, h, offset=offset).items()}
    z = orc.round_bf16(orc.make_pair_input(21, batch, n, c))
    m = _module(c, h, p, torch.bfloat16)
    print("pair bias", c, h, n, batch, offset, flush=True)
    zg = z.to(DEV).to(torch.bfloat16)
    got = m(zg)
    assert got.shape == (*batch, h, n, n) and got.dtype == torch.bfloat16
    want = orc.pair_bias(z, p)
    floor = orc.pair_bias(z.to(torch.bfloat16), {k: v.to(torch.bfloat16) for k, v in p.items()})
    _check("pair bias", got, want, bf16_ref=floor)
    assert torch.equal(zg.float().cpu(), z)
    # the transposed view gives the transposed bias, without a copy of z
    got_t = m(zg.transpose(-2, -3))
    _check("pair bias of the transposed view", got_t.transpose(-1, -2), want)


def test_pair_bias_full_size_sampled():
    """Pairformer shape N = 768, c_z = 128, 16 heads: whole rows against the oracle."""
    lib()
    n, rows = 768, [0, 1, 400, 767]
    gen = torch.Generator().manual_seed(800)
    p = {k: orc.round_bf16(v) for k, v in orc.make_pair_bias_params(gen, 128, 16).items()}
    m = _module(128, 16, p, torch.bfloat16)
    g = torch.Generator(device=DEV).manual_seed(5)
    zg = torch.randn(1, n, n, 128, device=DEV, generator=g).to(torch.bfloat16)
    got = m(zg)
    assert torch.isfinite(got).all()
    want = orc.pair_bias(zg[0, rows].float().cpu().unsqueeze(1), p)  # [rows, H, 1, N]
    _check("pair bias rows at N=768", got[0][:, rows].permute(1, 0, 2), want[:, :, 0])


@pytest.mark.parametrize("c,h,n,batch,offset", [(128, 16, 33, (), True), (96, 5, 20, (2,), False), (256, 64, 9, (), True),
                                                     (40, 3, 17, (), False), (64, 32, 70, (2,), True)])
def test_pair_bias_fp32(c, h, n, batch, offset):
    lib()
    gen = torch.Generator().manual_seed(900 + n)
    p = orc.make_pair_bias_params(gen, c, h, offset=offset)
    z = orc.make_pair_input(22, batch, n, c)
    got = _module(c, h, p, torch.float32)(z.to(DEV))
    report("pair bias fp32", got.cpu(), orc.pair_bias(z, p), atol=1e-4, rtol=0.0)


def test_pair_bias_rejects_unsupported():
    lib()
    z = torch.zeros(1, 8, 8, 128, device=DEV, dtype=torch.bfloat16)
    with pytest.raises(ValueError):  # 80 heads: beyond both the bf16 kernel (32) and the fp32 kernels (64)
        F3.pair_bias(z, torch.ones(128, device=DEV), None, torch.zeros(80, 128, device=DEV))
    with pytest.raises(ValueError):  # 320 channels: beyond the fp32 kernels too
        F3.pair_bias(torch.zeros(1, 8, 8, 320, device=DEV, dtype=torch.bfloat16), torch.ones(320, device=DEV), None,
                     torch.zeros(4, 320, device=DEV))


def test_pair_bias_bf16_shape_outside_the_bf16_kernel():
    """40 heads (more than one MFMA tile of heads) and 96 channels in bf16: the fp32 kernel on widened
    activations, rounded to bf16 once."""
    lib()
    for c, h in ((128, 40), (96, 5)):
        gen = torch.Generator().manual_seed(930 + h)
        p = {k: orc.round_bf16(v) for k, v in orc.make_pair_bias_params(gen, c, h, offset=True).items()}
        z = orc.round_bf16(orc.make_pair_input(23, (2,), 19, c))
        got = _module(c, h, p, torch.bfloat16)(z.to(DEV).to(torch.bfloat16))
        assert got.dtype == torch.bfloat16 and tuple(got.shape) == (2, h, 19, 19)
        want = orc.pair_bias(z, p)
        report("pair bias, bf16 through fp32", got.float().cpu(), want, atol=2e-2 * float(want.abs().max()), rtol=0.0)
