"""fp32 parity: the library's fp32 kernels against the fp32 CPU oracle on the same inputs.

Tolerance (north star, fp32): max-abs error <= 1e-4.  Inputs are N(0,1), weights N(0, 1/fan_in)
and LayerNorm affine near identity, so outputs are O(1) and an absolute bound is meaningful;
benchmark configuration 1 (N=64, c_z=128, 4 heads x 32, all-ones mask) is the first case."""
import random

import pytest
import torch

from gpu_util import lib, record_parity  # noqa: F401
from oracle import pairstack_oracle as orc

import of3pair

pytestmark = pytest.mark.gpu
DEV = "cuda"
FP32_TOL = 1e-4


def _maxerr(name, got, want):
    record_parity(name, got, want, None, "fp32: max|err| <= 1e-4")
    err = float((got.float().cpu() - want).abs().max())
    print("%s: max|err| = %.3g (max|want| = %.3g)" % (name, err, float(want.abs().max())), flush=True)
    assert err <= FP32_TOL, "%s: %.3g" % (name, err)


def _load(module, params):
    module.load_state_dict(params, strict=True)
    return module.to(DEV).eval()


@pytest.mark.parametrize("outgoing", [True, False])
@pytest.mark.parametrize("c,ch,n,batch,masked", [(128, 128, 64, (1,), False), (64, 64, 45, (2,), True), (96, 40, 33, (), True),
                                                  (36, 20, 19, (), True),  # channel counts off the multiples of 8: the plain FMA kernels
                                                  (48, 80, 29, (2,), True), (256, 64, 40, (), False),  # multiples of 16, not of 64; more than 128 channels
                                                  (16, 16, 9, (), True), (64, 256, 35, (), True)])  # the narrowest and the widest hidden width
def test_trimul_fp32(outgoing, c, ch, n, batch, masked):
    lib()
    gen = torch.Generator().manual_seed(300 + n)
    p = orc.make_trimul_params(gen, c, ch)
    z = torch.randn(*batch, n, n, c, generator=gen)
    mask = (torch.rand(*batch, n, n, generator=gen) > 0.2).float() if masked else None
    cls = of3pair.TriangleMultiplicationOutgoing if outgoing else of3pair.TriangleMultiplicationIncoming
    m = _load(cls(c, ch), p)
    got = m(z.to(DEV), mask=None if mask is None else mask.to(DEV))
    assert got.dtype == torch.float32
    _maxerr("trimul fp32", got, orc.trimul_update(z, mask, p, outgoing))


@pytest.mark.parametrize("starting", [True, False])
@pytest.mark.parametrize("c,d,heads,n,batch,masked", [(128, 32, 4, 64, (1,), False), (64, 16, 4, 45, (2,), True),
                                                     (48, 64, 2, 37, (), True), (36, 16, 3, 21, (), True),
                                                     (64, 32, 2, 150, (), True),  # more than one 128-query group
                                                     (128, 32, 4, 44, (2,), True), (32, 32, 1, 129, (), False),
                                                     (16, 32, 1, 9, (), True), (256, 32, 8, 40, (), True),  # narrowest and widest
                                                     # head width 16: the template stack's; several query groups; an odd
                                                     # number of heads (no pair of heads per 32-channel tile)
                                                     (64, 16, 4, 150, (), True), (128, 16, 2, 70, (2,), False),
                                                     (48, 16, 3, 40, (), True),
                                                     # the reference's unit test (test_triangular_attention.py:24-45):
                                                     # c_z = 128, head width 12, 4 heads, n_res = 22, batch 2, no mask;
                                                     # and other widths that are no multiples of 8
                                                     (128, 12, 4, 22, (2,), False), (40, 20, 2, 35, (), True), (64, 7, 3, 19, (), True)])
def test_triattn_fp32(starting, c, d, heads, n, batch, masked):
    lib()
    gen = torch.Generator().manual_seed(400 + n)
    p = orc.make_triattn_params(gen, c, d, heads)
    x = torch.randn(*batch, n, n, c, generator=gen)
    mask = None
    if masked:
        mask = (torch.rand(*batch, n, n, generator=gen) > 0.2).float()
        mask[..., 3, :] = 0.0   # a fully masked row (starting frame) and column (ending frame)
        mask[..., :, 5] = 0.0
    m = _load(of3pair.TriangleAttention(c, d, heads, starting=starting), p)
    got = m(x.to(DEV), mask=None if mask is None else mask.to(DEV))
    _maxerr("triattn fp32", got, orc.triattn_update(x, mask, p, heads, starting=starting))


@pytest.mark.parametrize("d,heads,pads", [(32, 2, 0), (16, 4, 0), (32, 2, 50)])
def test_triattn_fp32_large_logits_and_padding(d, heads, pads):
    """Logits far outside the range in which a softmax with the offset 0 is exact (queries whose largest
    logit lies beyond +-60 in base 2): the work-groups concerned must repeat the pass with running
    maxima, next to work-groups that never need it; with a padded tail (runs of masked keys the first
    pass leaves out, padded rows that only the second pass serves)."""
    lib()
    c, n = 64, 150
    gen = torch.Generator().manual_seed(4400 + d + pads)
    p = orc.make_triattn_params(gen, c, d, heads)
    p["mha.linear_q.weight"] = p["mha.linear_q.weight"] * 14.0   # q.k / sqrt(d) of +-40 and more
    p["linear_z.weight"][0] = p["linear_z.weight"][0] * 40.0     # head 0: a triangle bias of +-100
    x = torch.randn(n, n, c, generator=gen)
    mask = orc.tail_padding_mask((), n, pads) if pads else (torch.rand(n, n, generator=gen) > 0.2).float()
    m = _load(of3pair.TriangleAttention(c, d, heads), p)
    got = m(x.to(DEV), mask=mask.to(DEV))
    want = orc.triattn_update(x, mask, p, heads)
    if pads:  # padded rows: -1e9 absorbs moderate logits only, and these are not moderate; compare the real rows
        got, want = got[: n - pads], want[: n - pads]
    _maxerr("triattn fp32 large logits", got, want)


def test_trimul_fp32_reference_unit_test_shape():
    """The reference's own unit test of the module (test_triangular_multiplicative_update.py:28-52): c_z = 128,
    hidden width 11, batch 2, n_res = 128, uniform inputs and an integer 0/1 mask; here with the values checked."""
    lib()
    gen = torch.Generator().manual_seed(511)
    p = orc.make_trimul_params(gen, 128, 11)
    x = torch.rand(2, 128, 128, 128, generator=gen)
    mask = torch.randint(0, 2, (2, 128, 128), generator=gen)
    m = _load(of3pair.TriangleMultiplicationOutgoing(128, 11), p)
    got = m(x.to(DEV), mask.to(DEV))
    assert got.shape == x.shape
    _maxerr("trimul fp32 c_hidden=11", got, orc.trimul_update(x, mask.float(), p, True))


def test_block_config1_fp32():
    """benchmark configuration 1: B=1, N=64, c_z=128, c_hidden_mul=128, 4 heads x 32, all-ones mask, fp32."""
    lib()
    n, c, d, heads = 64, 128, 32, 4
    p = orc.make_block_params(0, c, c, d, heads)
    m = _load(of3pair.PairStack(c, c, d, heads), p)
    z = orc.make_pair_input(1, (1,), n, c)
    mask = torch.ones(1, n, n)
    zg = z.to(DEV)
    got = m(zg, mask.to(DEV))
    assert torch.equal(zg.cpu(), z)
    want = orc.pair_stack_block(z, mask, p, heads)
    _maxerr("block config 1 fp32", got, want)
    got2 = m(zg, mask.to(DEV), inplace_safe=True)   # in place: same result, z overwritten
    assert got2.data_ptr() == zg.data_ptr()
    _maxerr("block config 1 fp32 in place", got2, want)


def test_block_fp32_padded():
    lib()
    n, c, d, heads = 80, 64, 16, 4
    p = orc.make_block_params(3, c, c, d, heads)
    m = _load(of3pair.PairStack(c, c, d, heads), p)
    z = orc.make_pair_input(4, (2,), n, c)
    mask = orc.tail_padding_mask((2,), n, torch.tensor([9, 0]))
    got = m(z.to(DEV), mask.to(DEV))
    _maxerr("block fp32 padded", got, orc.pair_stack_block(z, mask, p, heads))


def test_block_fp32_n768():
    """the headline shape in fp32 (N=768, c_z=128, 4 heads x 32) against the oracle: the split-operand
    kernels at the size the bench times them at, every key tile and k-panel of the full loops."""
    lib()
    n, c, d, heads = 768, 128, 32, 4
    p = orc.make_block_params(0, c, c, d, heads)
    m = _load(of3pair.PairStack(c, c, d, heads), p)
    z = orc.make_pair_input(1, (1,), n, c)
    mask = orc.tail_padding_mask((1,), n, torch.tensor([40]))
    print("fp32 block n=768", flush=True)
    got = m(z.to(DEV), mask.to(DEV))
    _maxerr("block fp32 n=768", got, orc.pair_stack_block(z, mask, p, heads, row_chunk=32))


@pytest.mark.parametrize("seed", range(12))
def test_fp32_random_shapes(seed):
    """seeded random shapes through both fp32 modules: ragged N around the tile sizes (32-key tiles,
    128-query ranges, 256 x 128 contraction tiles), channel counts on and off the multiples of 64, masks
    from empty to dense, batch 1-2."""
    lib()
    rnd = random.Random(900 + seed)
    n = rnd.choice([1, 2, 3, 5, 31, 32, 33, 63, 65, 96, 127, 129, 130, 160, 200, 257, 260])
    c = rnd.choice([64, 128, 48, 80])
    ch = rnd.choice([64, 128, 32, 48])
    heads = rnd.choice([1, 2, 4])
    batch = rnd.choice([(), (1,), (2,)])
    keep = rnd.choice([0.0, 0.3, 0.8, 1.0])
    gen = torch.Generator().manual_seed(1000 + seed)
    z = torch.randn(*batch, n, n, c, generator=gen) * rnd.choice([0.5, 1.0, 3.0])
    mask = (torch.rand(*batch, n, n, generator=gen) < keep).float() if keep < 1.0 else None
    print("fp32 random shape seed=%d n=%d c=%d ch=%d heads=%d batch=%s keep=%.1f" % (seed, n, c, ch, heads, batch, keep), flush=True)
    outgoing, starting = bool(seed & 1), bool(seed & 2)
    pm = orc.make_trimul_params(gen, c, ch)
    cls = of3pair.TriangleMultiplicationOutgoing if outgoing else of3pair.TriangleMultiplicationIncoming
    got = _load(cls(c, ch), pm)(z.to(DEV), mask=None if mask is None else mask.to(DEV))
    _maxerr("trimul fp32 random", got, orc.trimul_update(z, mask, pm, outgoing))
    d = 16 if seed % 3 == 2 else 32
    pa = orc.make_triattn_params(gen, c, d, heads)
    got = _load(of3pair.TriangleAttention(c, d, heads, starting=starting), pa)(z.to(DEV), mask=None if mask is None else mask.to(DEV))
    _maxerr("triattn fp32 random", got, orc.triattn_update(z, mask, pa, heads, starting=starting))


@pytest.mark.parametrize("kind", ["offset", "odd_stride", "transposed"])
def test_fp32_views(kind):
    """fp32 inputs that are views: a pair tensor that starts 4 bytes into its storage, one whose position
    stride is odd (both leave the 8-byte row alignment the fast kernels ask for), and a transposed one."""
    lib()
    n, c, d, heads = 70, 128, 32, 4
    gen = torch.Generator().manual_seed(77)
    z = torch.randn(n, n, c, generator=gen)
    mask = (torch.rand(n, n, generator=gen) > 0.15).float()
    if kind == "offset":
        buf = torch.zeros(n * n * c + 1, device=DEV)
        zg = buf[1:].view(n, n, c)
        zg.copy_(z)
    elif kind == "odd_stride":
        buf = torch.zeros(n, n, c + 1, device=DEV)
        zg = buf[:, :, :c]
        zg.copy_(z)
    else:
        zg = z.transpose(0, 1).contiguous().to(DEV).transpose(0, 1)
    assert not zg.is_contiguous() or kind == "offset"
    print("fp32 view %s strides %s offset %d" % (kind, zg.stride(), zg.storage_offset()), flush=True)
    pm = orc.make_trimul_params(gen, c, c)
    got = _load(of3pair.TriangleMultiplicationIncoming(c, c), pm)(zg, mask=mask.to(DEV))
    _maxerr("trimul fp32 view", got, orc.trimul_update(z, mask, pm, False))
    pa = orc.make_triattn_params(gen, c, d, heads)
    got = _load(of3pair.TriangleAttention(c, d, heads, starting=False), pa)(zg, mask=mask.to(DEV))
    _maxerr("triattn fp32 view", got, orc.triattn_update(z, mask, pa, heads, starting=False))
    assert torch.equal(zg.cpu(), z), "the input view is left as it was"


def test_block_fp32_is_deterministic():
    """no atomics, no run-to-run ordering: two calls (one on another stream) give the same bits."""
    lib()
    n, c, d, heads = 200, 128, 32, 4
    p = orc.make_block_params(5, c, c, d, heads)
    m = _load(of3pair.PairStack(c, c, d, heads), p)
    z = orc.make_pair_input(9, (1,), n, c).to(DEV)
    mask = orc.tail_padding_mask((1,), n, torch.tensor([17])).to(DEV)
    a = m(z, mask)
    b = m(z, mask)
    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        c2 = m(z, mask)
    s.synchronize()
    torch.cuda.synchronize()
    assert torch.equal(a, b) and torch.equal(a, c2)
