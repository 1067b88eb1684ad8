"""Stage-by-stage checks of the HIP kernels through the C ABI, each against the same step
computed with torch in fp32 on bf16-rounded inputs.  These localise a failure to one
kernel; parity with the oracle for whole modules is in test_gpu_parity.py.

Tolerances: every kernel output is rounded once to bf16 (relative 2^-9 = 0.002), and MFMA
accumulation order differs from torch's, so outputs are compared with rtol 1e-2 plus an
absolute term scaled to the tensor (2e-2 relative to its magnitude is the north-star bound)."""
import math

import pytest
import torch

from gpu_util import bf, lib, report, s3, stream

pytestmark = pytest.mark.gpu
DEV = "cuda"
LOG2E = 1.4426950408889634


def _gen(seed):
    return torch.Generator(device="cpu").manual_seed(seed)


def _randn(gen, *shape, scale=1.0):
    return (torch.randn(*shape, generator=gen) * scale).to(DEV)


def _ln(x, w, b):
    return torch.nn.functional.layer_norm(x.float(), (x.shape[-1],), w.float(), b.float(), 1e-5)


# ---------------------------------------------------------------------------------------
def _to_panels(t):
    """[..., rows, k] -> k-panel layout [..., k/32, rows, 32]"""
    *lead, rows, k = t.shape
    return t.reshape(*lead, rows, k // 32, 32).transpose(-2, -3).contiguous()


@pytest.mark.parametrize("variant", [0, 1, 2, 3, 4])
@pytest.mark.parametrize("n", [128, 384, 640, 768])
def test_contract(variant, n):
    L = lib()
    gen = _gen(n + variant)
    planes, B, CH = 64, 1, 64  # 64 planes: enough tiles that persistent work-groups take several each
    np_ = L.of3_padded_n(n)
    a = bf(_randn(gen, planes, np_, np_))
    b = bf(_randn(gen, planes, np_, np_))
    x = torch.full((planes, np_, np_), float("nan"), dtype=torch.bfloat16, device=DEV)
    print("contract variant", variant, "n", n, flush=True)
    ap, bp = _to_panels(a), _to_panels(b)
    st = L.of3_trimul_contract(ap.data_ptr(), bp.data_ptr(), x.data_ptr(), B, n, CH, variant, stream())
    assert st == 0, L.of3_status_string(st)
    torch.cuda.synchronize()
    want = torch.bmm(a.float(), b.float().transpose(1, 2))
    report("contract", x, want, atol=2e-2 * math.sqrt(np_) , rtol=1e-2)


@pytest.mark.parametrize("variant", [0, 1, 2, 3, 4])
@pytest.mark.parametrize("n", [70, 200, 333])
def test_contract_ragged_n(variant, n):
    """N off the multiples of 32 and 128: the sum runs over the ceil(N / 32) panels that hold a k below N (fewer
    of them than the pipeline has stages at N = 70), the panels after them are never read (they hold NaN here)."""
    L = lib()
    gen = _gen(500 + n + variant)
    planes, B, CH = 64, 1, 64
    np_ = L.of3_padded_n(n)
    kk = (n + 31) // 32 * 32
    a = bf(_randn(gen, planes, np_, np_))
    b = bf(_randn(gen, planes, np_, np_))
    a[:, :, kk:] = float("nan")
    b[:, :, kk:] = float("nan")
    x = torch.full((planes, np_, np_), float("nan"), dtype=torch.bfloat16, device=DEV)
    print("contract ragged variant", variant, "n", n, flush=True)
    ap, bp = _to_panels(a), _to_panels(b)
    st = L.of3_trimul_contract(ap.data_ptr(), bp.data_ptr(), x.data_ptr(), B, n, CH, variant, stream())
    assert st == 0, L.of3_status_string(st)
    torch.cuda.synchronize()
    want = torch.bmm(a[:, :, :kk].float(), b[:, :, :kk].float().transpose(1, 2))
    report("contract ragged", x[:, :n, :n], want[:, :n, :n], atol=2e-2 * math.sqrt(kk), rtol=1e-2)


def _trimul_weights(gen, C, CH):
    w = {
        "ln_in_w": 1 + 0.1 * torch.randn(C, generator=gen), "ln_in_b": 0.1 * torch.randn(C, generator=gen),
        "ln_out_w": 1 + 0.1 * torch.randn(CH, generator=gen), "ln_out_b": 0.1 * torch.randn(CH, generator=gen),
        "a_p": torch.randn(CH, C, generator=gen) / math.sqrt(C), "a_g": torch.randn(CH, C, generator=gen) / math.sqrt(C),
        "b_p": torch.randn(CH, C, generator=gen) / math.sqrt(C), "b_g": torch.randn(CH, C, generator=gen) / math.sqrt(C),
        "g": torch.randn(C, C, generator=gen) / math.sqrt(C), "z": torch.randn(C, CH, generator=gen) / math.sqrt(CH),
    }
    return {k: bf(v.to(DEV)).contiguous() for k, v in w.items()}


@pytest.mark.parametrize("outgoing", [True, False])
@pytest.mark.parametrize("C,n,B", [(128, 70, 2), (128, 128, 1), (64, 50, 3)])
def test_trimul_proj(outgoing, C, n, B):
    L = lib()
    gen = _gen(17 + n)
    CH = C
    np_ = L.of3_padded_n(n)
    z = bf(_randn(gen, B, n, n, C))
    mask = (torch.rand(B, n, n, generator=gen) > 0.3).float().to(DEV)
    w = _trimul_weights(gen, C, CH)
    a = torch.full((B, CH, np_ // 32, np_, 32), float("nan"), dtype=torch.bfloat16, device=DEV)
    b = torch.full_like(a, float("nan"))
    print("trimul_proj", outgoing, C, n, B, flush=True)
    st = L.of3_trimul_proj(z.data_ptr(), s3(z), mask.data_ptr(), s3(mask), w["ln_in_w"].data_ptr(),
                           w["ln_in_b"].data_ptr(), w["a_p"].data_ptr(), w["a_g"].data_ptr(), w["b_p"].data_ptr(),
                           w["b_g"].data_ptr(), a.data_ptr(), b.data_ptr(), B, n, C, CH, int(outgoing), stream())
    assert st == 0, L.of3_status_string(st)
    torch.cuda.synchronize()
    zn = bf(_ln(z, w["ln_in_w"], w["ln_in_b"])).float()
    m = mask[..., None]
    ar = m * torch.sigmoid(zn @ w["a_g"].float().t()) * (zn @ w["a_p"].float().t())
    br = m * torch.sigmoid(zn @ w["b_g"].float().t()) * (zn @ w["b_p"].float().t())
    for name, got, ref in (("a", a, ar), ("b", b, br)):
        got = got.transpose(-2, -3).reshape(B, CH, np_, np_)  # k-panels -> [b][c][r][k]
        # expected [b][c][r][k]: outgoing (r,k) = (i,k); incoming (r,k) from ref[b,k,r,c]
        want = ref.permute(0, 3, 1, 2) if outgoing else ref.permute(0, 3, 2, 1)
        report("trimul_proj %s valid" % name, got[:, :, :n, :n], want, atol=2e-2, rtol=1e-2)
        # the contraction sums over the panels that hold a k below n: the last of them is padded with zeros,
        # the panels after it are not written at all
        kk = (n + 31) // 32 * 32
        pad = got[:, :, :n, n:kk]
        assert (pad.float() == 0).all(), "k-padding of %s must be zero" % name
        assert torch.isnan(got[:, :, :n, kk:].float()).all(), "panels past the last k of %s are left alone" % name


@pytest.mark.parametrize("add_residual", [0, 1])
@pytest.mark.parametrize("C,n,B", [(128, 70, 2), (64, 130, 1), (128, 150, 2), (128, 5, 3), (64, 291, 1)])
def test_trimul_out(add_residual, C, n, B):
    L = lib()
    gen = _gen(29 + n)
    CH = C
    np_ = L.of3_padded_n(n)
    z = bf(_randn(gen, B, n, n, C))
    w = _trimul_weights(gen, C, CH)
    x = bf(_randn(gen, B, CH, np_, np_, scale=3.0))
    out = torch.full_like(z, float("nan"))
    print("trimul_out", add_residual, C, n, B, flush=True)
    st = L.of3_trimul_out(x.data_ptr(), z.data_ptr(), s3(z), out.data_ptr(), w["ln_in_w"].data_ptr(),
                          w["ln_in_b"].data_ptr(), w["ln_out_w"].data_ptr(), w["ln_out_b"].data_ptr(),
                          w["g"].data_ptr(), w["z"].data_ptr(), B, n, C, CH, add_residual, stream())
    assert st == 0, L.of3_status_string(st)
    torch.cuda.synchronize()
    zn = bf(_ln(z, w["ln_in_w"], w["ln_in_b"])).float()
    xv = x[:, :, :n, :n].permute(0, 2, 3, 1)
    xn = bf(_ln(xv, w["ln_out_w"], w["ln_out_b"])).float()
    want = (xn @ w["z"].float().t()) * torch.sigmoid(zn @ w["g"].float().t())
    if add_residual:
        want = want + z.float()
    report("trimul_out", out, want, atol=3e-2, rtol=1e-2)


def _triattn_weights(gen, C, H, D):
    hd = H * D
    w = {
        "ln_w": 1 + 0.1 * torch.randn(C, generator=gen), "ln_b": 0.1 * torch.randn(C, generator=gen),
        "bias": torch.randn(H, C, generator=gen) / math.sqrt(C),
        "q": torch.randn(hd, C, generator=gen) / math.sqrt(C), "k": torch.randn(hd, C, generator=gen) / math.sqrt(C),
        "v": torch.randn(hd, C, generator=gen) / math.sqrt(C), "g": torch.randn(hd, C, generator=gen) / math.sqrt(C),
        "o": torch.randn(C, hd, generator=gen) / math.sqrt(hd),
    }
    return {k: bf(v.to(DEV)).contiguous() for k, v in w.items()}


@pytest.mark.parametrize("transposed", [False, True])
@pytest.mark.parametrize("C,D,n,B", [(128, 32, 70, 2), (64, 16, 130, 1), (128, 32, 161, 1), (128, 32, 6, 3), (64, 16, 3, 2)])
def test_triattn_proj(transposed, C, D, n, B):
    L = lib()
    H = 4
    gen = _gen(41 + n)
    np_ = L.of3_padded_n(n)
    zfull = bf(_randn(gen, B, n, n, C))
    mfull = (torch.rand(B, n, n, generator=gen) > 0.3).float().to(DEV)
    x = zfull.transpose(1, 2) if transposed else zfull
    mask = mfull.transpose(1, 2) if transposed else mfull
    w = _triattn_weights(gen, C, H, D)
    q = torch.full((B, n, H, np_, D), float("nan"), dtype=torch.bfloat16, device=DEV)
    k = torch.full_like(q, float("nan"))
    vt = torch.full((B, n, H, np_ // 32, D, 32), float("nan"), dtype=torch.bfloat16, device=DEV)
    tb = torch.full((B, H, n, np_), float("nan"), dtype=torch.float32, device=DEV)
    mb = torch.full((B, n, np_), float("nan"), dtype=torch.float32, device=DEV)
    print("triattn_proj", transposed, C, D, n, B, flush=True)
    st = L.of3_triattn_proj(x.data_ptr(), s3(x), mask.data_ptr(), s3(mask), w["ln_w"].data_ptr(), w["ln_b"].data_ptr(),
                            w["q"].data_ptr(), w["k"].data_ptr(), w["v"].data_ptr(), w["bias"].data_ptr(),
                            q.data_ptr(), k.data_ptr(), vt.data_ptr(), tb.data_ptr(), mb.data_ptr(), B, n, C, H, D,
                            1e9, stream())
    assert st == 0, L.of3_status_string(st)
    torch.cuda.synchronize()
    xn = bf(_ln(x, w["ln_w"], w["ln_b"])).float()  # [B, I, J, C]
    qr = (xn @ w["q"].float().t()).view(B, n, n, H, D).permute(0, 1, 3, 2, 4) * (LOG2E / math.sqrt(D))
    kr = (xn @ w["k"].float().t()).view(B, n, n, H, D).permute(0, 1, 3, 2, 4)
    vr = (xn @ w["v"].float().t()).view(B, n, n, H, D).permute(0, 1, 3, 4, 2)
    tbr = (xn @ w["bias"].float().t()).permute(0, 3, 1, 2) * LOG2E
    mbr = LOG2E * 1e9 * (mask - 1)
    report("q", q[:, :, :, :n], qr, atol=2e-2, rtol=1e-2)
    report("k", k[:, :, :, :n], kr, atol=2e-2, rtol=1e-2)
    vt = vt.transpose(-2, -3).reshape(B, n, H, D, np_)  # key panels -> [b][i][h][d][j]
    report("vt", vt[..., :n], vr, atol=2e-2, rtol=1e-2)
    report("tbias", tb[..., :n], tbr, atol=2e-2, rtol=1e-2)
    assert torch.equal(mb[..., :n], mbr), "mask bias"
    # the padding is written as far as the attention core reads: to the end of the last token's 32-key panel
    n32 = 32 * ((n + 31) // 32)
    assert torch.isinf(mb[..., n:n32]).all() and (mb[..., n:n32] < 0).all(), "padded keys must carry -inf"
    assert torch.isfinite(k[:, :, :, n:n32].float()).all() and torch.isfinite(vt[..., n:n32].float()).all()
    assert (tb[..., n:n32] == 0).all()


# logit_scale > 1 drives the logits far beyond the range in which a softmax without running maxima is
# exact (queries shifted up overflow exp2, queries shifted down lose every term): the kernel's second
# pass has to take over for those work-groups, next to work-groups that never need it
@pytest.mark.parametrize("D,n,B,logit_scale", [(32, 70, 2, 1.0), (32, 256, 1, 1.0), (16, 130, 1, 1.0),
                                               (32, 200, 1, 40.0), (16, 70, 1, 40.0)])
def test_triattn_flash(D, n, B, logit_scale):
    L = lib()
    H = 4
    gen = _gen(53 + n)
    np_ = L.of3_padded_n(n)
    q = bf(_randn(gen, B, n, H, np_, D))
    k = bf(_randn(gen, B, n, H, np_, D))
    vt = bf(_randn(gen, B, n, H, D, np_))
    tb = _randn(gen, B, H, n, np_).contiguous()
    if logit_scale != 1.0:
        tb[:, 0] *= logit_scale                      # head 0: logits of +-100 and more
        tb[:, 1, : n // 2] += 3.0 * logit_scale      # head 1: half of the queries far up ...
        tb[:, 1, n // 2:] -= 5.0 * logit_scale       # ... the others far down; heads 2, 3 stay moderate
    mask = (torch.rand(B, n, n, generator=gen) > 0.3).float().to(DEV)
    if logit_scale == 1.0:
        mask[:, 3, :] = 0  # a fully masked row (its -1e9 absorbs moderate logits only: ulp(1.44e9) = 128)
    mb = torch.full((B, n, np_), float("-inf"), device=DEV)
    mb[..., :n] = LOG2E * 1e9 * (mask - 1)
    o = torch.full((B, n, n, H * D), float("nan"), dtype=torch.bfloat16, device=DEV)
    print("triattn_flash", D, n, B, flush=True)
    vtp = _to_panels(vt)  # [b][i][h][d][j] -> [b][i][h][j/32][d][32]
    st = L.of3_triattn_flash(q.data_ptr(), k.data_ptr(), vtp.data_ptr(), tb.data_ptr(), mb.data_ptr(), o.data_ptr(),
                             B, n, H, D, stream())
    assert st == 0, L.of3_status_string(st)
    torch.cuda.synchronize()
    qf, kf, vf = q[:, :, :, :n].float(), k[:, :, :, :n].float(), vt[..., :n].float()
    s = torch.einsum("bihqd,bihkd->bihqk", qf, kf)
    s = (s + mb[:, :, None, None, :n]) + tb[:, None, :, :, :n]
    p = torch.softmax(s * math.log(2.0), dim=-1)
    want = torch.einsum("bihqk,bihdk->biqhd", p, vf).reshape(B, n, n, H * D)
    report("flash o", o, want, atol=2e-2, rtol=2e-2)


@pytest.mark.parametrize("seed", list(range(12)))
def test_triattn_flash_random_shapes(seed):
    """Seeded random shapes, mask densities and logit ranges: ragged N around the 32-key and 128-query
    tile sizes, work-groups that finish in the first pass next to ones that need the second."""
    import random

    L = lib()
    rnd = random.Random(1000 + seed)
    H = 4
    D = rnd.choice([16, 32])
    n = rnd.choice([1, 2, 31, 32, 33, 63, 65, 127, 128, 129, 160, 191, 193, 255, 257]) if seed < 8 else rnd.randint(1, 300)
    B = rnd.choice([1, 2])
    scale = rnd.choice([1.0, 1.0, 8.0, 30.0])
    density = rnd.choice([1.0, 0.9, 0.5])
    gen = _gen(7000 + seed)
    np_ = L.of3_padded_n(n)
    q = bf(_randn(gen, B, n, H, np_, D))
    k = bf(_randn(gen, B, n, H, np_, D))
    vt = bf(_randn(gen, B, n, H, D, np_))
    tb = (_randn(gen, B, H, n, np_) * scale).contiguous()
    mask = (torch.rand(B, n, n, generator=gen) < density).float().to(DEV)
    if scale == 1.0 and n > 3:
        mask[:, n // 2, :] = 0  # a fully masked row (moderate logits only: -1e9 absorbs |logit| < 64)
    else:
        mask[:, :, 0] = 1       # every row keeps a key, so the softmax does not hinge on the absorption
    mb = torch.full((B, n, np_), float("-inf"), device=DEV)
    mb[..., :n] = LOG2E * 1e9 * (mask - 1)
    o = torch.full((B, n, n, H * D), float("nan"), dtype=torch.bfloat16, device=DEV)
    print("flash random", seed, "D", D, "n", n, "B", B, "scale", scale, "density", density, flush=True)
    vtp = _to_panels(vt)
    st = L.of3_triattn_flash(q.data_ptr(), k.data_ptr(), vtp.data_ptr(), tb.data_ptr(), mb.data_ptr(), o.data_ptr(),
                             B, n, H, D, stream())
    assert st == 0, L.of3_status_string(st)
    torch.cuda.synchronize()
    qf, kf, vf = q[:, :, :, :n].float(), k[:, :, :, :n].float(), vt[..., :n].float()
    s = torch.einsum("bihqd,bihkd->bihqk", qf, kf)
    s = (s + mb[:, :, None, None, :n]) + tb[:, None, :, :, :n]
    p = torch.softmax(s * math.log(2.0), dim=-1)
    want = torch.einsum("bihqk,bihdk->biqhd", p, vf).reshape(B, n, n, H * D)
    report("flash o (random shapes)", o, want, atol=2e-2, rtol=2e-2)


@pytest.mark.parametrize("D,n,B,pads", [(32, 200, 2, "tail"), (16, 200, 2, "tail"), (32, 160, 1, "head"),
                                        (16, 97, 1, "middle"), (32, 300, 1, "outer")])
def test_triattn_flash_padding_masks(D, n, B, pads):
    """Block-shaped masks as padding produces them: runs of 32 and more masked keys (key tiles the
    kernel leaves out for rows that have an unmasked key) and rows whose keys are all masked (padded
    tokens: the reference's -1e9 absorbs the logits and the row becomes a uniform average; the kernel
    gets there in its first pass with the row's mask bias as the offset)."""
    L = lib()
    H = 4
    gen = _gen(911 + n + D)
    np_ = L.of3_padded_n(n)
    q = bf(_randn(gen, B, n, H, np_, D))
    k = bf(_randn(gen, B, n, H, np_, D))
    vt = bf(_randn(gen, B, n, H, D, np_))
    tb = _randn(gen, B, H, n, np_).contiguous()
    tok = torch.ones(B, n)
    if pads == "tail":
        tok[0, n - 70:] = 0
        if B > 1:
            tok[1, n - 33:] = 0
    elif pads == "head":
        tok[:, :45] = 0
    elif pads == "middle":
        tok[:, 20:60] = 0
    mask = (tok[:, :, None] * tok[:, None, :]).to(DEV)  # outer product: padded rows have no unmasked key
    if pads == "outer":  # keys masked in long runs for some rows only, every row keeps a key
        mask = torch.ones(B, n, n, device=DEV)
        mask[:, ::3, 64:200] = 0
        mask[:, 1::3, :96] = 0
    mb = torch.full((B, n, np_), float("-inf"), device=DEV)
    mb[..., :n] = LOG2E * 1e9 * (mask - 1)
    o = torch.full((B, n, n, H * D), float("nan"), dtype=torch.bfloat16, device=DEV)
    print("triattn_flash padding", D, n, B, pads, flush=True)
    vtp = _to_panels(vt)
    st = L.of3_triattn_flash(q.data_ptr(), k.data_ptr(), vtp.data_ptr(), tb.data_ptr(), mb.data_ptr(), o.data_ptr(),
                             B, n, H, D, stream())
    assert st == 0, L.of3_status_string(st)
    torch.cuda.synchronize()
    qf, kf, vf = q[:, :, :, :n].float(), k[:, :, :, :n].float(), vt[..., :n].float()
    s = torch.einsum("bihqd,bihkd->bihqk", qf, kf)
    s = (s + mb[:, :, None, None, :n]) + tb[:, None, :, :, :n]
    p = torch.softmax(s * math.log(2.0), dim=-1)
    want = torch.einsum("bihqk,bihdk->biqhd", p, vf).reshape(B, n, n, H * D)
    report("flash o (padding masks)", o, want, atol=2e-2, rtol=2e-2)
    if pads != "outer":  # a padded row is the plain average of v over all keys, for every query
        i_pad = int((tok[0] == 0).nonzero()[0])
        mean_v = vf[0, i_pad].mean(dim=-1)  # [h][d]
        got = o[0, i_pad].float().reshape(n, H, D)
        assert (got - mean_v[None]).abs().max() < 2e-2


@pytest.mark.parametrize("transposed,add_residual", [(False, 0), (True, 1)])
@pytest.mark.parametrize("C,D,n,B", [(128, 32, 70, 2), (64, 16, 130, 1), (128, 32, 5, 3), (128, 32, 150, 2)])
def test_triattn_out(transposed, add_residual, C, D, n, B):
    L = lib()
    H = 4
    gen = _gen(67 + n)
    zfull = bf(_randn(gen, B, n, n, C))
    x = zfull.transpose(1, 2) if transposed else zfull
    w = _triattn_weights(gen, C, H, D)
    o = bf(_randn(gen, B, n, n, H * D))
    out = torch.full_like(zfull, float("nan"))
    outv = out.transpose(1, 2) if transposed else out
    print("triattn_out", transposed, add_residual, C, D, n, B, flush=True)
    st = L.of3_triattn_out(o.data_ptr(), x.data_ptr(), s3(x), outv.data_ptr(), w["ln_w"].data_ptr(),
                           w["ln_b"].data_ptr(), w["g"].data_ptr(), w["o"].data_ptr(), B, n, C, H, D, add_residual,
                           stream())
    assert st == 0, L.of3_status_string(st)
    torch.cuda.synchronize()
    xn = bf(_ln(x, w["ln_w"], w["ln_b"])).float()
    og = bf(o.float() * torch.sigmoid(xn @ w["g"].float().t())).float()
    want = og @ w["o"].float().t()
    if add_residual:
        want = want + x.float()
    report("triattn_out", outv, want, atol=3e-2, rtol=1e-2)
