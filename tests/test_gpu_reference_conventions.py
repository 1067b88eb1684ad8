"""The reference's own acceptance conventions for alternative kernels, applied to the HIP path
against the fp32 CPU oracle (openfold3/tests/test_kernels.py):

  * a single module: max-abs difference < 2e-2 (test_kernels.py:60,95-96 for attention on uniform
    [0, 1) inputs at n_res = 200 with 4 heads of 32 and a random 0/1 mask; :282-302 for the
    triangle multiplication on N(0,1) inputs, seq_len 84, c_z = c_hidden = 128, all-ones mask,
    several templates), every Linear re-initialised N(0, 1/fan_in) (:381-385);
  * a whole PairFormer block: mean-abs difference < 2e-2 after F.layer_norm over the channel
    dimension (:469-492), inputs uniform [0, 1), masks random 0/1;
  * the template embedder: max-abs difference < 2e-2 on its output, 3 templates, n_token = 200, a
    random 0/1 pair mask (:652-725; here from the output of the feature embedding on, which is where
    the replaced part begins).

These sit beside the stricter rms / noise-floor criteria of tests/test_gpu_parity.py; the achieved
figures are written to the parity summary."""
import pytest
import torch

from gpu_util import lib, record_parity  # noqa: F401
from oracle import pairstack_oracle as orc

import of3pair

pytestmark = pytest.mark.gpu
DEV = "cuda"
EPS = 2e-2


def _load(module, params, dtype):
    module.load_state_dict(params, strict=True)
    return module.to(DEV).to(dtype).eval()


def _inputs(dtype, *tensors):
    if dtype == torch.bfloat16:
        return [orc.round_bf16(t) for t in tensors]
    return list(tensors)


def _params(p, dtype):
    return {k: orc.round_bf16(v) for k, v in p.items()} if dtype == torch.bfloat16 else p


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("outgoing", [True, False])
def test_trimul_max_abs(dtype, outgoing):
    lib()
    n_tmpl, n, c = 4, 84, 128
    gen = torch.Generator().manual_seed(2024)
    p = _params(orc.make_trimul_params(gen, c, c), dtype)
    (z,) = _inputs(dtype, torch.randn(1, n_tmpl, n, n, c, generator=gen))
    mask = torch.ones(1, n_tmpl, n, n)
    cls = of3pair.TriangleMultiplicationOutgoing if outgoing else of3pair.TriangleMultiplicationIncoming
    m = _load(cls(c, c), p, dtype)
    got = m(z.to(DEV).to(dtype), mask=mask.to(DEV))
    want = orc.trimul_update(z, mask, p, outgoing)
    rec = record_parity("trimul update (reference convention)", got, want, None,
                        "max|err| < 2e-2" if dtype == torch.float32 else
                        "PASSES ON max|err| <= error of the oracle run in bfloat16 (2.8-3.1e-2), NOT on 2e-2; the "
                        "reference states this test in fp32 only")
    bound = EPS
    if dtype == torch.bfloat16:
        # The reference states this test in fp32 only.  In bf16 the outputs reach |4|, where half a
        # bf16 ulp is already 1.6e-2: the reference's own bf16 path (the oracle's operations run in
        # bfloat16) is the yardstick wherever it lies above 2e-2.
        ref16 = orc.trimul_update(z.to(torch.bfloat16), mask.to(torch.bfloat16),
                                  {k: v.to(torch.bfloat16) for k, v in p.items()}, outgoing)
        bound = max(EPS, float((ref16.float() - want).abs().max()))
        print("bf16 reference path max|err| = %.4g, HIP path %.4g" % (bound, rec["max_abs_err"]), flush=True)
    assert rec["max_abs_err"] <= bound, rec


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("starting", [True, False])
def test_triattn_max_abs(dtype, starting):
    lib()
    n, c, d, heads = 200, 128, 32, 4
    gen = torch.Generator().manual_seed(2025)
    p = _params(orc.make_triattn_params(gen, c, d, heads), dtype)
    (x,) = _inputs(dtype, torch.rand(1, n, n, c, generator=gen))
    mask = torch.randint(0, 2, (1, n, n), generator=gen).float()
    m = _load(of3pair.TriangleAttention(c, d, heads, starting=starting), p, dtype)
    got = m(x.to(DEV).to(dtype), mask=mask.to(DEV))
    want = orc.triattn_update(x, mask, p, heads, starting=starting, row_chunk=50)
    rec = record_parity("triattn update (reference convention)", got, want, None, "max|err| < 2e-2")
    assert rec["max_abs_err"] < EPS, rec


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_pairformer_block_mean_abs_after_layer_norm(dtype):
    lib()
    n, cs, cz = 96, 384, 128
    p = _params(orc.make_pairformer_block_params(33, cs, cz, 128, 32, 4, 24, 16, 4), dtype)
    gen = torch.Generator().manual_seed(2026)
    s, z = _inputs(dtype, torch.rand(1, n, cs, generator=gen), torch.rand(1, n, n, cz, generator=gen))
    single_mask = torch.randint(0, 2, (1, n), generator=gen).float()
    pair_mask = torch.randint(0, 2, (1, n, n), generator=gen).float()
    blk = of3pair.PairFormerBlock(c_s=cs, c_z=cz, c_hidden_pair_bias=24, no_heads_pair_bias=16, c_hidden_mul=128,
                                  c_hidden_pair_att=32, no_heads_pair=4, transition_type="swiglu", transition_n=4,
                                  pair_dropout=0.25, fuse_projection_weights=False, inf=1e9)
    blk = _load(blk, p, dtype)
    s_got, z_got = blk(s.to(DEV).to(dtype), z.to(DEV).to(dtype), single_mask.to(DEV), pair_mask.to(DEV))
    s_want, z_want = orc.pairformer_block(s, z, single_mask, pair_mask, p, 4, 16)
    F = torch.nn.functional
    for name, got, want, c in (("s", s_got, s_want, cs), ("z", z_got, z_want, cz)):
        g = F.layer_norm(got.float().cpu(), (c,))
        w = F.layer_norm(want, (c,))
        rec = record_parity("pairformer block %s after layer_norm (reference convention)" % name, g, w, None,
                            "mean|err| < 2e-2")
        assert rec["mean_abs_err"] < EPS, rec


STACK_CFG = dict(c_t=64, c_hidden_tri_att=16, c_hidden_tri_mul=64, no_blocks=2, no_heads=4,
                 transition_type="swiglu", pair_transition_n=2, dropout_rate=0.25, tri_mul_first=True,
                 fuse_projection_weights=False, blocks_per_ckpt=None, inf=1e9, use_reentrant=False,
                 tune_chunk_size=False)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_template_embedder_max_abs(dtype):
    lib()
    n, nt, ct, cz = 200, 3, 64, 128
    gen = torch.Generator().manual_seed(2027)
    blocks = []
    for seed in range(2):
        b = dict(orc.make_block_params(60 + seed, ct, ct, 16, 4))
        b.update({"pair_transition." + k: v for k, v in orc.make_transition_params(gen, ct, 2).items()})
        blocks.append(_params(b, dtype))
    tail = _params(orc.make_template_tail_params(gen, ct, cz), dtype)
    (emb,) = _inputs(dtype, torch.rand(1, nt, n, n, ct, generator=gen))
    pair_mask = torch.randint(0, 2, (1, n, n), generator=gen).float()
    core = of3pair.TemplateEmbedderCore(ct, cz, STACK_CFG)
    sd = {}
    for i, b in enumerate(blocks):
        sd.update({"template_pair_stack.blocks.%d.%s" % (i, k): v for k, v in b.items()})
    sd.update(tail)
    core.load_state_dict(sd, strict=True)
    core = core.to(DEV).to(dtype).eval()
    got = core(emb.to(DEV).to(dtype), pair_mask.to(DEV))
    tn = orc.template_stack(emb, pair_mask[:, None], blocks, tail["template_pair_stack.layer_norm.weight"],
                            tail["template_pair_stack.layer_norm.bias"], 4)
    want = orc.template_tail(tn, tail["linear_t.weight"])
    rec = record_parity("template embedder output (reference convention)", got, want, None,
                        "max|err| < 2e-2" if dtype == torch.float32 else
                        "PASSES ON max|err| <= error of the oracle run in bfloat16 (5.5e-2), NOT on 2e-2")
    bound = EPS
    if dtype == torch.bfloat16:
        # as for the triangle multiplication above: where the reference's own bf16 path (the oracle's
        # operations run in bfloat16) lies above 2e-2, it is the yardstick
        bf = torch.bfloat16
        b16 = [{k: v.to(bf) for k, v in b.items()} for b in blocks]
        t16 = {k: v.to(bf) for k, v in tail.items()}
        tn16 = orc.template_stack(emb.to(bf), pair_mask[:, None].to(bf), b16, t16["template_pair_stack.layer_norm.weight"],
                                  t16["template_pair_stack.layer_norm.bias"], 4)
        ref16 = orc.template_tail(tn16, t16["linear_t.weight"])
        bound = max(EPS, float((ref16.float() - want).abs().max()))
        print("bf16 reference path max|err| = %.4g, HIP path %.4g" % (bound, rec["max_abs_err"]), flush=True)
    assert rec["max_abs_err"] <= bound, rec
