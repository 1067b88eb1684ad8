"""Known-answer vectors committed under tests/golden/ (float64 brute force, see
tests/golden/make_fixtures.py): the fp32 oracle must reproduce them on the CPU, and the HIP
modules must reproduce them on the GPU through the C-ABI within the bf16 tolerance."""
import os

import numpy as np
import pytest
import torch

from oracle import pairstack_oracle as orc

FIX = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "pairstack_small.npz")
FP32_TOL = 1e-4      # max-abs, fp32 path
BF16_REL = 2e-2      # max-abs relative to the largest expected magnitude, bf16 path


@pytest.fixture(scope="module")
def fx():
    d = np.load(FIX)
    get = lambda pre: {k[len(pre):]: torch.from_numpy(d[k]) for k in d.files if k.startswith(pre)}
    return d, torch.from_numpy(d["z"]), torch.from_numpy(d["mask"]), get("tm."), get("ta.")


def test_fixture_inputs_are_bf16_representable(fx):
    d, z, _, tm, ta = fx
    for t in [z, *tm.values(), *ta.values()]:
        assert torch.equal(t, t.bfloat16().float())


@pytest.mark.parametrize("outgoing", [True, False])
def test_oracle_trimul_reproduces_fixture(fx, outgoing):
    d, z, mask, tm, _ = fx
    got = orc.trimul_update(z, mask, tm, outgoing).numpy()
    want = d["trimul_outgoing" if outgoing else "trimul_incoming"]
    assert np.abs(got - want).max() < FP32_TOL


@pytest.mark.parametrize("starting", [True, False])
def test_oracle_triattn_reproduces_fixture(fx, starting):
    d, z, mask, _, ta = fx
    heads = int(d["dims"][3])
    got = orc.triattn_update(z, mask, ta, heads, starting=starting).numpy()
    want = d["triattn_starting" if starting else "triattn_ending"]
    assert np.abs(got - want).max() < FP32_TOL


def _bound(got, want):
    err = np.abs(got - want).max()
    assert err <= BF16_REL * np.abs(want).max(), (err, np.abs(want).max())


@pytest.mark.gpu
@pytest.mark.parametrize("outgoing", [True, False])
def test_gpu_trimul_reproduces_fixture(fx, outgoing):
    import of3pair

    d, z, mask, tm, _ = fx
    _, c, ch = (int(v) for v in d["dims"][:3])
    cls = of3pair.TriangleMultiplicationOutgoing if outgoing else of3pair.TriangleMultiplicationIncoming
    m = cls(c, ch)
    m.load_state_dict(tm)
    m = m.to("cuda", torch.bfloat16).eval()
    got = m(z.to("cuda", torch.bfloat16)[None], mask=mask.cuda()[None])[0].float().cpu().numpy()
    _bound(got, d["trimul_outgoing" if outgoing else "trimul_incoming"])


@pytest.mark.gpu
@pytest.mark.parametrize("starting", [True, False])
def test_gpu_triattn_reproduces_fixture(fx, starting):
    import of3pair

    d, z, mask, _, ta = fx
    _, c, _, heads, hd = (int(v) for v in d["dims"])
    m = of3pair.TriangleAttention(c, hd, heads, starting=starting)
    m.load_state_dict(ta)
    m = m.to("cuda", torch.bfloat16).eval()
    got = m(z.to("cuda", torch.bfloat16)[None], mask=mask.cuda()[None])[0].float().cpu().numpy()
    _bound(got, d["triattn_starting" if starting else "triattn_ending"])
