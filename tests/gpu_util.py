"""Helpers shared by the GPU tests: library loading, raw C-ABI calls on torch tensors and
error reporting that names where the worst mismatch sits."""
import os
import sys

import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.join(ROOT, "openfold-3_amd")):
    if p not in sys.path:
        sys.path.insert(0, p)

from of3pair import _lib  # noqa: E402
from of3pair import build as of3_build  # noqa: E402


def lib():
    if not of3_build.is_built():
        of3_build.build()
    return _lib.load()


def stream():
    return torch.cuda.current_stream().cuda_stream


def s3(t):
    return _lib.strides3(t.stride()[:3])


def bf(t):
    return t.to(torch.bfloat16)


def report(name, got, want, atol, rtol=0.0):
    """Asserts |got - want| <= atol + rtol*|want| elementwise; the message names the worst
    element so that an indexing slip can be read off the failure."""
    got = got.float()
    want = want.float()
    assert got.shape == want.shape, "%s: shape %s vs %s" % (name, tuple(got.shape), tuple(want.shape))
    assert torch.isfinite(got).all(), "%s: non-finite values in output" % name
    err = (got - want).abs()
    bound = atol + rtol * want.abs()
    bad = err > bound
    if bad.any():
        idx = torch.nonzero(bad)
        worst = torch.argmax(err - bound)
        widx = tuple(int(v) for v in torch.unravel_index(worst, err.shape))
        raise AssertionError(
            "%s: %d / %d elements out of tolerance (atol %.3g rtol %.3g); worst at %s got %.6g want %.6g; "
            "first bad index %s; max |want| %.4g" % (
                name, int(bad.sum()), bad.numel(), atol, rtol, widx, float(got[widx]), float(want[widx]),
                tuple(int(v) for v in idx[0]), float(want.abs().max())))
    return float(err.max())
