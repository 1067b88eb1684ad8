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


PARITY_RECORDS = []


def record_parity(name, got, want, bf16_ref=None, bound=None):
    """Keeps the achieved error figures of one comparison; when the session ends, tests/conftest.py
    writes them to the file the environment variable OF3_PARITY_SUMMARY names (nothing is written
    without it).  `bound` describes the assertion the figures were held against."""
    got, want = got.float().cpu(), want.float().cpu()
    err = (got - want).abs()
    rms_want = float(want.pow(2).mean().sqrt())
    rec = {
        "test": os.environ.get("PYTEST_CURRENT_TEST", "?").split(" ")[0].split("::", 1)[-1],
        "tensor": name, "elements": want.numel(),
        "max_abs_err": float(err.max()), "max_abs_want": float(want.abs().max()),
        "rms_err": float(err.pow(2).mean().sqrt()), "rms_want": rms_want,
        "mean_abs_err": float(err.mean()),
        "floor_rms": None if bf16_ref is None else float((bf16_ref.float().cpu() - want).pow(2).mean().sqrt()),
        "bound": bound or "",
    }
    PARITY_RECORDS.append(rec)
    return rec


def write_parity_summary(path):
    if not PARITY_RECORDS:
        return
    os.makedirs(os.path.dirname(os.path.abspath(path)), exist_ok=True)
    with open(path, "w") as f:
        f.write("# achieved errors of the GPU parity tests (HIP path vs fp32 CPU oracle), one line per compared tensor\n")
        f.write("# max_rel = max|err| / max|want| ; rms_rel = rms(err) / rms(want) ; floor = rms(err) / rms error of the\n")
        f.write("# oracle run in bfloat16 at the reference's rounding points (blank where the test has no such leg)\n")
        f.write("%-86s %-34s %10s %10s %9s %9s %9s %6s  %s\n" % ("test", "tensor", "max|err|", "max|want|", "max_rel",
                                                                  "rms_rel", "mean|err|", "floor", "bound"))
        for r in PARITY_RECORDS:
            floor = "" if not r["floor_rms"] else "%.2f" % (r["rms_err"] / r["floor_rms"])
            f.write("%-86s %-34s %10.3e %10.3e %9.2e %9.2e %9.2e %6s  %s\n" % (
                r["test"][:86], r["tensor"][:34], r["max_abs_err"], r["max_abs_want"],
                r["max_abs_err"] / max(r["max_abs_want"], 1e-30), r["rms_err"] / max(r["rms_want"], 1e-30),
                r["mean_abs_err"], floor, r["bound"]))
