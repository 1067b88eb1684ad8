"""Writes tests/golden/pairstack_small.npz: known-answer vectors for the four pair-stack
modules at sizes the HIP kernels accept (c_z = 64, 4 heads of 16), computed by the float64
explicit-loop statement in oracle/brute_force.py.

The reference ships no golden vectors for these modules (its tests assert shapes, or compare
a fused CUDA kernel with its own PyTorch path at run time), so the vectors are produced here,
from the index formulas, and committed as data.  Inputs and weights are rounded to bf16
before the float64 evaluation so that a bf16 kernel and the fp32 oracle consume bit-identical
values.  Run from the repository root:  python tests/golden/make_fixtures.py
"""
import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

from oracle import brute_force as bf  # noqa: E402
from oracle import pairstack_oracle as orc  # noqa: E402

N, C, CH, HEADS, D = 10, 64, 64, 4, 16
SEED_W, SEED_Z, SEED_M = 0, 1, 2


def main():
    gen_w = torch.Generator().manual_seed(SEED_W)
    tm = {k: orc.round_bf16(v) for k, v in orc.make_trimul_params(gen_w, C, CH).items()}
    ta = {k: orc.round_bf16(v) for k, v in orc.make_triattn_params(gen_w, C, D, HEADS).items()}
    z = orc.round_bf16(torch.randn(N, N, C, generator=torch.Generator().manual_seed(SEED_Z)))
    mask = (torch.rand(N, N, generator=torch.Generator().manual_seed(SEED_M)) > 0.25).float()
    mask[3, :] = 0.0  # one fully masked row: uniform softmax over all keys
    mask[0, :] = 1.0

    out = {"z": z.numpy(), "mask": mask.numpy(),
           "dims": np.array([N, C, CH, HEADS, D]), "seeds": np.array([SEED_W, SEED_Z, SEED_M])}
    for k, v in tm.items():
        out["tm." + k] = v.numpy()
    for k, v in ta.items():
        out["ta." + k] = v.numpy()
    out["trimul_outgoing"] = bf.trimul_update(z, mask, tm, True).astype(np.float32)
    out["trimul_incoming"] = bf.trimul_update(z, mask, tm, False).astype(np.float32)
    out["triattn_starting"] = bf.triattn_update(z, mask, ta, HEADS, starting=True).astype(np.float32)
    out["triattn_ending"] = bf.triattn_update(z, mask, ta, HEADS, starting=False).astype(np.float32)
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "pairstack_small.npz")
    np.savez_compressed(path, **out)
    print(path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
