"""Builds libof3pair.so (HIP, gfx950 only) in-tree with hipcc.

    python -m of3pair.build            # from the openfold-3_amd directory

The library lands in openfold-3_amd/lib/libof3pair.so next to its objects; nothing is
installed outside the tree.
"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(PKG_DIR)
CSRC = os.path.join(ROOT, "csrc")
LIB_DIR = os.path.join(ROOT, "lib")
LIB_PATH = os.path.join(LIB_DIR, "libof3pair.so")

SOURCES = [
    "of3pair_api.hip",
    "trimul_proj.hip",
    "trimul_contract.hip",
    "trimul_out.hip",
    "triattn_proj.hip",
    "triattn_flash.hip",
    "triattn_out.hip",
    "transition.hip",
    "pair_bias.hip",
    "template_tail.hip",
    "single_attn.hip",
    "single_transition.hip",
    "pair_f32.hip",
    "single_f32.hip",
]

# packed fp32 VALU ops are disabled on purpose (device code only)
HIPCC_FLAGS = [
    "-O3",
    "--offload-arch=gfx950",
    "-std=c++17",
    "-fPIC",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def _hipcc() -> str:
    return os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")


def _run(cmd):
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    # the host pass does not know the packed-fp32 feature and says so; that line is noise
    out = "\n".join(l for l in proc.stdout.splitlines() if "packed-fp32-ops" not in l)
    if proc.returncode != 0:
        raise RuntimeError("command failed: %s\n%s" % (" ".join(cmd), out))
    return out


def build(verbose: bool = False, jobs: int = 4) -> str:
    os.makedirs(LIB_DIR, exist_ok=True)
    objs = []

    def compile_one(src):
        obj = os.path.join(LIB_DIR, os.path.splitext(src)[0] + ".o")
        out = _run([_hipcc(), *HIPCC_FLAGS, "-c", os.path.join(CSRC, src), "-o", obj])
        if verbose and out.strip():
            print(out)
        return obj

    with ThreadPoolExecutor(max_workers=jobs) as ex:
        objs = list(ex.map(compile_one, SOURCES))
    _run([_hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB_PATH, *objs])
    return LIB_PATH


def is_built() -> bool:
    return os.path.exists(LIB_PATH)


if __name__ == "__main__":
    print(build(verbose="-v" in sys.argv))
