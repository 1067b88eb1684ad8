"""Builds libof3pair.so (HIP, gfx950 only) in-tree with hipcc.

    python -m of3pair.build            # from the openfold-3_amd directory

The library lands in openfold-3_amd/lib/libof3pair.so next to its objects; nothing is
installed outside the tree.
"""
from __future__ import annotations

import hashlib
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(PKG_DIR)
CSRC = os.path.join(ROOT, "csrc")
LIB_DIR = os.path.join(ROOT, "lib")
LIB_PATH = os.path.join(LIB_DIR, "libof3pair.so")
STAMP_PATH = os.path.join(LIB_DIR, "libof3pair.sources.sha256")
INCLUDE_DIR = os.path.join(os.path.dirname(ROOT), "include")

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


def _flags():
    """The compiler flags, plus what OF3_HIPCC_EXTRA adds (e.g. -DOF3_FLASH_WIDE_FROM=1 to run the tests on a
    kernel variant that the default thresholds would not pick at the tests' sizes)."""
    return HIPCC_FLAGS + os.environ.get("OF3_HIPCC_EXTRA", "").split()


def _hipcc() -> str:
    return os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")


def _run(cmd):
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    # the host pass does not know the packed-fp32 feature and says so; that line is noise
    out = "\n".join(l for l in proc.stdout.splitlines() if "packed-fp32-ops" not in l)
    if proc.returncode != 0:
        raise RuntimeError("command failed: %s\n%s" % (" ".join(cmd), out))
    return out


def source_digest() -> str:
    """sha256 over everything the library is compiled from: the kernel sources and headers, the public
    header and the compiler flags."""
    h = hashlib.sha256(" ".join(_flags()).encode())
    files = [os.path.join(CSRC, f) for f in SOURCES]
    files += [os.path.join(CSRC, f) for f in sorted(os.listdir(CSRC)) if f.endswith(".h")]
    if os.path.isdir(INCLUDE_DIR):
        files += [os.path.join(INCLUDE_DIR, f) for f in sorted(os.listdir(INCLUDE_DIR)) if f.endswith(".h")]
    for path in files:
        h.update(os.path.basename(path).encode())
        with open(path, "rb") as fh:
            h.update(fh.read())
    return h.hexdigest()


def build(verbose: bool = False, jobs: int = 4) -> str:
    os.makedirs(LIB_DIR, exist_ok=True)
    digest = source_digest()
    if os.path.exists(STAMP_PATH):
        os.remove(STAMP_PATH)  # no stamp while the objects are in flux
    objs = []

    def compile_one(src):
        obj = os.path.join(LIB_DIR, os.path.splitext(src)[0] + ".o")
        out = _run([_hipcc(), *_flags(), "-c", os.path.join(CSRC, src), "-o", obj])
        if verbose and out.strip():
            print(out)
        return obj

    with ThreadPoolExecutor(max_workers=jobs) as ex:
        objs = list(ex.map(compile_one, SOURCES))
    _run([_hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB_PATH, *objs])
    with open(STAMP_PATH, "w") as fh:
        fh.write(digest + "\n")
    return LIB_PATH


def is_built() -> bool:
    """True when the library exists and was built from the sources as they are now (the stamp
    written next to it holds the digest of the sources of that build)."""
    return os.path.exists(LIB_PATH) and not is_stale()


def is_stale() -> bool:
    """True when a library exists whose sources are known to have changed since it was built (a
    library without a stamp, e.g. one copied in from elsewhere, cannot be judged and is accepted)."""
    if not os.path.exists(LIB_PATH) or not os.path.exists(STAMP_PATH):
        return False
    with open(STAMP_PATH) as fh:
        return fh.read().strip() != source_digest()


if __name__ == "__main__":
    print(build(verbose="-v" in sys.argv))
