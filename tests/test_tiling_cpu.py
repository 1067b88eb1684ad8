"""The tiling of the position-wise passes and the order of the attention core's work-groups
(openfold-3_amd/csrc/of3_tiles.h) checked on the host: the header is plain C++ that the kernels and
tests/tiling_check.cpp both compile, so the index arithmetic that decides which addresses a tile touches is
exercised here for every small token count and a spread of larger ones, without a GPU."""
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.mark.skipif(shutil.which("g++") is None, reason="needs a host C++ compiler")
def test_tiles_stay_inside_and_cover_every_position(tmp_path):
    exe = str(tmp_path / "tiling_check")
    subprocess.run(["g++", "-std=c++17", "-O1", "-I" + os.path.join(ROOT, "openfold-3_amd", "csrc"),
                    os.path.join(ROOT, "tests", "tiling_check.cpp"), "-o", exe], check=True)
    counts = list(range(1, 140)) + [150, 160, 161, 191, 192, 193, 200, 255, 256, 257, 291, 300, 383, 384, 385, 500, 640, 700,
                                    768, 769, 1025, 1100, 2048, 2100]
    out = subprocess.run([exe] + [str(n) for n in counts], capture_output=True, text=True)
    assert out.returncode == 0, out.stdout[-400:]
    assert out.stdout.count("ok ") == len(counts)
