"""The tile numbering of the 16x16x32 attention kernels, compiled for the host (tests/host/fa16_work_cover.cpp drives
the functions of mindie-sd_amd/csrc/fa16_work.hpp that the kernels themselves call through whole grids): every tile
taken exactly once by every numbering, and the causal numbering's work per XCD within 5 % of the mean."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def checker(tmp_path_factory):
    exe = str(tmp_path_factory.mktemp("fa16") / "fa16_work_cover")
    subprocess.run(["g++", "-O2", "-std=c++17", "-I", os.path.join(ROOT, "mindie-sd_amd", "csrc"),
                    os.path.join(ROOT, "tests", "host", "fa16_work_cover.cpp"), "-o", exe], check=True)
    return exe


@pytest.mark.parametrize("groups,tiles", [
    (12, 128),    # Wan2.1-1.3B: 12 heads, 32760 tokens in 256-row tiles
    (40, 296),    # Wan2.1-14B 720p
    (40, 128), (48, 70), (1, 1), (1, 2), (1, 7), (3, 5), (7, 9), (8, 8), (9, 1), (5, 64), (24, 131), (2, 1000),
])
def test_every_tile_once(checker, groups, tiles):
    res = subprocess.run([checker, str(groups), str(tiles)], capture_output=True, text=True)
    assert res.returncode == 0, res.stdout + res.stderr
    assert "checks passed" in res.stdout
