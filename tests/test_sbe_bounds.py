"""The index arithmetic of the block-mask estimate kernels, compiled for the host (tests/host/sbe_bounds.cpp walks
the kernels' loops with the functions of mindie-sd_amd/csrc/sbe_index.hpp that the kernels themselves use) and
driven through whole launches with a bounds assertion on every access: the long-sequence shapes of the two DiT
workloads, both layouts, causal and not, heads processed in one or several workspace groups."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def checker(tmp_path_factory):
    exe = str(tmp_path_factory.mktemp("sbe") / "sbe_bounds")
    subprocess.run(["g++", "-O2", "-std=c++17", "-I", os.path.join(ROOT, "mindie-sd_amd", "csrc"),
                    os.path.join(ROOT, "tests", "host", "sbe_bounds.cpp"), "-o", exe], check=True)
    return exe


@pytest.mark.parametrize("s,heads,n,layout,causal,ws_heads", [
    (32760, 12, 12, 0, 0, 12),     # Wan2.1-1.3B shape
    (32760, 12, 12, 1, 1, 5),
    (75600, 40, 40, 0, 0, 40),     # Wan2.1-14B 720p shape
    (75600, 40, 40, 1, 1, 7),
    (8192, 16, 16, 0, 0, 16),      # the reference's own test shape
    (1031, 4, 2, 1, 1, 3), (128, 1, 1, 0, 0, 1), (1, 1, 1, 0, 1, 1), (2049, 2, 2, 0, 1, 1),
])
def test_every_access_in_range(checker, s, heads, n, layout, causal, ws_heads):
    res = subprocess.run([checker, str(s), str(heads), str(n), str(layout), str(causal), str(ws_heads)],
                         capture_output=True, text=True)
    assert res.returncode == 0, res.stdout + res.stderr
    assert "checks passed" in res.stdout
