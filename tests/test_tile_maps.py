"""The block -> tile numberings of the kernels, checked on the host: the check
program includes the kernels' own headers, is compiled with hipcc and runs on
the CPU (it launches nothing)."""

import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HIPCC = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"


@pytest.mark.skipif(not os.path.exists(HIPCC), reason="hipcc not installed")
def test_every_tile_and_row_is_visited_once(tmp_path):
    exe = tmp_path / "tile_maps_check"
    build = subprocess.run(
        [HIPCC, "--offload-arch=gfx950", "-std=c++20", "-O1",
         "-I", os.path.join(ROOT, "oslo_amd", "csrc"), "-I", os.path.join(ROOT, "include"),
         os.path.join(ROOT, "tests", "host", "tile_maps_check.hip"), "-o", str(exe)],
        capture_output=True, text=True)
    assert build.returncode == 0, build.stderr[-3000:]
    run = subprocess.run([str(exe)], capture_output=True, text=True, timeout=300)
    assert run.returncode == 0, run.stdout[-3000:]
    assert "tile maps ok" in run.stdout
