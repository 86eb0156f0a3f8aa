"""Index arithmetic of the fast kernels, checked on the CPU: tests/lds_layout_check.hip includes the
kernels' own headers (the swizzle, the tile loader's slot-to-chunk function, the workgroup mapping and the
head-group rule are host-callable), is compiled for the host only, walks every lane, wave and wave-load
of a tile for each padded head dimension and every workgroup of a range of grids."""

from __future__ import annotations

import pathlib
import subprocess

import pytest

ROOT = pathlib.Path(__file__).resolve().parent.parent
HIPCC = pathlib.Path("/opt/rocm/bin/hipcc")


def test_loader_slots_match_fragment_reads_and_reads_are_conflict_free(tmp_path):
    if not HIPCC.exists():
        pytest.skip("hipcc not installed")
    exe = tmp_path / "lds_layout_check"
    build = subprocess.run(
        [str(HIPCC), "-x", "hip", "--cuda-host-only", "-O1", "-std=c++17", "-Wno-unused-command-line-argument",
         f"-I{ROOT / 'flash-attention-triton_amd' / 'csrc'}", f"-I{ROOT / 'include'}",
         "-o", str(exe), str(ROOT / "tests" / "lds_layout_check.hip")],
        capture_output=True, text=True, timeout=300)
    assert build.returncode == 0, build.stderr[-2000:]
    run = subprocess.run([str(exe)], capture_output=True, text=True, timeout=60)
    assert run.returncode == 0, run.stdout + run.stderr
    lines = [l for l in run.stdout.splitlines() if l.startswith("DP")]
    assert len(lines) == 6 and all(l.endswith("ok") for l in lines), run.stdout
    mapping = [l for l in run.stdout.splitlines() if l.startswith("workgroup mapping")]
    assert len(mapping) == 1 and mapping[0].endswith("ok"), run.stdout
