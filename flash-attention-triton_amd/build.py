"""Build libfa2_gfx950.so in-tree with hipcc (cross-compiles for gfx950 without a GPU)."""

from __future__ import annotations

import pathlib
import subprocess

CSRC = pathlib.Path(__file__).resolve().parent / "csrc"
LIBRARY = CSRC / "libfa2_gfx950.so"


def build(force: bool = True) -> pathlib.Path:
    """Compile the HIP kernels and the C ABI.  ``force`` rebuilds even if the library exists."""
    cmd = ["make", "-j4", "-C", str(CSRC)]
    if force:
        cmd.append("-B")
    subprocess.run(cmd, check=True)
    if not LIBRARY.exists():
        raise RuntimeError(f"build did not produce {LIBRARY}")
    # The measurement probes next to the kernels (stand-alone executables under probes/bin).
    cmd = ["make", "-j2", "-C", str(CSRC / "probes")]
    if force:
        cmd.append("-B")
    subprocess.run(cmd, check=True)
    return LIBRARY


if __name__ == "__main__":
    print(build())
