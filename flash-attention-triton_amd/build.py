"""Build libfa2_gfx950.so in-tree with hipcc (cross-compiles for gfx950 without a GPU), and the C++
autograd node that sits on top of its C ABI."""

from __future__ import annotations

import pathlib
import subprocess
import sysconfig

PACKAGE = pathlib.Path(__file__).resolve().parent
CSRC = PACKAGE / "csrc"
LIBRARY = CSRC / "libfa2_gfx950.so"
TORCH_EXTENSION = PACKAGE / "_fa2_torch.so"


def build_torch_extension() -> pathlib.Path:
    """Compile csrc/fa2_torch_autograd.cpp (host C++ only) against the installed PyTorch and link
    it to libfa2_gfx950.so.  Needs no GPU and no HIP compiler."""
    import torch
    from torch.utils import cpp_extension

    includes = [*cpp_extension.include_paths("cuda"), sysconfig.get_paths()["include"], str(PACKAGE.parent / "include")]
    cmd = ["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-Wno-deprecated-declarations",
           "-DTORCH_EXTENSION_NAME=_fa2_torch", "-DTORCH_API_INCLUDE_EXTENSION_H",
           "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1",
           f"-D_GLIBCXX_USE_CXX11_ABI={int(torch._C._GLIBCXX_USE_CXX11_ABI)}"]
    cmd += [f"-I{p}" for p in includes]
    cmd += [str(CSRC / "fa2_torch_autograd.cpp"), "-o", str(TORCH_EXTENSION)]
    cmd += [f"-L{p}" for p in cpp_extension.library_paths("cuda")]
    cmd += ["-lc10", "-lc10_hip", "-ltorch_cpu", "-ltorch_hip", "-ltorch", "-ltorch_python",
            f"-L{CSRC}", "-lfa2_gfx950", "-Wl,-rpath,$ORIGIN/csrc"]
    subprocess.run(cmd, check=True)
    return TORCH_EXTENSION


def build(force: bool = True) -> pathlib.Path:
    """Compile the HIP kernels, the C ABI and the C++ autograd node.  ``force`` rebuilds even if
    the libraries exist."""
    cmd = ["make", "-j5", "-C", str(CSRC)]
    if force:
        cmd.append("-B")
    subprocess.run(cmd, check=True)
    if not LIBRARY.exists():
        raise RuntimeError(f"build did not produce {LIBRARY}")
    if force or not TORCH_EXTENSION.exists():
        build_torch_extension()
    return LIBRARY


if __name__ == "__main__":
    print(build())
