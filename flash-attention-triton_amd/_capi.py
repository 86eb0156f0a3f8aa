"""ctypes binding of libfa2_gfx950.so (declarations: include/fa2_gfx950.h).

The binding passes raw device pointers, sizes, element strides and the current HIP stream; it
holds no torch types in any signature.  There is no CPU or PyTorch fallback: if the library is
missing or reports an error, the caller gets an exception.
"""

from __future__ import annotations

import ctypes
import pathlib
import threading

LIBRARY_PATH = pathlib.Path(__file__).resolve().parent / "csrc" / "libfa2_gfx950.so"
ABI_VERSION = 1

FA2_DTYPE_F16 = 0
FA2_DTYPE_BF16 = 1
FA2_CONFIG_AUTO = -1
FA2_MAX_HEADDIM = 256

_i, _i64, _f, _p = ctypes.c_int, ctypes.c_int64, ctypes.c_float, ctypes.c_void_p


class ConfigInfo(ctypes.Structure):
    """Mirror of ``fa2_config_info``: one row of the gfx950 tile/wave table."""

    _fields_ = [(name, ctypes.c_int) for name in (
        "id", "headdim_padded",
        "fwd_block_q", "fwd_block_kv", "fwd_waves",
        "bwd_block_q", "bwd_block_kv", "bwd_waves",
        "dq_block_q", "dq_block_kv", "dq_waves")]

    def as_dict(self) -> dict:
        return {name: getattr(self, name) for name, _ in self._fields_}


# Every symbol include/fa2_gfx950.h declares, with its ctypes signature.
SIGNATURES = {
    "fa2_abi_version": (_i, []),
    "fa2_last_error_string": (ctypes.c_char_p, []),
    "fa2_status_string": (ctypes.c_char_p, [_i]),
    "fa2_config_count": (_i, []),
    "fa2_config_get": (_i, [_i, ctypes.POINTER(ConfigInfo)]),
    "fa2_pick_config": (_i, [_i, _i, _i, _i, _i]),
    "fa2_fwd": (_i, [_p] * 5 + [_i] * 6 + [_i64] * 12 + [_f, _i, _i, _p]),
    "fa2_bwd_preprocess": (_i, [_p] * 3 + [_i] * 5 + [_i64] * 6 + [_i, _p]),
    "fa2_bwd_workspace_bytes": (ctypes.c_size_t, [_i] * 7),
    "fa2_bwd": (_i, [_p] * 10 + [_i] * 6 + [_i64] * 21 + [_f, _i, _i, _i, _p]),
    "fa2_bwd_fused": (_i, [_p] * 11 + [_i] * 6 + [_i64] * 24 + [_f, _i, _i, _i, _p]),
}

_lib = None
_lock = threading.Lock()


def load() -> ctypes.CDLL:
    """Load the shared library once (thread-safe) and type every entry point."""
    global _lib
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is None:
            if not LIBRARY_PATH.exists():
                raise RuntimeError(
                    f"{LIBRARY_PATH} is missing: the HIP kernels are not built. "
                    "Build them with `python flash-attention-triton_amd/build.py` "
                    "(hipcc --offload-arch=gfx950); there is no fallback path."
                )
            lib = ctypes.CDLL(str(LIBRARY_PATH))
            for name, (restype, argtypes) in SIGNATURES.items():
                fn = getattr(lib, name)
                fn.restype = restype
                fn.argtypes = argtypes
            got = lib.fa2_abi_version()
            if got != ABI_VERSION:
                raise RuntimeError(f"libfa2_gfx950.so has ABI version {got}, binding expects {ABI_VERSION}")
            _lib = lib
    return _lib


def check(status: int, what: str) -> None:
    """Turn a non-zero fa2_status into RuntimeError carrying the library's message."""
    if status != 0:
        lib = load()
        name = lib.fa2_status_string(status).decode()
        detail = lib.fa2_last_error_string().decode()
        raise RuntimeError(f"{what} failed: {name}: {detail}")


def config_table() -> list[dict]:
    lib = load()
    rows = []
    for i in range(lib.fa2_config_count()):
        info = ConfigInfo()
        check(lib.fa2_config_get(i, ctypes.byref(info)), "fa2_config_get")
        rows.append(info.as_dict())
    return rows
