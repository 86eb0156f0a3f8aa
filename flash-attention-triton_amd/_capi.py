"""ctypes binding of libfa2_gfx950.so (declarations: include/fa2_gfx950.h).

The binding passes raw device pointers, sizes, element strides and the current HIP stream; it
holds no torch types in any signature.  There is no CPU or PyTorch fallback: if the library is
missing or reports an error, the caller gets an exception.
"""

from __future__ import annotations

import ctypes
import os
import pathlib
import threading

# The in-tree build; FA2_GFX950_LIBRARY names another build of the same ABI (e.g. one under test).
LIBRARY_PATH = pathlib.Path(os.environ.get("FA2_GFX950_LIBRARY") or
                            pathlib.Path(__file__).resolve().parent / "csrc" / "libfa2_gfx950.so")
ABI_VERSION = 5

FA2_DTYPE_F16 = 0
FA2_DTYPE_BF16 = 1
FA2_CONFIG_AUTO = -1
FA2_MAX_HEADDIM = 256
FA2_NOALLOC_MAX_ROWS = 4 << 20

_i, _i64, _f, _p = ctypes.c_int, ctypes.c_int64, ctypes.c_float, ctypes.c_void_p


class ConfigInfo(ctypes.Structure):
    """Mirror of ``fa2_config_info``: one row of the gfx950 tile/wave table."""

    _fields_ = [(name, ctypes.c_int) for name in (
        "id", "headdim_padded",
        "fwd_block_q", "fwd_block_kv", "fwd_waves",
        "bwd_block_q", "bwd_block_kv", "bwd_waves",
        "dq_block_q", "dq_block_kv", "dq_waves",
        "lds_direct", "fwd_wg_per_cu", "dq_wg_per_cu", "dkdv_wg_per_cu",
        "lds_stages", "dkdv_passes", "head_group", "dq_atomic", "fwd_exp_folded")]

    def as_dict(self) -> dict:
        return {name: getattr(self, name) for name, _ in self._fields_}


class Tensor(ctypes.Structure):
    """Mirror of ``fa2_tensor``: device pointer and the batch, head and sequence strides in elements."""

    _fields_ = [("ptr", _p), ("stride_batch", _i64), ("stride_head", _i64), ("stride_seq", _i64)]


class FwdArgs(ctypes.Structure):
    """Mirror of ``fa2_fwd_args``."""

    _fields_ = [("q", Tensor), ("k", Tensor), ("v", Tensor), ("o", Tensor), ("lse", _p),
                ("batch", _i), ("nheads", _i), ("seqlen_q", _i), ("seqlen_k", _i), ("headdim", _i),
                ("seqlen_q_rounded", _i), ("softmax_scale", _f), ("dtype", _i), ("config_id", _i)]


class BwdArgs(ctypes.Structure):
    """Mirror of ``fa2_bwd_args``."""

    _fields_ = [("q", Tensor), ("k", Tensor), ("v", Tensor), ("o", Tensor), ("d_o", Tensor),
                ("dq", Tensor), ("dk", Tensor), ("dv", Tensor), ("lse", _p), ("delta", _p),
                ("workspace", _p),
                ("batch", _i), ("nheads", _i), ("seqlen_q", _i), ("seqlen_k", _i), ("headdim", _i),
                ("seqlen_q_rounded", _i), ("softmax_scale", _f), ("dtype", _i), ("deterministic", _i),
                ("config_id", _i)]


# Every symbol include/fa2_gfx950.h declares, with its ctypes signature.
SIGNATURES = {
    "fa2_abi_version": (_i, []),
    "fa2_last_error_string": (ctypes.c_char_p, []),
    "fa2_status_string": (ctypes.c_char_p, [_i]),
    "fa2_config_count": (_i, []),
    "fa2_config_get": (_i, [_i, ctypes.POINTER(ConfigInfo)]),
    "fa2_pick_config": (_i, [_i, _i, _i, _i, _i]),
    "fa2_pick_config_forward_only": (_i, [_i, _i, _i, _i]),
    "fa2_fwd": (_i, [_p] * 5 + [_i] * 6 + [_i64] * 12 + [_f, _i, _i, _p]),
    "fa2_bwd_preprocess": (_i, [_p] * 3 + [_i] * 5 + [_i64] * 6 + [_i, _p]),
    "fa2_bwd_workspace_bytes": (ctypes.c_size_t, [_i] * 7),
    "fa2_bwd": (_i, [_p] * 10 + [_i] * 6 + [_i64] * 21 + [_f, _i, _i, _i, _p]),
    "fa2_bwd_fused": (_i, [_p] * 11 + [_i] * 6 + [_i64] * 24 + [_f, _i, _i, _i, _p]),
    "fa2_bwd_fused_noalloc": (_i, [_p] * 9 + [_i] * 6 + [_i64] * 24 + [_f, _i, _i, _i, _p]),
    "fa2_fwd_packed": (_i, [ctypes.POINTER(FwdArgs), _p]),
    "fa2_bwd_packed": (_i, [ctypes.POINTER(BwdArgs), _p]),
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
