"""FlashAttention-2 for AMD MI355X (gfx950): public API and autograd boundary.

Drop-in for ``flash_attention_triton.flash_attention_2`` of the reference
(src/flash_attention_triton/flash_attention_2.py): same public functions, same
``torch.autograd.Function`` contract, same assertion and exception types; the device work is
done by hand-written HIP kernels reached through the C ABI of ``libfa2_gfx950.so``.

Differences from the reference, all deliberate:

* bf16 inputs are computed with bf16 MFMA; the reference down-casts everything to fp16
  (flash_attention_2.py:316).  fp16 inputs use fp16 MFMA; any other dtype is down-cast to fp16
  and the output cast back, as in the reference.
* fp16/bf16 contiguous inputs are used as they are: no cast or copy kernels run.
* A forward that nothing will differentiate (under ``torch.no_grad()``, or with no input that
  requires a gradient) on bf16 inputs up to head dimension 128 multiplies Q by
  softmax_scale * log2(e) and rounds it to bf16 once, so that the score MFMAs deliver base-2
  exponents (4 % less time; the reference scales the fp32 scores, _triton_kernels_v2.py:137-152).
  Whenever a backward may follow, and always for fp16, the forward uses the reference's arithmetic:
  the backward recomputes the probabilities from Q itself and needs the log-sum-exp of exactly those
  scores.  ``KernelsConfigV2.exact_scale`` (through ``flash_attention_v2_custom``) or
  ``FA2_GFX950_EXACT_SCALE=1`` keeps the reference's arithmetic everywhere.
* The configuration selector knows one architecture, gfx950.
* ``deterministic=True`` does not serialise the backward into one program per head
  (flash_attention_2.py:204-207): dQ is produced by a query-tile-parallel kernel that accumulates
  in a fixed order without atomics.
* When the C++ autograd node is built (``_fa2_torch``, csrc/fa2_torch_autograd.cpp) the public
  functions record that node instead of the Python ``FlashAttentionV2Function``: same launches,
  same results, a third of the host time per step (the backward engine runs a C++ node on its
  device thread without the interpreter).  ``FA2_GFX950_PYTHON_AUTOGRAD=1`` keeps the Python class.
"""

from __future__ import annotations

import math
import os
import threading

import torch

from . import _capi
from ._configurators_v2 import BackwardConfig, KernelsConfigV2, init_to_zero_v2

# Architecture this package is written for, and what torch reports for it.
_GFX950_ARCH_PREFIX = "gfx950"
_MIN_CC = (9, 5)

_COMPUTE_DTYPES = {torch.float16: _capi.FA2_DTYPE_F16, torch.bfloat16: _capi.FA2_DTYPE_BF16}


# ================================ AUTOGRAD INTEGRATION ================================
def _strides3(t: torch.Tensor) -> tuple[int, int, int]:
    return t.stride(0), t.stride(1), t.stride(2)


_RAW_STREAM = getattr(torch._C, "_cuda_getCurrentRawStream", None)
# The binding functions behind torch.cuda.current_device(): the public wrappers add a lazy-init
# check per call, about a microsecond each, which shows at the smallest problem sizes.
_RAW_DEVICE = getattr(torch._C, "_cuda_getDevice", None) or torch.cuda.current_device


def _stream_handle() -> int:
    """hipStream_t of torch's current stream on the current device, as an integer."""
    if _RAW_STREAM is not None:  # same value as below without building a Stream object (~10 us)
        return _RAW_STREAM(_RAW_DEVICE())
    return torch.cuda.current_stream().cuda_stream


class _NoGuard:
    """Stands in for torch.cuda.device(...) when the tensors already live on the current device
    (the usual case): entering a device guard costs several microseconds per launch."""

    def __enter__(self):
        return None

    def __exit__(self, *exc):
        return False


_NO_GUARD = _NoGuard()

# Argument records of the packed entry points, kept per problem signature and per thread (a record
# is filled in and handed to the library by one thread at a time).
_FWD_ARGS: dict = {}
_BWD_ARGS: dict = {}
_MAX_RECORDS = 256


def _remember(table: dict, key, value) -> None:
    if len(table) >= _MAX_RECORDS:
        table.clear()
    table[key] = value


def _device_guard(device: torch.device):
    if device.index is None or device.index == _RAW_DEVICE():
        return _NO_GUARD
    return torch.cuda.device(device)


def _assert_forward_inputs(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, max_headdim: int) -> None:
    """The forward launcher's input checks (reference: flash_attention_2.py:85-90)."""
    batch, nheads, _, headdim = q.shape
    _, _, seqlen_k, _ = k.shape
    assert k.shape == (batch, nheads, seqlen_k, headdim)
    assert v.shape == (batch, nheads, seqlen_k, headdim)
    assert headdim <= max_headdim, f"Supports head dimensions only up to {max_headdim}"
    assert q.is_cuda and k.is_cuda and v.is_cuda, "All tensors must reside on CUDA device"
    assert q.dtype == k.dtype == v.dtype, "All tensors must be the same type"
    assert q.dtype in _COMPUTE_DTYPES, "Supports only fp16 and bf16"
    assert q.stride(-1) == k.stride(-1) == v.stride(-1) == 1, "Last dimension must be contiguous"


def _flash_attention_forward(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    softmax_scale: float | None,
    block_rows_size: int,
    block_cols_size: int,
    min_block_headdim: int,
    max_headdim: int,
    seqlen_cache_divisor: int,
    min_warps: int,
    max_warps: int,
    num_stages: int,
    forward_only: bool = False,
) -> tuple[torch.Tensor, torch.Tensor, float]:
    """Validate inputs, allocate O and the log-sum-exp, launch the forward kernel.

    Same signature, checks and return value as the reference launcher
    (flash_attention_2.py:61-144).  The tile arguments are accepted for compatibility; the tile
    shape comes from the table inside the library.  ``forward_only`` (not in the reference) says
    that no backward will read the log-sum-exp: the library may then pick a row whose forward folds
    the softmax scale into Q (``fa2_pick_config_forward_only``; bf16 up to head dimension 128).
    """
    batch, nheads, seqlen_q, headdim = q.shape
    _, _, seqlen_k, _ = k.shape

    _assert_forward_inputs(q, k, v, max_headdim)

    output = torch.empty_like(q)
    softmax_scale = softmax_scale or 1.0 / math.sqrt(headdim)

    # Row length of lse padded to a multiple of max_headdim (reference: flash_attention_2.py:98-99)
    seqlen_q_rounded = math.ceil(seqlen_q / max_headdim) * max_headdim
    lse = torch.empty((batch, nheads, seqlen_q_rounded), device=q.device, dtype=torch.float32)

    # The kernels take a positive scale.  A negative one (the reference passes any non-zero value
    # through) is folded into the sign of Q, which is exact: (-Q) K^T * |s| == Q K^T * s.
    q_in, kernel_scale = (q, softmax_scale) if softmax_scale > 0 else (-q, -softmax_scale)

    # One argument record per (shapes, strides, dtype, scale), kept between calls: only the five
    # pointers change from call to call.
    config_id = _forward_only_row(q.dtype, headdim, seqlen_q, seqlen_k) if forward_only else _capi.FA2_CONFIG_AUTO
    key = (q_in.shape, seqlen_k, q_in.stride(), k.stride(), v.stride(), output.stride(), q.dtype,
           seqlen_q_rounded, kernel_scale, config_id, threading.get_ident())
    args = _FWD_ARGS.get(key)
    if args is None:
        args = _capi.FwdArgs()
        for name, t in (("q", q_in), ("k", k), ("v", v), ("o", output)):
            rec = getattr(args, name)
            rec.stride_batch, rec.stride_head, rec.stride_seq = _strides3(t)
        args.batch, args.nheads, args.seqlen_q, args.seqlen_k = batch, nheads, seqlen_q, seqlen_k
        args.headdim, args.seqlen_q_rounded = headdim, seqlen_q_rounded
        args.softmax_scale, args.dtype = kernel_scale, _COMPUTE_DTYPES[q.dtype]
        args.config_id = config_id
        _remember(_FWD_ARGS, key, args)
    args.q.ptr, args.k.ptr, args.v.ptr = q_in.data_ptr(), k.data_ptr(), v.data_ptr()
    args.o.ptr, args.lse = output.data_ptr(), lse.data_ptr()

    lib = _capi.load()
    with _device_guard(q.device):
        status = lib.fa2_fwd_packed(args, _stream_handle())
    if status:
        _capi.check(status, "fa2_fwd")
    return output, lse, softmax_scale  # softmax_scale could have been updated


def _flash_attention_backward(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    output: torch.Tensor,
    lse: torch.Tensor,
    dq: torch.Tensor,
    dk: torch.Tensor,
    dv: torch.Tensor,
    d_output: torch.Tensor,
    softmax_scale: float | None,
    kernels_config: KernelsConfigV2,
) -> None:
    """Fill caller-allocated dq, dk, dv in place (reference: flash_attention_2.py:147-277)."""
    batch, nheads, seqlen_q, headdim = q.shape
    _, _, seqlen_k, _ = k.shape

    if not d_output.is_contiguous():
        d_output = d_output.contiguous()

    max_headdim = kernels_config.max_headdim
    seqlen_q_rounded = math.ceil(seqlen_q / max_headdim) * max_headdim

    assert headdim <= max_headdim
    assert lse.shape == (batch, nheads, seqlen_q_rounded)
    assert (
        q.is_contiguous()
        == k.is_contiguous()
        == v.is_contiguous()
        == output.is_contiguous()
        == True  # noqa: E712
    )
    assert dq.is_contiguous() == dk.is_contiguous() == dv.is_contiguous() == True  # noqa: E712
    assert q.dtype in _COMPUTE_DTYPES, "Supports only fp16 and bf16"
    assert d_output.dtype == q.dtype == output.dtype, "All tensors must be the same type"

    delta = torch.empty_like(lse)
    softmax_scale = softmax_scale or 1.0 / math.sqrt(headdim)
    deterministic = 1 if kernels_config.deterministic else 0
    config_id = _atomic_row(headdim) if kernels_config.atomic_dq else _capi.FA2_CONFIG_AUTO

    # Negative scale: run on -Q with |scale| (see the forward launcher); dK and dV are unchanged
    # and dQ comes out with the opposite sign.
    negated = softmax_scale < 0
    if negated:
        q, softmax_scale = -q, -softmax_scale

    # Both launches of the reference launcher (preprocess, then the main kernel) in one call:
    # with `o` in the record the library forms delta on the way.  Every tensor is contiguous here
    # (asserted above), so shapes, dtype, scale, mode and table row identify the record; the
    # workspace size is asked once per record (0 unless a sequence-parallel row was asked for: dQ
    # is written directly).
    key = (q.shape, seqlen_k, q.dtype, seqlen_q_rounded, softmax_scale, deterministic, config_id,
           threading.get_ident())
    cached = _BWD_ARGS.get(key)
    if cached is None:
        args = _capi.BwdArgs()
        for name, t in (("q", q), ("k", k), ("v", v), ("o", output), ("d_o", d_output), ("dq", dq),
                        ("dk", dk), ("dv", dv)):
            rec = getattr(args, name)
            rec.stride_batch, rec.stride_head, rec.stride_seq = _strides3(t)
        args.batch, args.nheads, args.seqlen_q, args.seqlen_k = batch, nheads, seqlen_q, seqlen_k
        args.headdim, args.seqlen_q_rounded = headdim, seqlen_q_rounded
        args.softmax_scale, args.dtype = softmax_scale, _COMPUTE_DTYPES[q.dtype]
        args.deterministic, args.config_id = deterministic, config_id
        ws_bytes = _capi.load().fa2_bwd_workspace_bytes(batch, nheads, seqlen_q, seqlen_k, headdim,
                                                        deterministic, config_id)
        cached = (args, ws_bytes)
        _remember(_BWD_ARGS, key, cached)
    args, ws_bytes = cached
    # lse and delta rows are indexed with the record's row length: it must be the one they were allocated with.
    assert lse.shape[2] == delta.shape[2] == args.seqlen_q_rounded
    workspace = torch.empty(ws_bytes, dtype=torch.uint8, device=q.device) if ws_bytes else None
    args.q.ptr, args.k.ptr, args.v.ptr = q.data_ptr(), k.data_ptr(), v.data_ptr()
    args.o.ptr, args.d_o.ptr = output.data_ptr(), d_output.data_ptr()
    args.dq.ptr, args.dk.ptr, args.dv.ptr = dq.data_ptr(), dk.data_ptr(), dv.data_ptr()
    args.lse, args.delta = lse.data_ptr(), delta.data_ptr()
    args.workspace = workspace.data_ptr() if workspace is not None else None

    lib = _capi.load()
    with _device_guard(q.device):
        status = lib.fa2_bwd_packed(args, _stream_handle())
    if status:
        _capi.check(status, "fa2_bwd")
    if negated:
        dq.neg_()


# FA2_GFX950_EXACT_SCALE=1 keeps forward-only calls on the rows of the reference's arithmetic too.
_EXACT_SCALE_ONLY = bool(os.environ.get("FA2_GFX950_EXACT_SCALE"))
_FORWARD_ONLY_ROWS: dict = {}


def _forward_only_row(dtype: torch.dtype, headdim: int, seqlen_q: int, seqlen_k: int) -> int:
    """Table row for a forward whose log-sum-exp no backward will read."""
    if _EXACT_SCALE_ONLY:
        return _capi.FA2_CONFIG_AUTO
    key = (dtype, headdim)
    row = _FORWARD_ONLY_ROWS.get(key)
    if row is None:
        row = _capi.load().fa2_pick_config_forward_only(_COMPUTE_DTYPES[dtype], headdim, seqlen_q, seqlen_k)
        if row < 0:
            _capi.check(-row, "fa2_pick_config_forward_only")
        _FORWARD_ONLY_ROWS[key] = row
    return row


_ATOMIC_ROWS: dict[int, int] = {}


def _atomic_row(headdim: int) -> int:
    """Id of the sequence-parallel (atomic dQ) table row for this head dimension."""
    if not _ATOMIC_ROWS:
        _ATOMIC_ROWS.update({row["headdim_padded"]: row["id"] for row in _capi.config_table() if row["dq_atomic"]})
    if headdim not in _ATOMIC_ROWS:
        raise ValueError(f"ATOMIC_DQ: the sequence-parallel atomic kernels exist for head dimensions "
                         f"{sorted(_ATOMIC_ROWS)}, got {headdim}")
    return _ATOMIC_ROWS[headdim]


def _compute_dtype(dtype: torch.dtype) -> torch.dtype:
    """bf16 stays bf16; everything else is computed in fp16 like the reference."""
    return torch.bfloat16 if dtype == torch.bfloat16 else torch.float16


class FlashAttentionV2Function(torch.autograd.Function):
    """Autograd function for FlashAttention v2 (reference: flash_attention_2.py:280-384)."""

    @staticmethod
    def forward(ctx, q, k, v, softmax_scale, kernels_config):  # noqa: ANN001, ANN205
        """Forward pass; saves (q, k, v, o, lse) in the compute dtype for backward."""
        initial_dtype = q.dtype
        compute_dtype = _compute_dtype(initial_dtype)

        # Contiguous fp16/bf16 inputs are used as they are.
        if not (q.dtype == k.dtype == v.dtype == compute_dtype
                and q.is_contiguous() and k.is_contiguous() and v.is_contiguous()):
            q, k, v = [proj.contiguous().to(compute_dtype) for proj in (q, k, v)]

        output, lse, ctx.softmax_scale = _flash_attention_forward(
            q,
            k,
            v,
            softmax_scale,
            kernels_config.block_rows_size,
            kernels_config.block_cols_size,
            kernels_config.min_block_headdim,
            kernels_config.max_headdim,
            kernels_config.seqlen_cache_divisor,
            kernels_config.min_warps,
            kernels_config.max_warps,
            kernels_config.num_stages,
            # Nothing will be differentiated (no_grad, or no input that requires a gradient): the
            # log-sum-exp saved below is never read.
            forward_only=not any(ctx.needs_input_grad[:3]) and not getattr(kernels_config, "exact_scale", False),
        )

        ctx.save_for_backward(q, k, v, output, lse)
        ctx.kernels_config = kernels_config

        # `output` is contiguous (allocated like the contiguous q).
        return output if initial_dtype == compute_dtype else output.to(initial_dtype)

    @staticmethod
    def backward(ctx, d_output):  # noqa: ANN001, ANN205
        """Gradients for q, k, v; the two non-tensor inputs get None."""
        q, k, v, output, lse = ctx.saved_tensors
        kernels_config = ctx.kernels_config

        # Like the reference (flash_attention_2.py:364) the backward is not differentiable.  It runs
        # under no_grad rather than the reference's inference_mode: gradients that are inference
        # tensors cannot be accumulated in place (a second backward into the same .grad, or q, k and
        # v being one tensor, raises "Inplace update to inference tensor").
        with torch.no_grad():
            dq = torch.empty_like(q)
            dk = torch.empty_like(k)
            dv = torch.empty_like(v)

            _flash_attention_backward(
                q,
                k,
                v,
                output,
                lse,
                dq,
                dk,
                dv,
                d_output.to(q.dtype),
                ctx.softmax_scale,
                kernels_config,
            )

        return dq, dk, dv, None, None


# ============================== AUTOGRAD NODE IN C++ ==============================
_CPP_NODE = None
_CPP_NODE_TRIED = False


def _cpp_node():
    """The extension module with the C++ autograd node, or None when it is not built or switched off."""
    global _CPP_NODE, _CPP_NODE_TRIED
    if not _CPP_NODE_TRIED:
        _CPP_NODE_TRIED = True
        if not os.environ.get("FA2_GFX950_PYTHON_AUTOGRAD"):
            _capi.load()  # the extension links against libfa2_gfx950.so: fail with this loader's message first
            try:
                from . import _fa2_torch
            except ImportError:
                _fa2_torch = None
            if _fa2_torch is not None and _fa2_torch.abi_version() == _capi.ABI_VERSION:
                _CPP_NODE = _fa2_torch
    return _CPP_NODE


def _apply(q, k, v, softmax_scale, kernels_config):  # noqa: ANN001, ANN202
    """Record the attention in the autograd graph: the C++ node when it is built, else the Python class.

    With the C++ node the reference's forward wrapper (flash_attention_2.py:283-384) is spelt out
    here: casts and copies are ordinary differentiable operations in front of the node, the input
    checks are the launcher's, a negative scale is folded into the sign of q.
    """
    node = _cpp_node()
    if node is None or kernels_config.atomic_dq:  # the C++ node always lets the table choose its backward row
        return FlashAttentionV2Function.apply(q, k, v, softmax_scale, kernels_config)
    initial_dtype = q.dtype
    compute_dtype = _compute_dtype(initial_dtype)
    if not (q.dtype == k.dtype == v.dtype == compute_dtype
            and q.is_contiguous() and k.is_contiguous() and v.is_contiguous()):
        q, k, v = [proj.contiguous().to(compute_dtype) for proj in (q, k, v)]
    _assert_forward_inputs(q, k, v, kernels_config.max_headdim)
    scale = softmax_scale or 1.0 / math.sqrt(q.shape[-1])
    if scale < 0:
        q, scale = -q, -scale
    # A forward that nothing will differentiate may take a forward-only row of the table.
    forward_only = (not (torch.is_grad_enabled() and (q.requires_grad or k.requires_grad or v.requires_grad))
                    and not getattr(kernels_config, "exact_scale", False) and not _EXACT_SCALE_ONLY)
    output = node.flash_attention_v2(q, k, v, scale, bool(kernels_config.deterministic), kernels_config.max_headdim,
                                     forward_only)
    return output if initial_dtype == compute_dtype else output.to(initial_dtype)


# ============================ gfx950 DEFAULT CONFIGURATIONS ============================
# Replaces the reference's eight Turing/Ampere x Triton-version constants
# (flash_attention_2.py:387-565).  The numbers restate the table compiled into the library
# (csrc/fa2_capi.hip); `_capi.config_table()` returns that table at run time.
GFX950_BACKWARD_CONFIGS_DETERMINISTIC = [
    BackwardConfig(
        {"BLOCK_Q_ROWS_SIZE": 64, "BLOCK_KV_COLS_SIZE": 128, "SEQUENCE_PARALLEL": False},
        num_warps=4,
        num_stages=2,
        pre_hook=init_to_zero_v2("DQ"),
    ),
]
GFX950_BACKWARD_CONFIGS_NON_DETERMINISTIC = [
    BackwardConfig(
        {"BLOCK_Q_ROWS_SIZE": 64, "BLOCK_KV_COLS_SIZE": 128, "SEQUENCE_PARALLEL": True},
        num_warps=4,
        num_stages=2,
        pre_hook=init_to_zero_v2("DQ"),
    ),
]
GFX950_KERNEL_CONFIG_DETERMINISTIC = KernelsConfigV2(
    block_rows_size=128,
    block_cols_size=64,
    min_block_headdim=32,
    max_headdim=_capi.FA2_MAX_HEADDIM,
    seqlen_cache_divisor=32,
    min_warps=4,
    max_warps=4,
    num_stages=2,
    backward_autotune_configs=GFX950_BACKWARD_CONFIGS_DETERMINISTIC,
)
GFX950_KERNEL_CONFIG_NON_DETERMINISTIC = KernelsConfigV2(
    block_rows_size=128,
    block_cols_size=64,
    min_block_headdim=32,
    max_headdim=_capi.FA2_MAX_HEADDIM,
    seqlen_cache_divisor=32,
    min_warps=4,
    max_warps=4,
    num_stages=2,
    backward_autotune_configs=GFX950_BACKWARD_CONFIGS_NON_DETERMINISTIC,
)

# The non-deterministic mode run the reference's way: one backward kernel per key tile, dQ
# accumulated with fp32 global atomics (KernelsConfigV2.atomic_dq).  Not in the table of defaults,
# because it is slower than the configuration above; pass it to flash_attention_v2_custom.
GFX950_BACKWARD_CONFIGS_SEQUENCE_PARALLEL_ATOMIC = [
    BackwardConfig(
        {"BLOCK_Q_ROWS_SIZE": 64, "BLOCK_KV_COLS_SIZE": 128, "SEQUENCE_PARALLEL": True, "ATOMIC_DQ": True},
        num_warps=4,
        num_stages=2,
        pre_hook=init_to_zero_v2("DQ"),
    ),
]
GFX950_KERNEL_CONFIG_SEQUENCE_PARALLEL_ATOMIC = KernelsConfigV2(
    block_rows_size=128,
    block_cols_size=64,
    min_block_headdim=32,
    max_headdim=_capi.FA2_MAX_HEADDIM,
    seqlen_cache_divisor=32,
    min_warps=4,
    max_warps=4,
    num_stages=2,
    backward_autotune_configs=GFX950_BACKWARD_CONFIGS_SEQUENCE_PARALLEL_ATOMIC,
)

_GPU_ARCHITECTURES = {
    "gfx950": {
        True: GFX950_KERNEL_CONFIG_DETERMINISTIC,
        False: GFX950_KERNEL_CONFIG_NON_DETERMINISTIC,
    },
}


# ========================= INTERNAL HELPERS FOR PUBLIC API =========================
def _current_arch_name() -> str:
    props = torch.cuda.get_device_properties(torch.cuda.current_device())
    return getattr(props, "gcnArchName", "") or ""


def _validate_runtime_compatibility(cc: tuple[int, int], arch_name: str | None = None) -> None:
    """Check that the current device can run the compiled kernels and that they are loadable.

    Plays the role of the reference's _validate_triton_compatibility
    (flash_attention_2.py:593-614): RuntimeError when the software stack does not fit the GPU.
    """
    if arch_name is None:
        arch_name = _current_arch_name()
    if not arch_name.startswith(_GFX950_ARCH_PREFIX):
        raise RuntimeError(
            f"Device architecture {arch_name!r} (compute capability {cc}) detected; "
            "libfa2_gfx950.so contains gfx950 (MI355X) code objects only"
        )
    _capi.load()  # raises RuntimeError when the library is missing or has the wrong ABI


_VALIDATED_DEVICES: dict[int, tuple[int, int]] = {}


def _validated_capability() -> tuple[int, int]:
    """Compute capability of the current device, checked once per device.

    The two device queries behind the check cost about 20 us per call, which is as much as the
    rest of the forward wrapper; a device that passed keeps passing, one that failed is asked again.
    """
    index = torch.cuda.current_device()
    cc = _VALIDATED_DEVICES.get(index)
    if cc is None:
        cc = torch.cuda.get_device_capability(index)
        _validate_runtime_compatibility(cc)
        _VALIDATED_DEVICES[index] = cc
    return cc


def _select_optimal_gpu_architecture(cc: tuple[int, int], deterministic: bool) -> KernelsConfigV2:
    """Pick the configuration for the device (reference: flash_attention_2.py:617-642).

    Raises:
        ValueError: If the compute capability is below what gfx950 reports.
    """
    if cc < _MIN_CC:
        raise ValueError(
            f"Unsupported GPU compute capability {cc}. Minimum required: {_MIN_CC} (gfx950)"
        )
    return _GPU_ARCHITECTURES["gfx950"][bool(deterministic)]


# =================================== PUBLIC API ===================================
def flash_attention_v2(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    softmax_scale: float | None = None,
    deterministic: bool = False,
) -> torch.Tensor:
    """Causal FlashAttention-2 with gfx950 kernels (reference: flash_attention_2.py:646-697).

    Args:
        q: Query tensor of shape (batch, nheads, seqlen_q, headdim).
        k: Key tensor of shape (batch, nheads, seqlen_k, headdim).
        v: Value tensor of shape (batch, nheads, seqlen_k, headdim).
        softmax_scale: Softmax scaling factor (default: 1/sqrt(headdim)).
        deterministic: Use the backward whose results are bit-identical from run to run.

    Returns:
        Attention output tensor, same shape and dtype as q.
    """
    cc = _validated_capability()

    kernels_config = _select_optimal_gpu_architecture(cc, deterministic)

    return _apply(q, k, v, softmax_scale, kernels_config)


_TILE_WARNING_SHOWN = False


def _warn_about_ignored_tile_fields(kernels_config: KernelsConfigV2) -> None:
    """Say once when a custom configuration asks for tile shapes other than the compiled ones.

    The reference hands these values to its kernels (flash_attention_2.py:137-141, 773-790); the
    gfx950 kernels exist in one tile shape per table row, so other values cannot be honoured."""
    global _TILE_WARNING_SHOWN
    if _TILE_WARNING_SHOWN:
        return
    compiled = GFX950_KERNEL_CONFIG_DETERMINISTIC
    asked = (kernels_config.block_rows_size, kernels_config.block_cols_size, kernels_config.min_warps)
    have = (compiled.block_rows_size, compiled.block_cols_size, compiled.min_warps)
    backward = [(c.kwargs.get("BLOCK_Q_ROWS_SIZE"), c.kwargs.get("BLOCK_KV_COLS_SIZE"))
                for c in kernels_config.backward_autotune_configs if hasattr(c, "kwargs")]
    have_bwd = (compiled.backward_autotune_configs[0].kwargs["BLOCK_Q_ROWS_SIZE"],
                compiled.backward_autotune_configs[0].kwargs["BLOCK_KV_COLS_SIZE"])
    if asked != have or any(b != have_bwd and b != (None, None) for b in backward):
        import warnings

        _TILE_WARNING_SHOWN = True
        warnings.warn(
            f"flash_attention_v2_custom: the gfx950 kernels are compiled for {have[0]}-row workgroups over "
            f"{have[1]}-row streamed tiles with {have[2]} wavefronts (backward {have_bwd[0]} x {have_bwd[1]}); the "
            f"configuration asks for {asked} (backward {backward}) and these fields are ignored.  max_headdim, "
            "exact_scale, SEQUENCE_PARALLEL and ATOMIC_DQ are honoured.", stacklevel=3)


def flash_attention_v2_custom(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    softmax_scale: float | None,
    kernels_configs: dict[tuple[int, int], KernelsConfigV2],
) -> torch.Tensor:
    """Causal FlashAttention-2 with a caller-supplied configuration per compute capability.

    Same contract as the reference (flash_attention_2.py:700-790): the dictionary is keyed by
    ``torch.cuda.get_device_capability()`` of the current device ((9, 5) on MI355X); a missing
    key raises ValueError.  Of the configuration, ``max_headdim``, ``exact_scale`` and the
    ``SEQUENCE_PARALLEL`` and ``ATOMIC_DQ`` flags of the backward configurations are honoured (the
    latter selects the atomic-add backward, ``GFX950_KERNEL_CONFIG_SEQUENCE_PARALLEL_ATOMIC``); the Triton tile, warp
    and stage counts are accepted and ignored (the reference hands them to its kernels, flash_attention_2.py:137-141;
    here the tile shapes are compiled in, one table row per padded head dimension).

    Example:
        configs = {(9, 5): KernelsConfigV2(
            block_rows_size=128, block_cols_size=64, min_block_headdim=32, max_headdim=128,
            seqlen_cache_divisor=32, min_warps=4, max_warps=4, num_stages=2,
            backward_autotune_configs=[BackwardConfig(
                {"BLOCK_Q_ROWS_SIZE": 64, "BLOCK_KV_COLS_SIZE": 128, "SEQUENCE_PARALLEL": False},
                num_warps=4, num_stages=2, pre_hook=init_to_zero_v2("DQ"))])}
        out = flash_attention_v2_custom(q, k, v, softmax_scale=None, kernels_configs=configs)
    """
    cc = torch.cuda.get_device_capability()

    if cc not in kernels_configs:
        raise ValueError(
            f"Missing kernel configuration for compute capability {cc}. "
            "KernelsConfig must be provided for the current GPU architecture"
        )
    _validate_runtime_compatibility(cc)

    kernels_config = kernels_configs[cc]
    _warn_about_ignored_tile_fields(kernels_config)
    if kernels_config.max_headdim > _capi.FA2_MAX_HEADDIM:
        raise ValueError(
            f"max_headdim={kernels_config.max_headdim} exceeds what the compiled kernels "
            f"support ({_capi.FA2_MAX_HEADDIM})"
        )

    return _apply(q, k, v, softmax_scale, kernels_config)
