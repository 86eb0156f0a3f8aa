"""``torch.library`` registration of the gfx950 kernels.

The reference wraps its kernels in a ``torch.autograd.Function`` whose backward runs under
``inference_mode`` (src/flash_attention_triton/flash_attention_2.py:283-384), which
``torch.compile`` cannot trace through.  This module registers the same two launches as
dispatcher operators with fake (meta) kernels and an autograd formula, so that a graph captured
by ``torch.compile`` or ``make_fx`` keeps them as opaque calls:

    fa2_gfx950::fwd(q, k, v, softmax_scale, deterministic)      -> (out, lse)
    fa2_gfx950::bwd(q, k, v, out, lse, d_out, softmax_scale, deterministic) -> (dq, dk, dv)

Both take contiguous fp16/bf16 ``(batch, nheads, seqlen, headdim)`` tensors on the GPU and call
the same launchers (and through them the same C ABI) as ``flash_attention_v2``;
``flash_attention_v2_op`` adds the dtype and scale handling of the public function around them.
"""

from __future__ import annotations

import math

import torch

from . import _capi
from . import flash_attention_2 as _fa2

_NAMESPACE = "fa2_gfx950"


def _config(deterministic: bool):
    return (_fa2.GFX950_KERNEL_CONFIG_DETERMINISTIC if deterministic
            else _fa2.GFX950_KERNEL_CONFIG_NON_DETERMINISTIC)


def _rounded(seqlen_q: int) -> int:
    """Padded row length of lse (reference rule: flash_attention_2.py:98)."""
    m = _capi.FA2_MAX_HEADDIM
    return math.ceil(seqlen_q / m) * m


@torch.library.custom_op(f"{_NAMESPACE}::fwd", mutates_args=(), device_types="cuda")
def fwd(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, softmax_scale: float,
        deterministic: bool) -> tuple[torch.Tensor, torch.Tensor]:
    # `deterministic` only selects the backward that autograd will launch for this call.
    cfg = _config(deterministic)
    out, lse, _ = _fa2._flash_attention_forward(
        q, k, v, softmax_scale, cfg.block_rows_size, cfg.block_cols_size, cfg.min_block_headdim,
        cfg.max_headdim, cfg.seqlen_cache_divisor, cfg.min_warps, cfg.max_warps, cfg.num_stages)
    return out, lse


@fwd.register_fake
def _(q, k, v, softmax_scale, deterministic):
    batch, nheads, seqlen_q, _ = q.shape
    out = torch.empty_like(q, memory_format=torch.contiguous_format)
    lse = q.new_empty((batch, nheads, _rounded(seqlen_q)), dtype=torch.float32)
    return out, lse


@torch.library.custom_op(f"{_NAMESPACE}::bwd", mutates_args=(), device_types="cuda")
def bwd(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, out: torch.Tensor, lse: torch.Tensor,
        d_out: torch.Tensor, softmax_scale: float,
        deterministic: bool) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    _fa2._flash_attention_backward(q, k, v, out, lse, dq, dk, dv, d_out.contiguous(), softmax_scale,
                                   _config(deterministic))
    return dq, dk, dv


@bwd.register_fake
def _(q, k, v, out, lse, d_out, softmax_scale, deterministic):
    fmt = torch.contiguous_format
    return (torch.empty_like(q, memory_format=fmt), torch.empty_like(k, memory_format=fmt),
            torch.empty_like(v, memory_format=fmt))


def _setup_context(ctx, inputs, output):
    q, k, v, softmax_scale, deterministic = inputs
    out, lse = output
    ctx.save_for_backward(q, k, v, out, lse)
    ctx.softmax_scale = softmax_scale
    ctx.deterministic = deterministic


def _backward(ctx, d_out, d_lse):
    q, k, v, out, lse = ctx.saved_tensors
    # The gradient of lse is not propagated (the reference returns the output only).
    dq, dk, dv = bwd(q, k, v, out, lse, d_out, ctx.softmax_scale, ctx.deterministic)
    return dq, dk, dv, None, None


fwd.register_autograd(_backward, setup_context=_setup_context)


def flash_attention_v2_op(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor,
                          softmax_scale: float | None = None,
                          deterministic: bool = False) -> torch.Tensor:
    """``flash_attention_v2`` routed through the registered operators (traceable).

    Same arguments, defaults and result as ``flash_attention_v2``
    (reference: flash_attention_2.py:646-697): inputs in any float dtype, output in the input
    dtype, ``softmax_scale`` of None or 0.0 meaning 1/sqrt(headdim).
    """
    initial_dtype = q.dtype
    compute_dtype = _fa2._compute_dtype(initial_dtype)
    q, k, v = [t.contiguous().to(compute_dtype) for t in (q, k, v)]
    scale = softmax_scale or 1.0 / math.sqrt(q.shape[-1])
    out, _ = fwd(q, k, v, scale, bool(deterministic))
    return out.to(initial_dtype)
