"""Configuration container of the gfx950 FlashAttention-2 kernels.

Mirrors ``KernelsConfigV2`` and ``init_to_zero_v2`` of the reference
(src/flash_attention_triton/_configurators_v2.py:9-93) so that code written against
``flash_attention_v2_custom`` keeps working, without importing Triton.  The fields keep their
names.  The tile shapes of the gfx950 kernels are compiled into ``libfa2_gfx950.so`` (one table row
per padded head dimension, chosen by the library from the problem), so of the fields below only
``max_headdim`` (largest accepted head dimension, padding of the log-sum-exp rows), the
``SEQUENCE_PARALLEL`` flag of the backward configurations (which backward mode is requested) and,
next to it, ``ATOMIC_DQ`` (run the reference's atomic-add formulation of that mode, see
``KernelsConfigV2.atomic_dq``) have an effect, plus one field the reference does not have,
``exact_scale``; the Triton tile, warp and stage counts are accepted and ignored.  The reference's
kernel-cache key helpers (_configurators_v2.py:40-78) have no counterpart: there is no run-time
compilation and therefore no kernel cache to key.
"""

from __future__ import annotations

from collections.abc import Callable
from dataclasses import dataclass, field
from typing import Any

import torch


@dataclass(frozen=True)
class BackwardConfig:
    """Stand-in for ``triton.Config`` in ``backward_autotune_configs``.

    Any object with the same attributes (``kwargs``, ``num_warps``, ``num_stages``,
    ``pre_hook``) is accepted, a real ``triton.Config`` included.  ``kwargs["SEQUENCE_PARALLEL"]``
    selects the non-deterministic backward (reference: flash_attention_2.py:204-207,
    _triton_kernels_v2.py:466-525); ``kwargs["ATOMIC_DQ"]`` beside it selects how that mode is run.
    """

    kwargs: dict[str, Any]
    num_warps: int = 4
    num_stages: int = 2
    pre_hook: Callable[..., Any] | None = None

    def __hash__(self) -> int:  # dict field: hash by content
        return hash((tuple(sorted(self.kwargs.items())), self.num_warps, self.num_stages))


@dataclass(frozen=True)
class KernelsConfigV2:
    """Configuration container for the FlashAttention-2 kernels (reference: _configurators_v2.py:9-38).

    Attributes:
        block_rows_size: Query rows per workgroup in the forward kernel (the compiled kernels
            use 128; other values are accepted and ignored).
        block_cols_size: Key rows per inner step of the forward kernel (compiled: 64).
        min_block_headdim: Smallest padded head dimension (power of two, at least 16).
        max_headdim: Largest supported head dimension.  Also the multiple to which the
            log-sum-exp row length is padded (reference: flash_attention_2.py:98).
        seqlen_cache_divisor: Kept for signature compatibility; the reference uses it to bound
            Triton recompilation, which does not exist here.
        min_warps: Wavefronts (64 lanes) per workgroup.
        max_warps: Kept for signature compatibility (dead in the reference as well).
        num_stages: LDS stages of the streamed tiles (compiled: 2).
        backward_autotune_configs: Backward configurations; the backward is deterministic
            unless one of them sets ``SEQUENCE_PARALLEL`` to True.
        exact_scale: Not in the reference.  A forward that nothing will differentiate may, for bf16
            inputs, run a kernel that multiplies Q by ``softmax_scale * log2(e)`` and rounds it to
            bf16 once (table rows with ``fwd_exp_folded``); True keeps such calls on the rows that
            apply the scale to the fp32 scores, as the reference does
            (_triton_kernels_v2.py:137-152), at about 4 % more forward time.  Forwards that a
            backward may follow, and fp16 inputs, always take those rows.
    """

    block_rows_size: int
    block_cols_size: int
    min_block_headdim: int
    max_headdim: int
    seqlen_cache_divisor: int
    min_warps: int
    max_warps: int
    num_stages: int
    backward_autotune_configs: list = field(default_factory=list)
    exact_scale: bool = False

    @property
    def deterministic(self) -> bool:
        """True unless a backward configuration asks for sequence-parallel dQ accumulation."""
        return not any(bool(getattr(c, "kwargs", {}).get("SEQUENCE_PARALLEL", False))
                       for c in self.backward_autotune_configs)

    @property
    def atomic_dq(self) -> bool:
        """True when a sequence-parallel backward configuration also sets ``ATOMIC_DQ``.

        The non-deterministic mode then runs as the reference formulates it
        (_triton_kernels_v2.py:336-339): one kernel per key tile that adds its dQ contributions into
        an fp32 accumulator with global atomics.  Without the flag (the default table) the mode runs
        the same two atomic-free kernels as the deterministic one, which on MI355X is two to three
        times faster; the flag is there for callers who want the reference's accumulation order
        semantics or want to measure it.  Head dimensions 32, 64 and 128 only.
        """
        return any(bool(getattr(c, "kwargs", {}).get("SEQUENCE_PARALLEL", False))
                   and bool(getattr(c, "kwargs", {}).get("ATOMIC_DQ", False))
                   for c in self.backward_autotune_configs)


def init_to_zero_v2(name: str) -> Callable[[dict[str, torch.Tensor]], torch.Tensor]:
    """Pre-hook that zeroes the tensor called ``name`` in a kernel-argument dictionary.

    Same contract as the reference (_configurators_v2.py:81-93).  The gfx950 library clears its
    own dQ workspace when a mode needs one, so the hook is never called by this package; it is
    kept so that configurations written for the reference still construct.
    """
    return lambda nargs: nargs[name].zero_()
