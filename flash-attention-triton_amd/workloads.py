"""Benchmark/parity workloads: the five causal-attention configurations and their seeded inputs.

Inputs are drawn on the CPU from ``torch.Generator().manual_seed(seed)`` in the order q, k, v, dO
(the order of the reference's test helpers, tests/test_flash_attention_2.py:60-62, 109), scaled by
the configuration's standard deviations, cast to its dtype and only then moved to the device, so
that the oracle and the kernels see bit-identical values on any machine.
"""

from __future__ import annotations

import math
from dataclasses import dataclass

import torch


@dataclass(frozen=True)
class Workload:
    name: str
    batch: int
    nheads: int
    seqlen: int
    headdim: int
    dtype: torch.dtype
    qk_std: float = 1.0
    explicit_scale: bool = False  # pass 1/sqrt(D) explicitly instead of None
    both_modes: bool = False      # exercised with deterministic=True and False
    description: str = ""

    @property
    def shape(self) -> tuple[int, int, int, int]:
        return (self.batch, self.nheads, self.seqlen, self.headdim)

    @property
    def softmax_scale(self) -> float | None:
        return 1.0 / math.sqrt(self.headdim) if self.explicit_scale else None

    @property
    def fwd_flops(self) -> float:
        """FlashAttention-2 paper convention: two GEMMs, 2 FLOP per MAC, causal halves the work."""
        return 4.0 * self.batch * self.nheads * self.seqlen**2 * self.headdim / 2.0

    @property
    def bwd_flops(self) -> float:
        return 2.5 * self.fwd_flops

    @property
    def fwd_bytes(self) -> float:
        """Algorithmic HBM bytes of the forward: read q, k, v, write o (2 B each) + lse (4 B)."""
        rows = self.batch * self.nheads * self.seqlen
        return 4.0 * rows * self.headdim * 2 + rows * 4


WORKLOADS = {
    "C1": Workload("C1", 2, 4, 512, 64, torch.float16, explicit_scale=True,
                   description="small fp16 case the reference's CPU oracle runs in seconds"),
    "C2": Workload("C2", 4, 16, 2048, 64, torch.bfloat16, both_modes=True,
                   description="bf16 D=64, deterministic and non-deterministic backward"),
    "C3": Workload("C3", 2, 32, 4096, 128, torch.bfloat16,
                   description="headline: 7B-style head layout, bf16 D=128"),
    "C4": Workload("C4", 1, 16, 16384, 128, torch.bfloat16, both_modes=True,
                   description="long sequence: stresses dQ accumulation and lse numerics"),
    "C5": Workload("C5", 8, 12, 3000, 64, torch.float16, qk_std=3.0,
                   description="ragged tail (N not a tile multiple), peaky softmax (q, k ~ N(0, 3^2))"),
}


def make_inputs(w: Workload, device="cpu", seed: int = 42, heads: int | None = None):
    """Seeded (q, k, v, dO) for workload ``w`` on ``device``.

    ``heads`` keeps only the first ``heads`` (batch, head) slices, returned as
    (heads, 1, seqlen, headdim); the values equal the corresponding slices of the full tensors.
    """
    gen = torch.Generator().manual_seed(seed)
    out = []
    for std in (w.qk_std, w.qk_std, 1.0, 1.0):
        t = torch.randn(w.shape, generator=gen, dtype=torch.float32)
        if std != 1.0:
            t = t * std
        t = t.to(w.dtype)
        if heads is not None:
            t = t.reshape(w.batch * w.nheads, 1, w.seqlen, w.headdim)[:heads].contiguous()
        out.append(t.to(device))
    return tuple(out)
