"""Naive causal attention on the CPU: the parity oracle (test infrastructure only).

This module restates, in plain PyTorch, the "vanilla attention" that the
reference's own test-suite uses as ground truth
(reference: tests/test_flash_attention_2.py:288-294):

    mask = triu(ones(N, N, bool), diagonal=1)
    O    = softmax((Q @ K^T) * scale  masked_fill(mask, -inf), dim=-1) @ V

The mask keeps ``row >= col`` anchored at the top-left corner, also when
``Nq != Nk`` (reference: src/flash_attention_triton/_triton_kernels_v2.py:139-147).

Everything here runs in fp32 or fp64 on the host.  It must never be imported by
the product package; only tests, ``__graft_entry__.smoke`` and the CPU baseline
leg of ``bench.py`` use it, and only as the checker.

Pinning status of each function (what independent evidence fixes it):

* ``naive_causal_attention``  pinned: brute-force scalar loops on tiny inputs,
  torch's own ``scaled_dot_product_attention(is_causal=True)`` (the second oracle of
  the reference, tests/test_flash_attention_2.py:313), the plain-C restatement in
  ``naive_attention.c``, and closed-form special cases (row 0 equals v[0]; V == 1
  gives O == 1; Q == 0 gives running means of V).
* ``naive_lse``               pinned: ``log(sum(exp(.)))`` by brute force; exp(S - lse)
  rows sum to one.
* ``naive_delta``             pinned: textbook row-wise dot product by brute force.
* ``naive_backward`` / ``closed_form_backward``  pinned: against each other (autograd
  versus hand-derived formulas), against fp64 central finite differences on tiny
  shapes, and by the invariants sum(q*dq) == sum(k*dk) per head and rows of dS
  summing to zero.
"""

from __future__ import annotations

import math

import torch


def default_scale(headdim: int) -> float:
    """Default softmax scale, 1/sqrt(D) (reference: flash_attention_2.py:94)."""
    return 1.0 / math.sqrt(headdim)


def causal_mask(seqlen_q: int, seqlen_k: int, device="cpu") -> torch.Tensor:
    """True where the score must be dropped: col > row (tests/test_flash_attention_2.py:288-290)."""
    return torch.triu(torch.ones((seqlen_q, seqlen_k), dtype=torch.bool, device=device), diagonal=1)


def masked_scores(q: torch.Tensor, k: torch.Tensor, scale: float) -> torch.Tensor:
    """scale * Q K^T with -inf above the diagonal (tests/test_flash_attention_2.py:291-292)."""
    qk = (q @ k.transpose(-2, -1)) * scale
    return qk.masked_fill(causal_mask(q.shape[-2], k.shape[-2], q.device), float("-inf"))


def naive_causal_attention(q, k, v, scale=None, dtype=torch.float32):
    """O = softmax(mask(scale * Q K^T)) V in ``dtype`` (tests/test_flash_attention_2.py:288-294)."""
    scale = scale or default_scale(q.shape[-1])
    q, k, v = (t.to(dtype) for t in (q, k, v))
    return torch.softmax(masked_scores(q, k, scale), dim=-1) @ v


def naive_lse(q, k, scale=None, dtype=torch.float32):
    """Row log-sum-exp of the masked, scaled scores (what _triton_kernels_v2.py:150-165 carries)."""
    scale = scale or default_scale(q.shape[-1])
    return torch.logsumexp(masked_scores(q.to(dtype), k.to(dtype), scale), dim=-1)


def naive_delta(o, d_o, dtype=torch.float32):
    """delta = rowsum(dO * O) (reference: _triton_kernels_v2.py:572-608)."""
    return (o.to(dtype) * d_o.to(dtype)).sum(-1)


def naive_backward(q, k, v, d_o, scale=None, dtype=torch.float32):
    """(O, dQ, dK, dV) of the naive attention through torch autograd, in ``dtype``."""
    scale = scale or default_scale(q.shape[-1])
    q, k, v = (t.detach().to(dtype).clone().requires_grad_(True) for t in (q, k, v))
    o = torch.softmax(masked_scores(q, k, scale), dim=-1) @ v
    dq, dk, dv = torch.autograd.grad(o, (q, k, v), d_o.to(dtype))
    return o.detach(), dq, dk, dv


def closed_form_backward(q, k, v, d_o, scale=None, dtype=torch.float64):
    """(O, dQ, dK, dV) from the hand-derived formulas, without autograd.

    P = softmax(S);  dV = P^T dO;  dP = dO V^T;  delta = rowsum(P * dP) = rowsum(dO * O);
    dS = P * (dP - delta);  dQ = scale * dS K;  dK = scale * dS^T Q
    (the tile maths of reference _triton_kernels_v2.py:299-348, untiled).
    """
    scale = scale or default_scale(q.shape[-1])
    q, k, v, d_o = (t.to(dtype) for t in (q, k, v, d_o))
    p = torch.softmax(masked_scores(q, k, scale), dim=-1)
    o = p @ v
    dv = p.transpose(-2, -1) @ d_o
    dp = d_o @ v.transpose(-2, -1)
    delta = (o * d_o).sum(-1, keepdim=True)
    ds = p * (dp - delta)
    dq = scale * (ds @ k)
    dk = scale * (ds.transpose(-2, -1) @ q)
    return o, dq, dk, dv


def sliced_forward_backward(q, k, v, d_o, scale=None, dtype=torch.float32, heads=None, backward=True):
    """Naive attention evaluated one (batch, head) slice at a time.

    Heads are independent, so the result equals the whole-tensor evaluation while the
    N x N score matrix stays at one slice.  ``heads`` limits the work to the first
    ``heads`` slices (used by the bounded CPU baseline); the returned tensors then
    cover only those slices, flattened over (batch, head).
    """
    b, h, nq, d = q.shape
    nk = k.shape[2]
    qf, kf, vf, gf = (t.reshape(b * h, -1, d) for t in (q, k, v, d_o))
    n = b * h if heads is None else min(heads, b * h)
    outs = []
    for i in range(n):
        if backward:
            outs.append(naive_backward(qf[i], kf[i], vf[i], gf[i], scale, dtype))
        else:
            outs.append((naive_causal_attention(qf[i], kf[i], vf[i], scale, dtype),))
    stacked = tuple(torch.stack(parts) for parts in zip(*outs))
    if heads is None:
        shapes = [(b, h, nq, d), (b, h, nq, d), (b, h, nk, d), (b, h, nk, d)]
        stacked = tuple(t.reshape(s) for t, s in zip(stacked, shapes))
    return stacked


def brute_force_attention(q, k, v, scale):
    """Scalar-loop causal attention for one head, fp64 python floats.  Tiny inputs only."""
    nq, d = q.shape
    nk = k.shape[0]
    out = [[0.0] * d for _ in range(nq)]
    lse = [0.0] * nq
    for i in range(nq):
        last = min(i, nk - 1)
        s = [scale * sum(float(q[i, c]) * float(k[j, c]) for c in range(d)) for j in range(last + 1)]
        m = max(s)
        w = [math.exp(x - m) for x in s]
        z = sum(w)
        lse[i] = m + math.log(z)
        for c in range(d):
            out[i][c] = sum(w[j] * float(v[j, c]) for j in range(last + 1)) / z
    return torch.tensor(out, dtype=torch.float64), torch.tensor(lse, dtype=torch.float64)
