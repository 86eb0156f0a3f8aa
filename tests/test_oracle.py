"""Pins the CPU oracle itself: brute force, library cross-check, closed forms, finite differences.

The reference holds no golden vectors for this path (its tests compare against naive attention
computed on the fly, tests/test_flash_attention_2.py:288-294), so the oracle is fixed by
independent evidence chosen so that a dropped term, a wrong sign or a transposed operand fails.
"""

from __future__ import annotations

import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import c_oracle
from oracle import naive_attention as oracle


def _rand(shape, seed, dtype=torch.float64):
    return torch.randn(shape, generator=torch.Generator().manual_seed(seed), dtype=dtype)


@pytest.mark.parametrize("nq,nk,d", [(7, 7, 4), (5, 9, 3), (9, 5, 6), (1, 1, 2), (16, 16, 8)])
def test_forward_matches_brute_force(nq, nk, d):
    q, k, v = _rand((nq, d), 1), _rand((nk, d), 2), _rand((nk, d), 3)
    scale = 0.37
    want_o, want_lse = oracle.brute_force_attention(q, k, v, scale)
    got_o = oracle.naive_causal_attention(q, k, v, scale, torch.float64)
    got_lse = oracle.naive_lse(q, k, scale, torch.float64)
    torch.testing.assert_close(got_o, want_o, atol=1e-12, rtol=1e-12)
    torch.testing.assert_close(got_lse, want_lse, atol=1e-12, rtol=1e-12)
    c_o, c_lse = c_oracle.forward(q.numpy(), k.numpy(), v.numpy(), scale)
    np.testing.assert_allclose(c_o, want_o.numpy(), atol=1e-12, rtol=1e-12)
    np.testing.assert_allclose(c_lse, want_lse.numpy(), atol=1e-12, rtol=1e-12)


def test_forward_matches_torch_sdpa():
    """Second oracle of the reference: tests/test_flash_attention_2.py:313."""
    q, k, v = (_rand((2, 3, 33, 16), s, torch.float32) for s in (4, 5, 6))
    scale = 0.21
    want = F.scaled_dot_product_attention(q, k, v, is_causal=True, scale=scale)
    got = oracle.naive_causal_attention(q, k, v, scale)
    torch.testing.assert_close(got, want, atol=2e-6, rtol=1e-5)


def test_default_scale_is_inverse_sqrt_headdim():
    q, k, v = (_rand((1, 1, 9, 16), s) for s in (7, 8, 9))
    a = oracle.naive_causal_attention(q, k, v, None, torch.float64)
    b = oracle.naive_causal_attention(q, k, v, 0.25, torch.float64)
    torch.testing.assert_close(a, b, atol=0, rtol=0)
    assert oracle.default_scale(64) == 1.0 / math.sqrt(64)


def test_closed_form_special_cases():
    n, d = 12, 5
    q, k, v = _rand((n, d), 10), _rand((n, d), 11), _rand((n, d), 12)
    # Row 0 sees only key 0.
    o = oracle.naive_causal_attention(q, k, v, 0.5, torch.float64)
    torch.testing.assert_close(o[0], v[0], atol=1e-14, rtol=0)
    # V == 1 gives O == 1 (rows of P sum to one).
    o1 = oracle.naive_causal_attention(q, k, torch.ones_like(v), 0.5, torch.float64)
    torch.testing.assert_close(o1, torch.ones_like(o1), atol=1e-14, rtol=0)
    # Q == 0 gives uniform probabilities: running means of V.
    o0 = oracle.naive_causal_attention(torch.zeros_like(q), k, v, 0.5, torch.float64)
    means = torch.cumsum(v, 0) / torch.arange(1, n + 1, dtype=torch.float64)[:, None]
    torch.testing.assert_close(o0, means, atol=1e-14, rtol=0)
    # exp(S - lse) sums to one on every row.
    lse = oracle.naive_lse(q, k, 0.5, torch.float64)
    p = torch.exp(oracle.masked_scores(q, k, 0.5) - lse[:, None])
    torch.testing.assert_close(p.sum(-1), torch.ones(n, dtype=torch.float64), atol=1e-14, rtol=0)
    # Q == 0: lse of row i is log(i + 1).
    lse0 = oracle.naive_lse(torch.zeros_like(q), k, 0.5, torch.float64)
    torch.testing.assert_close(lse0, torch.log(torch.arange(1, n + 1, dtype=torch.float64)), atol=1e-14, rtol=0)


def test_mask_is_top_left_anchored_when_lengths_differ():
    """Reference: _triton_kernels_v2.py:139-147 keeps row >= col with no offset."""
    q, k, v = _rand((3, 4), 13), _rand((6, 4), 14), _rand((6, 4), 15)
    o = oracle.naive_causal_attention(q, k, v, 1.0, torch.float64)
    torch.testing.assert_close(o[0], v[0], atol=1e-14, rtol=0)  # not the bottom-right convention
    q2 = _rand((6, 4), 16)
    k2, v2 = k[:3], v[:3]
    o2 = oracle.naive_causal_attention(q2, k2, v2, 1.0, torch.float64)
    # rows 3.. see all three keys: plain softmax attention
    full = torch.softmax(q2[3:] @ k2.T, -1) @ v2
    torch.testing.assert_close(o2[3:], full, atol=1e-14, rtol=0)


def test_delta_is_rowwise_dot():
    o, g = _rand((2, 2, 7, 5), 17), _rand((2, 2, 7, 5), 18)
    want = torch.einsum("bhnd,bhnd->bhn", o, g)
    torch.testing.assert_close(oracle.naive_delta(o, g, torch.float64), want, atol=1e-14, rtol=0)


@pytest.mark.parametrize("nq,nk,d", [(8, 8, 4), (6, 10, 3), (10, 6, 5)])
def test_backward_three_ways_agree(nq, nk, d):
    q, k, v, g = _rand((nq, d), 20), _rand((nk, d), 21), _rand((nk, d), 22), _rand((nq, d), 23)
    scale = 0.4
    o_a, dq_a, dk_a, dv_a = oracle.naive_backward(q, k, v, g, scale, torch.float64)
    o_c, dq_c, dk_c, dv_c = oracle.closed_form_backward(q, k, v, g, scale, torch.float64)
    for a, c in ((o_a, o_c), (dq_a, dq_c), (dk_a, dk_c), (dv_a, dv_c)):
        torch.testing.assert_close(a, c, atol=1e-12, rtol=1e-12)
    dq_n, dk_n, dv_n, delta_n = c_oracle.backward(q.numpy(), k.numpy(), v.numpy(), g.numpy(), scale)
    np.testing.assert_allclose(dq_n, dq_a.numpy(), atol=1e-12, rtol=1e-12)
    np.testing.assert_allclose(dk_n, dk_a.numpy(), atol=1e-12, rtol=1e-12)
    np.testing.assert_allclose(dv_n, dv_a.numpy(), atol=1e-12, rtol=1e-12)
    np.testing.assert_allclose(delta_n, (o_a * g).sum(-1).numpy(), atol=1e-12, rtol=1e-12)


def test_backward_matches_central_finite_differences():
    """d/dx sum(O * dO) by central differences through the plain-C forward."""
    nq, nk, d, scale, eps = 5, 6, 3, 0.6, 1e-6
    q, k, v, g = (_rand(s, i).numpy() for s, i in (((nq, d), 30), ((nk, d), 31), ((nk, d), 32), ((nq, d), 33)))
    dq, dk, dv, _ = c_oracle.backward(q, k, v, g, scale)

    def loss(q_, k_, v_):
        o, _ = c_oracle.forward(q_, k_, v_, scale)
        return float((o * g).sum())

    for grad, which in ((dq, 0), (dk, 1), (dv, 2)):
        num = np.zeros_like(grad)
        args = [q, k, v]
        for idx in np.ndindex(*grad.shape):
            plus = [a.copy() for a in args]
            minus = [a.copy() for a in args]
            plus[which][idx] += eps
            minus[which][idx] -= eps
            num[idx] = (loss(*plus) - loss(*minus)) / (2 * eps)
        np.testing.assert_allclose(grad, num, atol=1e-7, rtol=1e-6)


def test_backward_invariants():
    """sum(q*dq) == sum(k*dk) per head (QK^T is invariant under q -> a q, k -> k / a), and a
    constant shift of V along the sequence leaves dQ and dK unchanged (rows of dS sum to zero)."""
    q, k, v, g = (_rand((2, 3, 11, 4), s) for s in (40, 41, 42, 43))
    _, dq, dk, dv = oracle.closed_form_backward(q, k, v, g, 0.3)
    torch.testing.assert_close((q * dq).sum((-1, -2)), (k * dk).sum((-1, -2)), atol=1e-12, rtol=1e-12)
    _, dq2, dk2, _ = oracle.closed_form_backward(q, k, v + 3.0, g, 0.3)
    torch.testing.assert_close(dq2, dq, atol=1e-11, rtol=1e-11)
    torch.testing.assert_close(dk2, dk, atol=1e-11, rtol=1e-11)
    # dV of row j sums dO over the rows that attend to j, weighted by P: total mass is conserved.
    torch.testing.assert_close(dv.sum(-2), g.sum(-2), atol=1e-12, rtol=1e-12)


def test_sliced_evaluation_equals_whole_tensor():
    q, k, v, g = (_rand((2, 2, 9, 4), s, torch.float32) for s in (50, 51, 52, 53))
    whole = oracle.naive_backward(q, k, v, g, None, torch.float32)
    sliced = oracle.sliced_forward_backward(q, k, v, g, None, torch.float32)
    for a, b in zip(whole, sliced):
        torch.testing.assert_close(a, b, atol=1e-6, rtol=1e-6)
    part = oracle.sliced_forward_backward(q, k, v, g, None, torch.float32, heads=3)
    torch.testing.assert_close(part[0], whole[0].reshape(4, 9, 4)[:3], atol=1e-6, rtol=1e-6)
