"""GPU test of fa2_bwd_fused_noalloc, the backward entry point that takes no scratch from its caller.

It is called through the C ABI and compared bit for bit with fa2_bwd_fused (which gets its delta
scratch from the caller) on two calls in a row, the second with a smaller input, so that rows the
first call left in the library's scratch array lie beyond what the second call writes.  A third case
goes through the generic kernels (head dimension 50: the preprocess kernel writes delta), and the size limit is checked.
"""

from __future__ import annotations

import math

import pytest
import torch

pytestmark = pytest.mark.gpu


def _strides3(t):
    return [t.stride(0), t.stride(1), t.stride(2)]


def _inputs(b, h, nq, nk, d, dtype, seed):
    gen = torch.Generator().manual_seed(seed)
    q = torch.randn((b, h, nq, d), generator=gen).to(dtype).cuda()
    k = torch.randn((b, h, nk, d), generator=gen).to(dtype).cuda()
    v = torch.randn((b, h, nk, d), generator=gen).to(dtype).cuda()
    d_o = torch.randn((b, h, nq, d), generator=gen).to(dtype).cuda()
    return q, k, v, d_o


def _both_backwards(capi, b, h, nq, nk, d, dtype, seed):
    """(dq, dk, dv) from fa2_bwd_fused and from fa2_bwd_fused_noalloc on the same forward result."""
    lib = capi.load()
    q, k, v, d_o = _inputs(b, h, nq, nk, d, dtype, seed)
    code = capi.FA2_DTYPE_BF16 if dtype == torch.bfloat16 else capi.FA2_DTYPE_F16
    scale = 1.0 / math.sqrt(d)
    n_r = math.ceil(nq / 128) * 128
    st = torch.cuda.current_stream().cuda_stream
    o = torch.empty_like(q)
    lse = torch.empty((b, h, n_r), dtype=torch.float32, device="cuda")
    capi.check(lib.fa2_fwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), lse.data_ptr(), b, h, nq, nk, d,
                           n_r, *_strides3(q), *_strides3(k), *_strides3(v), *_strides3(o), scale, code,
                           capi.FA2_CONFIG_AUTO, st), "fa2_fwd")
    strides = [*_strides3(q), *_strides3(k), *_strides3(v), *_strides3(o), *_strides3(d_o)]

    def grads():
        # Filled with NaN so that an element the kernels fail to write cannot compare equal.
        return [torch.full_like(t, float("nan")) for t in (q, k, v)]

    want = grads()
    delta = torch.empty_like(lse)
    capi.check(lib.fa2_bwd_fused(q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), d_o.data_ptr(),
                                 lse.data_ptr(), delta.data_ptr(), None, *(t.data_ptr() for t in want),
                                 b, h, nq, nk, d, n_r, *strides, *(s for t in want for s in _strides3(t)),
                                 scale, code, 0, capi.FA2_CONFIG_AUTO, st), "fa2_bwd_fused")
    got = grads()
    capi.check(lib.fa2_bwd_fused_noalloc(q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), d_o.data_ptr(),
                                         lse.data_ptr(), *(t.data_ptr() for t in got),
                                         b, h, nq, nk, d, n_r, *strides, *(s for t in got for s in _strides3(t)),
                                         scale, code, 0, capi.FA2_CONFIG_AUTO, st), "fa2_bwd_fused_noalloc")
    torch.cuda.synchronize()
    return want, got


def _assert_same(want, got, what):
    for name, a, b in zip(("dq", "dk", "dv"), want, got):
        assert not torch.isnan(b).any(), f"{what}: {name} has unwritten or NaN elements"
        assert torch.equal(a, b), f"{what}: {name} differs from fa2_bwd_fused"


def test_noalloc_matches_fused_on_two_calls_in_a_row(capi):
    # First call: 2*3*640 rows of delta scratch; second call: fewer heads, a shorter and ragged
    # sequence, another head dimension - its rows overlap the start of what the first call left.
    want, got = _both_backwards(capi, 2, 3, 640, 640, 128, torch.bfloat16, seed=1)
    _assert_same(want, got, "first call (B=2 H=3 N=640 D=128 bf16)")
    want, got = _both_backwards(capi, 1, 2, 300, 300, 64, torch.float16, seed=2)
    _assert_same(want, got, "second, smaller call (B=1 H=2 N=300 D=64 fp16)")


def test_noalloc_generic_kernels_and_unequal_lengths(capi):
    # A head dimension that is not a multiple of 8 runs the generic kernels: the preprocess kernel,
    # not the dQ kernel, writes delta into the library's scratch.
    want, got = _both_backwards(capi, 2, 2, 200, 333, 50, torch.float16, seed=3)
    _assert_same(want, got, "generic path (B=2 H=2 Nq=200 Nk=333 D=50 fp16)")
    # Head dimension 48 with Nq != Nk: the padded fast kernels, delta formed inside the dQ kernel.
    want, got = _both_backwards(capi, 2, 2, 200, 333, 48, torch.float16, seed=4)
    _assert_same(want, got, "padded fast path (B=2 H=2 Nq=200 Nk=333 D=48 fp16)")


def test_noalloc_refuses_sizes_beyond_its_scratch(capi):
    lib = capi.load()
    rows = capi.FA2_NOALLOC_MAX_ROWS
    # batch * nheads * seqlen_q_rounded one tile above the limit; the size check comes before any
    # pointer is looked at, so small dummy tensors are enough.
    t = torch.zeros(8, dtype=torch.float16, device="cuda")
    n_r = 1024
    b = rows // n_r + 1
    args = [t.data_ptr()] * 9 + [b, 1, n_r, n_r, 64, n_r] + [0] * 24 + [0.125, capi.FA2_DTYPE_F16, 0,
                                                                       capi.FA2_CONFIG_AUTO, None]
    status = lib.fa2_bwd_fused_noalloc(*args)
    assert lib.fa2_status_string(status) == b"FA2_ERR_TOO_LARGE"
    assert b"FA2_NOALLOC_MAX_ROWS" in lib.fa2_last_error_string()
