"""GPU tests of the sequence-parallel backward run the reference's way: one kernel per key tile
that adds its dQ contributions into an fp32 accumulator with global atomics
(_triton_kernels_v2.py:336-339, 466-494), selected through flash_attention_v2_custom with
GFX950_KERNEL_CONFIG_SEQUENCE_PARALLEL_ATOMIC.  Same oracle and tolerance as the other parity tests.
dK and dV are accumulated in a fixed order and must not change from run to run; dQ is a sum whose
order the hardware picks and may differ in its last bits between runs."""

from __future__ import annotations

import math

import pytest
import torch

from oracle import naive_attention as oracle

pytestmark = pytest.mark.gpu

ATOL, RTOL = 2e-2, 1e-2


def _assert_close(name, got, want, atol=ATOL, rtol=RTOL):
    got = got.detach().float().cpu()
    want = want.detach().float().cpu()
    assert got.shape == want.shape, f"{name}: shape {tuple(got.shape)} != {tuple(want.shape)}"
    assert torch.isfinite(got).all(), f"{name} contains NaN or inf"
    err = (got - want).abs()
    bad = err > atol + rtol * want.abs()
    assert not bad.any(), (f"{name}: {int(bad.sum())} of {bad.numel()} elements outside atol={atol} rtol={rtol}; "
                           f"max abs err {err.max().item():.3e} (reference max {want.abs().max().item():.3e})")


def _seeded(shape_q, shape_k, dtype, qk_std=1.0, seed=42):
    gen = torch.Generator().manual_seed(seed)
    q = (torch.randn(shape_q, generator=gen) * qk_std).to(dtype)
    k = (torch.randn(shape_k, generator=gen) * qk_std).to(dtype)
    v = torch.randn(shape_k, generator=gen).to(dtype)
    d_o = torch.randn(shape_q, generator=gen).to(dtype)
    return q, k, v, d_o


def _run_atomic(fa2_module, q, k, v, d_o, scale):
    configs = {torch.cuda.get_device_capability(): fa2_module.GFX950_KERNEL_CONFIG_SEQUENCE_PARALLEL_ATOMIC}
    qg, kg, vg = (t.cuda().requires_grad_(True) for t in (q, k, v))
    out = fa2_module.flash_attention_v2_custom(qg, kg, vg, scale, configs)
    out.backward(d_o.cuda())
    torch.cuda.synchronize()
    return out.detach(), qg.grad, kg.grad, vg.grad


def _run_default(fa, q, k, v, d_o, scale, deterministic):
    qg, kg, vg = (t.cuda().requires_grad_(True) for t in (q, k, v))
    out = fa.flash_attention_v2(qg, kg, vg, scale, deterministic)
    out.backward(d_o.cuda())
    torch.cuda.synchronize()
    return out.detach(), qg.grad, kg.grad, vg.grad


CASES = [
    # (B, H, Nq, Nk, D, dtype, qk_std)
    (1, 1, 128, 128, 128, torch.bfloat16, 1.0),
    (2, 3, 512, 512, 64, torch.float16, 1.0),
    (1, 2, 75, 75, 64, torch.float16, 1.0),        # shorter than one tile
    (1, 2, 300, 300, 128, torch.bfloat16, 1.0),    # ragged tail
    (2, 2, 333, 200, 64, torch.bfloat16, 1.0),     # more queries than keys
    (2, 2, 200, 333, 128, torch.float16, 1.0),     # more keys than queries
    (1, 2, 130, 130, 32, torch.float16, 1.0),
    (1, 3, 640, 640, 64, torch.float16, 3.0),      # peaky softmax
    (1, 2, 1, 77, 64, torch.bfloat16, 1.0),        # single query
]


@pytest.mark.parametrize("case", CASES, ids=lambda c: f"B{c[0]}H{c[1]}Nq{c[2]}Nk{c[3]}D{c[4]}{str(c[5])[6:]}s{c[6]:g}")
def test_atomic_mode_matches_cpu_oracle(fa, fa2_module, case):
    b, h, nq, nk, d, dtype, std = case
    q, k, v, d_o = _seeded((b, h, nq, d), (b, h, nk, d), dtype, std)
    scale = 1.0 / math.sqrt(d)
    want = oracle.naive_backward(q, k, v, d_o, scale, torch.float32)
    got = _run_atomic(fa2_module, q, k, v, d_o, scale)
    for name, g, w in zip(("o", "dq", "dk", "dv"), got, want):
        assert g.dtype == dtype
        _assert_close(name, g, w)
    split = _run_default(fa, q, k, v, d_o, scale, True)
    assert torch.equal(got[0], split[0]), "the forward does not depend on the backward mode"
    for name, g, s in zip(("dq", "dk", "dv"), got[1:], split[1:]):
        _assert_close(f"{name} against the two-kernel backward", g, s.float())


@pytest.mark.parametrize("name", ["C2", "C4"])
def test_atomic_mode_at_benchmark_sizes(fa, fa2_module, workloads, name):
    """BASELINE's both-modes configuration (C2) and its long-sequence one (C4, written to stress the
    dQ atomics) at full size: the atomic backward against the deterministic one, and a rerun of
    itself (dQ may differ in its last bits between runs, dK and dV may not)."""
    w = workloads.WORKLOADS[name]
    q, k, v, d_o = workloads.make_inputs(w, "cpu")
    det = _run_default(fa, q, k, v, d_o, w.softmax_scale, True)
    first = _run_atomic(fa2_module, q, k, v, d_o, w.softmax_scale)
    again = _run_atomic(fa2_module, q, k, v, d_o, w.softmax_scale)
    for key, a, b, c in zip(("o", "dq", "dk", "dv"), first, again, det):
        _assert_close(f"{name} {key}, atomic against deterministic", a, c.float())
        if key == "dq":
            _assert_close(f"{name} dq, atomic rerun", a, b.float())
        else:
            assert torch.equal(a, b), f"{name} {key}: rerun differs"


def test_atomic_mode_through_the_c_abi(fa2_module, capi):
    """Workspace size, the library's own clearing of a dirty workspace, and the refusals."""
    lib = capi.load()
    b, h, n, d = 2, 2, 200, 64
    q, k, v, d_o = (t.cuda() for t in _seeded((b, h, n, d), (b, h, n, d), torch.float16))
    row = fa2_module._atomic_row(d)
    assert capi.config_table()[row]["dq_atomic"] == 1 and capi.config_table()[row]["headdim_padded"] == d
    ws_bytes = lib.fa2_bwd_workspace_bytes(b, h, n, n, d, 0, row)
    assert ws_bytes == b * h * 256 * d * 4  # 200 query rows round up to 256
    assert lib.fa2_bwd_workspace_bytes(b, h, n, n, d, 0, capi.FA2_CONFIG_AUTO) == 0
    scale = 1.0 / math.sqrt(d)
    n_r = 256
    st = torch.cuda.current_stream().cuda_stream
    s3 = fa2_module._strides3
    o = torch.empty_like(q)
    lse = torch.empty((b, h, n_r), dtype=torch.float32, device="cuda")
    delta = torch.empty_like(lse)
    capi.check(lib.fa2_fwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), lse.data_ptr(), b, h, n, n, d, n_r,
                           *s3(q), *s3(k), *s3(v), *s3(o), scale, capi.FA2_DTYPE_F16, capi.FA2_CONFIG_AUTO, st), "fwd")

    def backward(config, deterministic, workspace):
        grads = [torch.full_like(t, float("nan")) for t in (q, k, v)]
        status = lib.fa2_bwd_fused(q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), d_o.data_ptr(),
                                   lse.data_ptr(), delta.data_ptr(), workspace, *(g.data_ptr() for g in grads),
                                   b, h, n, n, d, n_r, *s3(q), *s3(k), *s3(v), *s3(o), *s3(d_o),
                                   *(s for g in grads for s in s3(g)), scale, capi.FA2_DTYPE_F16, deterministic,
                                   config, st)
        torch.cuda.synchronize()
        return status, grads

    status, want = backward(capi.FA2_CONFIG_AUTO, 1, None)
    assert status == 0
    dirty = torch.full((ws_bytes // 4,), 1e30, dtype=torch.float32, device="cuda")  # the library clears it
    status, got = backward(row, 0, dirty.data_ptr())
    assert status == 0, lib.fa2_last_error_string()
    for name, g, w in zip(("dq", "dk", "dv"), got, want):
        _assert_close(name, g, w.float())
    status, _ = backward(row, 0, None)
    assert lib.fa2_status_string(status) == b"FA2_ERR_WORKSPACE"
    status, _ = backward(row, 1, dirty.data_ptr())
    assert lib.fa2_status_string(status) == b"FA2_ERR_BAD_CONFIG"


def test_atomic_mode_refuses_other_head_dimensions(fa2_module):
    q = torch.zeros(1, 1, 64, 96, dtype=torch.float16, device="cuda", requires_grad=True)
    configs = {torch.cuda.get_device_capability(): fa2_module.GFX950_KERNEL_CONFIG_SEQUENCE_PARALLEL_ATOMIC}
    out = fa2_module.flash_attention_v2_custom(q, q, q, None, configs)
    with pytest.raises(ValueError, match="ATOMIC_DQ"):
        out.sum().backward()


def test_atomic_mode_from_concurrent_threads(fa2_module):
    """Four Python threads, each on its own stream with its own problem and its own workspace (the
    launcher allocates one per call), run the atomic backward at the same time: the only atomics in
    the library must not mix between callers.  dK and dV must have the serial call's bits, dQ the
    oracle's values."""
    import threading

    shapes = [(1, 2, 384, 64, torch.float16), (2, 2, 256, 128, torch.bfloat16), (1, 3, 300, 32, torch.float16),
              (1, 2, 640, 64, torch.bfloat16)]
    problems = [_seeded((b, h, n, d), (b, h, n, d), dt, seed=200 + i) for i, (b, h, n, d, dt) in enumerate(shapes)]
    serial = [_run_atomic(fa2_module, *p, None) for p in problems]
    wanted = [oracle.naive_backward(*p, None, torch.float32) for p in problems]
    configs = {torch.cuda.get_device_capability(): fa2_module.GFX950_KERNEL_CONFIG_SEQUENCE_PARALLEL_ATOMIC}
    rounds = 10
    results: list = [None] * len(problems)
    errors: list = []
    start = threading.Barrier(len(problems))

    def worker(i):
        try:
            stream = torch.cuda.Stream()
            q, k, v, d_o = (t.cuda() for t in problems[i])
            torch.cuda.synchronize()
            start.wait()
            with torch.cuda.stream(stream):
                for _ in range(rounds):
                    qg, kg, vg = (t.detach().requires_grad_(True) for t in (q, k, v))
                    out = fa2_module.flash_attention_v2_custom(qg, kg, vg, None, configs)
                    grads = torch.autograd.grad(out, (qg, kg, vg), d_o)
                stream.synchronize()
            results[i] = (out.detach(),) + tuple(grads)
        except Exception as exc:  # noqa: BLE001 - reported by the main thread
            errors.append((i, repr(exc)))
            start.abort()

    threads = [threading.Thread(target=worker, args=(i,)) for i in range(len(problems))]
    for t in threads:
        t.start()
    for t in threads:
        t.join(timeout=100)
    assert not errors, errors
    torch.cuda.synchronize()
    for i, (got, ser, want) in enumerate(zip(results, serial, wanted)):
        assert got is not None, f"thread {i} did not finish"
        assert torch.equal(got[0], ser[0]), f"thread {i}: o differs from the serial call"
        _assert_close(f"thread {i} dq", got[1], want[1])
        for name, a, b in zip(("dk", "dv"), got[2:], ser[2:]):
            assert torch.equal(a, b), f"thread {i}: {name} differs from the serial call"
