"""GPU tests beyond the fixed parity matrix: ragged shapes on the LDS-direct kernels, a seeded
randomised sweep, the row log-sum-exp at the long and the peaky benchmark sizes, concurrent callers
on one GPU, and the packed entry points.  Same oracle and tolerance as tests/test_parity_gpu.py."""

from __future__ import annotations

import ctypes
import math
import random
import threading

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


def _run(fa, q, k, v, d_o, scale, deterministic):
    qg, kg, vg = (t.cuda().requires_grad_(True) for t in (q, k, v))
    out = fa.flash_attention_v2(qg, kg, vg, scale, deterministic)
    out.backward(d_o.cuda())
    torch.cuda.synchronize()
    return out.detach(), qg.grad, kg.grad, vg.grad


def _gpu_reference(q, k, v, d_o, scale):
    """The oracle's formula in fp32 on the GPU (full-precision matmul), whole tensor at once."""
    torch.backends.cuda.matmul.allow_tf32 = False
    torch.set_float32_matmul_precision("highest")
    return oracle.naive_backward(q.cuda(), k.cuda(), v.cuda(), d_o.cuda(), scale, torch.float32)


# ---------------------------------------------------------------- ragged Nq != Nk on the fast kernels
# Head dimensions 32, 64 and 128 with 16-byte aligned rows run the LDS-direct kernels; these shapes
# walk their clamped-tile, partial-diagonal and "more keys than queries" branches over several tiles.
FAST_RAGGED = [
    (2, 3, 333, 200, 64, torch.float16),
    (2, 3, 200, 333, 128, torch.bfloat16),
    (1, 2, 700, 450, 32, torch.bfloat16),
    (1, 2, 450, 700, 64, torch.bfloat16),
    (1, 3, 1000, 129, 128, torch.float16),
    (1, 2, 129, 1000, 32, torch.float16),
    (1, 2, 513, 511, 128, torch.bfloat16),
]


@pytest.mark.parametrize("deterministic", [True, False], ids=["det", "seqpar"])
@pytest.mark.parametrize("case", FAST_RAGGED, ids=lambda c: f"B{c[0]}H{c[1]}Nq{c[2]}Nk{c[3]}D{c[4]}{str(c[5])[6:]}")
def test_ragged_shapes_on_fast_kernels(fa, case, deterministic):
    b, h, nq, nk, d, dtype = case
    q, k, v, d_o = _seeded((b, h, nq, d), (b, h, nk, d), dtype)
    scale = 1.0 / math.sqrt(d)
    want = oracle.naive_backward(q, k, v, d_o, scale, torch.float32)
    got = _run(fa, q, k, v, d_o, scale, deterministic)
    for name, g, w in zip(("o", "dq", "dk", "dv"), got, want):
        _assert_close(name, g, w)


# ---------------------------------------------------------------- the two autograd nodes
@pytest.mark.parametrize("case", [(2, 3, 333, 200, 64, torch.float16, None), (1, 2, 640, 640, 128, torch.bfloat16, 0.2),
                                  (1, 2, 300, 300, 96, torch.float32, None), (1, 2, 257, 257, 64, torch.bfloat16, -0.125)],
                         ids=["f16", "bf16-scale", "f32-input", "negative-scale"])
def test_cpp_autograd_node_equals_python_class(fa, fa2_module, case):
    """The public function records the C++ node (csrc/fa2_torch_autograd.cpp); the reference-shaped
    Python class FlashAttentionV2Function makes the same launches: outputs and gradients are equal
    bit for bit, input casts and a negative scale included."""
    b, h, nq, nk, d, dtype, scale = case
    assert fa2_module._cpp_node() is not None, "_fa2_torch.so is not built"
    q, k, v, d_o = _seeded((b, h, nq, d), (b, h, nk, d), dtype)
    cfg = fa2_module.GFX950_KERNEL_CONFIG_NON_DETERMINISTIC
    results = []
    for use_class in (False, True):
        qg, kg, vg = (t.cuda().requires_grad_(True) for t in (q, k, v))
        out = (fa2_module.FlashAttentionV2Function.apply(qg, kg, vg, scale, cfg) if use_class
               else fa.flash_attention_v2(qg, kg, vg, scale, False))
        out.backward(d_o.cuda())
        torch.cuda.synchronize()
        results.append((out.detach(), qg.grad, kg.grad, vg.grad))
    for name, a, c in zip(("o", "dq", "dk", "dv"), *results):
        assert a.dtype == c.dtype == dtype, name
        assert torch.equal(a, c), f"{name} differs between the C++ node and the Python class"


# ---------------------------------------------------------------- seeded randomised sweep
def test_randomised_shape_sweep(fa):
    """48 seeded cases of mixed head dimension, Nq != Nk, dtype and mode against the oracle's formula
    evaluated in fp32 on the GPU; stops at the first failure and names the case."""
    rng = random.Random(20240607)
    for case in range(48):
        d = rng.choice([32, 64, 128, 128, 64, 40, 96, 192, 256, 72])
        nq = rng.choice([rng.randint(1, 700), rng.randint(600, 1500), 64 * rng.randint(1, 12), 128 * rng.randint(1, 9)])
        nk = nq if rng.random() < 0.6 else rng.randint(1, 900)
        b, h = rng.randint(1, 2), rng.randint(1, 3)
        dtype = rng.choice([torch.float16, torch.bfloat16])
        deterministic = rng.random() < 0.5
        label = f"case {case}: B={b} H={h} Nq={nq} Nk={nk} D={d} {dtype} deterministic={deterministic}"
        print(label, flush=True)
        q, k, v, d_o = _seeded((b, h, nq, d), (b, h, nk, d), dtype, seed=case)
        scale = 1.0 / math.sqrt(d)
        want = _gpu_reference(q, k, v, d_o, scale)
        got = _run(fa, q, k, v, d_o, scale, deterministic)
        for name, g, w in zip(("o", "dq", "dk", "dv"), got, want):
            _assert_close(f"{label}: {name}", g, w)
        # The same forward with nothing to differentiate (bf16 up to 128 columns: a forward-only row).
        with torch.no_grad():
            out = fa.flash_attention_v2(q.cuda(), k.cuda(), v.cuda(), scale, deterministic)
        _assert_close(f"{label}: o, forward only", out, want[0])


# ---------------------------------------------------------------- lse at the long and the peaky sizes
@pytest.mark.parametrize("name", ["C4", "C5"])
def test_lse_at_benchmark_sizes(fa2_module, workloads, name):
    """Row log-sum-exp against logsumexp of the masked fp32 scores, per head, at N = 16384 (long
    rows: many rescales of the running sum) and at the ragged, peaky configuration."""
    w = workloads.WORKLOADS[name]
    q, k, v, _ = workloads.make_inputs(w, "cuda")
    cfg = fa2_module.GFX950_KERNEL_CONFIG_DETERMINISTIC
    _, lse, scale = fa2_module._flash_attention_forward(
        q, k, v, w.softmax_scale, cfg.block_rows_size, cfg.block_cols_size, cfg.min_block_headdim,
        cfg.max_headdim, cfg.seqlen_cache_divisor, cfg.min_warps, cfg.max_warps, cfg.num_stages)
    torch.cuda.synchronize()
    n = w.seqlen
    assert torch.count_nonzero(lse[..., n:]) == 0
    torch.backends.cuda.matmul.allow_tf32 = False
    torch.set_float32_matmul_precision("highest")
    for b in range(w.batch):
        for h in range(w.nheads):
            want = oracle.naive_lse(q[b:b + 1, h:h + 1], k[b:b + 1, h:h + 1], scale, torch.float32)
            _assert_close(f"{name} lse head ({b},{h})", lse[b:b + 1, h:h + 1, :n], want, atol=2e-3, rtol=1e-4)


# ---------------------------------------------------------------- both modes agree
def test_both_modes_agree_at_long_sequence(fa, workloads):
    """deterministic=True and False give the same gradients at N = 16384 (they run the same
    atomic-free kernels, so the agreement is exact; the reference asks for the parity tolerance)."""
    w = workloads.WORKLOADS["C4"]
    q, k, v, d_o = workloads.make_inputs(w, "cpu")
    a = _run(fa, q, k, v, d_o, w.softmax_scale, True)
    b = _run(fa, q, k, v, d_o, w.softmax_scale, False)
    for name, x, y in zip(("o", "dq", "dk", "dv"), a, b):
        assert torch.equal(x, y), f"{name} differs between the two backward modes"


# ---------------------------------------------------------------- concurrent callers on one GPU
def test_concurrent_threads_on_one_gpu(fa):
    """Eight Python threads, each on its own stream and its own problem, call forward + backward
    at the same time (the situation nn.DataParallel creates with one thread per replica, reference
    tests/test_flash_attention_2.py:438-448, here on the one GPU there is).  Every thread must get
    the bits the serial call gives: the library keeps no mutable state between calls, takes the
    stream per call, and the launcher's argument records are per thread."""
    shapes = [(1, 2, 384, 64), (2, 2, 256, 128), (1, 3, 300, 64), (1, 1, 512, 128),
              (2, 1, 200, 32), (1, 2, 640, 64), (1, 2, 129, 128), (1, 4, 256, 96)]
    problems = [_seeded(s, s, torch.bfloat16 if i % 2 else torch.float16, seed=100 + i) for i, s in enumerate(shapes)]
    serial = [_run(fa, *p, None, bool(i % 2)) for i, p in enumerate(problems)]
    rounds = 20
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
                    out = fa.flash_attention_v2(qg, kg, vg, None, bool(i % 2))
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
    for i, (got, want) in enumerate(zip(results, serial)):
        assert got is not None, f"thread {i} did not finish"
        for name, a, b in zip(("o", "dq", "dk", "dv"), got, want):
            assert torch.equal(a, b), f"thread {i}: {name} differs from the serial call"


# ---------------------------------------------------------------- packed entry points
def test_packed_entry_points_equal_the_long_ones(fa2_module, capi):
    """fa2_fwd_packed / fa2_bwd_packed give the bits fa2_fwd / fa2_bwd_fused / fa2_bwd give."""
    lib = capi.load()
    q, k, v, d_o = (t.cuda() for t in _seeded((2, 3, 333, 64), (2, 3, 200, 64), torch.bfloat16))
    b, h, nq, d = q.shape
    nk = k.shape[2]
    n_r = 512
    dtype = fa2_module._COMPUTE_DTYPES[q.dtype]
    scale = 0.11
    s3 = fa2_module._strides3
    stream = torch.cuda.current_stream().cuda_stream

    def tensor(t):
        return capi.Tensor(t.data_ptr() if t is not None else None, *(s3(t) if t is not None else (0, 0, 0)))

    o1, o2 = torch.empty_like(q), torch.empty_like(q)
    lse1 = torch.empty((b, h, n_r), device="cuda", dtype=torch.float32)
    lse2 = torch.empty_like(lse1)
    capi.check(lib.fa2_fwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), o1.data_ptr(), lse1.data_ptr(), b, h, nq, nk, d,
                           n_r, *s3(q), *s3(k), *s3(v), *s3(o1), scale, dtype, capi.FA2_CONFIG_AUTO, stream), "fa2_fwd")
    fwd = capi.FwdArgs(tensor(q), tensor(k), tensor(v), tensor(o2), lse2.data_ptr(), b, h, nq, nk, d, n_r, scale,
                       dtype, capi.FA2_CONFIG_AUTO)
    capi.check(lib.fa2_fwd_packed(ctypes.byref(fwd), stream), "fa2_fwd_packed")
    torch.cuda.synchronize()
    assert torch.equal(o1, o2) and torch.equal(lse1, lse2)

    def grads():
        return [torch.full_like(t, 7.0) for t in (q, k, v)]

    # fused: delta is formed on the way
    g1, g2 = grads(), grads()
    delta1, delta2 = torch.empty_like(lse1), torch.empty_like(lse1)
    capi.check(lib.fa2_bwd_fused(q.data_ptr(), k.data_ptr(), v.data_ptr(), o1.data_ptr(), d_o.data_ptr(),
                                 lse1.data_ptr(), delta1.data_ptr(), None, *(t.data_ptr() for t in g1),
                                 b, h, nq, nk, d, n_r, *s3(q), *s3(k), *s3(v), *s3(o1), *s3(d_o),
                                 *s3(g1[0]), *s3(g1[1]), *s3(g1[2]), scale, dtype, 0, capi.FA2_CONFIG_AUTO, stream),
               "fa2_bwd_fused")
    bwd = capi.BwdArgs(tensor(q), tensor(k), tensor(v), tensor(o1), tensor(d_o), tensor(g2[0]), tensor(g2[1]),
                       tensor(g2[2]), lse1.data_ptr(), delta2.data_ptr(), None, b, h, nq, nk, d, n_r, scale, dtype, 0,
                       capi.FA2_CONFIG_AUTO)
    capi.check(lib.fa2_bwd_packed(ctypes.byref(bwd), stream), "fa2_bwd_packed")
    torch.cuda.synchronize()
    assert torch.equal(delta1, delta2)
    for a, c in zip(g1, g2):
        assert torch.equal(a, c)

    # o.ptr == NULL: delta is an input, dk == dv == NULL skips the dK/dV kernel
    g3 = grads()
    bwd.o = tensor(None)
    bwd.dq, bwd.dk, bwd.dv = tensor(g3[0]), tensor(None), tensor(None)
    capi.check(lib.fa2_bwd_packed(ctypes.byref(bwd), stream), "fa2_bwd_packed (dq only)")
    torch.cuda.synchronize()
    assert torch.equal(g3[0], g1[0]) and (g3[1] == 7).all() and (g3[2] == 7).all()
    assert lib.fa2_status_string(lib.fa2_fwd_packed(None, stream)).decode() == "FA2_ERR_NULL_POINTER"


def test_preprocess_accepts_many_heads(fa2_module, capi):
    """batch * nheads above 65535 (the limit of a grid's second dimension) through fa2_bwd_preprocess."""
    lib = capi.load()
    b, h, n, d = 1, 70000, 16, 32
    gen = torch.Generator().manual_seed(3)
    o = torch.randn((b, h, n, d), generator=gen).to(torch.float16).cuda()
    d_o = torch.randn((b, h, n, d), generator=gen).to(torch.float16).cuda()
    delta = torch.empty((b, h, n), device="cuda", dtype=torch.float32)
    s3 = fa2_module._strides3
    capi.check(lib.fa2_bwd_preprocess(o.data_ptr(), d_o.data_ptr(), delta.data_ptr(), b, h, n, d, n, *s3(o), *s3(d_o),
                                      capi.FA2_DTYPE_F16, torch.cuda.current_stream().cuda_stream), "fa2_bwd_preprocess")
    torch.cuda.synchronize()
    torch.testing.assert_close(delta, (o.float() * d_o.float()).sum(-1), atol=1e-3, rtol=1e-4)
