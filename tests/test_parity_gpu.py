"""GPU parity tests: the HIP kernels, called through the public API and the C ABI, against the
oracle (naive fp32 causal attention) on the same seeded inputs.

Tolerance for O, dQ, dK, dV: ``allclose(atol=2e-2, rtol=1e-2)`` against the fp32 naive result
computed from the same half-precision inputs (the fallback bar of the task statement; the
"2x the Triton kernel's error" form cannot be evaluated because the reference kernels cannot
run beside these).  Deterministic mode: bit-identical across reruns.
"""

from __future__ import annotations

import math

import pytest
import torch
import torch.nn.functional as F

from oracle import naive_attention as oracle
from tests import golden_io

pytestmark = pytest.mark.gpu

ATOL, RTOL = 2e-2, 1e-2


def _assert_close(name, got, want, atol=ATOL, rtol=RTOL):
    got = got.detach().float().cpu()
    want = want.detach().float().cpu()
    assert got.shape == want.shape, f"{name}: shape {tuple(got.shape)} != {tuple(want.shape)}"
    assert not torch.isnan(got).any(), f"{name} contains NaN"
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


def _gpu_fp32_oracle(q, k, v, d_o, scale):
    """The oracle's own code on the GPU in fp32 (full-precision matmul), one head at a time."""
    torch.backends.cuda.matmul.allow_tf32 = False
    torch.set_float32_matmul_precision("highest")
    return oracle.sliced_forward_backward(q.cuda(), k.cuda(), v.cuda(), d_o.cuda(), scale, torch.float32)


# ------------------------------------------------------------------------- small shapes vs CPU oracle
SMALL_CASES = [
    # (B, H, Nq, Nk, D, dtype, qk_std)
    (1, 1, 128, 128, 128, torch.bfloat16, 1.0),
    (2, 4, 512, 512, 64, torch.float16, 1.0),
    (1, 2, 75, 75, 64, torch.float16, 1.0),       # shorter than one tile
    (1, 2, 300, 300, 128, torch.bfloat16, 1.0),   # ragged tail
    (2, 3, 333, 200, 48, torch.float16, 1.0),     # more queries than keys, head dim padded to 64
    (2, 3, 200, 333, 96, torch.bfloat16, 1.0),    # more keys than queries
    (1, 2, 130, 130, 32, torch.float16, 1.0),
    (1, 2, 100, 100, 40, torch.bfloat16, 1.0),    # head dim multiple of 8 but not of 16
    (1, 2, 100, 100, 50, torch.float16, 1.0),     # head dim not a multiple of 8: scalar access path
    (1, 1, 1, 1, 64, torch.float16, 1.0),         # single token
    (1, 2, 1, 77, 64, torch.bfloat16, 1.0),
    (1, 2, 77, 1, 64, torch.bfloat16, 1.0),
    (1, 4, 640, 640, 64, torch.float16, 3.0),     # peaky softmax
    (1, 2, 257, 257, 128, torch.float16, 1.0),
    (1, 2, 200, 200, 160, torch.bfloat16, 1.0),   # head dims above 128: padded to 192 / 256
    (1, 2, 333, 200, 192, torch.float16, 1.0),
    (2, 2, 300, 300, 256, torch.bfloat16, 1.0),
    (1, 1, 130, 130, 250, torch.float16, 1.0),    # above 128 and not a multiple of 8
    # several tiles at head dims above 128 (LDS-direct forward with rows of 256 in LDS, generic backward)
    (1, 2, 450, 200, 256, torch.bfloat16, 1.0),
    (1, 2, 200, 450, 192, torch.float16, 1.0),
    (2, 1, 333, 333, 200, torch.bfloat16, 1.0),   # padded into the row of 256
    (1, 2, 700, 700, 248, torch.float16, 1.0),
    (1, 1, 600, 600, 136, torch.float16, 3.0),    # padded into the row of 192, peaky softmax
    # head dims that are a multiple of 8 below the table row's: the padded LDS-direct kernels
    (2, 2, 333, 333, 8, torch.float16, 1.0),
    (1, 2, 200, 450, 24, torch.bfloat16, 1.0),
    (2, 2, 450, 200, 56, torch.float16, 1.0),
    (1, 2, 333, 333, 72, torch.bfloat16, 1.0),
    (2, 2, 200, 450, 88, torch.float16, 1.0),
    (1, 2, 333, 333, 104, torch.bfloat16, 1.0),
    (1, 2, 450, 200, 120, torch.float16, 1.0),
]


@pytest.mark.parametrize("deterministic", [True, False], ids=["det", "seqpar"])
@pytest.mark.parametrize("case", SMALL_CASES, ids=lambda c: f"B{c[0]}H{c[1]}Nq{c[2]}Nk{c[3]}D{c[4]}{str(c[5])[6:]}s{c[6]:g}")
def test_small_shapes_match_cpu_oracle(fa, case, deterministic):
    b, h, nq, nk, d, dtype, std = case
    q, k, v, d_o = _seeded((b, h, nq, d), (b, h, nk, d), dtype, std)
    scale = 1.0 / math.sqrt(d)
    want = oracle.naive_backward(q, k, v, d_o, scale, torch.float32)
    got = _run(fa, q, k, v, d_o, scale, deterministic)
    for name, g, w in zip(("o", "dq", "dk", "dv"), got, want):
        assert g.dtype == dtype
        _assert_close(name, g, w)


@pytest.mark.parametrize("name", golden_io.NAMES)
def test_golden_fixtures(fa, fa2_module, name):
    g = golden_io.load(name)
    out, dq, dk, dv = _run(fa, g["q"], g["k"], g["v"], g["d_o"], g["scale"], True)
    for key, got in (("o", out), ("dq", dq), ("dk", dk), ("dv", dv)):
        _assert_close(key, got, g[key])


# ------------------------------------------------------------------------- lse and delta through the launchers / C ABI
@pytest.mark.parametrize("shape", [(1, 2, 450, 300, 256, torch.bfloat16), (2, 1, 333, 500, 192, torch.float16),
                                   (1, 2, 513, 513, 160, torch.bfloat16)],
                         ids=lambda c: f"Nq{c[2]}Nk{c[3]}D{c[4]}")
def test_lse_at_large_head_dims(fa2_module, shape):
    """The forward kernels for head dimensions above 128 write the same lse layout (per-head check
    against logsumexp of the masked scores)."""
    b, h, nq, nk, d, dtype = shape
    q, k, v, _ = _seeded((b, h, nq, d), (b, h, nk, d), dtype)
    cfg = fa2_module.GFX950_KERNEL_CONFIG_DETERMINISTIC
    scale = 1 / math.sqrt(d)
    out, lse, _ = fa2_module._flash_attention_forward(
        q.cuda(), k.cuda(), v.cuda(), scale, cfg.block_rows_size, cfg.block_cols_size, cfg.min_block_headdim,
        cfg.max_headdim, cfg.seqlen_cache_divisor, cfg.min_warps, cfg.max_warps, cfg.num_stages)
    torch.cuda.synchronize()
    want = oracle.naive_lse(q, k, scale)
    _assert_close("lse", lse[..., :nq], want, atol=2e-3, rtol=1e-3)
    assert torch.count_nonzero(lse[..., nq:]) == 0, "padded lse rows must be written as zero"
    _assert_close("o", out, oracle.naive_causal_attention(q, k, v, scale))


@pytest.mark.parametrize("name", golden_io.NAMES)
def test_lse_and_delta_match_oracle(fa2_module, capi, name):
    g = golden_io.load(name)
    cfg = fa2_module.GFX950_KERNEL_CONFIG_DETERMINISTIC
    q, k, v, d_o = (g[x].cuda() for x in ("q", "k", "v", "d_o"))
    out, lse, scale = fa2_module._flash_attention_forward(
        q, k, v, g["scale"], cfg.block_rows_size, cfg.block_cols_size, cfg.min_block_headdim,
        cfg.max_headdim, cfg.seqlen_cache_divisor, cfg.min_warps, cfg.max_warps, cfg.num_stages)
    b, h, nq, d = q.shape
    n_r = math.ceil(nq / cfg.max_headdim) * cfg.max_headdim
    assert lse.shape == (b, h, n_r) and lse.dtype == torch.float32
    _assert_close("lse", lse[..., :nq], g["lse"], atol=2e-3, rtol=1e-3)
    assert torch.count_nonzero(lse[..., nq:]) == 0, "padded lse rows must be written as zero"

    delta = torch.full_like(lse, float("nan"))
    lib = capi.load()
    s3 = fa2_module._strides3
    rc = lib.fa2_bwd_preprocess(out.data_ptr(), d_o.data_ptr(), delta.data_ptr(), b, h, nq, d, n_r,
                                *s3(out), *s3(d_o), fa2_module._COMPUTE_DTYPES[q.dtype],
                                torch.cuda.current_stream().cuda_stream)
    capi.check(rc, "fa2_bwd_preprocess")
    torch.cuda.synchronize()
    want = oracle.naive_delta(out.cpu(), d_o.cpu())  # from the half-precision O the kernel saved
    _assert_close("delta", delta[..., :nq], want, atol=1e-3, rtol=1e-4)
    assert torch.count_nonzero(delta[..., nq:]) == 0
    _assert_close("delta vs exact", delta[..., :nq], g["delta"], atol=3e-2, rtol=1e-2)


def test_partial_gradients_through_c_abi(fa2_module, capi):
    """dq == NULL or dk == dv == NULL runs one of the two backward kernels; what it writes is
    bit-identical to the full call and the omitted outputs are left untouched."""
    g = golden_io.load(golden_io.NAMES[0])
    cfg = fa2_module.GFX950_KERNEL_CONFIG_DETERMINISTIC
    q, k, v, d_o = (g[x].cuda() for x in ("q", "k", "v", "d_o"))
    out, lse, scale = fa2_module._flash_attention_forward(
        q, k, v, g["scale"], cfg.block_rows_size, cfg.block_cols_size, cfg.min_block_headdim,
        cfg.max_headdim, cfg.seqlen_cache_divisor, cfg.min_warps, cfg.max_warps, cfg.num_stages)
    b, h, nq, d = q.shape
    nk = k.shape[2]
    n_r = lse.shape[-1]
    lib = capi.load()
    s3 = fa2_module._strides3
    dtype = fa2_module._COMPUTE_DTYPES[q.dtype]
    stream = torch.cuda.current_stream().cuda_stream
    delta = torch.empty_like(lse)
    capi.check(lib.fa2_bwd_preprocess(out.data_ptr(), d_o.data_ptr(), delta.data_ptr(), b, h, nq, d, n_r,
                                      *s3(out), *s3(d_o), dtype, stream), "fa2_bwd_preprocess")

    def run(want_dq, want_dkdv):
        dq, dk, dv = (torch.full_like(t, 7.0) for t in (q, k, v))
        capi.check(lib.fa2_bwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), d_o.data_ptr(), lse.data_ptr(),
                               delta.data_ptr(), None,
                               dq.data_ptr() if want_dq else None,
                               dk.data_ptr() if want_dkdv else None,
                               dv.data_ptr() if want_dkdv else None,
                               b, h, nq, nk, d, n_r, *s3(q), *s3(k), *s3(v), *s3(d_o),
                               *s3(dq), *s3(dk), *s3(dv), scale, dtype, 1, capi.FA2_CONFIG_AUTO, stream),
                   "fa2_bwd")
        torch.cuda.synchronize()
        return dq, dk, dv

    full = run(True, True)
    only_dq = run(True, False)
    only_dkdv = run(False, True)
    assert torch.equal(only_dq[0], full[0])
    assert torch.equal(only_dkdv[1], full[1]) and torch.equal(only_dkdv[2], full[2])
    assert (only_dq[1] == 7).all() and (only_dq[2] == 7).all() and (only_dkdv[0] == 7).all()
    _assert_close("dq", full[0], g["dq"])
    _assert_close("dk", full[1], g["dk"])
    _assert_close("dv", full[2], g["dv"])


@pytest.mark.parametrize("name", golden_io.NAMES)
def test_fused_backward_matches_two_call_path(fa2_module, capi, name):
    """fa2_bwd_fused == fa2_bwd_preprocess + fa2_bwd: delta to rounding (another summation order when
    the dQ kernel forms it), gradients within the parity tolerance of the fixture and close to the
    two-call path; bit-identical where the generic kernels run (delta then comes from the same
    preprocess kernel)."""
    g = golden_io.load(name)
    cfg = fa2_module.GFX950_KERNEL_CONFIG_DETERMINISTIC
    q, k, v, d_o = (g[x].cuda() for x in ("q", "k", "v", "d_o"))
    out, lse, scale = fa2_module._flash_attention_forward(
        q, k, v, g["scale"], cfg.block_rows_size, cfg.block_cols_size, cfg.min_block_headdim,
        cfg.max_headdim, cfg.seqlen_cache_divisor, cfg.min_warps, cfg.max_warps, cfg.num_stages)
    b, h, nq, d = q.shape
    nk = k.shape[2]
    n_r = lse.shape[-1]
    lib = capi.load()
    s3 = fa2_module._strides3
    dtype = fa2_module._COMPUTE_DTYPES[q.dtype]
    stream = torch.cuda.current_stream().cuda_stream

    delta2 = torch.full_like(lse, float("nan"))
    two = [torch.full_like(t, 7.0) for t in (q, k, v)]
    capi.check(lib.fa2_bwd_preprocess(out.data_ptr(), d_o.data_ptr(), delta2.data_ptr(), b, h, nq, d, n_r,
                                      *s3(out), *s3(d_o), dtype, stream), "fa2_bwd_preprocess")
    capi.check(lib.fa2_bwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), d_o.data_ptr(), lse.data_ptr(),
                           delta2.data_ptr(), None, *(t.data_ptr() for t in two),
                           b, h, nq, nk, d, n_r, *s3(q), *s3(k), *s3(v), *s3(d_o),
                           *s3(two[0]), *s3(two[1]), *s3(two[2]), scale, dtype, 1,
                           capi.FA2_CONFIG_AUTO, stream), "fa2_bwd")
    delta1 = torch.full_like(lse, float("nan"))
    one = [torch.full_like(t, 7.0) for t in (q, k, v)]
    capi.check(lib.fa2_bwd_fused(q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), d_o.data_ptr(),
                                 lse.data_ptr(), delta1.data_ptr(), None, *(t.data_ptr() for t in one),
                                 b, h, nq, nk, d, n_r, *s3(q), *s3(k), *s3(v), *s3(out), *s3(d_o),
                                 *s3(one[0]), *s3(one[1]), *s3(one[2]), scale, dtype, 1,
                                 capi.FA2_CONFIG_AUTO, stream), "fa2_bwd_fused")
    torch.cuda.synchronize()
    assert torch.count_nonzero(delta1[..., nq:]) == 0
    torch.testing.assert_close(delta1, delta2, atol=1e-5, rtol=1e-5)
    for key, a, bb in zip(("dq", "dk", "dv"), one, two):
        _assert_close(key, a, g[key])
        torch.testing.assert_close(a.float(), bb.float(), atol=2e-3, rtol=2e-3)
        if d not in (32, 64, 128):
            assert torch.equal(a, bb)
    # Partial gradients are not on offer here.
    rc = lib.fa2_bwd_fused(q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), d_o.data_ptr(),
                           lse.data_ptr(), delta1.data_ptr(), None, None, one[1].data_ptr(), one[2].data_ptr(),
                           b, h, nq, nk, d, n_r, *s3(q), *s3(k), *s3(v), *s3(out), *s3(d_o),
                           *s3(one[0]), *s3(one[1]), *s3(one[2]), scale, dtype, 1, capi.FA2_CONFIG_AUTO, stream)
    assert lib.fa2_status_string(rc).decode() == "FA2_ERR_NULL_POINTER"


# ------------------------------------------------------------------------- the five benchmark configurations at full size
def _workload_case(workloads, name):
    w = workloads.WORKLOADS[name]
    q, k, v, d_o = workloads.make_inputs(w, "cpu")
    return w, q, k, v, d_o


@pytest.mark.parametrize("name", ["C1", "C2", "C3", "C4", "C5"])
def test_baseline_configs_match_oracle(fa, workloads, name):
    """Full-size parity.  C1 against the CPU oracle on every head; the larger ones against the CPU
    oracle on two heads and against the same oracle code run in fp32 on the GPU on every head."""
    w, q, k, v, d_o = _workload_case(workloads, name)
    modes = (True, False) if w.both_modes else (False,)
    cpu_heads = w.batch * w.nheads if name == "C1" else 2
    if name == "C4":
        cpu_heads = 1
    flat = lambda t: t.reshape(w.batch * w.nheads, w.seqlen, w.headdim)  # noqa: E731
    cpu_want = oracle.sliced_forward_backward(q, k, v, d_o, w.softmax_scale, torch.float32, heads=cpu_heads)
    gpu_want = None if name == "C1" else _gpu_fp32_oracle(q, k, v, d_o, w.softmax_scale)
    for deterministic in modes:
        got = _run(fa, q, k, v, d_o, w.softmax_scale, deterministic)
        for key, g, cw in zip(("o", "dq", "dk", "dv"), got, cpu_want):
            _assert_close(f"{name} {key} (cpu oracle, det={deterministic})", flat(g)[:cpu_heads], cw)
        if gpu_want is not None:
            for key, g, gw in zip(("o", "dq", "dk", "dv"), got, gpu_want):
                _assert_close(f"{name} {key} (fp32 oracle on gpu, det={deterministic})", g, gw)
        # size-independent properties
        o, dq, dk, dv = (t.float() for t in got)
        torch.testing.assert_close(o[:, :, 0], v.cuda().float()[:, :, 0], atol=1e-6, rtol=0)  # row 0 == v[0]
        lhs = (q.cuda().float() * dq).sum((-1, -2))
        rhs = (k.cuda().float() * dk).sum((-1, -2))
        scale_ref = (q.cuda().float() * dq).abs().sum((-1, -2))
        assert ((lhs - rhs).abs() <= 2e-2 * scale_ref + 1e-2).all(), "sum(q*dq) != sum(k*dk)"
        torch.testing.assert_close(dv.sum(-2), d_o.cuda().float().sum(-2), atol=0.02 * math.sqrt(w.seqlen), rtol=2e-2)
    # The forward that nothing will differentiate (for bf16 a forward-only row of the table).
    with torch.no_grad():
        out = fa.flash_attention_v2(q.cuda(), k.cuda(), v.cuda(), w.softmax_scale, False)
    _assert_close(f"{name} o, forward only (cpu oracle)", flat(out)[:cpu_heads], cpu_want[0])
    if gpu_want is not None:
        _assert_close(f"{name} o, forward only (fp32 oracle on gpu)", out, gpu_want[0])


def test_constant_values_give_constant_output(fa, workloads):
    """V == 1 makes O == 1 exactly representable: checks the normalisation at full C3 size."""
    w, q, k, v, d_o = _workload_case(workloads, "C3")
    out = fa.flash_attention_v2(q.cuda(), k.cuda(), torch.ones_like(v).cuda())
    torch.testing.assert_close(out.float(), torch.ones_like(out, dtype=torch.float32), atol=8e-3, rtol=0)


# ------------------------------------------------------------------------- determinism
@pytest.mark.parametrize("name,reruns", [("C1", 100), ("C2", 10), ("C3", 3), ("C4", 3), ("C5", 5)])
def test_determinism(fa, workloads, name, reruns):
    """deterministic=True is bit-identical from run to run (reference: tests/test_flash_attention_2.py:321-342)."""
    w, q, k, v, d_o = _workload_case(workloads, name)
    ref = _run(fa, q, k, v, d_o, w.softmax_scale, True)
    for i in range(reruns):
        got = _run(fa, q, k, v, d_o, w.softmax_scale, True)
        for key, a, b in zip(("output", "dq", "dk", "dv"), got, ref):
            assert torch.equal(a, b), f"Non-determinism detected in deterministic mode at rerun {i} for {key}"


def test_non_determinism(fa, workloads):
    """deterministic=False: the reference allows the bits to differ between reruns and does not
    require it (tests/test_flash_attention_2.py:345-385 only reports).  Here both modes run the same
    atomic-free kernels, so reruns are held to the stronger property: identical bits, and equal to
    the deterministic mode's."""
    w, q, k, v, d_o = _workload_case(workloads, "C2")
    ref = _run(fa, q, k, v, d_o, w.softmax_scale, False)
    det = _run(fa, q, k, v, d_o, w.softmax_scale, True)
    for _ in range(5):
        got = _run(fa, q, k, v, d_o, w.softmax_scale, False)
        for key, a, b, c in zip(("output", "dq", "dk", "dv"), got, ref, det):
            assert torch.equal(a, b), f"{key}: rerun differs in the mode that has no atomics either"
            assert torch.equal(a, c), f"{key}: the two backward modes differ"


# ------------------------------------------------------------------------- the reference's own test matrix
REFERENCE_SHAPES = [(8, 12, 512, 32), (16, 16, 1024, 48), (32, 20, 1024, 64), (32, 20, 1024, 96), (64, 32, 2048, 128)]
REFERENCE_IDS = ["small", "medium", "medium+", "large", "large+"]


def _reference_inputs(shape):
    """fp32 inputs on the GPU with requires_grad, as tests/test_flash_attention_2.py:55-72 builds them."""
    torch.manual_seed(42)
    q, k, v = (torch.randn(shape, dtype=torch.float32, device="cuda", requires_grad=True) for _ in range(3))
    return q, k, v, 1.0 / math.sqrt(shape[-1])


@pytest.mark.parametrize("shape", REFERENCE_SHAPES, ids=REFERENCE_IDS)
def test_reference_matrix_forward(fa, shape):
    """Output shape, dtype, NaN-freeness and agreement with vanilla attention and torch SDPA on
    fp32 inputs with the reference's own tolerance (tests/test_flash_attention_2.py:236-318)."""
    q, k, v, scale = _reference_inputs(shape)
    out = fa.flash_attention_v2(q, k, v, scale)
    assert out.shape == q.shape and out.dtype == torch.float32
    assert not torch.isnan(out).any()
    with torch.no_grad():
        sdpa = F.scaled_dot_product_attention(q, k, v, is_causal=True, scale=scale)
        assert torch.allclose(out, sdpa, atol=1e-2, rtol=1e-3), "output doesn't match torch SDPA"
        heads = min(4, shape[0] * shape[1])
        flat = lambda t: t.reshape(-1, 1, shape[2], shape[3])[:heads]  # noqa: E731
        vanilla = oracle.naive_causal_attention(flat(q), flat(k), flat(v), scale)
        assert torch.allclose(flat(out), vanilla, atol=1e-2, rtol=1e-3), "output doesn't match vanilla attention"


@pytest.mark.parametrize("shape", REFERENCE_SHAPES[:4], ids=REFERENCE_IDS[:4])
def test_reference_matrix_gradients(fa, shape):
    """Gradients exist in the input dtype, hold no NaN, and match autograd of vanilla attention
    (the reference only checks for NaN: tests/test_flash_attention_2.py:256-271)."""
    q, k, v, scale = _reference_inputs(shape)
    d_o = torch.randn_like(q)
    fa.flash_attention_v2(q, k, v, scale).backward(d_o)
    for t in (q, k, v):
        assert t.grad is not None and t.grad.dtype == torch.float32 and not torch.isnan(t.grad).any()
    heads = min(4, shape[0] * shape[1])
    flat = lambda t: t.detach().reshape(-1, 1, shape[2], shape[3])[:heads]  # noqa: E731
    _, dq, dk, dv = oracle.naive_backward(flat(q), flat(k), flat(v), flat(d_o), scale, torch.float32)
    _assert_close("dq", flat(q.grad), dq)
    _assert_close("dk", flat(k.grad), dk)
    _assert_close("dv", flat(v.grad), dv)


def test_flash_attention_v2_custom_equals_default(fa, fa2_module):
    """A custom configuration equal to the default gives bit-identical O, dQ, dK, dV
    (tests/test_flash_attention_2.py:388-411)."""
    q, k, v, d_o = _seeded((4, 6, 512, 64), (4, 6, 512, 64), torch.float16)
    cc = torch.cuda.get_device_capability()
    configs = {cc: fa.KernelsConfigV2(
        block_rows_size=128, block_cols_size=64, min_block_headdim=32, max_headdim=128,
        seqlen_cache_divisor=32, min_warps=4, max_warps=4, num_stages=2,
        backward_autotune_configs=[fa.BackwardConfig(
            {"BLOCK_Q_ROWS_SIZE": 64, "BLOCK_KV_COLS_SIZE": 128, "SEQUENCE_PARALLEL": False},
            num_warps=4, num_stages=2, pre_hook=fa.init_to_zero_v2("DQ"))])}
    ref = _run(fa, q, k, v, d_o, None, True)
    qg, kg, vg = (t.cuda().requires_grad_(True) for t in (q, k, v))
    out = fa.flash_attention_v2_custom(qg, kg, vg, None, configs)
    out.backward(d_o.cuda())
    for key, a, b in zip(("output", "dq", "dk", "dv"), (out.detach(), qg.grad, kg.grad, vg.grad), ref):
        assert torch.equal(a, b), f"custom configuration differs from default for {key}"
    with pytest.raises(ValueError, match="Missing kernel configuration"):
        fa.flash_attention_v2_custom(qg, kg, vg, None, {(7, 5): configs[cc]})


def test_custom_max_headdim_after_default_on_the_python_class(fa, fa2_module):
    """N = 100 pads lse to 256 rows under the default max_headdim and to 128 under a custom
    max_headdim = 128 (flash_attention_2.py:98).  Both in a row, same shapes, through the Python
    autograd class, whose backward launcher keeps an argument record per problem: each call's
    backward must use its own row length, and the gradients must agree bit for bit."""
    q, k, v, d_o = _seeded((2, 3, 100, 64), (2, 3, 100, 64), torch.float16)
    cc = torch.cuda.get_device_capability()
    default = fa2_module.GFX950_KERNEL_CONFIG_DETERMINISTIC
    custom = fa.KernelsConfigV2(
        block_rows_size=128, block_cols_size=64, min_block_headdim=32, max_headdim=128,
        seqlen_cache_divisor=32, min_warps=4, max_warps=4, num_stages=2,
        backward_autotune_configs=default.backward_autotune_configs)
    want = oracle.naive_backward(q, k, v, d_o, None, torch.float32)
    results = []
    for cfg in (default, custom, default):
        qg, kg, vg = (t.cuda().requires_grad_(True) for t in (q, k, v))
        out = fa2_module.FlashAttentionV2Function.apply(qg, kg, vg, None, cfg)
        out.backward(d_o.cuda())
        torch.cuda.synchronize()
        results.append((out.detach(), qg.grad, kg.grad, vg.grad))
        for name, got, ref in zip(("o", "dq", "dk", "dv"), results[-1], want):
            _assert_close(f"{name} (max_headdim={cfg.max_headdim})", got, ref)
    for other in results[1:]:
        for name, a, b in zip(("o", "dq", "dk", "dv"), results[0], other):
            assert torch.equal(a, b), f"{name} depends on the lse padding"
    # The same pair through the public functions (the C++ node when it is built).
    qg, kg, vg = (t.cuda().requires_grad_(True) for t in (q, k, v))
    out = fa.flash_attention_v2_custom(qg, kg, vg, None, {cc: custom})
    out.backward(d_o.cuda())
    for name, a, b in zip(("o", "dq", "dk", "dv"), results[0], (out.detach(), qg.grad, kg.grad, vg.grad)):
        assert torch.equal(a, b), f"{name}: flash_attention_v2_custom(max_headdim=128) differs"


@pytest.mark.parametrize("shape", [(2, 3, 640, 640, 128), (2, 2, 333, 200, 48), (1, 4, 1024, 1024, 64), (1, 2, 77, 1, 64)],
                         ids=lambda s: "B%dH%dNq%dNk%dD%d" % s)
def test_forward_only_rows(fa, fa2_module, capi, shape):
    """A forward that nothing will differentiate takes, for bf16 inputs, a table row whose kernel
    folds softmax_scale * log2(e) into Q (rounded to bf16 once) instead of scaling the fp32 scores
    as the reference does (_triton_kernels_v2.py:137-152).  Its O and lse must meet the parity
    tolerance; a forward that a backward may follow, fp16 inputs, ``exact_scale`` configurations
    and the plain row through the C ABI must all give the reference arithmetic's bits."""
    b, h, nq, nk, d = shape
    cc = torch.cuda.get_device_capability()
    exact = {cc: fa.KernelsConfigV2(
        block_rows_size=128, block_cols_size=64, min_block_headdim=32, max_headdim=256,
        seqlen_cache_divisor=32, min_warps=4, max_warps=4, num_stages=2,
        backward_autotune_configs=fa2_module.GFX950_KERNEL_CONFIG_DETERMINISTIC.backward_autotune_configs,
        exact_scale=True)}
    lib = capi.load()
    rows = capi.config_table()
    for dtype, code in ((torch.bfloat16, capi.FA2_DTYPE_BF16), (torch.float16, capi.FA2_DTYPE_F16)):
        q, k, v, d_o = _seeded((b, h, nq, d), (b, h, nk, d), dtype)
        want = oracle.naive_causal_attention(q, k, v, None, torch.float32)
        training = _run(fa, q, k, v, d_o, None, True)[0]
        qc, kc, vc = q.cuda(), k.cuda(), v.cuda()
        with torch.no_grad():
            plain_inputs = fa.flash_attention_v2(qc, kc, vc)
            no_grad = fa.flash_attention_v2(qc.requires_grad_(True), kc, vc)
            exact_cfg = fa.flash_attention_v2_custom(qc, kc, vc, None, exact)
        _assert_close(f"o, forward-only ({dtype})", no_grad, want)
        assert torch.equal(no_grad, plain_inputs), "no_grad and inputs without requires_grad take the same row"
        assert torch.equal(exact_cfg, training), "exact_scale must give the bits of the forward a backward follows"
        only = rows[lib.fa2_pick_config_forward_only(code, d, nq, nk)]
        auto = rows[lib.fa2_pick_config(code, d, nq, nk, 0)]
        assert auto["fwd_exp_folded"] == 0 and only["headdim_padded"] == auto["headdim_padded"]
        if dtype == torch.float16:
            assert only["id"] == auto["id"] and torch.equal(no_grad, training)
        else:
            assert only["fwd_exp_folded"] == 1
        # The same two rows by id through the C ABI, lse included.
        n_r = math.ceil(nq / 128) * 128
        s3 = fa2_module._strides3
        st = torch.cuda.current_stream().cuda_stream
        outs = {}
        for row in (auto, only):
            o = torch.empty_like(qc)
            lse = torch.empty((b, h, n_r), dtype=torch.float32, device="cuda")
            capi.check(lib.fa2_fwd(qc.data_ptr(), kc.data_ptr(), vc.data_ptr(), o.data_ptr(), lse.data_ptr(), b, h, nq,
                                   nk, d, n_r, *s3(qc), *s3(kc), *s3(vc), *s3(o), 1.0 / math.sqrt(d), code, row["id"],
                                   st), "fa2_fwd")
            torch.cuda.synchronize()
            outs[row["id"]] = (o, lse)
        assert torch.equal(outs[auto["id"]][0], training) and torch.equal(outs[only["id"]][0], no_grad)
        want_lse = oracle.naive_lse(q, k, None)
        for row in (auto, only):
            torch.testing.assert_close(outs[row["id"]][1][..., :nq].cpu(), want_lse, atol=2e-2, rtol=1e-2)


def test_flash_attention_data_parallel(fa):
    """nn.DataParallel over the visible GPUs equals the direct call (tests/test_flash_attention_2.py:414-480)."""

    class AttentionModel(torch.nn.Module):
        def forward(self, q, k, v, scale):
            return fa.flash_attention_v2(q, k, v, scale)

    q, k, v, d_o = _seeded((4, 4, 256, 64), (4, 4, 256, 64), torch.float32)
    scale = 0.125
    ref = _run(fa, q, k, v, d_o, scale, False)
    model = torch.nn.DataParallel(AttentionModel().cuda())
    qg, kg, vg = (t.cuda().requires_grad_(True) for t in (q, k, v))
    out = model(qg, kg, vg, scale)
    out.backward(d_o.cuda())
    for a, b in zip((out.detach(), qg.grad, kg.grad, vg.grad), ref):
        assert torch.allclose(a, b, atol=1e-3, rtol=1e-3)


# ------------------------------------------------------------------------- boundary behaviour on the device
def test_non_contiguous_and_mixed_inputs(fa):
    """Inputs are made contiguous and brought to one compute dtype like the reference does
    (flash_attention_2.py:313-316); the output comes back in q's dtype."""
    q, k, v, d_o = _seeded((2, 3, 160, 64), (2, 3, 160, 64), torch.float16)
    want = oracle.naive_backward(q, k, v, d_o, None, torch.float32)
    # (B, N, H, D) storage viewed as (B, H, N, D): non-contiguous
    qn, kn, vn = (t.cuda().transpose(1, 2).contiguous().transpose(1, 2).requires_grad_(True) for t in (q, k, v))
    assert not qn.is_contiguous()
    out = fa.flash_attention_v2(qn, kn, vn)
    out.backward(d_o.cuda().transpose(1, 2).contiguous().transpose(1, 2))
    for name, g, w in zip(("o", "dq", "dk", "dv"), (out, qn.grad, kn.grad, vn.grad), want):
        _assert_close(name, g, w)
    # fp64 q with fp16 k, v: everything is computed in fp16, output in q's dtype
    out64 = fa.flash_attention_v2(q.cuda().double(), k.cuda(), v.cuda())
    assert out64.dtype == torch.float64
    _assert_close("o (fp64 in)", out64, want[0])


def test_zero_scale_means_default_and_explicit_scale_is_used(fa):
    """`softmax_scale or default`: 0.0 selects 1/sqrt(D) (flash_attention_2.py:94)."""
    q, k, v, _ = _seeded((1, 2, 96, 64), (1, 2, 96, 64), torch.bfloat16)
    a = fa.flash_attention_v2(q.cuda(), k.cuda(), v.cuda(), 0.0)
    b = fa.flash_attention_v2(q.cuda(), k.cuda(), v.cuda(), None)
    assert torch.equal(a, b)
    c = fa.flash_attention_v2(q.cuda(), k.cuda(), v.cuda(), 0.5)
    _assert_close("o (scale 0.5)", c, oracle.naive_causal_attention(q, k, v, 0.5))


def test_negative_scale(fa):
    """The reference passes any non-zero scale to its kernels (flash_attention_2.py:94); a negative
    one turns the softmax towards the smallest scores."""
    q, k, v, d_o = _seeded((1, 2, 200, 64), (1, 2, 200, 64), torch.float16)
    want = oracle.naive_backward(q, k, v, d_o, -0.2, torch.float32)
    got = _run(fa, q, k, v, d_o, -0.2, True)
    for name, g, w in zip(("o", "dq", "dk", "dv"), got, want):
        _assert_close(name, g, w)


def test_device_side_assertions(fa):
    q = torch.zeros(1, 2, 16, 64, device="cuda", dtype=torch.float16)
    with pytest.raises(AssertionError):
        fa.flash_attention_v2(q, torch.zeros(1, 2, 16, 32, device="cuda", dtype=torch.float16), q)
    big = torch.zeros(1, 1, 8, 264, device="cuda", dtype=torch.float16)
    with pytest.raises(AssertionError, match="Supports head dimensions only up to"):
        fa.flash_attention_v2(big, big, big)


# ------------------------------------------------------------------------- streams and graph capture
def test_side_stream_and_graph_replay(fa):
    """The library enqueues on the caller's current stream and allocates nothing itself, so a
    forward + backward recorded into a HIP graph replays with the same bits as the eager call, also
    after the inputs change in place.  Replays are interleaved with eager work and synchronisation."""
    q, k, v, d_o = _seeded((2, 4, 320, 64), (2, 4, 320, 64), torch.bfloat16)
    qs, ks, vs, gs = (t.cuda() for t in (q, k, v, d_o))
    for t in (qs, ks, vs):
        t.requires_grad_(True)

    def fwd_bwd():
        out = fa.flash_attention_v2(qs, ks, vs, None, True)
        return (out,) + torch.autograd.grad(out, (qs, ks, vs), gs)

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(2):  # warm-up on the side stream, as graph capture requires
            eager = fwd_bwd()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    want = oracle.naive_backward(q, k, v, d_o, None, torch.float32)
    for name, g, w in zip(("o", "dq", "dk", "dv"), eager, want):
        _assert_close(name, g.cpu(), w)

    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        captured = fwd_bwd()
    for replay in range(3):
        graph.replay()
        torch.cuda.synchronize()
        fresh = fwd_bwd()  # eager work between replays
        torch.cuda.synchronize()
        for a, b in zip(captured, fresh):
            assert torch.equal(a, b), f"replay {replay} differs from the eager result"
        with torch.no_grad():  # new input values, same storage
            qs.mul_(0.5)
            vs.add_(0.25)
