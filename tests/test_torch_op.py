"""The torch.library operators: registration and fake kernels on the CPU, numerics and tracing on
the GPU.  They launch the same kernels as flash_attention_v2, so results must be bit-identical."""

import math

import pytest
import torch


def _meta_inputs(dtype=torch.bfloat16, nq=300, nk=200, d=64):
    q = torch.empty(2, 3, nq, d, dtype=dtype, device="meta", requires_grad=True)
    k = torch.empty(2, 3, nk, d, dtype=dtype, device="meta", requires_grad=True)
    v = torch.empty(2, 3, nk, d, dtype=dtype, device="meta", requires_grad=True)
    return q, k, v


def test_operators_are_registered_with_schemas(fa):
    fwd = torch.ops.fa2_gfx950.fwd.default
    bwd = torch.ops.fa2_gfx950.bwd.default
    assert str(fwd._schema) == ("fa2_gfx950::fwd(Tensor q, Tensor k, Tensor v, float softmax_scale, "
                                "bool deterministic) -> (Tensor, Tensor)")
    assert str(bwd._schema) == ("fa2_gfx950::bwd(Tensor q, Tensor k, Tensor v, Tensor out, Tensor lse, "
                                "Tensor d_out, float softmax_scale, bool deterministic) -> "
                                "(Tensor, Tensor, Tensor)")
    assert "flash_attention_v2_op" in fa.__all__


def test_fake_kernels_give_shapes_and_dtypes(fa, capi):
    q, k, v = _meta_inputs()
    out, lse = torch.ops.fa2_gfx950.fwd(q, k, v, 0.125, True)
    n_r = math.ceil(300 / capi.FA2_MAX_HEADDIM) * capi.FA2_MAX_HEADDIM
    assert out.shape == q.shape and out.dtype == q.dtype and out.is_contiguous()
    assert lse.shape == (2, 3, n_r) and lse.dtype == torch.float32
    dq, dk, dv = torch.ops.fa2_gfx950.bwd(q, k, v, out, lse, out, 0.125, False)
    assert dq.shape == q.shape and dk.shape == k.shape and dv.shape == v.shape
    assert dq.dtype == dk.dtype == dv.dtype == q.dtype


def test_autograd_formula_on_meta_tensors(fa):
    """fp32 inputs are cast like the reference does; gradients come back in the input dtype."""
    q, k, v = _meta_inputs(torch.float32)
    out = fa.flash_attention_v2_op(q, k, v)
    assert out.dtype == torch.float32 and out.shape == q.shape and out.requires_grad
    dq, dk, dv = torch.autograd.grad(out, (q, k, v), torch.empty_like(out))
    assert (dq.shape, dk.shape, dv.shape) == (q.shape, k.shape, v.shape)
    assert dq.dtype == dk.dtype == dv.dtype == torch.float32


def test_traced_graph_keeps_the_operator_opaque(fa):
    from torch.fx.experimental.proxy_tensor import make_fx

    def f(q, k, v):
        return fa.flash_attention_v2_op(q, k, v, None, True)

    q, k, v = (t.detach() for t in _meta_inputs(torch.float16))
    graph = make_fx(f, tracing_mode="fake")(q, k, v)
    targets = [n.target for n in graph.graph.nodes if n.op == "call_function"]
    assert torch.ops.fa2_gfx950.fwd.default in targets


# ----------------------------------------------------------------------------------- GPU
def _gpu_inputs(dtype, shape=(2, 3, 200, 64), nk=None):
    g = torch.Generator().manual_seed(42)
    b, h, nq, d = shape
    nk = nk or nq
    q = torch.randn(b, h, nq, d, generator=g).to(dtype).cuda().requires_grad_(True)
    k = torch.randn(b, h, nk, d, generator=g).to(dtype).cuda().requires_grad_(True)
    v = torch.randn(b, h, nk, d, generator=g).to(dtype).cuda().requires_grad_(True)
    d_o = torch.randn(b, h, nq, d, generator=g).to(dtype).cuda()
    return q, k, v, d_o


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("deterministic", [True, False])
def test_operator_path_equals_function_path(fa, dtype, deterministic):
    q, k, v, d_o = _gpu_inputs(dtype, (2, 3, 333, 128), nk=200)
    want = fa.flash_attention_v2(q, k, v, None, deterministic)
    want_g = torch.autograd.grad(want, (q, k, v), d_o)
    got = fa.flash_attention_v2_op(q, k, v, None, deterministic)
    got_g = torch.autograd.grad(got, (q, k, v), d_o)
    assert got.dtype == dtype and torch.equal(got, want)
    for a, b in zip(got_g, want_g):
        assert a.dtype == dtype and torch.equal(a, b)


@pytest.mark.gpu
def test_opcheck(fa):
    q, k, v, d_o = _gpu_inputs(torch.bfloat16, (1, 2, 96, 64))
    utils = ("test_schema", "test_faketensor", "test_autograd_registration", "test_aot_dispatch_static")
    torch.library.opcheck(torch.ops.fa2_gfx950.fwd.default, (q, k, v, 0.125, True), test_utils=utils)
    out, lse = torch.ops.fa2_gfx950.fwd(q.detach(), k.detach(), v.detach(), 0.125, True)
    torch.library.opcheck(torch.ops.fa2_gfx950.bwd.default,
                          (q.detach(), k.detach(), v.detach(), out, lse, d_o, 0.125, True),
                          test_utils=("test_schema", "test_faketensor"))


@pytest.mark.gpu
def test_compiled_graph_matches_eager(fa):
    """torch.compile captures the whole function (no graph break) and gives the eager bits."""
    q, k, v, d_o = _gpu_inputs(torch.bfloat16, (2, 2, 256, 64))

    def f(q, k, v):
        return fa.flash_attention_v2_op(q * 1.0, k, v, None, True)

    want = f(q, k, v)
    want_g = torch.autograd.grad(want, (q, k, v), d_o)
    compiled = torch.compile(f, backend="aot_eager", fullgraph=True)
    got = compiled(q, k, v)
    got_g = torch.autograd.grad(got, (q, k, v), d_o)
    assert torch.equal(got, want)
    for a, b in zip(got_g, want_g):
        assert torch.equal(a, b)
