"""CPU-only tests: the oracle against the golden fixtures, the C-ABI library's exports and
argument validation (no kernel is launched), and the Python boundary's contract."""

from __future__ import annotations

import ctypes
import dataclasses
import pathlib
import re

import pytest
import torch

from oracle import naive_attention as oracle
from tests import golden_io

ROOT = pathlib.Path(__file__).resolve().parent.parent


# ------------------------------------------------------------------ oracle vs golden fixtures
@pytest.mark.parametrize("name", golden_io.NAMES)
def test_oracle_reproduces_golden_fixture(name):
    g = golden_io.load(name)
    o, dq, dk, dv = oracle.naive_backward(g["q"], g["k"], g["v"], g["d_o"], g["scale"], torch.float32)
    lse = oracle.naive_lse(g["q"], g["k"], g["scale"])
    for got, key in ((o, "o"), (dq, "dq"), (dk, "dk"), (dv, "dv"), (lse, "lse")):
        torch.testing.assert_close(got, g[key], atol=2e-5, rtol=2e-5)


# ------------------------------------------------------------------ C ABI: exports and errors
def _declared_functions() -> list[str]:
    text = (ROOT / "include" / "fa2_gfx950.h").read_text()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return re.findall(r"\b(fa2_[a-z0-9_]+)\s*\(", text)


def test_library_exports_every_declared_symbol(capi):
    lib = capi.load()
    names = sorted(set(_declared_functions()))
    assert names, "no declarations found in include/fa2_gfx950.h"
    for name in names:
        assert hasattr(lib, name), f"libfa2_gfx950.so does not export {name}"
    assert sorted(capi.SIGNATURES) == names, "ctypes binding and header disagree on the entry points"


def test_abi_version_and_table(capi):
    lib = capi.load()
    assert lib.fa2_abi_version() == capi.ABI_VERSION
    rows = capi.config_table()
    assert [r["id"] for r in rows] == list(range(len(rows)))
    # The rows FA2_CONFIG_AUTO picks from (plain), and the forward-only rows whose forward folds the
    # softmax scale into Q (what fa2_pick_config_forward_only returns for bf16 up to 128 columns).
    plain = [r for r in rows if not r["dq_atomic"] and not r["fwd_exp_folded"]]
    folded = [r for r in rows if r["fwd_exp_folded"]]
    assert [r["headdim_padded"] for r in plain] == [32, 64, 96, 128, 192, 256]
    assert [r["headdim_padded"] for r in folded] == [32, 64, 96, 128]
    assert plain[-1]["headdim_padded"] == capi.FA2_MAX_HEADDIM
    for r in rows:
        assert r["fwd_block_q"] == 32 * r["fwd_waves"]
        assert r["bwd_block_kv"] == 32 * r["bwd_waves"]
        assert r["dq_block_q"] == 32 * r["dq_waves"]
    by_dim = {r["headdim_padded"]: r for r in plain}
    for r in folded:  # a folded row differs from the plain row of its head dimension in that flag only
        twin = dict(by_dim[r["headdim_padded"]], id=r["id"], fwd_exp_folded=1)
        assert r == twin and not r["dq_atomic"]
    for d, want in ((1, 32), (32, 32), (33, 64), (48, 64), (64, 64), (96, 96), (100, 128), (128, 128),
                    (129, 192), (192, 192), (193, 256), (256, 256)):
        for dtype, seqlen in ((capi.FA2_DTYPE_F16, 512), (capi.FA2_DTYPE_BF16, 512), (capi.FA2_DTYPE_BF16, 16384)):
            idx = lib.fa2_pick_config(dtype, d, seqlen, seqlen, 0)
            assert idx >= 0 and rows[idx]["headdim_padded"] == want
            assert not rows[idx]["dq_atomic"] and not rows[idx]["fwd_exp_folded"]
            assert lib.fa2_pick_config(dtype, d, seqlen, seqlen, 1) == idx  # both backward modes share the row
            only = lib.fa2_pick_config_forward_only(dtype, d, seqlen, seqlen)
            assert only >= 0 and rows[only]["headdim_padded"] == want and not rows[only]["dq_atomic"]
            assert rows[only]["fwd_exp_folded"] == int(dtype == capi.FA2_DTYPE_BF16 and want <= 128)
    assert lib.fa2_pick_config_forward_only(capi.FA2_DTYPE_BF16, 257, 512, 512) == -4  # FA2_ERR_HEADDIM
    # LDS-direct kernels: all three up to 128 columns, forward and dQ only at 192 and 256.
    assert [r["lds_direct"] for r in plain] == [1, 1, 1, 1, 2, 2]
    # (batch, head) pairs dispatched together: a multiple of 8 (one XCD per head), fewer at 128 columns.
    assert all(r["head_group"] % 8 == 0 and r["head_group"] > 0 for r in rows)
    assert by_dim[128]["head_group"] < by_dim[64]["head_group"]
    assert lib.fa2_pick_config(capi.FA2_DTYPE_BF16, 257, 512, 512, 0) == -4  # FA2_ERR_HEADDIM
    assert lib.fa2_pick_config(7, 64, 512, 512, 0) == -3  # FA2_ERR_BAD_DTYPE
    info = capi.ConfigInfo()
    assert lib.fa2_config_get(99, ctypes.byref(info)) == 6  # FA2_ERR_BAD_CONFIG
    assert lib.fa2_config_get(0, None) == 1  # FA2_ERR_NULL_POINTER


def _fwd_args(capi, **over):
    a = dict(q=16, k=16, v=16, o=16, lse=16, batch=1, nheads=1, seqlen_q=8, seqlen_k=8, headdim=64,
             seqlen_q_rounded=128, scale=0.125, dtype=capi.FA2_DTYPE_F16, config=capi.FA2_CONFIG_AUTO)
    a.update(over)
    strides = [a["seqlen_q"] * a["headdim"], a["seqlen_q"] * a["headdim"], a["headdim"]] * 4
    if "strides" in over:
        strides = over["strides"]
    return [a["q"], a["k"], a["v"], a["o"], a["lse"], a["batch"], a["nheads"], a["seqlen_q"], a["seqlen_k"],
            a["headdim"], a["seqlen_q_rounded"], *strides, a["scale"], a["dtype"], a["config"], None]


@pytest.mark.parametrize("over,status", [
    (dict(q=None), "FA2_ERR_NULL_POINTER"),
    (dict(lse=None), "FA2_ERR_NULL_POINTER"),
    (dict(batch=0), "FA2_ERR_BAD_SHAPE"),
    (dict(seqlen_k=-3), "FA2_ERR_BAD_SHAPE"),
    (dict(seqlen_q=300, seqlen_q_rounded=256), "FA2_ERR_BAD_SHAPE"),
    (dict(headdim=264), "FA2_ERR_HEADDIM"),
    (dict(dtype=5), "FA2_ERR_BAD_DTYPE"),
    (dict(config=17), "FA2_ERR_BAD_CONFIG"),
    (dict(config=0, headdim=64), "FA2_ERR_BAD_CONFIG"),  # row 0 is built for headdim <= 32
    (dict(scale=float("nan")), "FA2_ERR_BAD_SHAPE"),
    (dict(strides=[-1] * 12), "FA2_ERR_BAD_STRIDE"),
])
def test_forward_rejects_bad_arguments_before_launching(capi, over, status):
    """Every error returns a status and a message; nothing is launched, thrown or aborted."""
    lib = capi.load()
    rc = lib.fa2_fwd(*_fwd_args(capi, **over))
    assert rc != 0
    assert lib.fa2_status_string(rc).decode() == status
    assert lib.fa2_last_error_string().decode() != ""
    with pytest.raises(RuntimeError, match=status):
        capi.check(rc, "fa2_fwd")


def test_backward_entry_points_reject_bad_arguments(capi):
    lib = capi.load()
    st = [512, 512, 64]
    rc = lib.fa2_bwd_preprocess(None, 16, 16, 1, 1, 8, 64, 128, *st, *st, capi.FA2_DTYPE_F16, None)
    assert lib.fa2_status_string(rc).decode() == "FA2_ERR_NULL_POINTER"
    rc = lib.fa2_bwd_preprocess(16, 16, 16, 1, 1, 8, 300, 128, *st, *st, capi.FA2_DTYPE_F16, None)
    assert lib.fa2_status_string(rc).decode() == "FA2_ERR_HEADDIM"
    rc = lib.fa2_bwd(16, 16, 16, 16, 16, None, None, 16, 16, 16, 1, 1, 8, 8, 64, 128, *(st * 7),
                     0.125, capi.FA2_DTYPE_F16, 1, capi.FA2_CONFIG_AUTO, None)
    assert lib.fa2_status_string(rc).decode() == "FA2_ERR_NULL_POINTER"
    assert "delta" in lib.fa2_last_error_string().decode()
    rc = lib.fa2_bwd(16, 16, 16, 16, 16, 16, None, 16, 16, 16, 1, 1, 0, 8, 64, 128, *(st * 7),
                     0.125, capi.FA2_DTYPE_F16, 1, capi.FA2_CONFIG_AUTO, None)
    assert lib.fa2_status_string(rc).decode() == "FA2_ERR_BAD_SHAPE"
    assert lib.fa2_bwd_workspace_bytes(2, 4, 512, 512, 64, 1, capi.FA2_CONFIG_AUTO) == 0
    # Either gradient group may be omitted, but not both, and dk/dv only together.
    rc = lib.fa2_bwd(16, 16, 16, 16, 16, 16, None, None, None, None, 1, 1, 8, 8, 64, 128, *(st * 7),
                     0.125, capi.FA2_DTYPE_F16, 1, capi.FA2_CONFIG_AUTO, None)
    assert lib.fa2_status_string(rc).decode() == "FA2_ERR_NULL_POINTER"
    assert "all NULL" in lib.fa2_last_error_string().decode()
    rc = lib.fa2_bwd(16, 16, 16, 16, 16, 16, None, 16, 16, None, 1, 1, 8, 8, 64, 128, *(st * 7),
                     0.125, capi.FA2_DTYPE_F16, 1, capi.FA2_CONFIG_AUTO, None)
    assert lib.fa2_status_string(rc).decode() == "FA2_ERR_NULL_POINTER"
    assert "dv" in lib.fa2_last_error_string().decode()
    # A forward-only row (its forward rounds Q * scale) is refused by the backward.
    only = lib.fa2_pick_config_forward_only(capi.FA2_DTYPE_BF16, 64, 8, 8)
    assert capi.config_table()[only]["fwd_exp_folded"] == 1
    rc = lib.fa2_bwd(16, 16, 16, 16, 16, 16, None, 16, 16, 16, 1, 1, 8, 8, 64, 128, *(st * 7),
                     0.125, capi.FA2_DTYPE_BF16, 1, only, None)
    assert lib.fa2_status_string(rc).decode() == "FA2_ERR_BAD_CONFIG"
    assert "forward-only" in lib.fa2_last_error_string().decode()


def test_missing_library_fails_loudly(capi, monkeypatch, tmp_path):
    monkeypatch.setattr(capi, "_lib", None)
    monkeypatch.setattr(capi, "LIBRARY_PATH", tmp_path / "libfa2_gfx950.so")
    with pytest.raises(RuntimeError, match="not built"):
        capi.load()


# ------------------------------------------------------------------ Python boundary contract
def test_public_names_match_reference(fa):
    """Reference: src/flash_attention_triton/__init__.py:13."""
    for name in ("KernelsConfigV2", "flash_attention_v2", "flash_attention_v2_custom", "init_to_zero_v2"):
        assert name in fa.__all__ and hasattr(fa, name)


def test_kernels_config_is_a_frozen_record_with_reference_fields(fa):
    fields = [f.name for f in dataclasses.fields(fa.KernelsConfigV2)]
    # The reference's nine fields in its order (_configurators_v2.py:27-38), then the one optional
    # field this package adds; a configuration written for the reference constructs unchanged.
    assert fields == ["block_rows_size", "block_cols_size", "min_block_headdim", "max_headdim",
                      "seqlen_cache_divisor", "min_warps", "max_warps", "num_stages",
                      "backward_autotune_configs", "exact_scale"]
    cfg = fa.KernelsConfigV2(128, 64, 32, 128, 32, 4, 4, 2, [
        fa.BackwardConfig({"BLOCK_Q_ROWS_SIZE": 64, "BLOCK_KV_COLS_SIZE": 128, "SEQUENCE_PARALLEL": False},
                          num_warps=4, num_stages=2, pre_hook=fa.init_to_zero_v2("DQ"))])
    with pytest.raises(dataclasses.FrozenInstanceError):
        cfg.block_rows_size = 64
    assert cfg.deterministic is True and cfg.exact_scale is False
    par = dataclasses.replace(cfg, backward_autotune_configs=[
        fa.BackwardConfig({"BLOCK_Q_ROWS_SIZE": 64, "BLOCK_KV_COLS_SIZE": 128, "SEQUENCE_PARALLEL": True})])
    assert par.deterministic is False


def test_init_to_zero_hook_zeroes_named_tensor(fa):
    hook = fa.init_to_zero_v2("DQ")
    t = torch.ones(4)
    assert hook({"DQ": t, "DK": torch.ones(2)}) is t
    assert torch.count_nonzero(t) == 0


def test_selector_and_validation(fa2_module, monkeypatch):
    sel = fa2_module._select_optimal_gpu_architecture
    assert sel((9, 5), True) is fa2_module.GFX950_KERNEL_CONFIG_DETERMINISTIC
    assert sel((9, 5), False) is fa2_module.GFX950_KERNEL_CONFIG_NON_DETERMINISTIC
    assert sel((9, 5), True).deterministic and not sel((9, 5), False).deterministic
    with pytest.raises(ValueError, match="Unsupported GPU compute capability"):
        sel((9, 4), False)
    with pytest.raises(RuntimeError, match="gfx950"):
        fa2_module._validate_runtime_compatibility((9, 4), "gfx942:sramecc+:xnack-")
    fa2_module._validate_runtime_compatibility((9, 5), "gfx950:sramecc+:xnack-")

    # flash_attention_v2_custom: a missing key for the current device is a ValueError
    monkeypatch.setattr(torch.cuda, "get_device_capability", lambda *a, **k: (9, 5))
    q = torch.zeros(1, 1, 4, 8)
    with pytest.raises(ValueError, match="Missing kernel configuration"):
        fa2_module.flash_attention_v2_custom(q, q, q, None, {(8, 0): sel((9, 5), True)})


def test_custom_tile_fields_are_reported_not_silently_dropped(fa, fa2_module, monkeypatch):
    """The reference passes a custom configuration's tile and warp values to its kernels
    (flash_attention_2.py:137-141); here they cannot change the compiled kernels, and the caller is
    told so once.  The compiled shapes themselves raise no warning."""
    import warnings

    monkeypatch.setattr(fa2_module, "_TILE_WARNING_SHOWN", False)
    ampere = fa.KernelsConfigV2(256, 256, 32, 256, 32, 8, 8, 1, [
        fa.BackwardConfig({"BLOCK_Q_ROWS_SIZE": 128, "BLOCK_KV_COLS_SIZE": 128, "SEQUENCE_PARALLEL": False})])
    with warnings.catch_warnings(record=True) as seen:
        warnings.simplefilter("always")
        fa2_module._warn_about_ignored_tile_fields(fa2_module.GFX950_KERNEL_CONFIG_DETERMINISTIC)
        fa2_module._warn_about_ignored_tile_fields(fa2_module.GFX950_KERNEL_CONFIG_SEQUENCE_PARALLEL_ATOMIC)
        assert not seen
        fa2_module._warn_about_ignored_tile_fields(ampere)
        fa2_module._warn_about_ignored_tile_fields(ampere)
    assert len(seen) == 1 and "ignored" in str(seen[0].message) and "exact_scale" in str(seen[0].message)


def test_launcher_assertions_mirror_reference(fa2_module):
    """Same AssertionErrors as flash_attention_2.py:85-90, raised before any FFI call."""
    cfg = fa2_module.GFX950_KERNEL_CONFIG_DETERMINISTIC
    tail = (cfg.block_rows_size, cfg.block_cols_size, cfg.min_block_headdim, cfg.max_headdim,
            cfg.seqlen_cache_divisor, cfg.min_warps, cfg.max_warps, cfg.num_stages)
    fwd = fa2_module._flash_attention_forward
    q = torch.zeros(1, 2, 8, 16, dtype=torch.float16)
    with pytest.raises(AssertionError):
        fwd(q, torch.zeros(1, 2, 8, 32, dtype=torch.float16), q, None, *tail)  # k shape
    with pytest.raises(AssertionError):
        fwd(q, q, torch.zeros(1, 3, 8, 16, dtype=torch.float16), None, *tail)  # v shape
    big = torch.zeros(1, 1, 4, 264, dtype=torch.float16)
    with pytest.raises(AssertionError, match="Supports head dimensions only up to 256"):
        fwd(big, big, big, None, *tail)
    with pytest.raises(AssertionError, match="must reside on CUDA device"):
        fwd(q, q, q, None, *tail)


def test_backward_record_follows_the_lse_row_length(fa2_module, monkeypatch):
    """The cached argument record of the backward launcher is per padded lse row length: the same
    shapes under another max_headdim (N = 100 pads to 256 or to 128, flash_attention_2.py:98) must
    not be handed the earlier call's seqlen_q_rounded, which the kernels index lse and delta with."""
    seen = []

    class FakeLibrary:
        @staticmethod
        def fa2_bwd_workspace_bytes(*_):
            return 0

        @staticmethod
        def fa2_bwd_packed(args, _stream):
            seen.append((args.seqlen_q, args.seqlen_q_rounded))
            return 0

    monkeypatch.setattr(fa2_module._capi, "load", lambda: FakeLibrary)
    monkeypatch.setattr(fa2_module, "_stream_handle", lambda: 0)
    base = fa2_module.GFX950_KERNEL_CONFIG_DETERMINISTIC
    q = torch.zeros(1, 2, 100, 64, dtype=torch.float16)
    grads = [torch.empty_like(q) for _ in range(3)]
    for max_headdim, rounded in ((256, 256), (128, 128), (256, 256)):
        cfg = dataclasses.replace(base, max_headdim=max_headdim)
        lse = torch.zeros(1, 2, rounded)
        fa2_module._flash_attention_backward(q, q, q, q, lse, *grads, q, None, cfg)
        with pytest.raises(AssertionError):  # an lse of another row length is refused, as in the reference
            fa2_module._flash_attention_backward(q, q, q, q, torch.zeros(1, 2, rounded + 128), *grads, q, None, cfg)
    assert seen == [(100, 256), (100, 128), (100, 256)]


def test_cpp_autograd_node_is_built_and_matches_the_library(capi, fa2_module):
    """The C++ autograd node (csrc/fa2_torch_autograd.cpp) loads without a GPU, is linked against
    the same ABI as the ctypes binding, and is what the public functions record."""
    node = fa2_module._cpp_node()
    assert node is not None, "flash-attention-triton_amd/_fa2_torch.so is not built (python flash-attention-triton_amd/build.py)"
    assert node.abi_version() == capi.ABI_VERSION
    q = torch.zeros(1, 2, 8, 16, dtype=torch.float16)
    with pytest.raises(AssertionError, match="must reside on CUDA device"):  # the launcher's checks come first
        fa2_module._apply(q, q, q, None, fa2_module.GFX950_KERNEL_CONFIG_DETERMINISTIC)


def test_noalloc_entry_point_refuses_sizes_beyond_its_scratch(capi):
    """The size check of fa2_bwd_fused_noalloc comes before anything touches a device."""
    lib = capi.load()
    n_r = 1024
    b = capi.FA2_NOALLOC_MAX_ROWS // n_r + 1
    args = [16] * 9 + [b, 1, n_r, n_r, 64, n_r] + [0] * 24 + [0.125, capi.FA2_DTYPE_F16, 0, capi.FA2_CONFIG_AUTO, None]
    status = lib.fa2_bwd_fused_noalloc(*args)
    assert lib.fa2_status_string(status) == b"FA2_ERR_TOO_LARGE"
    assert b"FA2_NOALLOC_MAX_ROWS" in lib.fa2_last_error_string()


def test_sequence_parallel_rows_and_workspace(capi, fa2_module):
    """The table's sequence-parallel rows are never picked automatically, size their workspace, and
    the configuration classes select them."""
    lib = capi.load()
    rows = capi.config_table()
    atomic = [r for r in rows if r["dq_atomic"]]
    assert sorted(r["headdim_padded"] for r in atomic) == [32, 64, 128]
    for d in (8, 32, 64, 96, 128, 200, 256):
        assert rows[lib.fa2_pick_config(capi.FA2_DTYPE_BF16, d, 512, 512, 0)]["dq_atomic"] == 0
    for r in atomic:
        d = r["headdim_padded"]
        assert lib.fa2_bwd_workspace_bytes(2, 3, 130, 77, d, 0, r["id"]) == 2 * 3 * 192 * d * 4
        assert lib.fa2_bwd_workspace_bytes(2, 3, 130, 77, d, 0, capi.FA2_CONFIG_AUTO) == 0
    assert fa2_module.GFX950_KERNEL_CONFIG_SEQUENCE_PARALLEL_ATOMIC.atomic_dq
    assert not fa2_module.GFX950_KERNEL_CONFIG_SEQUENCE_PARALLEL_ATOMIC.deterministic
    assert not fa2_module.GFX950_KERNEL_CONFIG_NON_DETERMINISTIC.atomic_dq
    assert not fa2_module.GFX950_KERNEL_CONFIG_DETERMINISTIC.atomic_dq


def test_workload_table_matches_baseline(workloads):
    w = workloads.WORKLOADS
    assert w["C1"].shape == (2, 4, 512, 64) and w["C1"].dtype == torch.float16
    assert w["C2"].shape == (4, 16, 2048, 64) and w["C2"].dtype == torch.bfloat16 and w["C2"].both_modes
    assert w["C3"].shape == (2, 32, 4096, 128) and w["C3"].dtype == torch.bfloat16
    assert w["C4"].shape == (1, 16, 16384, 128) and w["C4"].both_modes
    assert w["C5"].shape == (8, 12, 3000, 64) and w["C5"].qk_std == 3.0
    assert w["C3"].fwd_flops == pytest.approx(274.88e9, rel=1e-3)
    assert w["C3"].fwd_bytes == pytest.approx(269.5e6, rel=1e-3)
    q, k, v, g = workloads.make_inputs(w["C1"])
    q2, *_ = workloads.make_inputs(w["C1"], heads=3)
    assert q.dtype == torch.float16 and q.shape == (2, 4, 512, 64)
    torch.testing.assert_close(q2[:, 0], q.reshape(8, 512, 64)[:3], atol=0, rtol=0)


def test_traffic_stamp_ignores_comments_and_follows_code(tmp_path, monkeypatch):
    """bench.py drops the measured HBM traffic when the kernel sources have changed since the
    counter run.  The stamp it compares must not move when comments or layout change (nobody should
    have to re-stamp a summary by hand) and must move when code does."""
    import importlib

    bench = importlib.import_module("bench")
    src = tmp_path / "csrc"
    src.mkdir()
    (src / "k.hpp").write_text('// a comment\nint f(int x) { return x + 1; }  /* tail */\nconst char *s = "// not a comment";\n')
    (src / "Makefile").write_text("all:\n\ttrue\n")
    monkeypatch.setattr(bench, "KERNEL_SOURCES", src)
    base = bench.kernel_sources_hash()
    (src / "k.hpp").write_text('// another comment, more of it\n\nint f(int x)\n{\n  return x + 1;\n}\nconst char *s = "// not a comment";\n')
    assert bench.kernel_sources_hash() == base
    (src / "k.hpp").write_text('int f(int x) { return x + 2; }\nconst char *s = "// not a comment";\n')
    assert bench.kernel_sources_hash() != base
    (src / "k.hpp").write_text('int f(int x) { return x + 1; }\nconst char *s = "// not a comment!";\n')
    assert bench.kernel_sources_hash() != base
    # The committed summary carries the stamp of the committed sources.
    monkeypatch.undo()
    rows, source = bench._measured_traffic("C3")
    assert rows.get("fwd") and rows.get("bwd_dkdv") and rows.get("fwd_forward_only"), source
