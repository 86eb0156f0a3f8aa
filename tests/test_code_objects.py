"""What the compiler made of the kernels, read from the metadata of the code objects inside
libfa2_gfx950.so (no GPU needed): register and LDS use per kernel must leave room for the workgroups
per CU the gfx950 table states, and the LDS-direct kernels must not spill vector registers (a spill
inside a tile loop shares the vmcnt counter with the tile loads and stalls on them)."""

from __future__ import annotations

import pathlib
import re
import shutil
import subprocess

import pytest

LLVM = pathlib.Path("/opt/rocm/llvm/bin")
TOOLS = [LLVM / "llvm-objcopy", LLVM / "clang-offload-bundler", LLVM / "llvm-readelf"]
LDS_PER_CU = 160 * 1024
REGS_PER_LANE = 512  # VGPRs + accumulation registers per SIMD lane, shared by the waves on the SIMD

# No LDS-direct kernel may spill.  (The forward at 256 columns is instantiated in its padded form only:
# with the column count a compile-time 256 the compiler spilled about forty registers.)
KNOWN_SPILLS: dict = {}


def _kernel_records(library: pathlib.Path, tmp: pathlib.Path) -> list[dict]:
    fat = tmp / "fat.bin"
    subprocess.run([str(TOOLS[0]), "-O", "binary", "--only-section=.hip_fatbin", str(library), str(fat)], check=True)
    data = fat.read_bytes()
    starts = [m.start() for m in re.finditer(re.escape(b"__CLANG_OFFLOAD_BUNDLE__"), data)]
    assert starts, "no offload bundle in the library"
    records = []
    for i, s in enumerate(starts):
        e = starts[i + 1] if i + 1 < len(starts) else len(data)
        bundle, obj = tmp / f"bundle{i}.bin", tmp / f"code{i}.o"
        bundle.write_bytes(data[s:e])
        subprocess.run([str(TOOLS[1]), "--unbundle", "--type=o", f"--input={bundle}",
                        "--targets=hipv4-amdgcn-amd-amdhsa--gfx950", f"--output={obj}"], check=True)
        notes = subprocess.run([str(TOOLS[2]), "--notes", str(obj)], check=True, capture_output=True, text=True).stdout
        cur: dict = {}
        for line in notes.splitlines():
            m = re.match(r"\s*-?\s*\.(\w+):\s*(.*)", line)
            if not m:
                continue
            key, value = m.groups()
            if key == "agpr_count" and "name" in cur:  # keys are sorted: .agpr_count opens a kernel's record
                records.append(cur)
                cur = {}
            cur[key] = value.strip("'")
        if "name" in cur:
            records.append(cur)
    return records


def _parse(name: str):
    """(kernel, padded head dimension, padded variant?) from a mangled fa2 kernel name."""
    m = re.match(r"_ZN3fa2\d+(\w+?)I(?:DF16b|DF16_)Li(\d+)E((?:Li\d+E|Lb[01]E)*)", name)
    if not m:
        return None
    kernel, dp, rest = m.group(1), int(m.group(2)), m.group(3)
    flags = re.findall(r"Lb([01])E", rest)
    # fwd_direct<T, DP, BKV, PAD>; bwd_dq_direct<T, DP, BKV, FUSE_DELTA, PAD>; bwd_dkdv_direct<T, DP, BQ, PAD, ATOMIC>
    pad = {"fwd_direct_kernel": lambda f: f[0], "bwd_dq_direct_kernel": lambda f: f[1],
           "bwd_dkdv_direct_kernel": lambda f: f[0]}.get(kernel, lambda f: "0")(flags) == "1" if flags else False
    atomic = kernel == "bwd_dkdv_direct_kernel" and len(flags) > 1 and flags[1] == "1"
    return kernel, dp, pad, atomic


@pytest.fixture(scope="module")
def records(tmp_path_factory):
    import importlib

    capi = importlib.import_module("flash-attention-triton_amd._capi")
    if not capi.LIBRARY_PATH.exists():
        pytest.skip("library not built")
    if not all(t.exists() for t in TOOLS) or shutil.which("python3") is None:
        pytest.skip("ROCm LLVM tools not installed")
    return _kernel_records(capi.LIBRARY_PATH, tmp_path_factory.mktemp("code_objects"))


def test_every_kernel_fits_a_cu(records):
    assert len(records) > 50
    for r in records:
        assert int(r["group_segment_fixed_size"]) <= LDS_PER_CU, r["name"]
        assert int(r["vgpr_count"]) <= REGS_PER_LANE, r["name"]
        assert int(r["max_flat_workgroup_size"]) in (64, 256), r["name"]


def test_lds_direct_kernels_do_not_spill(records):
    seen = set()
    for r in records:
        parsed = _parse(r["name"])
        if not parsed or not parsed[0].endswith("_direct_kernel"):
            continue
        kernel, dp, pad, _ = parsed
        seen.add((kernel, dp))
        allowed = KNOWN_SPILLS.get((kernel, dp, pad), 0)
        assert int(r["vgpr_spill_count"]) <= allowed, f"{r['name']}: {r['vgpr_spill_count']} vector registers spilled"
    for dp in (32, 64, 96, 128):
        assert {("fwd_direct_kernel", dp), ("bwd_dq_direct_kernel", dp), ("bwd_dkdv_direct_kernel", dp)} <= seen
    for dp in (192, 256):
        assert {("fwd_direct_kernel", dp), ("bwd_dq_direct_kernel", dp)} <= seen


def test_registers_and_lds_leave_room_for_the_tables_workgroups(records):
    import importlib

    capi = importlib.import_module("flash-attention-triton_amd._capi")
    rows = {r["headdim_padded"]: r for r in capi.config_table() if not r["dq_atomic"] and not r["fwd_exp_folded"]}
    column = {"fwd_direct_kernel": "fwd_wg_per_cu", "bwd_dq_direct_kernel": "dq_wg_per_cu",
              "bwd_dkdv_direct_kernel": "dkdv_wg_per_cu"}
    checked = 0
    for r in records:
        parsed = _parse(r["name"])
        if not parsed or parsed[0] not in column or parsed[3]:
            continue
        kernel, dp, _, _ = parsed
        if kernel == "bwd_dkdv_direct_kernel" and dp > 128:
            continue
        regs = (int(r["vgpr_count"]) + 7) // 8 * 8  # the count includes the accumulation registers
        by_registers = min(8, REGS_PER_LANE // regs)  # waves per SIMD = workgroups per CU (4 waves, one per SIMD)
        by_lds = LDS_PER_CU // int(r["group_segment_fixed_size"])
        want = rows[dp][column[kernel]]
        assert min(by_registers, by_lds) >= want, (r["name"], by_registers, by_lds, want)
        checked += 1
    assert checked >= 3 * 4 * 2


# Two places in the kernels rest on facts about the compiler that no language rule guarantees: the
# score chains of the dK/dV kernel are inline-assembly MFMAs whose results are made safe to read with
# a hand-counted `s_nop 11` (the compiler's hazard recogniser does not see them), and the LDS-direct
# loads write M0 from inline assembly without naming it as a clobber (the backend never keeps a value
# in M0 across other code).  Both were validated, by reading the generated code and by the GPU parity
# tests, with the compiler release named here; with another release they have to be looked at again
# before this line is changed.
VALIDATED_COMPILER = "roc-7.2.0"


def test_hand_scheduled_code_was_validated_with_this_compiler():
    hipcc = pathlib.Path("/opt/rocm/bin/hipcc")
    if not hipcc.exists():
        pytest.skip("no hipcc here")
    out = subprocess.run([str(hipcc), "--version"], check=True, capture_output=True, text=True).stdout
    assert VALIDATED_COMPILER in out, (
        f"the kernels' hand-counted wait states (fa2_bwd_dkdv.hpp: VgprMfma, settle) and the unnamed M0 write "
        f"(fa2_common.hpp: load_lds_16) were validated with {VALIDATED_COMPILER}; this compiler reports:\n{out}")


def test_hand_counted_wait_states_are_in_the_code(records, tmp_path):
    """The dK/dV kernel's inline-assembly MFMA chains must still be followed by their `s_nop 11`
    before the first vector instruction reads them: one per chain and 32-row block in the source."""
    src = (pathlib.Path(__file__).resolve().parent.parent / "flash-attention-triton_amd" / "csrc" /
           "fa2_bwd_dkdv.hpp").read_text()
    assert src.count('asm volatile("s_nop 11" : "+v"(d))') == 1
    assert src.count("settle(s)") == 1 and src.count("settle(dp)") == 1
