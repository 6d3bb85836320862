"""The GEMM kernels read LDS from inline assembly and wait by hand; this compiles them to assembly
and checks that nothing touches a register before the wait that releases it (isa_wait_lint)."""
import os
import subprocess
import sys

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
import isa_mfma_lint  # noqa: E402
import isa_wait_lint  # noqa: E402

_compiled = {}  # a file is compiled once per session


def _assembly(tmp_path, name):
    if name in _compiled:
        return _compiled[name]
    from frink_amd import build as fb
    out = str(tmp_path / (name + ".s"))
    cmd = [fb.hipcc()] + fb.HIPCC_FLAGS + ["-x", "hip", "--cuda-device-only", "-S", os.path.join(fb.CSRC, name), "-o", out]
    r = subprocess.run(cmd, capture_output=True, text=True)
    assert r.returncode == 0, r.stderr[-2000:]
    _compiled[name] = open(out).read()
    return _compiled[name]


def test_no_use_of_lds_reads_before_their_waits(tmp_path):
    asm = _assembly(tmp_path, "frk_gemm.hip")
    names = isa_wait_lint.kernels(asm)
    assert sum("gemm_q4_k" in k for k in names) >= 3, names  # the two dense forms and the streaming kernel
    for k in names:
        assert isa_wait_lint.violations(asm, k) == [], k
    asm = _assembly(tmp_path, "frk_gemm_q6.hip")
    names = isa_wait_lint.kernels(asm)
    assert sum("gemm_q6_k" in k for k in names) == 2, names
    for k in names:
        assert isa_wait_lint.violations(asm, k) == [], k
    for name in ("frk_gemv_direct.hip", "frk_gemv_fused.hip"):
        asm = _assembly(tmp_path, name)
        names = isa_wait_lint.kernels(asm)
        assert names
        for k in names:
            assert isa_wait_lint.violations(asm, k) == [], k


def test_no_mfma_result_is_read_too_soon_across_a_block_boundary(tmp_path):
    """hipcc counts the wait states between an MFMA and a vector instruction that reads its result within one basic
    block only: a conditional piece of work placed between an MFMA and the shift of its sums once came out with the
    shift three instructions behind the MFMA (the last two registers of the sums read before they were written)."""
    for name in ("frk_gemm.hip", "frk_gemm_q6.hip", "frk_gemm_q8.hip", "frk_thin.hip"):
        asm = _assembly(tmp_path, name)
        assert "v_mfma" in asm, name
        assert isa_mfma_lint.violations(asm) == [], name


def test_mfma_lint_sees_a_reader_behind_a_branch():
    head = ["k:", "\tv_mfma_i32_32x32x32_i8 v[50:65], v[0:3], v[4:7], v[50:65]"]
    reader = ["\tv_lshlrev_b32_e32 v65, 3, v65", "\ts_endpgm"]
    # the compiler's own form within a block: enough wait states in front of the reader
    assert isa_mfma_lint.violations("\n".join(head + ["\ts_nop 15", "\ts_nop 1"] + reader)) == []
    # a skipped piece of work between the two: the reader is reached six wait states behind the MFMA
    branchy = head + ["\ts_cbranch_vccnz .LBB0_2", "\tv_mov_b32_e32 v1, v2", ".LBB0_2:", "\ts_waitcnt lgkmcnt(0)", "\ts_nop 2"] + reader
    got = isa_mfma_lint.violations("\n".join(branchy))
    assert len(got) == 1 and "line 8" in got[0], got
    # the next MFMA of a chain takes the sums as its accumulator: not a reader
    chain = head + [".LBB0_3:", "\tv_mfma_i32_32x32x32_i8 v[50:65], v[8:11], v[12:15], v[50:65]", "\ts_endpgm"]
    assert isa_mfma_lint.violations("\n".join(chain)) == []
    # a register that has been overwritten since is no longer the MFMA's
    over = head + ["\tv_mov_b32_e32 v65, 0", ".LBB0_4:", "\tv_add_u32_e32 v1, v65, v65", "\ts_endpgm"]
    assert [v for v in isa_mfma_lint.violations("\n".join(over)) if "v_add" in v] == []


def test_lint_sees_an_early_copy():
    asm = "\n".join([
        "k:",
        "\tds_read_b128 v[4:7], v1 offset:0",
        "\tds_read_b128 v[8:11], v1 offset:16",
        "\tv_mov_b64_e32 v[20:21], v[4:5]",
        "\ts_waitcnt lgkmcnt(1)",
        "\tv_add_u32_e32 v30, v4, v5",
        "\tv_add_u32_e32 v31, v8, v5",
        "\ts_waitcnt lgkmcnt(0)",
        "\tv_add_u32_e32 v31, v8, v5",
        "\ts_endpgm",
    ])
    got = isa_wait_lint.violations(asm, "k")
    assert len(got) == 2 and "line 4" in got[0] and "line 7" in got[1], got


def test_lint_follows_branches_and_loops():
    # a read that a loop's back edge leaves in flight is seen by the loop head's first instruction;
    # the block behind an unconditional branch is not reached from above
    asm = "\n".join([
        "k:",
        "\tv_mov_b32_e32 v4, 0",
        ".LBB0_1:",
        "\tv_add_u32_e32 v30, v4, v5",
        "\ts_waitcnt lgkmcnt(0)",
        "\tds_read_b128 v[4:7], v1 offset:0",
        "\ts_cbranch_scc1 .LBB0_1",
        "\ts_branch .LBB0_3",
        ".LBB0_2:",
        "\tv_add_u32_e32 v31, v6, v5",
        ".LBB0_3:",
        "\ts_waitcnt lgkmcnt(0)",
        "\tv_add_u32_e32 v31, v7, v5",
        "\ts_endpgm",
        ".Lfunc_end0:",
    ])
    got = isa_wait_lint.violations(asm, "k")
    assert len(got) == 1 and "line 4" in got[0] and "since line 6" in got[0], got


def test_lint_counts_memory_loads_and_loads_into_lds():
    # vmcnt counts a load into LDS like any other; the register load in front of it is released by
    # vmcnt(1), not before
    asm = "\n".join([
        "k:",
        "\tglobal_load_dwordx4 v[4:7], v[2:3], off",
        "\tglobal_load_lds_dwordx4 v1, s[2:3]",
        "\tv_add_u32_e32 v30, v4, v9",
        "\ts_waitcnt vmcnt(1)",
        "\tv_add_u32_e32 v30, v4, v9",
        "\tglobal_store_dword v[2:3], v30, off",
        "\ts_endpgm",
        ".Lfunc_end0:",
    ])
    got = isa_wait_lint.violations(asm, "k")
    assert len(got) == 1 and "line 4" in got[0] and "since line 2" in got[0], got


def test_lint_counts_lds_writes_and_permutes():
    # lgkmcnt(1) behind a read and a write releases the read: the write is the younger operation
    asm = "\n".join([
        "k:",
        "\tds_read_b128 v[4:7], v1 offset:0",
        "\tds_write_b32 v2, v3",
        "\ts_waitcnt lgkmcnt(1)",
        "\tv_add_u32_e32 v30, v4, v9",
        "\tds_read_b128 v[4:7], v1 offset:0",
        "\tds_bpermute_b32 v8, v2, v3",
        "\ts_waitcnt lgkmcnt(1)",
        "\tv_add_u32_e32 v30, v4, v8",
        "\ts_endpgm",
        ".Lfunc_end0:",
    ])
    got = isa_wait_lint.violations(asm, "k")
    assert len(got) == 1 and "line 9" in got[0] and "reads v8" in got[0], got
