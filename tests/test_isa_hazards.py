"""The hazard check over the compiled kernels (mixed_gemv_amd/isa_lint.py): that it sees each
hazard it is there for, on small hand-written listings, and that the library that was built
passed it.  The dot products of the VALU kernel are inline assembly the compiler cannot pad, so
this is what stands between a register copy placed by the register allocator and silently lost
partial sums."""
import json
import os

import pytest

from mixed_gemv_amd import build as lib_build
from mixed_gemv_amd import isa_lint

HEAD = "kernel_a:\n"
DOT = "\tv_dot2c_f32_f16_dpp v5, v1, v9 row_newbcast:3 row_mask:0xf bank_mask:0xf\n"


def findings(tmp_path, body):
    path = tmp_path / "k.s"
    path.write_text(HEAD + body + "\ts_endpgm\n")
    report = isa_lint.lint_file(str(path))
    return [f["rule"] for f in report["findings"]], report


def test_clean_chain_passes(tmp_path):
    body = ("\tbuffer_load_dwordx4 v[0:3], v20, s[4:7], 0 offen\n\ts_waitcnt vmcnt(0)\n"
            "\tv_and_b32_e32 v9, s3, v30\n\tv_pk_fma_f16 v9, v9, v31, v32\n\tv_pk_add_f16 v10, v9, v33\n"
            + DOT + "\tv_dot2c_f32_f16_dpp v5, v2, v10 row_newbcast:3 row_mask:0xf bank_mask:0xf\n"
            "\ts_nop 4\n\tv_add_f32_e32 v6, v5, v7\n")
    rules, report = findings(tmp_path, body)
    assert rules == [] and report["dot_instructions"] == 2 and report["kernels_with_dots"] == 1


def test_register_copy_in_the_middle_of_a_chain_is_found(tmp_path):
    # what a live-range split looks like: the accumulator moves to another register between two dots
    body = DOT + "\tv_mov_b32_e32 v40, v5\n\tv_dot2c_f32_f16_dpp v40, v2, v10 row_newbcast:4 row_mask:0xf bank_mask:0xf\n\ts_nop 4\n"
    rules, _ = findings(tmp_path, body)
    assert "dot-result-read-too-early" in rules


@pytest.mark.parametrize("gap,bad", [(0, True), (2, True), (3, False)])
def test_dot_result_needs_three_wait_states_before_any_other_reader(tmp_path, gap, bad):
    filler = "".join(f"\tv_mov_b32_e32 v{50 + i}, v60\n" for i in range(gap))
    rules, _ = findings(tmp_path, DOT + filler + "\tds_write_b32 v70, v5\n")
    assert ("dot-result-read-too-early" in rules) == bad
    rules, _ = findings(tmp_path, DOT + (f"\ts_nop {gap - 1}\n" if gap else "") + "\tv_add_f32_e32 v6, v5, v7\n")
    assert ("dot-result-read-too-early" in rules) == bad


def test_dot_result_as_multiplicand_or_overwritten(tmp_path):
    rules, _ = findings(tmp_path, DOT + "\tv_dot2c_f32_f16_dpp v8, v2, v5 row_newbcast:1 row_mask:0xf bank_mask:0xf\n\ts_nop 4\n")
    assert "dot-result-as-multiplicand" in rules
    rules, _ = findings(tmp_path, DOT + "\tv_mov_b32_e32 v5, 0\n")
    assert "dot-result-overwritten-too-early" in rules
    rules, _ = findings(tmp_path, DOT + "\tv_mov_b32_e32 v50, v60\n\tv_mov_b32_e32 v51, v60\n\tv_mov_b32_e32 v5, 0\n")
    assert rules == []


@pytest.mark.parametrize("gap,bad", [(0, True), (1, True), (2, False)])
def test_valu_write_then_dpp_read(tmp_path, gap, bad):
    filler = "".join(f"\tv_mov_b32_e32 v{50 + i}, v60\n" for i in range(gap))
    rules, _ = findings(tmp_path, "\tv_mov_b32_e32 v1, v44\n" + filler + DOT + "\ts_nop 4\n")
    assert ("valu-write-then-dpp-read" in rules) == bad
    # a load into the register is not a VALU write: the wait for its data is the compiler's business
    rules, _ = findings(tmp_path, "\tbuffer_load_dwordx4 v[0:3], v20, s[4:7], 0 offen\n\ts_waitcnt vmcnt(0)\n" + DOT + "\ts_nop 4\n")
    assert rules == []


def test_hazards_across_a_branch_are_followed(tmp_path):
    body = (DOT + "\ts_cbranch_scc1 .LBB0_2\n.LBB0_1:\n\ts_nop 4\n\tv_add_f32_e32 v6, v5, v7\n\ts_branch .LBB0_3\n"
            ".LBB0_2:\n\tv_mov_b32_e32 v41, v5\n.LBB0_3:\n")
    rules, _ = findings(tmp_path, body)
    assert rules == ["dot-result-read-too-early"]      # only the taken branch reads too early
    body = ("\tv_mov_b32_e32 v1, v44\n\ts_branch .LBB0_5\n.LBB0_4:\n\ts_nop 0\n.LBB0_5:\n" + DOT + "\ts_nop 4\n")
    rules, _ = findings(tmp_path, body)
    assert "valu-write-then-dpp-read" in rules          # the writer sits in the predecessor block


def test_the_built_library_passed_the_check():
    """A library built by mixed_gemv_amd.build leaves its objects beside it; then the report of the
    check must be there too, and clean.  (The report is a build product: a tree that holds only the
    library, as on a box that received it built, has neither objects nor report.)"""
    built_here = os.path.isdir(lib_build.OBJ_DIR) and any(f.endswith(".o") for f in os.listdir(lib_build.OBJ_DIR))
    if not os.path.exists(lib_build.LINT_REPORT):
        assert not built_here, "the library was built in this tree but the hazard check left no report"
        pytest.skip("no build products in this tree (the library arrived built)")
    reports = json.load(open(lib_build.LINT_REPORT))
    assert sum(r["dot_instructions"] for r in reports) >= lib_build.MIN_DOT_INSTRUCTIONS, "the check must have seen the VALU kernels"
    assert [f for r in reports for f in r["findings"]] == []


def test_a_check_that_sees_nothing_fails(tmp_path, monkeypatch):
    monkeypatch.setattr(lib_build, "OBJ_DIR", str(tmp_path))
    monkeypatch.setattr(lib_build, "LINT_REPORT", str(tmp_path / "isa_lint.json"))
    with pytest.raises(RuntimeError, match="no device assembly"):
        lib_build.lint_device_code(verbose=False)
    (tmp_path / "empty-hip-amdgcn-amd-amdhsa-gfx950.s").write_text("kernel_a:\n\ts_endpgm\n")
    with pytest.raises(RuntimeError, match="did not see the kernels"):
        lib_build.lint_device_code(verbose=False)
