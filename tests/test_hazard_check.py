"""The build check for what the compiler cannot see inside inline-assembly memory instructions
(tilegym_amd/csrc/check_hazards.py): wait states behind a vector write of a scalar operand, and no use of a load's
destination before a vmcnt wait.  The checker on hand-written snippets, then on the assembly of every kernel source
with inline-assembly loads."""
import importlib.util
import os
import shutil
import subprocess
import sys

import pytest

CSRC = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "tilegym_amd", "csrc")
spec = importlib.util.spec_from_file_location("check_hazards", os.path.join(CSRC, "check_hazards.py"))
check_hazards = importlib.util.module_from_spec(spec)
spec.loader.exec_module(check_hazards)

KERNEL = "kern:\n{body}\n\ts_endpgm\n"


def _scan(tmp_path, body):
    path = tmp_path / "k.s"
    path.write_text(KERNEL.format(body=body))
    return check_hazards.scan(str(path))


def test_adjacent_vector_write_of_a_scalar_offset_is_found(tmp_path):
    found = _scan(tmp_path, "\tv_readfirstlane_b32 s18, v51\n\tbuffer_load_dword v204, v226, s[52:55], s18 offen")
    assert len(found) == 1 and "after 0 wait states" in found[0]


def test_descriptor_registers_count_as_operands(tmp_path):
    body = "\tv_readlane_b32 s53, v255, 3\n\ts_mov_b32 m0, s4\n\ts_nop 0\n\tbuffer_load_dwordx4 v1, s[52:55], s7 offen lds"
    assert len(_scan(tmp_path, body)) == 1


def test_five_wait_states_clear_it(tmp_path):
    body = "\tv_readfirstlane_b32 s18, v51\n\ts_mov_b32 m0, s4\n\ts_nop 3\n\tbuffer_load_dwordx4 v1, s[52:55], s18 offen lds"
    assert _scan(tmp_path, body) == []
    body = "\tv_readfirstlane_b32 s18, v51\n\ts_mov_b32 m0, s4\n\ts_nop 2\n\tbuffer_load_dwordx4 v1, s[52:55], s18 offen lds"
    assert len(_scan(tmp_path, body)) == 1


def test_a_write_in_front_of_a_branch_reaches_the_target(tmp_path):
    body = ("\tv_cmp_lt_i32_e64 s[18:19], v1, v2\n\ts_cbranch_scc1 .LBB0_2\n\ts_nop 7\n.LBB0_2:\n"
            "\tbuffer_load_dword v3, v4, s[52:55], s18 offen")
    found = _scan(tmp_path, body)
    assert len(found) == 1 and "after 1 wait states" in found[0]


def test_scalar_arithmetic_is_no_finding(tmp_path):
    assert _scan(tmp_path, "\ts_lshl_b32 s18, s58, 2\n\tbuffer_load_dword v199, v58, s[48:51], s18 offen") == []


def _early(tmp_path, body):
    path = tmp_path / "k.s"
    path.write_text(KERNEL.format(body=body))
    return check_hazards.scan_early_use(str(path))


def test_a_copy_of_a_register_that_a_load_is_still_filling_is_found(tmp_path):
    body = "\tbuffer_load_dword v204, v226, s[52:55], s18 offen\n\tv_mov_b32_e32 v10, v204\n\ts_waitcnt vmcnt(0)"
    assert len(_early(tmp_path, body)) == 1
    # also an overwrite, and a use inside a register range
    body = "\tbuffer_load_dword v47, v226, s[52:55], s18 offen\n\tv_mfma_f32_16x16x128_f8f6f4 v[44:47], v[32:39], v[16:23], 0"
    assert len(_early(tmp_path, body)) == 1


def test_a_vmcnt_wait_on_every_path_clears_it(tmp_path):
    body = ("\tbuffer_load_dword v204, v226, s[52:55], s18 offen\n\ts_cbranch_scc1 .LBB0_2\n\ts_waitcnt vmcnt(3)\n"
            "\tv_mov_b32_e32 v10, v204\n.LBB0_2:\n\ts_waitcnt vmcnt(0) lgkmcnt(0)\n\tv_mov_b32_e32 v11, v204")
    assert _early(tmp_path, body) == []
    # a wait on lgkmcnt alone is none, and one branch without a wait is enough for a finding
    body = ("\tbuffer_load_dword v204, v226, s[52:55], s18 offen\n\ts_cbranch_scc1 .LBB0_2\n\ts_waitcnt vmcnt(3)\n"
            "\tv_mov_b32_e32 v10, v204\n.LBB0_2:\n\ts_waitcnt lgkmcnt(0)\n\tv_mov_b32_e32 v11, v204")
    assert len(_early(tmp_path, body)) == 1


def test_loads_into_lds_have_no_destination_register(tmp_path):
    assert _early(tmp_path, "\tbuffer_load_dwordx4 v1, s[52:55], s18 offen lds\n\tv_mov_b32_e32 v2, v1") == []


def test_spilled_registers_above_the_recorded_count_are_found(tmp_path):
    path = tmp_path / "k.s"
    meta = "    .name:           _ZN2tg23fp8_gemm_tile256_kernelENS_10GemmParamsE\n    .vgpr_spill_count: {n}\n"
    path.write_text(meta.format(n=3))
    assert len(check_hazards.scan_spills(str(path))) == 1
    path.write_text(meta.format(n=0))
    assert check_hazards.scan_spills(str(path)) == []


@pytest.mark.skipif(shutil.which("hipcc") is None and not os.path.exists("/opt/rocm/bin/hipcc"), reason="needs hipcc")
def test_no_kernel_breaks_either_rule():
    run = subprocess.run([sys.executable, os.path.join(CSRC, "check_hazards.py"), "--build"], capture_output=True, text=True,
                         timeout=900)
    assert run.returncode == 0, run.stdout[-4000:] + run.stderr[-2000:]
    assert "0 finding(s)" in run.stdout
