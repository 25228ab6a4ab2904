"""The build check for the scalar-operand rule of inline-assembly memory instructions (tilegym_amd/csrc/check_hazards.py):
the checker on hand-written snippets, then on the assembly of every kernel source with inline-assembly loads."""
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


@pytest.mark.skipif(shutil.which("hipcc") is None and not os.path.exists("/opt/rocm/bin/hipcc"), reason="needs hipcc")
def test_no_kernel_reads_a_scalar_operand_too_early():
    run = subprocess.run([sys.executable, os.path.join(CSRC, "check_hazards.py"), "--build"], capture_output=True, text=True,
                         timeout=900)
    assert run.returncode == 0, run.stdout[-4000:] + run.stderr[-2000:]
    assert "0 finding(s)" in run.stdout
