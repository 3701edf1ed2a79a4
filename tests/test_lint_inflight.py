"""The build-time hazard check of the hand-scheduled kernels (csrc/lint_inflight.py), on hand-written
assembly fixtures: it must accept a loop whose staging registers are covered by waits before they are touched, and
reject each of the hazards it exists for -- a register with a load in flight that is copied (the compiler's spill
or move), reused as a load's destination, stored, or used as an address, and an asm instruction that reads a
transcendental result without a wait state.  No GPU, no compiler."""
import importlib.util
import os

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def lint():
    path = os.path.join(ROOT, "ppl.llm.kernel.cuda_amd", "csrc", "lint_inflight.py")
    spec = importlib.util.spec_from_file_location("lint_inflight", path)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def asm_load(dst, addr="v2", base="s[4:5]"):
    return [";;#ASMSTART", "global_load_dwordx4 %s, %s, %s nt" % (dst, addr, base), ";;#ASMEND"]


def asm_wait(n):
    return [";;#ASMSTART", "s_waitcnt vmcnt(%d)" % n, ";;#ASMEND"]


CLEAN = (asm_load("v[10:13]") + asm_load("v[14:17]") + ["v_add_u32 v2, v2, v3", "v_mul_f32 v20, v21, v22"]
         + asm_wait(1) + ["v_perm_b32 v30, v10, v11, s8"]   # the first load has landed, the second has not
         + asm_wait(0) + ["v_perm_b32 v31, v14, v15, s8", "global_store_dwordx2 v2, v[30:31], s[6:7]", "s_endpgm"])


def test_clean_schedule_is_accepted(lint):
    problems, asm_loads, hazards = lint.lint("clean", CLEAN)
    assert (problems, asm_loads, hazards) == (0, 2, 0)


@pytest.mark.parametrize("what,lines", [
    ("copy of a staging register before its wait (what a spill or a register move does)",
     asm_load("v[10:13]") + ["v_mov_b32 v40, v11"] + asm_wait(0)),
    ("staging register written by an ordinary instruction while the load is in flight",
     asm_load("v[10:13]") + ["v_add_f32 v12, v1, v2"] + asm_wait(0)),
    ("wait that covers only the older of two loads",
     asm_load("v[10:13]") + asm_load("v[14:17]") + asm_wait(1) + ["v_perm_b32 v31, v14, v15, s8"]),
    ("second asm load into a register that still has one in flight",
     asm_load("v[10:13]") + asm_load("v[12:15]") + asm_wait(0)),
    ("compiler-scheduled load into a staging register",
     asm_load("v[10:13]") + ["global_load_dword v11, v2, s[4:5]"] + asm_wait(0)),
    ("staging register used as an address",
     asm_load("v[10:13]") + ["global_load_dword v50, v10, s[4:5]"] + asm_wait(0)),
    ("staging register stored before its wait",
     asm_load("v[10:13]") + ["global_store_dword v2, v13, s[6:7]"] + asm_wait(0)),
])
def test_register_hazards_are_rejected(lint, what, lines):
    problems, asm_loads, hazards = lint.lint("hazard", lines + ["s_endpgm"])
    assert asm_loads >= 1 and problems >= 1, what


def test_transcendental_result_read_by_the_next_asm_instruction(lint):
    bad = ["v_exp_f32_e32 v5, v4", ";;#ASMSTART", "v_mul_f32 v6, v5, v7", ";;#ASMEND"]
    assert lint.lint("trans", bad)[2] == 1
    spaced = ["v_exp_f32_e32 v5, v4", "v_add_f32 v9, v8, v8", ";;#ASMSTART", "v_mul_f32 v6, v5, v7", ";;#ASMEND"]
    assert lint.lint("trans", spaced)[2] == 0
    other_reg = ["v_exp_f32_e32 v5, v4", ";;#ASMSTART", "v_mul_f32 v6, v8, v7", ";;#ASMEND"]
    assert lint.lint("trans", other_reg)[2] == 0


def test_the_command_fails_on_a_hazard_and_on_nothing_to_check(lint, tmp_path, monkeypatch, capsys):
    def run(body):
        path = tmp_path / "k.s"
        path.write_text("_Z6kernelv:\n" + "\n".join(body) + "\ns_endpgm\n")
        monkeypatch.setattr("sys.argv", ["lint_inflight.py", str(path)])
        return lint.main()
    assert run(CLEAN[:-1]) == 0
    assert run(asm_load("v[10:13]") + ["v_mov_b32 v40, v11"] + asm_wait(0)) == 1
    assert run(["v_mov_b32 v1, v2"]) == 1  # no hand-scheduled kernel found: the check itself went wrong
    assert "0 hand-scheduled kernels checked" in capsys.readouterr().out
