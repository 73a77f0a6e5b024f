"""The build's check of the kernels' assembly (trueno_amd/csrc/check_asm_loads.py): a register written by a load in an
inline-asm block must not be named by compiler-generated code before the asm-block wait for that load."""
import importlib.util
import os

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
spec = importlib.util.spec_from_file_location("check_asm_loads", os.path.join(ROOT, "trueno_amd", "csrc", "check_asm_loads.py"))
check_asm_loads = importlib.util.module_from_spec(spec)
spec.loader.exec_module(check_asm_loads)

HEAD = "kernel_a:\n\t;;#ASMSTART\n\tglobal_load_dwordx4 v[30:33], v[2:3], off\n\t;;#ASMEND\n"
WAIT = "\t;;#ASMSTART\n\ts_waitcnt vmcnt(0)\n\t;;#ASMEND\n"


def _check(tmp_path, text):
    path = tmp_path / "k.s"
    path.write_text(text)
    return check_asm_loads.check(str(path))


def test_a_copy_before_the_wait_is_reported(tmp_path):
    errors = _check(tmp_path, HEAD + "\tv_mov_b64_e32 v[14:15], v[30:31]\n" + WAIT + "\tv_add_f32 v1, v30, v31\n\ts_endpgm\n")
    assert len(errors) == 1 and "kernel_a" in errors[0] and "v30" in errors[0]


def test_use_after_the_wait_is_fine(tmp_path):
    assert _check(tmp_path, HEAD + "\tv_mov_b32 v1, v2\n" + WAIT + "\tv_add_f32 v1, v30, v31\n\ts_endpgm\n") == []


def test_overwriting_a_register_in_flight_is_reported(tmp_path):
    assert len(_check(tmp_path, HEAD + "\tv_mov_b32 v33, 0\n" + WAIT + "\ts_endpgm\n")) == 1


def test_a_compiler_wait_for_everything_clears_the_loads(tmp_path):
    assert _check(tmp_path, HEAD + "\ts_waitcnt vmcnt(0)\n\tv_mov_b32 v1, v30\n\ts_endpgm\n") == []


def test_copies_into_lds_do_not_count_as_register_loads(tmp_path):
    text = "kernel_b:\n\t;;#ASMSTART\n\tglobal_load_lds_dwordx4 v[4:5], off\n\t;;#ASMEND\n\tv_mov_b32 v1, v4\n\ts_endpgm\n"
    assert _check(tmp_path, text) == []


LOAD2 = "\t;;#ASMSTART\n\tglobal_load_dwordx4 v[40:43], v[2:3], off\n\t;;#ASMEND\n"


def _wait(n):
    return f"\t;;#ASMSTART\n\ts_waitcnt vmcnt({n})\n\t;;#ASMEND\n"


def test_a_partial_wait_leaves_the_newest_loads_in_flight(tmp_path):
    """two loads, then vmcnt(1): the first has landed, the second has not"""
    text = HEAD + LOAD2 + _wait(1) + "\tv_mov_b32 v1, v30\n\tv_mov_b32 v5, v41\n\ts_endpgm\n"
    errors = _check(tmp_path, text)
    assert len(errors) == 1 and "v41" in errors[0]
    assert _check(tmp_path, HEAD + LOAD2 + _wait(0) + "\tv_mov_b32 v1, v30\n\tv_mov_b32 v5, v41\n\ts_endpgm\n") == []


def test_operations_issued_later_count_towards_a_wait(tmp_path):
    """load, two copies into LDS, vmcnt(2): the load is the oldest of three and has landed; with vmcnt(3) it may not have"""
    dma = "\tglobal_load_lds_dwordx4 v[4:5], off\n"
    assert _check(tmp_path, HEAD + dma + dma + _wait(2) + "\tv_mov_b32 v1, v30\n\ts_endpgm\n") == []
    assert len(_check(tmp_path, HEAD + dma + dma + _wait(3) + "\tv_mov_b32 v1, v30\n\ts_endpgm\n")) == 1


def test_a_load_in_flight_is_carried_around_a_loop(tmp_path):
    """the touch stands above the load in the text, but follows it on the loop's back edge"""
    text = ("kernel_c:\n.LBB0_1:\n\tv_mov_b32 v9, v31\n" + HEAD.split("\n", 1)[1] +
            "\ts_cbranch_scc1 .LBB0_1\n" + _wait(0) + "\ts_endpgm\n")
    errors = _check(tmp_path, text)
    assert len(errors) == 1 and "v31" in errors[0]
    # with the wait at the top of the loop body the same touch is fine, and so is a use behind the loop
    ok = ("kernel_d:\n.LBB1_1:\n" + _wait(0) + "\tv_mov_b32 v9, v31\n" + HEAD.split("\n", 1)[1] +
          "\ts_cbranch_scc1 .LBB1_1\n" + _wait(0) + "\tv_mov_b32 v30, 0\n\ts_endpgm\n")
    assert _check(tmp_path, ok) == []


def test_a_use_behind_a_loop_whose_last_rounds_issue_no_load(tmp_path):
    """load under a condition inside the loop, wait at the top of the next round: when the loop is left over the path on
    which no load was issued, the registers are free"""
    text = ("kernel_e:\n.LBB2_1:\n" + _wait(0) + "\ts_cbranch_scc0 .LBB2_3\n" + HEAD.split("\n", 1)[1] +
            "\ts_branch .LBB2_1\n.LBB2_3:\n\tv_add_f32 v30, v1, v2\n\ts_endpgm\n")
    assert _check(tmp_path, text) == []
