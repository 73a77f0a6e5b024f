"""The build's check of the kernels' assembly (trueno_amd/csrc/check_asm_loads.py): a register written by a load in an
inline-asm block must not be named by compiler-generated code before the asm-block wait for that load."""
import importlib.util
import os

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
spec = importlib.util.spec_from_file_location("check_asm_loads", os.path.join(ROOT, "trueno_amd", "csrc", "check_asm_loads.py"))
check_asm_loads = importlib.util.module_from_spec(spec)
spec.loader.exec_module(check_asm_loads)

HEAD = "kernel_a:\n\t;;#ASMSTART\n\tglobal_load_dwordx4 v[30:33], v[2:3], off\n\t;;#ASMEND\n"
WAIT = "\t;;#ASMSTART\n\ts_waitcnt vmcnt(5)\n\t;;#ASMEND\n"


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
