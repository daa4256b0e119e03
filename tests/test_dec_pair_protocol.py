"""The counter protocol of the decode pair kernel, checked on the CPU: tests/dec_pair_model.c walks the
kernel's work items over plow_amd/csrc/dec_pair_protocol.h (the very functions the kernel calls) under
random schedules, with waits that give up, over two launches on one scratch."""
import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))


def build_model(tmp_path):
    exe = os.path.join(str(tmp_path), "dec_pair_model")
    subprocess.check_call(["gcc", "-O1", "-Wall", "-Werror", "-o", exe, os.path.join(HERE, "dec_pair_model.c")])
    return exe


def test_protocol_leaves_scratch_zeroed_and_never_runs_early(tmp_path):
    r = subprocess.run([build_model(tmp_path)], capture_output=True, text=True)
    print(r.stdout[-400:])
    assert r.returncode == 0, r.stdout[-2000:]
    assert " 0 failures" in r.stdout


def test_model_sees_the_defect_of_resetting_from_the_last_down_item(tmp_path):
    r = subprocess.run([build_model(tmp_path), "--old-reset"], capture_output=True, text=True)
    assert r.returncode == 1
    assert "touched after reset" in r.stdout or "left at" in r.stdout
