"""The host-side soundness check of the barrier-free walk schedules (csrc/lean_schedule_check.hpp), which the
library runs on every schedule it builds: compiled with g++ into a small program over hand-made schedules.  A
sound schedule lets every wave finish; one in which a wave would wait for a slot state nobody posts is caught,
with the step and wave that wait."""
import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(os.path.dirname(HERE), "lvd-pg_amd", "csrc")


def test_lean_schedule_check(tmp_path):
    exe = str(tmp_path / "lean_check")
    subprocess.run(["g++", "-std=c++17", "-O1", "-Wall", "-Werror", "-I", CSRC, "-o", exe,
                    os.path.join(HERE, "lean_schedule_check_test.cpp")], check=True)
    out = subprocess.run([exe], check=True, capture_output=True, text=True).stdout
    got = dict((l.split()[0], int(l.split()[1])) for l in out.splitlines())
    assert got["forward_chain"] == -1
    assert got["forward_same_step"] == -1
    assert got["forward_reuse"] == -1
    assert got["forward_wrong_turn"] == 1 * 16 + 1        # step 1, wave 1
    assert got["forward_own_future"] == 0 * 16 + 3        # wave 3 never gets past its first step
    assert got["forward_overwrite"] == 1 * 16 + 4         # the second writer waits for a read that never comes
    assert got["backward_tree"] == -1
    assert got["backward_child_first"] == 0 * 16 + 0
