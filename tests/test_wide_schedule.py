"""The schedule of the wide walk kernels' two wave groups (csrc/wide_schedule.hpp) -- which node each group takes
in which step, so that every tile a node needs is in memory, or still in the group's registers, when the node asks
for it -- and the check the library runs on every schedule it builds: compiled with g++ over hand-made and
random trees."""
import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(os.path.dirname(HERE), "lvd-pg_amd", "csrc")


def test_wide_schedule(tmp_path):
    exe = str(tmp_path / "wide_schedule")
    subprocess.run(["g++", "-std=c++17", "-O1", "-Wall", "-Werror", "-I", CSRC, "-o", exe,
                    os.path.join(HERE, "wide_schedule_test.cpp")], check=True)
    out = subprocess.run([exe], check=True, capture_output=True, text=True).stdout
    got = dict((l.split()[0], int(l.split()[1])) for l in out.splitlines())
    assert got["chain_forward_steps"] == 5 and got["chain_backward_steps"] == 5
    assert got["chain_forward_fault"] == -1 and got["chain_backward_fault"] == -1
    assert got["chain_one_group"] == 1
    assert got["two_chains_steps"] <= 5 and got["two_chains_fault"] == -1 and got["two_chains_split"] == 1
    assert got["cross_too_early"] == 2
    assert got["cross_late_enough"] == -1
    assert got["slot_twice"] == 1
    assert got["own_group_two_back"] == -1
    assert got["other_group_two_back"] == 2
    assert got["random_faults"] == 0
    assert got["random_too_long"] == 0
    assert got["random_shorter"] == 1
