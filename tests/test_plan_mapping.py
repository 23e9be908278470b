"""Every workgroup id of a launch must lead to exactly one block of one tensor.
tests/plan_mapping.cpp links the library's planner and walks the whole grid of
each stage through a host restatement of the kernels' lookup."""

import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)


def test_every_block_is_visited_once(tmp_path):
    exe = str(tmp_path / "plan_mapping")
    subprocess.check_call(["g++", "-O2", "-std=c++17", "-Wall", "-o", exe,
                           os.path.join(HERE, "plan_mapping.cpp"),
                           os.path.join(ROOT, "torchft_amd", "csrc", "tftq_plan.cpp")])
    res = subprocess.run([exe], stdout=subprocess.PIPE, text=True, timeout=300)
    assert res.returncode == 0, res.stdout
    assert res.stdout.startswith("ok ")
