"""The kernels divide by a row scale with two fused multiply-adds instead of an
IEEE divide.  tests/exact_division.c proves by exhaustion (2.1e9 quotients)
that the result is the correctly rounded quotient for every e4m3 value and
every scale mantissa, so the GPU path can be bit-exact with the checker."""

import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))


def test_fma_division_is_exact(tmp_path):
    exe = str(tmp_path / "exact_division")
    subprocess.check_call(["gcc", "-O2", "-ffp-contract=off", "-o", exe,
                           os.path.join(HERE, "exact_division.c"), "-lm"])
    res = subprocess.run([exe], stdout=subprocess.PIPE, text=True, timeout=600)
    assert res.returncode == 0, res.stdout
    assert " 0 mismatches" in res.stdout


def test_three_operation_quotient_is_exact(tmp_path):
    """Averages over a group whose size is not a power of two divide by it with a
    multiplication and two fused multiply-adds; tests/exact_quotient.c proves by
    exhaustion (4.3e9 quotients) that this is the correctly rounded quotient."""
    exe = str(tmp_path / "exact_quotient")
    subprocess.check_call(["gcc", "-O2", "-fopenmp", "-ffp-contract=off", "-o", exe,
                           os.path.join(HERE, "exact_quotient.c"), "-lm"])
    res = subprocess.run([exe], stdout=subprocess.PIPE, text=True, timeout=900)
    assert res.returncode == 0, res.stdout
    assert " 0 mismatches" in res.stdout
