"""Runs tests/cabi/ft_cabi_check: a C++ program with no Python and no torch in it that calls
libftadam.so through include/ft_adam.h exactly as a foreign-language binding would (plain
pointers, sizes, a hipStream_t) and compares every result bit for bit with the CPU checker.
The program is built beforehand by `make -f tests/cabi/Makefile` (part of __graft_entry__.build)."""
import os
import subprocess

import pytest

pytestmark = pytest.mark.gpu

BINARY = os.path.join(os.path.dirname(os.path.abspath(__file__)), "cabi", "ft_cabi_check")


def test_native_program_through_the_c_abi(cuda):
    assert os.path.exists(BINARY), "tests/cabi/ft_cabi_check is not built: run `make -f tests/cabi/Makefile`"
    run = subprocess.run([BINARY], capture_output=True, text=True, timeout=110)
    print(run.stdout, flush=True)
    print(run.stderr, flush=True)
    assert run.returncode == 0, run.stdout[-2000:] + run.stderr[-2000:]
    assert "ALL PASSED" in run.stdout and "FAIL" not in run.stdout.replace("FAILED", "")
    assert run.stdout.count("\nok  ") + run.stdout.startswith("ok  ") >= 15
