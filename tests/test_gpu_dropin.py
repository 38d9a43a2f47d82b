"""A C program with ordinary host buffers, linked against the library like an SKL caller would be
(tests/c/dropin.c, built by tests/c/Makefile from __graft_entry__.build()): int8 GEMM with the fused
epilogue, panel pack / unpack and the fp8 conversion checked inside the program against plain loops."""
import os
import subprocess

import pytest

pytestmark = pytest.mark.gpu

HERE = os.path.dirname(os.path.abspath(__file__))


def test_c_caller_with_host_buffers(gpu):
    exe = os.path.join(HERE, "c", "dropin")
    if not os.path.exists(exe):
        pytest.fail("tests/c/dropin is not built: run __graft_entry__.build() (or make -C tests/c)")
    proc = subprocess.run([exe], capture_output=True, text=True, timeout=100)
    assert proc.returncode == 0 and "dropin ok" in proc.stdout, (proc.returncode, proc.stdout[-500:], proc.stderr[-2000:])
