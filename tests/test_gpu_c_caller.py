"""The C ABI called from C: llvq-hip/examples/c_caller.c (built by llvq_amd/csrc/Makefile) makes a small
LLVQ matrix, runs llvq_hip_gemv, llvq_hip_gemm and llvq_hip_gemm_static on it and checks every output
against a loop over the library's host decoder.  No Python, torch or C++ on the calling side: this is
the path a caller in a compiled language (the llvq-hip crate) takes."""
import os
import subprocess

import pytest

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_c_program_runs_the_three_products():
    exe = os.path.join(ROOT, "llvq_amd", "csrc", "c_caller")
    assert os.path.exists(exe), "build it first: python -c 'import __graft_entry__ as g; g.build()'"
    run = subprocess.run([exe], capture_output=True, text=True, timeout=120)
    print(run.stdout)
    assert run.returncode == 0, (run.returncode, run.stdout[-500:], run.stderr[-1000:])
    assert run.stdout.strip().endswith("ok")
