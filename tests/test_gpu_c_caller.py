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
    csrc = os.path.join(ROOT, "llvq_amd", "csrc")
    exe = os.path.join(csrc, "c_caller")
    if not os.path.exists(exe):  # normally built beside the library by __graft_entry__.build(); a one-second gcc run otherwise
        made = subprocess.run(["make", "-C", csrc, "c_caller", "-o", "libllvq_hip.so"], capture_output=True, text=True, timeout=120)
        assert made.returncode == 0, made.stderr[-1000:]
    run = subprocess.run([exe], capture_output=True, text=True, timeout=120)
    print(run.stdout)
    assert run.returncode == 0, (run.returncode, run.stdout[-500:], run.stderr[-1000:])
    assert run.stdout.strip().endswith("ok")
