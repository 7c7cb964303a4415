"""Register and scratch use of the kernels, read from the compiler's own report (the reference refuses a
kernel that spills, llvq-llm/src/fused_cuda.rs:234-239: local_bytes must be 0).  Cross-compiles for
gfx950 without a GPU."""
import os
import re
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "llvq_amd", "csrc")


@pytest.fixture(scope="module")
def usage(tmp_path_factory):
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(hipcc):
        pytest.skip("hipcc is not installed")
    out = tmp_path_factory.mktemp("res") / "llvq.o"
    cmd = [hipcc, "--offload-arch=gfx950", "-O3", "-std=c++17", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
           "-Rpass-analysis=kernel-resource-usage", "--cuda-device-only", "-c", "-o", str(out), "-x", "hip",
           os.path.join(CSRC, "llvq_hip.hip")]
    run = subprocess.run(cmd, capture_output=True, text=True, timeout=900)
    assert run.returncode == 0, run.stderr[-2000:]
    kernels, name = {}, None
    for line in run.stderr.splitlines():
        m = re.search(r"remark: Function Name: (\S+)", line)
        if m:
            name = m.group(1)
            kernels[name] = {}
            continue
        m = re.search(r"remark:\s+(VGPRs|AGPRs|ScratchSize \[bytes/lane\]|Occupancy \[waves/SIMD\]|LDS Size \[bytes/block\]): (\d+)", line)
        if m and name:
            kernels[name][m.group(1).split(" ")[0]] = int(m.group(2))
    assert kernels, "no resource remarks in the compiler output"
    return kernels


def test_the_gemv_and_decode_kernels_do_not_spill(usage):
    gemv = {k: v for k, v in usage.items() if "gemv_tiles_kernel" in k}
    assert len(gemv) == 12  # 2 output types x (full tile, half tile, lean image) x (natural, rotated basis)
    for name, u in usage.items():
        if "gemm_tiles_kernel" in name or "gemm_pipe_kernel" in name:
            continue
        assert u["ScratchSize"] == 0, f"{name} spills {u['ScratchSize']} bytes per lane"
    for name, u in gemv.items():
        # 1024 lanes per workgroup = 4 wavefronts per SIMD: 128 registers each is the ceiling
        assert u["VGPRs"] + u.get("AGPRs", 0) <= 128, (name, u)


def test_the_batched_kernel_spill_is_the_known_one(usage):
    """32 accumulator registers live across the decode phases at 16 wavefronts per CU: the compiler
    parks some of the decode state in scratch.  Measured alternatives (fewer wavefronts, accumulators
    re-read from LDS) were slower; this pins the amount so that growth is noticed."""
    gemm = {k: v for k, v in usage.items() if "gemm_tiles_kernel" in k}
    assert len(gemm) == 2
    for name, u in gemm.items():
        assert u["ScratchSize"] <= 256, (name, u)
        assert u["VGPRs"] <= 128


def test_the_pipelined_batched_kernel_keeps_its_spill_out_of_the_loops(usage):
    """Producers and consumers are separate branches, so 64 accumulators and the decode state share the
    128 registers; what the compiler still parks in scratch are per-lane constants of the consumers'
    set-up and epilogue (a few dwords), not operands of the matrix-core loop."""
    pipe = {k: v for k, v in usage.items() if "gemm_pipe_kernel" in k}
    assert len(pipe) == 2  # 8 or 12 producer wavefronts
    for name, u in pipe.items():
        assert u["ScratchSize"] <= 64, (name, u)
        assert u["VGPRs"] + u.get("AGPRs", 0) <= 128, (name, u)
