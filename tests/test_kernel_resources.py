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


def test_no_kernel_spills(usage):
    gemv = {k: v for k, v in usage.items() if "gemv_tiles_kernel" in k}
    # 2 output types x ((full tile, half tile, lean image) x (natural, rotated basis) + cap-13 stream x (whole, lean image))
    assert len(gemv) == 16
    seq = {k: v for k, v in usage.items() if "gemv_seq_kernel" in k}
    assert len(seq) == 10  # (full tile, lean image, half tile; full and lean again for the dense 49-bit blocks) x (two, three activation planes)
    gemv.update(seq)
    for name, u in usage.items():
        assert u["ScratchSize"] == 0, f"{name} spills {u['ScratchSize']} bytes per lane"
    for name, u in gemv.items():
        # 1024 lanes per workgroup = 4 wavefronts per SIMD: 128 registers each is the ceiling
        assert u["VGPRs"] + u.get("AGPRs", 0) <= 128, (name, u)


def test_the_batched_kernel_does_not_spill_either(usage):
    """Producers and consumers are separate branches of gemm_tiles_kernel, so the consumers' 64
    accumulators and the producers' decode state share the 128 registers instead of adding up."""
    gemm = {k: v for k, v in usage.items() if "gemm_tiles_kernel" in k}
    assert len(gemm) == 2  # 8 or 12 producer wavefronts
    for name, u in gemm.items():
        assert u["ScratchSize"] == 0, (name, u)
        assert u["VGPRs"] + u.get("AGPRs", 0) <= 128, (name, u)
