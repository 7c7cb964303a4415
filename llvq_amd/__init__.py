"""llvq_amd — MI355X-native fused Leech-lattice dequant-GEMV/GEMM behind LLVQ's
quantized-linear operator API.  The compute path is libllvq_hip.so (HIP, gfx950);
this package is the host-side mirror of the reference interface plus the
synthetic-input generator the benchmark and the tests share."""
from . import artifact, synth  # noqa: F401
from ._ffi import LlvqError, lib_path  # noqa: F401
from .fused import FusedMatrix, FusedModel, FusedProj, FusedRuntime, load  # noqa: F401
