"""Seeded synthetic LLVQ matrices and activations, shared by the benchmark and
the tests so that the CPU checker and the GPU path read identical bytes.

RNG is SplitMix64 as llvq-core/src/rng.rs:21-40 (vectorised: the state of draw
k is seed + k * gamma).  Draw order per matrix follows the reference's own
bench (llvq-cuda/src/bin/matvec.rs:410-418): per block `idx = next() %
(N(12) + 1)` then `gain = next() & 1`; then one gaussian per row scale
(`exp(-4 + 0.3 g)`), then one gaussian per tail value (`0.02 g`, narrowed to
f32).  Gain centroids are {0.8, 1.25}.  An activation is its own stream.
"""
import numpy as np

from .artifact import DIM, N12, N13, RawMatrix, pack_codes

_GAMMA = 0x9E3779B97F4A7C15
_M1 = 0xBF58476D1CE4E5B9
_M2 = 0x94D049BB133111EB
_MASK = (1 << 64) - 1


def fnv1a64(data: bytes) -> int:
    h = 0xCBF29CE484222325
    for b in data:
        h = ((h ^ b) * 0x100000001B3) & _MASK
    return h


class SplitMix64:
    """Counter-based view of rng.rs:21-40: `take(n)` returns the next n outputs."""

    def __init__(self, seed: int):
        self.state = seed & _MASK

    def take(self, n: int) -> np.ndarray:
        n = int(n)
        with np.errstate(over="ignore"):
            k = np.arange(1, n + 1, dtype=np.uint64)
            z = np.uint64(self.state) + k * np.uint64(_GAMMA)
            self.state = (self.state + n * _GAMMA) & _MASK
            z = (z ^ (z >> np.uint64(30))) * np.uint64(_M1)
            z = (z ^ (z >> np.uint64(27))) * np.uint64(_M2)
            return z ^ (z >> np.uint64(31))

    def next(self) -> int:
        return int(self.take(1)[0])

    def gaussian(self, n: int) -> np.ndarray:
        """Box–Muller, cosine branch (rng.rs:35-39): two draws per value."""
        d = self.take(2 * n)
        u1 = ((d[0::2] >> np.uint64(11)).astype(np.float64) + 1.0) * (1.0 / 9007199254740993.0)
        u2 = (d[1::2] >> np.uint64(11)).astype(np.float64) * (1.0 / 9007199254740992.0)
        return np.sqrt(-2.0 * np.log(u1)) * np.cos(2.0 * np.pi * u2)


def matrix_seed(seed: int, name: str) -> int:
    return (seed ^ fnv1a64(name.encode())) & _MASK


def make_matrix(name: str, d_out: int, d_in: int, seed: int = 0, index_bound: int = None,
                centroids=(0.8, 1.25), shell_cap: int = 12) -> RawMatrix:
    """Indices uniform below `index_bound` (default: the whole ball of the cap, origin included)."""
    if index_bound is None:
        index_bound = {12: N12, 13: N13}[shell_cap] + 1
    rng = SplitMix64(matrix_seed(seed, name))
    nb = d_out * (d_in // DIM)
    draws = rng.take(2 * nb)
    idx = draws[0::2] % np.uint64(index_bound)
    gain = draws[1::2] & np.uint64(1)
    row_scales = np.exp(-4.0 + 0.3 * rng.gaussian(d_out))
    tail = (0.02 * rng.gaussian(d_out * (d_in % DIM))).astype(np.float32)
    return RawMatrix(name, d_out, d_in, shell_cap, np.array(centroids, np.float64), row_scales, tail,
                     pack_codes(idx, gain, index_width={12: 47, 13: 48}[shell_cap]))


def make_activation(d_in: int, seed: int = 0, rows: int = 1) -> np.ndarray:
    """N(0,1) narrowed to binary16 (round to nearest even), shape [rows, d_in]."""
    rng = SplitMix64(matrix_seed(seed, f"activation:{d_in}"))
    return rng.gaussian(rows * d_in).astype(np.float16).reshape(rows, d_in)


# BASELINE configurations ----------------------------------------------------------
QWEN3_4B_LAYER = [  # (site, d_out, d_in) — the seven projections of one decoder layer
    ("self_attn.q_proj", 4096, 2560),
    ("self_attn.k_proj", 1024, 2560),
    ("self_attn.v_proj", 1024, 2560),
    ("self_attn.o_proj", 2560, 4096),
    ("mlp.gate_proj", 9728, 2560),
    ("mlp.up_proj", 9728, 2560),
    ("mlp.down_proj", 2560, 9728),
]


def config0(seed: int = 0) -> RawMatrix:
    """Single gate_proj of Qwen3-4B: 9728 x 2560, 106 blocks + 16 tail columns per row."""
    return make_matrix("model.layers.0.mlp.gate_proj.weight", 9728, 2560, seed)


def layer_matrices(layer: int = 0, seed: int = 0, shapes=QWEN3_4B_LAYER):
    return [make_matrix(f"model.layers.{layer}.{site}.weight", do, di, seed) for site, do, di in shapes]
