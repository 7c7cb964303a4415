"""Pins of the oracle's incoherence rotation (llvq-quant/src/rotation.rs).
The reference holds no numeric vectors for it (a rotation is a pure function of
(n, seed)); its own tests are properties (llvq-quant/tests/g5_rotation.rs), which
are repeated here, plus structure checks against library routines that a wrong
butterfly, a transposed mixing block or a wrong draw order would fail."""
import numpy as np
import scipy.linalg

from llvq_amd import artifact, synth
from llvq_amd.synth import SplitMix64

DIMS = [1, 3, 7, 16, 24, 96, 1024, 2048, 3072]  # g5_rotation.rs:13


def _matrix(rot):
    return np.stack([rot.apply(np.eye(rot.n)[j]) for j in range(rot.n)], axis=1)  # column j = Q e_j


def test_factorisation_and_draw_order(orc):
    """n = m k with m = 2^tz(n); signs are the first n Gaussian draws of the seed; the
    mixing block is the Gram-Schmidt of the next k*k draws, i.e. the Q factor of a QR."""
    for n in (24, 96, 40, 2560):
        seed = 0xABC0 + n
        rot = orc.Rotation(n, seed)
        m = n & -n
        assert (rot.m, rot.k) == (m, n // m)
        g = SplitMix64(seed).gaussian(n + rot.k * rot.k)
        assert np.array_equal(rot.signs, np.where(g[:n] < 0, -1.0, 1.0))
        A = g[n:].reshape(rot.k, rot.k)       # rows are the Gaussian vectors
        Qf, R = np.linalg.qr(A.T)             # Gram-Schmidt on rows = QR of the transpose
        Qf = Qf * np.sign(np.diag(R))          # positive diagonal = classical Gram-Schmidt
        assert np.allclose(rot.small, Qf.T, atol=1e-9)


def test_power_of_two_width_is_signed_hadamard(orc):
    for n in (1, 2, 16, 256):
        rot = orc.Rotation(n, 77)
        want = scipy.linalg.hadamard(n) / np.sqrt(n) * rot.signs[None, :]  # H D / sqrt n
        assert np.allclose(_matrix(rot), want, atol=1e-12)


def test_kronecker_structure(orc):
    """Q = (S kron I_m)(I_k kron H_m / sqrt m) D."""
    for n in (24, 96, 80):
        rot = orc.Rotation(n, 5)
        H = scipy.linalg.hadamard(rot.m) / np.sqrt(rot.m) if rot.m > 1 else np.ones((1, 1))
        want = np.kron(rot.small, np.eye(rot.m)) @ np.kron(np.eye(rot.k), H) @ np.diag(rot.signs)
        assert np.allclose(_matrix(rot), want, atol=1e-12)


def test_orthogonal_on_every_width(orc):  # g5_rotation.rs:16-42
    for n in DIMS:
        rot = orc.Rotation(n, 0x90001 + n)
        cols = np.stack([rot.apply(np.eye(n)[j]) for j in range(min(n, 64))], axis=1)
        assert np.allclose(cols.T @ cols, np.eye(cols.shape[1]), atol=1e-9)


def test_transpose_undoes_the_rotation(orc):  # g5_rotation.rs:45-72
    rng = SplitMix64(0x90002)
    for n in DIMS:
        rot = orc.Rotation(n, 0x90003 + n)
        v0 = rng.gaussian(n)
        assert np.abs(rot.apply_transpose(rot.apply(v0)) - v0).max() < 1e-9
        if n > 1:
            assert np.abs(rot.apply(v0) - v0).max() > 1e-6


def test_rotated_record_decodes_to_the_natural_basis(orc):
    """fused_path_matches_dense.rs: for a record with a rotation seed the dense arm
    (decode_matrix un-rotates) and the fused arm (activation rotated) give the same product."""
    raw = synth.make_matrix("model.layers.0.rot.weight", 8, 24 * 4 + 8, seed=3)
    raw.rotation_seed = 0x51DE
    om, _ = orc.read_matrix_raw(artifact.write_matrix_raw(raw))
    W = om.decode_matrix().astype(np.float64)
    x = SplitMix64(9).gaussian(raw.d_in)
    y_fused, a = om.fused_product(x)
    assert np.abs(W @ x - y_fused).max() < 1e-6 * a.max()
    # and un-rotating really changed the matrix: the stored (rotated) rows differ from W
    raw.rotation_seed = None
    on, _ = orc.read_matrix_raw(artifact.write_matrix_raw(raw))
    Wr = on.decode_matrix().astype(np.float64)
    rot = orc.Rotation(raw.d_in, 0x51DE)
    assert np.allclose(np.stack([rot.apply_transpose(r) for r in Wr]), W, atol=1e-6)
    assert np.abs(Wr - W).max() > 1e-4
