"""Parity of the batched matrix-core path (llvq_hip_gemm, M >= 2) against the
CPU oracle: Y = X W^T with W the oracle's decoded matrix, in f64.

Bar: |y - y_ref| / sum|w_i x_i| < 1e-3.  Weights enter the matrix cores as
binary16 (one rounding of value * centroid / sqrt(16 shell), 2^-11 relative per
weight), accumulation is f32; row scale and tail columns are applied in f32.
That rounding is of the order of 1e-4 of sum|w_i x_i|, so the plain relative
error of an output is below 1e-3 only where the sum does not cancel
(|y_ref| >= 0.2 sum|w_i x_i|); both are asserted.
"""
import numpy as np
import pytest

from llvq_amd import artifact, synth

pytestmark = pytest.mark.gpu

TOL = 1e-3


def _x16(x):
    import torch

    return torch.from_numpy(x.view(np.int16).copy()).view(torch.float16).cuda()


def _reference(orc, raw, X):
    om, _ = orc.read_matrix_raw(artifact.write_matrix_raw(raw))
    W = om.decode_matrix().astype(np.float64)  # [d_out, d_in], tail columns included
    X = X.astype(np.float64)
    return X @ W.T, np.abs(X) @ np.abs(W).T


def _check(Y, Y_ref, A_ref, tol=TOL, out_rounding=0.0):
    """out_rounding: half an ulp of the output type (2^-11 for binary16 outputs), which the result
    carries on top of the 1e-3 the computation is allowed."""
    Y = Y.astype(np.float64)
    e = np.abs(Y - Y_ref) / np.maximum(A_ref, 1e-30)
    assert e.max() < tol, f"max |dy|/sum|wx| = {e.max():.3e}"
    big = np.abs(Y_ref) >= 0.2 * A_ref
    if big.any():
        rel = (np.abs(Y - Y_ref)[big] / np.abs(Y_ref)[big]).max()
        assert rel < tol + out_rounding, f"max relative error {rel:.3e}"
    return e.max()


# d_in must keep activation rows 16-byte aligned (d_in % 8 == 0) for the matrix-core path
CASES = [
    # d_out, d_in, M.  A K-slice is 16 blocks per row; up to 256 activation rows four wavefronts
    # multiply (64-row tiles, the wavefronts left over share a tile's K-steps), beyond that eight.
    (64, 480, 16),      # one band, one full and one short K-slice, no tail
    (72, 184, 16),      # ragged band (72 = 64 + 8), 7 blocks + 16 tail columns
    (8, 2560, 2),       # tiny band, smallest batch
    (128, 2568, 17),    # ragged batch, tail
    (256, 4096, 64),    # 8B hidden size: 170 blocks + 16 tail
    (64, 384, 65),      # exactly one slice; two 64-row tiles, the second with one row
    (192, 976, 130),    # three tiles on four multiplying wavefronts: one of them idles
    (64, 416, 129),     # 17 blocks: a full slice and a slice of one block
    (64, 1000, 256),    # the widest batch of the four-wavefront variant
    (64, 376, 257),     # the narrowest of the eight-wavefront variant: 15 blocks, five tiles
    (320, 800, 300),    # 33 blocks = two full slices and one block; five tiles, three wavefronts idle
    (19000, 80, 257),   # 297 bands on 256 CUs: workgroups walk several units, short slices throughout
    (128, 4096, 512),   # eight tiles
    (64, 376, 511),
    (64, 488, 600),     # more rows than one launch holds
]


@pytest.mark.parametrize("d_out,d_in,M", CASES)
def test_gemm_shapes(gpu_rt, orc, d_out, d_in, M):
    import torch

    raw = synth.make_matrix(f"model.layers.0.gemm.{d_out}x{d_in}.weight", d_out, d_in, seed=7 * d_out + d_in)
    X = synth.make_activation(d_in, seed=M, rows=M)
    Y_ref, A_ref = _reference(orc, raw, X)
    proj = gpu_rt.upload(raw)
    try:
        Y32 = gpu_rt.forward_batched(proj, _x16(X), out_dtype=torch.float32).cpu().numpy()
        Y16 = gpu_rt.forward_batched(proj, _x16(X)).cpu().numpy()
        again = gpu_rt.forward_batched(proj, _x16(X), out_dtype=torch.float32).cpu().numpy()
    finally:
        gpu_rt.free(proj)
    e = _check(Y32, Y_ref, A_ref)
    assert e < 3e-4  # the binary16 weight rounding: 2^-11 = 4.9e-4 bounds a single term, sums of many stay near 1e-4
    _check(Y16.astype(np.float32), Y_ref, A_ref, out_rounding=2.0 ** -11)
    assert np.array_equal(Y32, again)  # fixed summation order, split or not


def test_gemm_origin_shell13_and_generic_blocks(gpu_rt, orc, boundary_indices):
    """Origins, shell-13 indices above N(12) and the class boundaries (which
    include every class that takes the generic walk)."""
    import torch

    d_out, nb, tw = 64, 40, 8
    d_in = 24 * nb + tw
    rng = synth.SplitMix64(2024)
    idx = rng.take(d_out * nb) % np.uint64(1 << 47)
    b = boundary_indices[boundary_indices < (1 << 47)]
    idx[: b.size] = b[: idx.size]
    idx[::5] = 0
    idx[1::11] = np.uint64((1 << 47) - 1)
    gains = (rng.take(idx.size) & np.uint64(1)).astype(np.uint8)
    raw = artifact.RawMatrix("model.layers.0.edge.weight", d_out, d_in, 12, [0.8, 1.25],
                             np.exp(rng.gaussian(d_out)), rng.gaussian(d_out * tw).astype(np.float32),
                             artifact.pack_codes(idx, gains))
    X = synth.make_activation(d_in, seed=77, rows=32)
    Y_ref, A_ref = _reference(orc, raw, X)
    proj = gpu_rt.upload(raw)
    Y = gpu_rt.forward_batched(proj, _x16(X), out_dtype=torch.float32).cpu().numpy()
    gpu_rt.free(proj)
    _check(Y, Y_ref, A_ref)


def test_gemm_degenerate_batches(gpu_rt, orc):
    """One row takes the GEMV; no rows is a no-op that leaves the output alone; a matrix with no whole
    block (tail columns only) goes row by row."""
    import torch

    raw = synth.make_matrix("model.layers.0.degenerate.weight", 24, 488, seed=3)
    X = synth.make_activation(488, seed=4, rows=3)
    proj = gpu_rt.upload(raw)
    tiny = synth.make_matrix("model.layers.0.tailonly.weight", 8, 16, seed=5)
    ptiny = gpu_rt.upload(tiny)
    try:
        xs = torch.from_numpy(X.view(np.int16).copy()).view(torch.float16).cuda()
        one = gpu_rt.forward_batched(proj, xs[:1], out_dtype=torch.float32).cpu().numpy()
        three = gpu_rt.forward_batched(proj, xs, out_dtype=torch.float32).cpu().numpy()
        assert np.abs(one[0] - three[0]).max() <= 2e-3 * np.abs(three[0]).max()  # GEMV (exact weights) vs matrix cores (binary16 weights)
        none = gpu_rt.forward_batched(proj, xs[:0], out_dtype=torch.float32)
        assert tuple(none.shape) == (0, 24)
        Xt = synth.make_activation(16, seed=6, rows=5)
        yt = gpu_rt.forward_batched(ptiny, torch.from_numpy(Xt.view(np.int16).copy()).view(torch.float16).cuda(),
                                    out_dtype=torch.float32).cpu().numpy()
        want = Xt.astype(np.float64) @ tiny.tail.reshape(8, 16).astype(np.float64).T
        assert np.abs(yt - want).max() <= 1e-5 * np.abs(want).max()
    finally:
        gpu_rt.free(proj)
        gpu_rt.free(ptiny)


def test_gemm_matches_gemv_rows(gpu_rt):
    """The batched kernel against the single-row kernel of the same library."""
    import torch

    raw = synth.make_matrix("model.layers.3.self_attn.k_proj.weight", 1024, 4096, seed=3)
    X = synth.make_activation(4096, seed=5, rows=16)
    proj = gpu_rt.upload(raw)
    Xd = _x16(X)
    Y = gpu_rt.forward_batched(proj, Xd, out_dtype=torch.float32)
    rows = torch.stack([gpu_rt.forward(proj, Xd[r], out_dtype=torch.float32).reshape(-1) for r in range(16)])
    gpu_rt.free(proj)
    scale = rows.abs().max().item()
    assert (Y - rows).abs().max().item() < 2e-3 * scale


@pytest.mark.parametrize("M", [48, 512])
def test_gemm_into_an_output_that_is_only_element_aligned(gpu_rt, M):
    """y as a view one element into a larger buffer (2 bytes off for binary16, 4 for f32): the kernels
    group four results into one store only where y keeps that alignment, and the bits are those of an
    aligned output either way.  48 rows finish through the partial sums, 512 also inside the launch."""
    import torch

    raw = synth.make_matrix("model.layers.3.self_attn.v_proj.weight", 1024, 2560, seed=4)
    proj = gpu_rt.upload(raw)
    try:
        X = _x16(synth.make_activation(2560, seed=6, rows=M))
        for dt in (torch.float16, torch.float32):
            want = gpu_rt.forward_batched(proj, X, out_dtype=dt)
            buf = torch.full((M * 1024 + 8,), float("nan"), dtype=dt, device="cuda")
            y = buf[1:1 + M * 1024].view(M, 1024)
            assert y.data_ptr() % 8 != 0
            gpu_rt.forward_batched_into(proj, X, y)
            gpu_rt.synchronize()
            assert torch.equal(y, want)
            assert bool(torch.isnan(buf[0])) and bool(torch.isnan(buf[1 + M * 1024:]).all())
    finally:
        gpu_rt.free(proj)


@pytest.mark.parametrize("site,d_out,d_in,M", [
    ("self_attn.k_proj", 1024, 4096, 64),     # few bands: the block range is split over units
    ("mlp.down_proj", 4096, 12288, 16),
    ("mlp.gate_proj", 12288, 4096, 256),
    ("self_attn.o_proj", 4096, 4096, 512),    # eight consumer wavefronts, bands shared between workgroups
    ("mlp.down_proj", 4096, 12288, 512),
])
def test_gemm_qwen3_8b_shapes(gpu_rt, orc, site, d_out, d_in, M):
    """BASELINE config 3 shapes; checked on a sample of activation rows to keep the f64 reference short."""
    import torch

    raw = synth.make_matrix(f"model.layers.0.{site}.weight", d_out, d_in, seed=8)
    X = synth.make_activation(d_in, seed=M + 1, rows=M)
    proj = gpu_rt.upload(raw)
    Y = gpu_rt.forward_batched(proj, _x16(X), out_dtype=torch.float32).cpu().numpy()
    gpu_rt.free(proj)
    pick = sorted({0, 1, 63, 64, M // 2, M - 65, M - 1} & set(range(M)))  # rows of every 64-row tile's ends
    Y_ref, A_ref = _reference(orc, raw, X[pick])
    _check(Y[pick], Y_ref, A_ref)
    assert np.isfinite(Y).all()


def test_gemm_2048_rows_in_chunks(gpu_rt, orc):
    """More activation rows than one launch holds: four launches of 512 rows, each row of the
    result against the oracle's on a sample that touches every chunk and its ends."""
    import torch

    d_out, d_in, M = 1024, 4096, 2048
    raw = synth.make_matrix("model.layers.0.self_attn.k_proj.weight", d_out, d_in, seed=21)
    X = synth.make_activation(d_in, seed=2048, rows=M)
    proj = gpu_rt.upload(raw)
    try:
        Y32 = gpu_rt.forward_batched(proj, _x16(X), out_dtype=torch.float32).cpu().numpy()
        Y16 = gpu_rt.forward_batched(proj, _x16(X)).cpu().numpy()
    finally:
        gpu_rt.free(proj)
    pick = sorted({0, 1, 511, 512, 513, 1023, 1024, 1500, 1535, 1536, 2046, 2047})
    Y_ref, A_ref = _reference(orc, raw, X[pick])
    e = _check(Y32[pick], Y_ref, A_ref)
    print(f"OBSERVED M=2048 max |dy|/sum|wx| = {e:.3e}")
    assert e < 3e-4
    _check(Y16[pick].astype(np.float32), Y_ref, A_ref, out_rounding=2.0 ** -11)
    assert np.isfinite(Y32).all() and np.isfinite(Y16.astype(np.float32)).all()


def test_gemm_partial_sums_of_the_call_before_do_not_leak(gpu_rt, orc):
    """Bands that several workgroups share are summed from a workspace.  Two matrices of one shape
    take turns, so the workspace holds the other one's partial sums at the same addresses whenever a
    call starts: every result must be that of the first call, bit for bit, and the first calls are
    checked against the oracle."""
    import torch

    d_out, d_in, M = 4096, 4096, 256  # 64 bands of 11 slices over 256 workgroups: every band has several pieces
    raws = [synth.make_matrix(f"model.layers.{i}.self_attn.o_proj.weight", d_out, d_in, seed=60 + i) for i in range(2)]
    Xs = [synth.make_activation(d_in, seed=70 + i, rows=M) for i in range(2)]
    projs = [gpu_rt.upload(r) for r in raws]
    try:
        xd = [_x16(X) for X in Xs]
        first = [gpu_rt.forward_batched(p, x, out_dtype=torch.float32) for p, x in zip(projs, xd)]
        for rounds in range(6):
            for i in (0, 1):
                again = gpu_rt.forward_batched(projs[i], xd[i], out_dtype=torch.float32)
                assert torch.equal(again, first[i]), f"round {rounds}, matrix {i}"
        pick = [0, 63, 64, 200, 255]
        for i in (0, 1):
            Y_ref, A_ref = _reference(orc, raws[i], Xs[i][pick])
            _check(first[i].cpu().numpy()[pick], Y_ref, A_ref)
    finally:
        for p in projs:
            gpu_rt.free(p)


def test_gemm_group_matches_the_oracle_and_the_single_calls(gpu_rt, orc):
    """Five projections that share their activation rows (more than one launch holds), as one call:
    every output against the oracle, and against the same projection called on its own (the two may
    split the block range differently, so they agree to rounding, not bit for bit)."""
    import torch

    d_in, M = 488, 70
    d_outs = [192, 72, 8, 64, 130]
    raws = [synth.make_matrix(f"model.layers.0.group{i}.weight", d, d_in, seed=40 + i) for i, d in enumerate(d_outs)]
    X = synth.make_activation(d_in, seed=9, rows=M)
    projs = [gpu_rt.upload(r) for r in raws]
    try:
        xd = _x16(X)
        for dtype in (torch.float32, torch.float16):
            ys = [torch.empty((M, d), dtype=dtype, device="cuda") for d in d_outs]
            gpu_rt.forward_batched_group_into(projs, xd, ys)
            for raw, p, y in zip(raws, projs, ys):
                Y_ref, A_ref = _reference(orc, raw, X)
                _check(y.float().cpu().numpy(), Y_ref, A_ref, out_rounding=0.0 if dtype == torch.float32 else 2.0 ** -11)
                single = gpu_rt.forward_batched(p, xd, out_dtype=dtype)
                assert (single.float() - y.float()).abs().max().item() <= 2e-3 * y.float().abs().max().item()
        with pytest.raises(Exception):
            other = gpu_rt.upload(synth.make_matrix("model.layers.0.other_width.weight", 8, 496, seed=1))
            try:
                gpu_rt.forward_batched_group_into([projs[0], other], xd, [ys[0], torch.empty((M, 8), dtype=ys[0].dtype, device="cuda")])
            finally:
                gpu_rt.free(other)
    finally:
        for p in projs:
            gpu_rt.free(p)


@pytest.mark.parametrize("M", [130, 257])
def test_gemm_bands_finished_in_the_launch(gpu_rt, orc, M):
    """More 64-row bands than workgroups: every workgroup walks whole bands alone and, where each
    multiplying wavefront owns a tile's every K-step (M > 128), finishes them in the launch — row scale,
    f32 tail, store — while the bands left over go through the workspace and the sum pass.  Three matrices
    in one call (299 bands, the first 256 walked alone), so that a short last band (6 rows), row counts
    that are no multiple of four (scalar stores) and tail columns all meet the in-launch epilogue, and a
    57-row band the sum pass; f32 and f16 outputs against the oracle."""
    import torch

    d_in = 88  # three blocks and 16 tail columns: one slice per band
    d_outs = [70, 16441, 2500]
    raws = [synth.make_matrix(f"model.layers.0.alone{i}.weight", d, d_in, seed=80 + i) for i, d in enumerate(d_outs)]
    X = synth.make_activation(d_in, seed=M, rows=M)
    projs = [gpu_rt.upload(r) for r in raws]
    try:
        xd = _x16(X)
        for dtype in (torch.float32, torch.float16):
            ys = [torch.full((M, d), float("nan"), dtype=dtype, device="cuda") for d in d_outs]
            gpu_rt.forward_batched_group_into(projs, xd, ys)
            again = [torch.empty_like(y) for y in ys]
            gpu_rt.forward_batched_group_into(projs, xd, again)
            for raw, y, y2 in zip(raws, ys, again):
                Y_ref, A_ref = _reference(orc, raw, X)
                _check(y.float().cpu().numpy(), Y_ref, A_ref, out_rounding=0.0 if dtype == torch.float32 else 2.0 ** -11)
                assert torch.equal(y, y2)
    finally:
        for p in projs:
            gpu_rt.free(p)


def test_reserved_workspaces_change_nothing(gpu_rt):
    """llvq_hip_reserve_batched only sizes buffers: the products before and after it are identical, for
    the group it was told about and at fewer rows than it was told."""
    import torch

    mats = [synth.make_matrix(f"model.layers.0.reserve.{i}.weight", do, 1000, seed=31 + i) for i, do in enumerate((192, 64))]
    projs = [gpu_rt.upload(m) for m in mats]
    try:
        X = _x16(synth.make_activation(1000, seed=5, rows=300))
        before = [gpu_rt.forward_batched(p, X, out_dtype=torch.float32) for p in projs]
        gpu_rt.reserve_batched(projs, 600)
        ys = [torch.empty((300, p.d_out), dtype=torch.float32, device="cuda") for p in projs]
        gpu_rt.forward_batched_group_into(projs, X, ys)
        for b, y in zip(before, ys):
            assert torch.equal(b, y)
        few = [gpu_rt.forward_batched(p, X[:40].contiguous(), out_dtype=torch.float32) for p in projs]
        for b, y in zip(before, few):
            assert torch.equal(b[:40], y) or float((b[:40] - y).abs().max()) < 1e-3 * float(b.abs().max())
        # and what it promises: calls up to the reserved row count take no device memory
        X6 = _x16(synth.make_activation(1000, seed=6, rows=600))
        y6 = [torch.empty((600, p.d_out), dtype=torch.float32, device="cuda") for p in projs]
        gpu_rt.synchronize()
        free_before = torch.cuda.mem_get_info()[0]
        for M in (600, 300, 100, 40):
            gpu_rt.forward_batched_group_into(projs, X6[:M], [y[:M] for y in y6])
        gpu_rt.synchronize()
        assert torch.cuda.mem_get_info()[0] == free_before
        with pytest.raises(Exception):
            gpu_rt.reserve_batched(projs, -1)
    finally:
        for p in projs:
            gpu_rt.free(p)
