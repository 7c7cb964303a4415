"""Parity of the HIP path against the CPU oracle, through the C ABI.

Bars: lattice points and (index, gain) fields bit-exact; GEMV within 1e-3 of the
f64 reference, measured as |y - y_ref| / sum|w_i x_i| (the reference's own V0
metric, llvq-cuda/src/bin/matvec.rs:114-120) and as plain relative error where
|y_ref| is not tiny.
"""
import numpy as np
import pytest

from llvq_amd import artifact, synth

pytestmark = pytest.mark.gpu

TOL = 1e-3  # north-star tolerance for GEMV/GEMM outputs (f32 accumulate)


def _dev(a):
    import torch

    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def _x16(x):
    import torch

    return torch.from_numpy(x.view(np.int16).copy()).view(torch.float16).cuda()


def _oracle_matrix(orc, raw):
    m, _ = orc.read_matrix_raw(artifact.write_matrix_raw(raw))
    return m


def _check_gemv(orc, y, raw, x):
    om = _oracle_matrix(orc, raw)
    y_ref, a_ref = om.fused_product(x.astype(np.float64))
    y = y.astype(np.float64)
    e_norm = np.abs(y - y_ref) / np.maximum(a_ref, 1e-30)
    assert e_norm.max() < TOL, f"max |dy|/sum|wx| = {e_norm.max():.3e}"
    big = np.abs(y_ref) > 1e-2 * a_ref
    if big.any():
        rel = np.abs(y - y_ref)[big] / np.abs(y_ref)[big]
        assert rel.max() < TOL, f"max relative error {rel.max():.3e}"
    return e_norm.max()


def test_decode_class_boundaries_bit_exact(gpu_rt, orc, boundary_indices):
    idx = boundary_indices[boundary_indices < (1 << 47)]  # what a 47-bit field can hold
    gains = (np.arange(idx.size) & 1).astype(np.uint8)
    pts, g, shells = gpu_rt.decode_blocks(_dev(artifact.pack_codes(idx, gains)))
    ref = orc.decode_many(idx, fast=False)
    assert np.array_equal(pts.cpu().numpy(), ref)
    assert np.array_equal(g.cpu().numpy(), gains)
    ref_shell = (ref.astype(np.int64) ** 2).sum(1) // 16
    assert np.array_equal(shells.cpu().numpy().astype(np.int64), ref_shell)


def test_decode_zero_run_free_classes(gpu_rt, orc):
    """Even classes with no zero coordinate: the case where 'last kind = zero run'
    must be decided by value (llvq-metal/shaders/cascade_archive.metal:186-205)."""
    picks = []
    for ci in range(orc.lib().orc_n_classes()):
        info = orc.class_info(ci)
        vals, counts, _ = orc.class_levels(ci)
        if not info["odd"] and 0 not in vals and info["lo"] < (1 << 47):
            hi = min(info["hi"], (1 << 47) - 1)
            picks += list(np.linspace(info["lo"], hi, 64, dtype=np.uint64))
    assert len(picks) >= 6 * 64
    idx = np.array(picks, dtype=np.uint64)
    pts, _, _ = gpu_rt.decode_blocks(_dev(artifact.pack_codes(idx, np.zeros(idx.size, np.uint8))))
    assert np.array_equal(pts.cpu().numpy(), orc.decode_many(idx))


def test_decode_million_uniform_ranks_bit_exact(gpu_rt, orc):
    rng = synth.SplitMix64(0x63_0001)
    idx = rng.take(1_000_000) % np.uint64(orc.N12 + 1)
    gains = (rng.take(idx.size) & np.uint64(1)).astype(np.uint8)
    pts, g, _ = gpu_rt.decode_blocks(_dev(artifact.pack_codes(idx, gains)))
    assert np.array_equal(pts.cpu().numpy(), orc.decode_many(idx))
    assert np.array_equal(g.cpu().numpy(), gains)


def test_decode_full_47bit_range(gpu_rt, orc):
    """Indices in (N(12), 2^47) fit the field and decode as shell-13 points."""
    rng = synth.SplitMix64(7)
    idx = rng.take(200_000) % np.uint64(1 << 47)
    pts, _, shells = gpu_rt.decode_blocks(_dev(artifact.pack_codes(idx, np.zeros(idx.size, np.uint8))))
    assert np.array_equal(pts.cpu().numpy(), orc.decode_many(idx))
    assert shells.max().item() == 13


def test_decode_empty(gpu_rt):
    import torch

    pts, g, s = gpu_rt.decode_blocks(torch.empty(0, dtype=torch.uint8, device="cuda"))
    assert pts.shape == (0, 24) and g.numel() == 0


# (d_out, d_in) of llvq-artifact/tests/fused_path_matches_dense.rs:45-51 plus ragged shapes
SMALL_SHAPES = [(8, 240), (8, 2560), (16, 9728), (8, 4096), (24, 96), (1, 24), (3, 47), (5, 2568), (7, 5120),
                (4, 16), (2, 23)]  # the last two have no whole block: tail columns only


@pytest.mark.parametrize("d_out,d_in", SMALL_SHAPES)
def test_gemv_small_shapes(gpu_rt, orc, d_out, d_in):
    import torch

    raw = synth.make_matrix(f"model.layers.0.test.{d_out}x{d_in}.weight", d_out, d_in, seed=d_out * 131 + d_in)
    x = synth.make_activation(d_in, seed=d_in)[0]
    proj = gpu_rt.upload(raw)
    try:
        y32 = gpu_rt.forward(proj, _x16(x), out_dtype=torch.float32).cpu().numpy()
        y16 = gpu_rt.forward(proj, _x16(x)).cpu().numpy()
    finally:
        gpu_rt.free(proj)
    e = _check_gemv(orc, y32, raw, x)
    assert e < 1e-5  # f32 out: the reference's own threshold (docs/mesures/e1v-cuda-2026-08-16.txt:95-96)
    _check_gemv(orc, y16.astype(np.float32), raw, x)


def test_gemv_rows_wider_than_the_full_tile(gpu_rt, orc):
    """d_in 17408 (the 14B intermediate size: 725 blocks + 8 tail columns): the activation
    planes leave no room for the 4096-block tile, so the half-tile variant runs."""
    import torch

    raw = synth.make_matrix("model.layers.0.mlp.down_proj.weight", 40, 17408, seed=14)
    x = synth.make_activation(17408, seed=14)[0]
    proj = gpu_rt.upload(raw)
    y = gpu_rt.forward(proj, _x16(x), out_dtype=torch.float32).cpu().numpy()
    gpu_rt.free(proj)
    assert _check_gemv(orc, y, raw, x) < 1e-5


def test_gemv_origin_and_shell13_blocks(gpu_rt, orc):
    """A matrix whose blocks are origins (decode to zero whatever the gain) and
    shell-13 indices above N(12)."""
    import torch

    d_out, d_in = 16, 24 * 8 + 5
    rng = synth.SplitMix64(99)
    idx = rng.take(d_out * 8) % np.uint64(1 << 47)
    idx[::3] = 0
    idx[1::7] = np.uint64((1 << 47) - 1)
    gains = (rng.take(idx.size) & np.uint64(1)).astype(np.uint8)
    raw = artifact.RawMatrix("model.layers.0.edge.weight", d_out, d_in, 12, [0.8, 1.25],
                             np.exp(rng.gaussian(d_out)), rng.gaussian(d_out * 5).astype(np.float32),
                             artifact.pack_codes(idx, gains))
    x = synth.make_activation(d_in, seed=5)[0]
    proj = gpu_rt.upload(raw)
    y = gpu_rt.forward(proj, _x16(x), out_dtype=torch.float32).cpu().numpy()
    gpu_rt.free(proj)
    _check_gemv(orc, y, raw, x)


def _class_ranges(orc, want):
    """Zero-based rank ranges [lo, hi) of the cap-12 classes that `want(odd, w, vals)` picks."""
    ranges = []
    for ci in range(383):
        info = orc.class_info(ci)
        vals, _, _ = orc.class_levels(ci)
        if info["shell"] <= 12 and want(info["odd"], info["w"], vals):
            ranges.append((info["lo"], info["hi"]))
    return ranges


def _is_rare(odd, w, vals):
    """The classes the kernels unrank by the generic walk: odd with five magnitudes, support weight 0 or 24,
    three word kinds."""
    if odd:
        return len(vals) > 4
    return not (w in (8, 12, 16) and len([v for v in vals if abs(v) % 4 == 2]) <= 2)


def _matrix_of_classes(ranges, d_out, nb, seed, name):
    rng = np.random.default_rng(seed)
    pick = rng.integers(0, len(ranges), size=d_out * nb)
    lo = np.array([r[0] for r in ranges], np.uint64)[pick]
    span = np.array([r[1] - r[0] for r in ranges], np.uint64)[pick]
    idx = lo + (rng.integers(0, 1 << 62, size=pick.size, dtype=np.uint64) % span) + np.uint64(1)  # index = 1 + zero-based rank
    gains = rng.integers(0, 2, size=idx.size).astype(np.uint8)
    return artifact.RawMatrix(name, d_out, nb * 24, 12, [0.8, 1.25], np.exp(rng.normal(size=d_out)),
                              np.zeros(0, np.float32), artifact.pack_codes(idx, gains))


def test_gemv_tiles_full_of_rare_class_blocks(gpu_rt, orc):
    """Every block from a class that takes the generic walk.  2560 rows of 40 blocks make tiles of ten rows:
    400 such blocks in a tile, six times what the kernel's two side queues for them hold, so the overflow
    path (the blocks ride in the odd queue, flagged) runs in every tile.  Uniform draws meet these classes
    0.07 % of the time."""
    import torch

    ranges = _class_ranges(orc, _is_rare)
    assert len(ranges) == 30
    raw = _matrix_of_classes(ranges, 2560, 40, 11, "model.layers.0.rare.weight")
    x = synth.make_activation(40 * 24, seed=12)[0]
    proj = gpu_rt.upload(raw)
    try:
        y = gpu_rt.forward(proj, _x16(x), out_dtype=torch.float32).cpu().numpy()
        X = torch.from_numpy(np.stack([x, x]).view(np.int16).copy()).view(torch.float16).cuda()
        Y = gpu_rt.forward_batched(proj, X, out_dtype=torch.float32).cpu().numpy()
    finally:
        gpu_rt.free(proj)
    assert _check_gemv(orc, y, raw, x) < 1e-5
    # the batched path rounds the weights to binary16: 1e-3 of sum|w x|, as tests/test_gpu_gemm.py states it
    y_ref, a_ref = _oracle_matrix(orc, raw).fused_product(x.astype(np.float64))
    assert (np.abs(Y[1].astype(np.float64) - y_ref) / np.maximum(a_ref, 1e-30)).max() < 1e-3


@pytest.mark.parametrize("share", [1.0, 0.5])
def test_gemv_tiles_full_of_second_free_kind_blocks(gpu_rt, orc, share):
    """Even-coset classes whose off-support slots hold two magnitudes besides zero have a decoder and a
    384-slot queue of their own (6 to 8 % of uniform draws, about 300 of a full tile).  2560 rows of 100 blocks
    make tiles of 1000 blocks: with every block from such a class 616 of them overflow into the even queue,
    flagged, in every tile; with half of them plain even-coset blocks the even queue's chunks mix the two."""
    import torch

    second = _class_ranges(orc, lambda odd, w, vals: not odd and not _is_rare(odd, w, vals)
                           and len([v for v in vals if v != 0 and abs(v) % 4 == 0]) > 1)
    plain = _class_ranges(orc, lambda odd, w, vals: not odd and not _is_rare(odd, w, vals)
                          and len([v for v in vals if v != 0 and abs(v) % 4 == 0]) <= 1)
    assert second and plain
    d_out, nb = 2560, 100
    raw = _matrix_of_classes(second, d_out, nb, 21, "model.layers.0.second.weight")
    if share < 1.0:
        other = _matrix_of_classes(plain, d_out, nb, 22, "x")
        keep = np.random.default_rng(23).random(d_out * nb) < share
        codes = raw.codes.reshape(-1, 6).copy()
        codes[~keep] = other.codes.reshape(-1, 6)[~keep]
        raw = artifact.RawMatrix(raw.name, d_out, nb * 24, 12, [0.8, 1.25], raw.row_scales, np.zeros(0, np.float32), codes.reshape(-1))
    x = synth.make_activation(nb * 24, seed=24)[0]
    proj = gpu_rt.upload(raw)
    try:
        y = gpu_rt.forward(proj, _x16(x), out_dtype=torch.float32).cpu().numpy()
    finally:
        gpu_rt.free(proj)
    assert _check_gemv(orc, y, raw, x) < 1e-5


def test_gemv_kernel_unranks_every_coordinate_exactly(gpu_rt, orc, boundary_indices):
    """The lattice points as the product kernels themselves unrank them (their own class find, queues and
    decoders, not the probe kernel's): one-hot activations read the matrix back column by column, and
    every one of the 24 coordinates of 163 840 blocks must be the oracle's integer — class boundaries,
    the rare classes, the classes with a second free kind, uniform cap-12 ranks and ranks over the whole
    47-bit field (shell 13), origins, both gain bits."""
    import torch

    d_out, nb = 4096, 40
    n = d_out * nb
    rng = synth.SplitMix64(0x5EED)
    idx = rng.take(n) % np.uint64(orc.N12 + 1)
    wide = rng.take(n // 8) % np.uint64(1 << 47)
    idx[: wide.size] = wide
    b = boundary_indices[boundary_indices < (1 << 47)]
    idx[wide.size: wide.size + b.size] = b
    at = wide.size + b.size
    for want, count in ((_is_rare, 4000), (lambda odd, w, vals: not odd and not _is_rare(odd, w, vals)
                                           and len([v for v in vals if v != 0 and abs(v) % 4 == 0]) > 1, 8000)):
        ranges = _class_ranges(orc, want)
        pick = np.random.default_rng(count).integers(0, len(ranges), size=count)
        lo = np.array([r[0] for r in ranges], np.uint64)[pick]
        span = np.array([r[1] - r[0] for r in ranges], np.uint64)[pick]
        idx[at: at + count] = lo + (rng.take(count) % span) + np.uint64(1)
        at += count
    idx[at: at + 64] = 0  # origins
    perm = np.random.default_rng(9).permutation(n)  # every tile gets its share of every kind
    idx = idx[perm]
    gains = (rng.take(n) & np.uint64(1)).astype(np.uint8)
    cent = [0.75, 1.5]
    raw = artifact.RawMatrix("model.layers.0.coords.weight", d_out, nb * 24, 12, cent, np.ones(d_out), np.zeros(0, np.float32),
                             artifact.pack_codes(idx, gains))
    proj = gpu_rt.upload(raw)
    try:
        eye = torch.eye(nb * 24, dtype=torch.float16, device="cuda")
        cols = [gpu_rt.forward(proj, eye[c], out_dtype=torch.float32).reshape(-1) for c in range(nb * 24)]
        W = torch.stack(cols).t().contiguous().cpu().numpy().astype(np.float64)  # [d_out, d_in]
        # the batched kernel's producers unrank on their own: the identity as 960 activation rows reads the matrix back too
        Wb = gpu_rt.forward_batched(proj, eye, out_dtype=torch.float32).t().contiguous().cpu().numpy().astype(np.float64)
    finally:
        gpu_rt.free(proj)
    pts = orc.decode_many(idx).astype(np.int64)  # [n, 24]
    n2 = (pts * pts).sum(axis=1).astype(np.float64)
    scale = np.where(n2 > 0, np.array(cent)[gains] / np.sqrt(np.maximum(n2, 1.0)), 0.0)
    got = W.reshape(n, 24)
    zero = n2 == 0
    assert zero.sum() >= 64 and np.all(got[zero] == 0.0)
    back = got[~zero] / scale[~zero, None]
    assert np.abs(back - np.rint(back)).max() < 1e-3
    assert np.array_equal(np.rint(back).astype(np.int64), pts[~zero])
    # batched path: a weight is rounded once to binary16 (2^-11 relative, under 0.02 for coordinates below 32), so the
    # integers are still unambiguous
    gotb = Wb.reshape(n, 24)
    assert np.all(gotb[zero] == 0.0)
    backb = gotb[~zero] / scale[~zero, None]
    assert np.abs(backb - np.rint(backb)).max() < 0.02
    assert np.array_equal(np.rint(backb).astype(np.int64), pts[~zero])


def test_gemv_config0_full_size(gpu_rt, orc):
    """BASELINE config 0: gate_proj 9728 x 2560, seed 0, against the oracle's f64 product."""
    import torch

    raw = synth.config0(seed=0)
    assert raw.encoded_bytes() == 6_887_440
    x = synth.make_activation(2560, seed=0)[0]
    proj = gpu_rt.upload(raw)
    y = gpu_rt.forward(proj, _x16(x), out_dtype=torch.float32).cpu().numpy()
    gpu_rt.free(proj)
    e = _check_gemv(orc, y, raw, x)
    assert e < 1e-5


def test_gemv_config1_full_size_groups(gpu_rt, orc):
    """BASELINE config 1: the seven projections of one Qwen3-4B layer at full size, through the four
    group launches a decode step makes (q/k/v, o, gate/up, down), f32 and binary16 outputs, against the
    oracle's f64 fused product.  Bars: 1e-5 of sum|w_i x_i| for f32 outputs, 1e-3 for binary16 ones
    (the reference's own, docs/mesures/e1v-cuda-2026-08-16.txt:95-96)."""
    import torch

    mats = synth.layer_matrices(0, seed=0)
    assert sum(m.encoded_bytes() for m in mats) == 27_243_632
    acts = {d: synth.make_activation(d, seed=0)[0] for d in (2560, 4096, 9728)}
    projs = [gpu_rt.upload(m) for m in mats]
    refs = [_oracle_matrix(orc, m).fused_product(acts[m.d_in].astype(np.float64)) for m in mats]
    try:
        worst = {}
        for dtype, bar in ((torch.float32, 1e-5), (torch.float16, 1e-3)):
            ys = []
            for group in (projs[0:3], projs[3:4], projs[4:6], projs[6:7]):
                ys += gpu_rt.forward_group(group, _x16(acts[group[0].d_in]), out_dtype=dtype)
            worst[dtype] = 0.0
            for m, y, (y_ref, a_ref) in zip(mats, ys, refs):
                assert y.shape[-1] == m.d_out
                e = np.abs(y.float().cpu().numpy().reshape(-1).astype(np.float64) - y_ref) / np.maximum(a_ref, 1e-30)
                assert e.max() < bar, f"{m.name} {dtype}: max |dy|/sum|wx| = {e.max():.3e}"
                worst[dtype] = max(worst[dtype], float(e.max()))
        print(f"config 1 worst |dy|/sum|wx|: f32 {worst[torch.float32]:.2e}, f16 {worst[torch.float16]:.2e}")
    finally:
        for p in projs:
            gpu_rt.free(p)


def test_gemv_group_matches_single(gpu_rt, orc):
    import torch

    mats = [synth.make_matrix(f"model.layers.1.self_attn.{n}.weight", do, 2560, seed=3)
            for n, do in (("q_proj", 96), ("k_proj", 32), ("v_proj", 32))]
    x = synth.make_activation(2560, seed=11)[0]
    projs = [gpu_rt.upload(m) for m in mats]
    ys = gpu_rt.forward_group(projs, _x16(x), out_dtype=torch.float32)
    for p, raw, y in zip(projs, mats, ys):
        single = gpu_rt.forward(p, _x16(x), out_dtype=torch.float32)
        assert torch.equal(single, y)
        _check_gemv(orc, y.cpu().numpy(), raw, x)
        gpu_rt.free(p)


def test_batched_rows_match_oracle(gpu_rt, orc):
    """Rows of a batch through llvq_hip_gemm.  Two or more rows take the matrix-core
    path, whose weights are binary16 (one rounding, 2^-11 relative, per weight), so
    the bar is the normalised error; a single row takes the GEMV kernel and its bar."""
    import torch

    raw = synth.make_matrix("model.layers.2.mlp.up_proj.weight", 64, 2560, seed=4)
    X = synth.make_activation(2560, seed=21, rows=16)
    proj = gpu_rt.upload(raw)
    Y = gpu_rt.forward_batched(proj, _x16(X), out_dtype=torch.float32).cpu().numpy()
    y0 = gpu_rt.forward_batched(proj, _x16(X[:1]), out_dtype=torch.float32).cpu().numpy()
    gpu_rt.free(proj)
    om = _oracle_matrix(orc, raw)
    for r in range(X.shape[0]):
        y_ref, a_ref = om.fused_product(X[r].astype(np.float64))
        e_norm = np.abs(Y[r].astype(np.float64) - y_ref) / np.maximum(a_ref, 1e-30)
        assert e_norm.max() < TOL, f"row {r}: max |dy|/sum|wx| = {e_norm.max():.3e}"
    assert _check_gemv(orc, y0[0], raw, X[0]) < 1e-5


def test_record_upload_path(gpu_rt, orc):
    """The library's own record reader: an on-disk LVQ4 file, parsed and uploaded through the C ABI."""
    import ctypes as C

    import torch

    from llvq_amd import _ffi

    mats = [synth.make_matrix(f"model.layers.0.self_attn.{n}.weight", 16, 2560, seed=8) for n in ("q_proj", "k_proj")]
    buf = artifact.write_file(mats, version=4)
    pos = C.c_size_t(0)
    ver, n = C.c_uint32(), C.c_uint32()
    _ffi.check(_ffi.lib().llvq_hip_read_header(buf, len(buf), C.byref(pos), C.byref(ver), C.byref(n)))
    assert (ver.value, n.value) == (4, 2)
    x = synth.make_activation(2560, seed=1)[0]
    p = pos.value
    for raw in mats:
        proj, p = gpu_rt.upload_record(buf, p)
        assert proj.name == raw.name
        y = gpu_rt.forward(proj, _x16(x), out_dtype=torch.float32).cpu().numpy()
        gpu_rt.free(proj)
        _check_gemv(orc, y, raw, x)
    assert p == len(buf) - 8


def test_full_size_properties_linearity_and_scaling(gpu_rt):
    """Size-independent properties at config-0 size: y(2x) = 2 y(x) exactly in
    binary floating point, and y is linear in the activation to rounding."""
    import torch

    raw = synth.config0(seed=0)
    proj = gpu_rt.upload(raw)
    x = _x16(synth.make_activation(2560, seed=0)[0])
    z = _x16(synth.make_activation(2560, seed=1)[0])
    y1 = gpu_rt.forward(proj, x, out_dtype=torch.float32)
    y2 = gpu_rt.forward(proj, (x * 2).contiguous(), out_dtype=torch.float32)
    assert torch.equal(y2, 2 * y1)
    half = torch.float16
    xz = (x.float() * 0.5 + z.float() * 0.5).to(half)  # may round: compare against f32 products of the rounded sum
    yz = gpu_rt.forward(proj, xz, out_dtype=torch.float32)
    exact = (xz.float() == x.float() * 0.5 + z.float() * 0.5)
    lin = 0.5 * y1 + 0.5 * gpu_rt.forward(proj, z, out_dtype=torch.float32)
    if bool(exact.all()):
        assert torch.allclose(yz, lin, rtol=1e-4, atol=1e-6)
    gpu_rt.free(proj)
