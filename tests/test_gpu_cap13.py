"""Matrices of shell cap 13: 48-bit indices, 49-bit blocks in a dense stream (llvq-search/src/pack.rs:48-82,
llvq-artifact/src/format.rs:87-89, :185-203) — the one input of the reference's operator besides the 6-byte record
(llvq-llm/src/fused.rs:1166-1180).  Bars as for cap 12: points and (index, gain) fields bit-exact; products within
1e-5 (f32 results) / 1e-3 (binary16 results) of the f64 oracle, in |y - y_ref| / sum|w_i x_i|."""
import numpy as np
import pytest

from llvq_amd import LlvqError, artifact, synth

from test_gpu_parity import _dev, _oracle_matrix, _x16

pytestmark = pytest.mark.gpu


def test_decode_stream_every_class_of_the_cap13_ball(gpu_rt, orc, boundary_indices):
    """The first, quarter, middle and last index of all 383 classes and the neighbours of every class boundary,
    N(13) itself, the origin, 200 000 uniform draws below N(13) + 1 and a few numbers past N(13) that the field can
    hold: points, gain bits and shells against the oracle, for streams that start a block at every bit offset."""
    rng = synth.SplitMix64(13)
    idx = np.concatenate([boundary_indices, rng.take(200_000) % np.uint64(orc.N13 + 1),
                          np.array([orc.N13 + 1, (1 << 48) - 1], np.uint64)])
    gains = (rng.take(idx.size) & np.uint64(1)).astype(np.uint8)
    codes = artifact.pack_codes(idx, gains, index_width=48)
    assert codes.size == (idx.size * 49 + 7) // 8
    pts, g, shells = gpu_rt.decode_stream(_dev(codes), idx.size, 13)
    ok = idx <= np.uint64(orc.N13)
    ref = orc.decode_many(idx[ok], fast=False)
    got = pts.cpu().numpy()
    assert np.array_equal(got[ok], ref)
    assert np.all(got[~ok] == 0) and np.all(shells.cpu().numpy()[~ok] == 0xFF)
    assert np.array_equal(g.cpu().numpy(), gains)
    assert np.array_equal(shells.cpu().numpy()[ok].astype(np.int64), (ref.astype(np.int64) ** 2).sum(1) // 16)
    # the cap-12 stream through the same entry point is the 6-byte probe
    idx12 = boundary_indices[boundary_indices < (1 << 47)]
    p12, _, _ = gpu_rt.decode_stream(_dev(artifact.pack_codes(idx12, np.zeros(idx12.size, np.uint8))), idx12.size, 12)
    assert np.array_equal(p12.cpu().numpy(), orc.decode_many(idx12, fast=False))


@pytest.mark.parametrize("d_out,d_in", [(4096, 2560), (1024, 4096), (7, 77), (333, 24 * 35 + 5), (64, 9728), (40, 17408), (5000, 48)])
def test_gemv_cap13_matches_the_oracle(gpu_rt, orc, d_out, d_in):
    """Shapes whose tiles start at odd bit offsets of the stream (odd rows x odd blocks per row), with and without
    tail columns, one wider than the full table image allows beside its planes (17 408: the lean image), many tiles
    per workgroup and fewer tiles than workgroups; f32 and binary16 results."""
    import torch

    raw = synth.make_matrix(f"model.layers.0.cap13.{d_out}x{d_in}.weight", d_out, d_in, seed=3, shell_cap=13)
    assert raw.shell_cap == 13 and raw.codes.size == (d_out * (d_in // 24) * 49 + 7) // 8
    x = synth.make_activation(d_in, seed=4)[0]
    proj = gpu_rt.upload(raw)
    try:
        y32 = gpu_rt.forward(proj, _x16(x), out_dtype=torch.float32).cpu().numpy().reshape(-1)
        y16 = gpu_rt.forward(proj, _x16(x), out_dtype=torch.float16).float().cpu().numpy().reshape(-1)
    finally:
        gpu_rt.free(proj)
    om = _oracle_matrix(orc, raw)
    y_ref, a_ref = om.fused_product(x.astype(np.float64))
    e32 = (np.abs(y32 - y_ref) / np.maximum(a_ref, 1e-30)).max()
    assert e32 < 1e-5, f"f32 results: {e32:.3e}"
    e16 = (np.abs(y16 - y_ref) / np.maximum(a_ref, 1e-30)).max()  # (a binary16 result carries its own half ulp)
    assert e16 < 1e-3, f"binary16 results: {e16:.3e}"


def test_gemv_cap13_kernel_unranks_every_coordinate_exactly(gpu_rt, orc, boundary_indices):
    """One-hot activations read a cap-13 matrix back column by column through the product kernel's own stream
    extraction, class find and decoders: all 24 coordinates of 61 440 blocks — every class boundary of the ball,
    uniform draws over it (60 % of them on shell 13), origins, both gain bits — are the oracle's integers."""
    import torch

    d_out, nb = 4096, 15
    n = d_out * nb
    rng = synth.SplitMix64(0xCA913)
    idx = rng.take(n) % np.uint64(orc.N13 + 1)
    idx[: boundary_indices.size] = boundary_indices
    idx[boundary_indices.size: boundary_indices.size + 64] = 0
    idx = idx[np.random.default_rng(5).permutation(n)]
    gains = (rng.take(n) & np.uint64(1)).astype(np.uint8)
    cent = [0.75, 1.5]
    raw = artifact.RawMatrix("model.layers.0.coords13.weight", d_out, nb * 24, 13, cent, np.ones(d_out), np.zeros(0, np.float32),
                             artifact.pack_codes(idx, gains, index_width=48))
    proj = gpu_rt.upload(raw)
    try:
        eye = torch.eye(nb * 24, dtype=torch.float16, device="cuda")
        W = torch.stack([gpu_rt.forward(proj, eye[c], out_dtype=torch.float32).reshape(-1) for c in range(nb * 24)])
        W = W.t().contiguous().cpu().numpy().astype(np.float64)
    finally:
        gpu_rt.free(proj)
    pts = orc.decode_many(idx).astype(np.int64)
    n2 = (pts * pts).sum(axis=1).astype(np.float64)
    scale = np.where(n2 > 0, np.array(cent)[gains] / np.sqrt(np.maximum(n2, 1.0)), 0.0)
    got = W.reshape(n, 24)
    zero = n2 == 0
    assert zero.sum() >= 64 and np.all(got[zero] == 0.0)
    back = got[~zero] / scale[~zero, None]
    assert np.abs(back - np.rint(back)).max() < 1e-3
    assert np.array_equal(np.rint(back).astype(np.int64), pts[~zero])


def test_cap13_groups_rotation_and_batched_rows(gpu_rt, orc):
    """A group of cap-13 matrices in one call; a call that mixes caps (one launch per cap); a cap-13 matrix stored
    in a rotated basis (a kernel of its own rotates the activation); batched rows (a loop over the rows' products)."""
    import torch

    mk = lambda name, do, cap: synth.make_matrix(f"model.layers.1.{name}.weight", do, 2560, seed=6, shell_cap=cap)
    raws = [mk("q13", 512, 13), mk("k13", 128, 13), mk("v12", 128, 12), mk("o13", 96, 13)]
    rot = synth.make_matrix("model.layers.1.rot13.weight", 192, 1536, seed=7, shell_cap=13)
    rot = artifact.RawMatrix(rot.name, rot.d_out, rot.d_in, 13, rot.centroids, rot.row_scales, rot.tail, rot.codes, rotation_seed=0x13)
    projs = [gpu_rt.upload(m) for m in raws]
    prot = gpu_rt.upload(rot)
    try:
        x = synth.make_activation(2560, seed=8)[0]
        ys = gpu_rt.forward_group(projs, _x16(x), out_dtype=torch.float32)
        for y, m in zip(ys, raws):
            y_ref, a_ref = _oracle_matrix(orc, m).fused_product(x.astype(np.float64))
            assert (np.abs(y.cpu().numpy().reshape(-1) - y_ref) / np.maximum(a_ref, 1e-30)).max() < 1e-5, m.name
        xr = synth.make_activation(1536, seed=9)[0]
        yr = gpu_rt.forward(prot, _x16(xr), out_dtype=torch.float32).cpu().numpy().reshape(-1)
        y_ref, a_ref = _oracle_matrix(orc, rot).fused_product(xr.astype(np.float64))
        assert (np.abs(yr - y_ref) / np.maximum(a_ref, 1e-30)).max() < 1e-5
        X = synth.make_activation(2560, seed=10, rows=5)
        Y = gpu_rt.forward_batched(projs[0], _x16(X), out_dtype=torch.float32)
        for r in range(5):
            assert torch.equal(Y[r], gpu_rt.forward(projs[0], _x16(X[r]), out_dtype=torch.float32).reshape(-1))
    finally:
        for p in projs + [prot]:
            gpu_rt.free(p)


def test_cap13_refusals(gpu_rt, orc):
    """Named refusals, nothing enqueued: an index past N(13) in the stream, a cap whose blocks are neither 48 nor 49
    bits, a sequence that mixes caps."""
    import torch

    idx = np.array([5, orc.N13 + 1, 7], np.uint64)
    bad = artifact.RawMatrix("model.layers.0.bad13.weight", 1, 72, 13, [0.8, 1.25], np.ones(1), np.zeros(0, np.float32),
                             artifact.pack_codes(idx, np.zeros(3, np.uint8), index_width=48))
    with pytest.raises(LlvqError) as err:
        gpu_rt.upload(bad)
    assert err.value.kind == "IndexOutOfRange"
    w11 = artifact.index_bits(11)
    cap11 = artifact.RawMatrix("model.layers.0.cap11.weight", 1, 72, 11, [0.8, 1.25], np.ones(1), np.zeros(0, np.float32),
                               artifact.pack_codes(np.array([1, 2, 3], np.uint64), np.zeros(3, np.uint8), index_width=w11))
    with pytest.raises(LlvqError) as err:
        gpu_rt.upload(cap11)
    assert err.value.kind == "Unsupported" and "cap 11" in str(err.value)
    p13 = gpu_rt.upload(synth.make_matrix("model.layers.0.seq13.weight", 64, 512, seed=1, shell_cap=13))
    p12 = gpu_rt.upload(synth.make_matrix("model.layers.0.seq12.weight", 64, 512, seed=1, shell_cap=12))
    try:
        x = torch.zeros(512, dtype=torch.float16, device="cuda")
        with pytest.raises(LlvqError) as err:  # one record width per sequence
            gpu_rt.plan_sequence([([p13], x, False), ([p12], x, False)])
        assert err.value.kind == "Unsupported" and "one shell cap" in str(err.value)
    finally:
        gpu_rt.free(p13)
        gpu_rt.free(p12)


@pytest.mark.parametrize("out", ["f16", "f32"])
def test_cap13_sequence_matches_the_separate_calls(gpu_rt, orc, out):
    """Cap-13 matrices through the sequence kernel: items of several widths (tiles that begin inside a byte of the
    dense stream, rows of one block, tail columns only, more tiles than workgroups), independent and ordered,
    against llvq_hip_gemv_group item by item, bit for bit, on two runs; one item against the CPU oracle."""
    import torch

    dt = torch.float16 if out == "f16" else torch.float32
    groups = [[(1024, 2560), (256, 2560)], [(640, 4096)], [(2432, 2560), (2432, 2560)], [(320, 9728)], [(40, 17)],
              [(5000, 48)], [(7, 24 * 700 + 5)], [(333, 2560)]]
    uploaded, items, xs = [], [], {}
    try:
        for gi, shapes in enumerate(groups):
            raws = [synth.make_matrix(f"model.layers.{gi}.s{j}.weight", do, di, seed=40 + gi, shell_cap=13) for j, (do, di) in enumerate(shapes)]
            projs = [gpu_rt.upload(m) for m in raws]
            uploaded.append((raws, projs))
            d_in = shapes[0][1]
            if d_in not in xs:
                xs[d_in] = synth.make_activation(d_in, seed=d_in)[0]
            items.append((projs, _x16(xs[d_in]), False))
        seq = gpu_rt.plan_sequence(items, out_dtype=dt)
        try:
            want = [gpu_rt.forward_group(projs, x, out_dtype=dt) for projs, x, _ in items]
            for run in range(2):
                for ys in seq.outputs:
                    for y in ys:
                        y.fill_(float("nan"))
                seq.run()
                seq.status()
                for gi, (ys, ws) in enumerate(zip(seq.outputs, want)):
                    for y, w in zip(ys, ws):
                        assert torch.equal(y.view(torch.int16 if out == "f16" else torch.int32), w.view(torch.int16 if out == "f16" else torch.int32)), \
                            f"run {run}, item {gi}: outputs differ from the separate call"
            if out == "f32":
                raw, x = uploaded[7][0][0], xs[2560]
                y_ref, a_ref = _oracle_matrix(orc, raw).fused_product(x.astype(np.float64))
                assert (np.abs(seq.outputs[7][0].cpu().numpy().reshape(-1) - y_ref) / np.maximum(a_ref, 1e-30)).max() < 1e-5
        finally:
            seq.close()
        # ordered: the second item reads what the first one wrote
        a = gpu_rt.upload(synth.make_matrix("model.layers.9.a.weight", 2560, 2560, seed=77, shell_cap=13))
        b = gpu_rt.upload(synth.make_matrix("model.layers.9.b.weight", 1000, 2560, seed=78, shell_cap=13))
        try:
            x = _x16(xs[2560])
            mid = gpu_rt.forward(a, x, out_dtype=torch.float16).reshape(-1)
            want_b = gpu_rt.forward(b, mid, out_dtype=torch.float16).reshape(-1)
            ya = torch.empty(2560, dtype=torch.float16, device="cuda")
            chain = gpu_rt.plan_sequence([([a], x, False, [ya]), ([b], ya, True)], out_dtype=torch.float16)
            try:
                chain.run()
                chain.status()
                assert torch.equal(chain.outputs[0][0].view(torch.int16), mid.view(torch.int16))
                assert torch.equal(chain.outputs[1][0].view(torch.int16), want_b.view(torch.int16))
            finally:
                chain.close()
        finally:
            gpu_rt.free(a)
            gpu_rt.free(b)
    finally:
        for _, projs in uploaded:
            for p in projs:
                gpu_rt.free(p)
