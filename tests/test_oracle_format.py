"""Pins of the oracle's byte-level side: bit stream, matrix record, header,
reconstruct / products, f16 conversions, SplitMix64 — against the reference's
own known answers and against independent routines (numpy, the host-side
Python mirror of the record layout)."""
import struct

import numpy as np
import pytest

from llvq_amd import artifact, synth


# ---- llvq-search/tests/g6_pack.rs ------------------------------------------------------
def test_bit_order_is_most_significant_first(orc):
    assert orc.pack_bits([(0b101, 3), (0b011, 3), (0b110, 3)]) == bytes([0b10101111, 0])
    assert orc.pack_bits([(0, 0), (0b1011, 4), (0, 0), (0b0110, 4)]) == bytes([0b10110110])
    with pytest.raises(ValueError):
        orc.pack_bits([(0b10000, 4)])


def test_bit_stream_round_trips_at_every_width(orc):
    for width in range(1, 65):
        hi = (1 << width) - 1
        vals = [0, 1, hi, hi // 2, hi // 3]
        buf = orc.pack_bits([(v, width) for v in vals])
        assert len(buf) == (5 * width + 7) // 8
        assert orc.read_bits(buf, [width] * 5) == vals


def test_index_stream_is_six_bytes_per_block(orc):
    rng = synth.SplitMix64(0x69AC1)
    idx = (rng.take(4096) >> np.uint64(17)) % np.uint64(orc.N13)
    gains = rng.take(4096) & np.uint64(1)
    buf = orc.pack_bits([w for i, g in zip(idx, gains) for w in ((int(i), 47), (int(g), 1))])
    assert len(buf) == 4096 * 6 == 24576
    # the vectorised packer of the product's host side writes the same bytes
    assert artifact.pack_codes(idx, gains).tobytes() == buf
    back = orc.read_bits(buf, [47, 1] * 4096)
    assert back[0::2] == [int(i) for i in idx] and back[1::2] == [int(g) for g in gains]


# ---- record layout: format.rs:166-203, g6_format.rs, hostile_files.rs --------------------
def _small(name="model.layers.0.self_attn.q_proj.weight", d_out=3, d_in=53, seed=5):
    return synth.make_matrix(name, d_out, d_in, seed=seed)


def test_record_field_order_and_passthrough(orc):
    raw = _small()
    buf = artifact.write_matrix_raw(raw)
    # field order and widths, by hand
    name = raw.name.encode()
    pos = 0
    assert struct.unpack_from("<I", buf, pos)[0] == len(name)
    pos += 4 + len(name)
    assert struct.unpack_from("<IIIIQI", buf, pos) == (3, 53, 12, 2, 0, 0)
    pos += 28
    assert np.frombuffer(buf, "<f8", 2, pos).tolist() == [0.8, 1.25]
    pos += 16
    assert np.array_equal(np.frombuffer(buf, "<f8", 3, pos), raw.row_scales)
    pos += 24
    assert np.array_equal(np.frombuffer(buf, "<f4", 3 * 5, pos), raw.tail)
    pos += 60
    assert struct.unpack_from("<Q", buf, pos)[0] == 3 * 2 * 6
    assert len(buf) == pos + 8 + 36
    # oracle reads it, and writes back the same bytes (g6_format.rs:233-262)
    m, end = orc.read_matrix_raw(buf)
    assert end == len(buf) and m.name == raw.name
    assert m.write() == buf
    idx, g = raw.unpack()
    assert np.array_equal(m.indices(), idx) and np.array_equal(m.gains(), g)
    assert np.array_equal(m.row_scales(), raw.row_scales) and np.array_equal(m.tail(), raw.tail.astype(np.float64))
    # and the Python mirror reads what it wrote
    r2, end2 = artifact.read_matrix_raw(buf)
    assert end2 == len(buf) and r2.codes.tobytes() == raw.codes.tobytes() and r2.rotation_seed is None


def test_header_versions(orc):
    for v, n in ((1, 8), (2, 8), (3, 8), (4, 16)):
        h = orc.write_header(v, 7)
        assert len(h) == n and h == artifact.write_header(v, 7)
        assert orc.read_header(h) == (v, 7, n)
        assert artifact.read_header(h) == (v, 7, n)
    assert orc.write_header(4, 1)[8:] == struct.pack("<Q", 0x338F420F11866319)
    bad = bytearray(orc.write_header(4, 1))
    bad[8] ^= 1
    with pytest.raises(orc.OracleError) as e:
        orc.read_header(bytes(bad))
    assert e.value.kind == "CodebookMismatch"
    with pytest.raises(artifact.CodebookMismatch):
        artifact.read_header(bytes(bad))


def _hostile_cases():
    """(bytes, reader, expected kind, expected `reading`) — llvq-artifact/tests/hostile_files.rs:45-214."""
    one = artifact.RawMatrix("model.layers.0.self_attn.q_proj.weight", 1, 48, 12, [1.0], [1.0], [],
                             np.frombuffer(bytes(12), np.uint8))  # 2 blocks x 47 bits = 12 bytes
    rec = artifact.write_matrix_raw(one)
    cases = []
    cases.append((bytes([0xDE, 0xAD, 0xBE, 0xEF, 0, 0, 0, 0]), "header", "NotAnArtifact", None))
    cases.append((b"", "header", "Truncated", "magic"))
    cases.append((artifact.write_header(4, 7)[:6], "header", "Truncated", "matrix count"))
    cases.append((rec[:9], "matrix", "Truncated", "name"))
    cases.append((struct.pack("<I", 0xFFFFFFFF) + b"abc", "matrix", "Truncated", "name"))
    cases.append((struct.pack("<I", 2) + bytes([0xFF, 0xFE]), "matrix", "BadName", None))
    at = 4 + len(one.name) + 8
    cases.append((rec[:at] + struct.pack("<I", 0xFFFF) + rec[at + 4:], "matrix", "Inconsistent", None))
    at = len(rec) - 12 - 8
    cases.append((rec[:at] + struct.pack("<Q", 2 ** 64 - 1) + rec[at + 8:], "matrix", "Truncated", "code stream"))
    cases.append((rec[:at] + struct.pack("<Q", 1) + rec[at + 8:at + 9], "matrix", "Truncated", "code stream"))
    return cases


def test_hostile_files_are_errors_never_crashes(orc):
    for buf, what, kind, reading in _hostile_cases():
        with pytest.raises(orc.OracleError) as e:
            (orc.read_header if what == "header" else orc.read_matrix_raw)(buf)
        assert e.value.kind == kind, (kind, e.value)
        if reading:
            assert e.value.what == reading
        # the Python mirror refuses the same files the same way
        with pytest.raises(artifact.ArtifactError) as e2:
            (artifact.read_header if what == "header" else artifact.read_matrix_raw)(buf)
        assert type(e2.value).__name__ == kind
        if reading:
            assert e2.value.reading == reading


def test_index_too_wide_is_refused_by_the_writer(orc):
    with pytest.raises(artifact.IndexTooWide):
        artifact.pack_codes(np.array([1, 1 << 47], np.uint64), np.array([0, 0]))
    m, _ = orc.read_matrix_raw(artifact.write_matrix_raw(_small()))
    m.c.indices[1] = 1 << 47
    with pytest.raises(orc.OracleError) as e:
        m.write()
    assert e.value.kind == "IndexTooWide"


def test_every_stored_field_is_load_bearing(orc):
    """g6_format.rs:151-189: corrupting any stored field moves the reconstruction."""
    raw = _small(d_out=4, d_in=77, seed=9)
    base = orc.read_matrix_raw(artifact.write_matrix_raw(raw))[0].decode_matrix()

    def decoded(**kw):
        f = dict(name=raw.name, d_out=raw.d_out, d_in=raw.d_in, shell_cap=12, centroids=raw.centroids.copy(),
                 row_scales=raw.row_scales.copy(), tail=raw.tail.copy(), codes=raw.codes.copy())
        f.update(kw)
        return orc.read_matrix_raw(artifact.write_matrix_raw(artifact.RawMatrix(**f)))[0].decode_matrix()

    c = raw.centroids.copy(); c[1] *= 1.5
    rs = raw.row_scales.copy(); rs[2] *= 2
    tl = raw.tail.copy(); tl[3] += 1
    idx, g = raw.unpack()
    i2 = idx.copy(); i2[5] = (i2[5] + 12345) % np.uint64(orc.N12)
    g2 = g.copy(); g2[7] ^= 1
    for changed in (decoded(centroids=c), decoded(row_scales=rs), decoded(tail=tl),
                    decoded(codes=artifact.pack_codes(i2, g)), decoded(codes=artifact.pack_codes(idx, g2))):
        assert not np.array_equal(changed, base)
    assert np.array_equal(decoded(), base)


# ---- numerics -------------------------------------------------------------------------------
def test_reconstruct_closed_form(orc):
    """quantizer.rs:354-367: centroid * row_scale / sqrt(16 m) * p, in f64, in that order."""
    raw = _small(d_out=2, d_in=48, seed=3)
    m, _ = orc.read_matrix_raw(artifact.write_matrix_raw(raw))
    w = m.decode_matrix()
    idx, g = raw.unpack()
    pts = orc.decode_many(idx)
    for r in range(2):
        for b in range(2):
            p = pts[r * 2 + b].astype(np.float64)
            shell = int((p ** 2).sum()) // 16
            picked = raw.centroids[g[r * 2 + b]] * raw.row_scales[r]
            expect = (p * (picked / np.sqrt(np.float64(16 * shell)))).astype(np.float32) if shell else np.zeros(24, np.float32)
            assert np.array_equal(w[r, 24 * b:24 * b + 24], expect)


def test_dense_equals_fused(orc):
    """llvq-artifact/tests/fused_path_matches_dense.rs:140-175, natural basis: 1e-6 of sum |w x|."""
    for d_out, d_in, seed in ((8, 240, 0x11), (8, 2560, 0x22), (16, 9728, 0x33), (8, 4096, 0x44), (24, 96, 0x55)):
        raw = synth.make_matrix(f"test.{d_out}x{d_in}", d_out, d_in, seed=seed, index_bound=1 << 47)
        m, _ = orc.read_matrix_raw(artifact.write_matrix_raw(raw))
        x = synth.SplitMix64(seed ^ 0xA11CE).gaussian(d_in)
        dense = orc.dense_matvec(m.decode_matrix(), x)
        fused, scale = m.fused_product(x)
        assert (np.abs(dense - fused) / np.maximum(scale, 1e-12)).max() < 1e-6


def test_f16_conversions_exhaustive(orc):
    L = orc.lib()
    bits = np.arange(65536, dtype=np.uint16)
    ref = bits.view(np.float16).astype(np.float32)
    got = np.array([L.orc_f16_to_f32(int(b)) for b in bits], np.float32)
    nan = np.isnan(ref)
    assert np.array_equal(got[~nan], ref[~nan]) and np.isnan(got[nan]).all()
    # narrowing: every f16 value round-trips, and midpoints / neighbours round to nearest even like numpy
    back = np.array([L.orc_f32_to_f16(float(v)) for v in ref[~nan]], np.uint16)
    assert np.array_equal(back, bits[~nan])
    rng = synth.SplitMix64(16)
    f = (rng.gaussian(20000) * np.exp(rng.gaussian(20000) * 6)).astype(np.float32)
    f = np.concatenate([f, np.array([65504, 65519.99, 65520, 1e-8, 5.96e-8, 2.98e-8, 2.9802322e-8, -0.0, 6.1e-5], np.float32)])
    with np.errstate(over="ignore"):
        expect = f.astype(np.float16).view(np.uint16)
    got = np.array([L.orc_f32_to_f16(float(v)) for v in f], np.uint16)
    assert np.array_equal(got, expect)


def test_splitmix_vectors(orc):
    """Published SplitMix64 outputs for seed 0, and the vectorised generator against the C one."""
    import ctypes as C

    s = C.c_uint64(0)
    first = [orc.lib().orc_splitmix_next(C.byref(s)) for _ in range(3)]
    assert first == [0xE220A8397B1DCDAF, 0x6E789E6AA1B965F4, 0x06C45D188009454F]
    assert synth.SplitMix64(0).take(3).tolist() == first
    s = C.c_uint64(0xA4C0DE)
    g_c = np.array([orc.lib().orc_splitmix_gaussian(C.byref(s)) for _ in range(1000)])
    g_np = synth.SplitMix64(0xA4C0DE).gaussian(1000)
    assert np.allclose(g_c, g_np, rtol=1e-12, atol=1e-14)
    assert abs(g_np.mean()) < 0.1 and abs(g_np.std() - 1) < 0.1


def test_host_packer_follows_the_bit_writer_at_every_block_width(orc):
    """llvq_amd.artifact.pack_codes / RawMatrix.unpack against the oracle's bit writer (pack.rs:48-82) for blocks of
    3 bits (the reference's own known answer, g6_pack.rs:17-27: 101 011 110 -> AF 00), 48 bits (cap 12) and 49 bits
    (cap 13, the dense stream: 48 bits of index, format.rs:87-89), and a cap-13 record through both readers."""
    from llvq_amd import synth

    assert artifact.pack_codes([0b10, 0b01, 0b11], [1, 1, 0], index_width=2).tobytes() == bytes([0b10101111, 0])
    rng = np.random.default_rng(49)
    for width, bound in ((47, orc.N12 + 1), (48, orc.N13 + 1)):
        idx = rng.integers(0, bound, size=1001, dtype=np.uint64)
        idx[:3] = [0, bound - 1, 1]
        gains = rng.integers(0, 2, size=idx.size).astype(np.uint8)
        want = orc.pack_bits([f for i, g in zip(idx.tolist(), gains.tolist()) for f in ((i, width), (g, 1))])
        got = artifact.pack_codes(idx, gains, index_width=width)
        assert got.tobytes() == want and got.size == (idx.size * (width + 1) + 7) // 8
    assert artifact.index_bits(13) == 48 and orc.lib().orc_index_bits(13) == 48
    raw = synth.make_matrix("model.layers.0.cap13.weight", 9, 24 * 5 + 3, seed=2, shell_cap=13)
    assert raw.codes.size == (9 * 5 * 49 + 7) // 8
    blob = artifact.write_matrix_raw(raw)
    om, _ = orc.read_matrix_raw(blob)
    back, _ = artifact.read_matrix_raw(blob)
    idx, gains = back.unpack()
    assert np.array_equal(idx, om.indices().astype(np.uint64)) and np.array_equal(gains, om.gains().astype(np.uint8))
    assert int(idx.max()) <= orc.N13 and int(idx.max()) >= (1 << 47)  # the draw reaches shell 13's upper half
    assert om.write() == blob
