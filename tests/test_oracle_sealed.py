"""Pins of the sealed-section oracle (oracle/sealed_oracle.py) and of the host
mirror's reader/writer (llvq_amd/artifact.py) against the reference's own
vectors: llvq-artifact/tests/raw_tensors.rs and tests/hostile_files.rs:172-213."""
import struct

import numpy as np
import pytest

from llvq_amd import artifact
from oracle import sealed_oracle as S


def test_f16_widening_matches_hand_computed_values():  # raw_tensors.rs:20-40
    for bits, want in [(0x0000, 0.0), (0x3C00, 1.0), (0xC000, -2.0), (0x3555, 0.33325195), (0x7BFF, 65504.0),
                       (0x0400, 6.1035156e-5), (0x0001, 5.9604645e-8), (0x03FF, 6.097555e-5), (0x8001, -5.9604645e-8)]:
        assert S.f16_to_f32(bits).tobytes() == np.float32(want).tobytes(), hex(bits)
    assert S.f16_to_f32(0x8000) == 0.0 and np.signbit(S.f16_to_f32(0x8000))
    assert S.f16_to_f32(0x7C00) == np.inf and S.f16_to_f32(0xFC00) == -np.inf and np.isnan(S.f16_to_f32(0x7E00))
    # every pattern agrees with numpy's own widening
    allb = np.arange(65536, dtype=np.uint16)
    mine = np.array([S.f16_to_f32(b) for b in allb[::37]], np.float32)
    assert np.array_equal(mine.view(np.uint32), allb[::37].view(np.float16).astype(np.float32).view(np.uint32))


def _small_quant():  # raw_tensors.rs:66-78
    return artifact.RawTensor("model.embed_tokens.weight", [2, 5], bits=4, group=2,
                              packed=[0x10, 0x32, 0x54, 0x76, 0x98], scales=[0x3C00] * 6,
                              biases=[0x0000, 0x3C00, 0x4000, 0x4200, 0x4400, 0x4500])


def test_quant_decode_known_values():  # raw_tensors.rs:97-126
    t, _ = artifact.read_raw(artifact.write_raw(_small_quant()), 0, 3)
    o = S.read_raw(S.Cursor(artifact.write_raw(_small_quant())), 3)
    want = S.to_f32(o)
    # q = 0..9 in order; groups of 2 with a short last group per row: biases 0,0,1,1,2 | 3,3,4,4,5
    assert want.tolist() == [0, 1, 3, 4, 6, 8, 9, 11, 12, 14]
    assert want[0] == 0.0 and want[4] == 6.0 and want[5] == 8.0
    assert (t.bits, t.group) == (4, 2) and t.packed.tolist() == [0x10, 0x32, 0x54, 0x76, 0x98]
    assert np.array_equal(o["scales"], t.scales) and np.array_equal(o["biases"], t.biases)


def test_f16_tensor_round_trip_and_byte_layout():  # raw_tensors.rs:49-62
    t = artifact.RawTensor("model.norm.weight", [2, 3], data=[0x3C00, 0xC000, 0x0001, 0x7BFF, 0x0000, 0x8000])
    b = artifact.write_raw(t)
    # tag, name, rank, dims, count, data — written out by hand
    name = b"model.norm.weight"
    want = (struct.pack("<I", 0) + struct.pack("<I", len(name)) + name + struct.pack("<I", 2) + struct.pack("<QQ", 2, 3)
            + struct.pack("<Q", 6) + struct.pack("<6H", 0x3C00, 0xC000, 0x0001, 0x7BFF, 0x0000, 0x8000))
    assert b == want
    o = S.read_raw(S.Cursor(b), 3)
    assert o["name"] == t.name and o["dims"] == [2, 3] and o["data"].tolist() == t.data.tolist()
    back, pos = artifact.read_raw(b, 0, 3)
    assert pos == len(b) and back.data.tolist() == t.data.tolist()


def test_legacy_v2_record_still_reads():  # raw_tensors.rs:129-144
    b = struct.pack("<I", 1) + b"w" + struct.pack("<I", 1) + struct.pack("<Q", 3) + struct.pack("<Q", 3) + struct.pack(
        "<3H", 0x3C00, 0xC000, 0x7BFF)
    for got in (S.read_raw(S.Cursor(b), 2), vars(artifact.read_raw(b, 0, 2)[0])):
        assert got["name"] == "w" and got["dims"] == [3]
    assert S.to_f32(S.read_raw(S.Cursor(b), 2)).tolist() == [1.0, -2.0, 65504.0]


def test_unknown_tag_is_refused_before_anything_else():  # hostile_files.rs:172-181, raw_tensors.rs:147-158
    b = struct.pack("<I", 99) + bytes(32)
    with pytest.raises(S.OracleSealedError) as e:
        S.read_raw(S.Cursor(b), 3)
    assert e.value.kind == "BadRawEncoding" and e.value.what == 99
    with pytest.raises(artifact.BadRawEncoding) as e2:
        artifact.read_raw(b, 0, 3)
    assert e2.value.tag == 99 and "encoding tag 99" in str(e2.value)


def test_lying_lengths_are_truncations():  # hostile_files.rs:184-213
    b = struct.pack("<I", 0) + struct.pack("<I", 1) + b"t" + struct.pack("<I", 1) + struct.pack("<Q", 4) + struct.pack(
        "<Q", 2 ** 64 - 1)
    with pytest.raises(S.OracleSealedError) as e:
        S.read_raw(S.Cursor(b), 3)
    assert (e.value.kind, e.value.what) == ("Truncated", "raw tensor data")
    with pytest.raises(artifact.Truncated) as e2:
        artifact.read_raw(b, 0, 3)
    assert e2.value.reading == "raw tensor data"
    blob = struct.pack("<I", 1) + b"b" + struct.pack("<Q", 2 ** 64 - 1)
    with pytest.raises(S.OracleSealedError) as e:
        S.read_blob(S.Cursor(blob))
    assert (e.value.kind, e.value.what) == ("Truncated", "blob")
    with pytest.raises(artifact.Truncated) as e2:
        artifact.read_blob(blob)
    assert e2.value.reading == "blob"


def test_inconsistent_quant_payloads_are_refused_by_the_writer():  # raw_tensors.rs:161-170
    t = _small_quant()
    t.scales = t.scales[:-1]
    with pytest.raises(artifact.Inconsistent):
        artifact.write_raw(t)


def test_sealed_file_round_trip():
    from llvq_amd import synth

    m = synth.make_matrix("model.layers.0.self_attn.q_proj.weight", 8, 48, seed=1)
    raws = [artifact.RawTensor("model.norm.weight", [48], data=np.arange(48, dtype=np.uint16) + 0x3C00), _small_quant()]
    blobs = [artifact.Blob("config.json", b'{"hidden_size": 48}'), artifact.Blob("tokenizer.json", b"{}")]
    buf = artifact.write_file([m], version=4, raws=raws, blobs=blobs)
    version, mats, r2, b2 = artifact.read_sealed(buf)
    assert version == 4 and len(mats) == 1 and mats[0].name == m.name
    assert [t.name for t in r2] == [t.name for t in raws] and r2[1].packed.tolist() == raws[1].packed.tolist()
    assert [(b.name, b.data) for b in b2] == [(b.name, b.data) for b in blobs]
    # a file that ends after the matrices is a truncation, not an empty model
    cut = buf[: len(artifact.write_header(4, 1)) + len(artifact.write_matrix_raw(m))]
    with pytest.raises(artifact.Truncated):
        artifact.read_sealed(cut)


def test_int8_writer_follows_the_reference_writer_on_hand_computed_groups():  # embedquant.rs:22-92
    """Four groups of four whose bytes can be worked out by hand.  (1) min -8, max 55.75: the scale is exactly
    0.25, so -7.375 sits at quotient 2.5 and must code as 3 (half away from zero; half-to-even would say 2),
    -7.125 at 3.5 codes as 4.  (2) a constant group: scale 1.0, codes 0, the bias carries the value.  (3) a
    range that rounds to zero in binary16 (two neighbouring subnormals): ungraded like the constant one.
    (4) min 0, max 255: scale 1, codes are the values."""
    from llvq_amd import decoder

    rows = np.array([[-8.0, -7.375, -7.125, 55.75, 3.0, 3.0, 3.0, 3.0, 0.0, 2.0 ** -24, 0.0, 2.0 ** -24, 0.0, 7.0, 255.0, 100.0]],
                    dtype=np.float16)
    t = decoder.quantize_rows_q8("model.embed_tokens.weight", rows, group=4)
    assert (t.bits, t.group, list(t.dims)) == (8, 4, [1, 16])
    assert np.asarray(t.packed).tolist() == [0, 3, 4, 255, 0, 0, 0, 0, 0, 0, 0, 0, 0, 7, 255, 100]
    assert np.asarray(t.scales).tolist() == [0x3400, 0x3C00, 0x3C00, 0x3C00]  # 0.25, 1, 1, 1
    assert np.asarray(t.biases).tolist() == [0xC800, 0x4200, 0x0000, 0x0000]  # -8, 3, 0, 0
