"""The shipped library without a GPU: exported symbols, its own codebook tables
and host decoder (the arithmetic the kernels run), its record reader."""
import ctypes as C
import os
import re
import struct

import numpy as np
import pytest

from llvq_amd import _ffi, artifact, synth

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_every_declared_symbol_is_exported():
    hdr = open(os.path.join(ROOT, "include", "llvq_hip.h")).read()
    declared = sorted(set(re.findall(r"\b(llvq_hip_[a-z_0-9]+)\s*\(", hdr)))
    assert declared == sorted(_ffi.EXPORTS)
    L = _ffi.lib()
    for name in declared:
        assert hasattr(L, name), name


def test_library_fingerprint_is_the_published_one():
    assert _ffi.lib().llvq_hip_codebook_fingerprint() == 0x338F420F11866319


def _host_decode(indices):
    L = _ffi.lib()
    out = np.zeros((len(indices), 24), np.int8)
    shells = np.zeros(len(indices), np.int32)
    s = C.c_int()
    for k, i in enumerate(indices):
        assert L.llvq_hip_host_decode(int(i), out[k].ctypes.data, C.byref(s)) == 1
        shells[k] = s.value
    return out, shells


def test_host_decoder_matches_oracle_on_boundaries_and_draws(orc, boundary_indices):
    """The library's decoder (table-driven even coset, FP64 walk of the odd coset) against
    the reference algorithm restated in the oracle: every class boundary, 60 000 draws."""
    got, shells = _host_decode(boundary_indices)
    ref = orc.decode_many(boundary_indices, fast=False)
    assert np.array_equal(got, ref)
    assert np.array_equal(shells, (ref.astype(np.int64) ** 2).sum(1) // 16)
    idx = synth.SplitMix64(0xBEEF).take(60_000) % np.uint64(orc.N13 + 1)
    assert np.array_equal(_host_decode(idx)[0], orc.decode_many(idx))
    out = np.zeros(24, np.int8)
    assert _ffi.lib().llvq_hip_host_decode(orc.N13 + 1, out.ctypes.data, None) == 0


def test_host_decoder_dense_sweep_of_small_classes(orc):
    """Consecutive indices across the first classes (every arrangement and sign pattern of
    shells 2 and 3's small classes), where a mixed-radix slip would show at once."""
    idx = np.arange(0, 120_000, dtype=np.uint64)
    assert np.array_equal(_host_decode(idx)[0], orc.decode_many(idx))


def test_record_reader_happy_path_and_hostile_files():
    L = _ffi.lib()
    raw = synth.make_matrix("model.layers.3.mlp.up_proj.weight", 4, 77, seed=2)
    buf = artifact.write_file([raw], version=4)
    pos = C.c_size_t(0)
    ver, n = C.c_uint32(), C.c_uint32()
    assert L.llvq_hip_read_header(buf, len(buf), C.byref(pos), C.byref(ver), C.byref(n)) == 0
    assert (ver.value, n.value, pos.value) == (4, 1, 16)
    info = _ffi.RecordInfo()
    assert L.llvq_hip_parse_matrix_record(buf, len(buf), C.byref(pos), C.byref(info)) == 0
    assert info.name.decode() == raw.name and (info.d_out, info.d_in, info.shell_cap, info.n_centroids) == (4, 77, 12, 2)
    assert buf[info.codes_off:info.codes_off + info.code_bytes] == raw.codes.tobytes()
    assert np.array_equal(np.frombuffer(buf, "<f8", 4, info.row_scales_off), raw.row_scales)
    assert pos.value == len(buf) - 8

    from test_oracle_format import _hostile_cases

    kinds = {"NotAnArtifact": 1, "Truncated": 2, "BadName": 3, "Inconsistent": 5}
    for hbuf, what, kind, reading in _hostile_cases():
        pos = C.c_size_t(0)
        if what == "header":
            rc = L.llvq_hip_read_header(hbuf, len(hbuf), C.byref(pos), C.byref(ver), C.byref(n))
        else:
            rc = L.llvq_hip_parse_matrix_record(hbuf, len(hbuf), C.byref(pos), C.byref(info))
        assert rc == kinds[kind], (kind, rc)
        msg = L.llvq_hip_last_error().decode()
        if reading:
            assert msg == f"file ends mid-{reading}"
        if kind == "Inconsistent":
            assert "shell cap 65535" in msg
    bad = bytearray(artifact.write_header(4, 1))
    bad[9] ^= 0x40
    pos = C.c_size_t(0)
    assert L.llvq_hip_read_header(bytes(bad), len(bad), C.byref(pos), C.byref(ver), C.byref(n)) == 10


def test_python_operator_refusals():
    from llvq_amd.fused import FusedMatrix

    raw = synth.make_matrix("model.layers.0.mlp.gate_proj.weight", 2, 48, seed=1)
    three = artifact.RawMatrix(raw.name, 2, 48, 12, [0.5, 1.0, 1.5], raw.row_scales, raw.tail, raw.codes)
    with pytest.raises(ValueError, match="3 centroids"):
        FusedMatrix(three)
    assert artifact.split_name("model.layers.17.self_attn.q_proj.weight") == (17, "self_attn.q_proj")
    with pytest.raises(artifact.ArtifactError):
        artifact.split_name("lm_head.weight")


def test_synthetic_configs():
    raw = synth.make_matrix("model.layers.0.self_attn.k_proj.weight", 8, 2560, seed=0)
    assert raw.nblocks == 106 and raw.tail_w == 16 and raw.codes.size == 8 * 106 * 6
    idx, g = raw.unpack()
    assert int(idx.max()) <= artifact.N12 and set(np.unique(g)) <= {0, 1}
    assert raw.encoded_bytes() == 8 * 106 * 6 + 8 * 16 * 4 + 8 * 8 + 16
    # BASELINE byte counts: config 0 = 6 887 440, one layer = 27 243 632
    shapes = {n: (o, i) for n, o, i in synth.QWEN3_4B_LAYER}
    total = sum(6 * o * (i // 24) + 4 * o * (i % 24) + 8 * o + 16 for o, i in shapes.values())
    assert total == 27_243_632
    o, i = shapes["mlp.gate_proj"]
    assert 6 * o * (i // 24) + 4 * o * (i % 24) + 8 * o + 16 == 6_887_440
    x = synth.make_activation(2560, 0)
    assert x.dtype == np.float16 and x.shape == (1, 2560)


# ---- rotation tables (fused.rs:1272-1331: "the tables describe the rotation") -------------
def test_rotation_tables_describe_the_rotation(orc):
    import ctypes as C

    from llvq_amd import _ffi
    from llvq_amd.synth import SplitMix64

    L = _ffi.lib()
    for n, seed in [(240, 1), (2560, 2), (9728, 3), (4096, 4), (96, 5)]:  # fused.rs:1274
        x = SplitMix64(seed ^ 0xF00D).gaussian(n)
        got = x.copy()
        _ffi.check(L.llvq_hip_host_rotate(n, seed, got.ctypes.data))
        want = orc.Rotation(n, seed).apply(x)
        dev = np.linalg.norm(got - want) / np.linalg.norm(want)
        assert dev < 1e-6, f"n={n}: relative deviation {dev:.3e}"  # the reference's own threshold
        assert abs(np.linalg.norm(got) / np.linalg.norm(x) - 1) < 1e-6  # 1/sqrt m, not 1/sqrt n


def test_rotation_with_a_wide_odd_factor_is_refused():
    from llvq_amd import LlvqError, _ffi

    v = np.zeros(33 * 8)
    with pytest.raises(LlvqError) as e:  # k = 33 > 32 (fused.rs:698-704)
        _ffi.check(_ffi.lib().llvq_hip_host_rotate(33 * 8, 1, v.ctypes.data))
    assert e.value.kind == "Unsupported" and "33" in str(e.value)


# ---- sealed sections through the library's own reader (sealed.rs:277-341) ----------------
def _parse_raw(buf, pos=0, version=3):
    info = _ffi.RawInfo()
    p = C.c_size_t(pos)
    _ffi.check(_ffi.lib().llvq_hip_parse_raw_tensor(bytes(buf), len(buf), C.byref(p), version, C.byref(info)))
    return info, p.value


def test_library_reads_raw_tensors_and_blobs():
    q = artifact.RawTensor("model.embed_tokens.weight", [2, 5], bits=4, group=2, packed=[0x10, 0x32, 0x54, 0x76, 0x98],
                           scales=[0x3C00] * 6, biases=[0x0000, 0x3C00, 0x4000, 0x4200, 0x4400, 0x4500])  # raw_tensors.rs:66-78
    f = artifact.RawTensor("model.norm.weight", [2, 3], data=[0x3C00, 0xC000, 0x0001, 0x7BFF, 0x0000, 0x8000])
    buf = artifact.write_raw(f) + artifact.write_raw(q) + artifact.write_blob(artifact.Blob("config.json", b"{}"))
    a, pos = _parse_raw(buf)
    assert a.name == b"model.norm.weight" and a.tag == 0 and a.rank == 2 and list(a.dims[:2]) == [2, 3] and a.count == 6
    assert np.frombuffer(buf, "<u2", 6, a.data_off).tolist() == f.data.tolist() and a.data_len == 12
    b, pos = _parse_raw(buf, pos)
    assert b.name == b"model.embed_tokens.weight" and (b.tag, b.bits, b.group, b.count) == (1, 4, 2, 6)
    assert buf[b.data_off:b.data_off + b.data_len] == bytes(q.packed)
    assert np.frombuffer(buf, "<u2", 6, b.biases_off).tolist() == q.biases.tolist()
    assert np.frombuffer(buf, "<u2", 6, b.scales_off).tolist() == q.scales.tolist()
    blob = _ffi.BlobInfo()
    p = C.c_size_t(pos)
    _ffi.check(_ffi.lib().llvq_hip_parse_blob(buf, len(buf), C.byref(p), C.byref(blob)))
    assert blob.name == b"config.json" and buf[blob.data_off:blob.data_off + blob.data_len] == b"{}" and p.value == len(buf)
    # legacy record: no tag below version 3 (raw_tensors.rs:129-144)
    legacy = struct.pack("<I", 1) + b"w" + struct.pack("<I", 1) + struct.pack("<Q", 3) + struct.pack("<Q", 3) + struct.pack(
        "<3H", 0x3C00, 0xC000, 0x7BFF)
    c, pos = _parse_raw(legacy, 0, 2)
    assert c.name == b"w" and c.tag == 0 and c.count == 3 and pos == len(legacy)


def test_library_refuses_hostile_sealed_sections():
    from llvq_amd import LlvqError

    with pytest.raises(LlvqError) as e:  # hostile_files.rs:172-181
        _parse_raw(struct.pack("<I", 99) + bytes(32))
    assert e.value.kind == "BadRawEncoding" and "encoding tag 99" in str(e.value)
    lying = struct.pack("<I", 0) + struct.pack("<I", 1) + b"t" + struct.pack("<I", 1) + struct.pack("<Q", 4) + struct.pack(
        "<Q", 2 ** 64 - 1)
    with pytest.raises(LlvqError) as e:  # hostile_files.rs:184-200
        _parse_raw(lying)
    assert e.value.kind == "Truncated" and "raw tensor data" in str(e.value)
    blob = struct.pack("<I", 1) + b"b" + struct.pack("<Q", 2 ** 64 - 1)
    info = _ffi.BlobInfo()
    p = C.c_size_t(0)
    with pytest.raises(LlvqError) as e:  # hostile_files.rs:203-213
        _ffi.check(_ffi.lib().llvq_hip_parse_blob(blob, len(blob), C.byref(p), C.byref(info)))
    assert e.value.kind == "Truncated" and str(e.value).endswith("mid-blob")
    with pytest.raises(LlvqError) as e:
        _parse_raw(struct.pack("<I", 0) + struct.pack("<I", 2) + b"\xff\xfe" + bytes(16))
    assert e.value.kind == "BadName"
    # every prefix of an honest record is a truncation, never a crash
    honest = artifact.write_raw(artifact.RawTensor("t", [3], data=[1, 2, 3]))
    for cut in range(len(honest)):
        with pytest.raises(LlvqError) as e:
            _parse_raw(honest[:cut])
        assert e.value.kind == "Truncated"


def test_header_is_plain_c_and_matches_the_python_mirror(tmp_path):
    """include/llvq_hip.h compiles as C99 (the boundary is a C ABI, not a C++ one), a C caller links and
    runs the host-only entry points, and the structs have the layout the ctypes mirror assumes."""
    import subprocess

    src = tmp_path / "abi.c"
    src.write_text(r'''
#include <stddef.h>
#include <stdio.h>
#include "llvq_hip.h"
int main(void) {
  signed char pt[24];
  int shell = 0;
  if (llvq_hip_codebook_fingerprint() != 0x338f420f11866319ULL) return 3;
  if (llvq_hip_host_decode(1, pt, &shell) != 1 || shell != 2) return 4;
  printf("%zu %zu %zu %zu %zu %zu %zu\n", sizeof(llvq_matrix_desc), sizeof(llvq_decoder_desc), sizeof(llvq_quant_rows),
         sizeof(llvq_raw_info), sizeof(llvq_blob_info), offsetof(llvq_decoder_desc, kv_mode), offsetof(llvq_decoder_desc, prefill_rows));
  return 0;
}
''')
    exe = tmp_path / "abi"
    libdir = os.path.dirname(_ffi.lib_path())
    cmd = ["gcc", "-std=c99", "-Wall", "-Wextra", "-Werror", "-pedantic", "-I", os.path.join(ROOT, "include"), str(src),
           "-o", str(exe), "-L", libdir, "-lllvq_hip", "-Wl,-rpath," + libdir, "-Wl,-rpath,/opt/rocm/lib"]
    built = subprocess.run(cmd, capture_output=True, text=True)
    assert built.returncode == 0, built.stderr[-2000:]
    run = subprocess.run([str(exe)], capture_output=True, text=True, timeout=120)
    assert run.returncode == 0, (run.returncode, run.stderr[-500:])
    got = [int(v) for v in run.stdout.split()]
    want = [C.sizeof(_ffi.MatrixDesc), C.sizeof(_ffi.DecoderDesc), C.sizeof(_ffi.QuantRows), C.sizeof(_ffi.RawInfo),
            C.sizeof(_ffi.BlobInfo), _ffi.DecoderDesc.kv_mode.offset, _ffi.DecoderDesc.prefill_rows.offset]
    assert got == want


def test_output_dtype_is_checked():
    """Outputs are binary16 or f32; anything else (bfloat16: two bytes written as four) is refused
    before a kernel sees the pointer."""
    import torch

    from llvq_amd import _ffi, fused

    rt = fused.FusedRuntime.__new__(fused.FusedRuntime)
    rt._torch, rt.handle, rt.projs = torch, None, []
    assert rt._out_code(torch.float16) == _ffi.F16
    assert rt._out_code(torch.float32) == _ffi.F32
    for bad in (torch.bfloat16, torch.float64, torch.int8):
        with pytest.raises(ValueError):
            rt._out_code(bad)


def _c_prototypes():
    """name -> (return type, [argument types]) of every function include/llvq_hip.h declares, types
    normalised to a small vocabulary shared with the Rust side."""
    import re

    text = open(os.path.join(ROOT, "include", "llvq_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", " ", text, flags=re.S)
    text = re.sub(r"^\s*#.*$", " ", text, flags=re.M)
    protos = {}
    for ret, name, args in re.findall(r"([A-Za-z_][\w \*]*?)\s*\b(llvq_hip_\w+)\s*\(([^;{}]*?)\)\s*;", text):
        protos[name] = (_c_type(ret), [] if args.strip() in ("", "void") else [_c_type(a) for a in args.split(",")])
    return protos


def _c_type(decl):
    import re

    d = decl.strip()
    d = re.sub(r"\[\d*\]\s*$", "*", d)                 # int8_t point[24] -> pointer
    if "*" not in d or d.endswith("*"):
        pass
    stars = d.count("*")
    base = d.replace("*", " ")
    words = [w for w in base.split() if w not in ("const", "struct")]
    # drop the parameter name, if there is one
    known = {"void", "int", "char", "float", "double", "size_t", "uint8_t", "int8_t", "uint16_t", "uint32_t", "uint64_t",
             "llvq_rt", "llvq_mat", "llvq_decoder", "llvq_matrix_desc", "llvq_record_info", "llvq_raw_info", "llvq_blob_info",
             "llvq_decoder_desc", "llvq_seq", "llvq_seq_item"}
    if len(words) > 1 and words[-1] not in known:
        words = words[:-1]
    ctype = " ".join(words)
    table = {"int": "c_int", "char": "c_char", "float": "f32", "double": "f64", "size_t": "usize", "uint8_t": "u8", "int8_t": "i8",
             "uint16_t": "u16", "uint32_t": "u32", "uint64_t": "u64", "void": "c_void", "llvq_rt": "LlvqRt", "llvq_mat": "LlvqMat",
             "llvq_decoder": "LlvqDecoder", "llvq_matrix_desc": "LlvqMatrixDesc", "llvq_record_info": "LlvqRecordInfo",
             "llvq_raw_info": "LlvqRawInfo", "llvq_blob_info": "LlvqBlobInfo", "llvq_decoder_desc": "LlvqDecoderDesc",
             "llvq_seq": "LlvqSeq", "llvq_seq_item": "LlvqSeqItem"}
    return table[ctype] + "*" * stars if stars else ("()" if ctype == "void" else table[ctype])


def _rust_prototypes():
    import re

    text = open(os.path.join(ROOT, "llvq-hip", "src", "lib.rs")).read()
    block = re.search(r'extern\s+"C"\s*\{(.*?)\n\}', text, flags=re.S).group(1)
    protos = {}
    for name, args, ret in re.findall(r"fn\s+(llvq_hip_\w+)\s*\(([^)]*)\)\s*(?:->\s*([^;]+))?;", block):
        types = []
        for a in [a for a in args.split(",") if a.strip()]:
            t = a.split(":", 1)[1].strip()
            stars = len(re.findall(r"\*(?:const|mut)", t))
            base = re.sub(r"\*(?:const|mut)\s*", "", t).strip()
            types.append(base + "*" * stars)
        r = (ret or "()").strip()
        stars = len(re.findall(r"\*(?:const|mut)", r))
        protos[name] = (re.sub(r"\*(?:const|mut)\s*", "", r).strip() + "*" * stars, types)
    return protos


def test_rust_crate_declares_the_header():
    """llvq-hip/src/lib.rs (source only: there is no Rust toolchain to build it with here) binds every
    function of include/llvq_hip.h with the header's argument and return types, and nothing else; the
    ctypes mirror exports the same set."""
    c, rust = _c_prototypes(), _rust_prototypes()
    assert set(c) == set(rust), (sorted(set(c) - set(rust)), sorted(set(rust) - set(c)))
    for name in sorted(c):
        assert c[name] == rust[name], f"{name}: header {c[name]}, crate {rust[name]}"
    assert set(_ffi.EXPORTS) == set(c), (sorted(set(c) - set(_ffi.EXPORTS)), sorted(set(_ffi.EXPORTS) - set(c)))
    for name in c:
        assert hasattr(_ffi.lib(), name)
    # the crate's repr(C) mirror of the one struct a Rust caller fills in field by field
    text = open(os.path.join(ROOT, "llvq-hip", "src", "lib.rs")).read()
    assert "pub const STATIC_SCRATCH_BYTES: usize = 64 << 20;" in text and _ffi.STATIC_SCRATCH_BYTES == 64 << 20
