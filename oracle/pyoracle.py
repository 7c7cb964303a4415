"""ctypes view of the CPU oracle (oracle/liboracle.so).  TEST INFRASTRUCTURE ONLY.

Imported by tests/, by the smoke test and by the benchmark's CPU-baseline leg;
the shipped package never imports it.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")
DIM = 24
N13 = 280974212784720
N12 = 111043117458000

ERR = {
    0: "Ok", 1: "NotAnArtifact", 2: "Truncated", 3: "BadName", 4: "UnexpectedName",
    5: "Inconsistent", 6: "PointOutsideCodebook", 7: "IndexTooWide", 8: "IndexOutOfRange",
    9: "BadRawEncoding", 10: "CodebookMismatch", 11: "UnknownVersion", 12: "Io",
}


def build():
    subprocess.check_call(["make", "-s", "-C", _HERE, "liboracle.so"])


class RawMatrixC(C.Structure):
    _fields_ = [
        ("name", C.c_char_p),
        ("d_out", C.c_uint32), ("d_in", C.c_uint32), ("shell_cap", C.c_uint32),
        ("n_centroids", C.c_uint32),
        ("rot_seed", C.c_uint64), ("has_rot", C.c_uint32),
        ("centroids", C.POINTER(C.c_double)),
        ("row_scales", C.POINTER(C.c_double)),
        ("tail", C.POINTER(C.c_double)),
        ("indices", C.POINTER(C.c_uint64)),
        ("gains", C.POINTER(C.c_uint32)),
        ("nblocks_total", C.c_size_t),
        ("code_off", C.c_size_t), ("code_len", C.c_size_t),
    ]


_lib = None


class RotationC(C.Structure):
    _fields_ = [("n", C.c_size_t), ("m", C.c_size_t), ("k", C.c_size_t),
                ("signs", C.POINTER(C.c_double)), ("small", C.POINTER(C.c_double))]


class Rotation:
    """llvq-quant/src/rotation.rs: Rotation::new(n, seed), apply, apply_transpose."""

    def __init__(self, n, seed):
        self.c = RotationC()
        rc = lib().orc_rotation_new(int(n), int(seed), C.byref(self.c))
        if rc:
            raise OracleError(rc)
        self.n, self.m, self.k = self.c.n, self.c.m, self.c.k
        self.signs = np.ctypeslib.as_array(self.c.signs, shape=(self.n,)).copy()
        self.small = np.ctypeslib.as_array(self.c.small, shape=(self.k, self.k)).copy()

    def apply(self, v):
        v = np.array(v, dtype=np.float64)
        assert v.size == self.n
        lib().orc_rotation_apply(C.byref(self.c), v.ctypes.data_as(C.POINTER(C.c_double)))
        return v

    def apply_transpose(self, v):
        v = np.array(v, dtype=np.float64)
        assert v.size == self.n
        lib().orc_rotation_apply_transpose(C.byref(self.c), v.ctypes.data_as(C.POINTER(C.c_double)))
        return v

    def __del__(self):
        try:
            lib().orc_rotation_free(C.byref(self.c))
        except Exception:
            pass


def lib():
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(_LIB_PATH):
        build()
    L = C.CDLL(_LIB_PATH)
    i32p = C.POINTER(C.c_int32)
    u8p = C.POINTER(C.c_uint8)
    L.orc_clmul.restype = C.c_uint64
    L.orc_clmul.argtypes = [C.c_uint64, C.c_uint64]
    L.orc_golay_codewords.restype = C.POINTER(C.c_uint32)
    L.orc_golay_of_weight.argtypes = [C.c_int, C.POINTER(C.POINTER(C.c_uint32))]
    L.orc_golay_contains.argtypes = [C.c_uint32]
    L.orc_leech_contains.argtypes = [i32p]
    L.orc_shell_index.restype = C.c_int64
    L.orc_shell_index.argtypes = [i32p]
    L.orc_enumerate_shell.restype = C.c_size_t
    L.orc_enumerate_shell.argtypes = [C.c_int, i32p, C.c_size_t]
    L.orc_shell_roundtrip_check.restype = C.c_longlong
    L.orc_shell_roundtrip_check.argtypes = [C.c_int, C.c_size_t, C.c_uint64, C.c_uint64]
    for f in (L.orc_splitmix_next,):
        f.restype = C.c_uint64
        f.argtypes = [C.POINTER(C.c_uint64)]
    for f in (L.orc_splitmix_f64, L.orc_splitmix_gaussian):
        f.restype = C.c_double
        f.argtypes = [C.POINTER(C.c_uint64)]
    L.orc_class_info.argtypes = [C.c_int, C.POINTER(C.c_uint64), C.POINTER(C.c_uint64)] + [C.POINTER(C.c_int)] * 4
    L.orc_shell_cardinality.restype = C.c_uint64
    L.orc_shell_cardinality.argtypes = [C.c_int]
    L.orc_index_bits.argtypes = [C.c_uint32]
    L.orc_index_decode.argtypes = [C.c_uint64, i32p]
    L.orc_fast_decode.argtypes = [C.c_uint64, i32p]
    L.orc_index_encode.argtypes = [i32p, C.POINTER(C.c_uint64)]
    L.orc_class_of.argtypes = [C.c_uint64]
    L.orc_class_levels.argtypes = [C.c_int, i32p, u8p, C.POINTER(C.c_int), C.POINTER(C.c_int)]
    L.orc_bitw_new.restype = C.c_void_p
    L.orc_bitw_push.argtypes = [C.c_void_p, C.c_uint64, C.c_uint32]
    L.orc_bitw_finish.restype = C.c_size_t
    L.orc_bitw_finish.argtypes = [C.c_void_p, C.POINTER(u8p)]
    L.orc_bitr_read.restype = C.c_uint64
    L.orc_bitr_read.argtypes = [C.c_char_p, C.POINTER(C.c_uint64), C.c_uint32]
    L.orc_free.argtypes = [C.c_void_p]
    L.orc_codebook_fingerprint.restype = C.c_uint64
    L.orc_read_header.argtypes = [C.c_char_p, C.c_size_t, C.POINTER(C.c_size_t), C.POINTER(C.c_uint32),
                                  C.POINTER(C.c_uint32), C.POINTER(C.c_char_p)]
    L.orc_write_header.restype = C.c_size_t
    L.orc_write_header.argtypes = [C.c_char_p, C.c_uint32, C.c_uint32]
    L.orc_read_matrix_raw.argtypes = [C.c_char_p, C.c_size_t, C.POINTER(C.c_size_t), C.POINTER(RawMatrixC),
                                      C.POINTER(C.c_char_p)]
    L.orc_raw_matrix_free.argtypes = [C.POINTER(RawMatrixC)]
    L.orc_write_matrix_raw.argtypes = [C.POINTER(RawMatrixC), C.POINTER(u8p), C.POINTER(C.c_size_t)]
    L.orc_reconstruct.argtypes = [i32p, C.c_uint32, C.POINTER(C.c_double), C.c_double, C.POINTER(C.c_double)]
    L.orc_rotation_new.argtypes = [C.c_size_t, C.c_uint64, C.POINTER(RotationC)]
    L.orc_rotation_free.argtypes = [C.POINTER(RotationC)]
    L.orc_rotation_free.restype = None
    L.orc_rotation_apply.argtypes = [C.POINTER(RotationC), C.POINTER(C.c_double)]
    L.orc_rotation_apply.restype = None
    L.orc_rotation_apply_transpose.argtypes = [C.POINTER(RotationC), C.POINTER(C.c_double)]
    L.orc_rotation_apply_transpose.restype = None
    L.orc_decode_matrix.argtypes = [C.POINTER(RawMatrixC), C.POINTER(C.c_float)]
    L.orc_fused_product.argtypes = [C.POINTER(RawMatrixC), C.POINTER(C.c_double), C.POINTER(C.c_double),
                                    C.POINTER(C.c_double)]
    L.orc_dense_matvec.argtypes = [C.POINTER(C.c_float), C.c_size_t, C.c_size_t, C.POINTER(C.c_double),
                                   C.POINTER(C.c_double)]
    L.orc_f16_to_f32.restype = C.c_float
    L.orc_f16_to_f32.argtypes = [C.c_uint16]
    L.orc_f32_to_f16.restype = C.c_uint16
    L.orc_f32_to_f16.argtypes = [C.c_float]
    L.orc_cpu_gemv.argtypes = [C.c_void_p, C.c_size_t, C.c_size_t, C.POINTER(C.c_double), C.POINTER(C.c_double),
                               C.c_void_p, C.c_void_p, C.c_void_p, C.c_int]
    L.orc_decode_batch.argtypes = [C.c_void_p, C.c_size_t, C.c_void_p, C.c_int]
    L.orc_cpu_decode_only.restype = C.c_uint64
    L.orc_cpu_decode_only.argtypes = [C.c_void_p, C.c_size_t]
    _lib = L
    return L


class OracleError(Exception):
    def __init__(self, code, what=""):
        self.code = code
        self.kind = ERR.get(code, str(code))
        self.what = what
        super().__init__(f"{self.kind}({what})" if what else self.kind)


def _pt(p):
    a = np.ascontiguousarray(p, dtype=np.int32)
    return a, a.ctypes.data_as(C.POINTER(C.c_int32))


def index_decode(idx):
    out = np.zeros(DIM, np.int32)
    ok = lib().orc_index_decode(int(idx), out.ctypes.data_as(C.POINTER(C.c_int32)))
    return out if ok else None


def fast_decode(idx):
    out = np.zeros(DIM, np.int32)
    ok = lib().orc_fast_decode(int(idx), out.ctypes.data_as(C.POINTER(C.c_int32)))
    return out if ok else None


def decode_many(indices, fast=True):
    """Decode an array of indices to an int8 [n, 24] array (every index must be valid)."""
    idx = np.ascontiguousarray(indices, dtype=np.uint64)
    out = np.zeros((idx.size, DIM), np.int8)
    rc = lib().orc_decode_batch(idx.ctypes.data, idx.size, out.ctypes.data, 1 if fast else 0)
    if rc:
        raise OracleError(rc)
    return out


def index_encode(p):
    a, ptr = _pt(p)
    out = C.c_uint64()
    ok = lib().orc_index_encode(ptr, C.byref(out))
    return out.value if ok else None


def leech_contains(p):
    a, ptr = _pt(p)
    return bool(lib().orc_leech_contains(ptr))


def shell_index(p):
    a, ptr = _pt(p)
    v = lib().orc_shell_index(ptr)
    return None if v < 0 else v


def golay_codewords():
    return np.ctypeslib.as_array(lib().orc_golay_codewords(), shape=(4096,)).copy()


def class_info(ci):
    lo, hi = C.c_uint64(), C.c_uint64()
    sh, odd, w, nl = C.c_int(), C.c_int(), C.c_int(), C.c_int()
    lib().orc_class_info(ci, C.byref(lo), C.byref(hi), C.byref(sh), C.byref(odd), C.byref(w), C.byref(nl))
    return dict(lo=lo.value, hi=hi.value, shell=sh.value, odd=bool(odd.value), w=w.value, n_levels=nl.value)


def class_levels(ci):
    v = (C.c_int32 * 5)()
    n = (C.c_uint8 * 5)()
    ln, nz = C.c_int(), C.c_int()
    lib().orc_class_levels(ci, v, n, C.byref(ln), C.byref(nz))
    return list(v)[: ln.value], list(n)[: ln.value], nz.value


def pack_bits(values_widths):
    L = lib()
    w = L.orc_bitw_new()
    for v, wd in values_widths:
        if L.orc_bitw_push(w, int(v), int(wd)):
            raise ValueError("value does not fit its width")
    out = C.POINTER(C.c_uint8)()
    n = L.orc_bitw_finish(w, C.byref(out))
    b = bytes(bytearray(out[:n]))
    L.orc_free(out)
    return b


def read_bits(buf, widths):
    pos = C.c_uint64(0)
    return [lib().orc_bitr_read(buf, C.byref(pos), int(w)) for w in widths]


class RawMatrix:
    """Owner of one parsed matrix record (llvq-artifact/src/format.rs:215-229)."""

    def __init__(self, c):
        self.c = c

    def __del__(self):
        try:
            lib().orc_raw_matrix_free(C.byref(self.c))
        except Exception:
            pass

    @property
    def name(self):
        return self.c.name.decode()

    @property
    def nblocks_total(self):
        return self.c.nblocks_total

    def indices(self):
        return np.ctypeslib.as_array(self.c.indices, shape=(max(self.c.nblocks_total, 1),))[: self.c.nblocks_total].copy()

    def gains(self):
        return np.ctypeslib.as_array(self.c.gains, shape=(max(self.c.nblocks_total, 1),))[: self.c.nblocks_total].copy()

    def row_scales(self):
        return np.ctypeslib.as_array(self.c.row_scales, shape=(max(self.c.d_out, 1),))[: self.c.d_out].copy()

    def centroids(self):
        return np.ctypeslib.as_array(self.c.centroids, shape=(max(self.c.n_centroids, 1),))[: self.c.n_centroids].copy()

    def tail(self):
        n = self.c.d_out * (self.c.d_in % DIM)
        return np.ctypeslib.as_array(self.c.tail, shape=(max(n, 1),))[:n].copy()

    def decode_matrix(self):
        w = np.zeros((self.c.d_out, self.c.d_in), np.float32)
        rc = lib().orc_decode_matrix(C.byref(self.c), w.ctypes.data_as(C.POINTER(C.c_float)))
        if rc:
            raise OracleError(rc)
        return w

    def fused_product(self, x):
        x = np.ascontiguousarray(x, dtype=np.float64)
        assert x.size == self.c.d_in
        y = np.zeros(self.c.d_out, np.float64)
        a = np.zeros(self.c.d_out, np.float64)
        dp = C.POINTER(C.c_double)
        rc = lib().orc_fused_product(C.byref(self.c), x.ctypes.data_as(dp), y.ctypes.data_as(dp), a.ctypes.data_as(dp))
        if rc:
            raise OracleError(rc)
        return y, a

    def write(self):
        out = C.POINTER(C.c_uint8)()
        n = C.c_size_t()
        rc = lib().orc_write_matrix_raw(C.byref(self.c), C.byref(out), C.byref(n))
        if rc:
            raise OracleError(rc)
        b = bytes(bytearray(out[: n.value]))
        lib().orc_free(out)
        return b


def read_header(buf, pos=0):
    p = C.c_size_t(pos)
    ver, nm = C.c_uint32(), C.c_uint32()
    what = C.c_char_p()
    rc = lib().orc_read_header(buf, len(buf), C.byref(p), C.byref(ver), C.byref(nm), C.byref(what))
    if rc:
        raise OracleError(rc, (what.value or b"").decode())
    return ver.value, nm.value, p.value


def write_header(version, n):
    b = C.create_string_buffer(16)
    k = lib().orc_write_header(b, version, n)
    if k == 0:
        raise OracleError(11)
    return b.raw[:k]


def read_matrix_raw(buf, pos=0):
    p = C.c_size_t(pos)
    m = RawMatrixC()
    what = C.c_char_p()
    rc = lib().orc_read_matrix_raw(buf, len(buf), C.byref(p), C.byref(m), C.byref(what))
    if rc:
        raise OracleError(rc, (what.value or b"").decode())
    return RawMatrix(m), p.value


def dense_matvec(w, x):
    w = np.ascontiguousarray(w, dtype=np.float32)
    x = np.ascontiguousarray(x, dtype=np.float64)
    y = np.zeros(w.shape[0], np.float64)
    dp = C.POINTER(C.c_double)
    lib().orc_dense_matvec(w.ctypes.data_as(C.POINTER(C.c_float)), w.shape[0], w.shape[1], x.ctypes.data_as(dp),
                           y.ctypes.data_as(dp))
    return y


def cpu_gemv(codes, d_out, d_in, centroids, row_scales, tail, x_f16, threads):
    codes = np.ascontiguousarray(codes, dtype=np.uint8)
    cen = np.ascontiguousarray(centroids, dtype=np.float64)
    rs = np.ascontiguousarray(row_scales, dtype=np.float64)
    tl = np.ascontiguousarray(tail, dtype=np.float32)
    xh = np.ascontiguousarray(x_f16, dtype=np.uint16)
    y = np.zeros(d_out, np.float32)
    dp = C.POINTER(C.c_double)
    rc = lib().orc_cpu_gemv(codes.ctypes.data, d_out, d_in, cen.ctypes.data_as(dp), rs.ctypes.data_as(dp),
                            tl.ctypes.data, xh.ctypes.data, y.ctypes.data, int(threads))
    if rc:
        raise OracleError(rc)
    return y


def cpu_decode_only(codes, nblocks):
    codes = np.ascontiguousarray(codes, dtype=np.uint8)
    return lib().orc_cpu_decode_only(codes.ctypes.data, int(nblocks))
