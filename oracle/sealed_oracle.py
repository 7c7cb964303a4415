"""CPU restatement of the sealed-file sections that follow the matrix records:
raw tensors (binary16, or int4/int8 codes with binary16 scale and bias per group)
and named blobs.  TEST INFRASTRUCTURE ONLY.

Follows llvq-artifact/src/sealed.rs: f16_to_f32 :47-62, RawTensor::to_f32 :113-136,
write_raw :214-275, read_raw :277-326, write_blob / read_blob :328-341; and the
q8 head arithmetic of llvq-llm/kernels/emb_q8.cu (weight = f32(s * q) + b, f32
fused multiply-add against the activation, binary16 out).

Pinned by the reference's own vectors (llvq-artifact/tests/raw_tensors.rs: nine
binary16 widenings, the 2 x 5 int4 tensor and its decoded values, the legacy v2
record) and its hostile-file cases (tests/hostile_files.rs:172-213)."""
import struct

import numpy as np


class OracleSealedError(Exception):
    def __init__(self, kind, what=None):
        self.kind, self.what = kind, what
        super().__init__(f"{kind}: {what}")


def f16_to_f32(bits):
    """sealed.rs:47-62, bit by bit."""
    bits = int(bits) & 0xFFFF
    sign = (bits >> 15) << 31
    exp = (bits >> 10) & 0x1F
    frac = bits & 0x3FF
    if exp == 0 and frac == 0:
        mag = 0
    elif exp == 0:
        z = 32 - frac.bit_length()  # leading zeros of a u32
        mag = ((134 - z) << 23) | ((frac << (z - 8)) & 0x007FFFFF)
    elif exp == 0x1F:
        mag = (0xFF << 23) | (frac << 13)
    else:
        mag = ((exp + 112) << 23) | (frac << 13)
    return np.frombuffer(struct.pack("<I", sign | mag), dtype="<f4")[0]


class Cursor:
    def __init__(self, buf, pos=0):
        self.buf, self.pos = bytes(buf), pos

    def get(self, n, what):
        if n > len(self.buf) - self.pos:
            raise OracleSealedError("Truncated", what)
        out = self.buf[self.pos:self.pos + n]
        self.pos += n
        return out

    def u32(self, what):
        return struct.unpack("<I", self.get(4, what))[0]

    def u64(self, what):
        return struct.unpack("<Q", self.get(8, what))[0]

    def string(self, what):
        n = self.u32(what)
        try:
            return self.get(n, what).decode("utf-8")
        except UnicodeDecodeError:
            raise OracleSealedError("BadName")

    def u16s(self, n, what):
        if n * 2 >= 1 << 64:  # a count whose byte size overflows u64 truncates by definition
            raise OracleSealedError("Truncated", what)
        return np.frombuffer(self.get(2 * n, what), dtype="<u2")


def read_raw(cur, version):
    """sealed.rs:277-326 → dict(name, dims, kind, ...)."""
    tag = cur.u32("raw tensor tag") if version >= 3 else 0
    if tag not in (0, 1):
        raise OracleSealedError("BadRawEncoding", tag)
    name = cur.string("raw tensor name")
    rank = cur.u32("raw tensor rank")
    dims = [cur.u64("raw tensor dims") for _ in range(rank)]
    if tag == 0:
        n = cur.u64("raw tensor length")
        return dict(name=name, dims=dims, kind="f16", data=cur.u16s(n, "raw tensor data"))
    bits = cur.u32("quant width") & 0xFF
    group = cur.u32("quant group")
    nbytes = cur.u64("quant packed length")
    packed = np.frombuffer(cur.get(nbytes, "quant packed data"), dtype=np.uint8)
    groups = cur.u64("quant group count")
    scales = cur.u16s(groups, "quant scales")
    biases = cur.u16s(groups, "quant biases")
    return dict(name=name, dims=dims, kind="quant", bits=bits, group=group, packed=packed, scales=scales, biases=biases)


def read_blob(cur):
    name = cur.string("blob name")
    n = cur.u64("blob length")
    return dict(name=name, data=cur.get(n, "blob"))


def to_f32(t):
    """RawTensor::to_f32 (sealed.rs:113-136)."""
    if t["kind"] == "f16":
        return np.array([f16_to_f32(b) for b in t["data"]], dtype=np.float32)
    n = int(np.prod(t["dims"], dtype=np.int64)) if t["dims"] else 1
    row_len = max(t["dims"][-1] if t["dims"] else 1, 1)
    gpr = -(-row_len // t["group"])
    out = np.empty(n, np.float32)
    for i in range(n):
        row, col = divmod(i, row_len)
        g = row * gpr + col // t["group"]
        qv = int(t["packed"][i]) if t["bits"] == 8 else (int(t["packed"][i // 2]) >> (4 * (i % 2))) & 0xF
        out[i] = np.float32(f16_to_f32(t["scales"][g]) * np.float32(qv)) + f16_to_f32(t["biases"][g])
    return out


def q8_rows_f32(packed, scales, biases, d, group=64):
    """Vectorised to_f32 for an int8 tensor [rows, d]: f32(s * q) + b, both steps rounded to f32."""
    rows = packed.size // d
    gpr = -(-d // group)
    s = scales.view(np.float16).astype(np.float32).reshape(rows, gpr)
    b = biases.view(np.float16).astype(np.float32).reshape(rows, gpr)
    q = packed.reshape(rows, d).astype(np.float32)
    idx = np.arange(d) // group
    return (s[:, idx] * q).astype(np.float32) + b[:, idx]


def q8_head_logits(packed, scales, biases, d, x_f16):
    """emb_q8.cu tv_q8_h: logits[row] = f16(sum_c (s q + b) x_c); f64 accumulation here."""
    W = q8_rows_f32(packed, scales, biases, d).astype(np.float64)
    x = np.asarray(x_f16, np.float16).astype(np.float64)
    return (W @ x).astype(np.float16).astype(np.float32)
