"""The `.llvq` container as this path needs it: header and matrix records.

Host-side mirror of llvq-artifact/src/format.rs (`read_header` :588,
`read_matrix_raw` :301, `write_matrix_raw` :238, `write_header` :563) with the
code stream kept packed — the device reads the file's bytes verbatim.  Errors
are the variants of llvq-artifact/src/error.rs:11-45.
"""
import struct

import numpy as np

DIM = 24
N13 = 280974212784720
N12 = 111043117458000
MAX_SHELL = 13
FINGERPRINT = 0x338F420F11866319
# N(cap) for cap = 0..13 (theta series of the Leech lattice, cumulative from shell 2)
_SHELL_SIZES = [0, 0, 196560, 16773120, 398034000, 4629381120, 34417656000, 187489935360,
                814879774800, 2975551488000, 9486551299680, 27052945920000, 70486236999360,
                169931095326720]


class ArtifactError(Exception):
    """One subclass per variant of llvq_artifact::Error that this path can raise."""


class NotAnArtifact(ArtifactError):
    pass


class Truncated(ArtifactError):
    def __init__(self, reading):
        self.reading = reading
        super().__init__(f"file ends mid-{reading}")


class BadName(ArtifactError):
    pass


class Inconsistent(ArtifactError):
    pass


class IndexTooWide(ArtifactError):
    pass


class CodebookMismatch(ArtifactError):
    pass


class BadRawEncoding(ArtifactError):
    """Error::BadRawEncoding { tag } (error.rs:34)"""

    def __init__(self, tag):
        self.tag = tag
        super().__init__(f"raw tensor encoding tag {tag} is unknown — file written by a newer writer, or corrupted")


class UnknownVersion(ArtifactError):
    pass


def index_bits(cap):
    """ceil(log2 N(cap)), floor 1 — llvq-quant/src/quantizer.rs:572-576."""
    n = sum(_SHELL_SIZES[2:cap + 1]) if cap >= 2 else 0
    return max(int(n).bit_length(), 1)


def gain_bits(n_centroids):
    """format.rs:87-89"""
    p, b = 1, 0
    while p < n_centroids:
        p <<= 1
        b += 1
    return b


class RawMatrix:
    """RawMatrix of format.rs:215-229 with `codes` left as the packed stream."""

    def __init__(self, name, d_out, d_in, shell_cap, centroids, row_scales, tail, codes,
                 rotation_seed=None):
        self.name = name
        self.d_out = int(d_out)
        self.d_in = int(d_in)
        self.shell_cap = int(shell_cap)
        self.centroids = np.ascontiguousarray(centroids, dtype=np.float64)
        self.row_scales = np.ascontiguousarray(row_scales, dtype=np.float64)
        self.tail = np.ascontiguousarray(tail, dtype=np.float32).reshape(-1)
        self.codes = np.ascontiguousarray(codes, dtype=np.uint8).reshape(-1)
        self.rotation_seed = rotation_seed

    @property
    def nblocks(self):
        return self.d_in // DIM

    @property
    def tail_w(self):
        return self.d_in % DIM

    def encoded_bytes(self):
        """codes + tail + row scales + centroids, as the file stores them."""
        return int(self.codes.size + 4 * self.tail.size + 8 * self.row_scales.size + 8 * self.centroids.size)

    def unpack(self):
        """(indices u64, gains u8) of the code stream: per block index_bits(cap) bits of index, then the gain bits,
        most significant first, blocks back to back (6 bytes per block at cap 12, 49 bits at cap 13)."""
        ib, gb = index_bits(self.shell_cap), gain_bits(self.centroids.size)
        n = self.d_out * self.nblocks
        if ib + gb == 48:
            b = self.codes[: 6 * n].reshape(n, 6).astype(np.uint64)
            v = np.zeros(n, np.uint64)
            for k in range(6):
                v = (v << np.uint64(8)) | b[:, k]
        else:
            w = ib + gb
            if w > 64:
                raise Inconsistent(f"{self.name}: {w} bits per block")
            bits = np.unpackbits(self.codes[: (n * w + 7) // 8])[: n * w].reshape(n, w)
            v = np.zeros(n, np.uint64)
            for k in range(w):
                v = (v << np.uint64(1)) | bits[:, k].astype(np.uint64)
        return v >> np.uint64(gb), (v & np.uint64((1 << gb) - 1)).astype(np.uint8)


def pack_codes(indices, gains, index_width=47):
    """Per block `index_width` bits of index then one gain bit, MSB first, blocks back to back
    (llvq-search/src/pack.rs:10-18, :48-82, format.rs:185-203) — 6 bytes per block at cap 12 (47 bits of
    index), 49 bits per block at cap 13 (48), the stream's last byte zero-padded."""
    idx = np.ascontiguousarray(indices, dtype=np.uint64)
    g = np.ascontiguousarray(gains, dtype=np.uint64)
    if not 1 <= index_width <= 62:
        raise Inconsistent(f"{index_width}-bit indices")
    if idx.size and int(idx.max()) >= (1 << index_width):
        raise IndexTooWide(f"index {int(idx.max())} does not fit in {index_width} bits")
    v = (idx << np.uint64(1)) | (g & np.uint64(1))
    be = v.astype(">u8").view(np.uint8).reshape(-1, 8)
    if index_width == 47:
        return np.ascontiguousarray(be[:, 2:]).reshape(-1)
    w = index_width + 1
    bits = np.unpackbits(be, axis=1)[:, 64 - w:]
    return np.packbits(np.ascontiguousarray(bits).reshape(-1))


def write_header(version, n_matrices):
    """format.rs:563-578"""
    if version not in (1, 2, 3, 4):
        raise UnknownVersion(f"no artifact format version {version} to write")
    out = b"LVQ" + str(version).encode() + struct.pack("<I", n_matrices)
    if version >= 4:
        out += struct.pack("<Q", FINGERPRINT)
    return out


def read_header(buf, pos=0):
    """format.rs:588-619 → (version, n_matrices, new_pos)"""
    if len(buf) - pos < 4:
        raise Truncated("magic")
    magic = bytes(buf[pos:pos + 4])
    if magic not in (b"LVQ1", b"LVQ2", b"LVQ3", b"LVQ4"):
        raise NotAnArtifact(f"not an LLVQ artifact: magic is {list(magic)}")
    version = magic[3] - ord("0")
    pos += 4
    if len(buf) - pos < 4:
        raise Truncated("matrix count")
    (n,) = struct.unpack_from("<I", buf, pos)
    pos += 4
    if version >= 4:
        if len(buf) - pos < 8:
            raise Truncated("codebook fingerprint")
        (fp,) = struct.unpack_from("<Q", buf, pos)
        pos += 8
        if fp != FINGERPRINT:
            raise CodebookMismatch(f"codebook fingerprint {fp:#018x} does not match this build's {FINGERPRINT:#018x}")
    return version, n, pos


def write_matrix_raw(m):
    """format.rs:238-298: the record's bytes."""
    nb = m.d_out * m.nblocks
    ib, gb = index_bits(m.shell_cap), gain_bits(m.centroids.size)
    need = (nb * (ib + gb) + 7) // 8
    if m.codes.size != need:
        raise Inconsistent(f"{m.name}: {m.codes.size} code bytes for {nb} blocks")
    if m.row_scales.size != m.d_out:
        raise Inconsistent(f"{m.name}: {m.row_scales.size} row scales for {m.d_out} rows")
    name = m.name.encode()
    head = struct.pack("<I", len(name)) + name + struct.pack(
        "<IIIIQI", m.d_out, m.d_in, m.shell_cap, m.centroids.size,
        m.rotation_seed or 0, 1 if m.rotation_seed is not None else 0)
    return b"".join([head, m.centroids.astype("<f8").tobytes(), m.row_scales.astype("<f8").tobytes(),
                     m.tail.astype("<f4").tobytes(), struct.pack("<Q", m.codes.size), m.codes.tobytes()])


def read_matrix_raw(buf, pos=0):
    """format.rs:301-382 → (RawMatrix, new_pos).  `buf` is bytes-like; arrays are views where possible."""
    mv = memoryview(buf)
    n = len(mv)

    def need(k, what):
        if n - pos < k:
            raise Truncated(what)

    need(4, "name length")
    (nl,) = struct.unpack_from("<I", mv, pos)
    pos += 4
    need(nl, "name")
    try:
        name = bytes(mv[pos:pos + nl]).decode("utf-8")
    except UnicodeDecodeError:
        raise BadName("matrix name is not valid UTF-8")
    pos += nl
    fields = []
    for what, fmt in (("d_out", "<I"), ("d_in", "<I"), ("shell cap", "<I")):
        need(4, what)
        fields.append(struct.unpack_from(fmt, mv, pos)[0])
        pos += 4
    d_out, d_in, cap = fields
    if cap > MAX_SHELL:
        raise Inconsistent(f"{name}: shell cap {cap} exceeds the supported ball (m <= {MAX_SHELL})")
    need(4, "centroid count")
    (nc,) = struct.unpack_from("<I", mv, pos)
    pos += 4
    need(8, "rotation seed")
    (seed,) = struct.unpack_from("<Q", mv, pos)
    pos += 8
    need(4, "rotation flag")
    (flag,) = struct.unpack_from("<I", mv, pos)
    pos += 4
    need(8 * nc, "centroids")
    centroids = np.frombuffer(mv, dtype="<f8", count=nc, offset=pos).copy()
    pos += 8 * nc
    need(8 * d_out, "row scales")
    row_scales = np.frombuffer(mv, dtype="<f8", count=d_out, offset=pos).copy()
    pos += 8 * d_out
    tn = d_out * (d_in % DIM)
    need(4 * tn, "tail")
    tail = np.frombuffer(mv, dtype="<f4", count=tn, offset=pos).copy()
    pos += 4 * tn
    need(8, "code length")
    (nbytes,) = struct.unpack_from("<Q", mv, pos)
    pos += 8
    need(nbytes, "code stream")
    codes = np.frombuffer(mv, dtype=np.uint8, count=nbytes, offset=pos)
    pos += nbytes
    if d_out * (d_in // DIM) * (index_bits(cap) + gain_bits(nc)) > nbytes * 8:
        raise Truncated("code stream")
    return RawMatrix(name, d_out, d_in, cap, centroids, row_scales, tail, codes,
                     seed if flag else None), pos


# ---- sealed sections: raw tensors and blobs (llvq-artifact/src/sealed.rs) ----------------
TAG_F16, TAG_QUANT = 0, 1


class RawTensor:
    """sealed.rs:80-92.  `data` is a uint16 array of binary16 bit patterns (kind "f16"),
    or for kind "quant": `packed` uint8, `scales` / `biases` uint16, `bits` in (4, 8), `group`."""

    def __init__(self, name, dims, data=None, bits=None, group=None, packed=None, scales=None, biases=None):
        self.name, self.dims = name, [int(d) for d in dims]
        self.kind = "f16" if data is not None else "quant"
        self.data = None if data is None else np.ascontiguousarray(data, dtype=np.uint16)
        self.bits, self.group = bits, group
        self.packed = None if packed is None else np.ascontiguousarray(packed, dtype=np.uint8)
        self.scales = None if scales is None else np.ascontiguousarray(scales, dtype=np.uint16)
        self.biases = None if biases is None else np.ascontiguousarray(biases, dtype=np.uint16)

    def __len__(self):
        return int(np.prod(self.dims, dtype=np.int64)) if self.dims else 1

    def nbytes(self):
        """RawTensor::bytes (sealed.rs:104-111)"""
        if self.kind == "f16":
            return self.data.size * 2
        return self.packed.size + (self.scales.size + self.biases.size) * 2


class Blob:
    def __init__(self, name, data):
        self.name, self.data = name, bytes(data)


def _put_str(s):
    b = s.encode()
    return struct.pack("<I", len(b)) + b


def write_raw(t: RawTensor) -> bytes:
    """sealed.rs:214-275"""
    out = [struct.pack("<I", TAG_F16 if t.kind == "f16" else TAG_QUANT), _put_str(t.name),
           struct.pack("<I", len(t.dims))] + [struct.pack("<Q", d) for d in t.dims]
    n = len(t)
    if t.kind == "f16":
        if t.data.size != n:
            raise Inconsistent(f"{t.name}: {t.data.size} values for dims {t.dims}")
        out += [struct.pack("<Q", t.data.size), t.data.astype("<u2").tobytes()]
    else:
        row_len = max(t.dims[-1] if t.dims else 1, 1)
        groups = (n // row_len) * ((row_len + t.group - 1) // t.group)
        if t.bits not in (4, 8):
            raise Inconsistent(f"{t.name}: unsupported quant width {t.bits}")
        need = n if t.bits == 8 else (n + 1) // 2
        if t.packed.size != need or t.scales.size != groups or t.biases.size != groups:
            raise Inconsistent(f"{t.name}: {t.packed.size} packed bytes / {t.scales.size} scales / {t.biases.size} biases "
                               f"for {n} values in groups of {t.group} (want {need} / {groups} / {groups})")
        out += [struct.pack("<IIQ", t.bits, t.group, t.packed.size), t.packed.tobytes(), struct.pack("<Q", groups),
                t.scales.astype("<u2").tobytes(), t.biases.astype("<u2").tobytes()]
    return b"".join(out)


def read_raw(buf, pos=0, version=4):
    """sealed.rs:277-326 → (RawTensor, new_pos)"""
    mv = memoryview(buf)
    n = len(mv)

    def take(k, what):
        nonlocal pos
        if k > n - pos:
            raise Truncated(what)
        at = pos
        pos += k
        return at

    tag = TAG_F16
    if version >= 3:
        (tag,) = struct.unpack_from("<I", mv, take(4, "raw tensor tag"))
    if tag not in (TAG_F16, TAG_QUANT):
        raise BadRawEncoding(tag)
    (nl,) = struct.unpack_from("<I", mv, take(4, "raw tensor name"))
    at = take(nl, "raw tensor name")
    try:
        name = bytes(mv[at:at + nl]).decode("utf-8")
    except UnicodeDecodeError:
        raise BadName("raw tensor name is not valid UTF-8")
    (rank,) = struct.unpack_from("<I", mv, take(4, "raw tensor rank"))
    dims = [struct.unpack_from("<Q", mv, take(8, "raw tensor dims"))[0] for _ in range(rank)]
    if tag == TAG_F16:
        (cnt,) = struct.unpack_from("<Q", mv, take(8, "raw tensor length"))
        if cnt > (1 << 62):
            raise Truncated("raw tensor data")
        at = take(2 * cnt, "raw tensor data")
        return RawTensor(name, dims, data=np.frombuffer(mv, dtype="<u2", count=cnt, offset=at)), pos
    bits, group = struct.unpack_from("<II", mv, take(8, "quant width"))
    (nbytes,) = struct.unpack_from("<Q", mv, take(8, "quant packed length"))
    at = take(nbytes, "quant packed data")
    packed = np.frombuffer(mv, dtype=np.uint8, count=nbytes, offset=at)
    (groups,) = struct.unpack_from("<Q", mv, take(8, "quant group count"))
    if groups > (1 << 62):
        raise Truncated("quant scales")
    scales = np.frombuffer(mv, dtype="<u2", count=groups, offset=take(2 * groups, "quant scales"))
    biases = np.frombuffer(mv, dtype="<u2", count=groups, offset=take(2 * groups, "quant biases"))
    return RawTensor(name, dims, bits=bits & 0xFF, group=group, packed=packed, scales=scales, biases=biases), pos


def write_blob(b: Blob) -> bytes:
    return _put_str(b.name) + struct.pack("<Q", len(b.data)) + b.data


def read_blob(buf, pos=0):
    """sealed.rs:336-341 → (Blob, new_pos)"""
    mv = memoryview(buf)
    n = len(mv)
    if n - pos < 4:
        raise Truncated("blob name")
    (nl,) = struct.unpack_from("<I", mv, pos)
    pos += 4
    if nl > n - pos:
        raise Truncated("blob name")
    try:
        name = bytes(mv[pos:pos + nl]).decode("utf-8")
    except UnicodeDecodeError:
        raise BadName("blob name is not valid UTF-8")
    pos += nl
    if n - pos < 8:
        raise Truncated("blob length")
    (k,) = struct.unpack_from("<Q", mv, pos)
    pos += 8
    if k > n - pos:
        raise Truncated("blob")
    return Blob(name, mv[pos:pos + k]), pos + k


def write_file(matrices, version=4, raws=(), blobs=()):
    """ArtifactWriter::seal / finish (format.rs:501-545): header, matrix records, raw tensors, blobs."""
    return b"".join([write_header(version, len(matrices))] + [write_matrix_raw(m) for m in matrices]
                    + [struct.pack("<I", len(raws))] + [write_raw(t) for t in raws]
                    + [struct.pack("<I", len(blobs))] + [write_blob(b) for b in blobs])


def read_file(buf):
    version, n, pos = read_header(buf)
    out = []
    for _ in range(n):
        m, pos = read_matrix_raw(buf, pos)
        out.append(m)
    return version, out


def read_sealed(buf):
    """The whole file: (version, matrices, raw tensors, blobs).  Files of version 1 end after the matrices."""
    version, n, pos = read_header(buf)
    mats = []
    for _ in range(n):
        m, pos = read_matrix_raw(buf, pos)
        mats.append(m)
    raws, blobs = [], []
    if version >= 2:
        if len(buf) - pos < 4:
            raise Truncated("raw tensor count")
        (nr,) = struct.unpack_from("<I", buf, pos)
        pos += 4
        for _ in range(nr):
            t, pos = read_raw(buf, pos, version)
            raws.append(t)
        if len(buf) - pos < 4:
            raise Truncated("blob count")
        (nbl,) = struct.unpack_from("<I", buf, pos)
        pos += 4
        for _ in range(nbl):
            b, pos = read_blob(buf, pos)
            blobs.append(b)
    return version, mats, raws, blobs


def split_name(name):
    """`model.layers.{b}.{proj}.weight` → (b, proj) — format.rs:442-453"""
    parts = name.split(".")
    if len(parts) < 5:
        raise ArtifactError(f"unexpected tensor name {name}")
    try:
        return int(parts[2]), ".".join(parts[3:-1])
    except ValueError:
        raise ArtifactError(f"unexpected tensor name {name}")
