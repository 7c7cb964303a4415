#include "artifact.hpp"

#include <cstdio>
#include <cstring>

#include "../../include/llvq_hip.h"
#include "codebook.hpp"

namespace llvq {
namespace {

struct Cursor {
  const uint8_t* buf;
  size_t len;
  size_t pos;
  size_t left() const { return len - pos; }
  bool u32(uint32_t* v) {
    if (left() < 4) return false;
    std::memcpy(v, buf + pos, 4);  // the file is little-endian, so is every target of this library
    pos += 4;
    return true;
  }
  bool u64(uint64_t* v) {
    if (left() < 8) return false;
    std::memcpy(v, buf + pos, 8);
    pos += 8;
    return true;
  }
};

int truncated(std::string* err, const char* what) {
  if (err) *err = std::string("file ends mid-") + what;  // error.rs:58
  return LLVQ_ERR_TRUNCATED;
}

bool valid_utf8(const uint8_t* s, size_t n) {
  size_t i = 0;
  while (i < n) {
    const uint8_t c = s[i];
    int extra;
    uint32_t cp;
    if (c < 0x80) { ++i; continue; }
    if ((c & 0xE0) == 0xC0) { extra = 1; cp = c & 0x1F; }
    else if ((c & 0xF0) == 0xE0) { extra = 2; cp = c & 0x0F; }
    else if ((c & 0xF8) == 0xF0) { extra = 3; cp = c & 0x07; }
    else return false;
    if (i + (size_t)extra >= n) return false;
    for (int k = 1; k <= extra; ++k) {
      if ((s[i + k] & 0xC0) != 0x80) return false;
      cp = (cp << 6) | (s[i + k] & 0x3F);
    }
    static const uint32_t min_cp[4] = {0, 0x80, 0x800, 0x10000};
    if (cp < min_cp[extra] || cp > 0x10FFFF || (cp >= 0xD800 && cp <= 0xDFFF)) return false;
    i += (size_t)extra + 1;
  }
  return true;
}

}  // namespace

int parse_header(const uint8_t* buf, size_t len, size_t* pos, uint32_t* version,
                 uint32_t* n_matrices, std::string* err) {
  Cursor c{buf, len, *pos};
  if (c.left() < 4) return truncated(err, "magic");
  const uint8_t* m = buf + c.pos;
  c.pos += 4;
  if (m[0] == 'L' && m[1] == 'V' && m[2] == 'Q' && m[3] >= '1' && m[3] <= '4') {
    *version = (uint32_t)(m[3] - '0');
  } else {
    if (err) {
      char t[96];
      std::snprintf(t, sizeof t, "not an LLVQ artifact: magic is [%u, %u, %u, %u]", m[0], m[1], m[2], m[3]);
      *err = t;
    }
    return LLVQ_ERR_NOT_AN_ARTIFACT;
  }
  if (!c.u32(n_matrices)) return truncated(err, "matrix count");
  if (*version >= 4) {  // format.rs:604-613
    uint64_t stored;
    if (!c.u64(&stored)) return truncated(err, "codebook fingerprint");
    const uint64_t mine = codebook_fingerprint();
    if (stored != mine) {
      if (err) {
        char t[160];
        std::snprintf(t, sizeof t, "codebook fingerprint %#018llx does not match this build's %#018llx",
                      (unsigned long long)stored, (unsigned long long)mine);
        *err = t;
      }
      return LLVQ_ERR_CODEBOOK_MISMATCH;
    }
  }
  *pos = c.pos;
  return LLVQ_OK;
}

int parse_matrix_record(const uint8_t* buf, size_t len, size_t* pos, RecordView* out,
                        std::string* err) {
  Cursor c{buf, len, *pos};
  RecordView r;
  uint32_t name_len;
  if (!c.u32(&name_len)) return truncated(err, "name length");
  if (c.left() < name_len) return truncated(err, "name");
  if (!valid_utf8(buf + c.pos, name_len)) {
    if (err) *err = "matrix name is not valid UTF-8";
    return LLVQ_ERR_BAD_NAME;
  }
  r.name.assign((const char*)buf + c.pos, name_len);
  c.pos += name_len;
  if (!c.u32(&r.d_out)) return truncated(err, "d_out");
  if (!c.u32(&r.d_in)) return truncated(err, "d_in");
  if (!c.u32(&r.shell_cap)) return truncated(err, "shell cap");
  if (r.shell_cap > (uint32_t)kMaxShell) {  // format.rs:311-319
    if (err)
      *err = r.name + ": shell cap " + std::to_string(r.shell_cap) +
             " exceeds the supported ball (m <= " + std::to_string(kMaxShell) + ")";
    return LLVQ_ERR_INCONSISTENT;
  }
  if (!c.u32(&r.n_centroids)) return truncated(err, "centroid count");
  if (!c.u64(&r.rotation_seed)) return truncated(err, "rotation seed");
  uint32_t flag;
  if (!c.u32(&flag)) return truncated(err, "rotation flag");
  r.has_rotation = flag != 0;

  // Lengths from the file are claims: check them against the bytes that are
  // actually there before sizing anything from them (format.rs:124-142).
  if ((uint64_t)r.n_centroids * 8 > c.left()) return truncated(err, "centroids");
  r.centroids_off = c.pos;
  r.centroids.resize(r.n_centroids);
  if (r.n_centroids) std::memcpy(r.centroids.data(), buf + c.pos, (size_t)r.n_centroids * 8);
  c.pos += (size_t)r.n_centroids * 8;
  if ((uint64_t)r.d_out * 8 > c.left()) return truncated(err, "row scales");
  r.row_scales_off = c.pos;
  r.row_scales.resize(r.d_out);
  if (r.d_out) std::memcpy(r.row_scales.data(), buf + c.pos, (size_t)r.d_out * 8);
  c.pos += (size_t)r.d_out * 8;
  const uint64_t tail_n = (uint64_t)r.d_out * (r.d_in % kDim);
  if (tail_n * 4 > c.left()) return truncated(err, "tail");
  r.tail_off = c.pos;
  r.tail.resize((size_t)tail_n);
  if (tail_n) std::memcpy(r.tail.data(), buf + c.pos, (size_t)tail_n * 4);  // an empty vector has no address to copy to
  c.pos += (size_t)tail_n * 4;

  uint64_t nbytes;
  if (!c.u64(&nbytes)) return truncated(err, "code length");
  if (nbytes > c.left()) return truncated(err, "code stream");
  r.codes_off = c.pos;
  r.codes = buf + c.pos;
  r.code_bytes = (size_t)nbytes;
  c.pos += (size_t)nbytes;

  // The stream must hold every block the dimensions promise (format.rs:352-361).
  uint64_t pow2 = 1;
  uint32_t gb = 0;
  while (pow2 < r.n_centroids) { pow2 <<= 1; ++gb; }
  const unsigned __int128 need =
      (unsigned __int128)r.d_out * (r.d_in / kDim) * (uint32_t)(index_bits(r.shell_cap) + (int)gb);
  if (need > (unsigned __int128)nbytes * 8) return truncated(err, "code stream");

  *out = std::move(r);
  *pos = c.pos;
  return LLVQ_OK;
}

namespace {

int read_name(Cursor& c, const char* what, std::string* name, std::string* err) {
  uint32_t n = 0;
  if (!c.u32(&n)) return truncated(err, what);
  if (c.left() < n) return truncated(err, what);
  if (!valid_utf8(c.buf + c.pos, n)) {
    if (err) *err = "a name is not valid UTF-8";
    return LLVQ_ERR_BAD_NAME;
  }
  name->assign(reinterpret_cast<const char*>(c.buf + c.pos), n);
  c.pos += n;
  return LLVQ_OK;
}

}  // namespace

int parse_raw_tensor(const uint8_t* buf, size_t len, size_t* pos, uint32_t version, RawTensorView* out,
                     std::string* err) {
  Cursor c{buf, len, *pos};
  RawTensorView t;
  if (version >= 3 && !c.u32(&t.tag)) return truncated(err, "raw tensor tag");
  // refused before anything else is parsed: past an unknown tag every byte would be read against the wrong layout
  if (t.tag != 0 && t.tag != 1) {
    if (err) *err = "raw tensor encoding tag " + std::to_string(t.tag) + " is unknown — file written by a newer writer, or corrupted";
    return LLVQ_ERR_BAD_RAW_ENCODING;
  }
  int rc = read_name(c, "raw tensor name", &t.name, err);
  if (rc) return rc;
  uint32_t rank = 0;
  if (!c.u32(&rank)) return truncated(err, "raw tensor rank");
  if ((uint64_t)rank * 8 > c.left()) return truncated(err, "raw tensor dims");
  t.dims.resize(rank);
  for (uint32_t i = 0; i < rank; ++i)
    if (!c.u64(&t.dims[i])) return truncated(err, "raw tensor dims");
  if (t.tag == 0) {
    if (!c.u64(&t.count)) return truncated(err, "raw tensor length");
    if (t.count > c.left() / 2) return truncated(err, "raw tensor data");  // also a count whose byte size overflows
    t.data_off = c.pos;
    t.data_len = (size_t)t.count * 2;
    c.pos += t.data_len;
  } else {
    uint64_t nbytes = 0;
    if (!c.u32(&t.bits)) return truncated(err, "quant width");
    t.bits &= 0xFFu;
    if (!c.u32(&t.group)) return truncated(err, "quant group");
    if (!c.u64(&nbytes)) return truncated(err, "quant packed length");
    if (nbytes > c.left()) return truncated(err, "quant packed data");
    t.data_off = c.pos;
    t.data_len = (size_t)nbytes;
    c.pos += t.data_len;
    if (!c.u64(&t.count)) return truncated(err, "quant group count");
    if (t.count > c.left() / 2) return truncated(err, "quant scales");
    t.scales_off = c.pos;
    c.pos += (size_t)t.count * 2;
    if (t.count > c.left() / 2) return truncated(err, "quant biases");
    t.biases_off = c.pos;
    c.pos += (size_t)t.count * 2;
  }
  *out = std::move(t);
  *pos = c.pos;
  return LLVQ_OK;
}

int parse_blob(const uint8_t* buf, size_t len, size_t* pos, BlobView* out, std::string* err) {
  Cursor c{buf, len, *pos};
  BlobView b;
  int rc = read_name(c, "blob name", &b.name, err);
  if (rc) return rc;
  uint64_t n = 0;
  if (!c.u64(&n)) return truncated(err, "blob length");
  if (n > c.left()) return truncated(err, "blob");
  b.data_off = c.pos;
  b.data_len = (size_t)n;
  c.pos += b.data_len;
  *out = std::move(b);
  *pos = c.pos;
  return LLVQ_OK;
}

}  // namespace llvq
