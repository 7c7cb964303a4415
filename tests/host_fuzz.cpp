// Host-side robustness driver, built with -fsanitize=address,undefined by tests/test_host_sanitized.py:
// every prefix of a sealed file and a few thousand corrupted copies go through the library's readers
// (the cases of llvq-artifact/tests/hostile_files.rs, generalised: always a status, never a fault), and
// the index decoder the kernels share with the host runs on class boundaries and random 48-bit ranks, and the
// rotation tables are built and applied for served and awkward widths.
// Each input lives in a heap block of exactly its size, so a read past the end is reported.
#include <algorithm>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <memory>
#include <string>
#include <vector>

#include "../llvq_amd/csrc/artifact.hpp"
#include "../llvq_amd/csrc/codebook.hpp"
#include "../llvq_amd/csrc/gemm_share.h"
#include "../llvq_amd/csrc/rotation.hpp"

using namespace llvq;

static uint64_t rng_state = 1;
static uint64_t next_u64() {  // SplitMix64
  uint64_t z = (rng_state += 0x9E3779B97F4A7C15ULL);
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ULL;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBULL;
  return z ^ (z >> 31);
}

// header, matrix records, raw tensors, blobs; stops at the first refusal.  Returns the records read.
static size_t read_all(const uint8_t* buf, size_t len) {
  size_t pos = 0, seen = 0;
  uint32_t version = 0, n = 0;
  std::string err;
  if (parse_header(buf, len, &pos, &version, &n, &err)) return seen;
  for (uint32_t i = 0; i < n; ++i) {
    RecordView r;
    if (parse_matrix_record(buf, len, &pos, &r, &err)) return seen;
    if (r.codes_off + r.code_bytes > len) { std::fprintf(stderr, "record view past the buffer\n"); std::abort(); }
    ++seen;
  }
  if (version < 2) return seen;
  auto read_u32 = [&](uint32_t* v) {
    if (pos + 4 > len) return false;
    std::memcpy(v, buf + pos, 4);
    pos += 4;
    return true;
  };
  uint32_t n_raw = 0, n_blob = 0;
  if (!read_u32(&n_raw)) return seen;
  for (uint32_t i = 0; i < n_raw; ++i) {
    RawTensorView t;
    if (parse_raw_tensor(buf, len, &pos, version, &t, &err)) return seen;
    if (t.data_off + t.data_len > len) { std::fprintf(stderr, "tensor view past the buffer\n"); std::abort(); }
    ++seen;
  }
  if (!read_u32(&n_blob)) return seen;
  for (uint32_t i = 0; i < n_blob; ++i) {
    BlobView b;
    if (parse_blob(buf, len, &pos, &b, &err)) return seen;
    if (b.data_off + b.data_len > len) { std::fprintf(stderr, "blob view past the buffer\n"); std::abort(); }
    ++seen;
  }
  return seen;
}

int main(int argc, char** argv) {
  if (argc < 4) return 2;
  std::FILE* f = std::fopen(argv[1], "rb");
  if (!f) return 2;
  std::vector<uint8_t> file;
  uint8_t tmp[4096];
  for (size_t k; (k = std::fread(tmp, 1, sizeof tmp, f)) > 0;) file.insert(file.end(), tmp, tmp + k);
  std::fclose(f);
  rng_state = std::strtoull(argv[2], nullptr, 10);
  const size_t n_mut = std::strtoull(argv[3], nullptr, 10);

  const size_t whole = read_all(file.data(), file.size());
  size_t cases = 0;
  // every prefix (all of the short ones, a stride through the long code streams)
  for (size_t len = 0; len < file.size(); len += (len < 4096 || file.size() - len < 4096) ? 1 : 97) {
    std::unique_ptr<uint8_t[]> p(new uint8_t[len ? len : 1]);
    std::memcpy(p.get(), file.data(), len);
    if (read_all(p.get(), len) > whole) return 3;
    ++cases;
  }
  // corrupted copies: a few bytes replaced, mostly inside the headers of the records
  for (size_t m = 0; m < n_mut; ++m) {
    std::unique_ptr<uint8_t[]> p(new uint8_t[file.size()]);
    std::memcpy(p.get(), file.data(), file.size());
    const int flips = 1 + (int)(next_u64() % 4);
    for (int k = 0; k < flips; ++k) {
      const size_t span = (next_u64() & 1) ? std::min<size_t>(file.size(), 512) : file.size();
      p[next_u64() % span] = (uint8_t)next_u64();
    }
    (void)read_all(p.get(), file.size());
    ++cases;
  }
  // the index decoder: boundaries of the 48-bit field, the ends of the valid range, random ranks
  int8_t pt[kDim];
  int shell = 0;
  size_t valid = 0;
  const uint64_t edges[] = {0, 1, 2, 196560, 196561, kN13 - 1, kN13, kN13 + 1, (1ULL << 47) - 1, 1ULL << 47, (1ULL << 48) - 1, ~0ULL};
  for (uint64_t e : edges) valid += host_decode(e, pt, &shell) ? 1 : 0;
  for (size_t m = 0; m < 200000; ++m) valid += host_decode(next_u64() >> 16, pt, &shell) ? 1 : 0;
  // The table that stands for the last eight slots of the odd-coset walk, against an independent
  // enumeration: for every multiset of four kinds over eight slots, entry r must be the r-th
  // arrangement in lexicographic order (kind 0 first; index.rs:97-117), as codes 3 - kind, first
  // slot in the lowest byte, and the multisets' entries must follow one another without gaps.
  {
    const Codebook& cb = codebook();
    size_t entries = 0;
    for (int t3 = 0; t3 <= 8; ++t3)
      for (int t2 = 0; t2 <= t3; ++t2)
        for (int t1 = 0; t1 <= t2; ++t1) {
          const uint32_t me = cb.tail_meta[t1 + 9 * t2 + 81 * t3];
          if ((me >> 12) != entries) { std::fprintf(stderr, "walk tail: multiset %d %d %d starts at %u, not %zu\n", t1, t2, t3, me >> 12, entries); return 6; }
          int seq[8];
          for (int i = 0; i < 8; ++i) seq[i] = i < t1 ? 0 : i < t2 ? 1 : i < t3 ? 2 : 3;
          uint32_t r = 0;
          do {
            uint64_t want = 0;
            for (int i = 0; i < 8; ++i) want |= (uint64_t)(3 - seq[i]) << (8 * i);
            if (cb.tail_codes[entries + r] != want) { std::fprintf(stderr, "walk tail: multiset %d %d %d, rank %u\n", t1, t2, t3, r); return 6; }
            ++r;
          } while (std::next_permutation(seq, seq + 8));
          if (r != (me & 0xFFFu)) { std::fprintf(stderr, "walk tail: multiset %d %d %d has %u arrangements, table says %u\n", t1, t2, t3, r, me & 0xFFFu); return 6; }
          entries += r;
        }
    if (entries != 65536) { std::fprintf(stderr, "walk tail: %zu entries\n", entries); return 6; }
  }
  // rotation tables of served and awkward widths (an odd factor above 32 is a refusal, not a fault)
  size_t rotations = 0;
  for (uint32_t n : {1u, 8u, 24u, 104u, 256u, 1000u, 2560u, 2568u, 4096u, 9728u, 17408u}) {
    RotationTables t;
    std::string why;
    if (!build_rotation(n, next_u64(), &t, &why)) continue;
    std::vector<double> v(n);
    for (uint32_t i = 0; i < n; ++i) v[i] = (double)(int64_t)(next_u64() >> 40) / (double)(1 << 23) - 1.0;
    double before = 0, after = 0;
    for (double x : v) before += x * x;
    host_rotate(t, &v);
    for (double x : v) after += x * x;
    if (!(after > 0.999 * before && after < 1.001 * before)) { std::fprintf(stderr, "rotation of width %u does not keep the norm\n", n); return 4; }
    ++rotations;
  }
  // the batched launch's work sharing: every slice has exactly one owner, workgroups hold consecutive
  // slices, loads differ by at most one, and no band receives more partial sums than the workspace holds
  size_t shares = 0;
  for (uint32_t cap : {1u, 3u, 256u, 304u})
    for (uint32_t spb : {1u, 2u, 7u, 11u, 26u, 32u, 46u, 683u})
      for (uint32_t bands : {1u, 2u, 5u, 16u, 40u, 96u, 192u, 255u, 256u, 257u, 304u, 1000u}) {
        const uint64_t total = (uint64_t)bands * spb;
        const GemmShare sh = gemm_share(bands, spb, cap);
        if (sh.n_wg == 0 || sh.n_wg > cap || sh.n_wg > total) { std::fprintf(stderr, "share: bad workgroup count\n"); return 5; }
        if (sh.shared0 != sh.whole * sh.n_wg || sh.shared0 > bands || bands - sh.shared0 >= sh.n_wg) { std::fprintf(stderr, "share: bands walked alone\n"); return 5; }
        const uint64_t left = (uint64_t)(bands - sh.shared0) * spb;
        if (!gemm_share_exact(sh, bands, spb)) { std::fprintf(stderr, "share: multipliers not exact\n"); return 5; }
        // the multipliers against plain division, over every dividend the walk can form
        for (uint32_t nq = 0; nq <= (uint32_t)left + spb; ++nq)
          if (share_div(nq, sh.inv_spb) != nq / spb || share_div(nq, sh.inv_base1) != nq / (sh.base + 1u) ||
              (sh.base && share_div(nq, sh.inv_base) != nq / sh.base)) { std::fprintf(stderr, "share: multiplier wrong at %u\n", nq); return 5; }
        if (gemm_first_slice(0, sh.base, sh.rem) != 0 || gemm_first_slice(sh.n_wg, sh.base, sh.rem) != left) { std::fprintf(stderr, "share: slices not covered\n"); return 5; }
        // every workgroup's walk, run by run as the kernel walks it: each slice of each band exactly once, pieces numbered
        // 0.. in workgroup order, loads within one slice of each other
        std::vector<uint8_t> seen((size_t)total, 0);
        std::vector<uint32_t> pieces_seen(bands, 0);
        uint32_t lo_load = ~0u, hi_load = 0;
        for (uint32_t c = 0; c < sh.n_wg; ++c) {
          const uint32_t n = gemm_slices_of(sh, spb, c);
          lo_load = n < lo_load ? n : lo_load;
          hi_load = n > hi_load ? n : hi_load;
          for (uint32_t t = 0; t < n;) {
            const GemmRun r = gemm_run_at(sh, spb, c, t);
            if (r.band >= bands || r.len == 0 || r.lo + r.len > spb || t + r.len > n) { std::fprintf(stderr, "share: run out of range\n"); return 5; }
            if (r.band < sh.shared0 && (r.lo != 0 || r.len != spb || r.piece != 0)) { std::fprintf(stderr, "share: a band walked alone is not whole\n"); return 5; }
            if (r.piece != pieces_seen[r.band]++) { std::fprintf(stderr, "share: piece numbering\n"); return 5; }
            for (uint32_t k = 0; k < r.len; ++k)
              if (seen[(size_t)r.band * spb + r.lo + k]++) { std::fprintf(stderr, "share: slice walked twice\n"); return 5; }
            t += r.len;
          }
        }
        if (hi_load - lo_load > 1) { std::fprintf(stderr, "share: uneven load\n"); return 5; }
        for (uint64_t k = 0; k < total; ++k)
          if (!seen[(size_t)k]) { std::fprintf(stderr, "share: slice not walked\n"); return 5; }
        for (uint32_t b = 0; b < bands; ++b)
          if (pieces_seen[b] != gemm_pieces_of(sh, spb, b) || pieces_seen[b] > sh.max_pieces) {
            std::fprintf(stderr, "share: %u pieces in band %u, formula %u, %u slots\n", pieces_seen[b], b, gemm_pieces_of(sh, spb, b), sh.max_pieces);
            return 5;
          }
        ++shares;
      }
  std::printf("ok: %zu records in the whole file, %zu hostile inputs, %zu decodable ranks, %zu rotations, %zu work shares\n", whole, cases, valid, rotations, shares);
  return 0;
}
