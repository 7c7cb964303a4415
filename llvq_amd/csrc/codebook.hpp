// Host-side construction of the LLVQ format-v1 codebook tables and their
// device-shaped packing.
//
// What is built here is the data the index format is defined by
// (llvq-search/src/index.rs:12-22): the extended Golay code in its canonical
// order (llvq-core/src/golay.rs:62-81), the class list in format order
// (llvq-search/src/classes.rs:144-254, index.rs:125-176) and, per class, the
// radices of the local rank (index.rs:24-36).  The construction below is an
// independent formulation (linear span for the code, recursive multiset
// generation plus an explicit sort key for the classes); it is checked against
// the published codebook fingerprint at runtime creation.
#pragma once
#include <cstdint>
#include <vector>

namespace llvq {

constexpr int kDim = 24;
constexpr uint64_t kN13 = 280974212784720ULL;  // llvq-core/src/leech.rs:54
constexpr uint64_t kFingerprint = 0x338f420f11866319ULL;  // llvq-artifact/tests/codebook_fingerprint.rs:58
constexpr int kMaxShell = 13;
constexpr int kClassSlots = 384;   // 383 classes + one sentinel, a power-of-two-friendly size
constexpr int kEndsPadded = 512;   // class ends padded for a fixed-depth search

struct KindCount {
  int value;
  int count;
};

// One equivalence class (parity coset, multiset of |values|) with its radices.
struct ClassDef {
  int shell = 0;
  bool odd = false;
  // even coset
  int w = 0;      // Golay weight of the support
  int p_req = 0;  // required parity of minus signs on the support
  std::vector<KindCount> word;  // values = 2 mod 4, descending
  std::vector<KindCount> free;  // values = 0 mod 4, nonzero, descending
  int n0 = 0;                   // zeros off the support
  uint64_t a_on = 1, a_off = 1; // arrangement counts on / off the support
  int sw_bits = 0, sf_bits = 0; // log2 of the sign radices
  // odd coset
  std::vector<KindCount> vals;  // descending, counts sum to 24
  uint64_t m_arr = 1;
  // layout
  uint64_t offset = 0, card = 0;
};

// Device-shaped class record, 64 bytes.  Problem 0 is the 24-slot arrangement
// of an odd class or the off-support arrangement of an even class; problem 1
// is the on-support arrangement of an even class.
struct alignas(16) DevClass {
  double m0, inv0;  // arrangement count of problem 0 and its reciprocal
  double m1, inv1;  // same for problem 1 (1.0 when unused)
  uint32_t tg0;     // packed prefix-sum thresholds of problem 0 (see decode_core.h)
  uint32_t tg1;     // same for problem 1
  uint32_t vals0;   // |value| per kind of problem 0, one nibble each, indexed by 4 - kind
  uint32_t vals1;   // same for problem 1
  uint32_t meta;    // see kMeta* below
  float inv_norm;   // 1 / sqrt(16 * shell)
  uint32_t shell;
  uint32_t golay_base;  // first codeword of the weight bucket (0 for odd classes)
};
static_assert(sizeof(DevClass) == 64, "DevClass must stay 64 bytes");

constexpr uint32_t kMetaOdd = 1u;          // bit 0
constexpr int kMetaWShift = 1;             // bits 1..5   support weight
constexpr int kMetaPreqShift = 6;          // bit 6       p_req
constexpr int kMetaSfShift = 7;            // bits 7..11  free-sign bits
constexpr int kMetaSwShift = 12;           // bits 12..16 support-sign bits (w-1, or 0)

struct Codebook {
  uint32_t golay[4096];
  int bucket_start[26];
  std::vector<ClassDef> classes;          // 383, format order
  // device-shaped tables
  DevClass dev_classes[kClassSlots];
  uint64_t ends[kEndsPadded];             // offset + card per class, then UINT64_MAX
  double rcp[32];                         // rcp[c] = 1/c, rcp[0] unused
  uint64_t n12 = 0;                       // points in the cap-12 ball (47-bit field)
};

const Codebook& codebook();

// ceil(log2(N(cap))) with a floor of 1 — llvq-quant/src/quantizer.rs:572-576.
int index_bits(uint32_t cap);

// Digest of the index map — llvq-artifact/src/codebook.rs:129-185 — computed
// with this library's tables and host decoder.
uint64_t codebook_fingerprint();

// Decode with the same arithmetic the kernels run (decode_core.h).
bool host_decode(uint64_t idx, int8_t point[kDim], int* shell);

}  // namespace llvq
