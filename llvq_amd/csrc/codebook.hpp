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
constexpr int kStartsPadded = 512; // class starts, padded with UINT64_MAX past N(13)
constexpr int kStartsLds = 320;    // what a 47-bit index can reach (class <= 317) plus its upper neighbour; the rare wide search reads the padded table
constexpr int kFastLds = 320;      // fast-path class records a 47-bit index can reach
constexpr int kLutShift = 36;      // class-find table is keyed on the index as a record holds it (1 .. N) >> 36
constexpr int kOnLutSlots = 4352;  // LDS slots for the support-arrangement table (4322 entries used)
constexpr int kLutSize = 4096;     // covers every index <= N(13) < 2^48 (a 47-bit field uses the lower half)
constexpr int kLut2Shift = 31;     // second-level buckets of the class-find table
constexpr int kLut2Span = 1 << (kLutShift - kLut2Shift);  // entries of a second-level table
constexpr int kLut2Lds = 54 * kLut2Span;  // second-level entries the lower half of the first level refers to (53 tables)
// Class-find table entries (16 bits).  First level, keyed on the index as a record holds it >> kLutShift:
//   bit 15 clear: the entry is where a second-level table begins in lut2 (a multiple of kLut2Span), that table
//   keyed on (index >> kLut2Shift) % kLut2Span; bit 15 set (kLutFinal): a final entry.  Every second-level entry is
//   final, with or without the bit.  Final entry (either level): bits 0..8 = class c0 holding the bucket's first
//   index; bit 13 clear: the bucket meets at most one class start, so the class is c0 or c0 + 1
//   (one comparison with starts[c0 + 1]) and bits 9..10 / 11..12 are the decoders of c0 / c0 + 1
//   (kLutKind*); bit 13 set: the bucket meets several class starts, bits 9..11 = k with the class
//   at most 2^k - 1 further, found by a halving search.
constexpr uint32_t kLutFinal = 0x8000u, kLutWide = 0x2000u;
enum : uint32_t { kLutKindOdd = 0, kLutKindEven = 1, kLutKindEvenSecond = 2, kLutKindGeneric = 3 };

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

// LDS-resident class record of the two fast decode paths, 48 bytes.
//   odd-coset walk:   inv0 = 1/m_arr, d1 = m_arr, u0 = packed thresholds, tab = signed value table
//   even-coset table: inv0 = 1/a_off, d1 = 1/a_on, u0 = first on_lut entry | second free value << 16,
//                     u1 = first off_lut entry, a_off/a_on as floats (both < 2^24), tab = signed value table
// `tab` is the 8-byte table a byte-permute indexes with a 3-bit code per coordinate:
//   odd:  code = (3 - kind) | (off-support ? 4 : 0); bytes 0..3 = a_kind, bytes 4..7 = -a_kind
//   even: code = on-support | primary-kind << 1 | minus << 2
struct alignas(16) FastClass {
  double inv0;
  double d1;
  uint32_t u0, u1;
  float inv_norm;
  uint32_t meta;     // kMeta* fields, path in bits 17..18, golay_base in bits 20..31
  float a_off, a_on;
  uint32_t tab_lo, tab_hi;
};
static_assert(sizeof(FastClass) == 48, "FastClass must stay 48 bytes");

constexpr int kMetaPathShift = 17;         // bits 17..18: which decoder a class takes
constexpr uint32_t kMetaSecondFree = 1u << 19;  // even-coset fast path: the class has a second non-zero off-support kind
constexpr int kMetaGolayShift = 20;        // bits 20..31: first codeword of the weight bucket
enum : uint32_t { kPathOdd = 0, kPathEven = 1, kPathGeneric = 2 };
constexpr int kTailSlots = 8;             // slots of the odd-coset walk that are looked up, not walked
constexpr int kTailMetaSlots = 732;       // 9^3 threshold triples, padded to a multiple of four
constexpr int kTailCodeSlots = 65536 + 2520;  // 4^8 arrangements, and the padding

struct Codebook {
  uint32_t golay[4096];
  int bucket_start[26];
  std::vector<ClassDef> classes;          // 383, format order
  // device-shaped tables
  DevClass dev_classes[kClassSlots];
  uint64_t starts[kStartsPadded];         // starts[c] = offset of class c + 1 (the first index of class c as a record holds it), starts[383] = N(13) + 1, then UINT64_MAX
  uint16_t lut[kLutSize];                 // first level of the class-find table (see kLutFinal)
  std::vector<uint16_t> lut2;             // its second-level tables, those of the lowest keys first
  double rcp[32];                         // rcp[c] = 1/c, rcp[0] unused
  // step[(m * 25 + c) * 2 + {0,1}] = {m / c, 1 - m / c}: the odd-coset walk's per-slot
  // update t' + 1 = (t + 1 - lo) * (m / c) + (1 - m / c), m = slots left after this one
  double step[24 * 25 * 2];
  // The last kTailSlots slots of the odd-coset walk are one table read.  With eight slots left the
  // walk's state is the three thresholds T1 <= T2 <= T3 <= 8 (counts of the four kinds still to
  // place) and a rank below the remaining multiset's arrangement count M <= 2520:
  // tail_meta[T1 + 9 T2 + 81 T3] = M | first entry << 12, and tail_codes[first + rank] holds the
  // eight slots' table codes (3 - kind), one per byte, first slot in the lowest byte — what the
  // walk itself produces, which is how the table is filled.  Padded so that any rank below 2520
  // stays inside the table.
  uint32_t tail_meta[kTailMetaSlots];
  std::vector<uint64_t> tail_codes;
  uint64_t n12 = 0;                       // points in the cap-12 ball (47-bit field)
  // fast paths
  FastClass fast[kClassSlots];
  // Arrangement tables of the even coset, slot space: entry r of a problem is the
  // r-th arrangement in lexicographic order (index.rs:97-117) as two 16-bit slot
  // masks, kind 0 in the low half and kind 1 in the high half.
  std::vector<uint32_t> on_lut;           // support problems (w in {8,12,16}, at most 2 word kinds)
  std::vector<uint32_t> off_lut;          // off-support problems (24-w slots, free kinds then the zero run)
  // Per codeword, the five move masks that deposit slot bits onto the set
  // positions of the word (dwords 0..3) and onto its unset positions (4..7).
  uint32_t expand[4096][8];
  uint8_t pdep4[256];                     // pdep4[mask << 4 | bits]: low bits of `bits` onto the set bits of `mask`
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
