// Unranking of a format-v1 index into its 24 lattice coordinates — the one
// piece of arithmetic shared by the kernels and by the host mirror that the
// fingerprint check and the CPU tests run.  Compiled for gfx950 by hipcc and
// for the host by the same translation units.
//
// What it computes is the map of llvq-search/src/index.rs:334-435 (equivalently
// fastdec.rs:321-399).  How it computes it is different, and chosen for a
// 64-lane SIMD with full-rate FP64 and slow 64-bit integer multiply/divide:
//
//  * Mixed-radix split of the local rank by FP64 multiplication with a stored
//    reciprocal.  q = floor((x + 1/2) * (1/d)) is exact whenever x < 2^51: the
//    true quotient (x + 1/2)/d is at least 1/(2d) away from every integer,
//    the computed one is off by at most q * 2^-52, and q * d <= x.
//
//  * Odd coset — multiset-permutation unranking without ever forming an
//    arrangement count.  With M arrangements of the remaining multiset, n slots
//    left and kind counts c_0.. (prefix sums T_0 = 0, T_1, ...), the reference
//    picks the kind j with  M T_j / n <= rank < M T_{j+1} / n  and continues
//    with rank' = rank - M T_j / n,  M' = M c_j / n  (fastdec.rs:173-194).
//    Writing rho = (rank + 1/2) / M  this is:  t = rho n;  j = the kind of
//    sorted element floor(t);  rho' = (t - T_j) / c_j  — and rho' equals
//    (rank' + 1/2) / M' exactly, so the half-unit guard band travels with the
//    recurrence.  A decision is wrong only if the accumulated error of rho,
//    measured in units of 1/M, reaches 1/2; that error grows by about
//    2^-52 M_i per step and M <= 5 354 228 880 < 2^33, so FP64 leaves a factor
//    > 2^10.  The k-1 comparisons of one step are done at once on thresholds
//    packed into 6-bit fields of one register (a guard bit per field turns the
//    per-field comparison into one subtraction).
//
//  * Even coset (support weight 8, 12 or 16, at most two word kinds — all but
//    0.04 % of uniformly drawn blocks) — no walk at all.  The two arrangement
//    ranks index tables of slot masks; slot masks and sign bits are moved to
//    coordinate positions by a five-step parallel bit deposit whose move masks
//    are stored per codeword.
//
//  * Every path ends in a 3-bit code per coordinate, four codes per dword, that
//    a byte permute turns into signed 8-bit lattice coordinates.
//
// Classes outside the fast paths (five magnitudes on the odd coset, support
// weight 0 or 24, three word kinds) take the generic walk of both cosets.
#pragma once
#include <cstdint>

#include "codebook.hpp"

#if defined(__HIPCC__)
#include <hip/hip_runtime.h>
#define LLVQ_HD __host__ __device__ __forceinline__
#else
#define LLVQ_HD inline
#endif

namespace llvq {

struct DecodeTables {
  const uint32_t* golay;    // 4096 codewords, canonical order
  const DevClass* cls;      // generic-walk class records
  const FastClass* fast;    // fast-path class records
  const uint64_t* starts;   // starts[c] = first index of class c as a record holds it (class 0 begins at 1); starts[383] = N(13) + 1 (a kernel's copy may end at kStartsLds)
  const uint64_t* starts_far;  // the whole padded table, for the wide search
  const uint16_t* lut;      // class-find table, first level (kLutFinal in codebook.hpp)
  const uint16_t* lut2;     // its second-level tables
  const double* rcp;        // rcp[c] = 1/c for c in 1..24
  const uint32_t* on_lut;   // even coset, support arrangements
  const uint32_t* off_lut;  // even coset, off-support arrangements
  const uint32_t* expand;   // 8 dwords per codeword: deposit masks for the word and for its complement
  const uint8_t* pdep4;     // 4-bit deposit table
  const double* step;       // {m/c, 1 - m/c} pairs, see Codebook::step (rows m >= kTailSlots are read)
  const uint32_t* tail_meta;   // the walk's last kTailSlots slots, see Codebook::tail_meta
  const uint64_t* tail_codes;
};

// Threshold packing: field f (bits 6f..6f+4) holds T_{4-f}; bit 6f+5 is the
// field's guard bit.  Fields of kinds a problem does not have hold n.
constexpr uint32_t kFieldOnes = 1u | (1u << 6) | (1u << 12) | (1u << 18);
constexpr uint32_t kFieldGuard = kFieldOnes << 5;

// bit k of a nibble -> bit 0 / 1 / 2 of byte k
constexpr uint32_t kSpread0 = 0x00204081u, kSpread1 = 0x00408102u, kSpread2 = 0x00810204u;

LLVQ_HD uint32_t popc32(uint32_t v) {
#if defined(__HIP_DEVICE_COMPILE__)
  return (uint32_t)__popc(v);
#else
  return (uint32_t)__builtin_popcount(v);
#endif
}

// a * b + c with 24-bit signed factors (one full-rate instruction on the device)
LLVQ_HD int mad24(int a, int b, int c) {
#if defined(__HIP_DEVICE_COMPILE__)
  int r;  // the compiler would widen this to a 64-bit multiply-add
  asm("v_mad_i32_i24 %0, %1, %2, %3" : "=v"(r) : "v"(a), "s"(b), "v"(c));
  return r;
#else
  return a * b + c;
#endif
}

LLVQ_HD double floor64(double v) { return __builtin_floor(v); }
// x < 2^52 as a double, exactly: the integer dropped into the mantissa of 2^52, which is then
// taken away (two instructions; the compiler's general conversion of a 64-bit integer takes four)
LLVQ_HD double small_u64_to_double(uint64_t x) {
  return __builtin_bit_cast(double, x | 0x4330000000000000ULL) - 4503599627370496.0;
}
LLVQ_HD double fma64(double a, double b, double c) { return __builtin_fma(a, b, c); }
LLVQ_HD uint32_t bfi32(uint32_t mask, uint32_t a, uint32_t b) { return (a & mask) | (b & ~mask); }

// signed byte `code` (0..7) of the 8-byte table {hi:lo}
LLVQ_HD int table_byte(uint32_t lo, uint32_t hi, uint32_t code) {
  const uint32_t w = code & 4u ? hi : lo;
  return (int)(int8_t)(w >> (8u * (code & 3u)));
}

// One slot of the arrangement walk.  Returns jj = 4 - kind.
LLVQ_HD uint32_t walk_step(double& rho, uint32_t& tg, uint32_t n, const double* rcp) {
  const double t = rho * (double)n;
  const uint32_t ti = (uint32_t)t;
  const uint32_t e = tg - (ti + 1u) * kFieldOnes;  // guard survives iff T_m > ti
  const uint32_t lt = (e >> 5) & kFieldOnes;
  const uint32_t jj = popc32(lt);
  const uint32_t sh = jj * 6u;
  const uint32_t lo = (tg >> sh) & 31u;
  const uint32_t hi = (((tg << 6) | n) >> sh) & 31u;
  tg -= lt;  // every threshold above the chosen kind loses one element
  rho = (t - (double)lo) * rcp[hi - lo];
  return jj;
}

// Final class-find entry of the index 1 <= i <= N(13), as a record holds it: one table probe on the top bits and,
// where that bucket meets several class starts, one on the bits below.
LLVQ_HD uint32_t class_entry(const DecodeTables& T, uint64_t i) {
  uint32_t e = T.lut[(uint32_t)(i >> kLutShift)];
  if (!(e & kLutFinal)) e = T.lut2[e + ((uint32_t)(i >> kLut2Shift) & (uint32_t)(kLut2Span - 1))];
  return e;
}
// The class from its entry: one comparison, or (0.09 % of uniformly drawn indices) a halving
// search over at most 2^k classes.  starts_far is padded with UINT64_MAX.
LLVQ_HD uint32_t class_from_entry(const DecodeTables& T, uint32_t e, uint64_t i) {
  uint32_t ci = e & 511u;
  if (!(e & kLutWide)) return ci + (T.starts_far[ci + 1u] <= i ? 1u : 0u);
  for (uint32_t step = (1u << ((e >> 9) & 7u)) >> 1; step; step >>= 1)
    if (T.starts_far[ci + step] <= i) ci += step;
  return ci;
}
LLVQ_HD uint32_t find_class(const DecodeTables& T, uint64_t i) { return class_from_entry(T, class_entry(T, i), i); }

// ---- odd coset, fast path (at most four magnitudes) ------------------------------
// local = g * m_arr + r_arr (index.rs:33-36).  Calls on_codes(q, sel) for q = 0..5:
// byte j of sel is the table code of coordinate 4q + j,
// code = (3 - kind) | (coordinate off the codeword's support ? 4 : 0).
// The walk carries t + 1 = rho n + 1 instead of rho: floor(t + 1) is the operand
// of the packed comparison, and the next slot's value is one fused multiply-add,
// (t + 1 - T_j) (m / c_j) + (1 - m / c_j) with m = n - 1, both factors from one
// 16-byte table entry.
// One slot of the walk: n slots are left, the kind's code 4 - kind is returned.
LLVQ_HD uint32_t odd_walk_slot(const DecodeTables& T, uint32_t n, double& t1, uint32_t& tg) {
  const uint32_t ti1 = (uint32_t)t1;                      // floor(t) + 1
  const uint32_t ltg = (uint32_t)mad24((int)ti1, -(int)kFieldOnes, (int)tg) & kFieldGuard;  // guard survives iff T_m > floor(t)
  const uint32_t jj = popc32(ltg);                        // 4 - kind
  const uint32_t sh = jj * 6u;
  const uint32_t lo = (tg >> sh) & 31u;
  const uint32_t hi = (((tg << 6) | n) >> sh) & 31u;
  tg -= ltg >> 5;
  if (n > 1u) {
    const double* e = T.step + 2u * ((n - 1u) * 25u + (hi - lo));
    t1 = fma64(t1 - (double)lo, e[0], e[1]);
  }
  return jj;
}

// The first sixteen slots of the walk (n = 24 .. 9 slots left) as they are produced; ends with
// the state the table of the last eight slots is entered with.
template <class OnCodes>
LLVQ_HD void odd_walk_head(const DecodeTables& T, const FastClass& f, uint64_t li, uint32_t& ncw, double& t1, uint32_t& tg,
                           OnCodes&& on_codes) {
  const double local = small_u64_to_double(li);
  const double g = floor64((local + 0.5) * f.inv0);
  const double r = fma64(-g, f.d1, local);
  t1 = fma64((r + 0.5) * f.inv0, 24.0, 1.0);
  ncw = ~T.golay[(uint32_t)g & 4095u];
  tg = f.u0;
#pragma unroll
  for (int q = 0; q < (kDim - kTailSlots) / 4; ++q) {
    uint32_t sel = 0;
#pragma unroll
    for (int j = 0; j < 4; ++j) sel |= odd_walk_slot(T, (uint32_t)(kDim - 4 * q - j), t1, tg) << (8 * j);
    // table index = jj - 1 (kinds 0..3 <-> jj 4..1), bit 2 = off the codeword's support
    on_codes(q, (sel - 0x01010101u) | ((((ncw >> (4 * q)) & 15u) * kSpread2) & 0x04040404u));
  }
}

template <class OnCodes>
LLVQ_HD void odd_codes(const DecodeTables& T, const FastClass& f, uint64_t li, OnCodes&& on_codes) {
  uint32_t ncw, tg;
  double t1;
  odd_walk_head(T, f, li, ncw, t1, tg, on_codes);
  // The last eight slots.  t1 - 1 = 8 rho with rho = (rank + 1/2) / M for the M arrangements of
  // what is left, so rank = floor(rho M); the thresholds T3, T2, T1 sit in fields 1, 2, 3.
  const uint32_t th = tg >> 6;
  const uint32_t me = T.tail_meta[(th & 15u) * 81u + ((th >> 6) & 15u) * 9u + ((th >> 12) & 15u)];
  const uint32_t rank = (uint32_t)(fma64(t1, 0.125, -0.125) * (double)(me & 0xFFFu));
  const uint64_t codes = T.tail_codes[(me >> 12) + rank];
  on_codes(4, (uint32_t)codes | ((((ncw >> 16) & 15u) * kSpread2) & 0x04040404u));
  on_codes(5, (uint32_t)(codes >> 32) | ((((ncw >> 20) & 15u) * kSpread2) & 0x04040404u));
}

// ---- even coset, fast path --------------------------------------------------------
// Deposits bit k of x onto the k-th selected position; e = four packed move-mask
// dwords.  Bits are copied, not moved: positions outside the selection hold
// leftovers and must be masked off by the caller.
LLVQ_HD uint32_t expand24(uint32_t x, const uint32_t* e) {
  const uint32_t e0 = e[0];
  x = bfi32((e0 >> 8) & 0x00FF0000u, x << 16, x);
  x = bfi32(e[3], x << 8, x);
  x = bfi32(e[2], x << 4, x);
  x = bfi32(e[1], x << 2, x);
  x = bfi32(e0, x << 1, x);
  return x;
}

// local = (((g A_on + r_on) A_off + r_off) S_w + r_sw) S_f + r_sf  (index.rs:24-32).
// Calls on_codes(q, sel, sel2) for q = 0..5: byte j of sel is
// on-support | primary-kind << 1 | minus << 2 of coordinate 4q + j (FastClass::tab);
// byte j of sel2 is second-free-kind | minus << 2.
// SEC = false is for classes without a second free kind (FastClass::meta & kMetaSecondFree clear): their
// off-support table entries have an empty high half, and sel2 is passed as zero.
template <bool SEC = true, class OnCodes>
LLVQ_HD void even_codes(const DecodeTables& T, const FastClass& f, uint64_t li, OnCodes&& on_codes) {
  const uint32_t p_req = (f.meta >> kMetaPreqShift) & 1u;
  const uint32_t sf = (f.meta >> kMetaSfShift) & 31u;
  const uint32_t sw = (f.meta >> kMetaSwShift) & 31u;
  const uint32_t r_sf = (uint32_t)li & ((1u << sf) - 1u);
  li >>= sf;
  const uint32_t r_sw = (uint32_t)li & ((1u << sw) - 1u);
  li >>= sw;
  const double rest = small_u64_to_double(li);
  const double q1 = floor64((rest + 0.5) * f.inv0);
  const uint32_t r_off = (uint32_t)fma64(-q1, (double)f.a_off, rest);
  const double g = floor64((q1 + 0.5) * f.d1);
  const uint32_t r_on = (uint32_t)fma64(-g, (double)f.a_on, q1);
  const uint32_t gi = ((f.meta >> kMetaGolayShift) + (uint32_t)g) & 4095u;
  const uint32_t cw = T.golay[gi];
  const uint32_t* e_on = T.expand + 8u * gi;
  const uint32_t* e_off = e_on + 4;
  const uint32_t on_e = T.on_lut[(f.u0 & 0xFFFFu) + r_on];
  const uint32_t off_e = T.off_lut[f.u1 + r_off];
  // word signs: bit s of r_sw for support slot s < w-1, the last one forced by
  // the parity rule (index.rs:375-388)
  const uint32_t signs_on = r_sw | (((popc32(r_sw) & 1u) ^ p_req) << sw);
  // free signs go to the nonzero off-support slots in slot order (index.rs:403-415)
  const uint32_t nz = SEC ? (off_e | (off_e >> 16)) & 0xFFFFu : off_e & 0xFFFFu;
  uint32_t signs_off = 0, r = r_sf;
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    const uint32_t m4 = (nz >> (4 * k)) & 15u;
    signs_off |= (uint32_t)T.pdep4[m4 * 16u + (r & 15u)] << (4 * k);
    r >>= popc32(m4);
  }
  const uint32_t prim = bfi32(cw, expand24(on_e & 0xFFFFu, e_on), expand24(off_e & 0xFFFFu, e_off));
  const uint32_t sec = SEC ? expand24(off_e >> 16, e_off) & ~cw : 0u;
  const uint32_t sign = bfi32(cw, expand24(signs_on, e_on), expand24(signs_off, e_off));
#pragma unroll
  for (int q = 0; q < 6; ++q) {
    const uint32_t s2 = (((sign >> (4 * q)) & 15u) * kSpread2) & 0x04040404u;
    const uint32_t sel = ((((cw >> (4 * q)) & 15u) * kSpread0) & 0x01010101u) |
                         ((((prim >> (4 * q)) & 15u) * kSpread1) & 0x02020202u) | s2;
    const uint32_t sel2 = SEC ? ((((sec >> (4 * q)) & 15u) * kSpread0) & 0x01010101u) | s2 : 0u;
    on_codes(q, sel, sel2);
  }
}

// ---- generic walk of both cosets (rare classes) -----------------------------------
template <class Emit>
LLVQ_HD void decode_odd(const DecodeTables& T, const DevClass& c, uint64_t li, Emit&& emit) {
  const double local = (double)li;
  const double g = floor64((local + 0.5) * c.inv0);
  const double r = fma64(-g, c.m0, local);
  double rho = (r + 0.5) * c.inv0;
  const uint32_t cw = T.golay[(uint32_t)g & 4095u];
  uint32_t tg = c.tg0;
  for (int p = 0; p < kDim; ++p) {
    const uint32_t jj = walk_step(rho, tg, (uint32_t)(kDim - p), T.rcp);
    const int v = (int)((c.vals0 >> (4u * jj)) & 15u);
    // forced signs (index.rs:417-431): a = v if v = 3 mod 4 else -v; a on the
    // codeword's support, -a off it.
    const uint32_t neg = ((cw >> p) ^ ((uint32_t)v >> 1)) & 1u;
    emit(p, neg ? -v : v);
  }
}

template <class Emit>
LLVQ_HD void decode_even(const DecodeTables& T, const DevClass& c, uint64_t li, Emit&& emit) {
  const uint32_t w = (c.meta >> kMetaWShift) & 31u;
  const uint32_t p_req = (c.meta >> kMetaPreqShift) & 1u;
  const uint32_t sf = (c.meta >> kMetaSfShift) & 31u;
  const uint32_t sw = (c.meta >> kMetaSwShift) & 31u;
  uint32_t r_sf = (uint32_t)li & ((1u << sf) - 1u);
  li >>= sf;
  const uint32_t r_sw = (uint32_t)li & ((1u << sw) - 1u);
  li >>= sw;
  const double rest = (double)li;
  const double q = floor64((rest + 0.5) * c.inv0);
  const double r_off = fma64(-q, c.m0, rest);
  const double g = floor64((q + 0.5) * c.inv1);
  const double r_on = fma64(-g, c.m1, q);
  double rho_off = (r_off + 0.5) * c.inv0;
  double rho_on = (r_on + 0.5) * c.inv1;
  const uint32_t cw = T.golay[(c.golay_base + (uint32_t)g) & 4095u];
  uint32_t signs_on = r_sw | (((popc32(r_sw) & 1u) ^ p_req) << sw);
  uint32_t tg_on = c.tg1, tg_off = c.tg0;
  uint32_t n_on = w, n_off = kDim - w;
  for (int p = 0; p < kDim; ++p) {
    int v;
    uint32_t neg;
    if ((cw >> p) & 1u) {
      const uint32_t jj = walk_step(rho_on, tg_on, n_on, T.rcp);
      --n_on;
      v = (int)((c.vals1 >> (4u * jj)) & 15u);
      neg = signs_on & 1u;
      signs_on >>= 1;
    } else {
      const uint32_t jj = walk_step(rho_off, tg_off, n_off, T.rcp);
      --n_off;
      v = (int)((c.vals0 >> (4u * jj)) & 15u);
      // the zero run is recognised by its value, never by its kind index
      neg = v ? (r_sf & 1u) : 0u;
      r_sf >>= (v ? 1 : 0);
    }
    emit(p, neg ? -v : v);
  }
}

// Decodes `idx` and calls emit(position, value) for positions 0..23 in order,
// taking the same path the GEMV kernel takes for the index's class.  Returns
// the class index, -1 for the origin, -2 for an index past N(13) (zeros).
template <class Emit>
LLVQ_HD int decode_index(const DecodeTables& T, uint64_t idx, Emit&& emit) {
  if (idx == 0 || idx > kN13) {
    for (int p = 0; p < kDim; ++p) emit(p, 0);
    return idx == 0 ? -1 : -2;
  }
  const uint32_t ci = find_class(T, idx);
  const uint64_t li = idx - T.starts[ci];
  const FastClass f = T.fast[ci];
  const uint32_t path = (f.meta >> kMetaPathShift) & 3u;
  if (path == kPathOdd) {
    odd_codes(T, f, li, [&](int q, uint32_t sel) {
      for (int j = 0; j < 4; ++j) emit(4 * q + j, table_byte(f.tab_lo, f.tab_hi, (sel >> (8 * j)) & 7u));
    });
  } else if (path == kPathEven) {
    const int fv1 = (int)(f.u0 >> 16);
    auto on_codes = [&](int q, uint32_t sel, uint32_t sel2) {
      for (int j = 0; j < 4; ++j) {
        const uint32_t c2 = (sel2 >> (8 * j)) & 7u;
        const int second = (c2 & 1u) ? ((c2 & 4u) ? -fv1 : fv1) : 0;
        emit(4 * q + j, table_byte(f.tab_lo, f.tab_hi, (sel >> (8 * j)) & 7u) + second);
      }
    };
    // the two instantiations the GEMV kernel bins even-coset blocks into
    if (f.meta & kMetaSecondFree) even_codes<true>(T, f, li, on_codes);
    else even_codes<false>(T, f, li, on_codes);
  } else {
    const DevClass c = T.cls[ci];
    if (c.meta & kMetaOdd) decode_odd(T, c, li, emit);
    else decode_even(T, c, li, emit);
  }
  return (int)ci;
}

}  // namespace llvq
