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
//  * Multiset-permutation unranking without ever forming an arrangement count.
//    With M arrangements of the remaining multiset, n slots left and kind
//    counts c_0.. (prefix sums T_0 = 0, T_1, ...), the reference picks the
//    kind j with  M T_j / n <= rank < M T_{j+1} / n  and continues with
//    rank' = rank - M T_j / n,  M' = M c_j / n  (fastdec.rs:173-194).  Writing
//    rho = (rank + 1/2) / M  this is:  t = rho n;  j = the kind of sorted
//    element floor(t);  rho' = (t - T_j) / c_j  — and rho' equals
//    (rank' + 1/2) / M' exactly, so the half-unit guard band travels with the
//    recurrence.  A decision is wrong only if the accumulated error of rho,
//    measured in units of 1/M, reaches 1/2; that error grows by about 2^-52 M_i
//    per step and M <= 5 354 228 880 < 2^33, so FP64 leaves a factor > 2^10.
//
//  * The k-1 comparisons of one step are done at once on thresholds packed
//    into 6-bit fields of one register (a guard bit per field turns the
//    per-field comparison into one subtraction), so a step costs the same for
//    2 and for 5 kinds and needs no per-lane indexed registers.
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
  const uint32_t* golay;   // 4096 codewords, canonical order
  const DevClass* cls;     // kClassSlots records
  const uint64_t* ends;    // kEndsPadded class ends
  const double* rcp;       // rcp[c] = 1/c for c in 1..24
};

// Threshold packing: field f (bits 6f..6f+4) holds T_{4-f}; bit 6f+5 is the
// field's guard bit.  Fields of kinds a problem does not have hold n.
constexpr uint32_t kFieldOnes = 1u | (1u << 6) | (1u << 12) | (1u << 18);
constexpr uint32_t kFieldGuard = kFieldOnes << 5;

LLVQ_HD uint32_t popc32(uint32_t v) {
#if defined(__HIP_DEVICE_COMPILE__)
  return (uint32_t)__popc(v);
#else
  return (uint32_t)__builtin_popcount(v);
#endif
}

LLVQ_HD double floor64(double v) {
#if defined(__HIP_DEVICE_COMPILE__)
  return __builtin_floor(v);
#else
  return __builtin_floor(v);
#endif
}

LLVQ_HD double fma64(double a, double b, double c) { return __builtin_fma(a, b, c); }

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

// Count of class ends <= i over the padded table: fixed nine probes.
LLVQ_HD uint32_t find_class(const uint64_t* ends, uint64_t i) {
  uint32_t lo = 0;
#pragma unroll
  for (uint32_t step = 256; step >= 1; step >>= 1)
    if (ends[lo + step - 1] <= i) lo += step;
  return lo;
}

// Decodes `idx` and calls emit(position, value) for positions 0..23 in order.
// Returns the class index, -1 for the origin, -2 for an index past N(13)
// (which emits zeros).
template <class Emit>
LLVQ_HD int decode_index(const DecodeTables& T, uint64_t idx, Emit&& emit) {
  if (idx == 0 || idx > kN13) {
    for (int p = 0; p < kDim; ++p) emit(p, 0);
    return idx == 0 ? -1 : -2;
  }
  const uint64_t i = idx - 1;
  uint32_t ci = find_class(T.ends, i);
  if (ci > 382u) ci = 382u;
  const uint64_t offset = ci ? T.ends[ci - 1] : 0;
  const DevClass c = T.cls[ci];
  uint64_t li = i - offset;

  if (c.meta & kMetaOdd) {
    // local = g * m_arr + r_arr  (index.rs:33-36)
    const double local = (double)li;
    const double g = floor64((local + 0.5) * c.inv0);
    const double r = fma64(-g, c.m0, local);
    double rho = (r + 0.5) * c.inv0;
    const uint32_t cw = T.golay[(uint32_t)g & 4095u];
    uint32_t tg = c.tg0;
#pragma unroll
    for (int p = 0; p < kDim; ++p) {
      const uint32_t jj = walk_step(rho, tg, (uint32_t)(kDim - p), T.rcp);
      const int v = (int)((c.vals0 >> (4u * jj)) & 15u);
      // forced signs (index.rs:417-431): a = v if v = 3 mod 4 else -v; a on the
      // codeword's support, -a off it.
      const uint32_t neg = ((cw >> p) ^ ((uint32_t)v >> 1)) & 1u;
      emit(p, neg ? -v : v);
    }
    return (int)ci;
  }

  // local = (((g A_on + r_on) A_off + r_off) S_w + r_sw) S_f + r_sf  (index.rs:24-32)
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
  // word signs: bit s of r_sw for support slot s < w-1, the last one forced by
  // the parity rule (index.rs:375-388)
  uint32_t signs_on = r_sw | (((popc32(r_sw) & 1u) ^ p_req) << sw);
  uint32_t tg_on = c.tg1, tg_off = c.tg0;
  uint32_t n_on = w, n_off = kDim - w;
#pragma unroll
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
      // free signs are consumed by the nonzero off-support slots only
      // (index.rs:403-415); the zero run is recognised by its value
      neg = v ? (r_sf & 1u) : 0u;
      r_sf >>= (v ? 1 : 0);
    }
    emit(p, neg ? -v : v);
  }
  return (int)ci;
}

}  // namespace llvq
