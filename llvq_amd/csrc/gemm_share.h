// How a batched launch shares its K-slices out over the workgroups: plain integer
// arithmetic, used by the kernels, by the host code that sizes the workspace, and by
// the host tests.
//
// A band (64 weight rows) is `spb` slices.  Where a launch has at least as many bands as
// workgroups, every workgroup first walks `whole` bands alone, from the first slice to the
// last: those bands have one partial sum and need no workspace.  The bands left over
// (fewer than there are workgroups) are numbered slice by slice, and workgroup c walks the
// consecutive slices [gemm_first_slice(c), gemm_first_slice(c + 1)) of that sequence:
// base + 1 of them for c < rem, base otherwise.  A left-over band whose slices fall to
// several workgroups gets one partial sum ("piece") from each, at most max_pieces of them.
#pragma once

#include <cstdint>

#if defined(__HIPCC__)
#include <hip/hip_runtime.h>
#define LLVQ_SHARE_FN __host__ __device__ inline
#else
#define LLVQ_SHARE_FN inline
#endif

namespace llvq {

struct GemmShare {
  uint32_t n_wg;        // workgroups of the launch (at most one per CU, at most one per slice)
  uint32_t whole;       // bands every workgroup walks alone: workgroup c has bands [c whole, c whole + whole)
  uint32_t shared0;     // the first left-over band: whole * n_wg
  uint32_t base, rem;   // of the left-over bands' slices workgroup c walks base + (c < rem)
  uint32_t max_pieces;  // partial sums a left-over band can receive (1 if there is none)
  // multipliers that divide by spb, base + 1 and base (share_div): a kernel divides with one multiply
  uint32_t inv_spb, inv_base1, inv_base;
};

// n / d for the d that `magic` was made for (share_magic), exact while n * d < 2^32
LLVQ_SHARE_FN uint32_t share_magic(uint32_t d) { return d > 1u ? (uint32_t)((1ULL << 32) / d) + 1u : 0u; }
LLVQ_SHARE_FN uint32_t share_div(uint32_t n, uint32_t magic) {
#if defined(__HIP_DEVICE_COMPILE__)
  return magic ? __umulhi(n, magic) : n;
#else
  return magic ? (uint32_t)(((uint64_t)n * magic) >> 32) : n;
#endif
}

// n_bands x spb slices (> 0), spread over at most `cap` workgroups
LLVQ_SHARE_FN GemmShare gemm_share(uint32_t n_bands, uint32_t spb, uint32_t cap) {
  GemmShare s;
  const uint64_t total = (uint64_t)n_bands * spb;
  s.n_wg = total < cap ? (uint32_t)total : cap;
  s.whole = n_bands / s.n_wg;  // 0 unless there are at least as many bands as workgroups
  s.shared0 = s.whole * s.n_wg;
  const uint64_t left = (uint64_t)(n_bands - s.shared0) * spb;
  s.base = (uint32_t)(left / s.n_wg);
  s.rem = (uint32_t)(left % s.n_wg);
  // a run of spb slices starting anywhere meets at most ceil((spb - 1) / base) + 1 workgroups;
  // with fewer slices than workgroups (base = 0) every slice of a band has its own
  s.max_pieces = left == 0 ? 1u : (s.base == 0 ? spb : (spb + s.base - 1) / s.base + 1);
  s.inv_spb = share_magic(spb);
  s.inv_base1 = share_magic(s.base + 1u);
  s.inv_base = share_magic(s.base);
  return s;
}

// Whether the multipliers are exact for every quotient the walk forms: the largest dividend is below
// the left-over slice count or a workgroup's slice count, the largest divisor is spb.
LLVQ_SHARE_FN bool gemm_share_exact(const GemmShare& s, uint32_t n_bands, uint32_t spb) {
  const uint64_t left = (uint64_t)(n_bands - s.shared0) * spb, mine = (uint64_t)s.whole * spb + s.base + 1u;
  const uint64_t n = left > mine ? left : mine;
  return n * spb < (1ULL << 32);
}

// the first left-over slice of workgroup c (c = n_wg gives their count)
LLVQ_SHARE_FN uint32_t gemm_first_slice(uint32_t c, uint32_t base, uint32_t rem) {
  return c * base + (c < rem ? c : rem);
}

// the workgroup that walks left-over slice g
LLVQ_SHARE_FN uint32_t gemm_owner(const GemmShare& s, uint32_t g) {
  const uint32_t head = s.rem * (s.base + 1u);
  return g < head ? share_div(g, s.inv_base1) : s.rem + share_div(g - head, s.inv_base);
}

// slices workgroup c walks in all
LLVQ_SHARE_FN uint32_t gemm_slices_of(const GemmShare& s, uint32_t spb, uint32_t c) {
  return s.whole * spb + gemm_first_slice(c + 1u, s.base, s.rem) - gemm_first_slice(c, s.base, s.rem);
}

// partial sums of a band: 1 for a band walked alone, else one per workgroup that met its slices
LLVQ_SHARE_FN uint32_t gemm_pieces_of(const GemmShare& s, uint32_t spb, uint32_t band) {
  if (band < s.shared0) return 1u;
  const uint32_t b = band - s.shared0;
  return gemm_owner(s, (b + 1u) * spb - 1u) - gemm_owner(s, b * spb) + 1u;
}

// The run (consecutive slices of one band) that starts at the t-th slice workgroup c walks;
// t must be a run's first slice: 0, or the end of the run before.
struct GemmRun {
  uint32_t band;     // the band
  uint32_t lo, len;  // its slices [lo, lo + len) are this workgroup's
  uint32_t piece;    // which of the band's partial sums they feed
};
LLVQ_SHARE_FN GemmRun gemm_run_at(const GemmShare& s, uint32_t spb, uint32_t c, uint32_t t) {
  GemmRun r;
  const uint32_t alone = s.whole * spb;
  if (t < alone) {
    r.band = c * s.whole + share_div(t, s.inv_spb);
    r.lo = 0;
    r.len = spb;
    r.piece = 0;
    return r;
  }
  const uint32_t g_lo = gemm_first_slice(c, s.base, s.rem), g_hi = gemm_first_slice(c + 1u, s.base, s.rem);
  const uint32_t u = g_lo + (t - alone), b = share_div(u, s.inv_spb);
  r.band = s.shared0 + b;
  r.lo = u - b * spb;
  r.len = spb - r.lo < g_hi - u ? spb - r.lo : g_hi - u;
  r.piece = c - gemm_owner(s, b * spb);
  return r;
}

}  // namespace llvq
