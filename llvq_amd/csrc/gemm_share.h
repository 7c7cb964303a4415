// How a batched launch shares its K-slices out over the workgroups: plain integer
// arithmetic, used by the kernels, by the host code that sizes the workspace, and by
// the host tests.
//
// The slices of a launch are numbered band by band (`spb` slices per band).  Workgroup
// c of n_wg walks the consecutive slices [gemm_first_slice(c), gemm_first_slice(c + 1)):
// base + 1 of them for c < rem, base otherwise.  A band whose slices fall to several
// workgroups gets one partial sum ("piece") from each, at most max_pieces of them.
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
  uint32_t base, rem;   // workgroup c walks base + (c < rem) slices
  uint32_t max_pieces;  // partial sums a band can receive
};

// total = bands x spb slices (> 0), spread over at most `cap` workgroups
LLVQ_SHARE_FN GemmShare gemm_share(uint64_t total, uint32_t spb, uint32_t cap) {
  GemmShare s;
  s.n_wg = total < cap ? (uint32_t)total : cap;
  s.base = (uint32_t)(total / s.n_wg);
  s.rem = (uint32_t)(total % s.n_wg);
  // a run of spb slices starting anywhere meets at most ceil((spb - 1) / base) + 1 workgroups
  s.max_pieces = (spb + s.base - 1) / s.base + 1;
  return s;
}

// the first slice of workgroup c (c = n_wg gives the slice count)
LLVQ_SHARE_FN uint32_t gemm_first_slice(uint32_t c, uint32_t base, uint32_t rem) {
  return c * base + (c < rem ? c : rem);
}

// the workgroup that walks slice g
LLVQ_SHARE_FN uint32_t gemm_owner(uint32_t g, uint32_t base, uint32_t rem) {
  const uint32_t head = rem * (base + 1u);
  return g < head ? g / (base + 1u) : rem + (g - head) / base;
}

}  // namespace llvq
