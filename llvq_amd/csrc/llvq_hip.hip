// C ABI and gfx950 kernels of the fused Leech-lattice dequant-GEMV.
//
// Data layout in HBM, per matrix: the packed code stream exactly as the file
// holds it (6 bytes per block, big-endian (idx << 1) | gain, rows
// back to back), f32 row scales, f32 tail columns, two f32 gain centroids.
// Per runtime: one 45 KB table image (Golay words, class records, class ends,
// reciprocals) that every workgroup copies into LDS.
#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>
#include <type_traits>

#include <algorithm>
#include <cstdio>
#include <cmath>
#include <cstring>
#include <string>
#include <utility>
#include <vector>

#include "../../include/llvq_hip.h"
#include "artifact.hpp"
#include "codebook.hpp"
#include "decode_core.h"
#include "rotation.hpp"

namespace llvq {

// ---- table image --------------------------------------------------------------
// What every workgroup copies into LDS.  The rarely used generic class records
// and the large even-coset tables stay in HBM (they live in L2).
struct TableImage {
  uint64_t starts[kStartsLds];  // first: read twice per block, its offset then needs no add of its own
  FastClass fast[kFastLds];
  double rcp[32];
  double step[(24 - kTailSlots) * 25 * 2];  // rows m >= kTailSlots: the walk's last slots are looked up
  uint8_t pdep4[256];
  uint32_t tail_meta[kTailMetaSlots];
  uint16_t lut[2048];        // a 47-bit field only reaches the lower half of the host table
  uint16_t lut2[kLut2Lds];   // the second-level tables that half refers to
  uint32_t golay[4096];
  uint32_t on_lut[kOnLutSlots];
};
static_assert(sizeof(TableImage) % 16 == 0, "table image is copied in 16-byte units");
constexpr size_t kLdsImageBytes = sizeof(TableImage);  // Golay words and the support-arrangement table included
static_assert(kLdsImageBytes % 16 == 0, "LDS part of the table image is copied in 16-byte units");

struct GlobalTables {
  const TableImage* image;
  const uint64_t* starts;  // the padded table of class starts (kStartsPadded)
  const DevClass* cls;
  const uint32_t* off_lut;
  const uint32_t* expand;
  const uint64_t* tail_codes;
  // what a 48-bit index (shell cap 13) can reach and the LDS image leaves out: every fast-path class record,
  // the whole first level of the class-find table and all its second-level tables
  const FastClass* wide_fast;
  const uint16_t* wide_lut;
  const uint16_t* wide_lut2;
};

constexpr size_t kLdsImageBytesLean = offsetof(TableImage, golay);  // without the Golay words and the support-arrangement table
static_assert(kLdsImageBytesLean % 16 == 0, "LDS part of the table image is copied in 16-byte units");
constexpr size_t kLdsImageBytesLeanest = offsetof(TableImage, lut);  // without the class lookup table either
static_assert(kLdsImageBytesLeanest % 16 == 0, "LDS part of the table image is copied in 16-byte units");

// kFull: the whole image goes to LDS; otherwise its last two tables (33 KB) are
// read through L2, for a kernel that needs the LDS for something else.  kLut = false
// leaves the 4 KB class lookup table (one read per block) in L2 as well.
// kWide: for 48-bit indices the class records, class starts and class-find tables are the full ones in device
// memory (read through L2); the LDS copies cover what a 47-bit index reaches.
template <bool kFull = true, bool kLut = true, bool kWide = false>
__device__ __forceinline__ DecodeTables stage_tables(uint8_t* smem, const GlobalTables& g) {
  static_assert(kLut || !kFull, "the tables that stay in L2 are the image's last ones");
  const uint4* src = reinterpret_cast<const uint4*>(g.image);
  uint4* dst = reinterpret_cast<uint4*>(smem);
  constexpr size_t kBytes = kFull ? sizeof(TableImage) : (kLut ? kLdsImageBytesLean : kLdsImageBytesLeanest);
  // five loads per lane in flight at a time (one pass for a 1024-lane workgroup): a load and its
  // store per loop iteration would pay the L2 latency once per iteration
  constexpr uint32_t kUnits = (uint32_t)(kBytes / 16), kLast = kUnits - 1u;
  const uint32_t st = blockDim.x;
  for (uint32_t i0 = threadIdx.x; i0 < kUnits; i0 += 5u * st) {
    const uint32_t i1 = i0 + st, i2 = i1 + st, i3 = i2 + st, i4 = i3 + st;
    const uint4 r0 = src[i0], r1 = src[min(i1, kLast)], r2 = src[min(i2, kLast)], r3 = src[min(i3, kLast)], r4 = src[min(i4, kLast)];
    __builtin_amdgcn_sched_barrier(0);  // keep the loads together, ahead of the first store
    dst[i0] = r0;
    if (i1 < kUnits) dst[i1] = r1;
    if (i2 < kUnits) dst[i2] = r2;
    if (i3 < kUnits) dst[i3] = r3;
    if (i4 < kUnits) dst[i4] = r4;
  }
  const TableImage* s = reinterpret_cast<const TableImage*>(smem);
  const TableImage* far = kFull ? s : g.image;
  if constexpr (kWide)
    return DecodeTables{far->golay, g.cls, g.wide_fast, g.starts, g.starts, g.wide_lut, g.wide_lut2, s->rcp, far->on_lut, g.off_lut,
                        g.expand, s->pdep4, s->step - kTailSlots * 25 * 2, s->tail_meta, g.tail_codes};
  return DecodeTables{far->golay, g.cls, s->fast, s->starts, g.starts, kLut ? s->lut : g.image->lut, kLut ? s->lut2 : g.image->lut2, s->rcp, far->on_lut, g.off_lut,
                      g.expand, s->pdep4, s->step - kTailSlots * 25 * 2, s->tail_meta, g.tail_codes};
}

// 6-byte big-endian record at a 2-byte-aligned offset of a 4-byte-aligned buffer
// (global or LDS): two dword reads, one funnel shift, two byte swaps.
__device__ __forceinline__ uint64_t read_record(const uint8_t* buf, size_t byte) {
  const uint32_t* w = reinterpret_cast<const uint32_t*>(buf + (byte & ~(size_t)3));
  const uint32_t w0 = w[0], w1 = w[1];
  const bool odd = (byte & 2) != 0;
  const uint32_t first = odd ? __builtin_amdgcn_alignbit(w1, w0, 16) : w0;  // bytes 0..3
  const uint32_t second = odd ? (w1 >> 16) : (w1 & 0xFFFFu);                // bytes 4..5
  return ((uint64_t)__builtin_bswap32(first) << 16) | (uint64_t)(__builtin_bswap32(second) >> 16);
}

// Sum over each row of 16 lanes, left in all 16 (four cross-lane moves inside the row).
template <int CTRL>
__device__ __forceinline__ float dpp_move(float x) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), CTRL, 0xF, 0xF, false));
}
__device__ __forceinline__ float row16_sum(float x) {
  x += dpp_move<0xB1>(x);   // quad_perm [1,0,3,2]: lane ^ 1
  x += dpp_move<0x4E>(x);   // quad_perm [2,3,0,1]: lane ^ 2
  x += dpp_move<0x141>(x);  // row_half_mirror: the other quad of the half row
  x += dpp_move<0x140>(x);  // row_mirror: the other half of the row
  return x;
}

// Sum over the wavefront, the same value in every lane: the four rows' sums are read as scalars.
__device__ __forceinline__ float wave_sum(float v) {
  v = row16_sum(v);
  return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 0)) + __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 16)) +
         __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 32)) + __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 48));
}

// Inclusive prefix sum over the wavefront's lanes: four shifts inside each row of 16 lanes, then the
// rows' totals are handed on (row 0 to row 1 and row 2 to row 3, then rows 0-1 to rows 2-3).
__device__ __forceinline__ uint32_t wave_prefix_sum(uint32_t v) {
  v += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x111, 0xF, 0xF, true);  // row_shr:1
  v += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x112, 0xF, 0xF, true);  // row_shr:2
  v += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x114, 0xF, 0xF, true);  // row_shr:4
  v += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x118, 0xF, 0xF, true);  // row_shr:8
  v += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x142, 0xA, 0xF, true);  // row_bcast:15 into rows 1 and 3
  v += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x143, 0xC, 0xF, true);  // row_bcast:31 into rows 2 and 3
  return v;
}

constexpr uint32_t kDenseBits = 49;  // bits per block at shell cap 13: a 48-bit index and the gain bit

// ---- parity probe: unrank records to points -----------------------------------
template <bool WIDE>
__global__ __launch_bounds__(256) void decode_blocks_kernel(GlobalTables g, const uint8_t* __restrict__ codes,
                                                            size_t nblocks, int8_t* __restrict__ points,
                                                            uint8_t* __restrict__ gains,
                                                            uint8_t* __restrict__ shells) {
  extern __shared__ __align__(16) uint8_t smem[];
  const DecodeTables T = stage_tables<true, true, WIDE>(smem, g);
  __syncthreads();
  if constexpr (WIDE) {
    // 49-bit blocks of a dense stream (shell cap 13): block b is the 49 bits from bit 49 b on, read byte by byte
    // (at most seven bytes hold it), so that no byte past the stream's ceil(49 nblocks / 8) is touched
    for (size_t b = (size_t)blockIdx.x * blockDim.x + threadIdx.x; b < nblocks; b += (size_t)gridDim.x * blockDim.x) {
      const uint64_t bit = (uint64_t)b * kDenseBits;
      const uint32_t sh = (uint32_t)(bit & 7u), nbytes = (sh + kDenseBits + 7u) >> 3;
      uint64_t acc = 0;
      for (uint32_t k = 0; k < 7u; ++k) acc = (acc << 8) | (k < nbytes ? codes[(bit >> 3) + k] : 0u);
      const uint64_t rec = (acc >> (56u - sh - kDenseBits)) & ((1ULL << kDenseBits) - 1u);  // index << 1 | gain
      int8_t* out = points + b * kDim;
      const int ci = decode_index(T, rec >> 1, [&](int p, int v) { out[p] = (int8_t)v; });
      if (gains) gains[b] = (uint8_t)(rec & 1);
      if (shells) shells[b] = ci >= 0 ? (uint8_t)T.cls[ci].shell : (ci == -1 ? 0 : 0xFF);
    }
    return;
  }
  for (size_t b = (size_t)blockIdx.x * blockDim.x + threadIdx.x; b < nblocks;
       b += (size_t)gridDim.x * blockDim.x) {
    // the stream's last record is read byte by byte: the two-dword read would touch up to two
    // bytes past a buffer the caller sized to 6 * nblocks
    uint64_t rec;
    if (b + 1 < nblocks) {
      rec = read_record(codes, 6 * b);
    } else {
      rec = 0;
      for (int k = 0; k < 6; ++k) rec = (rec << 8) | codes[6 * b + k];
    }
    int8_t* out = points + b * kDim;
    const int ci = decode_index(T, rec >> 1, [&](int p, int v) { out[p] = (int8_t)v; });
    if (gains) gains[b] = (uint8_t)(rec & 1);
    if (shells) shells[b] = ci >= 0 ? (uint8_t)T.cls[ci].shell : (ci == -1 ? 0 : 0xFF);
  }
}

// ---- fused dequant-GEMV ---------------------------------------------------------
// One persistent 1024-lane workgroup per CU.  The rows of up to four matrices
// that share an activation are cut into tiles of at most kTileBlocks blocks; a
// workgroup takes tiles round-robin and runs four phases on each:
//   P0  every lane loads its own four consecutive 6-byte records from HBM into
//       registers (issued a tile ahead; the records never pass through LDS);
//   P1  the lane parses them, finds each block's class (two table probes and a
//       comparison) and queues the block with its rank within the class: odd
//       coset, even coset, and even-coset classes with a second free kind each
//       have a queue, because they are different straight-line programs and
//       binning keeps every lane of a wavefront on the same one; blocks of the
//       rare generic classes go to two small side queues;
//   P2  wavefronts take 64 queued blocks at a time, unrank them to 8-bit
//       coordinates, reduce them against the activation with integer dot
//       products and write one partial sum per block;
//   P3  sixteen lanes per row add the row's partial sums in a fixed order,
//       apply the row scale and the tail columns, and store y.
// Results do not depend on the queue order, so they are reproducible.
//
// The activation is held in LDS as block-scaled fixed point: per 24-column
// block a power-of-two scale and three signed byte planes (x = scale *
// (65536 d2 + 256 d1 + d0), |65536 d2 + ...| <= 2^22), i.e. every binary16
// value within 2^12 of its block's largest is exact and the rest round at
// 2^-23 of that largest.  Integer sums of 24 products are exact; the three
// plane sums are combined and scaled in f32.
constexpr int kWgThreads = 1024;
constexpr int kWaves = kWgThreads / 64;
constexpr int kTileBlocks = 4096;  // default tile capacity; the kernel is instantiated per capacity
constexpr int kMaxGroup = 4;
constexpr int kPlaneDwords = 18;  // 3 planes x 6 dwords per 24-column block
constexpr int kGenericSlots = 64; // queue of blocks that take the generic walk

struct MatArg {
  const uint8_t* codes;
  const float* rscale;
  const float* tail;
  void* y;
  float g0, g1;
  uint32_t d_out;
  uint32_t tile_begin;  // first tile of this matrix in the launch
};

// What a launch may do to produce its activation before the product.
enum : uint32_t {
  kPrologueNone = 0,
  kPrologueSiluMul = 1,    // x[i] = f16(f16(silu(x2[i])) * x[i])           (model.rs:831)
  kPrologueAddRmsNorm = 2  // r = f16(x[i] + x2[i]) (x2 may be null: r = x[i]); resid_out = r;
                           // x[i] = f16(r / sqrt(mean(r^2) + eps) * norm_w[i])  (model.rs:781, :827-829)
};

struct GroupArgs {
  GlobalTables tables;
  const __half* x;
  const float* x_f32;  // when set, the activation is these f32 values (a rotated activation) and x is unused
  const __half* x2;
  const __half* norm_w;
  __half* resid_out;  // written by workgroup 0 only; must not alias x
  float eps;
  uint32_t prologue;
  uint32_t nblocks, tail_w, n_mats, rows_per_tile, n_tiles;
  float inv_nblocks;  // 1 / nblocks, for the block -> column split
  // the basis of these matrices, when they are stored rotated and the launch rotates its
  // own activation (rot_m = 0: no rotation; see rotate_lds)
  const uint32_t* rot_signbits;
  const float* rot_small;
  float rot_inv;
  uint32_t rot_m, rot_k;
  MatArg m[kMaxGroup];
};


// x <- (S (x) I_m)(I_k (x) H_m / sqrt m) x in place on n = k m f32 values in LDS whose
// signs D are already applied (llvq-quant/src/rotation.rs:97-105; f32 like the reference's
// device rotation, llvq-cuda/kernels/llvq_rot.cuh).  `small` is the k x k block in device
// memory.  Every thread of a 1024-thread workgroup calls it; the values are final after
// the caller's next barrier.
//  * Walsh-Hadamard levels: for m >= 512 a wavefront takes a run of 512 values, eight per
//    lane, and does nine levels without a barrier (three in registers, six by lane
//    exchange); the levels above 512, and every level of a narrower m, are radix-2
//    passes over LDS (groups are contiguous, so one pass covers all of them).
//  * the k x k block across groups, with the 1/sqrt m factor applied first, is a small
//    dense product S (k x k) . C (k x m): a wavefront takes 32 columns of C at a time and
//    runs it as f32 matrix-core steps of depth 2 (S padded with zeros to 32 x 32); it reads
//    its columns whole before it writes them, and no other wavefront touches them.
typedef float rot_acc_t __attribute__((ext_vector_type(16)));
__device__ __forceinline__ void rotate_lds(float* v, uint32_t n, uint32_t m, uint32_t k, float inv,
                                           const float* __restrict__ small) {
  const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
  const uint32_t l32 = lane & 31u, lh = lane >> 5;
  const uint32_t steps = (k + 1u) >> 1;  // depth-2 steps that cover k
  // S[l32][2 s + lh], requested before the butterflies so that the loads are back by the time they are used
  float s_frag[kRotKMax / 2];
#pragma unroll
  for (uint32_t s = 0; s < kRotKMax / 2; ++s) {
    const uint32_t t = 2u * s + lh;
    s_frag[s] = (k > 1 && m >= 32 && l32 < k && t < k) ? small[l32 * k + t] : 0.f;
  }
  uint32_t len0 = 1;
  if (m >= 512) {
    for (uint32_t c = wave; c < (n >> 9); c += 16) {
      float4* src = reinterpret_cast<float4*>(v + (c << 9) + lane * 8u);
      const float4 lo = src[0], hi = src[1];
      float r[8] = {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
#pragma unroll
      for (int l = 1; l < 8; l <<= 1)
#pragma unroll
        for (int i = 0; i < 8; ++i)
          if (!(i & l)) {
            const float u = r[i], w = r[i | l];
            r[i] = u + w;
            r[i | l] = u - w;
          }
#pragma unroll
      for (int l = 1; l < 64; l <<= 1) {
        const bool upper = (lane & (uint32_t)l) != 0;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          const float other = __shfl_xor(r[i], l, 64);
          r[i] = upper ? other - r[i] : r[i] + other;
        }
      }
      src[0] = make_float4(r[0], r[1], r[2], r[3]);
      src[1] = make_float4(r[4], r[5], r[6], r[7]);
    }
    len0 = 512;
  }
  __syncthreads();
  for (uint32_t len = len0; len < m; len <<= 1) {
    for (uint32_t p = tid; p < (n >> 1); p += 1024) {
      const uint32_t j = (p / len) * (len << 1) + (p % len);
      const float u = v[j], w = v[j + len];
      v[j] = u + w;
      v[j + len] = u - w;
    }
    __syncthreads();
  }
  if (k == 1) {
    for (uint32_t i = tid; i < n; i += 1024) v[i] = v[i] * inv;
    return;
  }
  if (m >= 32) {
    for (uint32_t tile = wave; tile < (m >> 5); tile += 16) {
      const uint32_t j = (tile << 5) + l32;
      float c_frag[kRotKMax / 2];
#pragma unroll
      for (uint32_t s = 0; s < kRotKMax / 2; ++s) {
        const uint32_t t = 2u * s + lh;
        const float x = v[(t < k ? t * m : 0u) + j];  // always a valid address, so the reads go out together
        c_frag[s] = t < k ? x * inv : 0.f;
      }
      rot_acc_t acc;
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[r] = 0.f;
#pragma unroll
      for (uint32_t s = 0; s < kRotKMax / 2; ++s)
        if (s < steps) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(s_frag[s], c_frag[s], acc, 0, 0, 0);
      // acc[r] is row 8 (r / 4) + 4 lh + r % 4 of column j
#pragma unroll
      for (uint32_t r = 0; r < 16; ++r) {
        const uint32_t g = 8u * (r >> 2) + 4u * lh + (r & 3u);
        if (g < k) v[g * m + j] = acc[r];
      }
    }
    return;
  }
  // narrow groups (m < 32): one thread per column
  for (uint32_t j = tid; j < m; j += 1024) {
    float col[kRotKMax];
#pragma unroll
    for (uint32_t t = 0; t < kRotKMax; ++t) col[t] = t < k ? v[t * m + j] * inv : 0.f;
    for (uint32_t g = 0; g < k; ++g) {
      float acc = 0.f;
#pragma unroll
      for (uint32_t t = 0; t < kRotKMax; ++t)
        if (t < k) acc = fmaf(small[g * k + t], col[t], acc);
      v[g * m + j] = acc;
    }
  }
}

constexpr int kSmallTileBlocks = 2048;  // tile of the variant for rows too wide for the full tile's LDS
constexpr int kSecSlots = 384;          // queue of even-coset blocks whose class has a second free kind (7.6 % of uniform draws)
// Per queue slot an 8-byte entry and its 2-byte block number, per tile slot a partial sum; the 32
// bytes between them keep the area at least as large as a derived activation's staging needs it
// (see prologue_fits / rotation_fits).
__host__ __device__ constexpr size_t gemv_stage_bytes(uint32_t tile) { return ((size_t)tile + kSecSlots) * 10 + 32 + (size_t)tile * 4; }
__host__ __device__ constexpr size_t gemv_lds_bytes(uint32_t nblocks, uint32_t tile = kTileBlocks,
                                                    size_t image_bytes = kLdsImageBytes) {
  return image_bytes + (size_t)nblocks * (kPlaneDwords + 1) * 4 + (32 + (nblocks & 1u)) * 4 + gemv_stage_bytes(tile) +
         2 * (size_t)kGenericSlots * 10 + 32;
}

template <typename OutT>
__device__ __forceinline__ void store_out(void* y, uint32_t r, float v);
template <>
__device__ __forceinline__ void store_out<float>(void* y, uint32_t r, float v) {
  reinterpret_cast<float*>(y)[r] = v;
}
template <>
__device__ __forceinline__ void store_out<__half>(void* y, uint32_t r, float v) {
  reinterpret_cast<__half*>(y)[r] = __float2half_rn(v);
}

// Loads and stores of values that another workgroup of the SAME launch produces or consumes (gemv_seq.h): device
// scope, so that they meet in memory and not in an XCD's own L2, which the L2 of another XCD is not coherent with.
// They replace the device-scope fences such an exchange would otherwise need — whose acquire side empties the
// XCD's L2 of the decode tables every time.
template <bool kDeviceScope>
__device__ __forceinline__ __half load_half(const __half* p) {
  if constexpr (kDeviceScope)
    return __ushort_as_half(__hip_atomic_load(reinterpret_cast<const unsigned short*>(p), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
  else
    return *p;
}
template <bool kDeviceScope>
__device__ __forceinline__ void store_half(__half* p, __half v) {
  if constexpr (kDeviceScope)
    __hip_atomic_store(reinterpret_cast<unsigned short*>(p), __half_as_ushort(v), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  else
    *p = v;
}

// One 24-column block of the activation -> scale and byte planes.
template <bool kDeviceScope = false>
__device__ __forceinline__ void load_block_f16(const __half* x, float (&v)[kDim]) {
  if constexpr (kDeviceScope) {
    if ((reinterpret_cast<uintptr_t>(x) & 3) == 0) {
      const uint32_t* src = reinterpret_cast<const uint32_t*>(x);
#pragma unroll
      for (int k = 0; k < kDim / 2; ++k) {
        const uint32_t w = __hip_atomic_load(src + k, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        v[2 * k] = __half2float(__ushort_as_half((unsigned short)(w & 0xFFFFu)));
        v[2 * k + 1] = __half2float(__ushort_as_half((unsigned short)(w >> 16)));
      }
    } else {
#pragma unroll
      for (int j = 0; j < kDim; ++j) v[j] = __half2float(load_half<true>(x + j));
    }
    return;
  }
  if ((reinterpret_cast<uintptr_t>(x) & 15) == 0) {
    const uint4* src = reinterpret_cast<const uint4*>(x);
#pragma unroll
    for (int k = 0; k < 3; ++k) {
      const uint4 u = src[k];
      const uint32_t w[4] = {u.x, u.y, u.z, u.w};
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        v[8 * k + 2 * j] = __half2float(__ushort_as_half((unsigned short)(w[j] & 0xFFFFu)));
        v[8 * k + 2 * j + 1] = __half2float(__ushort_as_half((unsigned short)(w[j] >> 16)));
      }
    }
  } else {  // the activation of a batched row need not be 16-byte aligned
#pragma unroll
    for (int j = 0; j < kDim; ++j) v[j] = __half2float(x[j]);
  }
}

// PLANES = 3: x = scale (65536 d2 + 256 d1 + d0), |...| <= 2^22, for results stored as f32; PLANES = 2: x = scale (256 d1 + d0),
// |...| <= 2^14, for results stored as binary16 — an activation is then rounded at 2^-15 of its block's largest value,
// a sixteenth of the half ulp the stored result carries anyway, and a block costs a third fewer dot products.
template <int PLANES>
__device__ __forceinline__ void quantize_values(const float (&v)[kDim], uint32_t* planes, float* scale);

template <int PLANES>
__device__ __forceinline__ void quantize_block(const __half* x, uint32_t* planes, float* scale) {
  float v[kDim];
  load_block_f16(x, v);
  quantize_values<PLANES>(v, planes, scale);
}

// f32 activation (a rotated one, fused_cuda.rs:384): same block-scaled fixed point
template <int PLANES>
__device__ __forceinline__ void quantize_block_f32(const float* x, uint32_t* planes, float* scale) {
  float v[kDim];
#pragma unroll
  for (int j = 0; j < kDim; ++j) v[j] = x[j];
  quantize_values<PLANES>(v, planes, scale);
}

template <int PLANES>
__device__ __forceinline__ void quantize_values(const float (&v)[kDim], uint32_t* planes, float* scale) {
  static_assert(PLANES == 2 || PLANES == 3, "two or three byte planes");
  constexpr int kBits = PLANES == 3 ? 22 : 14;
  float amax = 0.f;
#pragma unroll
  for (int j = 0; j < kDim; ++j) amax = fmaxf(amax, fabsf(v[j]));
  bool bad = false;
#pragma unroll
  for (int j = 0; j < kDim; ++j) bad |= !(fabsf(v[j]) <= 3.4028234e38f);  // inf or NaN
  int e = 0;
  (void)frexpf(amax, &e);  // amax = m 2^e, m in [0.5, 1)
  const float up = ldexpf(1.f, kBits - e);
  *scale = bad ? __builtin_nanf("") : (amax == 0.f ? 0.f : ldexpf(1.f, e - kBits));
  uint32_t p0[6], p1[6], p2[6];
#pragma unroll
  for (int q = 0; q < 6; ++q) p0[q] = p1[q] = p2[q] = 0;
#pragma unroll
  for (int j = 0; j < kDim; ++j) {
    const int xq = (amax == 0.f || bad) ? 0 : (int)rintf(v[j] * up);  // |xq| <= 2^kBits
    const int d0 = (int)(int8_t)(xq & 0xFF);
    const int x1 = (xq - d0) >> 8;
    const int d1 = (int)(int8_t)(x1 & 0xFF);
    const int d2 = (x1 - d1) >> 8;  // zero with two planes: |x1| <= 64
    p0[j >> 2] |= (uint32_t)(d0 & 0xFF) << (8 * (j & 3));
    p1[j >> 2] |= (uint32_t)(d1 & 0xFF) << (8 * (j & 3));
    p2[j >> 2] |= (uint32_t)(d2 & 0xFF) << (8 * (j & 3));
  }
#pragma unroll
  for (int q = 0; q < 6; ++q) {
    planes[q] = p0[q];
    planes[6 + q] = p1[q];
    if (PLANES == 3) planes[12 + q] = p2[q];
  }
}

template <int PLANES>
__device__ __forceinline__ float planes_to_float(int d0, int d1, int d2) {
  if (PLANES == 2) return fmaf((float)d1, 256.f, (float)d0);
  return fmaf((float)d2, 65536.f, fmaf((float)d1, 256.f, (float)d0));
}

__device__ __forceinline__ void tile_of(const GroupArgs& a, uint32_t tile, MatArg& M, uint32_t& r0, uint32_t& rows) {
  M = a.m[0];  // constant indices only: a dynamic one would move the arguments to scratch
#pragma unroll
  for (uint32_t k = 1; k < kMaxGroup; ++k)
    if (k < a.n_mats && tile >= a.m[k].tile_begin) M = a.m[k];
  r0 = (tile - M.tile_begin) * a.rows_per_tile;
  rows = min(a.rows_per_tile, M.d_out - r0);
}

// A lane's share of a tile's code bytes: NB consecutive 6-byte records, 3 NB / 2 dwords, from the
// byte the first of them starts at.  A tile starts on a row boundary, i.e. at an even byte (a
// multiple of four whenever rows-per-tile x blocks-per-row is even), so these are vector loads at
// two- or four-byte alignment; consecutive lanes read consecutive memory.  Unconditional: a lane
// past the tile's end reads the tile's first records again and ignores them — a guarded load is
// merged with the register's old value at once, and that merge waits for the load.
template <int NB>
struct LaneRecords {
  static_assert(NB == 2 || NB == 4, "a lane takes two or four records");
  uint32_t w[NB * 3 / 2];
};
typedef uint32_t dwords4_a2 __attribute__((ext_vector_type(4), aligned(2)));
typedef uint32_t dwords3_a2 __attribute__((ext_vector_type(3), aligned(2)));
typedef uint32_t dwords2_a2 __attribute__((ext_vector_type(2), aligned(2)));
template <int NB>
__device__ __forceinline__ void prefetch_records(const GroupArgs& a, uint32_t tile, uint32_t tid, LaneRecords<NB>& r) {
  if (tile >= a.n_tiles || a.nblocks == 0) return;  // rows of tail columns only have no code bytes
  MatArg M;
  uint32_t r0, rows;
  tile_of(a, tile, M, r0, rows);
  // a lane whose records all lie past the tile's end re-reads the tile's first ones: every byte read lies
  // inside the tile or within 6 NB bytes behind it, which the 64 bytes of slack behind a matrix's last
  // record cover
  const uint32_t share = (uint32_t)NB * 6u;
  const uint32_t at = tid * (uint32_t)NB < rows * a.nblocks ? tid * share : 0u;
  const uint8_t* src = M.codes + (size_t)r0 * a.nblocks * 6 + at;
  // streaming loads: the code bytes are read once
  if constexpr (NB == 4) {
    const dwords4_a2 lo = __builtin_nontemporal_load(reinterpret_cast<const dwords4_a2*>(src));
    const dwords2_a2 hi = __builtin_nontemporal_load(reinterpret_cast<const dwords2_a2*>(src + 16));
    r.w[0] = lo.x; r.w[1] = lo.y; r.w[2] = lo.z; r.w[3] = lo.w; r.w[4] = hi.x; r.w[5] = hi.y;
  } else {
    const dwords3_a2 v = __builtin_nontemporal_load(reinterpret_cast<const dwords3_a2*>(src));
    r.w[0] = v.x; r.w[1] = v.y; r.w[2] = v.z;
  }
}

// Record j of a lane's share as the 48-bit big-endian number it is: one byte permute for its
// low 32 bits, one for its high 16.
template <int NB>
__device__ __forceinline__ void lane_record(const LaneRecords<NB>& r, int j, uint32_t& lo32, uint32_t& hi16) {
  const int d = 3 * (j / 2) + (j & 1);
  const uint32_t a = r.w[d], b = r.w[d + 1];  // the record's bytes lie in these two dwords
  if (j & 1) {  // starts at byte 2 of a
    lo32 = __builtin_amdgcn_perm(b, a, 0x04050607u);
    hi16 = __builtin_amdgcn_perm(b, a, 0x0c0c0203u);
  } else {      // starts at byte 0 of a
    lo32 = __builtin_amdgcn_perm(b, a, 0x02030405u);
    hi16 = __builtin_amdgcn_perm(b, a, 0x0c0c0001u);
  }
}

// ---- records of the cap-13 ball: 49 bits per block in a dense stream -------------------------------
// At shell cap 13 an index takes 48 bits (N(13) < 2^48), so a block is 49 bits — index, then the gain bit,
// most significant bit first — and blocks follow one another without padding (llvq-search/src/pack.rs:48-82,
// llvq-artifact/src/format.rs:87-89): block b of a matrix starts at bit 49 b of its code stream.  A lane takes
// four consecutive blocks, 196 bits, from the eight dwords that hold them: the stream position of its first
// block, cut to a dword boundary, plus the bits `s0` left over.  Unconditional loads, as for the 6-byte records:
// a lane past the tile's end reads the tile's first blocks again; every byte read lies inside the tile or within
// 32 bytes behind it, which the slack behind a matrix's code stream covers.
struct DenseRecords {
  uint32_t w[8];
  uint32_t s0;  // bits of w[0] ahead of the lane's first block (0..31)
};
typedef uint32_t dwords4_a4 __attribute__((ext_vector_type(4), aligned(4)));
__device__ __forceinline__ void prefetch_records(const GroupArgs& a, uint32_t tile, uint32_t tid, DenseRecords& r) {
  if (tile >= a.n_tiles || a.nblocks == 0) return;
  MatArg M;
  uint32_t r0, rows;
  tile_of(a, tile, M, r0, rows);
  const uint64_t tile_bit = (uint64_t)r0 * a.nblocks * kDenseBits;    // the tile's first bit in the matrix's stream
  const uint64_t tile_base = (tile_bit >> 3) & ~(uint64_t)3;           // ... cut to a dword
  const uint32_t rem = (uint32_t)(tile_bit - 8u * tile_base);           // 0..31
  const uint32_t first = tid * 4u < rows * a.nblocks ? tid * 4u : 0u;  // the lane's first block in the tile
  const uint32_t lane_bit = rem + first * kDenseBits;
  const uint8_t* src = M.codes + tile_base + (size_t)(lane_bit >> 5) * 4;
  const dwords4_a4 lo = __builtin_nontemporal_load(reinterpret_cast<const dwords4_a4*>(src));
  const dwords4_a4 hi = __builtin_nontemporal_load(reinterpret_cast<const dwords4_a4*>(src + 16));
  r.w[0] = lo.x; r.w[1] = lo.y; r.w[2] = lo.z; r.w[3] = lo.w; r.w[4] = hi.x; r.w[5] = hi.y; r.w[6] = hi.z; r.w[7] = hi.w;
  r.s0 = lane_bit & 31u;
}

// The index (ilo, ihi) and gain bit of record i of a lane's share.  6-byte records: 47 bits of index.
template <int NB>
__device__ __forceinline__ const LaneRecords<NB>& prepared_records(const LaneRecords<NB>& rec) { return rec; }
template <int NB>
__device__ __forceinline__ void record_index(const LaneRecords<NB>& rec, int i, uint32_t& ilo, uint32_t& ihi, uint32_t& gain) {
  uint32_t lo32, hi16;
  lane_record(rec, i, lo32, hi16);
  gain = lo32 & 1u;
  ilo = __builtin_amdgcn_alignbit(hi16, lo32, 1);
  ihi = hi16 >> 1;
}
// 49-bit blocks: the dwords become big-endian words and the lane's bits are moved to the front of them, once;
// block j is then the 49 bits from bit 49 j on.  48 bits of index.
struct DenseWords {
  uint32_t n[7];
};
__device__ __forceinline__ DenseWords prepared_records(const DenseRecords& rec) {
  uint32_t be[8];
  DenseWords d;
#pragma unroll
  for (int i = 0; i < 8; ++i) be[i] = __builtin_bswap32(rec.w[i]);
#pragma unroll
  for (int i = 0; i < 7; ++i) d.n[i] = (uint32_t)((((uint64_t)be[i] << 32) | be[i + 1]) >> (32u - rec.s0));
  return d;
}
__device__ __forceinline__ void record_index(const DenseWords& r, int j, uint32_t& ilo, uint32_t& ihi, uint32_t& gain) {
  constexpr uint32_t kW = kDenseBits;
  const int d = (int)(kW * (uint32_t)j) >> 5;
  const uint32_t sh = (kW * (uint32_t)j) & 31u;
  const uint64_t top = (((uint64_t)r.n[d] << 32) | r.n[d + 1]);
  const uint64_t x = sh ? (top << sh) | (uint64_t)(r.n[d + 2 > 6 ? 6 : d + 2] >> (32u - sh)) : top;  // 64 bits from the block's first
  const uint64_t v = x >> (64u - kW);                                                                  // the block: index << 1 | gain
  gain = (uint32_t)v & 1u;
  ilo = (uint32_t)(v >> 1);
  ihi = (uint32_t)(v >> 33);
}
template <class Rec> struct RecordTraits { static constexpr bool kWide = false; };
template <> struct RecordTraits<DenseRecords> { static constexpr bool kWide = true; };

// Phase timestamps for tuning builds (-DLLVQ_PHASE_TIMING): wave 0 of each
// workgroup stores the realtime counter at every phase boundary of its first tile.
#ifdef LLVQ_PHASE_TIMING
__device__ unsigned long long g_phase_stamps[1024 * 8];
#define LLVQ_STAMP(k)                                                                     \
  do {                                                                                    \
    if (threadIdx.x == 0 && tile == blockIdx.x) g_phase_stamps[blockIdx.x * 8 + (k)] = wall_clock64(); \
  } while (0)
#else
#define LLVQ_STAMP(k) do {} while (0)
#endif

// The same number as one the compiler can relate to nothing it knows.  Used where what it would derive costs
// more than the plain form: the address of an element of a second array with the same index (formed from the
// first element's address by a 64-bit multiply-add), a table key re-shaped into three instructions, a 16-bit
// entry zero-extended again.
__device__ __forceinline__ uint32_t detached(uint32_t v) {
  asm("" : "+v"(v));
  return v;
}

static_assert(kLutFinal == 0x8000u, "the final flag is the top bit of a 16-bit entry");

// Classes of NB indices as records hold them (1 .. N, below 2^47; 0 walks the tables harmlessly) side by side:
// the class, its first index and its decoder
// (kLutKind*).  Two table probes and one comparison each, every read unconditional so that the NB
// reads of a step go out together; the indices whose bucket meets several class starts (0.09 % of
// uniform draws) take the halving search afterwards, under a wavefront-wide test.
template <int NB, bool WIDE = false>
__device__ __forceinline__ void find_classes(const DecodeTables& T, const uint32_t (&zlo)[NB], const uint32_t (&zhi)[NB],
                                             uint32_t (&ci)[NB], uint64_t (&start)[NB], uint32_t (&kind)[NB]) {
  uint32_t e[NB], e2[NB];
  // (48-bit indices reach the whole first-level table; T's class-find tables are then the full ones, in device memory)
#pragma unroll
  for (int i = 0; i < NB; ++i) {
    // a bit-field extract and a scaled add; the entry as the 32-bit word the load returns (upper half zero)
    const uint32_t key = detached(__builtin_amdgcn_ubfe(zhi[i], kLutShift - 32, WIDE ? 12 : 11));
    e[i] = detached(T.lut[key]);
  }
#pragma unroll
  for (int i = 0; i < NB; ++i) {
    // a first-level entry that is not final is where its second-level table begins, a multiple of the span
    const uint32_t at = (__builtin_amdgcn_alignbit(zhi[i], zlo[i], kLut2Shift) & (uint32_t)(kLut2Span - 1)) | e[i];
    e2[i] = T.lut2[e[i] < kLutFinal ? at : 0u];  // the flag is the entry's top bit: one comparison
  }
  uint64_t s0[NB], s1[NB];
#pragma unroll
  for (int i = 0; i < NB; ++i) {
    e[i] = e[i] < kLutFinal ? e2[i] : e[i];
    s0[i] = T.starts[e[i] & 511u];
    s1[i] = T.starts[(e[i] & 511u) + 1u];
  }
  uint32_t wide = 0;
#pragma unroll
  for (int i = 0; i < NB; ++i) {
    const uint64_t z = ((uint64_t)zhi[i] << 32) | zlo[i];
    const bool up = s1[i] <= z;
    ci[i] = (e[i] & 511u) + (up ? 1u : 0u);
    start[i] = up ? s1[i] : s0[i];
    kind[i] = (e[i] >> (up ? 11 : 9)) & 3u;
    wide |= e[i] & kLutWide;
  }
  if (__any(wide != 0u)) {
#pragma unroll
    for (int i = 0; i < NB; ++i)
      if (e[i] & kLutWide) {
        const uint32_t c = class_from_entry(T, e[i], ((uint64_t)zhi[i] << 32) | zlo[i]);
        const uint32_t meta = T.fast[c].meta, path = (meta >> kMetaPathShift) & 3u;
        ci[i] = c;
        start[i] = T.starts_far[c];
        kind[i] = path == kPathOdd ? (uint32_t)kLutKindOdd
                                   : path == kPathEven ? ((meta & kMetaSecondFree) ? (uint32_t)kLutKindEvenSecond : (uint32_t)kLutKindEven)
                                                       : (uint32_t)kLutKindGeneric;
      }
  }
}

// P1 of the GEMV and GEMM kernels: each of the LANES lanes taking part (the first
// LANES of the workgroup) classifies up to NB blocks of the tile and bins them: slots first, first + LANES, ...
// (`first` is the lane's index in the workgroup unless the caller hands out the slots itself).
// `record(f)` returns the 48-bit record of tile slot f < nblk;
// `origin(f)` is called for an origin block (index 0) and returns whether the
// block must still be queued (flagged, with the odd-coset blocks) or is settled.
// Queue entry: slot (12 bits) | class << 16 | gain << 25 | origin << 30 | generic walk << 31.
// The halving searches of a lane's blocks run side by side (independent LDS
// chains); a wavefront claims queue space with one atomic per queue.  Blocks of
// the rare generic classes take ~2000 dependent instructions: they go to a
// small queue that P2 hands out first; what does not fit rides in the odd queue.
constexpr uint32_t kEntryOrigin = 0x40000000u, kEntryGeneric = 0x80000000u;
template <int NB, int LANES = kWgThreads, typename RecordFn, typename OriginFn>
__device__ __forceinline__ void classify_and_bin(const DecodeTables& T, uint32_t nblk, uint32_t capacity, uint32_t* queue,
                                                 uint32_t* gqueue, uint32_t* ctrl, RecordFn record, OriginFn origin,
                                                 uint32_t first = threadIdx.x) {
  const uint32_t tid = first, lane = threadIdx.x & 63u;
  uint32_t entry[NB], ci[NB];
  uint64_t zi[NB];  // the record's index, ~0 when the lane has no block / an origin
  bool queued_origin[NB];
  // Every LDS read of this phase is unconditional (a lane without a block reads a valid slot and
  // ignores it), so that the NB reads of a step go out together: a guarded read is waited for
  // where it is issued, and the phase is a chain of dependent reads.
  uint64_t recs[NB];
#pragma unroll
  for (int i = 0; i < NB; ++i) recs[i] = record(min(tid + (uint32_t)i * LANES, nblk - 1u));
#pragma unroll
  for (int i = 0; i < NB; ++i) {
    const uint32_t f = tid + (uint32_t)i * LANES;
    zi[i] = ~0ULL;
    entry[i] = 0;
    ci[i] = 0;
    queued_origin[i] = false;
    if (f < nblk) {
      const uint64_t rec = recs[i];
      entry[i] = f | ((uint32_t)(rec & 1) << 25);
      if ((rec >> 1) == 0) {  // the origin decodes to zero whatever the gain (index.rs:335-337)
        queued_origin[i] = origin(f);
        if (queued_origin[i]) entry[i] |= kEntryOrigin;
      } else {
        zi[i] = rec >> 1;
      }
    }
  }
  uint32_t zlo[NB], zhi[NB], kind[NB];
  uint64_t start[NB];
#pragma unroll
  for (int i = 0; i < NB; ++i) {  // a lane without a block, or with an origin, walks the tables with index 0
    zlo[i] = zi[i] != ~0ULL ? (uint32_t)zi[i] : 0u;
    zhi[i] = zi[i] != ~0ULL ? (uint32_t)(zi[i] >> 32) : 0u;
  }
  find_classes<NB>(T, zlo, zhi, ci, start, kind);
  uint32_t path[NB], odd_rank[NB], even_rank[NB], n_o = 0, n_e = 0;
#pragma unroll
  for (int i = 0; i < NB; ++i) {
    const uint32_t decoder = kind[i] == kLutKindOdd ? (uint32_t)kPathOdd : kind[i] == kLutKindGeneric ? (uint32_t)kPathGeneric : (uint32_t)kPathEven;
    path[i] = zi[i] != ~0ULL ? decoder : (queued_origin[i] ? (uint32_t)kPathOdd : 3u);
    entry[i] |= ci[i] << 16;
    if (path[i] == kPathGeneric) {
      entry[i] |= kEntryGeneric;
      const uint32_t slot = atomicAdd(&ctrl[2], 1u);
      if (slot < (uint32_t)kGenericSlots) {
        gqueue[slot] = entry[i];
        path[i] = 3u;  // placed
      }
    }
    const uint64_t mo = __ballot(path[i] == kPathOdd || path[i] == kPathGeneric), me = __ballot(path[i] == kPathEven);
    odd_rank[i] = n_o + __builtin_amdgcn_mbcnt_hi((uint32_t)(mo >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)mo, 0));
    even_rank[i] = n_e + __builtin_amdgcn_mbcnt_hi((uint32_t)(me >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)me, 0));
    n_o += (uint32_t)__popcll(mo);
    n_e += (uint32_t)__popcll(me);
  }
  uint32_t base_o = 0, base_e = 0;
  if (lane == 0) {
    base_o = atomicAdd(&ctrl[0], n_o);
    base_e = atomicAdd(&ctrl[1], n_e);
  }
  base_o = __shfl(base_o, 0, 64);
  base_e = __shfl(base_e, 0, 64);
#pragma unroll
  for (int i = 0; i < NB; ++i) {
    if (path[i] == kPathOdd || path[i] == kPathGeneric) queue[base_o + odd_rank[i]] = entry[i];  // odd from the bottom
    if (path[i] == kPathEven) queue[capacity - 1 - (base_e + even_rank[i])] = entry[i];          // even from the top
  }
}

// ---- P1 of the GEMV kernel --------------------------------------------------------------
// Each lane classifies the NB consecutive records it loaded itself and queues them with
// everything P2 needs, so that the record is parsed once:
//   qa[slot] = { local rank, bits 0..31;  local rank, bits 32..44 | class << 13 | gain << 22 | flags }
//   qf[slot] = the block's number in the tile (row * blocks per row + column)
// (the largest class holds fewer than 2^45 indices).  Three queues — the odd coset from the bottom
// of qa / qf, the even coset from their top, and even-coset classes with a second free kind in a
// small queue of their own (what does not fit there rides in the even queue, flagged) — because the
// three are different straight-line programs.  Blocks of the rare generic classes go to two small
// queues, by coset; what does not fit rides in the odd queue, flagged.
constexpr uint32_t kQaClassShift = 13, kQaGainShift = 22;
constexpr uint32_t kQaSecond = 0x40000000u;
enum : uint32_t { kCtrlOdd = 0, kCtrlEven = 1, kCtrlGenOdd = 2, kCtrlTicket = 3, kCtrlSec = 4, kCtrlGenEven = 5, kCtrlWords = 8 };

struct GemvQueues {
  uint2* qa;        // [tile + kSecSlots]: the odd queue from 0 up, the even queue from tile - 1 down, the small even queue from tile up
  uint16_t* qf;     // [tile + kSecSlots]
  uint2* gqa;       // [2][kGenericSlots]: odd-coset generic blocks, then even-coset ones
  uint16_t* gqf;
  uint32_t* ctrl;   // [kCtrlWords]
  float* partial;   // [tile]
};

// What a lane knows of its NB blocks after classification and before they are queued: the two
// words of each block's queue entry and, packed in `where`, bits 2i..2i+1 = the queue block i joins
// (0 odd, 1 even, 2 the small even queue, 3 none), bit 8 + i = block i is the origin, bit 12 + i =
// block i is a generic block of the even coset.
template <int NB>
struct Classified {
  uint32_t e0[NB], e1[NB];
  uint32_t where;
};

// First half of P1: table reads only, nothing is written — it may run while another tile's queues are in use.
template <int NB, class Rec>
__device__ __forceinline__ void classify_records(const DecodeTables& T, const Rec& rec, uint32_t nblk, Classified<NB>& c,
                                                 uint32_t tid = threadIdx.x) {
  constexpr bool kWide = RecordTraits<Rec>::kWide;
  // Every LDS read below is unconditional, from a valid slot, so that the NB reads of a step go
  // out together (a guarded read is waited for where it is issued).  A lane past the tile's end
  // walks the tables with whatever bytes follow the tile and queues nothing.
  uint32_t zlo[NB], zhi[NB], gain[NB], ci[NB], kind[NB];
  uint64_t start[NB];
  bool live[NB];  // a block of the tile that is not the origin (which decodes to zero whatever the gain, index.rs:335-337)
  uint32_t where = 0;
  bool any_origin = false;
  const auto& records = prepared_records(rec);
  const uint32_t share = nblk > tid * NB ? nblk - tid * NB : 0u;  // this lane's blocks are its first `share` (NB or more: all)
#pragma unroll
  for (int i = 0; i < NB; ++i) {
    uint32_t ilo, ihi;  // the 47-bit (48-bit) index
    record_index(records, i, ilo, ihi, gain[i]);
    // The tables are keyed on the index as the record holds it.  A 48-bit field can hold numbers past N(13):
    // the host refuses such a matrix, and a lane past the tile's end, which reads whatever bits follow, must
    // still walk the tables inside them: such a number counts as the origin
    if (kWide) {
      const uint64_t v = ((uint64_t)ihi << 32) | ilo;
      const bool inside = v <= kN13;
      ilo = inside ? ilo : 0u;
      ihi = inside ? ihi : 0u;
    }
    const bool origin = (ilo | ihi) == 0u, mine = (uint32_t)i < share;
    live[i] = mine && !origin;
    any_origin |= mine && origin;
    zlo[i] = ilo;
    zhi[i] = ihi;
  }
  if (__any(any_origin)) {  // rare: a block at the origin is flagged for settle_origins
    asm volatile("");       // (a branch, not selects on the common path)
#pragma unroll
    for (int i = 0; i < NB; ++i) where |= ((uint32_t)i < share && (zlo[i] | zhi[i]) == 0u) ? 1u << (8 + i) : 0u;
  }
  find_classes<NB, kWide>(T, zlo, zhi, ci, start, kind);
  // Which queue a block joins.  A generic block (rare) joins none here: it is settled when the block is queued
  // (its coset's small queue, or the odd queue, flagged, when that one is full).
  bool any_generic = false;
#pragma unroll
  for (int i = 0; i < NB; ++i) {
    const uint64_t li = (((uint64_t)zhi[i] << 32) | zlo[i]) - start[i];
    c.e0[i] = (uint32_t)li;
    c.e1[i] = (uint32_t)(li >> 32) | (ci[i] << kQaClassShift) | (gain[i] << kQaGainShift);
    where |= (live[i] ? kind[i] : 3u) << (2 * i);
    any_generic |= live[i] && kind[i] == kLutKindGeneric;
  }
  static_assert(kLutKindGeneric == 3u, "a generic block and a block that joins no queue share the code 3");
  if (__any(any_generic)) {
#pragma unroll
    for (int i = 0; i < NB; ++i)
      if (live[i] && kind[i] == kLutKindGeneric) where |= (1u << (16 + i)) | ((T.fast[ci[i]].meta & kMetaOdd) ? 0u : 1u << (12 + i));
  }
  c.where = where;
}

// Second half of P1: the lane's classified blocks go to the tile's queues (LDS writes and counters).
template <int NB>
__device__ __forceinline__ void queue_classified(Classified<NB>& c, uint32_t capacity, const GemvQueues& Q, uint32_t tid = threadIdx.x) {
  const uint32_t lane = tid & 63u;
  uint32_t kq[NB];
#pragma unroll
  for (int i = 0; i < NB; ++i) kq[i] = (c.where >> (2 * i)) & 3u;
  if (__any((c.where >> 16) & 15u)) {  // generic blocks: to the small queue of their coset while it has room
#pragma unroll
    for (int i = 0; i < NB; ++i)
      if ((c.where >> (16 + i)) & 1u) {
        const uint32_t even = (c.where >> (12 + i)) & 1u;
        const uint32_t slot = atomicAdd(&Q.ctrl[even ? kCtrlGenEven : kCtrlGenOdd], 1u);
        c.e1[i] |= 0x80000000u;  // the walk, not a fast decoder
        if (slot < (uint32_t)kGenericSlots) {
          Q.gqa[even * kGenericSlots + slot] = make_uint2(c.e0[i], c.e1[i]);
          Q.gqf[even * kGenericSlots + slot] = (uint16_t)(tid * NB + (uint32_t)i);
        } else {
          kq[i] = 0u;  // rides in the odd queue, flagged
        }
      }
  }
  // A block's rank in its queue among the wavefront's blocks.  Three 10-bit counters packed in a
  // dword (a wavefront classifies at most 256 blocks): a lane's own blocks in order, behind the
  // blocks of the lanes below it — one prefix sum over the wavefront by lane shifts.
  uint32_t sh[NB], running[NB], total = 0;
#pragma unroll
  for (int i = 0; i < NB; ++i) {
    sh[i] = __umul24(kq[i], 10u);
    running[i] = total;
    total += (1u << sh[i]) & 0x3FFFFFFFu;  // a block that joins no queue (3) counts nowhere
  }
  const uint32_t through = wave_prefix_sum(total);  // this lane's blocks included
  const uint32_t below = through - total;
  const uint32_t all = (uint32_t)__builtin_amdgcn_readlane((int)through, 63);
  const uint32_t n_o = all & 1023u, n_e = (all >> 10) & 1023u, n_s = (all >> 20) & 1023u;
  uint32_t base_o = 0, base_e = 0, base_s = 0;
  if (lane == 0) {
    base_o = atomicAdd(&Q.ctrl[kCtrlOdd], n_o);
    base_s = atomicAdd(&Q.ctrl[kCtrlSec], n_s);
    // what the small queue cannot take rides in the even queue behind this wavefront's own entries
    const uint32_t spill = base_s + n_s > (uint32_t)kSecSlots ? base_s + n_s - max(base_s, (uint32_t)kSecSlots) : 0u;
    base_e = atomicAdd(&Q.ctrl[kCtrlEven], n_e + spill);
  }
  base_o = __builtin_amdgcn_readfirstlane(base_o);
  base_e = __builtin_amdgcn_readfirstlane(base_e);
  base_s = __builtin_amdgcn_readfirstlane(base_s);
  // odd from the bottom, even from the top, the small queue behind both
  const uint32_t top = capacity - 1u - base_e, small = capacity + base_s;
  const bool spills = base_s + n_s > (uint32_t)kSecSlots;  // wavefront-uniform, rare
  auto place = [&](int i, uint32_t pos, uint32_t e1) {
    if (kq[i] != 3u) {
      Q.qa[pos] = make_uint2(c.e0[i], e1);
      Q.qf[detached(pos)] = (uint16_t)(tid * NB + (uint32_t)i);
    }
  };
  if (!spills) {  // a branch of its own: the rare case's arithmetic stays out of the common one
    // the three queues' first slots in vector registers, formed once, and a signed step: the even queue runs down
    const uint32_t v_odd = detached(base_o), v_top = detached(top), v_small = detached(small);
#pragma unroll
    for (int i = 0; i < NB; ++i) {
      const uint32_t rank = __builtin_amdgcn_ubfe(below + running[i], sh[i], 10);
      const uint32_t first = kq[i] == 1u ? v_top : (kq[i] == 2u ? v_small : v_odd);
      const int step = kq[i] == 1u ? -1 : 1;
      place(i, (uint32_t)__mul24((int)rank, step) + first, c.e1[i]);
    }
  } else {
    const uint32_t fits = base_s >= (uint32_t)kSecSlots ? 0u : (uint32_t)kSecSlots - base_s;  // small-queue ranks below this fit
#pragma unroll
    for (int i = 0; i < NB; ++i) {
      const uint32_t rank = __builtin_amdgcn_ubfe(below + running[i], sh[i], 10);
      const uint32_t up = base_o + rank, down = top - rank, behind = small + rank;
      uint32_t pos = kq[i] == 1u ? down : up;
      pos = kq[i] == 2u ? behind : pos;
      const bool out = kq[i] == 2u && rank >= fits;
      place(i, out ? top - (n_e + (rank - fits)) : pos, c.e1[i] | (out ? kQaSecond : 0u));
    }
  }
}

// The origin blocks of a lane's share decode to zero: their partial sums are written here.
template <int NB>
__device__ __forceinline__ void settle_origins(uint32_t where, float* partial, uint32_t tid = threadIdx.x) {
  if (__any((where >> 8) & 15u)) {
#pragma unroll
    for (int i = 0; i < NB; ++i)
      if ((where >> (8 + i)) & 1u) partial[tid * NB + (uint32_t)i] = 0.f;
  }
}

template <int NB, class Rec>
__device__ __forceinline__ void classify_stream(const DecodeTables& T, const Rec& rec, uint32_t nblk, uint32_t capacity,
                                                const GemvQueues& Q) {
  Classified<NB> c;
  classify_records<NB>(T, rec, nblk, c);
  settle_origins<NB>(c.where, Q.partial);
  queue_classified<NB>(c, capacity, Q);
}

// P2 of the GEMV kernels: unrank the tile's queued blocks and reduce them against the activation planes.
// Chunks of 64 queued blocks are handed out through a counter: the two generic chunks first (longest),
// then the chunks of the three fast decoders.  `hook(done, last, state)` (kHook) runs in every wavefront before
// each of its chunks of the fast decoders, with the number it has finished, and once more (last = true) when
// there is none left for it: where a caller puts work that does not depend on this tile and fills the issue
// slots this tile's decoders leave.  `state` is 0 at first and then whatever the hook returned last; the
// function returns the final one.
struct UnrankOperands {
  const uint32_t* xplanes;  // [nb][kPlaneDwords]
  const float* xscale;      // [nb]
  uint32_t nb;              // blocks per row
  float inv_nb;             // 1 / nb, for the block -> column split
  float g0, g1;             // the matrix's gain centroids
  uint32_t hook_state = 0;  // the state the hook is first called with
};

template <int TILE, bool kHook, int PLANES, class Hook>
__device__ __forceinline__ uint32_t unrank_tile(const DecodeTables& T, const GemvQueues& Q, const UnrankOperands& op, Hook&& hook) {
  constexpr int kTileBlocks = TILE;
  uint32_t tid = threadIdx.x;
  // inside a persistent loop over tiles: lane-derived values are formed here, per call, not carried around that loop
  if constexpr (kHook) asm volatile("" : "+v"(tid));
  const uint32_t lane = tid & 63u;
  uint32_t* ctrl = Q.ctrl;
  float* partial = Q.partial;
  const uint32_t* xplanes = op.xplanes;
  const float* xscale = op.xscale;
  const uint32_t nb = op.nb;
  const uint32_t n_odd = ctrl[kCtrlOdd], n_even = ctrl[kCtrlEven], n_sec = min(ctrl[kCtrlSec], (uint32_t)kSecSlots);
  const uint32_t n_gen_o = min(ctrl[kCtrlGenOdd], (uint32_t)kGenericSlots), n_gen_e = min(ctrl[kCtrlGenEven], (uint32_t)kGenericSlots);
  const uint32_t c_gen_o = n_gen_o ? 1u : 0u, c_gen_e = n_gen_e ? 1u : 0u, c_gen = c_gen_o + c_gen_e;
  const uint32_t c_odd = (n_odd + 63u) >> 6, c_even = (n_even + 63u) >> 6, c_sec = (n_sec + 63u) >> 6;
  auto ticket = [&]() {
    uint32_t t = 0;
    if (lane == 0) t = atomicAdd(&ctrl[kCtrlTicket], 1u);
    return (uint32_t)__shfl(t, 0, 64);
  };
  // what every decoder starts from: the block's local rank, class, column and scale
  struct Block {
    uint64_t li;
    uint32_t f, ci, col;
    float g;
  };
  auto open_block = [&](uint2 e, uint32_t f) {
    Block b;
    b.li = ((uint64_t)(e.y & 0x1FFFu) << 32) | e.x;
    b.ci = (e.y >> kQaClassShift) & 0x1FFu;
    b.f = f;
    const uint32_t row = (uint32_t)(((float)f + 0.5f) * op.inv_nb);
    b.col = f - __umul24(row, nb);  // both below 2^24: the full-rate multiply
    b.g = (e.y >> kQaGainShift) & 1u ? op.g1 : op.g0;
    return b;
  };
  // generic walk of one queued block (rare classes): coordinates packed four to a dword, then
  // the same integer dot products as the fast paths
  auto generic_block = [&](uint2 e, uint32_t f) {
    const Block b = open_block(e, f);
    const uint32_t* xp = xplanes + __umul24(b.col, (uint32_t)kPlaneDwords);
    const DevClass c = T.cls[b.ci];
    uint32_t w[6] = {0, 0, 0, 0, 0, 0};
    auto emit = [&](int p, int v) { w[p >> 2] |= ((uint32_t)v & 0xFFu) << (8 * (p & 3)); };
    if (c.meta & kMetaOdd) decode_odd(T, c, b.li, emit);
    else decode_even(T, c, b.li, emit);
    int d0 = 0, d1 = 0, d2 = 0;
#pragma unroll
    for (int q = 0; q < 6; ++q) {
      d0 = __builtin_amdgcn_sdot4((int)w[q], (int)xp[q], d0, false);
      d1 = __builtin_amdgcn_sdot4((int)w[q], (int)xp[6 + q], d1, false);
      if (PLANES == 3) d2 = __builtin_amdgcn_sdot4((int)w[q], (int)xp[12 + q], d2, false);
    }
    partial[b.f] = planes_to_float<PLANES>(d0, d1, d2) * xscale[b.col] * (c.inv_norm * b.g);
  };
  auto odd_block = [&](uint2 e, uint32_t f) {
    const Block b = open_block(e, f);
    const uint32_t* xp = xplanes + __umul24(b.col, (uint32_t)kPlaneDwords);
    const FastClass fc = T.fast[b.ci];
    int d0 = 0, d1 = 0, d2 = 0;
    odd_codes(T, fc, b.li, [&](int q, uint32_t sel) {
      const int w = (int)__builtin_amdgcn_perm(fc.tab_hi, fc.tab_lo, sel);
      d0 = __builtin_amdgcn_sdot4(w, (int)xp[q], d0, false);
      d1 = __builtin_amdgcn_sdot4(w, (int)xp[6 + q], d1, false);
      if (PLANES == 3) d2 = __builtin_amdgcn_sdot4(w, (int)xp[12 + q], d2, false);
    });
    partial[b.f] = planes_to_float<PLANES>(d0, d1, d2) * xscale[b.col] * (fc.inv_norm * b.g);
  };
  auto even_block = [&](uint2 e, uint32_t f, auto second) {
    constexpr bool kSecond = decltype(second)::value;
    const Block b = open_block(e, f);
    const uint32_t* xp = xplanes + __umul24(b.col, (uint32_t)kPlaneDwords);
    const FastClass fc = T.fast[b.ci];
    const uint32_t fv1 = fc.u0 >> 16;
    const uint32_t tab2_lo = fv1 << 8, tab2_hi = ((0u - fv1) & 0xFFu) << 8;
    int d0 = 0, d1 = 0, d2 = 0;
    even_codes<kSecond>(T, fc, b.li, [&](int q, uint32_t sel, uint32_t sel2) {
      int w = (int)__builtin_amdgcn_perm(fc.tab_hi, fc.tab_lo, sel);
      if (kSecond) w |= (int)__builtin_amdgcn_perm(tab2_hi, tab2_lo, sel2);
      d0 = __builtin_amdgcn_sdot4(w, (int)xp[q], d0, false);
      d1 = __builtin_amdgcn_sdot4(w, (int)xp[6 + q], d1, false);
      if (PLANES == 3) d2 = __builtin_amdgcn_sdot4(w, (int)xp[12 + q], d2, false);
    });
    partial[b.f] = planes_to_float<PLANES>(d0, d1, d2) * xscale[b.col] * (fc.inv_norm * b.g);
  };
  uint32_t chunk = ticket();
  // the generic chunks, kept out of the loop below: their code and registers are not the hot path's
  while (chunk < c_gen) {
    const uint32_t even = (chunk == 1u || !c_gen_o) ? 1u : 0u;
    if (lane < (even ? n_gen_e : n_gen_o)) generic_block(Q.gqa[even * kGenericSlots + lane], Q.gqf[even * kGenericSlots + lane]);
    chunk = ticket();
  }
  // Even and odd chunks alternate while both queues last: the even coset waits for tables in L2,
  // the odd one issues arithmetic, and wavefronts on either kind at the same time overlap the two.
  // The chunks of the small even queue come first (their queue ends in a partial chunk as well).
  const uint32_t c_pair = min(c_odd, c_even);
  const uint32_t c_all = c_gen + c_sec + c_odd + c_even;
  uint32_t done = 0, hook_state = op.hook_state;
  for (;; ++done, chunk = ticket()) {
    if constexpr (kHook) hook_state = hook(done, chunk >= c_all, hook_state);
    if (chunk >= c_all) break;
    const uint32_t ts = chunk - c_gen;
    if (ts < c_sec) {
      const uint32_t k = ts * 64u + lane;
      if (k < n_sec) even_block(Q.qa[kTileBlocks + k], Q.qf[detached(kTileBlocks + k)], std::true_type{});
      continue;
    }
    const uint32_t t = ts - c_sec;
    const bool paired = t < 2u * c_pair;
    const bool is_odd = paired ? (t & 1u) != 0u : c_odd > c_even;
    const uint32_t ordinal = paired ? t >> 1 : t - c_pair;
    const uint32_t k = ordinal * 64u + lane;
    if (is_odd) {
      const uint32_t at = min(k, (uint32_t)kTileBlocks - 1u);
      const uint2 e = Q.qa[at];
      // generic blocks that found their small queue full wait for the pass below
      if (k < n_odd && !(e.y >> 31)) odd_block(e, Q.qf[detached(at)]);
    } else {
      const uint32_t at = kTileBlocks - 1 - min(k, (uint32_t)kTileBlocks - 1u);
      const uint2 e = Q.qa[at];
      const bool mine = k < n_even;
      // blocks with a second free kind that found their queue full ride here, flagged
      if (__any(mine && (e.y & kQaSecond))) {
        if (mine) even_block(e, Q.qf[at], std::true_type{});
      } else {
        if (mine) even_block(e, Q.qf[at], std::false_type{});
      }
    }
  }
  if (ctrl[kCtrlGenOdd] > (uint32_t)kGenericSlots || ctrl[kCtrlGenEven] > (uint32_t)kGenericSlots) {
    // more generic blocks than the small queues hold (hostile input): the rest sit flagged in the odd queue
    for (uint32_t k = tid; k < n_odd; k += kWgThreads) {
      const uint2 e = Q.qa[k];
      if (e.y >> 31) generic_block(e, Q.qf[k]);
    }
  }
  return hook_state;
}

// Where a launch's activation comes from, and what it may do to produce it before the product.
struct ActivationSource {
  const __half* x;
  const float* x_f32;  // when set, the activation is these f32 values (a rotated activation) and x is unused
  const __half* x2;
  const __half* norm_w;
  __half* resid_out;
  float eps;
  uint32_t prologue;   // kPrologue*
  uint32_t nb, tail_w;
  const uint32_t* rot_signbits;
  const float* rot_small;
  float rot_inv;
  uint32_t rot_m, rot_k;
  bool writes_resid;   // this workgroup is the one that stores the new residual
  bool device_scope = false;  // a finished activation is read at device scope (another workgroup of this launch stored it)
};

// Fills the activation planes, scales and tail values in LDS from `a`, by every lane of the workgroup.
// `raw` (the tile's queue entries, block numbers and partial sums, free at this point) is the staging
// area of a derived or rotated activation; `request` is called once, right behind the loads of the
// activation's operands (the caller's first code bytes go out there).  Returns whether the staging
// area was used: the caller then needs a barrier before the area becomes queues again.  kInPlace: `raw` is the
// planes' own memory (rows of at most as many blocks as the workgroup has lanes, natural basis only).
template <int TILE, bool ROT, int PLANES, bool kInPlace = false, class Request>
__device__ __forceinline__ bool stage_activation(const ActivationSource& a, uint32_t* xplanes, float* xscale, float* xtail, uint8_t* raw,
                                                 float* partial, Request&& request_first_tile) {
  constexpr int kTileBlocks = TILE;
  constexpr int kRawBytes = TILE * 6 + 32;  // what a derived binary16 activation may take of the staging area
  uint32_t tid = threadIdx.x;
  // staged from inside a loop over tiles: lane-derived indices are formed here, not carried through the loop in registers
  if constexpr (kInPlace) asm volatile("" : "+v"(tid));
  const uint32_t lane = tid & 63u, wave = tid >> 6;
  const uint32_t nb = a.nb;
  const __half* xsrc = a.x;
  // A launch over matrices stored in a rotated basis rotates its activation itself: the
  // values go, signs applied, as f32 to the area the first tile's queues and
  // partial sums will use (free until then), are rotated there and quantised from there.
  const bool rotated = ROT && a.rot_m != 0;
  float* xf = reinterpret_cast<float*>(raw);
  const uint32_t d_in = nb * kDim + a.tail_w;
  auto signed_f32 = [&](uint32_t i, float v) { return ((a.rot_signbits[i >> 5] >> (i & 31u)) & 1u) ? -v : v; };
  if (a.prologue != kPrologueNone) {
    // Every workgroup derives the activation for itself (a few thousand values)
    // instead of waiting for a kernel of its own; it is staged, as binary16, where
    // the tile's queues will go.
    __half* xs = reinterpret_cast<__half*>(raw);
    // All of a lane's values are requested before the first is used (a load and its use per loop
    // iteration would pay the memory latency once per iteration): the rounds are counted at compile
    // time (3 covers 3072 values, 6 and 12 the wider rows), their loads are unconditional (a lane past
    // the row's end reads its last value) and a scheduling barrier keeps them ahead of the arithmetic.
    constexpr int kPerMax = (kRawBytes / 2 + kWgThreads - 1) / kWgThreads;
    const bool silu = a.prologue == kPrologueSiluMul;
    const __half* src1 = a.x2 ? a.x2 : a.x;
    const __half* src2 = silu ? a.x : a.norm_w;
    auto derive = [&](auto rounds, uint32_t base) {
      constexpr int kPer = decltype(rounds)::value;
      __half in0[kPer], in1[kPer], in2[kPer];
#pragma unroll
      for (int k = 0; k < kPer; ++k) {
        const uint32_t i = min(base + tid + (uint32_t)k * kWgThreads, d_in - 1u);
        in0[k] = load_half<kInPlace>(a.x + i);
        in1[k] = load_half<kInPlace>(src1 + i);
        in2[k] = src2[i];  // the norm's gains are constants (with SiLU this is x again, and unused)
      }
      request_first_tile();
      __builtin_amdgcn_sched_barrier(0);
      if (silu) {
#pragma unroll
        for (int k = 0; k < kPer; ++k) {
          const uint32_t i = base + tid + (uint32_t)k * kWgThreads;
          if (i < d_in) {
            const float g = __half2float(in1[k]);
            const float sg = __half2float(__float2half_rn(g / (1.0f + __expf(-g))));
            const __half h = __float2half_rn(sg * __half2float(in0[k]));
            if (rotated) xf[i] = signed_f32(i, __half2float(h));
            else xs[i] = h;
          }
        }
      } else {
        float* red = partial + kTileBlocks - kWaves;  // the end of the partial sums: beyond the f32 staging of a rotated launch
        float v[kPer];
        float ss = 0.f;
#pragma unroll
        for (int k = 0; k < kPer; ++k) {
          const uint32_t i = base + tid + (uint32_t)k * kWgThreads;
          v[k] = 0.f;
          if (i < d_in) {
            float r = __half2float(in0[k]);
            if (a.x2) r = __half2float(__float2half_rn(r + __half2float(in1[k])));
            if (a.resid_out && a.writes_resid) store_half<kInPlace>(a.resid_out + i, __float2half_rn(r));
            v[k] = r;
            ss += r * r;
          }
        }
        ss = wave_sum(ss);
        if (lane == 0) red[wave] = ss;
        __syncthreads();
        float total = 0.f;
#pragma unroll
        for (int w = 0; w < kWaves; ++w) total += red[w];
        const float inv = 1.0f / sqrtf(total / (float)d_in + a.eps);
#pragma unroll
        for (int k = 0; k < kPer; ++k) {
          const uint32_t i = base + tid + (uint32_t)k * kWgThreads;
          if (i < d_in) {
            const __half h = __float2half_rn(v[k] * inv * __half2float(in2[k]));
            if (rotated) xf[i] = signed_f32(i, __half2float(h));
            else xs[i] = h;
          }
        }
      }
    };
    const uint32_t n_per = (d_in + kWgThreads - 1) / kWgThreads;
    if constexpr (kInPlace) {
      // at most six rounds of operands in registers at a time: the wider SiLU rows go in runs of 6144 values
      // (a row sum of squares over more than 6144 values is refused by the host for this variant)
      if (n_per <= 3) derive(std::integral_constant<int, 3>{}, 0u);
      else
        for (uint32_t base = 0; base < d_in; base += 6u * kWgThreads) derive(std::integral_constant<int, 6>{}, base);
    } else {
      if (n_per <= 3) derive(std::integral_constant<int, kPerMax < 3 ? kPerMax : 3>{}, 0u);
      else if (n_per <= 6) derive(std::integral_constant<int, kPerMax < 6 ? kPerMax : 6>{}, 0u);
      else derive(std::integral_constant<int, kPerMax>{}, 0u);
    }
    __syncthreads();
    xsrc = xs;
  } else if (rotated) {
    request_first_tile();
    // eight values per lane and pass; a width that is not a multiple of eight ends one value at a time
    const uint32_t n8 = d_in & ~7u;
    for (uint32_t i = tid * 8u; i < n8; i += kWgThreads * 8u) {
      const uint4 h = *reinterpret_cast<const uint4*>(a.x + i);
      const uint32_t sg = a.rot_signbits[i >> 5] >> (i & 31u);
      const uint32_t w[4] = {h.x, h.y, h.z, h.w};
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const float lo = __half2float(__ushort_as_half((unsigned short)(w[q] & 0xFFFFu)));
        const float hi = __half2float(__ushort_as_half((unsigned short)(w[q] >> 16)));
        xf[i + 2 * q] = ((sg >> (2 * q)) & 1u) ? -lo : lo;
        xf[i + 2 * q + 1] = ((sg >> (2 * q + 1)) & 1u) ? -hi : hi;
      }
    }
    for (uint32_t i = n8 + tid; i < d_in; i += kWgThreads) xf[i] = signed_f32(i, __half2float(a.x[i]));
    __syncthreads();
  }
  if (rotated) {
    rotate_lds(xf, d_in, a.rot_m, a.rot_k, a.rot_inv, a.rot_small);
    __syncthreads();
    for (uint32_t col = tid; col < nb; col += kWgThreads)
      quantize_block_f32<PLANES>(xf + (size_t)col * kDim, xplanes + (size_t)col * kPlaneDwords, xscale + col);
    if (tid < a.tail_w) xtail[tid] = xf[(size_t)nb * kDim + tid];
  } else if (a.prologue != kPrologueNone) {
    if constexpr (kInPlace) {
      // the staging area is the planes' own: every lane reads its block before any lane writes (nb <= lanes)
      float v[kDim];
      load_block_f16(xsrc + (size_t)min(tid, nb ? nb - 1u : 0u) * kDim, v);
      const float tail_v = tid < a.tail_w ? __half2float(xsrc[(size_t)nb * kDim + tid]) : 0.f;
      __syncthreads();
      if (tid < nb) quantize_values<PLANES>(v, xplanes + (size_t)tid * kPlaneDwords, xscale + tid);
      if (tid < a.tail_w) xtail[tid] = tail_v;
    } else {
      for (uint32_t col = tid; col < nb; col += kWgThreads)
        quantize_block<PLANES>(xsrc + (size_t)col * kDim, xplanes + (size_t)col * kPlaneDwords, xscale + col);
      if (tid < a.tail_w) xtail[tid] = __half2float(xsrc[(size_t)nb * kDim + tid]);
    }
  } else {
    // a finished activation from global memory: this lane's block is requested, then the first tile's
    // code bytes, then the block is quantised (rows wider than 1024 blocks take further rounds)
    float v[kDim];
#pragma unroll
    for (int j = 0; j < kDim; ++j) v[j] = 0.f;
    if ((tid & ~63u) < nb) {  // wavefronts with a block to read (a row of tail columns only has none)
      const uint32_t c0 = min(tid, nb - 1u);
      if (a.x_f32) {
#pragma unroll
        for (int j = 0; j < kDim; ++j) v[j] = a.x_f32[(size_t)c0 * kDim + j];
      } else {
        // (an activation another workgroup of this launch stored is read at device scope; any other through the caches)
        if (kInPlace && a.device_scope) load_block_f16<true>(xsrc + (size_t)c0 * kDim, v);
        else load_block_f16<false>(xsrc + (size_t)c0 * kDim, v);
      }
    }
    float tail_v = 0.f;
    if (tid < a.tail_w) {
      if (a.x_f32) tail_v = a.x_f32[(size_t)nb * kDim + tid];
      else if (kInPlace && a.device_scope) tail_v = __half2float(load_half<true>(xsrc + (size_t)nb * kDim + tid));
      else tail_v = __half2float(xsrc[(size_t)nb * kDim + tid]);
    }
    request_first_tile();
    __builtin_amdgcn_sched_barrier(0);
    if (tid < nb) quantize_values<PLANES>(v, xplanes + (size_t)tid * kPlaneDwords, xscale + tid);
    if (tid < a.tail_w) xtail[tid] = tail_v;
    for (uint32_t col = tid + kWgThreads; col < nb; col += kWgThreads) {
      if (a.x_f32) quantize_block_f32<PLANES>(a.x_f32 + (size_t)col * kDim, xplanes + (size_t)col * kPlaneDwords, xscale + col);
      else quantize_block<PLANES>(xsrc + (size_t)col * kDim, xplanes + (size_t)col * kPlaneDwords, xscale + col);
    }
  }
  return a.prologue != kPrologueNone || rotated;
}

// LEAN: the Golay words and the support-arrangement table stay in L2, which leaves
// room for the full tile beside the activation planes of a very wide row.
// ROT: the launch can rotate its own activation (GroupArgs::rot_m); kept out of the other
// instantiations, whose hot loop it would otherwise cost registers and a few per cent.
// WIDE: the matrices are cap-13 ones (49-bit blocks in a dense stream, 48-bit indices): a lane extracts its blocks
// from the stream, and the class tables a 47-bit index cannot reach are read from device memory.
template <typename OutT, int TILE = kTileBlocks, bool LEAN = false, bool ROT = false, bool WIDE = false>
__global__ __launch_bounds__(kWgThreads) void gemv_tiles_kernel(GroupArgs a) {
  static_assert(!WIDE || (TILE == 4 * kWgThreads && !ROT), "the dense-stream variant takes four blocks per lane and no in-launch rotation");
  // the tile capacity of this instantiation (these shadow the namespace-level defaults)
  constexpr int kTileBlocks = TILE;
  constexpr int kP1Blocks = TILE / kWgThreads;
  constexpr int kPlanes = std::is_same<OutT, __half>::value ? 2 : 3;  // byte planes of the activation (quantize_values)
  extern __shared__ __align__(16) uint8_t smem[];
#ifdef LLVQ_PHASE_TIMING
  if (threadIdx.x == 0) g_phase_stamps[blockIdx.x * 8 + 3] = wall_clock64();
#endif
  const DecodeTables T = stage_tables<!LEAN, true, WIDE>(smem, a.tables);
  // A lane loads the records it classifies itself, HBM -> registers; the next tile's loads are
  // issued while the current one is being decoded.  The first tile's are issued right behind the
  // loads of the activation: the memory counter retires in order, so whatever is requested
  // after them would wait for HBM with them, and they are not needed before the activation is.
  typename std::conditional<WIDE, DenseRecords, LaneRecords<kP1Blocks>>::type pre;
#pragma unroll
  for (int k = 0; k < (int)(sizeof(pre.w) / sizeof(pre.w[0])); ++k) pre.w[k] = 0;
  if constexpr (WIDE) pre.s0 = 0;
  auto request_first_tile = [&]() { prefetch_records(a, blockIdx.x, threadIdx.x, pre); };
  const uint32_t nb = a.nblocks;
  uint32_t* xplanes = reinterpret_cast<uint32_t*>(smem + (LEAN ? kLdsImageBytesLean : kLdsImageBytes));
  float* xscale = reinterpret_cast<float*>(xplanes + (size_t)nb * kPlaneDwords);
  float* xtail = xscale + nb;
  // queue entries | block numbers | 32 bytes | partial sums: also the staging area of a derived or rotated activation
  uint8_t* raw = reinterpret_cast<uint8_t*>(xtail + 32 + (nb & 1u));  // 8-byte aligned: the queue entries are read as 64-bit words
  GemvQueues Q;
  Q.qa = reinterpret_cast<uint2*>(raw);
  Q.qf = reinterpret_cast<uint16_t*>(Q.qa + kTileBlocks + kSecSlots);
  Q.partial = reinterpret_cast<float*>(Q.qf + kTileBlocks + kSecSlots + 16);
  Q.gqa = reinterpret_cast<uint2*>(Q.partial + kTileBlocks);
  Q.gqf = reinterpret_cast<uint16_t*>(Q.gqa + 2 * kGenericSlots);
  Q.ctrl = reinterpret_cast<uint32_t*>(Q.gqf + 2 * kGenericSlots);
  float* partial = Q.partial;
  uint32_t* ctrl = Q.ctrl;
  static_assert((kTileBlocks + kSecSlots) % 4 == 0 && kGenericSlots % 2 == 0, "the arrays behind the 16-bit ones stay 8-byte aligned");
  const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
  const ActivationSource src{a.x, a.x_f32, a.x2, a.norm_w, a.resid_out, a.eps, a.prologue, nb, a.tail_w,
                             a.rot_signbits, a.rot_small, a.rot_inv, a.rot_m, a.rot_k, blockIdx.x == 0};
  if (stage_activation<kTileBlocks, ROT, kPlanes>(src, xplanes, xscale, xtail, raw, partial, request_first_tile))
    __syncthreads();  // the staging area becomes the tile's queues

#ifdef LLVQ_PHASE_TIMING
  if (threadIdx.x == 0) g_phase_stamps[blockIdx.x * 8 + 7] = wall_clock64();
#endif
  for (uint32_t tile = blockIdx.x; tile < a.n_tiles; tile += gridDim.x) {
    LLVQ_STAMP(0);
    MatArg M;
    uint32_t r0, rows;
    tile_of(a, tile, M, r0, rows);
    const uint32_t nblk = rows * nb;

    if (tid < (uint32_t)kCtrlWords) ctrl[tid] = 0;
    // P3 operands (row scales, tail weights): fetched now, used after the decode
    const uint32_t sub = lane >> 4, l16 = lane & 15u;
    constexpr int kP3Rounds = 2;  // 64 rows per round cover every tile of the usual shapes
    float rs_pre[kP3Rounds], tl_pre[kP3Rounds][2];
#pragma unroll
    for (int j = 0; j < kP3Rounds; ++j) {
      const uint32_t row = (wave * 4 + sub) + (uint32_t)j * (kWaves * 4);
      const bool ok = row < rows;
      rs_pre[j] = ok ? M.rscale[r0 + row] : 0.f;
      tl_pre[j][0] = (ok && l16 < a.tail_w) ? M.tail[(size_t)(r0 + row) * a.tail_w + l16] : 0.f;
      tl_pre[j][1] = (ok && l16 + 16 < a.tail_w) ? M.tail[(size_t)(r0 + row) * a.tail_w + l16 + 16] : 0.f;
    }
    __syncthreads();
    LLVQ_STAMP(1);

    // P1: classify and bin (a tile of tail-only rows has no blocks: its queues stay empty)
    if (nblk != 0) classify_stream<kP1Blocks>(T, pre, nblk, kTileBlocks, Q);
    __syncthreads();
    LLVQ_STAMP(2);
    prefetch_records(a, tile + gridDim.x, tid, pre);

    // P2: unrank and reduce
    unrank_tile<kTileBlocks, false, kPlanes>(T, Q, UnrankOperands{xplanes, xscale, nb, a.inv_nblocks, M.g0, M.g1}, [](uint32_t, bool, uint32_t) { return 0u; });
    LLVQ_STAMP(4);
    __syncthreads();
    LLVQ_STAMP(5);
    // P3: 16 lanes per row, fixed summation order
    for (uint32_t base = 0; base < rows; base += kWaves * 4) {
      const uint32_t j = base / (kWaves * 4);
      const uint32_t row = base + wave * 4 + sub;
      const bool ok = row < rows;
      float s = 0.f;
      if (ok)
        for (uint32_t b = l16; b < nb; b += 16u) s += partial[row * nb + b];  // fixed order per lane
      float rs, t0, t1;
      if (j < (uint32_t)kP3Rounds) {
        rs = j == 0 ? rs_pre[0] : rs_pre[1];
        t0 = j == 0 ? tl_pre[0][0] : tl_pre[1][0];
        t1 = j == 0 ? tl_pre[0][1] : tl_pre[1][1];
      } else {
        rs = ok ? M.rscale[r0 + row] : 0.f;
        t0 = (ok && l16 < a.tail_w) ? M.tail[(size_t)(r0 + row) * a.tail_w + l16] : 0.f;
        t1 = (ok && l16 + 16 < a.tail_w) ? M.tail[(size_t)(r0 + row) * a.tail_w + l16 + 16] : 0.f;
      }
      float v = s * rs;
      v = fmaf(t0, l16 < a.tail_w ? xtail[l16] : 0.f, v);
      v = fmaf(t1, l16 + 16 < a.tail_w ? xtail[l16 + 16] : 0.f, v);
#pragma unroll
      for (int o = 8; o >= 1; o >>= 1) v += __shfl_xor(v, o, 16);  // fixed tree inside each group of 16 lanes
      if (ok && l16 == 0) store_out<OutT>(M.y, r0 + row, v);
    }
    __syncthreads();
    LLVQ_STAMP(6);
  }
}


// The instantiations of gemv_tiles_kernel by (f32 output, tile, lean image, in-launch rotation).
template <typename OutT, bool ROT>
__host__ const void* gemv_kernel_of(uint32_t tile, bool lean) {
  if (lean) return reinterpret_cast<const void*>(gemv_tiles_kernel<OutT, kTileBlocks, true, ROT>);
  if (tile == (uint32_t)kTileBlocks) return reinterpret_cast<const void*>(gemv_tiles_kernel<OutT, kTileBlocks, false, ROT>);
  return reinterpret_cast<const void*>(gemv_tiles_kernel<OutT, kSmallTileBlocks, false, ROT>);
}
__host__ const void* gemv_kernel(bool f32, uint32_t tile, bool lean, bool rot) {
  if (f32) return rot ? gemv_kernel_of<float, true>(tile, lean) : gemv_kernel_of<float, false>(tile, lean);
  return rot ? gemv_kernel_of<__half, true>(tile, lean) : gemv_kernel_of<__half, false>(tile, lean);
}
// ... and for cap-13 matrices (full tile only, with the whole or the lean table image, no in-launch rotation)
__host__ const void* gemv_kernel_wide(bool f32, bool lean) {
  if (f32) return lean ? reinterpret_cast<const void*>(gemv_tiles_kernel<float, kTileBlocks, true, false, true>)
                       : reinterpret_cast<const void*>(gemv_tiles_kernel<float, kTileBlocks, false, false, true>);
  return lean ? reinterpret_cast<const void*>(gemv_tiles_kernel<__half, kTileBlocks, true, false, true>)
              : reinterpret_cast<const void*>(gemv_tiles_kernel<__half, kTileBlocks, false, false, true>);
}
template <class Fn>
__host__ void for_each_gemv_kernel(Fn&& fn) {
  for (int f32 = 0; f32 < 2; ++f32) {
    for (int rot = 0; rot < 2; ++rot) {
      fn(gemv_kernel(f32, kTileBlocks, false, rot));
      fn(gemv_kernel(f32, kSmallTileBlocks, false, rot));
      fn(gemv_kernel(f32, kTileBlocks, true, rot));
    }
    fn(gemv_kernel_wide(f32, false));
    fn(gemv_kernel_wide(f32, true));
  }
}

// ---- incoherence rotation of an activation ----------------------------------------
// x' = Q x for Q = (S (x) I_m)(I_k (x) H_m / sqrt m) D (llvq-quant/src/rotation.rs:97-105),
// in f32 like the reference's device rotation (llvq-cuda/kernels/llvq_rot.cuh): signs on
// load, radix-2 Walsh-Hadamard butterflies inside each group of m, then the k x k block
// across groups with the 1/sqrt m factor applied first.  One workgroup per activation row.
struct RotArgs {
  const __half* x;        // [rows, n]
  void* out;              // [rows, n] f32 or f16
  const uint32_t* signbits;
  const float* small;     // k x k
  uint32_t n, m, k;
  float inv;
};

// the identity rotation: binary16 -> f32
__global__ __launch_bounds__(256) void widen_kernel(const __half* __restrict__ x, float* __restrict__ out, uint32_t n) {
  const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) out[i] = __half2float(x[i]);
}

template <typename OutT>
__global__ __launch_bounds__(1024) void rotate_kernel(RotArgs a) {
  extern __shared__ __align__(16) float rot_s[];
  const uint32_t tid = threadIdx.x, n = a.n, m = a.m, k = a.k;
  const __half* x = a.x + (size_t)blockIdx.x * n;
  for (uint32_t i = tid; i < n; i += 1024) {
    const float v = __half2float(x[i]);
    rot_s[i] = ((a.signbits[i >> 5] >> (i & 31u)) & 1u) ? -v : v;
  }
  __syncthreads();
  rotate_lds(rot_s, n, m, k, a.inv, a.small);
  __syncthreads();
  OutT* out = reinterpret_cast<OutT*>(a.out) + (size_t)blockIdx.x * n;
  for (uint32_t i = tid; i < n; i += 1024) out[i] = (OutT)rot_s[i];
}

}  // namespace llvq

#include "gemv_seq.h"
#include "gemm_kernel.h"
#include "decoder.h"

// =================================================================================
// C ABI
// =================================================================================
using namespace llvq;

struct llvq_rt {
  int device = 0;
  hipStream_t stream = nullptr;
  uint8_t* blob = nullptr;  // one device allocation holding every table
  uint8_t* static_scratch = nullptr;  // this device's copy of `scratch` (kStaticScratchBytes)
  GlobalTables tables{};
  int cu_count = 0;
  // rotations by (width, seed) — shared by every matrix that consumes the same activation
  // (llvq-llm/src/fused.rs:672-674) — and the scratch rotated activations land in
  struct DevRotation {
    uint32_t n = 0, m = 0, k = 0;
    uint64_t seed = 0;
    float inv = 1.f;
    uint32_t* signbits = nullptr;
    float* small = nullptr;
  };
  std::vector<DevRotation*> rotations;
  float* rot_scratch = nullptr;   // one rotated activation, f32
  size_t rot_scratch_elems = 0;
  __half* rot_rows = nullptr;     // rotated batch rows, f16 (matrix-core path)
  size_t rot_rows_bytes = 0;
  // workspace of the batched kernels: partial sums [S, n_bands, M, 64]
  float* gemm_ws = nullptr;
  size_t gemm_ws_bytes = 0;
  // a batch's activations in K-step tiles [n_steps, m_pad, 32] (pipelined batched kernel)
  __half* gemm_xt = nullptr;
  size_t gemm_xt_bytes = 0;
};

struct llvq_mat {
  std::string name;
  uint32_t d_out = 0, d_in = 0, nblocks = 0, tail_w = 0;
  uint32_t record_bits = 48;  // 48: 6-byte records (shell cap 12); 49: the dense stream of shell cap 13
  float g[2] = {0, 0};
  uint8_t* codes = nullptr;  // device
  float* rscale = nullptr;   // device
  float* tail = nullptr;     // device
  uint64_t device_bytes = 0;
  uint64_t encoded_bytes = 0;
  bool has_rotation = false;
  uint64_t rotation_seed = 0;
  const llvq_rt::DevRotation* rot = nullptr;  // owned by the runtime
};

struct llvq_seq {
  uint8_t* blob = nullptr;  // one device allocation: tiles | items | counters | status
  SeqArgs args{};
  uint32_t tile = 0, grid = 0, n_items = 0;
  bool lean = false, f32 = false, wide = false;
  size_t lds = 0;
  uint32_t* own_status = nullptr;  // the status word inside `blob` (args.status may point at a word several sequences share)
};

static thread_local std::string g_last_error;

// Workspace of llvq_hip_gemm_static: device memory the library never allocates or frees.  The
// array's name is only a host-side handle; its device address differs per GPU and is asked for
// once per device, with that device current, at llvq_hip_runtime_create.
constexpr size_t kStaticScratchBytes = (size_t)LLVQ_STATIC_SCRATCH_BYTES;
static __device__ __align__(256) uint8_t scratch[kStaticScratchBytes];
constexpr int kMaxDevices = 64;
static uint8_t* g_scratch_ptr[kMaxDevices] = {};

static int fail(int code, const std::string& msg) {
  g_last_error = msg;
  return code;
}
static int hip_fail(hipError_t e, const char* what) {
  return fail(LLVQ_ERR_DEVICE, std::string(what) + ": " + hipGetErrorString(e));
}
#define HIP_TRY(expr)                                  \
  do {                                                 \
    hipError_t e_ = (expr);                            \
    if (e_ != hipSuccess) return hip_fail(e_, #expr);  \
  } while (0)

extern "C" {

const char* llvq_hip_last_error(void) { return g_last_error.c_str(); }
const char* llvq_hip_version(void) { return "llvq-hip 0.1 (gfx950)"; }

uint64_t llvq_hip_codebook_fingerprint(void) { return codebook_fingerprint(); }

int llvq_hip_host_decode(uint64_t idx, int8_t point[24], int* shell) {
  return host_decode(idx, point, shell) ? 1 : 0;
}

int llvq_hip_runtime_create(int device, void* hip_stream, llvq_rt** out) {
  if (!out) return fail(LLVQ_ERR_INVALID_ARGUMENT, "runtime_create: out is null");
  *out = nullptr;
  const Codebook& cb = codebook();
  if (cb.classes.size() != 383 || codebook_fingerprint() != kFingerprint)
    return fail(LLVQ_ERR_CODEBOOK_MISMATCH, "this build's index map does not reproduce the published fingerprint");
  HIP_TRY(hipSetDevice(device));
  auto* rt = new llvq_rt();
  rt->device = device;
  rt->stream = reinterpret_cast<hipStream_t>(hip_stream);
  hipDeviceProp_t prop;
  hipError_t e = hipGetDeviceProperties(&prop, device);
  if (e != hipSuccess) { delete rt; return hip_fail(e, "hipGetDeviceProperties"); }
  rt->cu_count = prop.multiProcessorCount;
  if (device >= 0 && device < kMaxDevices) {
    if (!g_scratch_ptr[device]) {
      void* p = nullptr;
      e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
      if (e != hipSuccess) { delete rt; return hip_fail(e, "hipGetSymbolAddress(scratch)"); }
      g_scratch_ptr[device] = reinterpret_cast<uint8_t*>(p);
    }
    rt->static_scratch = g_scratch_ptr[device];
  }
  // one blob: LDS image | generic class records | off-support table | deposit masks | walk-tail codes
  if (cb.on_lut.size() > (size_t)kOnLutSlots) { delete rt; return fail(LLVQ_ERR_UNSUPPORTED, "support-arrangement table outgrew its LDS slot"); }
  const size_t off_starts = sizeof(TableImage);
  static_assert(sizeof(TableImage) % 8 == 0, "the class starts follow the image 8-byte aligned");
  const size_t off_cls = (off_starts + sizeof(cb.starts) + 15) & ~(size_t)15;
  const size_t off_lut = off_cls + sizeof(cb.dev_classes);
  const size_t off_exp = (off_lut + cb.off_lut.size() * 4 + 15) & ~(size_t)15;
  const size_t off_tail = off_exp + sizeof(cb.expand);
  static_assert(sizeof(cb.expand) % 16 == 0, "the walk-tail codes are read as 8-byte units");
  // ... | every fast-path class record | the whole class-find table, both levels (for 48-bit indices)
  const size_t off_wfast = (off_tail + cb.tail_codes.size() * 8 + 15) & ~(size_t)15;
  const size_t off_wlut = off_wfast + sizeof(cb.fast);
  const size_t off_wlut2 = off_wlut + sizeof(cb.lut);
  const size_t total = off_wlut2 + cb.lut2.size() * 2;
  std::vector<uint8_t> host(total, 0);
  auto* img = reinterpret_cast<TableImage*>(host.data());
  std::memcpy(img->golay, cb.golay, sizeof img->golay);
  std::memcpy(img->fast, cb.fast, sizeof img->fast);
  std::memcpy(img->starts, cb.starts, sizeof img->starts);
  std::memcpy(img->lut, cb.lut, sizeof img->lut);
  // a 47-bit index reaches no class past kFastLds - 2 and no second-level table past kLut2Lds
  uint32_t lut2_used = 0;
  for (uint16_t e : img->lut)
    if (!(e & kLutFinal)) lut2_used = std::max<uint32_t>(lut2_used, (uint32_t)e + (uint32_t)kLut2Span);
  if (lut2_used > (uint32_t)kLut2Lds || lut2_used > cb.lut2.size() || cb.starts[kFastLds - 1] < (1ULL << 47)) {
    delete rt;
    return fail(LLVQ_ERR_UNSUPPORTED, "class-find tables outgrew their LDS slots");
  }
  std::memcpy(img->lut2, cb.lut2.data(), (size_t)lut2_used * 2);
  std::memcpy(host.data() + off_starts, cb.starts, sizeof(cb.starts));
  std::memcpy(img->rcp, cb.rcp, sizeof img->rcp);
  std::memcpy(img->step, cb.step + kTailSlots * 25 * 2, sizeof img->step);
  std::memcpy(img->tail_meta, cb.tail_meta, sizeof img->tail_meta);
  std::memcpy(img->pdep4, cb.pdep4, sizeof img->pdep4);
  std::memcpy(img->on_lut, cb.on_lut.data(), cb.on_lut.size() * 4);
  std::memcpy(host.data() + off_cls, cb.dev_classes, sizeof(cb.dev_classes));
  std::memcpy(host.data() + off_lut, cb.off_lut.data(), cb.off_lut.size() * 4);
  std::memcpy(host.data() + off_exp, cb.expand, sizeof(cb.expand));
  std::memcpy(host.data() + off_tail, cb.tail_codes.data(), cb.tail_codes.size() * 8);
  std::memcpy(host.data() + off_wfast, cb.fast, sizeof(cb.fast));
  std::memcpy(host.data() + off_wlut, cb.lut, sizeof(cb.lut));
  std::memcpy(host.data() + off_wlut2, cb.lut2.data(), cb.lut2.size() * 2);
  e = hipMalloc(reinterpret_cast<void**>(&rt->blob), total);
  if (e != hipSuccess) { delete rt; return hip_fail(e, "hipMalloc(tables)"); }
  e = hipMemcpy(rt->blob, host.data(), total, hipMemcpyHostToDevice);
  if (e != hipSuccess) { (void)hipFree(rt->blob); delete rt; return hip_fail(e, "hipMemcpy(tables)"); }
  rt->tables.image = reinterpret_cast<const TableImage*>(rt->blob);
  rt->tables.starts = reinterpret_cast<const uint64_t*>(rt->blob + off_starts);
  rt->tables.cls = reinterpret_cast<const DevClass*>(rt->blob + off_cls);
  rt->tables.off_lut = reinterpret_cast<const uint32_t*>(rt->blob + off_lut);
  rt->tables.expand = reinterpret_cast<const uint32_t*>(rt->blob + off_exp);
  rt->tables.tail_codes = reinterpret_cast<const uint64_t*>(rt->blob + off_tail);
  rt->tables.wide_fast = reinterpret_cast<const FastClass*>(rt->blob + off_wfast);
  rt->tables.wide_lut = reinterpret_cast<const uint16_t*>(rt->blob + off_wlut);
  rt->tables.wide_lut2 = reinterpret_cast<const uint16_t*>(rt->blob + off_wlut2);
  // the activation tile of a wide matrix pushes dynamic LDS past the 64 KB default
  const int max_lds = 160 * 1024;
  for_each_gemv_kernel([&](const void* kernel) { (void)hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, max_lds); });
  (void)hipFuncSetAttribute(reinterpret_cast<const void*>(rotate_kernel<float>), hipFuncAttributeMaxDynamicSharedMemorySize, max_lds);
  (void)hipFuncSetAttribute(reinterpret_cast<const void*>(rotate_kernel<__half>), hipFuncAttributeMaxDynamicSharedMemorySize, max_lds);
  (void)hipFuncSetAttribute(reinterpret_cast<const void*>(gemm_tiles_kernel<8>), hipFuncAttributeMaxDynamicSharedMemorySize, max_lds);
  (void)hipFuncSetAttribute(reinterpret_cast<const void*>(gemm_tiles_kernel<12>), hipFuncAttributeMaxDynamicSharedMemorySize, max_lds);
  *out = rt;
  return LLVQ_OK;
}

void llvq_hip_runtime_destroy(llvq_rt* rt) {
  if (!rt) return;
  (void)hipSetDevice(rt->device);
  (void)hipFree(rt->blob);
  (void)hipFree(rt->gemm_ws);
  (void)hipFree(rt->gemm_xt);
  (void)hipFree(rt->rot_scratch);
  (void)hipFree(rt->rot_rows);
  for (auto* r : rt->rotations) {
    (void)hipFree(r->signbits);
    (void)hipFree(r->small);
    delete r;
  }
  delete rt;
}

#ifdef LLVQ_PHASE_TIMING
// Tuning builds only: the phase timestamps of the last gemv_tiles_kernel launch ([workgroup][8]) and the stage
// timestamps of the last gemm_tiles_kernel launch ([workgroup][wavefront][4]).
int llvq_hip_debug_phase_stamps(unsigned long long* out, size_t n) {
  return (int)hipMemcpyFromSymbol(out, HIP_SYMBOL(g_phase_stamps), n * sizeof(unsigned long long));
}
int llvq_hip_debug_gemm_stamps(unsigned long long* out, size_t n) {
  return (int)hipMemcpyFromSymbol(out, HIP_SYMBOL(g_gemm_stamps), n * sizeof(unsigned long long));
}
#endif

int llvq_hip_synchronize(llvq_rt* rt) {
  if (!rt) return fail(LLVQ_ERR_INVALID_ARGUMENT, "synchronize: runtime is null");
  HIP_TRY(hipStreamSynchronize(rt->stream));
  return LLVQ_OK;
}

// The device tables of rotation (n, seed), built once per runtime.  Also makes
// sure the f32 scratch holds n values.
static int runtime_rotation(llvq_rt* rt, uint32_t n, uint64_t seed, const llvq_rt::DevRotation** out) {
  for (auto* r : rt->rotations)
    if (r->n == n && r->seed == seed) { *out = r; return LLVQ_OK; }
  RotationTables t;
  std::string err;
  if (!build_rotation(n, seed, &t, &err)) return fail(LLVQ_ERR_UNSUPPORTED, err);
  if ((size_t)n * sizeof(float) > 160 * 1024 - 64)
    return fail(LLVQ_ERR_UNSUPPORTED, "width " + std::to_string(n) + " does not fit the rotation kernel's LDS");
  auto* r = new llvq_rt::DevRotation();
  r->n = t.n; r->m = t.m; r->k = t.k; r->seed = seed; r->inv = t.inv;
  hipError_t e = hipMalloc(reinterpret_cast<void**>(&r->signbits), t.signbits.size() * 4);
  if (e == hipSuccess) e = hipMemcpy(r->signbits, t.signbits.data(), t.signbits.size() * 4, hipMemcpyHostToDevice);
  if (e == hipSuccess) e = hipMalloc(reinterpret_cast<void**>(&r->small), t.small.size() * 4);
  if (e == hipSuccess) e = hipMemcpy(r->small, t.small.data(), t.small.size() * 4, hipMemcpyHostToDevice);
  if (e == hipSuccess && n > rt->rot_scratch_elems) {
    (void)hipFree(rt->rot_scratch);
    rt->rot_scratch = nullptr;
    rt->rot_scratch_elems = 0;
    e = hipMalloc(reinterpret_cast<void**>(&rt->rot_scratch), (size_t)n * sizeof(float));
    if (e == hipSuccess) rt->rot_scratch_elems = n;
  }
  if (e != hipSuccess) {
    (void)hipFree(r->signbits);
    (void)hipFree(r->small);
    delete r;
    return hip_fail(e, "rotation tables");
  }
  rt->rotations.push_back(r);
  *out = r;
  return LLVQ_OK;
}

static int upload_impl(llvq_rt* rt, const std::string& name, uint32_t d_out, uint32_t d_in,
                       uint32_t shell_cap, uint32_t n_centroids, const double* centroids,
                       const double* row_scales, const float* tail, const uint8_t* codes,
                       size_t code_bytes, bool has_rotation, uint64_t rotation_seed, llvq_mat** out) {
  if (shell_cap > (uint32_t)kMaxShell)
    return fail(LLVQ_ERR_INCONSISTENT, name + ": shell cap " + std::to_string(shell_cap) +
                                           " exceeds the supported ball (m <= 13)");
  // one gain bit is compiled into the kernels (llvq-llm/src/fused.rs:1168-1177)
  if (n_centroids != 2)
    return fail(LLVQ_ERR_UNSUPPORTED, name + ": " + std::to_string(n_centroids) +
                                          " centroids, but the kernels hard-code 1 gain bit");
  const int ib = index_bits(shell_cap);
  if (ib + 1 != 48 && ib + 1 != (int)kDenseBits)
    return fail(LLVQ_ERR_UNSUPPORTED, name + ": shell cap " + std::to_string(shell_cap) + " packs " +
                                          std::to_string(ib + 1) +
                                          " bits per block; the kernels read 6-byte records (cap 12) and the 49-bit stream of cap 13");
  const uint32_t record_bits = (uint32_t)ib + 1u;
  const uint32_t nblocks = d_in / kDim, tail_w = d_in % kDim;
  const uint64_t total_blocks = (uint64_t)d_out * nblocks;
  if ((unsigned __int128)total_blocks * record_bits > (unsigned __int128)code_bytes * 8)
    return fail(LLVQ_ERR_TRUNCATED, "file ends mid-code stream");
  if (d_out == 0 || d_in == 0) return fail(LLVQ_ERR_INVALID_ARGUMENT, name + ": empty matrix");
  if ((total_blocks && !codes) || !centroids || !row_scales || (tail_w && !tail))
    return fail(LLVQ_ERR_INVALID_ARGUMENT, name + ": a required array is null");
  // Index range (format.rs:389-392).  The bound is N(13) whatever the cap; a
  // 47-bit field cannot exceed it (2^47 < N(13)), so at cap 12 this never fires.
  if (ib < 64 && ((1ULL << ib) - 1) > kN13) {
    // (only the 48-bit field of cap 13 can: block b is the record_bits bits from bit record_bits * b on)
    for (uint64_t b = 0; b < total_blocks; ++b) {
      const uint64_t bit = b * record_bits;
      const uint32_t sh = (uint32_t)(bit & 7u), nbytes = (sh + record_bits + 7u) >> 3;
      uint64_t acc = 0;
      for (uint32_t k = 0; k < 7u; ++k) acc = (acc << 8) | (k < nbytes ? codes[(bit >> 3) + k] : 0u);
      const uint64_t v = (acc >> (56u - sh - record_bits)) & ((1ULL << record_bits) - 1u);
      if ((v >> 1) > kN13)
        return fail(LLVQ_ERR_INDEX_OUT_OF_RANGE,
                    name + ": index " + std::to_string(v >> 1) + " is not a codebook member");
    }
  }

  HIP_TRY(hipSetDevice(rt->device));
  const llvq_rt::DevRotation* rot = nullptr;
  if (has_rotation) {
    const int rc = runtime_rotation(rt, d_in, rotation_seed, &rot);
    if (rc) return rc;
  }
  auto* m = new llvq_mat();
  m->has_rotation = has_rotation;
  m->rotation_seed = rotation_seed;
  m->rot = rot;
  m->name = name;
  m->d_out = d_out;
  m->d_in = d_in;
  m->nblocks = nblocks;
  m->tail_w = tail_w;
  m->record_bits = record_bits;
  m->g[0] = (float)centroids[0];  // fused.rs:1209
  m->g[1] = (float)centroids[1];
  std::vector<float> rs(d_out);
  for (uint32_t r = 0; r < d_out; ++r) rs[r] = (float)row_scales[r];  // fused.rs:1210
  const size_t code_len = (size_t)((total_blocks * record_bits + 7) / 8);
  const size_t code_alloc = ((code_len + 3) & ~(size_t)3) + 64;  // slack so wide loads may run past the last record
  const size_t tail_len = (size_t)d_out * tail_w * sizeof(float);
  auto cleanup = [&](hipError_t e, const char* what) {
    (void)hipFree(m->codes);
    (void)hipFree(m->rscale);
    (void)hipFree(m->tail);
    delete m;
    return hip_fail(e, what);
  };
  hipError_t e;
  if ((e = hipMalloc(reinterpret_cast<void**>(&m->codes), code_alloc)) != hipSuccess) return cleanup(e, "hipMalloc(codes)");
  if ((e = hipMemset(m->codes, 0, code_alloc)) != hipSuccess) return cleanup(e, "hipMemset(codes)");
  if (code_len && (e = hipMemcpy(m->codes, codes, code_len, hipMemcpyHostToDevice)) != hipSuccess) return cleanup(e, "hipMemcpy(codes)");
  // 64 floats of slack: the batched kernel reads the scales of a whole 64-row band, four at a time
  rs.resize((size_t)d_out + 64, 0.f);
  if ((e = hipMalloc(reinterpret_cast<void**>(&m->rscale), rs.size() * sizeof(float))) != hipSuccess) return cleanup(e, "hipMalloc(rscale)");
  if ((e = hipMemcpy(m->rscale, rs.data(), rs.size() * sizeof(float), hipMemcpyHostToDevice)) != hipSuccess) return cleanup(e, "hipMemcpy(rscale)");
  // zero-length arrays become one-element dummies (fused_cuda.rs:1084-1098)
  if ((e = hipMalloc(reinterpret_cast<void**>(&m->tail), tail_len ? tail_len : sizeof(float))) != hipSuccess) return cleanup(e, "hipMalloc(tail)");
  if (tail_len && (e = hipMemcpy(m->tail, tail, tail_len, hipMemcpyHostToDevice)) != hipSuccess) return cleanup(e, "hipMemcpy(tail)");
  m->device_bytes = code_alloc + rs.size() * sizeof(float) + (tail_len ? tail_len : sizeof(float));
  m->encoded_bytes = code_len + (uint64_t)d_out * 8 + tail_len + 16;
  *out = m;
  return LLVQ_OK;
}

int llvq_hip_matrix_upload(llvq_rt* rt, const llvq_matrix_desc* d, llvq_mat** out) {
  if (!rt || !d || !out) return fail(LLVQ_ERR_INVALID_ARGUMENT, "matrix_upload: null argument");
  *out = nullptr;
  return upload_impl(rt, d->name ? d->name : "", d->d_out, d->d_in, d->shell_cap, d->n_centroids,
                     d->centroids, d->row_scales, d->tail, d->codes, d->code_bytes,
                     d->has_rotation != 0, d->rotation_seed, out);
}

int llvq_hip_read_header(const uint8_t* buf, size_t len, size_t* pos, uint32_t* version,
                         uint32_t* n_matrices) {
  if (!buf || !pos || !version || !n_matrices || *pos > len)
    return fail(LLVQ_ERR_INVALID_ARGUMENT, "read_header: bad argument");
  std::string err;
  const int rc = parse_header(buf, len, pos, version, n_matrices, &err);
  return rc ? fail(rc, err) : LLVQ_OK;
}

int llvq_hip_parse_matrix_record(const uint8_t* buf, size_t len, size_t* pos, llvq_record_info* out) {
  if (!buf || !pos || !out || *pos > len) return fail(LLVQ_ERR_INVALID_ARGUMENT, "parse_matrix_record: bad argument");
  RecordView r;
  std::string err;
  size_t p = *pos;
  const int rc = parse_matrix_record(buf, len, &p, &r, &err);
  if (rc) return fail(rc, err);
  std::memset(out, 0, sizeof *out);
  std::strncpy(out->name, r.name.c_str(), sizeof out->name - 1);
  out->d_out = r.d_out;
  out->d_in = r.d_in;
  out->shell_cap = r.shell_cap;
  out->n_centroids = r.n_centroids;
  out->rotation_seed = r.rotation_seed;
  out->has_rotation = r.has_rotation ? 1 : 0;
  out->centroids_off = r.centroids_off;
  out->row_scales_off = r.row_scales_off;
  out->tail_off = r.tail_off;
  out->codes_off = r.codes_off;
  out->code_bytes = r.code_bytes;
  *pos = p;
  return LLVQ_OK;
}

int llvq_hip_parse_raw_tensor(const uint8_t* buf, size_t len, size_t* pos, uint32_t version, llvq_raw_info* out) {
  if (!buf || !pos || !out || *pos > len) return fail(LLVQ_ERR_INVALID_ARGUMENT, "parse_raw_tensor: bad argument");
  RawTensorView t;
  std::string err;
  size_t p = *pos;
  const int rc = parse_raw_tensor(buf, len, &p, version, &t, &err);
  if (rc) return fail(rc, err);
  std::memset(out, 0, sizeof *out);
  std::strncpy(out->name, t.name.c_str(), sizeof out->name - 1);
  out->rank = (uint32_t)t.dims.size();
  for (size_t i = 0; i < t.dims.size() && i < 8; ++i) out->dims[i] = t.dims[i];
  out->tag = t.tag;
  out->bits = t.bits;
  out->group = t.group;
  out->count = t.count;
  out->data_off = t.data_off;
  out->data_len = t.data_len;
  out->scales_off = t.scales_off;
  out->biases_off = t.biases_off;
  *pos = p;
  return LLVQ_OK;
}

int llvq_hip_parse_blob(const uint8_t* buf, size_t len, size_t* pos, llvq_blob_info* out) {
  if (!buf || !pos || !out || *pos > len) return fail(LLVQ_ERR_INVALID_ARGUMENT, "parse_blob: bad argument");
  BlobView b;
  std::string err;
  size_t p = *pos;
  const int rc = parse_blob(buf, len, &p, &b, &err);
  if (rc) return fail(rc, err);
  std::memset(out, 0, sizeof *out);
  std::strncpy(out->name, b.name.c_str(), sizeof out->name - 1);
  out->data_off = b.data_off;
  out->data_len = b.data_len;
  *pos = p;
  return LLVQ_OK;
}

int llvq_hip_matrix_from_record(llvq_rt* rt, const uint8_t* buf, size_t len, size_t* pos,
                                llvq_mat** out) {
  if (!rt || !buf || !pos || !out || *pos > len)
    return fail(LLVQ_ERR_INVALID_ARGUMENT, "matrix_from_record: bad argument");
  *out = nullptr;
  RecordView r;
  std::string err;
  size_t p = *pos;
  int rc = parse_matrix_record(buf, len, &p, &r, &err);
  if (rc) return fail(rc, err);
  rc = upload_impl(rt, r.name, r.d_out, r.d_in, r.shell_cap, r.n_centroids, r.centroids.data(),
                   r.row_scales.data(), r.tail.data(), r.codes, r.code_bytes, r.has_rotation, r.rotation_seed, out);
  if (rc == LLVQ_OK) *pos = p;
  return rc;
}

void llvq_hip_matrix_free(llvq_rt* rt, llvq_mat* m) {
  if (!m) return;
  if (rt) (void)hipSetDevice(rt->device);
  (void)hipFree(m->codes);
  (void)hipFree(m->rscale);
  (void)hipFree(m->tail);
  delete m;
}

int llvq_hip_matrix_info(const llvq_mat* m, uint32_t* d_out, uint32_t* d_in, uint32_t* nblocks,
                         uint32_t* tail_w, uint64_t* device_bytes) {
  if (!m) return fail(LLVQ_ERR_INVALID_ARGUMENT, "matrix_info: matrix is null");
  if (d_out) *d_out = m->d_out;
  if (d_in) *d_in = m->d_in;
  if (nblocks) *nblocks = m->nblocks;
  if (tail_w) *tail_w = m->tail_w;
  if (device_bytes) *device_bytes = m->device_bytes;
  return LLVQ_OK;
}

const char* llvq_hip_matrix_name(const llvq_mat* m) { return m ? m->name.c_str() : ""; }

// Rows per tile.  The workgroups take tiles in rounds of `grid`; a launch lasts rounds x (a tile's
// blocks + what a tile costs whatever its size: barriers, row sums, the wait for its first code
// bytes, taken as kTileFixedBlocks blocks' worth).  For k = 1, 2, ... rounds the best tile is the
// smallest that needs no more than k rounds; the cheapest of those that fit the tile capacity wins
// (7168 rows of 213 blocks on 256 CUs: 14 rows in exactly 2 rounds, not 19 rows in 1.5).
constexpr uint32_t kTileFixedBlocks = 400;
static uint32_t pick_rows_per_tile(const llvq_mat* const* mats, int n, uint32_t nblocks, uint32_t grid, uint32_t tile) {
  const uint32_t cap = nblocks ? (tile / nblocks ? tile / nblocks : 1u) : 0xFFFFFFFFu;
  uint64_t total = 0;
  for (int i = 0; i < n; ++i) total += mats[i]->d_out;
  auto tiles_at = [&](uint32_t r) {
    uint64_t t = 0;
    for (int i = 0; i < n; ++i) t += (mats[i]->d_out + r - 1) / r;
    return t;
  };
  uint32_t best = cap == 0xFFFFFFFFu ? (uint32_t)((total + grid - 1) / grid) : cap;
  if (best < 1) best = 1;
  uint64_t best_cost = ((tiles_at(best) + grid - 1) / grid) * ((uint64_t)best * nblocks + kTileFixedBlocks);
  for (uint32_t k = 1; k <= 16; ++k) {
    uint32_t r = (uint32_t)((total + (uint64_t)k * grid - 1) / ((uint64_t)k * grid));
    if (r < 1) r = 1;
    for (uint32_t tries = 0; tries < 64 && r <= cap && tiles_at(r) > (uint64_t)k * grid; ++tries) ++r;
    if (r > cap || tiles_at(r) > (uint64_t)k * grid) continue;
    const uint64_t cost = (uint64_t)k * ((uint64_t)r * nblocks + kTileFixedBlocks);
    if (cost < best_cost || (cost == best_cost && r > best)) {
      best_cost = cost;
      best = r;
    }
  }
  return best;
}

// Whether a launch over rows of this width can stage a derived activation where
// its first tile's queues go.
struct GemvShape {
  uint32_t tile;
  bool lean;
  size_t lds;
};

// The kernel variant for rows of nblocks blocks: the full tile with the whole table
// image in LDS where that fits, else the full tile with the lean image, else the half tile.
static GemvShape pick_gemv_shape(uint32_t nblocks) {
  GemvShape s{(uint32_t)kTileBlocks, false, gemv_lds_bytes(nblocks, kTileBlocks)};
  if (s.lds <= 160 * 1024) return s;
  s = GemvShape{(uint32_t)kTileBlocks, true, gemv_lds_bytes(nblocks, kTileBlocks, kLdsImageBytesLean)};
  if (s.lds <= 160 * 1024) return s;
  return GemvShape{(uint32_t)kSmallTileBlocks, false, gemv_lds_bytes(nblocks, kSmallTileBlocks)};
}

static bool prologue_fits(const llvq_mat* m0) {
  return (size_t)m0->d_in * 2 <= (size_t)pick_gemv_shape(m0->nblocks).tile * 6 + 32;
}

// Whether a launch over rows of this width can rotate its own activation: the f32
// values take the place of the first tile's queues and partial sums.
static bool rotation_fits(const llvq_mat* m0) {
  if (m0->record_bits != 48) return false;  // the dense-stream kernels have no in-launch rotation: a kernel of its own rotates
  const size_t tile = pick_gemv_shape(m0->nblocks).tile;
  return (size_t)m0->d_in * 4 + 64 <= tile * 6 + 32 + tile * 8;
}

struct Prologue {
  uint32_t kind = kPrologueNone;
  const void* x2 = nullptr;
  const void* norm_w = nullptr;
  void* resid_out = nullptr;
  float eps = 0.f;
};

static int launch_group(llvq_rt* rt, const llvq_mat* const* mats, int n, const void* x, void* const* y,
                        int y_dtype, const Prologue* pro = nullptr, const float* x_f32 = nullptr,
                        const llvq_rt::DevRotation* rot = nullptr) {
  const llvq_mat* m0 = mats[0];
  if (y_dtype != LLVQ_F32 && y_dtype != LLVQ_F16) return fail(LLVQ_ERR_INVALID_ARGUMENT, "gemv: unknown output dtype");
  const GemvShape shape = pick_gemv_shape(m0->nblocks);
  const uint32_t tile = shape.tile;
  const size_t lds = shape.lds;
  if (lds > 160 * 1024 || m0->nblocks > tile)
    return fail(LLVQ_ERR_UNSUPPORTED, m0->name + ": d_in " + std::to_string(m0->d_in) + " does not fit the LDS activation tile");
  // as many workgroups as fit a CU's 160 KB of LDS side by side
  const uint32_t per_cu = (uint32_t)((160 * 1024) / lds) < 1u ? 1u : (uint32_t)((160 * 1024) / lds);
  const uint32_t wg_per_cu = per_cu > (uint32_t)(2048 / kWgThreads) ? (uint32_t)(2048 / kWgThreads) : per_cu;
  const uint32_t grid_cap = (uint32_t)(rt->cu_count > 0 ? rt->cu_count : 256) * wg_per_cu;
  GroupArgs a{};
  a.tables = rt->tables;
  a.x = reinterpret_cast<const __half*>(x);
  a.x_f32 = x_f32;
  if (pro) {
    if ((size_t)m0->d_in * 2 > (size_t)tile * 6 + 32)
      return fail(LLVQ_ERR_UNSUPPORTED, m0->name + ": d_in too wide for a fused activation prologue");
    a.prologue = pro->kind;
    a.x2 = reinterpret_cast<const __half*>(pro->x2);
    a.norm_w = reinterpret_cast<const __half*>(pro->norm_w);
    a.resid_out = reinterpret_cast<__half*>(pro->resid_out);
    a.eps = pro->eps;
  }
  if (rot) {
    if (!rotation_fits(m0) || rot->n != m0->d_in)
      return fail(LLVQ_ERR_UNSUPPORTED, m0->name + ": d_in too wide for a rotation inside the launch");
    a.rot_signbits = rot->signbits;
    a.rot_small = rot->small;
    a.rot_inv = rot->inv;
    a.rot_m = rot->m;
    a.rot_k = rot->k;
  }
  a.nblocks = m0->nblocks;
  a.tail_w = m0->tail_w;
  a.n_mats = (uint32_t)n;
  a.inv_nblocks = m0->nblocks ? 1.0f / (float)m0->nblocks : 0.f;
  a.rows_per_tile = pick_rows_per_tile(mats, n, m0->nblocks, grid_cap, tile);
  uint32_t tiles = 0;
  for (int i = 0; i < n; ++i) {
    a.m[i] = MatArg{mats[i]->codes, mats[i]->rscale, mats[i]->tail, y[i], mats[i]->g[0], mats[i]->g[1],
                    mats[i]->d_out, tiles};
    tiles += (mats[i]->d_out + a.rows_per_tile - 1) / a.rows_per_tile;
  }
  a.n_tiles = tiles;
  const uint32_t grid = tiles < grid_cap ? tiles : grid_cap;
  const bool wide = m0->record_bits != 48;
  for (int i = 1; i < n; ++i)
    if (mats[i]->record_bits != m0->record_bits)
      return fail(LLVQ_ERR_INVALID_ARGUMENT, mats[i]->name + ": matrices of one launch must share their shell cap");
  if (wide && (tile != (uint32_t)kTileBlocks || rot))
    return fail(LLVQ_ERR_UNSUPPORTED, m0->name + ": rows too wide for the cap-13 kernels");
  const void* kernel = wide ? gemv_kernel_wide(y_dtype == LLVQ_F32, shape.lean) : gemv_kernel(y_dtype == LLVQ_F32, tile, shape.lean, rot != nullptr);
  void* params[] = {&a};
  HIP_TRY(hipLaunchKernel(kernel, dim3(grid), dim3(kWgThreads), params, lds, rt->stream));
  HIP_TRY(hipGetLastError());
  return LLVQ_OK;
}

// Enqueues x' = Q x for `rows` activation rows of width rot->n.
static int launch_rotate(llvq_rt* rt, const llvq_rt::DevRotation* rot, const void* x_f16, uint32_t rows, void* out,
                         bool out_f16) {
  RotArgs a{};
  a.x = reinterpret_cast<const __half*>(x_f16);
  a.out = out;
  a.signbits = rot->signbits;
  a.small = rot->small;
  a.n = rot->n;
  a.m = rot->m;
  a.k = rot->k;
  a.inv = rot->inv;
  const size_t lds = (size_t)rot->n * sizeof(float);
  if (out_f16) hipLaunchKernelGGL(rotate_kernel<__half>, dim3(rows), dim3(1024), lds, rt->stream, a);
  else hipLaunchKernelGGL(rotate_kernel<float>, dim3(rows), dim3(1024), lds, rt->stream, a);
  HIP_TRY(hipGetLastError());
  return LLVQ_OK;
}

static bool same_basis(const llvq_mat* a, const llvq_mat* b) {
  return a->record_bits == b->record_bits && a->has_rotation == b->has_rotation && (!a->has_rotation || a->rotation_seed == b->rotation_seed);
}

// One activation through projections that share it: consecutive matrices in the
// same basis go out as one launch (at most kMaxGroup).  A launch in a rotated basis
// rotates the activation itself (`pro`, when given, derives it first); rows too wide
// for that get it rotated once, into the runtime's scratch, by a kernel of its own
// (never together with `pro`: the caller stages the activation first then).
static int forward_group(llvq_rt* rt, const llvq_mat* const* mats, int n, const void* x, void* const* y, int y_dtype,
                         const Prologue* pro = nullptr) {
  int i = 0;
  while (i < n) {
    int j = i + 1;
    while (j < n && j - i < kMaxGroup && same_basis(mats[i], mats[j])) ++j;
    const float* xr = nullptr;
    if (mats[i]->has_rotation && rotation_fits(mats[i])) {
      const int rc = launch_group(rt, mats + i, j - i, x, y + i, y_dtype, pro, nullptr, mats[i]->rot);
      if (rc) return rc;
      i = j;
      continue;
    }
    if (pro && mats[i]->has_rotation) return fail(LLVQ_ERR_UNSUPPORTED, mats[i]->name + ": prologue with a rotation outside the launch");
    if (mats[i]->has_rotation) {
      // the scratch may still hold this very rotation if the previous run used it; rotating again is cheap and always right
      const int rc = launch_rotate(rt, mats[i]->rot, x, 1, rt->rot_scratch, false);
      if (rc) return rc;
      xr = rt->rot_scratch;
    }
    const int rc = launch_group(rt, mats + i, j - i, x, y + i, y_dtype, pro, xr);
    if (rc) return rc;
    i = j;
  }
  return LLVQ_OK;
}

static int launch_gemv(llvq_rt* rt, const llvq_mat* m, const void* x, void* y, int y_dtype) {
  return forward_group(rt, &m, 1, x, &y, y_dtype);
}

int llvq_hip_gemv(llvq_rt* rt, const llvq_mat* m, const void* x, void* y, int y_dtype) {
  if (!rt || !m || !x || !y) return fail(LLVQ_ERR_INVALID_ARGUMENT, "gemv: null argument");
  HIP_TRY(hipSetDevice(rt->device));
  return launch_gemv(rt, m, x, y, y_dtype);
}

int llvq_hip_rotate(llvq_rt* rt, const llvq_mat* m, const void* x_f16_dev, float* xr_f32_dev) {
  if (!rt || !m || !x_f16_dev || !xr_f32_dev) return fail(LLVQ_ERR_INVALID_ARGUMENT, "rotate: null argument");
  HIP_TRY(hipSetDevice(rt->device));
  if (m->has_rotation) return launch_rotate(rt, m->rot, x_f16_dev, 1, xr_f32_dev, false);
  hipLaunchKernelGGL(widen_kernel, dim3((m->d_in + 255) / 256), dim3(256), 0, rt->stream,
                     reinterpret_cast<const __half*>(x_f16_dev), xr_f32_dev, m->d_in);
  HIP_TRY(hipGetLastError());
  return LLVQ_OK;
}

int llvq_hip_gemv_rotated(llvq_rt* rt, const llvq_mat* m, const float* xr_f32_dev, void* y, int y_dtype) {
  if (!rt || !m || !xr_f32_dev || !y) return fail(LLVQ_ERR_INVALID_ARGUMENT, "gemv_rotated: null argument");
  HIP_TRY(hipSetDevice(rt->device));
  return launch_group(rt, &m, 1, nullptr, &y, y_dtype, nullptr, xr_f32_dev);
}

int llvq_hip_host_rotate(uint32_t n, uint64_t seed, double* v) {
  if (!v) return fail(LLVQ_ERR_INVALID_ARGUMENT, "host_rotate: null vector");
  RotationTables t;
  std::string err;
  if (!build_rotation(n, seed, &t, &err)) return fail(LLVQ_ERR_UNSUPPORTED, err);
  std::vector<double> w(v, v + n);
  host_rotate(t, &w);
  std::memcpy(v, w.data(), (size_t)n * sizeof(double));
  return LLVQ_OK;
}

int llvq_hip_matrix_rotation(const llvq_mat* m, uint32_t* has_rotation, uint64_t* seed) {
  if (!m) return fail(LLVQ_ERR_INVALID_ARGUMENT, "matrix_rotation: matrix is null");
  if (has_rotation) *has_rotation = m->has_rotation ? 1u : 0u;
  if (seed) *seed = m->rotation_seed;
  return LLVQ_OK;
}

int llvq_hip_gemv_group(llvq_rt* rt, const llvq_mat* const* mats, int n, const void* x,
                        void* const* y, int y_dtype) {
  if (!rt || !mats || !x || !y || n < 0) return fail(LLVQ_ERR_INVALID_ARGUMENT, "gemv_group: bad argument");
  for (int i = 0; i < n; ++i) {
    if (!mats[i] || !y[i]) return fail(LLVQ_ERR_INVALID_ARGUMENT, "gemv_group: null matrix or output");
    if (mats[i]->d_in != mats[0]->d_in)
      return fail(LLVQ_ERR_INVALID_ARGUMENT, mats[i]->name + ": projections of one group must share d_in");
  }
  HIP_TRY(hipSetDevice(rt->device));
  return forward_group(rt, mats, n, x, y, y_dtype);
}

// ---- sequences of group products in one launch (gemv_seq.h) -------------------------------
// One item of a sequence as the library's own callers state it: what a launch_group call takes.
struct SeqSpec {
  const llvq_mat* const* mats = nullptr;
  int n = 0;
  const void* x = nullptr;
  void* const* y = nullptr;
  int y_dtype = LLVQ_F16;
  bool after_previous = false;
  Prologue pro{};
};

// three byte planes of the activation for f32 results, two for binary16 results, as gemv_tiles_kernel
static const void* seq_kernel(uint32_t tile, bool lean, bool f32, bool wide) {
  if (wide) {  // cap-13 matrices: full tiles only
    if (f32) return lean ? reinterpret_cast<const void*>(gemv_seq_kernel<kTileBlocks, true, 3, true>) : reinterpret_cast<const void*>(gemv_seq_kernel<kTileBlocks, false, 3, true>);
    return lean ? reinterpret_cast<const void*>(gemv_seq_kernel<kTileBlocks, true, 2, true>) : reinterpret_cast<const void*>(gemv_seq_kernel<kTileBlocks, false, 2, true>);
  }
  if (f32) {
    if (lean) return reinterpret_cast<const void*>(gemv_seq_kernel<kTileBlocks, true, 3>);
    if (tile == (uint32_t)kTileBlocks) return reinterpret_cast<const void*>(gemv_seq_kernel<kTileBlocks, false, 3>);
    return reinterpret_cast<const void*>(gemv_seq_kernel<kSmallTileBlocks, false, 3>);
  }
  if (lean) return reinterpret_cast<const void*>(gemv_seq_kernel<kTileBlocks, true, 2>);
  if (tile == (uint32_t)kTileBlocks) return reinterpret_cast<const void*>(gemv_seq_kernel<kTileBlocks, false, 2>);
  return reinterpret_cast<const void*>(gemv_seq_kernel<kSmallTileBlocks, false, 2>);
}

// The kernel variant for a sequence whose widest rows have max_nb blocks (as pick_gemv_shape).
static GemvShape pick_seq_shape(uint32_t max_nb) {
  GemvShape s{(uint32_t)kTileBlocks, false, gemv_seq_lds_bytes(max_nb, kTileBlocks, kLdsImageBytes)};
  if (s.lds <= 160 * 1024) return s;
  s = GemvShape{(uint32_t)kTileBlocks, true, gemv_seq_lds_bytes(max_nb, kTileBlocks, kLdsImageBytesLean)};
  if (s.lds <= 160 * 1024) return s;
  return GemvShape{(uint32_t)kSmallTileBlocks, false, gemv_seq_lds_bytes(max_nb, kSmallTileBlocks, kLdsImageBytes)};
}

constexpr uint32_t kSeqSpinLimit = 1u << 20;  // polls of a wait before it gives up (about a second)

static int seq_create(llvq_rt* rt, const SeqSpec* specs, int n, llvq_seq** out) {
  if (n <= 0) return fail(LLVQ_ERR_INVALID_ARGUMENT, "sequence_create: no items");
  uint32_t max_nb = 0;
  bool dependent = false;
  for (int i = 0; i < n; ++i) {
    const SeqSpec& sp = specs[i];
    if (!sp.mats || sp.n <= 0 || !sp.x || !sp.y) return fail(LLVQ_ERR_INVALID_ARGUMENT, "sequence_create: item " + std::to_string(i) + " has a null or empty field");
    if (sp.y_dtype != LLVQ_F32 && sp.y_dtype != LLVQ_F16) return fail(LLVQ_ERR_INVALID_ARGUMENT, "sequence_create: unknown output dtype");
    if (sp.after_previous && i == 0) return fail(LLVQ_ERR_INVALID_ARGUMENT, "sequence_create: the first item has no item before it");
    if (sp.y_dtype != specs[0].y_dtype) return fail(LLVQ_ERR_INVALID_ARGUMENT, "sequence_create: the items of a sequence share one output dtype");
    for (int j = 0; j < sp.n; ++j) {
      const llvq_mat* m = sp.mats[j];
      if (!m || !sp.y[j]) return fail(LLVQ_ERR_INVALID_ARGUMENT, "sequence_create: null matrix or output in item " + std::to_string(i));
      if (m->d_in != sp.mats[0]->d_in) return fail(LLVQ_ERR_INVALID_ARGUMENT, m->name + ": projections of one item must share d_in");
      if (m->has_rotation) return fail(LLVQ_ERR_UNSUPPORTED, m->name + ": a sequence takes natural-basis matrices only");
      if (m->record_bits != specs[0].mats[0]->record_bits) return fail(LLVQ_ERR_UNSUPPORTED, m->name + ": the matrices of a sequence share one shell cap");
    }
    if (sp.mats[0]->nblocks > 1024u) return fail(LLVQ_ERR_UNSUPPORTED, sp.mats[0]->name + ": rows wider than 24 576 columns do not fit a sequence");
    max_nb = std::max(max_nb, sp.mats[0]->nblocks);
    dependent |= sp.after_previous;
  }
  const GemvShape shape = pick_seq_shape(max_nb);
  if (shape.lds > 160 * 1024 || max_nb > shape.tile) return fail(LLVQ_ERR_UNSUPPORTED, "sequence_create: the widest rows do not fit the LDS activation tile");
  const bool wide = specs[0].mats[0]->record_bits != 48;
  if (wide && shape.tile != (uint32_t)kTileBlocks) return fail(LLVQ_ERR_UNSUPPORTED, "sequence_create: rows this wide do not fit a sequence of cap-13 matrices");
  for (int i = 0; i < n; ++i)
    if (specs[i].pro.kind == kPrologueAddRmsNorm && specs[i].mats[0]->d_in > 6u * kWgThreads)
      return fail(LLVQ_ERR_UNSUPPORTED, specs[i].mats[0]->name + ": d_in too wide for a fused norm inside a sequence");
  const uint32_t grid_cap = (uint32_t)(rt->cu_count > 0 ? rt->cu_count : 256);
  std::vector<SeqTile> tiles;
  std::vector<SeqItem> items((size_t)n);
  for (int i = 0; i < n; ++i) {
    const SeqSpec& sp = specs[i];
    const llvq_mat* m0 = sp.mats[0];
    const uint32_t nb = m0->nblocks;
    // Ordered items, and an item that is a launch by itself, are balanced one by one, like launches (everyone waits
    // for an item's slowest workgroup); independent items fill their tiles, because the round-robin runs on across
    // item boundaries.
    uint32_t rpt = (dependent || n == 1) ? pick_rows_per_tile(sp.mats, sp.n, nb, grid_cap, shape.tile) : (nb ? std::max(1u, shape.tile / nb) : 256u);
    SeqItem& I = items[(size_t)i];
    std::memset(&I, 0, sizeof I);
    I.x = reinterpret_cast<const __half*>(sp.x);
    I.x2 = reinterpret_cast<const __half*>(sp.pro.x2);
    I.norm_w = reinterpret_cast<const __half*>(sp.pro.norm_w);
    I.resid_out = reinterpret_cast<__half*>(sp.pro.resid_out);
    I.eps = sp.pro.eps;
    I.prologue = sp.pro.kind;
    I.nb = nb;
    I.tail_w = m0->tail_w;
    I.inv_nb = nb ? 1.0f / (float)nb : 0.f;
    I.y_f16 = sp.y_dtype == LLVQ_F16 ? 1u : 0u;
    I.first_tile = (uint32_t)tiles.size();
    I.wait_item = sp.after_previous ? (uint32_t)(i - 1) : kSeqNoWait;
    I.signals = (i + 1 < n && specs[i + 1].after_previous) ? 1u : 0u;
    const size_t ysz = sp.y_dtype == LLVQ_F16 ? 2 : 4;
    for (int j = 0; j < sp.n; ++j) {
      const llvq_mat* m = sp.mats[j];
      for (uint32_t r0 = 0; r0 < m->d_out; r0 += rpt) {
        SeqTile t{};
        t.rows = std::min(rpt, m->d_out - r0);
        t.nblk = t.rows * nb;
        const uint64_t first_bit = (uint64_t)r0 * nb * m->record_bits;  // 6-byte records begin on a byte; dense 49-bit blocks need not
        t.codes = m->codes + (first_bit >> 3);
        t.bit0 = (uint32_t)(first_bit & 7u);
        t.rscale = m->rscale + r0;
        t.tail = m->tail + (size_t)r0 * m->tail_w;
        t.y = reinterpret_cast<uint8_t*>(sp.y[j]) + (size_t)r0 * ysz;
        t.g0 = m->g[0];
        t.g1 = m->g[1];
        t.item = (uint32_t)i;
        tiles.push_back(t);
      }
    }
  }
  if (tiles.size() > 0x7FFFFFFFu) return fail(LLVQ_ERR_UNSUPPORTED, "sequence_create: too many tiles");
  const uint32_t n_tiles = (uint32_t)tiles.size();
  const uint32_t grid = std::min(n_tiles, grid_cap);
  for (int i = 0; i < n; ++i) {
    const uint32_t t0 = items[(size_t)i].first_tile, t1 = i + 1 < n ? items[(size_t)i + 1].first_tile : n_tiles;
    items[(size_t)i].expected = std::min(t1 - t0, grid);
  }
  for (int i = 0; i < n; ++i)
    if (items[(size_t)i].wait_item != kSeqNoWait) items[(size_t)i].wait_expected = items[items[(size_t)i].wait_item].expected;
  HIP_TRY(hipSetDevice(rt->device));
  auto* q = new llvq_seq();
  const size_t off_items = tiles.size() * sizeof(SeqTile);
  const size_t off_counters = (off_items + items.size() * sizeof(SeqItem) + 255) & ~(size_t)255;
  const size_t off_status = off_counters + (((size_t)n * 4 + 255) & ~(size_t)255);
  const size_t total = off_status + 256;
  hipError_t e = hipMalloc(reinterpret_cast<void**>(&q->blob), total);
  if (e == hipSuccess) e = hipMemset(q->blob, 0, total);
  if (e == hipSuccess) e = hipMemcpy(q->blob, tiles.data(), off_items, hipMemcpyHostToDevice);
  if (e == hipSuccess) e = hipMemcpy(q->blob + off_items, items.data(), items.size() * sizeof(SeqItem), hipMemcpyHostToDevice);
  if (e != hipSuccess) {
    (void)hipFree(q->blob);
    delete q;
    return hip_fail(e, "sequence tables");
  }
  q->args.tables = rt->tables;
  q->args.tiles = reinterpret_cast<const SeqTile*>(q->blob);
  q->args.items = reinterpret_cast<const SeqItem*>(q->blob + off_items);
  q->args.n_tiles = n_tiles;
  q->args.max_nb = max_nb;
  q->args.counters = reinterpret_cast<uint32_t*>(q->blob + off_counters);
  q->args.status = reinterpret_cast<uint32_t*>(q->blob + off_status);
  q->own_status = q->args.status;
  q->args.run = 0;
  q->args.spin_limit = kSeqSpinLimit;
  q->args.hold_item = kSeqNoWait;
  q->args.stamps = nullptr;
  q->args.item0 = items[0];
  q->tile = shape.tile;
  q->lean = shape.lean;
  q->f32 = specs[0].y_dtype == LLVQ_F32;
  q->wide = wide;
  // the activation planes of a wide row push dynamic LDS past the 64 KB default
  (void)hipFuncSetAttribute(seq_kernel(shape.tile, shape.lean, q->f32, q->wide), hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
  q->lds = shape.lds;
  q->grid = grid;
  q->n_items = (uint32_t)n;
  *out = q;
  return LLVQ_OK;
}

static int seq_run(llvq_rt* rt, llvq_seq* q) {
  q->args.run += 1;
  SeqArgs a = q->args;
  void* params[] = {&a};
  const void* kernel = seq_kernel(q->tile, q->lean, q->f32, q->wide);
  // An ordinary launch, also with ordered items: at most one workgroup per CU (by its LDS) and no more workgroups than
  // CUs, so on a device this stream has to itself every workgroup is resident and the waits end.  (A cooperative launch
  // would guarantee it, but costs some 200 us per launch here: 4B decode fell from 237 to 85 tokens/s with it.)  Should
  // another queue hold CUs for longer than the bounded wait, the run gives up and says so; it cannot hang.
  HIP_TRY(hipLaunchKernel(kernel, dim3(q->grid), dim3(kWgThreads), params, q->lds, rt->stream));
  HIP_TRY(hipGetLastError());
  q->args.hold_item = kSeqNoWait;
  return LLVQ_OK;
}

// After a run that gave up: its counters are short, so the next run starts over from zero.
static int seq_reset(llvq_seq* q) {
  HIP_TRY(hipMemset(q->args.counters, 0, (size_t)q->n_items * 4));
  HIP_TRY(hipMemset(q->args.status, 0, 4));
  q->args.run = 0;
  return LLVQ_OK;
}

int llvq_hip_sequence_create(llvq_rt* rt, const llvq_seq_item* items, int n_items, llvq_seq** out) {
  if (!rt || !items || !out || n_items <= 0) return fail(LLVQ_ERR_INVALID_ARGUMENT, "sequence_create: bad argument");
  *out = nullptr;
  std::vector<SeqSpec> specs((size_t)n_items);
  for (int i = 0; i < n_items; ++i) {
    specs[(size_t)i].mats = items[i].mats;
    specs[(size_t)i].n = items[i].n_mats;
    specs[(size_t)i].x = items[i].x_f16_dev;
    specs[(size_t)i].y = items[i].y_dev;
    specs[(size_t)i].y_dtype = items[i].y_dtype;
    specs[(size_t)i].after_previous = items[i].after_previous != 0;
  }
  return seq_create(rt, specs.data(), n_items, out);
}

int llvq_hip_sequence_run(llvq_rt* rt, llvq_seq* seq) {
  if (!rt || !seq) return fail(LLVQ_ERR_INVALID_ARGUMENT, "sequence_run: null argument");
  HIP_TRY(hipSetDevice(rt->device));
  return seq_run(rt, seq);
}

int llvq_hip_sequence_status(llvq_rt* rt, llvq_seq* seq) {
  if (!rt || !seq) return fail(LLVQ_ERR_INVALID_ARGUMENT, "sequence_status: null argument");
  HIP_TRY(hipSetDevice(rt->device));
  HIP_TRY(hipStreamSynchronize(rt->stream));
  uint32_t st = 0;
  HIP_TRY(hipMemcpy(&st, seq->args.status, sizeof st, hipMemcpyDeviceToHost));
  if (!st) return LLVQ_OK;
  // the counters of a run that gave up are short: start over from zero
  const int rc = seq_reset(seq);
  if (rc) return rc;
  return fail(LLVQ_ERR_DEVICE, "sequence: a workgroup gave up waiting for an item; the run's outputs are incomplete");
}

#ifdef LLVQ_SEQ_STAMPS
// Tuning builds only: where the next runs of `seq` store their phase timestamps (device memory of
// grid x kSeqStampTiles x 8 64-bit words, or null).
extern "C" int llvq_hip_sequence_debug(llvq_seq* seq, void* stamps_dev, uint32_t* grid) {
  seq->args.stamps = reinterpret_cast<unsigned long long*>(stamps_dev);
  if (grid) *grid = seq->grid;
  return LLVQ_OK;
}
#endif

int llvq_hip_sequence_tune(llvq_seq* seq, uint32_t spin_limit, int hold_item) {
  if (!seq) return fail(LLVQ_ERR_INVALID_ARGUMENT, "sequence_tune: null sequence");
  if (hold_item >= (int)seq->n_items) return fail(LLVQ_ERR_INVALID_ARGUMENT, "sequence_tune: no such item");
  seq->args.spin_limit = spin_limit ? spin_limit : kSeqSpinLimit;
  seq->args.hold_item = hold_item >= 0 ? (uint32_t)hold_item : kSeqNoWait;
  return LLVQ_OK;
}

void llvq_hip_sequence_destroy(llvq_rt* rt, llvq_seq* seq) {
  if (!seq) return;
  if (rt) {
    (void)hipSetDevice(rt->device);
    (void)hipStreamSynchronize(rt->stream);
  }
  (void)hipFree(seq->blob);
  delete seq;
}

// Grows a device buffer of the runtime to `need` bytes (contents are not kept).
static int grow_buffer(void** buf, size_t* have, size_t need) {
  if (need <= *have) return LLVQ_OK;
  (void)hipFree(*buf);  // waits for launches that still use it
  *buf = nullptr;
  *have = 0;
  HIP_TRY(hipMalloc(buf, need));
  *have = need;
  return LLVQ_OK;
}

// Batches of up to this many activation rows leave the matrix cores little to do:
// twelve of the sixteen wavefronts unrank and four multiply (four consumers cover 256 rows).
constexpr uint32_t kGemmNarrowRows = 256;

// Where a batched call's device workspaces come from: the runtime's buffers, grown with
// hipMalloc on first use of a larger shape, or (fixed != null) a region the caller of this
// file's helpers provides, which is carved up and never outgrown.
struct GemmWorkspace {
  uint8_t* fixed = nullptr;
  size_t fixed_bytes = 0, used = 0;
};
static int workspace_take(llvq_rt* rt, GemmWorkspace* w, void** runtime_buf, size_t* runtime_have, size_t need, void** out) {
  if (!w || !w->fixed) {
    const int rc = grow_buffer(runtime_buf, runtime_have, need);
    *out = *runtime_buf;
    return rc;
  }
  const size_t at = (w->used + 255) & ~(size_t)255;
  if (need > w->fixed_bytes || at > w->fixed_bytes - need)
    return fail(LLVQ_ERR_UNSUPPORTED, "gemm_static: this shape needs " + std::to_string(at + need) +
                                          " bytes of workspace, the static one holds " + std::to_string(w->fixed_bytes));
  *out = w->fixed + at;
  w->used = at + need;
  return LLVQ_OK;
}

// Workspace bytes of one batched launch (launch_gemm) over these matrices at M rows: the partial
// sums and the K-step-tiled copy of the activations.
static void gemm_workspace_bytes(const llvq_rt* rt, const llvq_mat* const* mats, int n, uint32_t M, size_t* ws_bytes, size_t* xt_bytes) {
  const uint32_t grid_cap = (uint32_t)(rt->cu_count > 0 ? rt->cu_count : 256);
  const llvq_mat* m0 = mats[0];
  uint32_t n_bands = 0;
  for (int i = 0; i < n; ++i) n_bands += (mats[i]->d_out + kGemmRows - 1) / kGemmRows;
  const uint32_t consumers = M <= kGemmNarrowRows ? 4u : 8u;
  uint32_t ct_shift = 0;
  while (((uint32_t)kGemmColTile << ct_shift) < M) ++ct_shift;
  const uint32_t kparts = consumers >> ct_shift;
  const uint32_t spb = (m0->nblocks + kGemmKb - 1) / kGemmKb;
  const GemmShare share = gemm_share(n_bands ? n_bands : 1, spb ? spb : 1, grid_cap);
  // bands walked by one workgroup alone are finished in the launch when every consumer owns its tile's every K-step
  const uint32_t ws_band0 = kparts == 1 ? share.shared0 : 0u;
  const uint32_t m_pad = (M + kGemmColTile - 1) / kGemmColTile * kGemmColTile;
  const uint32_t n_steps = spb * (kGemmKb * 24 / 32);
  *ws_bytes = (size_t)(n_bands - (ws_band0 < n_bands ? ws_band0 : n_bands)) * share.max_pieces * kparts * M * kGemmRows * sizeof(float);
  *xt_bytes = (size_t)n_steps * m_pad * 64;
}

// Sizes the runtime's batched-path buffers for calls over these matrices (grouped as
// llvq_hip_gemm_group groups them) at up to max_rows activation rows, so that those calls find
// them large enough and allocate nothing.
static int reserve_batched(llvq_rt* rt, const llvq_mat* const* mats, int n, uint32_t max_rows) {
  if (n <= 0 || max_rows < 2) return LLVQ_OK;
  size_t ws = 0, xt = 0, rows = 0;
  const uint32_t chunk = max_rows < (uint32_t)kGemmMaxM ? max_rows : (uint32_t)kGemmMaxM;
  for (int i0 = 0; i0 < n;) {
    int i1 = i0 + 1;
    while (i1 < n && i1 - i0 < kGemmMaxGroup && mats[i1]->has_rotation == mats[i0]->has_rotation &&
           (!mats[i0]->has_rotation || mats[i1]->rot == mats[i0]->rot))
      ++i1;
    bool six_byte = true;
    for (int i = i0; i < i1; ++i) six_byte &= mats[i]->record_bits == 48;
    if (mats[i0]->nblocks && six_byte) {  // (cap-13 matrices take the row loop, which has no workspace)
      // every row count up to the chunk: the partial-sum layout is not monotone in M where the consumers' split changes
      for (uint32_t M : {chunk, (uint32_t)64, (uint32_t)128, (uint32_t)256}) {
        if (M > chunk) continue;
        size_t w = 0, x = 0;
        gemm_workspace_bytes(rt, mats + i0, i1 - i0, M, &w, &x);
        ws = w > ws ? w : ws;
        xt = x > xt ? x : xt;
      }
    }
    if (mats[i0]->has_rotation) {
      const size_t r = (size_t)max_rows * mats[i0]->d_in * sizeof(__half);
      rows = r > rows ? r : rows;
    }
    i0 = i1;
  }
  int rc = grow_buffer(reinterpret_cast<void**>(&rt->gemm_ws), &rt->gemm_ws_bytes, ws);
  if (!rc) rc = grow_buffer(reinterpret_cast<void**>(&rt->gemm_xt), &rt->gemm_xt_bytes, xt);
  if (!rc) rc = grow_buffer(reinterpret_cast<void**>(&rt->rot_rows), &rt->rot_rows_bytes, rows);
  return rc;
}

// One launch over n <= kGemmMaxGroup matrices of equal d_in that take the same activations
// (already in the matrices' basis), M <= kGemmMaxM rows.
static int launch_gemm(llvq_rt* rt, const llvq_mat* const* mats, int n, const void* x, uint32_t M, void* const* y,
                       int y_dtype, GemmWorkspace* wsp = nullptr) {
  const uint32_t grid_cap = (uint32_t)(rt->cu_count > 0 ? rt->cu_count : 256);
  const bool f32 = y_dtype == LLVQ_F32;
  const llvq_mat* m0 = mats[0];
  const __half* xh = reinterpret_cast<const __half*>(x);
  GemmArgs a{};
  GemmReduceArgs r{};
  a.tables = rt->tables;
  a.n_mats = r.n_mats = (uint32_t)n;
  for (int i = 0; i < n; ++i) {
    a.mat[i] = GemmMat{mats[i]->codes, mats[i]->rscale, mats[i]->tail, y[i], mats[i]->g[0], mats[i]->g[1], mats[i]->d_out, a.n_bands};
    r.mat[i] = GemmReduceMat{mats[i]->rscale, mats[i]->tail, y[i], mats[i]->d_out, a.n_bands};
    a.n_bands += (mats[i]->d_out + kGemmRows - 1) / kGemmRows;
  }
  a.y_f32 = f32 ? 1u : 0u;
  a.x = xh;
  a.ldx = m0->d_in;
  a.tail_w = m0->tail_w;
  a.M = M;
  a.m_pad = (M + kGemmColTile - 1) / kGemmColTile * kGemmColTile;
  a.nblocks = m0->nblocks;
  // the consumer wavefronts over the batch's 64-row tiles, the count rounded up to a power of two
  const uint32_t consumers = M <= kGemmNarrowRows ? 4u : 8u;
  a.ct_shift = 0;
  while (((uint32_t)kGemmColTile << a.ct_shift) < M) ++a.ct_shift;
  const uint32_t kparts = consumers >> a.ct_shift;
  // The launch's slices, band by band, are shared out evenly over the workgroups (one per CU): a
  // band whose slices fall to several of them leaves one partial sum per workgroup.
  a.spb = (m0->nblocks + kGemmKb - 1) / kGemmKb;
  const uint64_t total = (uint64_t)a.n_bands * a.spb;
  if (total > 0xFFFFFFFFull) return fail(LLVQ_ERR_UNSUPPORTED, m0->name + ": too many K-slices for one batched launch");
  const GemmShare share = gemm_share(a.n_bands, a.spb, grid_cap);
  if (!gemm_share_exact(share, a.n_bands, a.spb)) return fail(LLVQ_ERR_UNSUPPORTED, m0->name + ": rows too wide for the batched launch's slice arithmetic");
  const uint32_t n_wg = share.n_wg;
  a.share = share;
  a.ws_band0 = kparts == 1 ? share.shared0 : 0u;
  const uint32_t ws_bands = a.n_bands - a.ws_band0;  // bands with partial sums in the workspace
  void* ws_buf = nullptr;
  void* xt_buf = nullptr;
  const size_t mark = wsp ? wsp->used : 0;  // a launch's carvings are released when it has been enqueued: the stream orders the next
  size_t ws_bytes = 0, xt_bytes = 0;
  gemm_workspace_bytes(rt, mats, n, M, &ws_bytes, &xt_bytes);
  if (ws_bytes != (size_t)ws_bands * share.max_pieces * kparts * M * kGemmRows * sizeof(float))
    return fail(LLVQ_ERR_DEVICE, "gemm: workspace sizing disagrees with the launch");
  int rc = LLVQ_OK;
  if (ws_bytes) rc = workspace_take(rt, wsp, reinterpret_cast<void**>(&rt->gemm_ws), &rt->gemm_ws_bytes, ws_bytes, &ws_buf);
  if (rc) return rc;
  // every slice has all its twelve K-steps in the tiled copy, zeros past the matrix's last block
  const uint32_t n_steps = (m0->nblocks + kGemmKb - 1) / kGemmKb * (kGemmKb * 24 / 32);
  if (xt_bytes != (size_t)n_steps * a.m_pad * 64) return fail(LLVQ_ERR_DEVICE, "gemm: activation-copy sizing disagrees with the launch");
  // the kernel reads the copy through a buffer descriptor: 32-bit offsets
  if (xt_bytes >= (1ull << 32)) return fail(LLVQ_ERR_UNSUPPORTED, m0->name + ": rows too wide for the batched launch's 32-bit activation offsets");
  rc = workspace_take(rt, wsp, reinterpret_cast<void**>(&rt->gemm_xt), &rt->gemm_xt_bytes, xt_bytes, &xt_buf);
  if (rc) return rc;
  if (wsp) wsp->used = mark;
  hipLaunchKernelGGL(tile_activations_kernel, dim3((uint32_t)((xt_bytes / 16 + 255) / 256)), dim3(256), 0, rt->stream, xh, M,
                     m0->d_in, m0->nblocks * 24u, a.m_pad, n_steps, reinterpret_cast<uint4*>(xt_buf));
  HIP_TRY(hipGetLastError());
  a.xt = reinterpret_cast<__half*>(xt_buf);
  a.ws = reinterpret_cast<float*>(ws_buf);
  const dim3 grid(n_wg), wg(kWgThreads);
  if (consumers == 4) hipLaunchKernelGGL(gemm_tiles_kernel<12>, grid, wg, gemm_lds_bytes(), rt->stream, a);
  else hipLaunchKernelGGL(gemm_tiles_kernel<8>, grid, wg, gemm_lds_bytes(), rt->stream, a);
  HIP_TRY(hipGetLastError());
  r.ws = a.ws;
  r.x = xh;
  r.M = M;
  r.ldx = m0->d_in;
  r.nblocks = m0->nblocks;
  r.tail_w = m0->tail_w;
  r.n_bands = a.n_bands;
  r.spb = a.spb;
  r.share = share;
  r.ws_band0 = a.ws_band0;
  r.kparts = kparts;
  if (ws_bands == 0) return LLVQ_OK;  // every band was finished by the workgroup that walked it
  const uint32_t rgrid = ws_bands * ((M + kReduceRowsM - 1) / kReduceRowsM);
  if (f32) hipLaunchKernelGGL(gemm_reduce_kernel<float>, dim3(rgrid), dim3(256), 0, rt->stream, r);
  else hipLaunchKernelGGL(gemm_reduce_kernel<__half>, dim3(rgrid), dim3(256), 0, rt->stream, r);
  HIP_TRY(hipGetLastError());
  return LLVQ_OK;
}

// Matrices [0, n) of one group: same d_in, same basis.  The matrix-core kernel reads activations as
// 16-byte vectors; a single row, or a shape that breaks that alignment, runs as GEMV launches instead.
static int gemm_same_basis(llvq_rt* rt, const llvq_mat* const* mats, int n, const void* x, int M, void* const* y, int y_dtype,
                           GemmWorkspace* wsp = nullptr) {
  const llvq_mat* m0 = mats[0];
  const size_t esz = y_dtype == LLVQ_F32 ? 4 : 2;
  const uint8_t* xb = reinterpret_cast<const uint8_t*>(x);
  bool six_byte = true;  // the matrix-core kernel's producers read 6-byte records: cap-13 matrices take the row loop
  for (int i = 0; i < n; ++i) six_byte &= mats[i]->record_bits == 48;
  const bool mfma_ok = M >= 2 && m0->d_in % 8 == 0 && (reinterpret_cast<uintptr_t>(x) & 15) == 0 && m0->nblocks > 0 && six_byte;
  if (!mfma_ok) {
    for (int i = 0; i < n; ++i)
      for (int r = 0; r < M; ++r) {
        const int rc = launch_gemv(rt, mats[i], xb + (size_t)r * m0->d_in * 2, reinterpret_cast<uint8_t*>(y[i]) + (size_t)r * mats[i]->d_out * esz, y_dtype);
        if (rc) return rc;
      }
    return LLVQ_OK;
  }
  if (wsp && wsp->fixed) {
    // a caller-provided region is never outgrown part-way: every launch's carvings (released once it is enqueued)
    // are sized before the first launch, since a short last chunk can need more than a full one, and a call
    // that does not fit is refused whole
    auto after = [](size_t used, size_t bytes) { return ((used + 255) & ~(size_t)255) + bytes; };
    const size_t base = m0->has_rotation ? after(wsp->used, (size_t)M * m0->d_in * sizeof(__half)) : wsp->used;
    size_t need = base;
    for (int m_lo = 0; m_lo < M; m_lo += kGemmMaxM) {
      const uint32_t mc = (uint32_t)(M - m_lo < kGemmMaxM ? M - m_lo : kGemmMaxM);
      for (int i0 = 0; i0 < n; i0 += kGemmMaxGroup) {
        size_t ws = 0, xt = 0;
        gemm_workspace_bytes(rt, mats + i0, n - i0 < kGemmMaxGroup ? n - i0 : kGemmMaxGroup, mc, &ws, &xt);
        const size_t top = after(ws ? after(base, ws) : base, xt);
        if (top > need) need = top;
      }
    }
    if (need > wsp->fixed_bytes)
      return fail(LLVQ_ERR_UNSUPPORTED, "gemm_static: this shape needs " + std::to_string(need) +
                                            " bytes of workspace, the static one holds " + std::to_string(wsp->fixed_bytes));
  }
  if (m0->has_rotation) {
    // rows are rotated (f32 inside) and narrowed to the binary16 the matrix cores take
    void* rows = nullptr;
    const int rc0 = workspace_take(rt, wsp, reinterpret_cast<void**>(&rt->rot_rows), &rt->rot_rows_bytes,
                                   (size_t)M * m0->d_in * sizeof(__half), &rows);
    if (rc0) return rc0;
    const int rc = launch_rotate(rt, m0->rot, x, (uint32_t)M, rows, true);
    if (rc) return rc;
    xb = reinterpret_cast<const uint8_t*>(rows);
  }
  for (int m_lo = 0; m_lo < M; m_lo += kGemmMaxM) {
    const uint32_t mc = (uint32_t)(M - m_lo < kGemmMaxM ? M - m_lo : kGemmMaxM);
    for (int i0 = 0; i0 < n; i0 += kGemmMaxGroup) {
      const int cnt = n - i0 < kGemmMaxGroup ? n - i0 : kGemmMaxGroup;
      void* ys[kGemmMaxGroup];
      for (int i = 0; i < cnt; ++i) ys[i] = reinterpret_cast<uint8_t*>(y[i0 + i]) + (size_t)m_lo * mats[i0 + i]->d_out * esz;
      const int rc = launch_gemm(rt, mats + i0, cnt, xb + (size_t)m_lo * m0->d_in * 2, mc, ys, y_dtype, wsp);
      if (rc) return rc;
    }
  }
  return LLVQ_OK;
}

int llvq_hip_gemm_group(llvq_rt* rt, const llvq_mat* const* mats, int n, const void* x, int M, void* const* y, int y_dtype) {
  if (!rt || !mats || !y || n < 0 || M < 0) return fail(LLVQ_ERR_INVALID_ARGUMENT, "gemm_group: bad argument");
  if (y_dtype != LLVQ_F32 && y_dtype != LLVQ_F16) return fail(LLVQ_ERR_INVALID_ARGUMENT, "gemm_group: unknown output dtype");
  for (int i = 0; i < n; ++i) {
    if (!mats[i]) return fail(LLVQ_ERR_INVALID_ARGUMENT, "gemm_group: null matrix");
    if (mats[i]->d_in != mats[0]->d_in)
      return fail(LLVQ_ERR_INVALID_ARGUMENT, mats[i]->name + ": projections of one group must share d_in");
  }
  if (M == 0 || n == 0) return LLVQ_OK;  // no rows: nothing is read or written, so the pointers may be null
  if (!x) return fail(LLVQ_ERR_INVALID_ARGUMENT, "gemm_group: null activation");
  for (int i = 0; i < n; ++i)
    if (!y[i]) return fail(LLVQ_ERR_INVALID_ARGUMENT, "gemm_group: null output");
  HIP_TRY(hipSetDevice(rt->device));
  // consecutive matrices that share a basis go into one launch; the activation is rotated once per basis
  for (int i0 = 0; i0 < n;) {
    int i1 = i0 + 1;
    while (i1 < n && mats[i1]->has_rotation == mats[i0]->has_rotation && (!mats[i0]->has_rotation || mats[i1]->rot == mats[i0]->rot)) ++i1;
    const int rc = gemm_same_basis(rt, mats + i0, i1 - i0, x, M, y + i0, y_dtype);
    if (rc) return rc;
    i0 = i1;
  }
  return LLVQ_OK;
}

int llvq_hip_gemm(llvq_rt* rt, const llvq_mat* m, const void* x, int M, void* y, int y_dtype) {
  if (!rt || !m || M < 0) return fail(LLVQ_ERR_INVALID_ARGUMENT, "gemm: bad argument");
  if (M == 0) return LLVQ_OK;  // no rows: nothing is read or written, so the pointers may be null
  if (!x || !y) return fail(LLVQ_ERR_INVALID_ARGUMENT, "gemm: null activation or output");
  return llvq_hip_gemm_group(rt, &m, 1, x, M, &y, y_dtype);
}

int llvq_hip_reserve_batched(llvq_rt* rt, const llvq_mat* const* mats, int n, int max_rows) {
  if (!rt || !mats || n < 0 || max_rows < 0) return fail(LLVQ_ERR_INVALID_ARGUMENT, "reserve_batched: bad argument");
  for (int i = 0; i < n; ++i) {
    if (!mats[i]) return fail(LLVQ_ERR_INVALID_ARGUMENT, "reserve_batched: null matrix");
    if (mats[i]->d_in != mats[0]->d_in)
      return fail(LLVQ_ERR_INVALID_ARGUMENT, mats[i]->name + ": projections of one group must share d_in");
  }
  HIP_TRY(hipSetDevice(rt->device));
  return reserve_batched(rt, mats, n, (uint32_t)max_rows);
}

int llvq_hip_gemm_static(llvq_rt* rt, const llvq_mat* m, const void* x, int M, void* y, int y_dtype) {
  if (!rt || !m || M < 0) return fail(LLVQ_ERR_INVALID_ARGUMENT, "gemm_static: bad argument");
  if (y_dtype != LLVQ_F32 && y_dtype != LLVQ_F16) return fail(LLVQ_ERR_INVALID_ARGUMENT, "gemm_static: unknown output dtype");
  if (M == 0) return LLVQ_OK;
  if (!x || !y) return fail(LLVQ_ERR_INVALID_ARGUMENT, "gemm_static: null activation or output");
  if (!rt->static_scratch) return fail(LLVQ_ERR_UNSUPPORTED, "gemm_static: no static workspace on this device");
  HIP_TRY(hipSetDevice(rt->device));
  GemmWorkspace w;
  w.fixed = rt->static_scratch;
  w.fixed_bytes = kStaticScratchBytes;
  return gemm_same_basis(rt, &m, 1, x, M, &y, y_dtype, &w);
}

int llvq_hip_decode_blocks(llvq_rt* rt, const uint8_t* codes_dev, size_t nblocks, int8_t* points_dev,
                           uint8_t* gains_dev, uint8_t* shells_dev) {
  if (!rt) return fail(LLVQ_ERR_INVALID_ARGUMENT, "decode_blocks: runtime is null");
  if (nblocks == 0) return LLVQ_OK;  // an empty stream is valid and writes nothing
  if (!points_dev || !codes_dev) return fail(LLVQ_ERR_INVALID_ARGUMENT, "decode_blocks: null argument");
  if (reinterpret_cast<uintptr_t>(codes_dev) & 3) return fail(LLVQ_ERR_INVALID_ARGUMENT, "decode_blocks: codes must start on a 4-byte boundary");
  HIP_TRY(hipSetDevice(rt->device));
  size_t grid = (nblocks + 255) / 256;
  const size_t cap = (size_t)(rt->cu_count > 0 ? rt->cu_count : 256) * 2;
  if (grid > cap) grid = cap;
  hipLaunchKernelGGL(decode_blocks_kernel<false>, dim3((uint32_t)grid), dim3(256), kLdsImageBytes, rt->stream,
                     rt->tables, codes_dev, nblocks, points_dev, gains_dev, shells_dev);
  HIP_TRY(hipGetLastError());
  return LLVQ_OK;
}

int llvq_hip_decode_stream(llvq_rt* rt, const uint8_t* codes_dev, size_t nblocks, uint32_t shell_cap, int8_t* points_dev,
                           uint8_t* gains_dev, uint8_t* shells_dev) {
  if (!rt) return fail(LLVQ_ERR_INVALID_ARGUMENT, "decode_stream: runtime is null");
  if (shell_cap > (uint32_t)kMaxShell) return fail(LLVQ_ERR_INCONSISTENT, "decode_stream: shell cap " + std::to_string(shell_cap) + " exceeds the supported ball (m <= 13)");
  const int bits = index_bits(shell_cap) + 1;
  if (bits == 48) return llvq_hip_decode_blocks(rt, codes_dev, nblocks, points_dev, gains_dev, shells_dev);
  if (bits != (int)kDenseBits)
    return fail(LLVQ_ERR_UNSUPPORTED, "decode_stream: shell cap " + std::to_string(shell_cap) + " packs " + std::to_string(bits) +
                                          " bits per block; the kernels read 6-byte records (cap 12) and the 49-bit stream of cap 13");
  if (nblocks == 0) return LLVQ_OK;
  if (!points_dev || !codes_dev) return fail(LLVQ_ERR_INVALID_ARGUMENT, "decode_stream: null argument");
  HIP_TRY(hipSetDevice(rt->device));
  size_t grid = (nblocks + 255) / 256;
  const size_t cap = (size_t)(rt->cu_count > 0 ? rt->cu_count : 256) * 2;
  if (grid > cap) grid = cap;
  hipLaunchKernelGGL(decode_blocks_kernel<true>, dim3((uint32_t)grid), dim3(256), kLdsImageBytes, rt->stream,
                     rt->tables, codes_dev, nblocks, points_dev, gains_dev, shells_dev);
  HIP_TRY(hipGetLastError());
  return LLVQ_OK;
}

}  // extern "C"

// =================================================================================
// Batch-1 decode loop (C ABI)
// =================================================================================
struct llvq_decoder {
  llvq_rt* rt = nullptr;
  uint32_t n_layers = 0, hidden = 0, n_heads = 0, n_kv = 0, head_dim = 0, inter = 0, vocab = 0, max_pos = 0;
  float eps = 1e-6f;
  std::vector<const llvq_mat*> proj;  // [n_layers * 7]: q k v o gate up down
  uint8_t* blob = nullptr;            // every dense tensor and buffer below, one allocation
  __half *ln1 = nullptr, *ln2 = nullptr, *qn = nullptr, *kn = nullptr, *fnorm = nullptr;
  __half *embed = nullptr, *head = nullptr, *cos_t = nullptr, *sin_t = nullptr;
  bool embed_q8 = false, head_q8 = false;  // int8 rows instead of binary16
  QuantRows embed_q{}, head_q{};
  __half *kcache = nullptr, *vcache = nullptr;  // [n_layers][n_kv][max_pos][head_dim]
  __half *h = nullptr, *h_alt = nullptr, *normed = nullptr, *q = nullptr, *k = nullptr, *v = nullptr, *ctx = nullptr, *o = nullptr;
  __half *gate = nullptr, *up = nullptr, *act = nullptr, *down = nullptr;
  float* logits = nullptr;
  float* best_val = nullptr;
  uint32_t* best_idx = nullptr;
  uint32_t* token = nullptr;    // the token the next step embeds
  uint32_t* history = nullptr;  // [max_pos] tokens chosen by the head
  float* attn_part = nullptr;   // [n_heads][kAttnMaxSplits][head_dim + 2] partial attention sums
  bool kv_q8 = false;           // int8 KV cache (kvq.rs) instead of binary16
  KvQ8 q8{};                    // layer 0's arrays; a layer's are at + layer * (cache_layer or cache_layer / 64 groups)
  uint32_t* attn_counters = nullptr;  // [n_kv], zero between launches
  uint32_t pos = 0;
  uint32_t head_grid = 0;
  // rows of positions at once (llvq_hip_decoder_prefill): [prefill_rows, width] buffers, one allocation
  uint32_t prefill_rows = 0;
  uint8_t* pblob = nullptr;
  __half *ph = nullptr, *ph_alt = nullptr, *pnormed = nullptr, *pq = nullptr, *pk = nullptr, *pv = nullptr, *pctx = nullptr, *po = nullptr;
  __half *pgate = nullptr, *pup = nullptr, *pact = nullptr, *pdown = nullptr;
  uint32_t* ptokens = nullptr;
  // llvq_hip_decoder_generate_phased: events recorded at the phase boundaries of a step (null otherwise)
  std::vector<hipEvent_t>* marks = nullptr;
  size_t next_mark = 0;
  // A position's projections as sequences (empty: one launch of gemv_tiles_kernel per projection group).
  //   chained: seqs[0] = layer 0's q/k/v, seqs[L + 1] = layer L's o_proj, gate/up, down_proj and layer L + 1's q/k/v,
  //            each item ordered behind the one before it;
  //   single:  seqs[4 L + j] = layer L's q/k/v, o_proj, gate/up, down_proj, one item each.
  // They share one status word.
  std::vector<llvq_seq*> seqs;
  bool seq_chained = false;
  uint32_t* seq_status = nullptr;
};

namespace {

// A phase boundary of a timed step: the next event of the decoder's list goes onto the stream.
void phase_mark(llvq_decoder* d) {
  if (d->marks && d->next_mark < d->marks->size()) (void)hipEventRecord((*d->marks)[d->next_mark++], d->rt->stream);
}

// The head over dec->normed and the argmax, which overwrites *dec->token (and history[slot] when recording).
void launch_head(llvq_decoder* d, uint32_t history_slot, bool record) {
  hipStream_t st = d->rt->stream;
  if (d->head_q8)
    hipLaunchKernelGGL(lm_head_q8_kernel, dim3(d->head_grid), dim3(kHeadThreads), d->hidden * sizeof(float), st, d->head_q, d->normed,
                       d->vocab, d->hidden, d->logits, d->best_val, d->best_idx);
  else
    hipLaunchKernelGGL(lm_head_kernel, dim3(d->head_grid), dim3(kHeadThreads), d->hidden * sizeof(float), st, d->head, d->normed,
                       d->vocab, d->hidden, d->logits, d->best_val, d->best_idx);
  phase_mark(d);
  hipLaunchKernelGGL(argmax_final_kernel, dim3(1), dim3(1024), 0, st, d->best_val, d->best_idx,
                     d->head_grid * (kHeadThreads / 64), d->token, record ? d->history : (uint32_t*)nullptr, history_slot);
  phase_mark(d);
}

// Binds a position's projections as sequences (llvq_decoder::seqs), each item with the activation prologue its
// launch would have.  The residual stream alternates between the decoder's two buffers exactly as decoder_step's
// launches alternate them: layer 0's q/k/v reads h; every later prologue reads one buffer and stores the other.
// A model a sequence cannot take (rotated matrices, rows too wide) leaves seqs empty: one launch per group then.
int decoder_bind_sequences(llvq_decoder* d, bool chained) {
  llvq_rt* rt = d->rt;
  d->seq_chained = chained;
  __half *h = d->h, *h_alt = d->h_alt;
  auto give_up = [&](int rc) {
    for (llvq_seq* q : d->seqs) llvq_hip_sequence_destroy(rt, q);
    d->seqs.clear();
    return rc == LLVQ_ERR_UNSUPPORTED ? (int)LLVQ_OK : rc;
  };
  void* qkv_out[3] = {d->q, d->k, d->v};
  void* o_out[1] = {d->o};
  void* gu_out[2] = {d->gate, d->up};
  void* dn_out[1] = {d->down};
  auto qkv_item = [&](uint32_t L, bool ordered) {
    SeqSpec sp;
    sp.mats = d->proj.data() + (size_t)L * 7;
    sp.n = 3;
    sp.x = h;
    sp.y = qkv_out;
    sp.after_previous = ordered;
    sp.pro.kind = kPrologueAddRmsNorm;
    sp.pro.norm_w = d->ln1 + (size_t)L * d->hidden;
    sp.pro.eps = d->eps;
    if (L) {  // the previous layer's MLP output joins the residual stream here
      sp.pro.x2 = d->down;
      sp.pro.resid_out = h_alt;
      std::swap(h, h_alt);
    }
    return sp;
  };
  auto bind = [&](std::vector<SeqSpec>& items) {
    llvq_seq* q = nullptr;
    const int rc = seq_create(rt, items.data(), (int)items.size(), &q);
    if (rc) return rc;
    q->args.status = d->seq_status;
    d->seqs.push_back(q);
    return (int)LLVQ_OK;
  };
  if (!chained) {
    for (uint32_t L = 0; L < d->n_layers; ++L) {
      const llvq_mat* const* P = d->proj.data() + (size_t)L * 7;
      std::vector<SeqSpec> one(1);
      one[0] = qkv_item(L, false);
      int rc = bind(one);
      if (rc) return give_up(rc);
      SeqSpec o;
      o.mats = P + 3; o.n = 1; o.x = d->ctx; o.y = o_out;
      one[0] = o;
      if ((rc = bind(one))) return give_up(rc);
      SeqSpec gu;
      gu.mats = P + 4; gu.n = 2; gu.x = h; gu.y = gu_out;
      gu.pro.kind = kPrologueAddRmsNorm;
      gu.pro.norm_w = d->ln2 + (size_t)L * d->hidden;
      gu.pro.eps = d->eps;
      gu.pro.x2 = d->o;
      gu.pro.resid_out = h_alt;
      std::swap(h, h_alt);
      one[0] = gu;
      if ((rc = bind(one))) return give_up(rc);
      SeqSpec dn;
      dn.mats = P + 6; dn.n = 1; dn.x = d->up; dn.y = dn_out;
      dn.pro.kind = kPrologueSiluMul;
      dn.pro.x2 = d->gate;
      one[0] = dn;
      if ((rc = bind(one))) return give_up(rc);
    }
    return LLVQ_OK;
  }
  for (uint32_t L = 0; L <= d->n_layers; ++L) {
    std::vector<SeqSpec> items;
    if (L == 0) {
      items.push_back(qkv_item(0, false));
    } else {
      const llvq_mat* const* P = d->proj.data() + (size_t)(L - 1) * 7;
      SeqSpec o;
      o.mats = P + 3; o.n = 1; o.x = d->ctx; o.y = o_out;
      items.push_back(o);
      SeqSpec gu;
      gu.mats = P + 4; gu.n = 2; gu.x = h; gu.y = gu_out; gu.after_previous = true;
      gu.pro.kind = kPrologueAddRmsNorm;
      gu.pro.norm_w = d->ln2 + (size_t)(L - 1) * d->hidden;
      gu.pro.eps = d->eps;
      gu.pro.x2 = d->o;
      gu.pro.resid_out = h_alt;
      std::swap(h, h_alt);
      items.push_back(gu);
      SeqSpec dn;
      dn.mats = P + 6; dn.n = 1; dn.x = d->up; dn.y = dn_out; dn.after_previous = true;
      dn.pro.kind = kPrologueSiluMul;
      dn.pro.x2 = d->gate;
      items.push_back(dn);
      if (L < d->n_layers) items.push_back(qkv_item(L, true));
    }
    const int rc = bind(items);
    if (rc) return give_up(rc);
  }
  return LLVQ_OK;
}

// After the stream has drained: whether a workgroup of any sequence gave up waiting since the last check.
int decoder_check_sequences(llvq_decoder* d) {
  if (d->seqs.empty()) return LLVQ_OK;
  uint32_t st = 0;
  HIP_TRY(hipMemcpy(&st, d->seq_status, sizeof st, hipMemcpyDeviceToHost));
  if (!st) return LLVQ_OK;
  for (llvq_seq* q : d->seqs) {
    const int rc = seq_reset(q);
    if (rc) return rc;
  }
  return fail(LLVQ_ERR_DEVICE, "decoder: a workgroup gave up waiting for a projection of the same launch; the position's results are incomplete");
}

// Enqueues one position: embeds *dec->token, runs the layers at position dec->pos,
// and (want_logits) the head and the argmax, which overwrites *dec->token.
int decoder_step(llvq_decoder* d, bool want_logits, uint32_t history_slot, bool record) {
  llvq_rt* rt = d->rt;
  hipStream_t st = rt->stream;
  if (d->pos >= d->max_pos) return fail(LLVQ_ERR_INVALID_ARGUMENT, "decoder: position " + std::to_string(d->pos) + " is past max_positions");
  // the two residual buffers, by local name: a step that fails part-way leaves the decoder as it found it
  __half *h = d->h, *h_alt = d->h_alt;
  phase_mark(d);
  if (d->embed_q8)
    hipLaunchKernelGGL(embed_q8_kernel, dim3((d->hidden + 255) / 256), dim3(256), 0, st, d->embed_q, d->token, d->vocab, d->hidden, h);
  else
    hipLaunchKernelGGL(embed_kernel, dim3((d->hidden + 255) / 256), dim3(256), 0, st, d->embed, d->token, d->vocab, d->hidden, h);
  phase_mark(d);
  const size_t cache_layer = (size_t)d->n_kv * d->max_pos * d->head_dim;
  const uint32_t T = d->pos + 1;
  // about 64 cached positions per workgroup (one batch of four per position class), at most kAttnMaxSplits ranges
  uint32_t n_splits = (T + 63) / 64;
  if (n_splits > (uint32_t)kAttnMaxSplits) n_splits = kAttnMaxSplits;
  const uint32_t groups_per_kv = d->n_heads / d->n_kv;
  // the queries and the sixteen position classes' running results
  size_t attn_lds = ((size_t)groups_per_kv * d->head_dim + (size_t)16 * groups_per_kv * (d->head_dim + 2)) * sizeof(float);
  const size_t merge_lds = (size_t)groups_per_kv * 2 * n_splits * sizeof(float);  // the merge reuses the staging area
  if (attn_lds < merge_lds) attn_lds = merge_lds;
  const size_t group_layer = cache_layer / kKvGroup;
  // few partials: the last workgroup of a kv head merges them; many: a chip-wide merge kernel does
  const uint32_t merge_inline = n_splits <= (uint32_t)kAttnInlineSplits ? 1u : 0u;
  // Projections in the natural basis derive their activation in the launch's
  // prologue; a rotated basis needs the activation as a tensor first (it goes
  // through the rotation kernel), and so do rows too wide for the staging area:
  // their prologue runs as a kernel of its own.
  auto project = [&](const llvq_mat* const* mats, int n, const __half* x, void* const* outs, const Prologue& pro) -> int {
    // every launch of the group can derive (and, in a rotated basis, rotate) the activation itself
    bool fused = prologue_fits(mats[0]);
    for (int i = 0; i < n; ++i) fused &= !mats[i]->has_rotation || rotation_fits(mats[i]);
    if (fused) return forward_group(rt, mats, n, x, outs, LLVQ_F16, &pro);
    const __half* staged = nullptr;
    if (pro.kind == kPrologueAddRmsNorm) {
      hipLaunchKernelGGL(add_rmsnorm_kernel, dim3(1), dim3(kNormThreads), 0, st, x, reinterpret_cast<const __half*>(pro.x2),
                         reinterpret_cast<const __half*>(pro.norm_w), reinterpret_cast<__half*>(pro.resid_out), d->normed,
                         d->hidden, pro.eps);
      staged = d->normed;
    } else {
      hipLaunchKernelGGL(silu_mul_kernel, dim3((d->inter + 255) / 256), dim3(256), 0, st, reinterpret_cast<const __half*>(pro.x2),
                         x, d->act, d->inter);
      staged = d->act;
    }
    return forward_group(rt, mats, n, staged, outs, LLVQ_F16);
  };
  // q/k norm, rope and the cache append of this position ride in the attention launch
  auto attention = [&](uint32_t L) {
    KvQ8 lq8 = d->q8;
    if (d->kv_q8) {
      lq8.kq += L * cache_layer; lq8.vq += L * cache_layer;
      lq8.ks += L * group_layer; lq8.kb += L * group_layer; lq8.vs += L * group_layer; lq8.vb += L * group_layer;
    }
    __half* kc = d->kv_q8 ? nullptr : d->kcache + L * cache_layer;
    __half* vc = d->kv_q8 ? nullptr : d->vcache + L * cache_layer;
    AttnNew nw{};
    nw.q_raw = d->q;
    nw.k_raw = d->k;
    nw.v_raw = d->v;
    nw.qn = d->qn + (size_t)L * d->head_dim;
    nw.kn = d->kn + (size_t)L * d->head_dim;
    nw.cos_t = d->cos_t;
    nw.sin_t = d->sin_t;
    nw.kcache = kc;
    nw.vcache = vc;
    nw.eps = d->eps;
    auto attend = [&](auto kernel) {
      hipLaunchKernelGGL(kernel, dim3(d->n_kv * n_splits), dim3(kAttnThreads), attn_lds, st, nw, kc, vc, lq8, d->ctx, d->attn_part,
                         d->attn_counters, d->n_heads, d->n_kv, d->head_dim, T, d->max_pos, 1.0f / sqrtf((float)d->head_dim), n_splits,
                         merge_inline);
    };
    if (d->kv_q8) {
      if (groups_per_kv <= 2) attend(attn_decode_kernel<true, 2>);
      else if (groups_per_kv <= 4) attend(attn_decode_kernel<true, 4>);
      else if (groups_per_kv <= 5) attend(attn_decode_kernel<true, 5>);
      else attend(attn_decode_kernel<true, kAttnMaxGroup>);
    } else {
      if (groups_per_kv <= 2) attend(attn_decode_kernel<false, 2>);
      else if (groups_per_kv <= 4) attend(attn_decode_kernel<false, 4>);
      else if (groups_per_kv <= 5) attend(attn_decode_kernel<false, 5>);
      else attend(attn_decode_kernel<false, kAttnMaxGroup>);
    }
    if (!merge_inline)
      hipLaunchKernelGGL(attn_merge_kernel, dim3(d->n_heads), dim3(128), 0, st, d->attn_part, d->ctx, d->head_dim, n_splits);
  };
  if (!d->seqs.empty() && d->seq_chained) {
    // the projections between two attention launches are one persistent launch each
    int rc = seq_run(rt, d->seqs[0]);
    if (rc) return rc;
    for (uint32_t L = 0; L < d->n_layers; ++L) {
      attention(L);
      rc = seq_run(rt, d->seqs[(size_t)L + 1]);
      if (rc) return rc;
    }
    h = d->n_layers ? d->h_alt : d->h;  // where the last post-attention residual went (decoder_bind_sequences)
  } else if (!d->seqs.empty()) {
    // one launch per projection group, through the sequence kernel's tile loop
    for (uint32_t L = 0; L < d->n_layers; ++L) {
      int rc = seq_run(rt, d->seqs[(size_t)L * 4]);
      if (rc) return rc;
      attention(L);
      for (int j = 1; j < 4; ++j)
        if ((rc = seq_run(rt, d->seqs[(size_t)L * 4 + j]))) return rc;
    }
    h = d->n_layers ? d->h_alt : d->h;
  } else {
  // The residual stream alternates between two buffers: a projection launch whose
  // prologue adds the previous branch reads one and (workgroup 0) writes the other.
  for (uint32_t L = 0; L < d->n_layers; ++L) {
    const llvq_mat* const* P = d->proj.data() + (size_t)L * 7;
    // the previous layer's MLP output joins the residual stream in the q/k/v launch
    Prologue ln1;
    ln1.kind = kPrologueAddRmsNorm;
    ln1.norm_w = d->ln1 + (size_t)L * d->hidden;
    ln1.eps = d->eps;
    if (L) {
      ln1.x2 = d->down;
      ln1.resid_out = h_alt;
    }
    void* qkv_out[3] = {d->q, d->k, d->v};
    int rc = project(P, 3, h, qkv_out, ln1);
    if (rc) return rc;
    if (L) std::swap(h, h_alt);
    attention(L);
    void* o_out[1] = {d->o};
    rc = forward_group(rt, P + 3, 1, d->ctx, o_out, LLVQ_F16);
    if (rc) return rc;
    Prologue ln2;
    ln2.kind = kPrologueAddRmsNorm;
    ln2.norm_w = d->ln2 + (size_t)L * d->hidden;
    ln2.eps = d->eps;
    ln2.x2 = d->o;
    ln2.resid_out = h_alt;
    void* gu_out[2] = {d->gate, d->up};
    rc = project(P + 4, 2, h, gu_out, ln2);
    if (rc) return rc;
    std::swap(h, h_alt);
    Prologue act;
    act.kind = kPrologueSiluMul;
    act.x2 = d->gate;
    void* d_out[1] = {d->down};
    rc = project(P + 6, 1, d->up, d_out, act);
    if (rc) return rc;
  }
  }
  phase_mark(d);
  if (want_logits) {
    hipLaunchKernelGGL(add_rmsnorm_kernel, dim3(1), dim3(kNormThreads), 0, st, h, d->down, d->fnorm, h, d->normed, d->hidden, d->eps);
    launch_head(d, history_slot, record);
  }
  HIP_TRY(hipGetLastError());
  d->pos += 1;
  return LLVQ_OK;
}
// n <= prefill_rows positions at once, starting at dec->pos: tokens from dec->ptokens.
// With want_logits the head runs on the last row and leaves its argmax in *dec->token.
int decoder_prefill_pass(llvq_decoder* d, uint32_t n, bool want_logits, uint32_t history_slot, bool record) {
  llvq_rt* rt = d->rt;
  hipStream_t st = rt->stream;
  if (d->pos + n > d->max_pos) return fail(LLVQ_ERR_INVALID_ARGUMENT, "decoder_prefill: positions past max_positions");
  const uint32_t qd = d->n_heads * d->head_dim;
  __half *ph = d->ph, *ph_alt = d->ph_alt;  // by local name: a pass that fails part-way leaves the decoder as it found it
  if (d->embed_q8)
    hipLaunchKernelGGL(embed_q8_kernel, dim3((d->hidden + 255) / 256, n), dim3(256), 0, st, d->embed_q, d->ptokens, d->vocab, d->hidden, ph);
  else
    hipLaunchKernelGGL(embed_kernel, dim3((d->hidden + 255) / 256, n), dim3(256), 0, st, d->embed, d->ptokens, d->vocab, d->hidden, ph);
  const size_t cache_layer = (size_t)d->n_kv * d->max_pos * d->head_dim, group_layer = cache_layer / kKvGroup;
  const float scale = 1.0f / sqrtf((float)d->head_dim);
  auto rows = [&](const llvq_mat* m, const __half* x, __half* y) { return llvq_hip_gemm(rt, m, x, (int)n, y, LLVQ_F16); };
  for (uint32_t L = 0; L < d->n_layers; ++L) {
    const llvq_mat* const* P = d->proj.data() + (size_t)L * 7;
    // residual + previous MLP branch, then the input norm (the branch of layer 0 is absent)
    hipLaunchKernelGGL(add_rmsnorm_kernel, dim3(n), dim3(kNormThreads), 0, st, ph, L ? d->pdown : (const __half*)nullptr,
                       d->ln1 + (size_t)L * d->hidden, L ? ph_alt : (__half*)nullptr, d->pnormed, d->hidden, d->eps);
    if (L) std::swap(ph, ph_alt);
    void* const qkv[3] = {d->pq, d->pk, d->pv};
    int rc = llvq_hip_gemm_group(rt, P, 3, d->pnormed, (int)n, qkv, LLVQ_F16);
    if (rc) return rc;
    KvQ8 lq8 = d->q8;
    if (d->kv_q8) {
      lq8.kq += L * cache_layer; lq8.vq += L * cache_layer;
      lq8.ks += L * group_layer; lq8.kb += L * group_layer; lq8.vs += L * group_layer; lq8.vb += L * group_layer;
    }
    __half* kc = d->kv_q8 ? nullptr : d->kcache + L * cache_layer;
    __half* vc = d->kv_q8 ? nullptr : d->vcache + L * cache_layer;
    AttnNew nw{};
    nw.qn = d->qn + (size_t)L * d->head_dim;
    nw.kn = d->kn + (size_t)L * d->head_dim;
    nw.cos_t = d->cos_t;
    nw.sin_t = d->sin_t;
    nw.kcache = kc;
    nw.vcache = vc;
    nw.eps = d->eps;
    const dim3 hgrid(d->n_heads + 2 * d->n_kv, n), agrid(d->n_kv, n);
    auto attend = [&](auto kernel) {
      hipLaunchKernelGGL(kernel, agrid, dim3(64), 0, st, d->pq, kc, vc, lq8, d->pctx, d->n_heads, d->n_kv, d->head_dim, d->pos, d->max_pos, scale);
    };
    const uint32_t grp = d->n_heads / d->n_kv;
    // 32 rows per workgroup on the matrix cores where the head width is the one that kernel is built for
    const bool on_mfma = d->head_dim == 128 && grp <= (uint32_t)kAttnMaxGroup;
    const dim3 mgrid(d->n_kv, (n + kAttnTile - 1) / kAttnTile);
    auto attend_mfma = [&](auto kernel, uint32_t waves) {
      hipLaunchKernelGGL(kernel, mgrid, dim3(waves * 64), 0, st, d->pq, kc, vc, lq8, d->pctx, d->n_heads, d->n_kv, d->pos, n, d->max_pos, scale);
    };
    if (d->kv_q8) {
      hipLaunchKernelGGL(norm_rope_append_rows_kernel<true>, hgrid, dim3(64), 0, st, d->pq, d->pk, d->pv, nw, lq8, d->n_heads, d->n_kv,
                         d->head_dim, d->pos, d->max_pos);
      if (on_mfma) {
        if (grp <= 2) attend_mfma(attn_rows_mfma_kernel<true, 2>, 2);
        else if (grp <= 4) attend_mfma(attn_rows_mfma_kernel<true, 4>, 4);
        else if (grp <= 5) attend_mfma(attn_rows_mfma_kernel<true, 5>, 5);
        else attend_mfma(attn_rows_mfma_kernel<true, kAttnMaxGroup>, kAttnMaxGroup);
      } else if (grp <= 2) attend(attn_rows_kernel<true, 2>);
      else if (grp <= 4) attend(attn_rows_kernel<true, 4>);
      else if (grp <= 5) attend(attn_rows_kernel<true, 5>);
      else attend(attn_rows_kernel<true, kAttnMaxGroup>);
    } else {
      hipLaunchKernelGGL(norm_rope_append_rows_kernel<false>, hgrid, dim3(64), 0, st, d->pq, d->pk, d->pv, nw, lq8, d->n_heads, d->n_kv,
                         d->head_dim, d->pos, d->max_pos);
      if (on_mfma) {
        if (grp <= 2) attend_mfma(attn_rows_mfma_kernel<false, 2>, 2);
        else if (grp <= 4) attend_mfma(attn_rows_mfma_kernel<false, 4>, 4);
        else if (grp <= 5) attend_mfma(attn_rows_mfma_kernel<false, 5>, 5);
        else attend_mfma(attn_rows_mfma_kernel<false, kAttnMaxGroup>, kAttnMaxGroup);
      } else if (grp <= 2) attend(attn_rows_kernel<false, 2>);
      else if (grp <= 4) attend(attn_rows_kernel<false, 4>);
      else if (grp <= 5) attend(attn_rows_kernel<false, 5>);
      else attend(attn_rows_kernel<false, kAttnMaxGroup>);
    }
    rc = rows(P[3], d->pctx, d->po);
    if (rc) return rc;
    hipLaunchKernelGGL(add_rmsnorm_kernel, dim3(n), dim3(kNormThreads), 0, st, ph, d->po, d->ln2 + (size_t)L * d->hidden, ph_alt,
                       d->pnormed, d->hidden, d->eps);
    std::swap(ph, ph_alt);
    void* const gate_up[2] = {d->pgate, d->pup};
    rc = llvq_hip_gemm_group(rt, P + 4, 2, d->pnormed, (int)n, gate_up, LLVQ_F16);
    if (rc) return rc;
    const uint32_t na = n * d->inter;
    hipLaunchKernelGGL(silu_mul_kernel, dim3((na + 255) / 256 < 4096u ? (na + 255) / 256 : 4096u), dim3(256), 0, st, d->pgate, d->pup, d->pact, na);
    rc = rows(P[6], d->pact, d->pdown);
    if (rc) return rc;
  }
  if (want_logits) {
    const size_t last = (size_t)(n - 1) * d->hidden;
    hipLaunchKernelGGL(add_rmsnorm_kernel, dim3(1), dim3(kNormThreads), 0, st, ph + last, d->pdown + last, d->fnorm, d->h, d->normed,
                       d->hidden, d->eps);
    launch_head(d, history_slot, record);
  }
  HIP_TRY(hipGetLastError());
  d->pos += n;
  (void)qd;
  return LLVQ_OK;
}

// The prompt through decoder_prefill_pass, prefill_rows positions at a time; the head runs after the last one.
int decoder_prefill(llvq_decoder* d, const uint32_t* tokens, size_t n, uint32_t history_slot, bool record) {
  if (!d->prefill_rows) return fail(LLVQ_ERR_UNSUPPORTED, "decoder_prefill: the decoder was created with prefill_rows = 0");
  for (size_t at = 0; at < n; at += d->prefill_rows) {
    const uint32_t c = (uint32_t)(n - at < d->prefill_rows ? n - at : d->prefill_rows);
    HIP_TRY(hipMemcpyAsync(d->ptokens, tokens + at, c * sizeof(uint32_t), hipMemcpyHostToDevice, d->rt->stream));
    const int rc = decoder_prefill_pass(d, c, at + c == n, history_slot, record);
    if (rc) return rc;
  }
  return LLVQ_OK;
}

}  // namespace

extern "C" {

int llvq_hip_decoder_create(llvq_rt* rt, const llvq_decoder_desc* c, llvq_decoder** out) {
  if (!rt || !c || !out) return fail(LLVQ_ERR_INVALID_ARGUMENT, "decoder_create: null argument");
  *out = nullptr;
  if (!c->projections || !c->input_norm || !c->post_norm || !c->q_norm || !c->k_norm || !c->final_norm ||
      (!c->embed && !c->embed_q8.codes))
    return fail(LLVQ_ERR_INVALID_ARGUMENT, "decoder_create: a required tensor is null");
  for (const llvq_quant_rows* qr : {&c->embed_q8, &c->lm_head_q8})
    if (qr->codes) {
      if (!qr->scales || !qr->biases) return fail(LLVQ_ERR_INVALID_ARGUMENT, "decoder_create: an int8 tensor without scales or biases");
      // what the kernels compile in (fused_cuda.rs:418-447): 8 bits, groups of 64, whole 16-byte runs per row
      if (qr->bits != 8 || qr->group != kEmbedGroup || c->hidden % 16)
        return fail(LLVQ_ERR_UNSUPPORTED, "decoder_create: int" + std::to_string(qr->bits) + " g" + std::to_string(qr->group) +
                                              " — the kernels hard-code int8 g64 and hidden % 16 = 0");
    }
  if (c->n_layers == 0 || c->hidden == 0 || c->hidden % 8 || c->hidden > 8192 || c->n_heads == 0 || c->n_kv_heads == 0 ||
      c->n_heads % c->n_kv_heads || c->n_heads / c->n_kv_heads > (uint32_t)kAttnMaxGroup || c->head_dim == 0 || c->head_dim % 8 || c->head_dim > 128 || c->intermediate == 0 ||
      c->vocab == 0 || c->max_positions == 0 || c->max_positions > 8192 ||
      (c->kv_mode != LLVQ_KV_F16 && c->kv_mode != LLVQ_KV_Q8) || (c->kv_mode == LLVQ_KV_Q8 && c->head_dim % 64))
    return fail(LLVQ_ERR_UNSUPPORTED,
                "decoder_create: shape outside what the kernels hold (hidden % 8 = 0 and <= 8192, head_dim % 8 = 0 and <= 128, "
                "heads a multiple of kv heads and at most 8 per kv head, max_positions <= 8192, kv_mode f16 or q8 with head_dim % 64 = 0)");
  if (c->prefill_rows > 4096) return fail(LLVQ_ERR_UNSUPPORTED, "decoder_create: the batched prompt path takes at most 4096 rows per pass");
  const uint32_t qd = c->n_heads * c->head_dim, kvd = c->n_kv_heads * c->head_dim;
  static const char* kSite[7] = {"q_proj", "k_proj", "v_proj", "o_proj", "gate_proj", "up_proj", "down_proj"};
  const uint32_t want_out[7] = {qd, kvd, kvd, c->hidden, c->intermediate, c->intermediate, c->hidden};
  const uint32_t want_in[7] = {c->hidden, c->hidden, c->hidden, qd, c->hidden, c->hidden, c->intermediate};
  for (uint32_t L = 0; L < c->n_layers; ++L)
    for (int j = 0; j < 7; ++j) {
      const llvq_mat* m = c->projections[(size_t)L * 7 + j];
      if (!m) return fail(LLVQ_ERR_INVALID_ARGUMENT, "decoder_create: layer " + std::to_string(L) + " " + kSite[j] + " is null");
      if (m->d_out != want_out[j] || m->d_in != want_in[j])
        return fail(LLVQ_ERR_INCONSISTENT, "decoder_create: layer " + std::to_string(L) + " " + kSite[j] + " is " +
                                               std::to_string(m->d_out) + "x" + std::to_string(m->d_in) + ", the architecture needs " +
                                               std::to_string(want_out[j]) + "x" + std::to_string(want_in[j]));
    }
  HIP_TRY(hipSetDevice(rt->device));
  auto* d = new llvq_decoder();
  d->rt = rt;
  d->n_layers = c->n_layers; d->hidden = c->hidden; d->n_heads = c->n_heads; d->n_kv = c->n_kv_heads;
  d->head_dim = c->head_dim; d->inter = c->intermediate; d->vocab = c->vocab; d->max_pos = c->max_positions;
  d->eps = (float)c->rms_eps;
  d->kv_q8 = c->kv_mode == LLVQ_KV_Q8;
  d->proj.assign(c->projections, c->projections + (size_t)c->n_layers * 7);
  d->head_grid = 1024;
  while (d->head_grid > 1 && (uint64_t)d->head_grid * (kHeadThreads / 64) > c->vocab) d->head_grid >>= 1;

  // RoPE tables exactly as Rotary::new builds them (model.rs:163-179): f32 inverse
  // frequencies from an f64 power, f32 angle = position * inv_freq, sin/cos narrowed to binary16.
  const uint32_t half_d = c->head_dim / 2;
  std::vector<__half> cos_h((size_t)c->max_positions * half_d), sin_h(cos_h.size());
  for (uint32_t i = 0; i < half_d; ++i) {
    const float inv = 1.0f / (float)std::pow(c->rope_theta, (double)(2 * i) / (double)c->head_dim);
    for (uint32_t p = 0; p < c->max_positions; ++p) {
      const float ang = (float)p * inv;
      cos_h[(size_t)p * half_d + i] = __float2half_rn(std::cos(ang));
      sin_h[(size_t)p * half_d + i] = __float2half_rn(std::sin(ang));
    }
  }

  // one allocation, 256-byte aligned pieces
  size_t total = 0;
  auto take = [&](size_t bytes) { const size_t at = total; total += (bytes + 255) & ~(size_t)255; return at; };
  const size_t hb = sizeof(__half);
  const size_t o_ln1 = take((size_t)c->n_layers * c->hidden * hb), o_ln2 = take((size_t)c->n_layers * c->hidden * hb);
  const size_t o_qn = take((size_t)c->n_layers * c->head_dim * hb), o_kn = take((size_t)c->n_layers * c->head_dim * hb);
  const size_t o_fn = take((size_t)c->hidden * hb);
  const size_t vh = (size_t)c->vocab * c->hidden, vg = (size_t)c->vocab * ((c->hidden + kEmbedGroup - 1) / kEmbedGroup);
  const bool eq8 = c->embed_q8.codes != nullptr;
  // the head: its own int8 or binary16 tensor, else tied to the embedding in whichever encoding that is
  const bool hq8 = c->lm_head_q8.codes != nullptr || (!c->lm_head && eq8);
  const bool head_own = c->lm_head_q8.codes != nullptr || c->lm_head != nullptr;
  const size_t o_emb = take(eq8 ? vh : vh * hb), o_emb_s = take(eq8 ? vg * hb : 0), o_emb_b = take(eq8 ? vg * hb : 0);
  const size_t o_head = head_own ? take(hq8 ? vh : vh * hb) : o_emb;
  const size_t o_head_s = head_own ? take(hq8 ? vg * hb : 0) : o_emb_s, o_head_b = head_own ? take(hq8 ? vg * hb : 0) : o_emb_b;
  const size_t o_cos = take(cos_h.size() * hb), o_sin = take(sin_h.size() * hb);
  const size_t cache_vals = (size_t)c->n_layers * c->n_kv_heads * c->max_positions * c->head_dim;
  const bool q8 = c->kv_mode == LLVQ_KV_Q8;
  const size_t o_kc = take(cache_vals * (q8 ? 1 : hb)), o_vc = take(cache_vals * (q8 ? 1 : hb));
  const size_t o_ks = take(q8 ? cache_vals / kKvGroup * hb : 0), o_kb = take(q8 ? cache_vals / kKvGroup * hb : 0);
  const size_t o_vs = take(q8 ? cache_vals / kKvGroup * hb : 0), o_vb = take(q8 ? cache_vals / kKvGroup * hb : 0);
  const size_t o_h = take(c->hidden * hb), o_h2 = take(c->hidden * hb), o_nm = take(c->hidden * hb), o_q = take(qd * hb), o_k = take(kvd * hb), o_v = take(kvd * hb);
  const size_t o_ctx = take(qd * hb), o_o = take(c->hidden * hb), o_g = take(c->intermediate * hb), o_u = take(c->intermediate * hb);
  const size_t o_act = take(c->intermediate * hb), o_dn = take(c->hidden * hb);
  const size_t o_log = take((size_t)c->vocab * sizeof(float));
  const size_t n_best = (size_t)d->head_grid * (kHeadThreads / 64);
  const size_t o_bv = take(n_best * sizeof(float)), o_bi = take(n_best * sizeof(uint32_t));
  const size_t o_tok = take(sizeof(uint32_t)), o_hist = take((size_t)c->max_positions * sizeof(uint32_t));
  const size_t o_ap = take((size_t)c->n_heads * kAttnMaxSplits * (c->head_dim + 2) * sizeof(float)), o_ac = take((size_t)c->n_kv_heads * sizeof(uint32_t));
  const size_t o_seqst = take(256);
  hipError_t e = hipMalloc(reinterpret_cast<void**>(&d->blob), total);
  if (e != hipSuccess) { delete d; return hip_fail(e, "hipMalloc(decoder)"); }
  auto put = [&](size_t at, const void* src, size_t bytes) { return hipMemcpy(d->blob + at, src, bytes, hipMemcpyHostToDevice); };
  e = hipMemset(d->blob, 0, total);
  if (e == hipSuccess) e = put(o_ln1, c->input_norm, (size_t)c->n_layers * c->hidden * hb);
  if (e == hipSuccess) e = put(o_ln2, c->post_norm, (size_t)c->n_layers * c->hidden * hb);
  if (e == hipSuccess) e = put(o_qn, c->q_norm, (size_t)c->n_layers * c->head_dim * hb);
  if (e == hipSuccess) e = put(o_kn, c->k_norm, (size_t)c->n_layers * c->head_dim * hb);
  if (e == hipSuccess) e = put(o_fn, c->final_norm, (size_t)c->hidden * hb);
  if (e == hipSuccess && !eq8) e = put(o_emb, c->embed, vh * hb);
  if (e == hipSuccess && eq8) e = put(o_emb, c->embed_q8.codes, vh);
  if (e == hipSuccess && eq8) e = put(o_emb_s, c->embed_q8.scales, vg * hb);
  if (e == hipSuccess && eq8) e = put(o_emb_b, c->embed_q8.biases, vg * hb);
  if (e == hipSuccess && head_own && !hq8) e = put(o_head, c->lm_head, vh * hb);
  if (e == hipSuccess && head_own && hq8) e = put(o_head, c->lm_head_q8.codes, vh);
  if (e == hipSuccess && head_own && hq8) e = put(o_head_s, c->lm_head_q8.scales, vg * hb);
  if (e == hipSuccess && head_own && hq8) e = put(o_head_b, c->lm_head_q8.biases, vg * hb);
  if (e == hipSuccess) e = put(o_cos, cos_h.data(), cos_h.size() * hb);
  if (e == hipSuccess) e = put(o_sin, sin_h.data(), sin_h.size() * hb);
  if (e != hipSuccess) { (void)hipFree(d->blob); delete d; return hip_fail(e, "decoder upload"); }
  auto H = [&](size_t at) { return reinterpret_cast<__half*>(d->blob + at); };
  d->ln1 = H(o_ln1); d->ln2 = H(o_ln2); d->qn = H(o_qn); d->kn = H(o_kn); d->fnorm = H(o_fn);
  d->embed = H(o_emb); d->head = H(o_head); d->cos_t = H(o_cos); d->sin_t = H(o_sin);
  d->embed_q8 = eq8;
  d->head_q8 = hq8;
  d->embed_q = QuantRows{d->blob + o_emb, H(o_emb_s), H(o_emb_b)};
  d->head_q = QuantRows{d->blob + o_head, H(o_head_s), H(o_head_b)};
  d->kcache = H(o_kc); d->vcache = H(o_vc);
  if (q8) {
    d->q8.kq = d->blob + o_kc; d->q8.vq = d->blob + o_vc;
    d->q8.ks = H(o_ks); d->q8.kb = H(o_kb); d->q8.vs = H(o_vs); d->q8.vb = H(o_vb);
  }
  d->h = H(o_h); d->h_alt = H(o_h2); d->normed = H(o_nm); d->q = H(o_q); d->k = H(o_k); d->v = H(o_v); d->ctx = H(o_ctx); d->o = H(o_o);
  d->gate = H(o_g); d->up = H(o_u); d->act = H(o_act); d->down = H(o_dn);
  d->logits = reinterpret_cast<float*>(d->blob + o_log);
  d->best_val = reinterpret_cast<float*>(d->blob + o_bv);
  d->best_idx = reinterpret_cast<uint32_t*>(d->blob + o_bi);
  d->token = reinterpret_cast<uint32_t*>(d->blob + o_tok);
  d->history = reinterpret_cast<uint32_t*>(d->blob + o_hist);
  d->attn_part = reinterpret_cast<float*>(d->blob + o_ap);
  d->attn_counters = reinterpret_cast<uint32_t*>(d->blob + o_ac);
  d->seq_status = reinterpret_cast<uint32_t*>(d->blob + o_seqst);
  if (c->prefill_rows) {
    // row buffers of the batched prompt path, one allocation
    const size_t R = c->prefill_rows;
    size_t ptotal = 0;
    auto ptake = [&](size_t bytes) { const size_t at = ptotal; ptotal += (bytes + 255) & ~(size_t)255; return at; };
    const size_t p_h = ptake(R * c->hidden * hb), p_h2 = ptake(R * c->hidden * hb), p_nm = ptake(R * c->hidden * hb);
    const size_t p_q = ptake(R * qd * hb), p_k = ptake(R * kvd * hb), p_v = ptake(R * kvd * hb), p_ctx = ptake(R * qd * hb);
    const size_t p_o = ptake(R * c->hidden * hb), p_g = ptake(R * c->intermediate * hb), p_u = ptake(R * c->intermediate * hb);
    const size_t p_act = ptake(R * c->intermediate * hb), p_dn = ptake(R * c->hidden * hb), p_tok = ptake(R * sizeof(uint32_t));
    e = hipMalloc(reinterpret_cast<void**>(&d->pblob), ptotal);
    if (e == hipSuccess) e = hipMemset(d->pblob, 0, ptotal);
    if (e != hipSuccess) { (void)hipFree(d->pblob); (void)hipFree(d->blob); delete d; return hip_fail(e, "hipMalloc(decoder prefill rows)"); }
    auto PH = [&](size_t at) { return reinterpret_cast<__half*>(d->pblob + at); };
    d->prefill_rows = c->prefill_rows;
    d->ph = PH(p_h); d->ph_alt = PH(p_h2); d->pnormed = PH(p_nm); d->pq = PH(p_q); d->pk = PH(p_k); d->pv = PH(p_v); d->pctx = PH(p_ctx);
    d->po = PH(p_o); d->pgate = PH(p_g); d->pup = PH(p_u); d->pact = PH(p_act); d->pdown = PH(p_dn);
    d->ptokens = reinterpret_cast<uint32_t*>(d->pblob + p_tok);
    // the batched products of a pass find their workspaces sized: no allocation (and no implicit
    // device synchronisation) between the launches of a prompt
    for (uint32_t L = 0; L < c->n_layers; ++L) {
      const llvq_mat* const* P = d->proj.data() + (size_t)L * 7;
      int rc = reserve_batched(rt, P, 3, c->prefill_rows);
      if (!rc) rc = reserve_batched(rt, P + 3, 1, c->prefill_rows);
      if (!rc) rc = reserve_batched(rt, P + 4, 2, c->prefill_rows);
      if (!rc) rc = reserve_batched(rt, P + 6, 1, c->prefill_rows);
      if (rc) { (void)hipFree(d->pblob); (void)hipFree(d->blob); delete d; return rc; }
    }
  }
  if (c->launch_mode > LLVQ_LAUNCH_CHAINED) {
    (void)hipFree(d->pblob); (void)hipFree(d->blob); delete d;
    return fail(LLVQ_ERR_INVALID_ARGUMENT, "decoder_create: unknown launch_mode");
  }
  if (c->launch_mode != LLVQ_LAUNCH_PER_GROUP) {
    const int rc = decoder_bind_sequences(d, c->launch_mode == LLVQ_LAUNCH_CHAINED);
    if (rc) { (void)hipFree(d->pblob); (void)hipFree(d->blob); delete d; return rc; }
  }
  *out = d;
  return LLVQ_OK;
}

void llvq_hip_decoder_destroy(llvq_decoder* d) {
  if (!d) return;
  (void)hipSetDevice(d->rt->device);
  (void)hipStreamSynchronize(d->rt->stream);
  for (llvq_seq* q : d->seqs) llvq_hip_sequence_destroy(d->rt, q);
  (void)hipFree(d->pblob);
  (void)hipFree(d->blob);
  delete d;
}

int llvq_hip_decoder_reset(llvq_decoder* d) {
  if (!d) return fail(LLVQ_ERR_INVALID_ARGUMENT, "decoder_reset: null decoder");
  d->pos = 0;  // the cache is overwritten position by position; nothing else carries state
  return LLVQ_OK;
}

int llvq_hip_decoder_position(const llvq_decoder* d) { return d ? (int)d->pos : -1; }

int llvq_hip_decoder_seek(llvq_decoder* d, uint32_t position) {
  if (!d) return fail(LLVQ_ERR_INVALID_ARGUMENT, "decoder_seek: null decoder");
  if (position >= d->max_pos) return fail(LLVQ_ERR_INVALID_ARGUMENT, "decoder_seek: position past max_positions");
  d->pos = position;
  return LLVQ_OK;
}

int llvq_hip_decoder_forward_token(llvq_decoder* d, uint32_t token, float* logits_host, uint32_t* argmax_host) {
  if (!d) return fail(LLVQ_ERR_INVALID_ARGUMENT, "decoder_forward_token: null decoder");
  if (token >= d->vocab) return fail(LLVQ_ERR_INVALID_ARGUMENT, "decoder_forward_token: token " + std::to_string(token) + " is outside the vocabulary");
  HIP_TRY(hipSetDevice(d->rt->device));
  hipLaunchKernelGGL(set_token_kernel, dim3(1), dim3(1), 0, d->rt->stream, d->token, token);
  const int rc = decoder_step(d, true, 0, false);
  if (rc) return rc;
  if (logits_host) HIP_TRY(hipMemcpyAsync(logits_host, d->logits, (size_t)d->vocab * sizeof(float), hipMemcpyDeviceToHost, d->rt->stream));
  if (argmax_host) HIP_TRY(hipMemcpyAsync(argmax_host, d->token, sizeof(uint32_t), hipMemcpyDeviceToHost, d->rt->stream));
  HIP_TRY(hipStreamSynchronize(d->rt->stream));
  return decoder_check_sequences(d);
}

static int generate_impl(llvq_decoder* d, const uint32_t* prompt, size_t n_prompt, size_t max_new, uint32_t* out, bool batched,
                         const char* who, double* phase_ms = nullptr) {
  if (!d || (n_prompt && !prompt) || (max_new && !out)) return fail(LLVQ_ERR_INVALID_ARGUMENT, std::string(who) + ": null argument");
  if (max_new == 0) return LLVQ_OK;  // model.rs:1052-1054
  if (n_prompt == 0) return fail(LLVQ_ERR_INVALID_ARGUMENT, std::string(who) + ": empty prompt");
  if (n_prompt + max_new - 1 > d->max_pos)
    return fail(LLVQ_ERR_INVALID_ARGUMENT, std::string(who) + ": " + std::to_string(n_prompt + max_new - 1) + " positions exceed max_positions " + std::to_string(d->max_pos));
  for (size_t i = 0; i < n_prompt; ++i)
    if (prompt[i] >= d->vocab) return fail(LLVQ_ERR_INVALID_ARGUMENT, std::string(who) + ": prompt token outside the vocabulary");
  HIP_TRY(hipSetDevice(d->rt->device));
  d->pos = 0;
  // Phase timing: five events per timed step (start, after the embedding, after the layers, after the
  // head, after the argmax); the step that ends the prompt is the first timed one.
  std::vector<hipEvent_t> marks;
  struct MarksGuard {
    llvq_decoder* d;
    std::vector<hipEvent_t>* m;
    ~MarksGuard() {
      d->marks = nullptr;
      for (hipEvent_t e : *m) (void)hipEventDestroy(e);
    }
  } guard{d, &marks};
  if (phase_ms) {
    marks.resize(5 * max_new);
    for (auto& e : marks) {
      e = nullptr;
      HIP_TRY(hipEventCreate(&e));
    }
  }
  if (batched) {
    const int rc = decoder_prefill(d, prompt, n_prompt, 0, true);
    if (rc) return rc;
  } else {
    for (size_t i = 0; i < n_prompt; ++i) {
      hipLaunchKernelGGL(set_token_kernel, dim3(1), dim3(1), 0, d->rt->stream, d->token, prompt[i]);
      if (phase_ms && i + 1 == n_prompt) { d->marks = &marks; d->next_mark = 0; }
      const int rc = decoder_step(d, i + 1 == n_prompt, 0, true);
      if (rc) return rc;
    }
  }
  for (size_t t = 1; t < max_new; ++t) {
    const int rc = decoder_step(d, true, (uint32_t)t, true);
    if (rc) return rc;
  }
  HIP_TRY(hipMemcpyAsync(out, d->history, max_new * sizeof(uint32_t), hipMemcpyDeviceToHost, d->rt->stream));
  HIP_TRY(hipStreamSynchronize(d->rt->stream));
  {
    const int rc = decoder_check_sequences(d);
    if (rc) return rc;
  }
  if (phase_ms) {
    auto between = [&](size_t a, size_t b, double* ms) -> int {
      float f = 0.f;
      HIP_TRY(hipEventElapsedTime(&f, marks[a], marks[b]));
      *ms = (double)f;
      return LLVQ_OK;
    };
    for (size_t t = 0; t < max_new; ++t) {
      double* row = phase_ms + 4 * t;
      row[0] = row[1] = row[2] = row[3] = 0.0;
      int rc = between(5 * t + 2, 5 * t + 3, &row[0]);           // final norm + head of the step that chose token t
      if (!rc) rc = between(5 * t + 3, 5 * t + 4, &row[1]);      // argmax
      if (!rc && t + 1 < max_new) rc = between(5 * (t + 1), 5 * (t + 1) + 1, &row[2]);      // embedding of token t
      if (!rc && t + 1 < max_new) rc = between(5 * (t + 1) + 1, 5 * (t + 1) + 2, &row[3]);  // the layers over it
      if (rc) return rc;
    }
  }
  return LLVQ_OK;
}

int llvq_hip_decoder_generate(llvq_decoder* d, const uint32_t* prompt, size_t n_prompt, size_t max_new, uint32_t* out) {
  return generate_impl(d, prompt, n_prompt, max_new, out, false, "decoder_generate");
}

int llvq_hip_decoder_generate_prefilled(llvq_decoder* d, const uint32_t* prompt, size_t n_prompt, size_t max_new, uint32_t* out) {
  return generate_impl(d, prompt, n_prompt, max_new, out, true, "decoder_generate_prefilled");
}

int llvq_hip_decoder_generate_phased(llvq_decoder* d, const uint32_t* prompt, size_t n_prompt, size_t max_new, uint32_t* out,
                                     double* phase_ms) {
  if (max_new && !phase_ms) return fail(LLVQ_ERR_INVALID_ARGUMENT, "decoder_generate_phased: null phase array");
  return generate_impl(d, prompt, n_prompt, max_new, out, false, "decoder_generate_phased", phase_ms);
}

int llvq_hip_decoder_prefill(llvq_decoder* d, const uint32_t* tokens, size_t n, float* logits_host, uint32_t* argmax_host) {
  if (!d || !tokens || n == 0) return fail(LLVQ_ERR_INVALID_ARGUMENT, "decoder_prefill: null or empty argument");
  if (d->pos + n > d->max_pos) return fail(LLVQ_ERR_INVALID_ARGUMENT, "decoder_prefill: positions past max_positions");
  for (size_t i = 0; i < n; ++i)
    if (tokens[i] >= d->vocab) return fail(LLVQ_ERR_INVALID_ARGUMENT, "decoder_prefill: token outside the vocabulary");
  HIP_TRY(hipSetDevice(d->rt->device));
  const int rc = decoder_prefill(d, tokens, n, 0, false);
  if (rc) return rc;
  if (logits_host) HIP_TRY(hipMemcpyAsync(logits_host, d->logits, (size_t)d->vocab * sizeof(float), hipMemcpyDeviceToHost, d->rt->stream));
  if (argmax_host) HIP_TRY(hipMemcpyAsync(argmax_host, d->token, sizeof(uint32_t), hipMemcpyDeviceToHost, d->rt->stream));
  HIP_TRY(hipStreamSynchronize(d->rt->stream));
  return LLVQ_OK;
}

#ifdef LLVQ_SEQ_STAMPS
llvq_seq* llvq_hip_decoder_debug_sequence(llvq_decoder* d, int index) {
  return d && index >= 0 && (size_t)index < d->seqs.size() ? d->seqs[(size_t)index] : nullptr;
}
#endif

}  // extern "C"
