// Fused dequant-GEMM for batched activations: Y[M, d_out] = X[M, d_in] W^T with
// W unranked on the fly and contracted on the matrix cores (f16 operands, f32
// accumulate).  Included by llvq_hip.hip after the GEMV kernel, whose helpers
// (table staging, record reads, queues) it shares.
//
// The reference runs a batch as a row loop over its GEMV
// (llvq-llm/src/model.rs:521-529); this kernel decodes every block once for
// all M rows instead.
//
// Work unit: a band of 64 weight rows x a range of blocks of those rows.  One
// persistent 1024-lane workgroup per CU walks its unit in K-slices of at most
// 32 blocks per row (768 columns, 2048 blocks):
//   P0  the slice's code bytes, 16-byte loads -> LDS (next slice's loads are
//       already in flight while this one is decoded);
//   P1  classify and bin the blocks (odd / even / generic queues);
//   P2  unrank; every block writes its 24 weights, already multiplied by
//       centroid[gain] / sqrt(16 shell), as binary16 into the W slice in LDS;
//   P3  16 wavefronts run v_mfma_f32_32x32x16_f16 over the slice: A fragments
//       from LDS, B fragments (activations) straight from global memory / L2,
//       fetched one batch ahead.  Up to 256 activation rows the wavefront grid
//       is 2 row tiles x 8 column tiles of 32; beyond, every wavefront takes
//       both row tiles of one of 16 column tiles.  Accumulators (16 or 32
//       registers) stay live across slices.
// Epilogue: row scale and the f32 tail columns in f32, then the store.  When a
// matrix has too few bands to occupy the chip its block range is split over
// several units; each writes its partial sums to a workspace and a second,
// chip-wide kernel (gemm_reduce_kernel) adds them in split order and applies
// the epilogue, so the result does not depend on scheduling.
#pragma once

namespace llvq {

typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float float16_t __attribute__((ext_vector_type(16)));

constexpr int kGemmRows = 64;                 // weight rows of a band
#ifndef LLVQ_GEMM_KB
#define LLVQ_GEMM_KB 32
#endif
constexpr int kGemmKb = LLVQ_GEMM_KB;         // blocks per row and K-slice (32: 768 columns = 24 K-steps of 32, 2048 blocks = two 64-block chunks per wavefront)
constexpr int kGemmTile = kGemmRows * kGemmKb;  // blocks per K-slice
constexpr int kGemmP1Blocks = (kGemmTile + kWgThreads - 1) / kWgThreads;
constexpr int kGemmRowChunks = (kGemmKb * 6 + 14 + 15) / 16;  // 16-byte units holding one row's code bytes at any even alignment
constexpr int kGemmRowBytes = kGemmRowChunks * 16;
constexpr int kGemmWStride = kGemmKb * 24 + 8;  // binary16 elements per W row in LDS; the pad spreads rows over banks
constexpr int kGemmMaxM = 512;                // activation rows per launch (32 column tiles of 16)
static_assert(kGemmRows * kGemmRowChunks <= kWgThreads, "one 16-byte load per lane covers a slice's code bytes");
static_assert(kGemmTile <= 4096, "queue entries keep the block slot in 12 bits");

struct GemmArgs {
  GlobalTables tables;
  const __half* x;        // [M, ldx] row-major
  const uint8_t* codes;
  const float* rscale;
  const float* tail;
  void* y;                // [M, d_out]
  float* ws;              // [S, n_bands, M, 64] partial sums when S > 1
  float g0, g1;
  uint32_t M, ldx, d_out, nblocks, tail_w;
  uint32_t n_bands, S, bps;  // split count, blocks per split
  uint32_t ct_shift;         // log2 of the column tiles the wavefronts spread over (0..4)
};

// The batched kernel keeps the Golay words and the support-arrangement table in L2:
// the 33 KB they would take in LDS buy a W slice of 32 blocks per row instead of 20.
constexpr size_t kGemmImageBytes = kLdsImageBytesLean;
constexpr size_t gemm_lds_bytes() {
  return kGemmImageBytes + (size_t)kGemmRows * kGemmRowBytes + (size_t)kGemmTile * 4 + kGenericSlots * 4 + 16 +
         (size_t)kGemmRows * kGemmWStride * 2;
}
static_assert(gemm_lds_bytes() <= 160 * 1024, "GEMM workgroup state must fit one CU's LDS");

// four packed signed bytes -> four binary16 values w * s, one rounding each
__device__ __forceinline__ uint2 scaled_halves(uint32_t w, float s, float bias) {
  const uint32_t u = w ^ 0x80808080u;  // bytes + 128, unsigned
  const float f0 = fmaf((float)(u & 0xFFu), s, bias);
  const float f1 = fmaf((float)((u >> 8) & 0xFFu), s, bias);
  const float f2 = fmaf((float)((u >> 16) & 0xFFu), s, bias);
  const float f3 = fmaf((float)(u >> 24), s, bias);
  const __half2 lo = __float22half2_rn(make_float2(f0, f1)), hi = __float22half2_rn(make_float2(f2, f3));
  uint2 r;
  r.x = *reinterpret_cast<const uint32_t*>(&lo);
  r.y = *reinterpret_cast<const uint32_t*>(&hi);
  return r;
}

template <typename OutT>
__device__ __forceinline__ void store_y(void* y, size_t at, float v);
template <>
__device__ __forceinline__ void store_y<float>(void* y, size_t at, float v) {
  reinterpret_cast<float*>(y)[at] = v;
}
template <>
__device__ __forceinline__ void store_y<__half>(void* y, size_t at, float v) {
  reinterpret_cast<__half*>(y)[at] = __float2half_rn(v);
}

// P2 of the batched kernels: the wavefronts that call this draw 64-block chunks of the
// tile's queues (generic walks first, then odd, then even classes) from a shared
// counter until none is left; every block's 24 weights, multiplied by
// centroid[gain] / sqrt(16 shell) and rounded once to binary16, go to row `row`,
// columns [24 b, 24 b + 24) of the W slice.  CAP = queue capacity, WSTRIDE = binary16
// elements per W row; slot f of the tile is block b = f - row kb of row = f / kb.
template <int CAP, int WSTRIDE, typename RecordAt>
__device__ __forceinline__ void unrank_queues_to_slice(const DecodeTables& T, const uint32_t* queue, const uint32_t* gqueue,
                                                       uint32_t* ctrl, uint32_t kb, uint32_t inv_kb, float g0, float g1,
                                                       _Float16* W, RecordAt record_at) {
  const uint32_t lane = threadIdx.x & 63u;
  const uint32_t n_odd = ctrl[0], n_even = ctrl[1], n_gen = min(ctrl[2], (uint32_t)kGenericSlots);
  const uint32_t c_gen = n_gen ? 1u : 0u, c_odd = (n_odd + 63u) >> 6, c_even = (n_even + 63u) >> 6;
  for (;;) {
    uint32_t chunk = 0;
    if (lane == 0) chunk = atomicAdd(&ctrl[3], 1u);
    chunk = __shfl(chunk, 0, 64);
    if (chunk >= c_gen + c_odd + c_even) break;
    const bool from_gen = chunk < c_gen, from_odd = chunk < c_gen + c_odd;
    const uint32_t k = from_gen ? lane : (from_odd ? (chunk - c_gen) * 64u + lane : (chunk - c_gen - c_odd) * 64u + lane);
    if (k < (from_gen ? n_gen : (from_odd ? n_odd : n_even))) {
      const uint32_t entry = from_gen ? gqueue[k] : (from_odd ? queue[k] : queue[CAP - 1 - k]);
      const uint32_t f = entry & 0xFFFu, ci = (entry >> 16) & 0x1FFu;
      const uint32_t row = (f * inv_kb) >> 16, b = f - row * kb;
      const uint64_t rec = record_at(row, b);
      const uint64_t li = (rec >> 1) - 1 - T.starts[ci];
      const float g = (entry >> 25) & 1u ? g1 : g0;
      _Float16* wrow = W + (size_t)row * WSTRIDE + b * 24u;
      if (entry & kEntryOrigin) {
        uint4* dst = reinterpret_cast<uint4*>(wrow);
        dst[0] = dst[1] = dst[2] = make_uint4(0, 0, 0, 0);
      } else if (from_odd) {
        if (entry >> 31) {  // generic walk
          const DevClass c = T.cls[ci];
          const float s = c.inv_norm * g;
          auto emit = [&](int p, int v) { wrow[p] = (_Float16)((float)v * s); };
          if (c.meta & kMetaOdd) decode_odd(T, c, li, emit);
          else decode_even(T, c, li, emit);
        } else {
          const FastClass fc = T.fast[ci];
          const float s = fc.inv_norm * g, bias = -128.f * s;
          odd_codes(T, fc, li, [&](int q, uint32_t sel) {
            const uint32_t w = __builtin_amdgcn_perm(fc.tab_hi, fc.tab_lo, sel);
            *reinterpret_cast<uint2*>(wrow + 4 * q) = scaled_halves(w, s, bias);
          });
        }
      } else {
        const FastClass fc = T.fast[ci];
        const float s = fc.inv_norm * g, bias = -128.f * s;
        const uint32_t fv1 = fc.u0 >> 16;
        const uint32_t tab2_lo = fv1 << 8, tab2_hi = ((0u - fv1) & 0xFFu) << 8;
        even_codes(T, fc, li, [&](int q, uint32_t sel, uint32_t sel2) {
          const uint32_t w = __builtin_amdgcn_perm(fc.tab_hi, fc.tab_lo, sel) | __builtin_amdgcn_perm(tab2_hi, tab2_lo, sel2);
          *reinterpret_cast<uint2*>(wrow + 4 * q) = scaled_halves(w, s, bias);
        });
      }
    }
  }
}

// Wavefront grid of the MFMA phase: every wavefront owns both 32-row tiles of the band
// and one 32-column tile of the batch.  A batch of fewer than sixteen column tiles
// leaves wavefronts over; they take the same tiles on interleaved K-steps (kpart) and
// the unit's epilogue adds their sums in kpart order.
#ifdef LLVQ_PHASE_TIMING
#define LLVQ_GSTAMP(k)                                                                                  \
  do {                                                                                                  \
    if (threadIdx.x == 0 && unit == blockIdx.x && si == 0) g_phase_stamps[blockIdx.x * 8 + (k)] = wall_clock64(); \
  } while (0)
#else
#define LLVQ_GSTAMP(k) do {} while (0)
#endif

template <typename OutT>
__global__ __launch_bounds__(kWgThreads) void gemm_tiles_kernel(GemmArgs a) {
  extern __shared__ __align__(16) uint8_t smem[];
  const DecodeTables T = stage_tables<false>(smem, a.tables);
  uint8_t* raw = smem + kGemmImageBytes;
  uint32_t* queue = reinterpret_cast<uint32_t*>(raw + kGemmRows * kGemmRowBytes);
  uint32_t* gqueue = queue + kGemmTile;
  uint32_t* ctrl = gqueue + kGenericSlots;
  _Float16* W = reinterpret_cast<_Float16*>(ctrl + 4);
  const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
  const uint32_t nb = a.nblocks;
  const uint32_t n_units = a.n_bands * a.S;

  // 32-row and 32-column tiles per wavefront.  Two column tiles would halve the operand
  // traffic per MFMA, but 64 accumulator registers beside the decode phases' state spill
  // (measured: 124 instead of 196 TFLOP/s at M = 512).
  constexpr int RT = 2, CT = 1;
  const uint32_t ctn = 1u << a.ct_shift, kparts = 16u >> a.ct_shift;
  const uint32_t ctile = wave & (ctn - 1u), kpart = wave >> a.ct_shift;
  const uint32_t l32 = lane & 31u, lh = lane >> 5;
  uint32_t my_m[CT];  // the activation rows this lane feeds and receives
#pragma unroll
  for (int c = 0; c < CT; ++c) my_m[c] = (ctile * CT + c) * 32u + l32;

  // code bytes of (unit, slice) -> one register per lane
  auto prefetch = [&](uint32_t r0, uint32_t rows, uint32_t k0, uint32_t kb, uint4& pre) {
    const uint32_t row = tid / kGemmRowChunks, j = tid - row * kGemmRowChunks;
    if (row < rows && kb) {
      const size_t byte0 = ((size_t)(r0 + row) * nb + k0) * 6;
      const uint32_t off = (uint32_t)(byte0 & 15);
      const uint32_t n16 = (off + kb * 6 + 15) >> 4;
      if (j < n16) pre = reinterpret_cast<const uint4*>(a.codes + (byte0 - off))[j];
    }
  };

#ifdef LLVQ_PHASE_TIMING
  if (threadIdx.x == 0) g_phase_stamps[blockIdx.x * 8 + 7] = wall_clock64();
#endif
  for (uint32_t unit = blockIdx.x; unit < n_units; unit += gridDim.x) {
    const uint32_t band = unit / a.S, split = unit - band * a.S;
    const uint32_t r0 = band * kGemmRows, rows = min((uint32_t)kGemmRows, a.d_out - r0);
    const uint32_t kb_lo = min(nb, split * a.bps), kb_hi = min(nb, kb_lo + a.bps);
    float16_t acc[RT][CT];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
#pragma unroll
      for (int c = 0; c < CT; ++c)
#pragma unroll
        for (int j = 0; j < 16; ++j) acc[rt][c][j] = 0.f;

    uint4 pre = make_uint4(0, 0, 0, 0);
    // Units walk their slices from different starting points (a fixed function of
    // the band), so that the CUs do not all pull the same activation columns
    // through the same L2 channels at the same time.
    const uint32_t n_slices = (kb_hi - kb_lo + kGemmKb - 1) / kGemmKb;
    uint32_t sj = n_slices ? (band * 5u) % n_slices : 0u;
    if (n_slices) prefetch(r0, rows, kb_lo + sj * kGemmKb, min((uint32_t)kGemmKb, kb_hi - (kb_lo + sj * kGemmKb)), pre);
    for (uint32_t si = 0; si < n_slices; ++si) {
      const uint32_t k0 = kb_lo + sj * kGemmKb;
      const uint32_t kb = min((uint32_t)kGemmKb, kb_hi - k0);
      sj = sj + 1 == n_slices ? 0u : sj + 1;
      const uint32_t nblk = rows * kb;
      const uint32_t inv_kb = (65536u + kb - 1u) / kb;  // floor(f / kb) = (f * inv_kb) >> 16 for f < 2048, kb <= 32
      // P0
      if (tid < 4) ctrl[tid] = 0;
      if (tid < (uint32_t)(kGemmRows * kGemmRowChunks)) reinterpret_cast<uint4*>(raw)[tid] = pre;
      __syncthreads();
      LLVQ_GSTAMP(0);
      if (si + 1 < n_slices) prefetch(r0, rows, kb_lo + sj * kGemmKb, min((uint32_t)kGemmKb, kb_hi - (kb_lo + sj * kGemmKb)), pre);

      auto record_at = [&](uint32_t row, uint32_t b) -> uint64_t {
        const uint32_t off = ((((r0 + row) * nb + k0) & 7u) * 6u) & 15u;  // (6 n) mod 16 depends on n mod 8 only
        return read_record(raw, row * kGemmRowBytes + off + 6u * b);
      };

      // P1: classify and bin.  An origin block is queued: its 24 zero weights are
      // written in P2, because the W slice may still be read by the previous slice's P3 now.
      classify_and_bin<kGemmP1Blocks>(
          T, nblk, kGemmTile, queue, gqueue, ctrl,
          [&](uint32_t f) {
            const uint32_t row = (f * inv_kb) >> 16;
            return record_at(row, f - row * kb);
          },
          [](uint32_t) { return true; });
      __syncthreads();
      LLVQ_GSTAMP(1);

      // P2: unrank into the W slice
      unrank_queues_to_slice<kGemmTile, kGemmWStride>(T, queue, gqueue, ctrl, kb, inv_kb, a.g0, a.g1, W, record_at);
      LLVQ_GSTAMP(2);
      __syncthreads();
      LLVQ_GSTAMP(3);

      // P3: acc += W_slice (64 x 24 kb) * X^T (24 kb x M).  K runs in steps of 32
      // (two MFMAs of 16): lane (l32, lh) holds columns [32 p + 16 lh, +16) of its
      // row as two fragments, for W and X alike, so an activation row is read in
      // 64-byte runs.  Columns past the slice are zeroed on both sides.
      if (ctile * CT * 32u < a.M) {  // column tiles beyond the batch have nothing to add
        const uint32_t kcols = kb * 24u, psteps = (kcols + 31u) >> 5;
        const __half* xrow[CT];
        bool m_in[CT];
#pragma unroll
        for (int c = 0; c < CT; ++c) {
          xrow[c] = a.x + (size_t)k0 * 24u + (size_t)min(my_m[c], a.M - 1u) * a.ldx + lh * 16u;
          m_in[c] = my_m[c] < a.M;
        }
        const _Float16* arow = W + (size_t)l32 * kGemmWStride + lh * 16u;
        constexpr int G = CT == 1 ? 2 : 1;  // K-steps per batch of activation loads
        const half8_t zero = {0, 0, 0, 0, 0, 0, 0, 0};
        half8_t cur[G][CT][2], nxt[G][CT][2];
        auto fetch = [&](uint32_t i0, half8_t (&dst)[G][CT][2]) {  // owned K-steps i0 .. i0+G-1
#pragma unroll
          for (int g = 0; g < G; ++g)
#pragma unroll
            for (int c = 0; c < CT; ++c)
#pragma unroll
              for (int f = 0; f < 2; ++f) {
                const uint32_t p = kpart + (i0 + g) * kparts, kc = p * 32u + lh * 16u + f * 8u;
                dst[g][c][f] = (m_in[c] && kc < kcols) ? *reinterpret_cast<const half8_t*>(xrow[c] + p * 32u + f * 8u) : zero;
              }
        };
        const uint32_t n_own = kpart < psteps ? (psteps - kpart + kparts - 1u) / kparts : 0u;
        fetch(0, cur);
        for (uint32_t i0 = 0; i0 < n_own; i0 += G) {
          if (i0 + G < n_own) fetch(i0 + G, nxt);
#pragma unroll
          for (int g = 0; g < G; ++g) {
            if (i0 + g < n_own) {
              const uint32_t p = kpart + (i0 + g) * kparts;
#pragma unroll
              for (int f = 0; f < 2; ++f) {
                const bool kin = p * 32u + lh * 16u + f * 8u < kcols;
#pragma unroll
                for (int rt = 0; rt < RT; ++rt) {
                  const half8_t av = kin ? *reinterpret_cast<const half8_t*>(arow + (size_t)rt * 32 * kGemmWStride + p * 32u + f * 8u) : zero;
#pragma unroll
                  for (int c = 0; c < CT; ++c)
                    acc[rt][c] = __builtin_amdgcn_mfma_f32_32x32x16_f16(av, cur[g][c][f], acc[rt][c], 0, 0, 0);
                }
              }
            }
          }
#pragma unroll
          for (int g = 0; g < G; ++g)
#pragma unroll
            for (int c = 0; c < CT; ++c)
#pragma unroll
              for (int f = 0; f < 2; ++f) cur[g][c][f] = nxt[g][c][f];
        }
      }
      LLVQ_GSTAMP(4);
      // no barrier here: the next slice's P0/P1 touch only raw, queues and
      // counters, and its P2 starts behind two barriers every wavefront reaches
      // after leaving P3
    }

    // ---- epilogue ----
    // acc[rt][c][j] belongs to weight row r0 + rt*32 + 8 (j/4) + 4 lh + j%4 and activation row my_m[c].
    // The tail columns (f32 weights, kept out of the binary16 contraction) are
    // staged in the W area: tl[row][t] as f32 and xt[m][t] as binary16.
    const uint32_t tw = a.tail_w;
    float* tl = reinterpret_cast<float*>(W);
    __half* xt = reinterpret_cast<__half*>(tl + kGemmRows * (kDim - 1));
    static_assert((size_t)(2 * kGemmRows + kGemmMaxM) * (kDim - 1) * 2 <= (size_t)kGemmRows * kGemmWStride * 2,
                  "tail staging fits the W area");
    auto stage_tail = [&]() {  // call with every wavefront past its last read of W
      for (uint32_t o = tid; o < rows * tw; o += kWgThreads) tl[o] = a.tail[(size_t)r0 * tw + o];
      const __half* xtail = a.x + (size_t)nb * 24u;
      for (uint32_t o = tid; o < a.M * tw; o += kWgThreads) {
        const uint32_t m = o / tw, t = o - m * tw;
        xt[o] = xtail[(size_t)m * a.ldx + t];
      }
    };
    const bool vec_ok = (a.d_out & 3u) == 0;  // four consecutive rows of one activation row store as one vector
    __syncthreads();  // every wavefront is past its last read of W
    if (kparts > 1) {
      // sums of the K-step shares -> the kpart 0 wavefront of each column group, one
      // 32 x 32 tile at a time through the W area: red[kpart - 1][ctile][j4][lane]
      float4* red = reinterpret_cast<float4*>(W);
      static_assert((size_t)15 * 4 * 64 * 16 <= (size_t)kGemmRows * kGemmWStride * 2, "K-step shares fit the W area");
#pragma unroll
      for (int rt = 0; rt < RT; ++rt)
#pragma unroll
        for (int c = 0; c < CT; ++c) {
          if (kpart > 0) {
#pragma unroll
            for (int j4 = 0; j4 < 4; ++j4)
              red[(((kpart - 1u) * ctn + ctile) * 4u + j4) * 64u + lane] =
                  make_float4(acc[rt][c][4 * j4], acc[rt][c][4 * j4 + 1], acc[rt][c][4 * j4 + 2], acc[rt][c][4 * j4 + 3]);
          }
          __syncthreads();
          if (kpart == 0) {
            for (uint32_t kp = 1; kp < kparts; ++kp)
#pragma unroll
              for (int j4 = 0; j4 < 4; ++j4) {
                const float4 v = red[(((kp - 1u) * ctn + ctile) * 4u + j4) * 64u + lane];
                acc[rt][c][4 * j4] += v.x;
                acc[rt][c][4 * j4 + 1] += v.y;
                acc[rt][c][4 * j4 + 2] += v.z;
                acc[rt][c][4 * j4 + 3] += v.w;
              }
          }
          __syncthreads();
        }
    }
    if (a.S > 1) {
      // gemm_reduce_kernel finishes these rows.  The workspace is [split][band][m][64]:
      // a unit's partial sums are one contiguous piece, and rows past the end of the
      // last band are written but never read.
#pragma unroll
      for (int c = 0; c < CT; ++c) {
        if (kpart == 0 && my_m[c] < a.M) {
          float* dst = a.ws + (((size_t)split * a.n_bands + band) * a.M + my_m[c]) * kGemmRows;
#pragma unroll
          for (int rt = 0; rt < RT; ++rt)
#pragma unroll
            for (int j4 = 0; j4 < 4; ++j4)
              *reinterpret_cast<float4*>(dst + rt * 32u + 8u * j4 + 4u * lh) =
                  make_float4(acc[rt][c][4 * j4], acc[rt][c][4 * j4 + 1], acc[rt][c][4 * j4 + 2], acc[rt][c][4 * j4 + 3]);
        }
      }
    } else {
      if (tw) stage_tail();
      __syncthreads();
#pragma unroll
      for (int c = 0; c < CT; ++c) {
        if (kpart == 0 && my_m[c] < a.M) {
#pragma unroll
          for (int rt = 0; rt < RT; ++rt)
#pragma unroll
            for (int j4 = 0; j4 < 4; ++j4) {
              const uint32_t row = rt * 32u + 8u * j4 + 4u * lh;
              float v[4];
#pragma unroll
              for (int i = 0; i < 4; ++i) {
                const uint32_t r = min(row + i, rows - 1u);
                float ts = 0.f;
                for (uint32_t t = 0; t < tw; ++t) ts = fmaf(tl[r * tw + t], __half2float(xt[my_m[c] * tw + t]), ts);
                v[i] = fmaf(acc[rt][c][4 * j4 + i], a.rscale[r0 + r], ts);
              }
              const size_t at = (size_t)my_m[c] * a.d_out + r0 + row;
              if (vec_ok && row + 3 < rows) {
                if constexpr (sizeof(OutT) == 4) {
                  *reinterpret_cast<float4*>(reinterpret_cast<float*>(a.y) + at) = make_float4(v[0], v[1], v[2], v[3]);
                } else {
                  const __half2 lo = __float22half2_rn(make_float2(v[0], v[1])), hi = __float22half2_rn(make_float2(v[2], v[3]));
                  uint2 pk;
                  pk.x = *reinterpret_cast<const uint32_t*>(&lo);
                  pk.y = *reinterpret_cast<const uint32_t*>(&hi);
                  *reinterpret_cast<uint2*>(reinterpret_cast<__half*>(a.y) + at) = pk;
                }
              } else {
#pragma unroll
                for (int i = 0; i < 4; ++i)
                  if (row + i < rows) store_y<OutT>(a.y, at + i, v[i]);
              }
            }
        }
      }
    }
#ifdef LLVQ_PHASE_TIMING
    if (threadIdx.x == 0 && unit == blockIdx.x) g_phase_stamps[blockIdx.x * 8 + 5] = wall_clock64();
#endif
    __syncthreads();  // W, raw and counters are reused by the next unit
  }
}

// Second pass of a split launch: y[m][r] = (sum over splits, in split order, of the
// partial sums) * rscale[r] + tail[r] . x_tail[m].  One workgroup per (band, 16
// activation rows), one lane per four consecutive weight rows of one activation row;
// the band's tail weights and the activation tails are staged in LDS once, and the
// partial sums are read with all their loads in flight (eight splits at a time).
struct GemmReduceArgs {
  const float* ws;  // [S, n_bands, M, 64]
  const __half* x;  // [M, ldx]
  const float* rscale;
  const float* tail;
  void* y;
  uint32_t M, ldx, d_out, nblocks, tail_w, S, n_bands;
};

constexpr int kReduceRowsM = 16;  // activation rows per workgroup

template <typename OutT>
__global__ __launch_bounds__(256) void gemm_reduce_kernel(GemmReduceArgs a) {
  __shared__ float tl[kGemmRows * kDim];            // [row][pitch], pitch odd
  __shared__ float xt[kReduceRowsM * (kDim - 1)];   // [m][tail_w]
  const uint32_t mchunks = (a.M + kReduceRowsM - 1) / kReduceRowsM;
  const uint32_t band = blockIdx.x / mchunks, mc = blockIdx.x - band * mchunks;
  const uint32_t r0 = band * kGemmRows, rows = min((uint32_t)kGemmRows, a.d_out - r0);
  const uint32_t tw = a.tail_w, pitch = tw | 1u;
  const uint32_t tid = threadIdx.x, quad = tid & 15u, ml = tid >> 4;
  const uint32_t m = mc * kReduceRowsM + ml, row = quad * 4u;
  for (uint32_t o = tid; o < rows * tw; o += 256) {
    const uint32_t r = o / tw, t = o - r * tw;
    tl[r * pitch + t] = a.tail[(size_t)r0 * tw + o];
  }
  for (uint32_t o = tid; o < kReduceRowsM * tw; o += 256) {
    const uint32_t mm = mc * kReduceRowsM + o / tw, t = o % tw;
    xt[o] = mm < a.M ? __half2float(a.x[(size_t)mm * a.ldx + (size_t)a.nblocks * 24u + t]) : 0.f;
  }
  __syncthreads();
  if (m >= a.M || row >= rows) return;
  const size_t sstride = (size_t)a.n_bands * a.M * kGemmRows;
  const float* src = a.ws + ((size_t)band * a.M + m) * kGemmRows + row;
  float sum[4] = {0.f, 0.f, 0.f, 0.f};
  for (uint32_t s0 = 0; s0 < a.S; s0 += 8) {
    float4 p[8];
#pragma unroll
    for (int u = 0; u < 8; ++u)
      p[u] = s0 + u < a.S ? *reinterpret_cast<const float4*>(src + (size_t)(s0 + u) * sstride) : make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
    for (int u = 0; u < 8; ++u)
      if (s0 + u < a.S) {
        sum[0] += p[u].x;
        sum[1] += p[u].y;
        sum[2] += p[u].z;
        sum[3] += p[u].w;
      }
  }
  float v[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const uint32_t r = min(row + i, rows - 1u);
    float ts = 0.f;
    for (uint32_t t = 0; t < tw; ++t) ts = fmaf(tl[r * pitch + t], xt[ml * tw + t], ts);
    v[i] = fmaf(sum[i], a.rscale[r0 + r], ts);
  }
  const size_t at = (size_t)m * a.d_out + r0 + row;
  if ((a.d_out & 3u) == 0 && row + 3 < rows) {
    if constexpr (sizeof(OutT) == 4) {
      *reinterpret_cast<float4*>(reinterpret_cast<float*>(a.y) + at) = make_float4(v[0], v[1], v[2], v[3]);
    } else {
      const __half2 lo = __float22half2_rn(make_float2(v[0], v[1])), hi = __float22half2_rn(make_float2(v[2], v[3]));
      uint2 pk;
      pk.x = *reinterpret_cast<const uint32_t*>(&lo);
      pk.y = *reinterpret_cast<const uint32_t*>(&hi);
      *reinterpret_cast<uint2*>(reinterpret_cast<__half*>(a.y) + at) = pk;
    }
  } else {
#pragma unroll
    for (int i = 0; i < 4; ++i)
      if (row + i < rows) store_y<OutT>(a.y, at + i, v[i]);
  }
}

}  // namespace llvq
