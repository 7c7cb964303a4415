// Fused dequant-GEMM for batched activations: Y[M, d_out] = X[M, d_in] W^T with
// W unranked on the fly and contracted on the matrix cores (f16 operands, f32
// accumulate).  Included by llvq_hip.hip after the GEMV kernel, whose helpers
// (table staging, record reads, queues) it shares.
//
// The reference runs a batch as a row loop over its GEMV
// (llvq-llm/src/model.rs:521-529); this kernel decodes every block once for
// all M rows instead.
//
// The work is cut into K-slices: 16 blocks per row of a band of 64 weight rows (384
// columns = 12 K-steps of 32, 1024 blocks).  The launch's slices, numbered band by band,
// are shared out evenly over one persistent 1024-lane workgroup per CU.  A workgroup's
// 16 wavefronts split into two roles, and the unranking and the contraction of
// consecutive slices run at the same time:
//   producers (the first 8 or 12) slice g: code bytes -> LDS (loads issued two
//                                slices ahead), classify and bin the blocks (odd /
//                                even / generic queues), unrank; every block writes
//                                its 24 weights, already multiplied by
//                                centroid[gain] / sqrt(16 shell) and rounded once to
//                                binary16, into W[g & 1] in LDS;
//   consumers (the other 8 or 4) v_mfma_f32_32x32x16_f16 over slice g - 1 from
//                                W[(g - 1) & 1]: every consumer owns all 64 weight
//                                rows x 64 activation rows (64 accumulator
//                                registers, live across a band's slices), A
//                                fragments from LDS, B fragments from global
//                                memory / L2 through a buffer descriptor, each
//                                16-byte piece in flight for most of two K-steps.
// The unranking is integer and f64 VALU work and the contraction runs on the
// matrix cores, so the two overlap on every SIMD.  Because the roles are separate
// branches of one kernel, the accumulators and the decode state are never live
// together: both fit the 128 registers a 1024-lane workgroup leaves each
// wavefront (one wavefront doing both in turn spills beyond 32 accumulators).
// A narrow batch leaves the matrix cores little to do, and 12 wavefronts unrank.
//
// A stage ends in one workgroup barrier.  In stage g the producers unrank slice g
// and then classify slice g + 1 (three sets of code bytes and counters, two sets of
// queues), the consumers multiply slice g - 1; so the W buffer written in stage g is
// complete before it is read in stage g + 1 and is not overwritten before stage g + 2.
//
// A band one workgroup walked alone, by consumers that own a 64-row tile each, is finished
// where its sums are: row scale, the f32 tail columns (on the matrix cores, f32 operands),
// the store to y.  Every other sum goes to the workspace [band][piece][K-share][m][64]: a
// band whose slices fell to several workgroups has one piece from each, and consumers
// left over by a batch of few 64-row tiles take the same tile on interleaved K-steps.
// gemm_reduce_kernel adds those partial sums in that fixed order and applies row scale
// and the tail, so the result does not depend on scheduling.
#pragma once

#include "gemm_share.h"

namespace llvq {

typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float float16_t __attribute__((ext_vector_type(16)));

constexpr int kGemmRows = 64;    // weight rows of a band
constexpr int kGemmMaxM = 512;   // activation rows per launch (eight consumers x 64)

// The batched kernel keeps the Golay words, the support-arrangement table and the class
// lookup table in L2: the 37 KB they would take in LDS buy the second W buffer and the
// buffers that let classification and unranking of consecutive slices share a stage.
constexpr size_t kGemmImageBytes = kLdsImageBytesLeanest;

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

// The producers' unranking: the wavefronts that call this draw 64-block chunks of the
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
      const uint64_t li = (rec >> 1) - T.starts[ci];
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

constexpr int kGemmKb = 16;                                   // blocks per row and K-slice
constexpr int kGemmTile = kGemmRows * kGemmKb;                // blocks per K-slice
constexpr int kGemmMinProducers = 512;                        // lanes of the producer role, at least
constexpr int kGemmRowChunks = (kGemmKb * 6 + 14 + 15) / 16;  // 16-byte units holding one row's code bytes at any even alignment
constexpr int kGemmRowBytes = kGemmRowChunks * 16;
constexpr int kGemmWStride = kGemmKb * 24 + 8;                // binary16 elements per W row in LDS
constexpr int kGemmColTile = 64;                              // activation rows per consumer
static_assert(kGemmRows * kGemmRowChunks <= kGemmMinProducers, "one 16-byte load per producer lane covers a slice's code bytes");
static_assert(kGemmMaxM <= (kWgThreads - kGemmMinProducers) / 64 * kGemmColTile, "the consumers cover a launch's activation rows");

// table image | code bytes of three slices | two block queues | two generic queues | three counter sets | two W buffers
constexpr size_t gemm_lds_bytes() {
  return kGemmImageBytes + 3 * (size_t)kGemmRows * kGemmRowBytes + 2 * (size_t)kGemmTile * 4 + 2 * kGenericSlots * 4 + 96 +
         2 * (size_t)kGemmRows * kGemmWStride * 2;
}
static_assert(gemm_lds_bytes() <= 160 * 1024, "GEMM workgroup state must fit one CU's LDS");

__device__ __forceinline__ void wg_barrier() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
}

// The consumers' side of a barrier.  They only read LDS and have nothing to publish, so the
// barrier must not wait for their global loads: those stay in flight across it.
__device__ __forceinline__ void consumer_barrier() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

// The activations as the consumers read them: xt[p][m][32] holds columns [32 p, 32 p + 32)
// of activation row m, so the 64 rows x 64 bytes a consumer needs for one K-step are one
// contiguous 4 KB run (in x they are 64 half cache lines, 2 ldx bytes apart).  Columns from
// `kcols` on (the tail columns, which the f32 epilogue handles) and rows from M on are
// zero, which leaves the consumers' loads unconditional.  One lane per 16 bytes.
__global__ __launch_bounds__(256) void tile_activations_kernel(const __half* x, uint32_t M, uint32_t ldx, uint32_t kcols,
                                                               uint32_t m_pad, uint32_t n_steps, uint4* xt) {
  const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= (size_t)n_steps * m_pad * 4) return;
  const uint32_t c = (uint32_t)(idx & 3), m = (uint32_t)((idx >> 2) % m_pad), p = (uint32_t)((idx >> 2) / m_pad);
  const uint32_t col = p * 32u + c * 8u;  // kcols is a multiple of 8: a 16-byte piece is all inside or all outside
  xt[idx] = (m < M && col < kcols) ? *reinterpret_cast<const uint4*>(x + (size_t)m * ldx + col) : make_uint4(0, 0, 0, 0);
}

// The workgroups share the launch's slices out evenly (gemm_share.h): whole bands first, where there
// are at least as many bands as workgroups, then consecutive slices of the bands left over, so that
// the chip is busy whatever the matrix's shape.  A band whose slices fall to several workgroups gets
// one partial sum from each ("pieces", numbered in workgroup order).  Both roles step through the
// same slices, the consumers one stage behind.
struct SliceWalk {
  uint32_t t;                   // slices this workgroup walked before this one; valid below its slice count
  uint32_t band, j;             // band, and the slice's place in it: blocks [16 j, 16 j + 16) of every row
  uint32_t run_lo, run_len, si; // this workgroup's slices of the band, and how many of them are done
  uint32_t mat, r0, rows;       // the band's matrix, its first row there, its row count
  uint32_t piece;               // which of the band's partial sums this workgroup's run of slices feeds
};

// Stage timestamps of tuning builds (-DLLVQ_PHASE_TIMING): lane 0 of EVERY wavefront stores the realtime counter at
// the boundaries of the workgroup's stage kGemmStampStage.  Producers: 0 stage begins, 1 its share of the slice
// unranked, 2 its share of the next slice classified, 3 through the barrier.  Consumers: 0 stage begins, 1 its K-steps
// multiplied, 3 through the barrier.
#ifdef LLVQ_PHASE_TIMING
constexpr uint32_t kGemmStampStage = 3;
__device__ unsigned long long g_gemm_stamps[1024 * 16 * 4];
#define LLVQ_GSTAMP(k)                                                                                                 \
  do {                                                                                                                 \
    if (lane == 0 && stage_no == kGemmStampStage) g_gemm_stamps[((size_t)blockIdx.x * 16 + wave) * 4 + (k)] = wall_clock64(); \
  } while (0)
#else
#define LLVQ_GSTAMP(k) do {} while (0)
#endif

// A launch covers up to four matrices that share their activations (q/k/v, gate/up): their
// bands are numbered through, matrix i owning bands [band_begin, next band_begin).
constexpr int kGemmMaxGroup = 4;
struct GemmMat {
  const uint8_t* codes;
  const float* rscale;  // d_out row scales and 64 floats of slack
  const float* tail;
  void* y;
  float g0, g1;
  uint32_t d_out, band_begin;
};
struct GemmArgs {
  GlobalTables tables;
  const __half* xt;       // [n_steps, m_pad, 32]: tile_activations_kernel's output
  float* ws;              // [n_bands - ws_band0, max_pieces, kparts, M, 64] partial sums
  const __half* x;        // [M, ldx] the activations as the caller gave them (the tail columns are read from here)
  GemmMat mat[kGemmMaxGroup];
  uint32_t n_mats;
  uint32_t y_f32;            // output type: binary32, else binary16
  uint32_t ldx, tail_w;
  uint32_t M, m_pad, nblocks;
  uint32_t n_bands;          // bands of all matrices
  uint32_t spb;              // slices per band
  GemmShare share;           // which workgroup walks what (gemm_share.h)
  uint32_t ws_band0;         // the first band with a place in the workspace
  uint32_t ct_shift;         // log2 of the 64-row activation tiles the consumers spread over
};


// PW = producer wavefronts (8 or 12); the other 16 - PW consume.
template <int PW>
__global__ __launch_bounds__(kWgThreads) void gemm_tiles_kernel(GemmArgs a) {
  constexpr int kProducers = PW * 64, kConsumers = 16 - PW;
  static_assert(kProducers >= kGemmMinProducers && (kConsumers == 8 || kConsumers == 4), "roles");
  extern __shared__ __align__(16) uint8_t smem[];
  const DecodeTables T = stage_tables<false, false>(smem, a.tables);
  uint8_t* raw0 = smem + kGemmImageBytes;
  constexpr uint32_t kRawBuf = kGemmRows * kGemmRowBytes;
  uint32_t* queue0 = reinterpret_cast<uint32_t*>(raw0 + 3 * kRawBuf);
  uint32_t* gqueue0 = queue0 + 2 * kGemmTile;
  uint32_t* ctrl0 = gqueue0 + 2 * kGenericSlots;  // three sets of eight counters: queue lengths, unrank ticket, classify ticket
  _Float16* W0 = reinterpret_cast<_Float16*>(ctrl0 + 24);
  constexpr uint32_t kWBuf = kGemmRows * kGemmWStride;  // elements per W buffer
  const uint32_t tid = threadIdx.x, lane = tid & 63u;
  const uint32_t wave = (uint32_t)__builtin_amdgcn_readfirstlane((int)(tid >> 6));
  const uint32_t nb = a.nblocks;
  const uint32_t n_mine = gemm_slices_of(a.share, a.spb, blockIdx.x);  // slices this workgroup walks

  auto enter_band = [&](SliceWalk& w) {
    w.mat = 0;
#pragma unroll
    for (uint32_t k = 1; k < (uint32_t)kGemmMaxGroup; ++k)
      if (k < a.n_mats && w.band >= a.mat[k].band_begin) w.mat = k;
    w.r0 = (w.band - a.mat[w.mat].band_begin) * kGemmRows;
    w.rows = min((uint32_t)kGemmRows, a.mat[w.mat].d_out - w.r0);
  };
  // A workgroup's slices of one band are walked from a band-dependent starting point, round the
  // run: workgroups that hold the same slices of different bands then do not all pull the same
  // activation columns through the same L2 channels at the same time.
  auto enter_run = [&](SliceWalk& w) {
    const GemmRun r = gemm_run_at(a.share, a.spb, blockIdx.x, w.t);
    w.band = r.band;
    w.run_lo = r.lo;
    w.run_len = r.len;
    w.piece = r.piece;
    w.si = 0;
    w.j = w.run_lo + (w.band * 5u) % w.run_len;
    enter_band(w);
  };
  auto start_walk = [&](SliceWalk& w) {
    w.t = 0;
    enter_run(w);
  };
  auto advance = [&](SliceWalk& w) {
    ++w.t;
    if (++w.si == w.run_len) {
      if (w.t < n_mine) enter_run(w);
    } else {
      w.j = w.j + 1 == w.run_lo + w.run_len ? w.run_lo : w.j + 1;
    }
  };
  auto live = [&](const SliceWalk& w) { return w.t < n_mine; };
  auto slice_blocks = [&](const SliceWalk& w) { return min((uint32_t)kGemmKb, nb - w.j * kGemmKb); };

  // Both W buffers start as zeros: a slice shorter than 16 blocks per row leaves columns the
  // consumers still multiply (by zero activations), which must therefore be finite.
  for (uint32_t o = tid; o < 2 * kWBuf / 8; o += kWgThreads) reinterpret_cast<uint4*>(W0)[o] = make_uint4(0, 0, 0, 0);

  if (wave < (uint32_t)PW) {
    // ---------------- producers ----------------
    // Stage g, one barrier at its end: code bytes of slice g + 2 -> LDS (loaded a stage earlier),
    // loads of slice g + 3 issued, unranking of slice g, then classification of slice g + 1.
    // A wavefront that runs out of chunks to unrank goes on to its share of the next slice's
    // classification, whose dependent table reads then overlap the others' arithmetic.
    // Buffers: code bytes and counters of slice s in set s mod 3, queues and W in set s mod 2.
    auto prefetch = [&](const SliceWalk& w, uint4& pre) {
      if (!live(w)) return;
      const uint32_t k0 = w.j * kGemmKb, kb = slice_blocks(w);
      // Unconditional: a lane past the band's rows or the row's units repeats the last ones (what it
      // stores is never read).  A guarded load is merged with the register's old value at once, and
      // that merge waits for the load, which is meant to stay in flight for a stage.
      const uint32_t row_raw = tid / kGemmRowChunks, row = min(row_raw, w.rows - 1u), j = tid - row_raw * kGemmRowChunks;
      const size_t byte0 = ((size_t)(w.r0 + row) * nb + k0) * 6;
      const uint32_t off = (uint32_t)(byte0 & 15);
      const uint32_t n16 = (off + kb * 6 + 15) >> 4;
      pre = reinterpret_cast<const uint4*>(a.mat[w.mat].codes + (byte0 - off))[min(j, n16 - 1u)];
    };
    auto stage_raw = [&](uint32_t set, const uint4& pre) {
      if (tid < 8) ctrl0[set * 8 + tid] = 0;
      if (tid < (uint32_t)(kGemmRows * kGemmRowChunks)) reinterpret_cast<uint4*>(raw0 + set * kRawBuf)[tid] = pre;
    };
    struct SliceView {  // what the phases of one slice need
      uint32_t k0, kb, r0, nblk, inv_kb, set3, set2;
      float g0, g1;
    };
    auto view = [&](const SliceWalk& w, uint32_t s) {
      SliceView v;
      v.k0 = w.j * kGemmKb;
      v.kb = slice_blocks(w);
      v.r0 = w.r0;
      v.nblk = w.rows * v.kb;
      v.inv_kb = (65536u + v.kb - 1u) / v.kb;  // floor(f / kb) = (f * inv_kb) >> 16 for f < 2048, kb <= 32
      v.set3 = s % 3u;
      v.set2 = s & 1u;
      v.g0 = a.mat[w.mat].g0;
      v.g1 = a.mat[w.mat].g1;
      return v;
    };
    auto classify = [&](const SliceView& v) {  // P1.  An origin block is queued like any other: its 24 zero weights must be written.
      const uint8_t* raw = raw0 + v.set3 * kRawBuf;
      uint32_t* ctrl = ctrl0 + v.set3 * 8;
      auto record = [&](uint32_t f) {
        const uint32_t row = (f * v.inv_kb) >> 16, b = f - row * v.kb;
        const uint32_t off = ((((v.r0 + row) * nb + v.k0) & 7u) * 6u) & 15u;  // (6 n) mod 16 depends on n mod 8 only
        return read_record(raw, row * kGemmRowBytes + off + 6u * b);
      };
      auto origin = [](uint32_t) { return true; };
      uint32_t* queue = queue0 + v.set2 * kGemmTile;
      uint32_t* gqueue = gqueue0 + v.set2 * kGenericSlots;
      if constexpr (kGemmTile % kProducers == 0) {
        // the slice's blocks divide evenly over the producers, and so do its sixteen chunks to unrank
        classify_and_bin<kGemmTile / kProducers, kProducers>(T, v.nblk, kGemmTile, queue, gqueue, ctrl, record, origin);
      } else {
        // 64 blocks at a time, handed out by a counter: the wavefronts that drew fewer chunks to
        // unrank arrive first and take more of this, so the stage ends for all at about the same time
        for (;;) {
          uint32_t unit = 0;
          if (lane == 0) unit = atomicAdd(&ctrl[4], 1u);
          unit = (uint32_t)__builtin_amdgcn_readfirstlane((int)unit);
          if (unit * 64u >= v.nblk) break;
          classify_and_bin<1, 64>(T, v.nblk, kGemmTile, queue, gqueue, ctrl, record, origin, unit * 64u + lane);
        }
      }
    };
    auto unrank = [&](const SliceView& v) {  // P2
      const uint8_t* raw = raw0 + v.set3 * kRawBuf;
      unrank_queues_to_slice<kGemmTile, kGemmWStride>(
          T, queue0 + v.set2 * kGemmTile, gqueue0 + v.set2 * kGenericSlots, ctrl0 + v.set3 * 8, v.kb, v.inv_kb, v.g0, v.g1,
          W0 + v.set2 * kWBuf, [&](uint32_t row, uint32_t b) -> uint64_t {
            const uint32_t off = ((((v.r0 + row) * nb + v.k0) & 7u) * 6u) & 15u;
            return read_record(raw, row * kGemmRowBytes + off + 6u * b);
          });
    };
    SliceWalk w0, w1, w2, w3;  // slices g, g + 1, g + 2, g + 3
    start_walk(w0);
    w1 = w0;
    advance(w1);
    w2 = w1;
    if (live(w2)) advance(w2);
    w3 = w2;
    if (live(w3)) advance(w3);
    uint4 pre = make_uint4(0, 0, 0, 0);
    prefetch(w0, pre);
    stage_raw(0, pre);
    prefetch(w1, pre);
    wg_barrier();  // slice 0's code bytes and the table image are in LDS
    if (live(w1)) stage_raw(1, pre);
    prefetch(w2, pre);
    classify(view(w0, 0));
    wg_barrier();
    uint32_t g = 0;
#ifdef LLVQ_PHASE_TIMING
    uint32_t stage_no = 0;
#endif
    while (live(w0)) {
#ifdef LLVQ_PHASE_TIMING
      ++stage_no;
#endif
      LLVQ_GSTAMP(0);
      if (live(w2)) stage_raw((g + 2u) % 3u, pre);
      prefetch(w3, pre);
      unrank(view(w0, g));
      LLVQ_GSTAMP(1);
      if (live(w1)) classify(view(w1, g + 1u));
      LLVQ_GSTAMP(2);
      wg_barrier();
      LLVQ_GSTAMP(3);
      ++g;
      w0 = w1;
      w1 = w2;
      w2 = w3;
      if (live(w3)) advance(w3);
    }
    wg_barrier();  // the consumers' last stage
  } else {
    // ---------------- consumers ----------------
    // Consumer c owns activation rows [64 ctile, +64) on the K-steps p = kpart (mod kparts) of
    // every slice: 12 / kparts steps, whatever the slice's length (past a short last slice's end
    // the activations are zero and the W buffer holds finite leftovers).  The loop is
    // branch-free, and the B fragments of two K-steps are in flight at any time, across
    // barriers and from one slice into the next: step i of the sequence lives in ring slot i mod 2.
    const uint32_t c = wave - (uint32_t)PW;
    const uint32_t ctn = 1u << a.ct_shift, kparts = (uint32_t)kConsumers >> a.ct_shift;
    const uint32_t ctile = c & (ctn - 1u), kpart = c >> a.ct_shift;
    const uint32_t m0 = ctile * kGemmColTile;
    const bool tile_live = m0 < a.M;  // a consumer past the batch's last tile multiplies that tile again and stores nothing
    // K-step p of the matrix: 32 binary16 values per activation row, rows 64 bytes apart.  The loads go through a
    // buffer descriptor over the tiled copy: a 32-bit lane offset in a vector register, the K-step's offset (the same
    // in every lane) in a scalar one, the place inside the step in the instruction.  No 64-bit address arithmetic, and
    // the loads are counted in order (vmcnt), which generic-pointer loads are not: with those every wait drains them all.
    // This lane's byte offset in a K-step of the tiled copy, from a lane number asked for on the spot: it is worked
    // out again at every stage's start and behind every epilogue, because kept alive through an epilogue it would be
    // a register the epilogue does not have.
    auto lane_offset = [&]() {
      uint32_t ln;
      asm volatile("v_mbcnt_lo_u32_b32 %0, -1, 0\n\tv_mbcnt_hi_u32_b32 %0, -1, %0" : "=v"(ln));
      return (min(m0, a.m_pad - kGemmColTile) + (ln & 31u)) * 64u + (ln >> 5) * 32u;
    };
    const uint32_t step_bytes = a.m_pad * 64u;
    const uint32_t own_bytes = kparts * step_bytes;  // between two of this consumer's K-steps
    const uint32_t n_own = (uint32_t)(kGemmKb * 24 / 32) / kparts;  // 12, 6 or 3 K-steps
    const __amdgpu_buffer_rsrc_t xt_rsrc = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<__half*>(a.xt), 0, a.spb * (uint32_t)(kGemmKb * 24 / 32) * step_bytes, 0x00020000);
    auto slice_base = [&](const SliceWalk& w) {  // twelve K-steps per slice; byte offset of this consumer's first
      return (w.j * (uint32_t)(kGemmKb * 24 / 32) + kpart) * step_bytes;
    };
    auto piece = [&](uint32_t lane_off, uint32_t step_off, int ct, int f) {
      typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
      const u32x4 v = __builtin_amdgcn_raw_buffer_load_b128(xt_rsrc, (int)lane_off,
                                                            __builtin_amdgcn_readfirstlane((int)step_off) + (ct * 32 * 64 + f * 16), 0);
      return __builtin_bit_cast(half8_t, v);
    };
    // B fragments of two K-steps: slot s holds the steps of parity s, as four 16-byte pieces [column half][K half]
    half8_t ring[2][2][2];
    auto fetch = [&](uint32_t lane_off, uint32_t step_off, half8_t (&dst)[2][2]) {
#pragma unroll
      for (int f = 0; f < 2; ++f)
#pragma unroll
        for (int ct = 0; ct < 2; ++ct) dst[ct][f] = piece(lane_off, step_off, ct, f);
    };

    SliceWalk w;
    start_walk(w);
    uint32_t xs = slice_base(w);
    {
      const uint32_t lane_off = lane_offset();
      fetch(lane_off, xs, ring[0]);
      fetch(lane_off, xs + own_bytes, ring[1]);
    }

    consumer_barrier();  // the table image (unused here) and slice 0's code bytes
    consumer_barrier();  // slice 0 classified
    consumer_barrier();  // stage 0: slice 0 unranked, nothing to multiply yet

    uint32_t buf = 0;
    float16_t acc[2][2];
    auto clear_acc = [&]() {
#pragma unroll
      for (int rt = 0; rt < 2; ++rt)
#pragma unroll
        for (int ct = 0; ct < 2; ++ct)
#pragma unroll
          for (int j = 0; j < 16; ++j) acc[rt][ct][j] = 0.f;
    };
    clear_acc();
#ifdef LLVQ_PHASE_TIMING
    uint32_t stage_no = 1;
#endif
    while (live(w)) {
#ifdef LLVQ_PHASE_TIMING
      ++stage_no;
#endif
      LLVQ_GSTAMP(0);
      const bool last_of_unit = w.si + 1 == w.run_len;  // the band ends, or this workgroup's share of it
      // The loads run ahead into the unit's next slice.  At the unit's end they re-read this
      // slice (the ring starts afresh behind the epilogue, which needs the registers).
      // (the slice after this one is worked out here and again at the stage's end: kept, its ten fields would be
      // live through the products, and this kernel has no register to spare)
      uint32_t xs_next = xs;
      if (!last_of_unit) {
        SliceWalk nx = w;
        advance(nx);
        xs_next = slice_base(nx);
      }
      const uint8_t* wbuf = reinterpret_cast<const uint8_t*>(W0 + buf * kWBuf);
      const uint32_t lane_off = lane_offset();
      uint32_t a_lane;  // this lane's byte offset in a W buffer, per stage for the same reason
      {
        uint32_t ln;
        asm volatile("v_mbcnt_lo_u32_b32 %0, -1, 0\n\tv_mbcnt_hi_u32_b32 %0, -1, %0" : "=v"(ln));
        a_lane = ((ln & 31u) * kGemmWStride + (ln >> 5) * 16u + kpart * 32u) * 2u;
      }
      auto step_src = [&](uint32_t i) { return i < n_own ? xs + i * own_bytes : xs_next + (i - n_own) * own_bytes; };
      // K-step k from its slot; every 16-byte piece of the slot is asked for again, for the step two on, as soon as
      // the products that read it are issued: a piece is in flight for most of two K-steps
      auto multiply = [&](uint32_t k, half8_t (&b)[2][2]) {
        const uint8_t* ap = wbuf + a_lane + k * kparts * 64u;
        const uint32_t nx = step_src(k + 2);
#pragma unroll
        for (int f = 0; f < 2; ++f) {
#pragma unroll
          for (int rt = 0; rt < 2; ++rt) {
            const half8_t av = *reinterpret_cast<const half8_t*>(ap + rt * 32 * kGemmWStride * 2 + f * 16);
            acc[rt][0] = __builtin_amdgcn_mfma_f32_32x32x16_f16(av, b[0][f], acc[rt][0], 0, 0, 0);
            acc[rt][1] = __builtin_amdgcn_mfma_f32_32x32x16_f16(av, b[1][f], acc[rt][1], 0, 0, 0);
          }
#pragma unroll
          for (int ct = 0; ct < 2; ++ct) b[ct][f] = piece(lane_off, nx, ct, f);
        }
      };
      uint32_t i = 0;
      for (; i + 1 < n_own; i += 2) {
        multiply(i, ring[0]);
        multiply(i + 1, ring[1]);
      }
      if (i < n_own) {  // an odd count (three K-steps): the slots change places
        multiply(i, ring[0]);
#pragma unroll
        for (int ct = 0; ct < 2; ++ct)
#pragma unroll
          for (int f = 0; f < 2; ++f) {
            const half8_t t = ring[0][ct][f];
            ring[0][ct][f] = ring[1][ct][f];
            ring[1][ct][f] = t;
          }
      }
      LLVQ_GSTAMP(1);
      consumer_barrier();
      LLVQ_GSTAMP(3);

      const SliceWalk done = w;
      advance(w);
      xs = slice_base(w);  // past the last slice: an address that is not read
      buf ^= 1u;
      if (last_of_unit) {
        // the unit's sums: acc[rt][ct][j] belongs to weight row r0 + 32 rt + 8 (j / 4) + 4 lh + j % 4
        // and activation row m0 + 32 ct + l32
        if (tile_live) {
          // this lane's activation row and its place in a 64-row result, worked out here: offsets kept
          // from the kernel's start would cost registers through every stage
          uint32_t ln;  // this lane's number, asked for here
          asm volatile("v_mbcnt_lo_u32_b32 %0, -1, 0\n\tv_mbcnt_hi_u32_b32 %0, -1, %0" : "=v"(ln));
          const uint32_t lane_l = ln & 31u, lane_h = ln >> 5, lane_m = m0 + lane_l, lane_r = 4u * lane_h;
          if (done.band >= a.ws_band0) {
            // one of several partial sums of its band: to the workspace
#pragma unroll
            for (int ct = 0; ct < 2; ++ct) {
              const uint32_t my_m = lane_m + 32u * ct;
              if (my_m < a.M) {
                float* dst = a.ws + ((((size_t)(done.band - a.ws_band0) * a.share.max_pieces + done.piece) * kparts + kpart) * a.M + my_m) * kGemmRows;
#pragma unroll
                for (int rt = 0; rt < 2; ++rt)
#pragma unroll
                  for (int j4 = 0; j4 < 4; ++j4)
                    *reinterpret_cast<float4*>(dst + rt * 32u + 8u * j4 + lane_r) =
                        make_float4(acc[rt][ct][4 * j4], acc[rt][ct][4 * j4 + 1], acc[rt][ct][4 * j4 + 2], acc[rt][ct][4 * j4 + 3]);
              }
            }
          } else {
            // the band's only sums (walked alone, and this consumer owns its tile's every K-step): finished here
            const GemmMat& mt = a.mat[done.mat];
            // row scale, four rows at a time (past a short last band's rows the array has 64 floats of slack)
#pragma unroll
            for (int rt = 0; rt < 2; ++rt) {
#pragma unroll
              for (int j4 = 0; j4 < 4; ++j4) {
                const float4 rs = *reinterpret_cast<const float4*>(mt.rscale + done.r0 + 32u * rt + 8u * j4 + lane_r);
#pragma unroll
                for (int ct = 0; ct < 2; ++ct) {
                  acc[rt][ct][4 * j4] *= rs.x;
                  acc[rt][ct][4 * j4 + 1] *= rs.y;
                  acc[rt][ct][4 * j4 + 2] *= rs.z;
                  acc[rt][ct][4 * j4 + 3] *= rs.w;
                }
              }
              __builtin_amdgcn_sched_barrier(0);
            }
            // the f32 tail columns, two at a time: v_mfma_f32_32x32x2_f32 takes row l32, column lh of
            // the weights and column l32, row lh of the activations
            const uint32_t tw = a.tail_w;
            for (uint32_t t0 = 0; t0 < tw; t0 += 2) {
              const uint32_t t = t0 + lane_h;
              float av[2], bv[2];
#pragma unroll
              for (int rt = 0; rt < 2; ++rt) {
                const uint32_t r = 32u * rt + lane_l;
                av[rt] = (t < tw && r < done.rows) ? mt.tail[(done.r0 + r) * tw + t] : 0.f;
              }
#pragma unroll
              for (int ct = 0; ct < 2; ++ct) {
                const uint32_t my_m = lane_m + 32u * ct;
                bv[ct] = (t < tw && my_m < a.M) ? __half2float(a.x[my_m * a.ldx + nb * 24u + t]) : 0.f;
              }
#pragma unroll
              for (int rt = 0; rt < 2; ++rt)
#pragma unroll
                for (int ct = 0; ct < 2; ++ct) acc[rt][ct] = __builtin_amdgcn_mfma_f32_32x32x2f32(av[rt], bv[ct], acc[rt][ct], 0, 0, 0);
            }
            // four results go out as one store where rows of y keep a vector's alignment: d_out a multiple of four and
            // y itself on a 4-element boundary (a view into a caller's buffer need not be)
            const bool vec = (mt.d_out & 3u) == 0 && (reinterpret_cast<uintptr_t>(mt.y) & (a.y_f32 ? 15u : 7u)) == 0;
            uint32_t ln_again;  // asked for once more: the row offset does not stay alive through the tail products
            asm volatile("v_mbcnt_lo_u32_b32 %0, -1, 0\n\tv_mbcnt_hi_u32_b32 %0, -1, %0" : "=v"(ln_again));
            const uint32_t store_r = 4u * (ln_again >> 5);
#pragma unroll
            for (int ct = 0; ct < 2; ++ct) {
              const uint32_t my_m = lane_m + 32u * ct;
              if (my_m < a.M) {
#pragma unroll
                for (int rt = 0; rt < 2; ++rt)
#pragma unroll
                  for (int j4 = 0; j4 < 4; ++j4) {
                    const uint32_t row = 32u * rt + 8u * j4 + store_r;
                    const size_t at = (size_t)my_m * mt.d_out + done.r0 + row;
                    const float v0 = acc[rt][ct][4 * j4], v1 = acc[rt][ct][4 * j4 + 1], v2 = acc[rt][ct][4 * j4 + 2], v3 = acc[rt][ct][4 * j4 + 3];
                    if (vec && row + 3u < done.rows) {
                      if (a.y_f32) {
                        *reinterpret_cast<float4*>(reinterpret_cast<float*>(mt.y) + at) = make_float4(v0, v1, v2, v3);
                      } else {
                        const __half2 lo = __float22half2_rn(make_float2(v0, v1)), hi = __float22half2_rn(make_float2(v2, v3));
                        uint2 pk;
                        pk.x = *reinterpret_cast<const uint32_t*>(&lo);
                        pk.y = *reinterpret_cast<const uint32_t*>(&hi);
                        *reinterpret_cast<uint2*>(reinterpret_cast<__half*>(mt.y) + at) = pk;
                      }
                    } else {
                      const float v[4] = {v0, v1, v2, v3};
#pragma unroll
                      for (int i = 0; i < 4; ++i)
                        if (row + i < done.rows) {
                          if (a.y_f32) store_y<float>(mt.y, at + i, v[i]);
                          else store_y<__half>(mt.y, at + i, v[i]);
                        }
                    }
                  }
              }
            }
          }
        }
        clear_acc();
        if (live(w)) {
          const uint32_t lane_off = lane_offset();
          fetch(lane_off, xs, ring[0]);
          fetch(lane_off, xs + own_bytes, ring[1]);
        }
      }
    }
  }
}

// Second pass, for the bands that have partial sums in the workspace: y[m][r] = (their sum, in
// index order) * rscale[r] + tail[r] . x_tail[m].  One workgroup per (band, 16
// activation rows), one lane per four consecutive weight rows of one activation row;
// the band's tail weights and the activation tails are staged in LDS once, and the
// partial sums are read with all their loads in flight (eight splits at a time).
struct GemmReduceMat {
  const float* rscale;
  const float* tail;
  void* y;
  uint32_t d_out, band_begin;
};
struct GemmReduceArgs {
  const float* ws;  // [n_bands - ws_band0, max_pieces, kparts, M, 64]
  const __half* x;  // [M, ldx]
  GemmReduceMat mat[kGemmMaxGroup];
  uint32_t n_mats;
  uint32_t M, ldx, nblocks, tail_w, n_bands;
  uint32_t spb, kparts, ws_band0;  // as in GemmArgs: which workgroups fed a band, and the bands that have partial sums
  GemmShare share;
};

constexpr int kReduceRowsM = 16;  // activation rows per workgroup

template <typename OutT>
__global__ __launch_bounds__(256) void gemm_reduce_kernel(GemmReduceArgs a) {
  __shared__ float tl[kGemmRows * kDim];            // [row][pitch], pitch odd
  __shared__ float xt[kReduceRowsM * (kDim - 1)];   // [m][tail_w]
  const uint32_t mchunks = (a.M + kReduceRowsM - 1) / kReduceRowsM;
  const uint32_t wsb = blockIdx.x / mchunks, mc = blockIdx.x - wsb * mchunks, band = a.ws_band0 + wsb;
  uint32_t mi = 0;
#pragma unroll
  for (uint32_t k = 1; k < (uint32_t)kGemmMaxGroup; ++k)
    if (k < a.n_mats && band >= a.mat[k].band_begin) mi = k;
  const GemmReduceMat mt = a.mat[mi];
  const uint32_t r0 = (band - mt.band_begin) * kGemmRows, rows = min((uint32_t)kGemmRows, mt.d_out - r0);
  const uint32_t tw = a.tail_w, pitch = tw | 1u;
  const uint32_t tid = threadIdx.x, quad = tid & 15u, ml = tid >> 4;
  const uint32_t m = mc * kReduceRowsM + ml, row = quad * 4u;
  // the band's partial sums: one per workgroup that walked some of its slices, times the K-step shares.
  // The first eight are requested before the tail operands are staged (the two do not depend on each
  // other, and each is a trip to memory); every load is unconditional, from a valid slot.
  const uint32_t n_sums = gemm_pieces_of(a.share, a.spb, band) * a.kparts;
  const size_t sstride = (size_t)a.M * kGemmRows;
  const float* src = a.ws + ((size_t)wsb * a.share.max_pieces * a.kparts * a.M + min(m, a.M - 1u)) * kGemmRows + row;
  float4 p[8];
#pragma unroll
  for (int u = 0; u < 8; ++u) p[u] = *reinterpret_cast<const float4*>(src + (size_t)min((uint32_t)u, n_sums - 1u) * sstride);
  for (uint32_t o = tid; o < rows * tw; o += 256) {
    const uint32_t r = o / tw, t = o - r * tw;
    tl[r * pitch + t] = mt.tail[(size_t)r0 * tw + o];
  }
  for (uint32_t o = tid; o < kReduceRowsM * tw; o += 256) {
    const uint32_t mm = mc * kReduceRowsM + o / tw, t = o % tw;
    xt[o] = mm < a.M ? __half2float(a.x[(size_t)mm * a.ldx + (size_t)a.nblocks * 24u + t]) : 0.f;
  }
  __syncthreads();
  if (m >= a.M || row >= rows) return;
  float sum[4] = {0.f, 0.f, 0.f, 0.f};
  for (uint32_t s0 = 0; s0 < n_sums; s0 += 8) {
    if (s0) {
#pragma unroll
      for (int u = 0; u < 8; ++u) p[u] = *reinterpret_cast<const float4*>(src + (size_t)min(s0 + u, n_sums - 1u) * sstride);
    }
#pragma unroll
    for (int u = 0; u < 8; ++u)
      if (s0 + u < n_sums) {
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
    v[i] = fmaf(sum[i], mt.rscale[r0 + r], ts);
  }
  const size_t at = (size_t)m * mt.d_out + r0 + row;
  if ((mt.d_out & 3u) == 0 && (reinterpret_cast<uintptr_t>(mt.y) & (4 * sizeof(OutT) - 1)) == 0 && row + 3 < rows) {
    if constexpr (sizeof(OutT) == 4) {
      *reinterpret_cast<float4*>(reinterpret_cast<float*>(mt.y) + at) = make_float4(v[0], v[1], v[2], v[3]);
    } else {
      const __half2 lo = __float22half2_rn(make_float2(v[0], v[1])), hi = __float22half2_rn(make_float2(v[2], v[3]));
      uint2 pk;
      pk.x = *reinterpret_cast<const uint32_t*>(&lo);
      pk.y = *reinterpret_cast<const uint32_t*>(&hi);
      *reinterpret_cast<uint2*>(reinterpret_cast<__half*>(mt.y) + at) = pk;
    }
  } else {
#pragma unroll
    for (int i = 0; i < 4; ++i)
      if (row + i < rows) store_y<OutT>(mt.y, at + i, v[i]);
  }
}

}  // namespace llvq
