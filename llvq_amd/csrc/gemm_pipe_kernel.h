// Fused dequant-GEMM for wide batches: the same product as gemm_tiles_kernel
// (gemm_kernel.h), with the unranking and the matrix-core contraction of
// consecutive K-slices running at the same time on one CU.
//
// The 16 wavefronts of a workgroup split into two roles:
//   producers (the first 8 or 12) P0/P1/P2 of slice g: code bytes -> LDS, classify
//                                and bin, unrank into W[g & 1] (binary16, scaled);
//   consumers (the other 8 or 4) v_mfma_f32_32x32x16_f16 over slice g - 1 from
//                                W[(g - 1) & 1]: every consumer owns all 64 weight
//                                rows x 64 activation rows (64 accumulator
//                                registers), A fragments from LDS, B fragments
//                                from global memory / L2.
// The unranking is integer VALU work and the contraction runs on the matrix
// cores, so the two overlap on every SIMD (two wavefronts of each role per SIMD).
// Because the roles are separate branches of one kernel, the accumulators and the
// decode state are never live together: both fit the 128 registers a
// 1024-lane workgroup leaves each wavefront, which the single-role kernel does
// not manage beyond 32 accumulators.
//
// A stage has three workgroup barriers (after P0, after P1, after P2); the
// consumers cross the same three while they work through their K-steps, so the
// W buffer written in stage g is complete before it is read in stage g + 1 and
// is not overwritten before stage g + 2.  A slice is 16 blocks per row (384
// columns = 12 K-steps of 32): two W buffers of that size fill the LDS the
// single-role kernel spends on one slice of 32.
//
// Every consumer writes its sums to the workspace [split x K-share][band][m][64];
// gemm_reduce_kernel adds them in that order and applies row scale and tail.
#pragma once

namespace llvq {

constexpr int kPipeKb = 16;                                   // blocks per row and K-slice
constexpr int kPipeTile = kGemmRows * kPipeKb;                // blocks per K-slice
constexpr int kPipeMinProducers = 512;                        // lanes of the producer role, at least
constexpr int kPipeRowChunks = (kPipeKb * 6 + 14 + 15) / 16;  // 16-byte units holding one row's code bytes at any even alignment
constexpr int kPipeRowBytes = kPipeRowChunks * 16;
constexpr int kPipeWStride = kPipeKb * 24 + 8;                // binary16 elements per W row in LDS
constexpr int kPipeColTile = 64;                              // activation rows per consumer
static_assert(kGemmRows * kPipeRowChunks <= kPipeMinProducers, "one 16-byte load per producer lane covers a slice's code bytes");
static_assert(kGemmMaxM <= (kWgThreads - kPipeMinProducers) / 64 * kPipeColTile, "the consumers cover a launch's activation rows");

constexpr size_t gemm_pipe_lds_bytes() {
  return kGemmImageBytes + 2 * (size_t)kGemmRows * kPipeRowBytes + (size_t)kPipeTile * 4 + kGenericSlots * 4 + 32 +
         2 * (size_t)kGemmRows * kPipeWStride * 2;
}
static_assert(gemm_pipe_lds_bytes() <= 160 * 1024, "pipelined GEMM workgroup state must fit one CU's LDS");

__device__ __forceinline__ void wg_barrier() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
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

// Position of a role in the workgroup's sequence of (unit, slice) pairs.  Both roles
// step through the same sequence, the consumers one stage behind.
struct PipeWalk {
  uint32_t unit, si, n_slices, sj;  // sj: the slice walked at step si (units start at a band-dependent offset)
  uint32_t band, split, r0, rows, kb_lo, kb_hi;
};

#ifdef LLVQ_PHASE_TIMING
#define LLVQ_PSTAMP(base, k)                                                                                          \
  do {                                                                                                                \
    if (tid == ((base) ? (uint32_t)PW * 64u : 0u) && stage_no == 3) g_phase_stamps[((base) + blockIdx.x) * 8 + (k)] = wall_clock64(); \
  } while (0)
#else
#define LLVQ_PSTAMP(base, k) do {} while (0)
#endif

struct GemmPipeArgs {
  GlobalTables tables;
  const __half* xt;       // [n_steps, m_pad, 32]: tile_activations_kernel's output
  const uint8_t* codes;
  float* ws;              // [S * kparts, n_bands, M, 64] partial sums
  float g0, g1;
  uint32_t M, m_pad, d_out, nblocks;
  uint32_t n_bands, S, bps;  // split count, blocks per split (a multiple of the slice)
  uint32_t ct_shift;         // log2 of the 64-row activation tiles the consumers spread over
};

// PW = producer wavefronts (8 or 12); the other 16 - PW consume.  A narrow batch leaves the
// matrix cores little to do, and more of the workgroup unranks.
template <int PW>
__global__ __launch_bounds__(kWgThreads) void gemm_pipe_kernel(GemmPipeArgs a) {
  constexpr int kProducers = PW * 64, kConsumers = 16 - PW;
  constexpr int kP1Blocks = (kPipeTile + kProducers - 1) / kProducers;
  static_assert(kProducers >= kPipeMinProducers && (kConsumers == 8 || kConsumers == 4), "roles");
  extern __shared__ __align__(16) uint8_t smem[];
  const DecodeTables T = stage_tables<false>(smem, a.tables);
  uint8_t* raw0 = smem + kGemmImageBytes;
  constexpr uint32_t kRawBuf = kGemmRows * kPipeRowBytes;
  uint32_t* queue = reinterpret_cast<uint32_t*>(raw0 + 2 * kRawBuf);
  uint32_t* gqueue = queue + kPipeTile;
  uint32_t* ctrl0 = gqueue + kGenericSlots;  // two sets of four counters
  _Float16* W0 = reinterpret_cast<_Float16*>(ctrl0 + 8);
  constexpr uint32_t kWBuf = kGemmRows * kPipeWStride;  // elements per W buffer
  const uint32_t tid = threadIdx.x, lane = tid & 63u;
  const uint32_t wave = (uint32_t)__builtin_amdgcn_readfirstlane((int)(tid >> 6));
  const uint32_t nb = a.nblocks;
  const uint32_t n_units = a.n_bands * a.S;

  auto open_unit = [&](PipeWalk& w, uint32_t unit) {
    w.unit = unit;
    w.si = 0;
    if (unit >= n_units) return;
    w.band = unit / a.S;
    w.split = unit - w.band * a.S;
    w.r0 = w.band * kGemmRows;
    w.rows = min((uint32_t)kGemmRows, a.d_out - w.r0);
    w.kb_lo = min(nb, w.split * a.bps);
    w.kb_hi = min(nb, w.kb_lo + a.bps);
    w.n_slices = (w.kb_hi - w.kb_lo + kPipeKb - 1) / kPipeKb;  // >= 1: the host leaves no split empty
    w.sj = (w.band * 5u) % w.n_slices;
  };
  auto advance = [&](PipeWalk& w) {
    w.sj = w.sj + 1 == w.n_slices ? 0u : w.sj + 1;
    if (++w.si == w.n_slices) open_unit(w, w.unit + gridDim.x);
  };

  if (wave < (uint32_t)PW) {
    // ---------------- producers ----------------
    // Stage g: P1 of slice g | barrier | code bytes of slice g + 1 -> the other raw buffer, P2 of slice g | barrier.
    auto prefetch = [&](const PipeWalk& w, uint4& pre) {
      if (w.unit >= n_units) return;
      const uint32_t k0 = w.kb_lo + w.sj * kPipeKb, kb = min((uint32_t)kPipeKb, w.kb_hi - k0);
      const uint32_t row = tid / kPipeRowChunks, j = tid - row * kPipeRowChunks;
      if (row < w.rows) {
        const size_t byte0 = ((size_t)(w.r0 + row) * nb + k0) * 6;
        const uint32_t off = (uint32_t)(byte0 & 15);
        const uint32_t n16 = (off + kb * 6 + 15) >> 4;
        if (j < n16) pre = reinterpret_cast<const uint4*>(a.codes + (byte0 - off))[j];
      }
    };
    auto stage_raw = [&](uint32_t buf, const uint4& pre) {
      if (tid < 4) ctrl0[buf * 4 + tid] = 0;
      if (tid < (uint32_t)(kGemmRows * kPipeRowChunks)) reinterpret_cast<uint4*>(raw0 + buf * kRawBuf)[tid] = pre;
    };
    PipeWalk w, ahead;
    open_unit(w, blockIdx.x);
    uint4 pre = make_uint4(0, 0, 0, 0);
    prefetch(w, pre);
    stage_raw(0, pre);
    ahead = w;
    advance(ahead);
    prefetch(ahead, pre);  // slice 1, stored during stage 0
    wg_barrier();          // slice 0's code bytes and the table image are in LDS
    uint32_t buf = 0;
#ifdef LLVQ_PHASE_TIMING
    uint32_t stage_no = 0;
#endif
    while (w.unit < n_units) {
#ifdef LLVQ_PHASE_TIMING
      ++stage_no;
#endif
      LLVQ_PSTAMP(0, 0);
      const uint32_t k0 = w.kb_lo + w.sj * kPipeKb;
      const uint32_t kb = min((uint32_t)kPipeKb, w.kb_hi - k0);
      const uint32_t r0 = w.r0, nblk = w.rows * kb;
      const uint32_t inv_kb = (65536u + kb - 1u) / kb;  // floor(f / kb) = (f * inv_kb) >> 16 for f < 2048, kb <= 32
      const uint8_t* raw = raw0 + buf * kRawBuf;
      uint32_t* ctrl = ctrl0 + buf * 4;
      auto record_at = [&](uint32_t row, uint32_t b) -> uint64_t {
        const uint32_t off = ((((r0 + row) * nb + k0) & 7u) * 6u) & 15u;  // (6 n) mod 16 depends on n mod 8 only
        return read_record(raw, row * kPipeRowBytes + off + 6u * b);
      };
      // P1.  An origin block is queued like any other: its 24 zero weights must be written.
      classify_and_bin<kP1Blocks, kProducers>(
          T, nblk, kPipeTile, queue, gqueue, ctrl,
          [&](uint32_t f) {
            const uint32_t row = (f * inv_kb) >> 16;
            return record_at(row, f - row * kb);
          },
          [](uint32_t) { return true; });
      LLVQ_PSTAMP(0, 1);
      wg_barrier();
      LLVQ_PSTAMP(0, 2);
      // the next slice's code bytes and counters: that buffer was last read in the stage before
      if (ahead.unit < n_units) stage_raw(buf ^ 1u, pre);
      w = ahead;
      advance(ahead);
      prefetch(ahead, pre);
      // P2
      unrank_queues_to_slice<kPipeTile, kPipeWStride>(T, queue, gqueue, ctrl, kb, inv_kb, a.g0, a.g1, W0 + buf * kWBuf, record_at);
      if ((kb * 24u) & 31u) {
        // the matrix's last K-step ends inside a 32-column step: zero weights up to the step's end
        // (the buffer holds an older slice there; the activations are zero from the same column on)
        const uint32_t kcols = kb * 24u, pad = 32u - (kcols & 31u);
        for (uint32_t o = tid; o < kGemmRows * pad; o += kProducers) {
          const uint32_t row = o / pad;
          W0[buf * kWBuf + row * kPipeWStride + kcols + (o - row * pad)] = (_Float16)0.f;
        }
      }
      LLVQ_PSTAMP(0, 3);
      wg_barrier();
      LLVQ_PSTAMP(0, 4);
      buf ^= 1u;
    }
    // the consumers' last stage
    wg_barrier();
    wg_barrier();
  } else {
    // ---------------- consumers ----------------
    // Consumer c owns activation rows [64 ctile, +64) on the K-steps p = kpart (mod kparts).
    const uint32_t c = wave - (uint32_t)PW;
    const uint32_t ctn = 1u << a.ct_shift, kparts = (uint32_t)kConsumers >> a.ct_shift;
    const uint32_t ctile = c & (ctn - 1u), kpart = c >> a.ct_shift;
    const uint32_t l32 = lane & 31u, lh = lane >> 5;
    const uint32_t m0 = ctile * kPipeColTile;
    const bool tile_live = m0 < a.M, second_live = m0 + 32u < a.M;
    const uint32_t my_m[2] = {m0 + l32, m0 + 32u + l32};
    // K-step p of the matrix: 32 binary16 values per activation row, rows 64 bytes apart
    const __half* xt_lane = a.xt + (size_t)min(my_m[0], a.m_pad - 1u) * 32u + lh * 16u;
    const size_t step_stride = (size_t)a.m_pad * 32u;

    wg_barrier();  // the table image (unused here) and slice 0's code bytes
    // stage 0: nothing to multiply yet
    wg_barrier();
    wg_barrier();

    PipeWalk w;
    open_unit(w, blockIdx.x);
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
    while (w.unit < n_units) {
#ifdef LLVQ_PHASE_TIMING
      ++stage_no;
#endif
      LLVQ_PSTAMP(256, 0);
      const uint32_t k0 = w.kb_lo + w.sj * kPipeKb;  // a multiple of 4 blocks: the slice starts on a K-step
      const uint32_t kb = min((uint32_t)kPipeKb, w.kb_hi - k0);
      const uint32_t kcols = kb * 24u, psteps = (kcols + 31u) >> 5;
      const uint32_t n_own = (tile_live && kpart < psteps) ? (psteps - kpart + kparts - 1u) / kparts : 0u;
      const _Float16* arow = W0 + buf * kWBuf + (size_t)l32 * kPipeWStride + lh * 16u;
      const __half* xs = xt_lane + (size_t)(k0 * 3u / 4u + kpart) * step_stride;  // 24 k0 / 32 K-steps precede the slice
      // B fragments of three K-steps in flight: step i lives in ring slot i mod 3
      half8_t ring[3][2][2];
      auto fetch = [&](uint32_t i, half8_t (&dst)[2][2]) {
        const __half* src = xs + (size_t)(i * kparts) * step_stride;
#pragma unroll
        for (int ct = 0; ct < 2; ++ct)
#pragma unroll
          for (int f = 0; f < 2; ++f) dst[ct][f] = *reinterpret_cast<const half8_t*>(src + ct * 32 * 32 + f * 8);
      };
      auto multiply = [&](uint32_t i, const half8_t (&b)[2][2]) {
        const uint32_t p = kpart + i * kparts;
#pragma unroll
        for (int f = 0; f < 2; ++f) {
#pragma unroll
          for (int rt = 0; rt < 2; ++rt) {
            const half8_t av = *reinterpret_cast<const half8_t*>(arow + (size_t)rt * 32 * kPipeWStride + p * 32u + f * 8u);
            acc[rt][0] = __builtin_amdgcn_mfma_f32_32x32x16_f16(av, b[0][f], acc[rt][0], 0, 0, 0);
            if (second_live) acc[rt][1] = __builtin_amdgcn_mfma_f32_32x32x16_f16(av, b[1][f], acc[rt][1], 0, 0, 0);
          }
        }
      };
      auto run = [&](uint32_t i_lo, uint32_t i_hi) {  // i_lo is a multiple of 3; steps i_lo and i_lo + 1 are in flight
        for (uint32_t i = i_lo; i < i_hi; i += 3) {
          if (i + 2 < n_own) fetch(i + 2, ring[2]);
          multiply(i, ring[0]);
          if (i + 1 < i_hi) {
            if (i + 3 < n_own) fetch(i + 3, ring[0]);
            multiply(i + 1, ring[1]);
          }
          if (i + 2 < i_hi) {
            if (i + 4 < n_own) fetch(i + 4, ring[1]);
            multiply(i + 2, ring[2]);
          }
        }
      };
      // a quarter of the K-steps beside the producers' P1, the rest beside their P2
      const uint32_t i_a = n_own >= 12 ? 3u : 0u;
      if (n_own > 0) fetch(0, ring[0]);
      if (n_own > 1) fetch(1, ring[1]);
      run(0, i_a);
      LLVQ_PSTAMP(256, 1);
      wg_barrier();
      LLVQ_PSTAMP(256, 2);
      run(i_a, n_own);
      LLVQ_PSTAMP(256, 3);
      wg_barrier();
      LLVQ_PSTAMP(256, 4);

      if (w.si + 1 == w.n_slices) {
        // the unit's sums: acc[rt][ct][j] belongs to weight row r0 + 32 rt + 8 (j / 4) + 4 lh + j % 4
        // and activation row my_m[ct]
        if (tile_live) {
#pragma unroll
          for (int ct = 0; ct < 2; ++ct) {
            if (my_m[ct] < a.M) {
              float* dst = a.ws + (((size_t)(w.split * kparts + kpart) * a.n_bands + w.band) * a.M + my_m[ct]) * kGemmRows;
#pragma unroll
              for (int rt = 0; rt < 2; ++rt)
#pragma unroll
                for (int j4 = 0; j4 < 4; ++j4)
                  *reinterpret_cast<float4*>(dst + rt * 32u + 8u * j4 + 4u * lh) =
                      make_float4(acc[rt][ct][4 * j4], acc[rt][ct][4 * j4 + 1], acc[rt][ct][4 * j4 + 2], acc[rt][ct][4 * j4 + 3]);
            }
          }
        }
        clear_acc();
      }
      advance(w);
      buf ^= 1u;
    }
  }
}

}  // namespace llvq
