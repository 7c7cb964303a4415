// A sequence of fused dequant-GEMV group products in ONE launch.  Included by llvq_hip.hip after the
// GEMV kernel, whose phases (record loads, classification, queues, unranking) it shares.
//
// The reference issues two launches per projection and notes that launch latency is about half
// of a decode token (llvq-llm/src/fused_cuda.rs:789-795); a launch of gemv_tiles_kernel pays for its
// boundary (ramp, drain, table staging, cold L2) what a quarter of its tiles cost.  Here the tiles of
// every item of a list — an item is what one llvq_hip_gemv_group call would be — are numbered through
// and dealt round-robin to one persistent 1024-lane workgroup per CU, which stages the decode tables
// once and then never stops at an item's end:
//
//   * everything that does not depend on the activation runs ahead.  While a workgroup unranks tile
//     t, each of its wavefronts, at a different point of the chunk loop, classifies its share of the
//     workgroup's next tile (table reads only, results in registers) — the chain of dependent LDS
//     reads that leaves the vector ALUs half idle when all sixteen wavefronts run it at once hides
//     behind the other wavefronts' arithmetic — and requests the code bytes of the tile after that;
//   * two barriers per tile: [queue tile t, row sums of tile t - 1] | [unrank tile t, classify t + 1];
//   * an item whose activation is produced by an earlier item of the list (`wait_item`) waits, just
//     before it reads that activation, for a per-item counter that every workgroup bumps when its last
//     rows of the earlier item have arrived in memory (outputs and activations are stored and loaded at
//     device scope, past the XCDs' own L2s, so no cache is flushed).  A workgroup only ever waits
//     for items below the one it is working on and takes its tiles in ascending order, so with every
//     workgroup resident (grid <= CUs, one workgroup per CU by its LDS, the device otherwise idle) the waits end.
//     They are bounded all the same: a wait that reaches `spin_limit` polls sets `*status` and the
//     workgroup returns, which makes every wait behind it give up in turn.
//
// Results are those of the per-item launches bit for bit: every block writes its own partial sum and
// the row sums have a fixed order, whatever the tiling.
#pragma once

namespace llvq {

constexpr uint32_t kSeqNoWait = 0xFFFFFFFFu;

struct SeqTile {          // one tile of the sequence: whole rows of one matrix, at most TILE blocks
  const uint8_t* codes;   // the first row's first record
  const float* rscale;    // the first row's scale
  const float* tail;      // the first row's tail weights
  void* y;                // the first row's output element
  float g0, g1;           // the matrix's gain centroids
  uint32_t rows;
  uint32_t nblk;          // rows x blocks per row
  uint32_t item;
  uint32_t bit0;          // dense 49-bit blocks: bits of the byte at `codes` ahead of the tile's first block (0..7); 0 for 6-byte records
  uint32_t pad[2];
};
static_assert(sizeof(SeqTile) == 64, "a tile descriptor is one 64-byte scalar load");

struct SeqItem {
  const __half* x;        // the activation, or the prologue's first operand
  const __half* x2;
  const __half* norm_w;
  __half* resid_out;      // stored by the workgroup that takes the item's first tile
  float eps;
  uint32_t prologue;      // kPrologue*
  uint32_t nb, tail_w;
  float inv_nb;
  uint32_t y_f16;
  uint32_t first_tile;
  uint32_t wait_item;     // kSeqNoWait, or the item that must be complete before the activation is read
  uint32_t expected;      // workgroups that take part in this item
  uint32_t signals;       // a later item waits for this one
  uint32_t wait_expected; // `expected` of wait_item
  uint32_t pad;
};
static_assert(sizeof(SeqItem) == 80, "item records are read with scalar loads");

struct SeqArgs {
  GlobalTables tables;
  const SeqTile* tiles;
  const SeqItem* items;
  uint32_t n_tiles, max_nb;
  uint32_t* counters;   // per item: workgroups that have finished it, counted on from run to run
  uint32_t* status;     // set to 1 by a workgroup that gave up waiting
  uint32_t run;         // 1, 2, ...: item i is complete in this run at counters[i] == run * expected
  uint32_t spin_limit;
  uint32_t hold_item;  // kSeqNoWait, or an item this run must treat as never complete (tests of the give-up path)
  unsigned long long* stamps;  // tuning builds (-DLLVQ_SEQ_STAMPS): [grid][kSeqStampTiles][8] realtime-counter readings, or null
  SeqItem item0;        // items[0] again, as a kernel argument: most workgroups start there, and need not wait for the table
};

// Phase timestamps of tuning builds: lane 0 of every workgroup stores the realtime counter (100 MHz) at the phase
// boundaries of its first kSeqStampTiles tiles.  Slots: 0 round begins, 1 previous rows finished, 2 signalled,
// 3 wait over, 4 activation staged, 5 queues and planes ready (barrier),
// 6 unranked (this wavefront), 7 round ends (barrier).
constexpr uint32_t kSeqStampTiles = 8;
#ifdef LLVQ_SEQ_STAMPS
#define LLVQ_SEQ_STAMP(k)                                                                                          \
  do {                                                                                                             \
    if (threadIdx.x == 0 && s.stamps && round < kSeqStampTiles) s.stamps[((size_t)blockIdx.x * kSeqStampTiles + round) * 8 + (k)] = wall_clock64(); \
  } while (0)
#else
#define LLVQ_SEQ_STAMP(k) do {} while (0)
#endif

__host__ __device__ constexpr size_t gemv_seq_lds_bytes(uint32_t max_nb, uint32_t tile, size_t image_bytes) {
  return gemv_lds_bytes(max_nb, tile, image_bytes) + 2 * kCtrlWords * 4;  // a second set of counters and the wait's verdict
}

// Pointers that a kernel reads out of a table in memory carry no address space, and loads through them would be
// generic ("flat") ones: those count on two wait counters out of order, so every wait after one — an LDS read's
// included — has to drain all loads in flight, among them the code bytes requested for the next tile.  The tables'
// pointers are the same in every lane and point into device memory: said so (made scalar, typed global), loads
// through them are global ones with a scalar base, counted in order.
template <typename T>
__device__ __forceinline__ T* uniform_global(T* p) {
  typedef T __attribute__((address_space(1))) global_t;
  const uint64_t bits = reinterpret_cast<uint64_t>(p);
  const uint32_t lo = (uint32_t)__builtin_amdgcn_readfirstlane((int)bits), hi = (uint32_t)__builtin_amdgcn_readfirstlane((int)(bits >> 32));
  return (T*)reinterpret_cast<global_t*>(((uint64_t)hi << 32) | lo);
}
__device__ __forceinline__ SeqTile seq_tile_at(const SeqTile* tiles, uint32_t i) {
  SeqTile t = tiles[i];
  t.codes = uniform_global(t.codes);
  t.rscale = uniform_global(t.rscale);
  t.tail = uniform_global(t.tail);
  t.y = uniform_global(t.y);
  return t;
}
__device__ __forceinline__ SeqItem seq_item_of(SeqItem I) {
  I.x = uniform_global(I.x);
  I.x2 = uniform_global(I.x2);
  I.norm_w = uniform_global(I.norm_w);
  I.resid_out = uniform_global(I.resid_out);
  return I;
}

template <int NB>
__device__ __forceinline__ void seq_request_records(const SeqTile& t, uint32_t tid, LaneRecords<NB>& r) {
  if (t.nblk == 0) return;  // rows of tail columns only have no code bytes
  // a lane whose records all lie past the tile's end re-reads the tile's first ones (see prefetch_records)
  const uint32_t at = tid * (uint32_t)NB < t.nblk ? tid * (uint32_t)NB * 6u : 0u;
  const uint8_t* src = t.codes + at;
  if constexpr (NB == 4) {
    const dwords4_a2 lo = __builtin_nontemporal_load(reinterpret_cast<const dwords4_a2*>(src));
    const dwords2_a2 hi = __builtin_nontemporal_load(reinterpret_cast<const dwords2_a2*>(src + 16));
    r.w[0] = lo.x; r.w[1] = lo.y; r.w[2] = lo.z; r.w[3] = lo.w; r.w[4] = hi.x; r.w[5] = hi.y;
  } else {
    const dwords3_a2 v = __builtin_nontemporal_load(reinterpret_cast<const dwords3_a2*>(src));
    r.w[0] = v.x; r.w[1] = v.y; r.w[2] = v.z;
  }
}

// The same for the dense 49-bit blocks of a cap-13 matrix (prefetch_records): eight dwords from the dword that
// holds the lane's first block.  seq_dense_bit: where that block begins, in bits from the dword boundary at or
// below the tile's first byte.
__device__ __forceinline__ uint32_t seq_dense_bit(const SeqTile& t, uint32_t tid) {
  const uint32_t first = tid * 4u < t.nblk ? tid * 4u : 0u;
  const uint32_t skew = (uint32_t)reinterpret_cast<uintptr_t>(t.codes) & 3u;  // `codes` is a byte address: back to its dword
  return skew * 8u + t.bit0 + first * kDenseBits;
}
__device__ __forceinline__ void seq_request_records(const SeqTile& t, uint32_t tid, DenseRecords& r) {
  if (t.nblk == 0) return;
  const uint32_t skew = (uint32_t)reinterpret_cast<uintptr_t>(t.codes) & 3u;
  const uint32_t lane_bit = seq_dense_bit(t, tid);
  const uint8_t* src = t.codes - skew + (size_t)(lane_bit >> 5) * 4;
  const dwords4_a4 lo = __builtin_nontemporal_load(reinterpret_cast<const dwords4_a4*>(src));
  const dwords4_a4 hi = __builtin_nontemporal_load(reinterpret_cast<const dwords4_a4*>(src + 16));
  r.w[0] = lo.x; r.w[1] = lo.y; r.w[2] = lo.z; r.w[3] = lo.w; r.w[4] = hi.x; r.w[5] = hi.y; r.w[6] = hi.z; r.w[7] = hi.w;
  r.s0 = lane_bit & 31u;
}

// Row scales and tail weights of a tile's first 128 rows, requested ahead of the row sums.
struct RowOperands {
  float rs[2], tl[2][2];
};
__device__ __forceinline__ void seq_request_row_operands(const SeqTile& t, uint32_t tail_w, RowOperands& o) {
  uint32_t tid = threadIdx.x;
  asm volatile("" : "+v"(tid));
  const uint32_t lane = tid & 63u, wave = tid >> 6, sub = lane >> 4, l16 = lane & 15u;
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const uint32_t row = (wave * 4 + sub) + (uint32_t)j * (kWaves * 4);
    const bool ok = row < t.rows;
    o.rs[j] = ok ? t.rscale[row] : 0.f;
    o.tl[j][0] = (ok && l16 < tail_w) ? t.tail[(size_t)row * tail_w + l16] : 0.f;
    o.tl[j][1] = (ok && l16 + 16 < tail_w) ? t.tail[(size_t)row * tail_w + l16 + 16] : 0.f;
  }
}

// P3: 16 lanes per row add the row's partial sums in the order gemv_tiles_kernel adds them, apply
// the row scale and the tail columns, and store y.
__device__ __forceinline__ void seq_finish_rows(const SeqTile& t, const float* partial, const float* xtail, uint32_t nb, uint32_t tail_w,
                                                uint32_t y_f16, const RowOperands& o) {
  uint32_t tid = threadIdx.x;
  asm volatile("" : "+v"(tid));  // lane-derived values are formed per call, not carried around the loop over tiles
  const uint32_t lane = tid & 63u, wave = tid >> 6, sub = lane >> 4, l16 = lane & 15u;
  for (uint32_t base = 0; base < t.rows; base += kWaves * 4) {
    const uint32_t j = base / (kWaves * 4);
    const uint32_t row = base + wave * 4 + sub;
    const bool ok = row < t.rows;
    float s = 0.f;
    if (ok)
      for (uint32_t b = l16; b < nb; b += 16u) s += partial[row * nb + b];  // fixed order per lane
    float rs, t0, t1;
    if (j < 2u) {
      rs = j == 0 ? o.rs[0] : o.rs[1];
      t0 = j == 0 ? o.tl[0][0] : o.tl[1][0];
      t1 = j == 0 ? o.tl[0][1] : o.tl[1][1];
    } else {
      rs = ok ? t.rscale[row] : 0.f;
      t0 = (ok && l16 < tail_w) ? t.tail[(size_t)row * tail_w + l16] : 0.f;
      t1 = (ok && l16 + 16 < tail_w) ? t.tail[(size_t)row * tail_w + l16 + 16] : 0.f;
    }
    float v = s * rs;
    v = fmaf(t0, l16 < tail_w ? xtail[l16] : 0.f, v);
    v = fmaf(t1, l16 + 16 < tail_w ? xtail[l16 + 16] : 0.f, v);
#pragma unroll
    for (int q = 8; q >= 1; q >>= 1) v += __shfl_xor(v, q, 16);  // fixed tree inside each group of 16 lanes
    if (ok && l16 == 0) {  // device scope: a later item of this launch may read it from another XCD
      if (y_f16) store_half<true>(reinterpret_cast<__half*>(t.y) + row, __float2half_rn(v));
      else __hip_atomic_store(reinterpret_cast<float*>(t.y) + row, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
  }
}

// What a lane carries from one tile to the next, in one set of registers: first the code bytes of its
// share of the workgroup's next tile (requested during the current tile's unranking), then, in their
// place, that share classified (consumed when the next tile's queues are filled).
template <int NB>
struct Carried {
  uint32_t r[2 * NB + 1];
};
template <int NB>
__device__ __forceinline__ void carried_records(const Carried<NB>& c, LaneRecords<NB>& rec) {
#pragma unroll
  for (int k = 0; k < NB * 3 / 2; ++k) rec.w[k] = c.r[k];
}
template <int NB>
__device__ __forceinline__ void carry_records(const LaneRecords<NB>& rec, Carried<NB>& c) {
#pragma unroll
  for (int k = 0; k < NB * 3 / 2; ++k) c.r[k] = rec.w[k];
}
// Dense blocks take the eight words in front; the ninth stays what it is (the `where` word of a classified share:
// before a workgroup's first tile it says "nothing to queue", and must go on saying so while records are carried).
// The bit offset of the lane's first block is worked out again where the records are classified (seq_dense_bit).
static_assert(sizeof(DenseRecords) == sizeof(Carried<4>), "a lane's dense blocks fit the carried registers");
__device__ __forceinline__ void carried_records(const Carried<4>& c, DenseRecords& rec) {
#pragma unroll
  for (int k = 0; k < 8; ++k) rec.w[k] = c.r[k];
}
__device__ __forceinline__ void carry_records(const DenseRecords& rec, Carried<4>& c) {
#pragma unroll
  for (int k = 0; k < 8; ++k) c.r[k] = rec.w[k];
}
template <class Rec>
__device__ __forceinline__ void clear_records(Rec& rec) {
  if constexpr (RecordTraits<Rec>::kWide) {
#pragma unroll
    for (int k = 0; k < 8; ++k) rec.w[k] = 0;
    rec.s0 = 0;
  } else {
#pragma unroll
    for (size_t k = 0; k < sizeof(rec.w) / sizeof(rec.w[0]); ++k) rec.w[k] = 0;
  }
}
template <int NB>
__device__ __forceinline__ void carry_classified(const Classified<NB>& cls, Carried<NB>& c) {
#pragma unroll
  for (int i = 0; i < NB; ++i) {
    c.r[2 * i] = cls.e0[i];
    c.r[2 * i + 1] = cls.e1[i];
  }
  c.r[2 * NB] = cls.where;
}
template <int NB>
__device__ __forceinline__ void carried_classified(const Carried<NB>& c, Classified<NB>& cls) {
#pragma unroll
  for (int i = 0; i < NB; ++i) {
    cls.e0[i] = c.r[2 * i];
    cls.e1[i] = c.r[2 * i + 1];
  }
  cls.where = c.r[2 * NB];
}

// The lane's index in the workgroup as a value the compiler cannot see through: what is derived from it is formed
// where it is used, not once before the loop over tiles and then carried around it in registers the decoders need.
__device__ __forceinline__ uint32_t opaque_tid() {
  uint32_t t = threadIdx.x;
  asm volatile("" : "+v"(t));
  return t;
}

// WIDE: every matrix of the sequence is a cap-13 one (49-bit blocks in a dense stream, as in gemv_tiles_kernel).
template <int TILE, bool LEAN, int PLANES, bool WIDE = false>
__global__ __launch_bounds__(kWgThreads) void gemv_seq_kernel(SeqArgs s) {
  constexpr int kP1Blocks = TILE / kWgThreads;
  static_assert(!WIDE || TILE == 4 * kWgThreads, "the dense-stream variant takes four blocks per lane");
  using Records = typename std::conditional<WIDE, DenseRecords, LaneRecords<kP1Blocks>>::type;
  extern __shared__ __align__(16) uint8_t smem[];
  const uint32_t tid = threadIdx.x, wave = tid >> 6;
  const uint32_t G = gridDim.x, n_tiles = s.n_tiles;
  if (blockIdx.x >= n_tiles) return;
  const DecodeTables T = stage_tables<!LEAN, true, WIDE>(smem, s.tables);
  const uint32_t max_nb = s.max_nb;
  uint32_t* xplanes = reinterpret_cast<uint32_t*>(smem + (LEAN ? kLdsImageBytesLean : kLdsImageBytes));
  float* xscale = reinterpret_cast<float*>(xplanes + (size_t)max_nb * kPlaneDwords);
  float* xtail = xscale + max_nb;
  uint8_t* raw = reinterpret_cast<uint8_t*>(xtail + 32 + (max_nb & 1u));
  GemvQueues Q;
  Q.qa = reinterpret_cast<uint2*>(raw);
  Q.qf = reinterpret_cast<uint16_t*>(Q.qa + TILE + kSecSlots);
  Q.partial = reinterpret_cast<float*>(Q.qf + TILE + kSecSlots + 16);
  Q.gqa = reinterpret_cast<uint2*>(Q.partial + TILE);
  Q.gqf = reinterpret_cast<uint16_t*>(Q.gqa + 2 * kGenericSlots);
  uint32_t* ctrl_sets = reinterpret_cast<uint32_t*>(Q.gqf + 2 * kGenericSlots);  // two sets of counters, then the wait's verdict
  uint32_t* verdict = ctrl_sets + 2 * kCtrlWords;
  if (tid < 2u * kCtrlWords) ctrl_sets[tid] = 0;

  // The loop below is entered with an empty tile in hand: nothing is queued or unranked for it, and the
  // classification of the workgroup's first real tile takes the place the next tile's always takes.
  SeqTile cur{};
  cur.item = kSeqNoWait;
  uint32_t nxt = blockIdx.x;  // the tile after `cur`
  SeqTile next = seq_tile_at(s.tiles, nxt);
  Carried<kP1Blocks> carried;
#pragma unroll
  for (int k = 0; k < 2 * kP1Blocks + 1; ++k) carried.r[k] = 0;
  carried.r[2 * kP1Blocks] = 0xFFu;  // no block of the empty tile joins a queue

  uint32_t it = kSeqNoWait;  // the item whose activation is in LDS
  uint32_t nb = 0, tail_w = 0, y_f16 = 0, it_signals = 0;
  float inv_nb = 0.f;
  SeqTile prev{};            // its rows are finished at the top of the next round
  RowOperands ops{};
  uint32_t parity = 0;
  // This workgroup has stored its last rows of item `it`: tell the items that wait for it.  The rows (and a
  // new residual) went out as device-scope stores, which pass through this XCD's L2 to memory; every wavefront
  // waits until its own have arrived, and one lane then counts the workgroup in.  No device-scope fence on either
  // side: a release would write the whole L2 back and an acquire would empty it of the decode tables.
  auto signal_item = [&]() {
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (tid == 0) __hip_atomic_fetch_add(s.counters + it, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  };
  // A first item that waits for nothing is staged right away, as a launch of its own would: the loads of its
  // operands go out behind the table image's, the first tile's code bytes behind those (the memory counter retires
  // in order, and the code bytes are needed last).
  uint32_t first_state = 0;  // 1: the first tile's code bytes are requested
  {
    SeqItem I = s.item0;
    if (next.item != 0) I = s.items[next.item];
    I = seq_item_of(I);
    if (I.wait_item == kSeqNoWait) {
      Records rec;
      clear_records(rec);
      const ActivationSource src{I.x, nullptr, I.x2, I.norm_w, I.resid_out, I.eps, I.prologue, I.nb, I.tail_w,
                                 nullptr, nullptr, 1.f, 0u, 0u, nxt == I.first_tile, false};
      (void)stage_activation<TILE, false, PLANES, true>(src, xplanes, xscale, xtail, reinterpret_cast<uint8_t*>(xplanes), Q.partial,
                                                        [&] { seq_request_records(next, tid, rec); });
      carry_records(rec, carried);
      first_state = 1;
      it = next.item;
      nb = I.nb;
      tail_w = I.tail_w;
      inv_nb = I.inv_nb;
      y_f16 = I.y_f16;
      it_signals = I.signals;
    }
  }
  __syncthreads();
#ifdef LLVQ_SEQ_STAMPS
  uint32_t round = 0;
#endif
  for (;;) {
    // ---- the current tile's blocks join their queues; the previous tile's rows are finished
    LLVQ_SEQ_STAMP(0);
    Q.ctrl = ctrl_sets + parity * kCtrlWords;
    Classified<kP1Blocks> cls;
    carried_classified(carried, cls);
    queue_classified<kP1Blocks>(cls, TILE, Q, opaque_tid());
    const uint32_t origins = cls.where;
    seq_finish_rows(prev, Q.partial, xtail, nb, tail_w, y_f16, ops);
    LLVQ_SEQ_STAMP(1);
    // What a wavefront does for the NEXT tile in the gaps of a chunk loop: state 0 nothing done, 1 its code bytes
    // requested (after the wavefront's first few chunks, a different number per wavefront of a SIMD), 2 classified
    // (when the wavefront has no chunk left: the others are still on theirs).
    const bool more = nxt < n_tiles;
    const uint32_t request_after = wave >> 2;
    auto classify_next = [&]() {
      Records rec;
      carried_records(carried, rec);
      if constexpr (WIDE) rec.s0 = seq_dense_bit(next, opaque_tid()) & 31u;
      Classified<kP1Blocks> c;
      classify_records<kP1Blocks>(T, rec, next.nblk, c, opaque_tid());
      carry_classified(c, carried);
    };
    auto for_next_tile = [&](uint32_t done, bool last, uint32_t state) {
      if (!more) return 2u;
      if (state == 0u && (last || done >= request_after)) {
        Records rec;
        clear_records(rec);
        seq_request_records(next, opaque_tid(), rec);
        carry_records(rec, carried);
        return 1u;
      }
      return state;
    };
    if (cur.item != it && cur.item != kSeqNoWait) {  // the same for every lane
      // the rows of the previous tile are finished with the old item's tail values before the new item's replace them
      if (it != kSeqNoWait && it_signals) signal_item();
      else __syncthreads();
      LLVQ_SEQ_STAMP(2);
      const SeqItem I = seq_item_of(s.items[cur.item]);
      if (I.wait_item != kSeqNoWait) {
        if (tid == 0) {
          const uint32_t target = s.run * I.wait_expected + (I.wait_item == s.hold_item ? 1u : 0u);
          uint32_t ok = 0;
          for (uint32_t spins = 0; spins <= s.spin_limit; ++spins) {
            const uint32_t v = __hip_atomic_load(s.counters + I.wait_item, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if ((int32_t)(v - target) >= 0) { ok = 1; break; }
            __builtin_amdgcn_s_sleep(1);
          }
          *verdict = ok;
          if (!ok) __hip_atomic_store(s.status, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        __syncthreads();
        if (*verdict == 0) return;  // gave up: every lane leaves, and so will whoever waits for this workgroup
        // what the awaited item stored is read below with device-scope loads, which do not stop at this XCD's L2
      }
      LLVQ_SEQ_STAMP(3);
      // a derived activation is staged where the planes themselves go: the queues are already in use
      const ActivationSource src{I.x, nullptr, I.x2, I.norm_w, I.resid_out, I.eps, I.prologue, I.nb, I.tail_w,
                                 nullptr, nullptr, 1.f, 0u, 0u, nxt - G == I.first_tile, I.wait_item != kSeqNoWait};
      (void)stage_activation<TILE, false, PLANES, true>(src, xplanes, xscale, xtail, reinterpret_cast<uint8_t*>(xplanes), Q.partial, [] {});
      it = cur.item;
      nb = I.nb;
      tail_w = I.tail_w;
      inv_nb = I.inv_nb;
      y_f16 = I.y_f16;
      it_signals = I.signals;
      LLVQ_SEQ_STAMP(4);
    }
    __syncthreads();
    LLVQ_SEQ_STAMP(5);

    // ---- the current tile is unranked; each wavefront requests and classifies its share of the next tile on the way
    if (tid < (uint32_t)kCtrlWords) ctrl_sets[(parity ^ 1u) * kCtrlWords + tid] = 0;
    settle_origins<kP1Blocks>(origins, Q.partial, opaque_tid());
    const uint32_t state = unrank_tile<TILE, true, PLANES>(T, Q, UnrankOperands{xplanes, xscale, nb, inv_nb, cur.g0, cur.g1, first_state}, for_next_tile);
    first_state = 0;
    if (state == 1u) classify_next();
    seq_request_row_operands(cur, tail_w, ops);
    LLVQ_SEQ_STAMP(6);
    __syncthreads();
    LLVQ_SEQ_STAMP(7);
#ifdef LLVQ_SEQ_STAMPS
    ++round;
#endif
    prev = cur;
    if (!more) break;
    cur = next;
    nxt += G;
    next = seq_tile_at(s.tiles, min(nxt, n_tiles - 1u));
    parity ^= 1u;
  }
  seq_finish_rows(prev, Q.partial, xtail, nb, tail_w, y_f16, ops);
  if (it_signals) signal_item();
}

}  // namespace llvq
