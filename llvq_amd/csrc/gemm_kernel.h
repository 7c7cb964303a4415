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
// 20 blocks per row (480 columns, 1280 blocks):
//   P0  the slice's code bytes, 16-byte loads -> LDS (next slice's loads are
//       already in flight while this one is decoded);
//   P1  classify and bin the blocks (odd / even / generic queues);
//   P2  unrank; every block writes its 24 weights, already multiplied by
//       centroid[gain] / sqrt(16 shell), as binary16 into the W slice in LDS;
//   P3  16 wavefronts run v_mfma_f32_16x16x32_f16 over the slice: A fragments
//       from LDS, B fragments (activations) straight from global memory / L2;
//       the wavefront grid is 2 row groups x 8 column groups and accumulators
//       (<= 32 registers) stay live across slices.
// Epilogue: row scale and the f32 tail columns in f32, then the store.  When a
// matrix has too few bands to occupy the chip its block range is split over
// several units; each writes its partial sums to a workspace and the unit that
// arrives last at the band's counter adds them in a fixed order, so the result
// does not depend on scheduling.
#pragma once

namespace llvq {

typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float float4_t __attribute__((ext_vector_type(4)));

constexpr int kGemmRows = 64;                 // weight rows of a band
constexpr int kGemmKb = 20;                   // blocks per row and K-slice: 480 columns = 15 MFMA k-steps
constexpr int kGemmTile = kGemmRows * kGemmKb;  // 1280 blocks per K-slice
constexpr int kGemmP1Blocks = (kGemmTile + kWgThreads - 1) / kWgThreads;
constexpr int kGemmRowChunks = 9;             // 16-byte units holding one row's <= 120 code bytes at any even alignment
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
  float* ws;              // [S, M, d_out] partial sums when S > 1
  uint32_t* counters;     // [n_bands], zero between launches
  float g0, g1;
  uint32_t M, ldx, d_out, nblocks, tail_w;
  uint32_t n_bands, S, bps;  // split count, blocks per split
};

constexpr size_t gemm_lds_bytes() {
  return kLdsImageBytes + (size_t)kGemmRows * kGemmRowBytes + (size_t)kGemmTile * 4 + kGenericSlots * 4 + 16 +
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

// CT = column tiles (16 activation rows each) per wavefront: M <= 128 CT.
template <int CT, typename OutT>
__global__ __launch_bounds__(kWgThreads) void gemm_tiles_kernel(GemmArgs a) {
  extern __shared__ __align__(16) uint8_t smem[];
  const DecodeTables T = stage_tables(smem, a.tables);
  uint8_t* raw = smem + kLdsImageBytes;
  uint32_t* queue = reinterpret_cast<uint32_t*>(raw + kGemmRows * kGemmRowBytes);
  uint32_t* gqueue = queue + kGemmTile;
  uint32_t* ctrl = gqueue + kGenericSlots;
  _Float16* W = reinterpret_cast<_Float16*>(ctrl + 4);
  const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
  const uint32_t nb = a.nblocks;
  const uint32_t n_units = a.n_bands * a.S;
  // stale W contents are multiplied by zero activations in a slice's padding
  // columns, so they must be finite from the start
  for (uint32_t i = tid; i < (uint32_t)(kGemmRows * kGemmWStride / 8); i += kWgThreads)
    reinterpret_cast<uint4*>(W)[i] = make_uint4(0, 0, 0, 0);

  // wavefront grid of the MFMA phase
  const uint32_t rg = wave & 1u, cg = wave >> 1;  // row group (32 rows), column group
  const uint32_t l16 = lane & 15u, lq = lane >> 4;

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

  for (uint32_t unit = blockIdx.x; unit < n_units; unit += gridDim.x) {
    const uint32_t band = unit / a.S, split = unit - band * a.S;
    const uint32_t r0 = band * kGemmRows, rows = min((uint32_t)kGemmRows, a.d_out - r0);
    const uint32_t kb_lo = min(nb, split * a.bps), kb_hi = min(nb, kb_lo + a.bps);
    float4_t acc[2][CT];
#pragma unroll
    for (int rt = 0; rt < 2; ++rt)
#pragma unroll
      for (int ct = 0; ct < CT; ++ct) acc[rt][ct] = float4_t{0.f, 0.f, 0.f, 0.f};

    uint4 pre = make_uint4(0, 0, 0, 0);
    prefetch(r0, rows, kb_lo, min((uint32_t)kGemmKb, kb_hi - kb_lo), pre);
    for (uint32_t k0 = kb_lo; k0 < kb_hi; k0 += kGemmKb) {
      const uint32_t kb = min((uint32_t)kGemmKb, kb_hi - k0);
      const uint32_t nblk = rows * kb;
      const uint32_t inv_kb = (65536u + kb - 1u) / kb;  // floor(f / kb) = (f * inv_kb) >> 16 for f < 1536, kb <= 24
      // P0
      if (tid < 4) ctrl[tid] = 0;
      if (tid < (uint32_t)(kGemmRows * kGemmRowChunks)) reinterpret_cast<uint4*>(raw)[tid] = pre;
      __syncthreads();
      if (k0 + kGemmKb < kb_hi) prefetch(r0, rows, k0 + kGemmKb, min((uint32_t)kGemmKb, kb_hi - k0 - kGemmKb), pre);

      auto record_at = [&](uint32_t row, uint32_t b) -> uint64_t {
        const uint32_t off = ((((r0 + row) * nb + k0) & 7u) * 6u) & 15u;  // (6 n) mod 16 depends on n mod 8 only
        return read_record(raw, row * kGemmRowBytes + off + 6u * b);
      };

      // P1: classify and bin
      {
        uint32_t entry[kGemmP1Blocks], ci[kGemmP1Blocks], kbits[kGemmP1Blocks], kmax = 0;
        uint64_t zi[kGemmP1Blocks];
#pragma unroll
        for (int i = 0; i < kGemmP1Blocks; ++i) {
          const uint32_t f = tid + (uint32_t)i * kWgThreads;
          zi[i] = ~0ULL;
          entry[i] = 0;
          ci[i] = 0;
          kbits[i] = 0;
          if (f < nblk) {
            const uint32_t row = (f * inv_kb) >> 16, b = f - row * kb;
            const uint64_t rec = record_at(row, b);
            entry[i] = f | ((uint32_t)(rec & 1) << 25);
            if ((rec >> 1) == 0) {
              entry[i] |= 0x40000000u;  // the origin: P2 writes 24 zero weights (W may still be read by P3 now)
            } else {
              zi[i] = (rec >> 1) - 1;
              const uint32_t e = T.lut[(uint32_t)(zi[i] >> kLutShift)];
              ci[i] = e & 511u;
              kbits[i] = 1u << ((e >> 9) & 7u);
              kmax = max(kmax, kbits[i]);
            }
          }
        }
        uint32_t kw = 1;
#pragma unroll
        for (uint32_t t = 1; t <= 6; ++t) kw = __any(kmax >= (1u << t)) ? (1u << t) : kw;
        for (uint32_t step = kw >> 1; step; step >>= 1) {
#pragma unroll
          for (int i = 0; i < kGemmP1Blocks; ++i)
            if (step < kbits[i] && T.starts[ci[i] + step] <= zi[i]) ci[i] += step;
        }
        uint32_t path[kGemmP1Blocks], odd_rank[kGemmP1Blocks], even_rank[kGemmP1Blocks], n_o = 0, n_e = 0;
#pragma unroll
        for (int i = 0; i < kGemmP1Blocks; ++i) {
          path[i] = zi[i] != ~0ULL ? ((T.fast[ci[i]].meta >> kMetaPathShift) & 3u)
                                   : ((entry[i] & 0x40000000u) ? (uint32_t)kPathOdd : 3u);
          entry[i] |= ci[i] << 16;
          if (path[i] == kPathGeneric) {
            entry[i] |= 0x80000000u;
            const uint32_t slot = atomicAdd(&ctrl[2], 1u);
            if (slot < (uint32_t)kGenericSlots) {
              gqueue[slot] = entry[i];
              path[i] = 3u;
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
        for (int i = 0; i < kGemmP1Blocks; ++i) {
          if (path[i] == kPathOdd || path[i] == kPathGeneric) queue[base_o + odd_rank[i]] = entry[i];
          if (path[i] == kPathEven) queue[kGemmTile - 1 - (base_e + even_rank[i])] = entry[i];
        }
      }
      __syncthreads();

      // P2: unrank into the W slice
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
        const uint32_t entry = from_gen ? gqueue[k] : (from_odd ? queue[k] : queue[kGemmTile - 1 - k]);
        const uint32_t f = entry & 0xFFFu, ci = (entry >> 16) & 0x1FFu;
        const uint32_t row = (f * inv_kb) >> 16, b = f - row * kb;
        const uint64_t rec = record_at(row, b);
        const uint64_t li = (rec >> 1) - 1 - T.starts[ci];
        const float g = (entry >> 25) & 1u ? a.g1 : a.g0;
        _Float16* wrow = W + (size_t)row * kGemmWStride + b * 24u;
        if (entry & 0x40000000u) {
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
      __syncthreads();

      // P3: acc += W_slice (64 x 24 kb) * X^T (24 kb x M); k runs in steps of 32,
      // the columns of a last partial step are zero on the activation side
      if (cg * 16u < a.M) {  // column groups beyond the batch have nothing to add
        const uint32_t kcols = kb * 24u, ksteps = (kcols + 31u) >> 5;
        const __half* xk = a.x + (size_t)k0 * 24u;
        constexpr int D = 8 / CT;  // k-steps whose B fragments are fetched together
        const _Float16* arow0 = W + (size_t)(rg * 32u + l16) * kGemmWStride + lq * 8u;
        for (uint32_t ks0 = 0; ks0 < ksteps; ks0 += D) {
          half8_t bf[D][CT];
#pragma unroll
          for (int d = 0; d < D; ++d) {
            const uint32_t kc = (ks0 + d) * 32u + lq * 8u;
#pragma unroll
            for (int ct = 0; ct < CT; ++ct) {
              const uint32_t m = (cg + 8u * ct) * 16u + l16;
              half8_t v = {0, 0, 0, 0, 0, 0, 0, 0};
              if (kc < kcols && m < a.M) v = *reinterpret_cast<const half8_t*>(xk + (size_t)m * a.ldx + kc);
              bf[d][ct] = v;
            }
          }
#pragma unroll
          for (int d = 0; d < D; ++d) {
            if (ks0 + d < ksteps) {
              const half8_t a0 = *reinterpret_cast<const half8_t*>(arow0 + (ks0 + d) * 32u);
              const half8_t a1 = *reinterpret_cast<const half8_t*>(arow0 + 16 * kGemmWStride + (ks0 + d) * 32u);
#pragma unroll
              for (int ct = 0; ct < CT; ++ct) {
                acc[0][ct] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a0, bf[d][ct], acc[0][ct], 0, 0, 0);
                acc[1][ct] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a1, bf[d][ct], acc[1][ct], 0, 0, 0);
              }
            }
          }
        }
      }
      // no barrier here: the next slice's P0/P1 touch only raw, queues and
      // counters, and its P2 starts behind two barriers every wavefront reaches
      // after leaving P3
    }

    // ---- epilogue ----
    // acc[rt][ct][i] belongs to weight row r0 + rg*32 + rt*16 + lq*4 + i and activation row (cg + 8 ct)*16 + l16
    const uint32_t tw = a.tail_w;
    const __half* xtail = a.x + (size_t)nb * 24u;
    if (a.S == 1) {
#pragma unroll
      for (int rt = 0; rt < 2; ++rt)
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) {
          const uint32_t m = (cg + 8u * ct) * 16u + l16;
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const uint32_t row = rg * 32u + rt * 16u + lq * 4u + i;
            if (row < rows && m < a.M) {
              float v = acc[rt][ct][i] * a.rscale[r0 + row];
              for (uint32_t t = 0; t < tw; ++t)
                v = fmaf(a.tail[(size_t)(r0 + row) * tw + t], __half2float(xtail[(size_t)m * a.ldx + t]), v);
              store_y<OutT>(a.y, (size_t)m * a.d_out + r0 + row, v);
            }
          }
        }
    } else {
#pragma unroll
      for (int rt = 0; rt < 2; ++rt)
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) {
          const uint32_t m = (cg + 8u * ct) * 16u + l16;
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const uint32_t row = rg * 32u + rt * 16u + lq * 4u + i;
            if (row < rows && m < a.M) a.ws[((size_t)split * a.M + m) * a.d_out + r0 + row] = acc[rt][ct][i];
          }
        }
      // the unit that arrives last at the band's counter adds the partial sums
      __threadfence();
      __syncthreads();
      if (tid == 0) ctrl[0] = __hip_atomic_fetch_add(&a.counters[band], 1u, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_AGENT);
      __syncthreads();
      const bool last = ctrl[0] == a.S - 1;
      __syncthreads();  // ctrl[0] is rewritten by the next unit's first slice
      if (last) {
        __threadfence();
        for (uint32_t o = tid; o < rows * a.M; o += kWgThreads) {
          const uint32_t m = o / rows, row = o - m * rows;
          float s = 0.f;
          for (uint32_t sp = 0; sp < a.S; ++sp)
            s += a.ws[((size_t)sp * a.M + m) * a.d_out + r0 + row];
          float v = s * a.rscale[r0 + row];
          for (uint32_t t = 0; t < tw; ++t)
            v = fmaf(a.tail[(size_t)(r0 + row) * tw + t], __half2float(xtail[(size_t)m * a.ldx + t]), v);
          store_y<OutT>(a.y, (size_t)m * a.d_out + r0 + row, v);
        }
        if (tid == 0) a.counters[band] = 0;  // ready for the next launch
      }
    }
    __syncthreads();  // W, raw and counters are reused by the next unit
  }
}

}  // namespace llvq
