// Batch-1 greedy decode loop of a Qwen3-architecture model whose seven
// projections per layer are LLVQ matrices: the counterpart of
// Block::forward_cached / Qwen3::hidden_cached / Qwen3::generate
// (llvq-llm/src/model.rs:766-835, :968-982, :1041-1073) at l = 1.
// Included by llvq_hip.hip after the GEMV launcher it drives.
//
// Everything between two projections runs in small hand-written kernels on the
// runtime's stream; the token chosen at one step is read by the next step's
// embedding kernel from device memory, so the host never waits inside a
// generation.  Activations between kernels are binary16 (the run dtype of the
// reference); every kernel computes in f32 and rounds once on output:
//   embed -> h
//   [per layer] add + RMSNorm -> qkv GEMV group -> per-head RMSNorm + RoPE +
//   cache append -> attention over the cache -> o GEMV -> add + RMSNorm ->
//   gate/up GEMV group -> SiLU(gate) * up -> down GEMV
//   add + final RMSNorm -> f16 lm_head GEMV (logits rounded to binary16, as the
//   reference's f16 matmul leaves them) -> argmax, lowest index on ties.
#pragma once

namespace llvq {

constexpr int kNormThreads = 1024;

__device__ __forceinline__ float block_sum_1024(float v, float* red) {
  v = wave_sum(v);
  const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
  __syncthreads();  // red may still be read from a previous call
  if (lane == 0) red[wave] = v;
  __syncthreads();
  float s = 0.f;
#pragma unroll
  for (int w = 0; w < kNormThreads / 64; ++w) s += red[w];  // same order in every lane
  return s;
}

// h[row] = embed[token[row]], row = blockIdx.y
__global__ __launch_bounds__(256) void embed_kernel(const __half* __restrict__ table, const uint32_t* __restrict__ token,
                                                    uint32_t vocab, uint32_t hidden, __half* __restrict__ h) {
  const uint32_t t = min(token[blockIdx.y], vocab - 1u);
  h += (size_t)blockIdx.y * hidden;
  for (uint32_t i = blockIdx.x * blockDim.x + threadIdx.x; i < hidden; i += gridDim.x * blockDim.x)
    h[i] = table[(size_t)t * hidden + i];
}

// r = f16(h + delta) when delta is given (else h), written to h_out when that is given
// (it may be h itself); normed = f16(r / sqrt(mean(r^2) + eps) * w)
// (candle_nn::RmsNorm: f32 inside, one rounding on the way out).
__global__ __launch_bounds__(kNormThreads) void add_rmsnorm_kernel(const __half* h, const __half* __restrict__ delta,
                                                                   const __half* __restrict__ w, __half* h_out,
                                                                   __half* __restrict__ normed, uint32_t n, float eps) {
  __shared__ float red[kNormThreads / 64];
  // one workgroup per row of n values
  h += (size_t)blockIdx.x * n;
  if (delta) delta += (size_t)blockIdx.x * n;
  if (h_out) h_out += (size_t)blockIdx.x * n;
  normed += (size_t)blockIdx.x * n;
  constexpr int kPer = 8;  // n <= 8192
  float v[kPer];
  float ss = 0.f;
#pragma unroll
  for (int k = 0; k < kPer; ++k) {
    const uint32_t i = threadIdx.x + (uint32_t)k * kNormThreads;
    v[k] = 0.f;
    if (i < n) {
      float x = __half2float(h[i]);
      if (delta) x = __half2float(__float2half_rn(x + __half2float(delta[i])));  // the residual stream is binary16
      if (h_out) h_out[i] = __float2half_rn(x);
      v[k] = x;
      ss += x * x;
    }
  }
  const float total = block_sum_1024(ss, red);
  const float inv = 1.0f / sqrtf(total / (float)n + eps);
#pragma unroll
  for (int k = 0; k < kPer; ++k) {
    const uint32_t i = threadIdx.x + (uint32_t)k * kNormThreads;
    if (i < n) normed[i] = __float2half_rn(v[k] * inv * __half2float(w[i]));
  }
}

// int8 KV cache (llvq-llm/src/kvq.rs:110-165): asymmetric 8-bit codes per group
// of 64 along head_dim, binary16 scale and bias, chosen from the token alone:
//   s = f16((max - min) / 255), b = f16(min), q = clamp(round((x - b) / (s > 0 ? s : 1)), 0, 255)
// and a reader gets back f16(q s + b).  The reference keeps that reconstructed
// value in its cache; here the codes themselves are stored (1.06 bytes per
// value instead of 2) and the same value is rebuilt on every read.
constexpr uint32_t kKvGroup = 64;
struct KvQ8 {
  uint8_t* kq;    // [n_kv][max_pos][head_dim]
  uint8_t* vq;
  __half* ks;     // [n_kv][max_pos][head_dim / 64] scales
  __half* kb;     //                                biases
  __half* vs;
  __half* vb;
};

// One group of 64 values held one per lane -> code, scale, bias.
__device__ __forceinline__ uint8_t kv_quantize_group(float x, __half* s_out, __half* b_out) {
  float mn = x, mx = x;
#pragma unroll
  for (int o = 32; o >= 1; o >>= 1) {
    mn = fminf(mn, __shfl_xor(mn, o, 64));
    mx = fmaxf(mx, __shfl_xor(mx, o, 64));
  }
  const __half sh = __float2half_rn(__fdiv_rn(__fsub_rn(mx, mn), 255.0f));
  const __half bh = __float2half_rn(mn);
  const float s = __half2float(sh), b = __half2float(bh);
  const float safe = s > 0.f ? s : 1.0f;
  const float q = fminf(fmaxf(roundf(__fdiv_rn(__fsub_rn(x, b), safe)), 0.f), 255.f);
  *s_out = sh;
  *b_out = bh;
  return (uint8_t)q;
}

__device__ __forceinline__ float kv_dequant(uint32_t q, float s, float b) {
  return __half2float(__float2half_rn(__fadd_rn(__fmul_rn((float)q, s), b)));
}

// One wavefront: per-head RMSNorm of a q or k head (model.rs:800-808), then RoPE at
// the absolute position in the rotate-half convention (candle_nn::rotary_emb::rope:
// out[i] = x[i] cos - x[i + d/2] sin, out[i + d/2] = x[i] sin + x[i + d/2] cos, with
// the binary16 cos/sin tables of Rotary::new, model.rs:163-179).  Each step rounds to
// binary16 as the reference's tensors do; the results are left, widened, in
// stage[0, head_dim) — an LDS area of this wavefront alone.  head_dim <= 256 (the callers take 128).
__device__ __forceinline__ void wave_lds_sync() {
  // LDS operations of one wavefront execute in order; only the compiler must not move them
  __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
  __builtin_amdgcn_wave_barrier();
}
__device__ __forceinline__ void norm_rope_wave(const __half* __restrict__ src, const __half* __restrict__ w,
                                               const __half* __restrict__ cos_t, const __half* __restrict__ sin_t,
                                               uint32_t pos, uint32_t head_dim, float eps, float* stage, uint32_t lane) {
  const uint32_t half_d = head_dim >> 1;
  if (head_dim == 128) {
    // the served width: a lane's two elements (lane, lane + 64) are a rotation pair, so nothing
    // crosses lanes but the sum of squares, and every load goes out before the first use
    const float x1 = __half2float(src[lane]), x2 = __half2float(src[lane + 64]);
    const float w1 = __half2float(w[lane]), w2 = __half2float(w[lane + 64]);
    const float c = __half2float(cos_t[(size_t)pos * 64 + lane]), sn = __half2float(sin_t[(size_t)pos * 64 + lane]);
    const float ss = wave_sum(x1 * x1 + x2 * x2);
    const float inv = 1.0f / sqrtf(ss / 128.0f + eps);
    const float n1 = __half2float(__float2half_rn(x1 * inv * w1)), n2 = __half2float(__float2half_rn(x2 * inv * w2));
    stage[lane] = __half2float(__float2half_rn(n1 * c - n2 * sn));
    stage[lane + 64] = __half2float(__float2half_rn(n1 * sn + n2 * c));
    wave_lds_sync();
    return;
  }
  float x[4];  // elements lane, lane + 64, lane + 128, lane + 192
  float ss = 0.f;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const uint32_t i = lane + 64u * j;
    x[j] = i < head_dim ? __half2float(src[i]) : 0.f;
    ss += x[j] * x[j];
  }
  ss = wave_sum(ss);
  const float inv = 1.0f / sqrtf(ss / (float)head_dim + eps);
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const uint32_t i = lane + 64u * j;
    if (i < head_dim) stage[i] = __half2float(__float2half_rn(x[j] * inv * __half2float(w[i])));
  }
  wave_lds_sync();
  float r1[2], r2[2];  // rotated pairs (i, i + d/2) for i = lane, lane + 64
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const uint32_t i = lane + 64u * j;
    r1[j] = r2[j] = 0.f;
    if (i < half_d) {
      const float c = __half2float(cos_t[(size_t)pos * half_d + i]), sn = __half2float(sin_t[(size_t)pos * half_d + i]);
      const float x1 = stage[i], x2 = stage[i + half_d];
      r1[j] = __half2float(__float2half_rn(x1 * c - x2 * sn));
      r2[j] = __half2float(__float2half_rn(x1 * sn + x2 * c));
    }
  }
  wave_lds_sync();
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const uint32_t i = lane + 64u * j;
    if (i < half_d) {
      stage[i] = r1[j];
      stage[i + half_d] = r2[j];
    }
  }
  wave_lds_sync();
}

// What the attention launch is handed about the position being decoded: the raw
// q / k / v rows the projections left, the layer's q and k norm weights and the
// rotary tables.  The launch norms and rotates its own query heads, and the one
// workgroup whose range ends at the new position does the same for k, appends
// k and v to the cache and uses them from LDS.
struct AttnNew {
  const __half* q_raw;  // [n_heads, head_dim]
  const __half* k_raw;  // [n_kv, head_dim]
  const __half* v_raw;  // [n_kv, head_dim]
  const __half* qn;     // [head_dim]
  const __half* kn;     // [head_dim]
  const __half* cos_t;  // [max_pos, head_dim / 2]
  const __half* sin_t;
  __half* kcache;       // this layer's binary16 cache (null with the int8 cache)
  __half* vcache;
  float eps;
};

constexpr int kAttnThreads = 256;
constexpr int kAttnWaves = kAttnThreads / 64;
constexpr int kAttnMaxSplits = 64;  // the cache is cut into at most this many ranges (host picks by length; 128 was measured slower at 8188 positions)
constexpr int kAttnMaxGroup = 8;    // query heads per kv head
constexpr int kAttnInlineSplits = 16;  // up to this many ranges, the workgroup that finishes last merges them itself

// ---- rows of positions at once (prompt processing through the batched product) ----
// One wavefront per (head, row): q heads are normed and rotated in place, k heads are
// normed, rotated and appended to the cache at position pos0 + row, v heads are appended.
// Grid (n_heads + 2 n_kv, rows).  Same arithmetic as the one-position path.
template <bool Q8>
__global__ __launch_bounds__(64) void norm_rope_append_rows_kernel(__half* __restrict__ q, const __half* __restrict__ k,
                                                                   const __half* __restrict__ v, AttnNew nw, KvQ8 q8,
                                                                   uint32_t n_heads, uint32_t n_kv, uint32_t head_dim,
                                                                   uint32_t pos0, uint32_t max_pos) {
  __shared__ float stage[256];
  const uint32_t head = blockIdx.x, row = blockIdx.y, lane = threadIdx.x;
  const uint32_t pos = pos0 + row, kvgroups = head_dim / kKvGroup;
  if (head < n_heads) {
    __half* qh = q + ((size_t)row * n_heads + head) * head_dim;
    norm_rope_wave(qh, nw.qn, nw.cos_t, nw.sin_t, pos, head_dim, nw.eps, stage, lane);
    for (uint32_t i = lane; i < head_dim; i += 64) qh[i] = __float2half_rn(stage[i]);
    return;
  }
  const bool is_k = head < n_heads + n_kv;
  const uint32_t kvh = is_k ? head - n_heads : head - n_heads - n_kv;
  const __half* src = (is_k ? k : v) + ((size_t)row * n_kv + kvh) * head_dim;
  if (is_k) norm_rope_wave(src, nw.kn, nw.cos_t, nw.sin_t, pos, head_dim, nw.eps, stage, lane);
  else {
    for (uint32_t i = lane; i < head_dim; i += 64) stage[i] = __half2float(src[i]);
    wave_lds_sync();
  }
  const size_t crow = (size_t)kvh * max_pos + pos;
  if constexpr (Q8) {
    uint8_t* cq = is_k ? q8.kq : q8.vq;
    __half* cs = is_k ? q8.ks : q8.vs;
    __half* cb = is_k ? q8.kb : q8.vb;
    for (uint32_t g = 0; g < kvgroups; ++g) {
      __half sh, bh;
      const uint8_t code = kv_quantize_group(stage[g * kKvGroup + lane], &sh, &bh);
      cq[crow * head_dim + g * kKvGroup + lane] = code;
      if (lane == 0) {
        cs[crow * kvgroups + g] = sh;
        cb[crow * kvgroups + g] = bh;
      }
    }
  } else {
    __half* dst = (is_k ? nw.kcache : nw.vcache) + crow * head_dim;
    for (uint32_t i = lane; i < head_dim; i += 64) dst[i] = __float2half_rn(stage[i]);
  }
}

// Causal attention of a row of queries over the cache (model.rs:812-822 with the mask of
// :938-960): one wavefront per (kv head, row) serves every query head of the group; the
// query at row r sees positions 0 .. pos0 + r.  Lane (pj, sub) = (lane / 16, lane % 16)
// holds dims [8 sub, 8 sub + 8) of the positions j = pj (mod 4); each of the four position
// classes keeps its own running maximum, sum and weighted V sum (f32), merged at the end.
// head_dim <= 128, a multiple of 8; G >= query heads per kv head sizes the register arrays.  q is already normed and rotated; ctx is rounded once.
template <bool Q8, int G>
__global__ __launch_bounds__(64) void attn_rows_kernel(const __half* __restrict__ q, const __half* __restrict__ kcache,
                                                       const __half* __restrict__ vcache, KvQ8 q8, __half* __restrict__ ctx,
                                                       uint32_t n_heads, uint32_t n_kv, uint32_t head_dim, uint32_t pos0,
                                                       uint32_t max_pos, float scale) {
  const uint32_t kvh = blockIdx.x, row = blockIdx.y, lane = threadIdx.x;
  const uint32_t groups = n_heads / n_kv, T = pos0 + row + 1;
  const uint32_t sub = lane & 15u, pj = lane >> 4, i0 = sub * 8u;
  const bool active = i0 < head_dim;
  const uint32_t kvgroups = head_dim / kKvGroup;
  const size_t base = (size_t)kvh * max_pos;
  float qv[G][8], acc[G][8], m[G], l[G];
#pragma unroll
  for (int g = 0; g < G; ++g) {
    m[g] = -INFINITY;
    l[g] = 0.f;
#pragma unroll
    for (int t = 0; t < 8; ++t) {
      acc[g][t] = 0.f;
      qv[g][t] = ((uint32_t)g < groups && active)
                     ? __half2float(q[((size_t)row * n_heads + kvh * groups + g) * head_dim + i0 + t]) * scale
                     : 0.f;
    }
  }
  // U positions of this lane's class per pass: their rows are requested together, then used in order
  constexpr int U = 4;
  for (uint32_t jb = pj; jb < T; jb += 4 * U) {
    uint4 kraw[U], vraw[U];
    float ks[U], kb[U], vs[U], vb[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const uint32_t j = jb + 4u * u;
      kraw[u] = vraw[u] = make_uint4(0, 0, 0, 0);
      ks[u] = kb[u] = vs[u] = vb[u] = 0.f;
      if (active && j < T) {
        if constexpr (Q8) {
          const uint2 kc = *reinterpret_cast<const uint2*>(q8.kq + (base + j) * head_dim + i0);
          const uint2 vc = *reinterpret_cast<const uint2*>(q8.vq + (base + j) * head_dim + i0);
          const size_t gi = (base + j) * kvgroups + i0 / kKvGroup;
          kraw[u].x = kc.x; kraw[u].y = kc.y;
          vraw[u].x = vc.x; vraw[u].y = vc.y;
          ks[u] = __half2float(q8.ks[gi]); kb[u] = __half2float(q8.kb[gi]);
          vs[u] = __half2float(q8.vs[gi]); vb[u] = __half2float(q8.vb[gi]);
        } else {
          kraw[u] = *reinterpret_cast<const uint4*>(kcache + (base + j) * head_dim + i0);
          vraw[u] = *reinterpret_cast<const uint4*>(vcache + (base + j) * head_dim + i0);
        }
      }
    }
    // scores of the U positions first (independent exchanges), then the running sums in order
    float sc[U][G], vfs[U][8];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      float kf[8];
      if constexpr (Q8) {
#pragma unroll
        for (int t = 0; t < 4; ++t) {
          kf[t] = kv_dequant((kraw[u].x >> (8 * t)) & 0xFFu, ks[u], kb[u]);
          kf[4 + t] = kv_dequant((kraw[u].y >> (8 * t)) & 0xFFu, ks[u], kb[u]);
          vfs[u][t] = kv_dequant((vraw[u].x >> (8 * t)) & 0xFFu, vs[u], vb[u]);
          vfs[u][4 + t] = kv_dequant((vraw[u].y >> (8 * t)) & 0xFFu, vs[u], vb[u]);
        }
      } else {
        const uint32_t kw[4] = {kraw[u].x, kraw[u].y, kraw[u].z, kraw[u].w}, vw[4] = {vraw[u].x, vraw[u].y, vraw[u].z, vraw[u].w};
#pragma unroll
        for (int t = 0; t < 4; ++t) {
          kf[2 * t] = __half2float(__ushort_as_half((unsigned short)(kw[t] & 0xFFFFu)));
          kf[2 * t + 1] = __half2float(__ushort_as_half((unsigned short)(kw[t] >> 16)));
          vfs[u][2 * t] = __half2float(__ushort_as_half((unsigned short)(vw[t] & 0xFFFFu)));
          vfs[u][2 * t + 1] = __half2float(__ushort_as_half((unsigned short)(vw[t] >> 16)));
        }
      }
      if (!active) {
#pragma unroll
        for (int t = 0; t < 8; ++t) kf[t] = vfs[u][t] = 0.f;
      }
#pragma unroll
      for (int g = 0; g < G; ++g) {
        float d = 0.f;
#pragma unroll
        for (int t = 0; t < 8; ++t) d = fmaf(qv[g][t], kf[t], d);
        sc[u][g] = row16_sum(d);
      }
    }
#pragma unroll
    for (int u = 0; u < U; ++u)
      if (jb + 4u * u < T) {
#pragma unroll
        for (int g = 0; g < G; ++g)
          if ((uint32_t)g < groups) {
            const float d = sc[u][g];
            const float mn = fmaxf(m[g], d);
            const float c = __expf(m[g] - mn), p = __expf(d - mn);  // c = 0 on the first position (m = -inf)
            l[g] = fmaf(l[g], c, p);
#pragma unroll
            for (int t = 0; t < 8; ++t) acc[g][t] = fmaf(acc[g][t], c, p * vfs[u][t]);
            m[g] = mn;
          }
      }
  }
  // merge the four position classes (a class with no position has m = -inf and weight 0)
#pragma unroll
  for (int off = 16; off <= 32; off <<= 1)
#pragma unroll
    for (int g = 0; g < G; ++g)
      if ((uint32_t)g < groups) {
        const float mo = __shfl_xor(m[g], off, 64), lo = __shfl_xor(l[g], off, 64);
        const float mn = fmaxf(m[g], mo);
        const float c1 = m[g] == -INFINITY ? 0.f : __expf(m[g] - mn), c2 = mo == -INFINITY ? 0.f : __expf(mo - mn);
        l[g] = l[g] * c1 + lo * c2;
#pragma unroll
        for (int t = 0; t < 8; ++t) {
          const float ao = __shfl_xor(acc[g][t], off, 64);
          acc[g][t] = acc[g][t] * c1 + ao * c2;
        }
        m[g] = mn;
      }
  if (pj == 0 && active)
#pragma unroll
    for (int g = 0; g < G; ++g)
      if ((uint32_t)g < groups) {
        __half* dst = ctx + ((size_t)row * n_heads + kvh * groups + g) * head_dim + i0;
        const float inv = 1.0f / l[g];
#pragma unroll
        for (int t = 0; t < 8; ++t) dst[t] = __float2half_rn(acc[g][t] * inv);
      }
}

// The same causal attention for 32 rows at a time on the matrix cores (head_dim = 128).
// Workgroup (kv head, block of 32 rows); wavefront w serves query head w of the group and all
// 32 rows.  The cache is walked in tiles of 32 positions, staged in LDS once for all heads:
// K as stored ([position][dim]), V transposed ([dim][position], positions in the order the
// second product wants them).  Per tile and wavefront:
//   S^T = K Q^T      8 x v_mfma_f32_32x32x16_f16; A = K rows from LDS, B = the wavefront's
//                    query rows, held in registers for the whole walk.  Lane (q, h) of the
//                    result holds row q's scores of positions 8a + 4h + b (a, b < 4);
//   online softmax   per row in its two lanes: running maximum and sum in f32, one exchange
//                    between the halves of the wavefront; the causal mask is applied here;
//   O^T += V^T P^T   8 x the same MFMA; B = the probabilities just computed, rounded to
//                    binary16 in the lanes that hold them (no cross-lane movement: the K
//                    index of the product is permuted to match, V^T is stored in that order).
// Scores, maxima, sums and O stay in f32; the context is rounded once.  The next tile's K and
// V rows are requested before the current tile is multiplied.  Positions past the pass's last
// row are read as that row (their probabilities are zero; the values must be finite).
constexpr int kAttnTile = 32;
constexpr int kAttnKPitch = 128 + 8;   // binary16 elements per K row in LDS
constexpr int kAttnVPitch = 32 + 8;    // per V^T row
template <bool Q8, int G>
__global__ __launch_bounds__(G * 64) void attn_rows_mfma_kernel(const __half* __restrict__ q, const __half* __restrict__ kcache,
                                                                const __half* __restrict__ vcache, KvQ8 q8,
                                                                __half* __restrict__ ctx, uint32_t n_heads, uint32_t n_kv,
                                                                uint32_t pos0, uint32_t n_rows, uint32_t max_pos, float scale) {
  typedef _Float16 h8 __attribute__((ext_vector_type(8)));
  typedef float f16v __attribute__((ext_vector_type(16)));
  constexpr uint32_t kDimH = 128, kThreads = G * 64;
  constexpr int CH = (kAttnTile * kDimH / 8 + kThreads - 1) / kThreads;  // 16-byte pieces of a tile per lane
  __shared__ __align__(16) _Float16 kt[kAttnTile * kAttnKPitch];
  __shared__ __align__(16) _Float16 vt[kDimH * kAttnVPitch];
  const uint32_t kvh = blockIdx.x, row0 = blockIdx.y * kAttnTile;
  const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
  const uint32_t groups = n_heads / n_kv;
  const uint32_t l32 = lane & 31u, lh = lane >> 5;
  const bool has_head = wave < groups;
  const uint32_t head = kvh * groups + min(wave, groups - 1u);
  const uint32_t my_row = min(row0 + l32, n_rows - 1u);      // rows past the pass repeat its last row and store nothing
  const uint32_t qpos = pos0 + my_row;
  const uint32_t last_pos = pos0 + n_rows - 1u;              // last cached position
  const uint32_t t_end = pos0 + min(row0 + kAttnTile - 1u, n_rows - 1u);
  const uint32_t n_tiles = t_end / kAttnTile + 1u;
  const size_t base = (size_t)kvh * max_pos;
  constexpr uint32_t kvgroups = kDimH / kKvGroup;

  // query rows: B fragments of the first product, dims [16 s + 8 h, +8) of row q
  h8 qf[8];
  {
    const __half* qrow = q + ((size_t)my_row * n_heads + head) * kDimH + lh * 8u;
#pragma unroll
    for (int s8 = 0; s8 < 8; ++s8) qf[s8] = *reinterpret_cast<const h8*>(qrow + s8 * 16);
  }
  f16v o[4];
#pragma unroll
  for (int dt = 0; dt < 4; ++dt)
#pragma unroll
    for (int j = 0; j < 16; ++j) o[dt][j] = 0.f;
  float m_run = -INFINITY, l_run = 0.f;

  // staging, 16-byte pieces: piece c of K = position c / 16, dims [8 (c % 16), +8) (rows are read and
  // stored whole); piece c of V = position c % 32, dims [8 (c / 32), +8) (the transposing 2-byte stores
  // of a wavefront then fall into different LDS banks)
  uint4 kreg[CH], vreg[CH];
  float ksc[CH], kbi[CH], vsc[CH], vbi[CH];
  auto request = [&](uint32_t tile) {
#pragma unroll
    for (int u = 0; u < CH; ++u) {
      const uint32_t c = tid + (uint32_t)u * kThreads;
      if (c < kAttnTile * kDimH / 8) {
        const uint32_t kpos = min(tile * kAttnTile + c / 16u, last_pos), kd0 = (c & 15u) * 8u;
        const uint32_t vpos = min(tile * kAttnTile + (c & 31u), last_pos), vd0 = (c >> 5) * 8u;
        if constexpr (Q8) {
          const uint2 kc = *reinterpret_cast<const uint2*>(q8.kq + (base + kpos) * kDimH + kd0);
          const uint2 vc = *reinterpret_cast<const uint2*>(q8.vq + (base + vpos) * kDimH + vd0);
          const size_t kgi = (base + kpos) * kvgroups + kd0 / kKvGroup, vgi = (base + vpos) * kvgroups + vd0 / kKvGroup;
          kreg[u] = make_uint4(kc.x, kc.y, 0, 0);
          vreg[u] = make_uint4(vc.x, vc.y, 0, 0);
          ksc[u] = __half2float(q8.ks[kgi]); kbi[u] = __half2float(q8.kb[kgi]);
          vsc[u] = __half2float(q8.vs[vgi]); vbi[u] = __half2float(q8.vb[vgi]);
        } else {
          kreg[u] = *reinterpret_cast<const uint4*>(kcache + (base + kpos) * kDimH + kd0);
          vreg[u] = *reinterpret_cast<const uint4*>(vcache + (base + vpos) * kDimH + vd0);
        }
      }
    }
  };
  auto deposit = [&]() {
#pragma unroll
    for (int u = 0; u < CH; ++u) {
      const uint32_t c = tid + (uint32_t)u * kThreads;
      if (c < kAttnTile * kDimH / 8) {
        const uint32_t kp = c / 16u, kd0 = (c & 15u) * 8u, p = c & 31u, vd0 = (c >> 5) * 8u;
        h8 kv8, vv8;
        if constexpr (Q8) {
#pragma unroll
          for (int t = 0; t < 4; ++t) {
            kv8[t] = (_Float16)kv_dequant((kreg[u].x >> (8 * t)) & 0xFFu, ksc[u], kbi[u]);
            kv8[4 + t] = (_Float16)kv_dequant((kreg[u].y >> (8 * t)) & 0xFFu, ksc[u], kbi[u]);
            vv8[t] = (_Float16)kv_dequant((vreg[u].x >> (8 * t)) & 0xFFu, vsc[u], vbi[u]);
            vv8[4 + t] = (_Float16)kv_dequant((vreg[u].y >> (8 * t)) & 0xFFu, vsc[u], vbi[u]);
          }
        } else {
          kv8 = __builtin_bit_cast(h8, kreg[u]);
          vv8 = __builtin_bit_cast(h8, vreg[u]);
        }
        *reinterpret_cast<h8*>(kt + kp * kAttnKPitch + kd0) = kv8;
        // position p = 16 hh + 8 a + 4 h + b sits at column 16 hh + 8 h + 4 a + b of its V^T row
        const uint32_t col = (p & 16u) + ((p >> 2) & 1u) * 8u + ((p >> 3) & 1u) * 4u + (p & 3u);
#pragma unroll
        for (int t = 0; t < 8; ++t) vt[(vd0 + t) * kAttnVPitch + col] = vv8[t];
      }
    }
  };

  request(0);
  for (uint32_t tile = 0; tile < n_tiles; ++tile) {
    __syncthreads();  // the previous tile has been read by every wavefront
    deposit();
    __syncthreads();
    if (tile + 1 < n_tiles) request(tile + 1);
    // S^T = K Q^T
    f16v sacc;
#pragma unroll
    for (int j = 0; j < 16; ++j) sacc[j] = 0.f;
#pragma unroll
    for (int s8 = 0; s8 < 8; ++s8) {
      const h8 kf = *reinterpret_cast<const h8*>(kt + l32 * kAttnKPitch + s8 * 16 + lh * 8u);
      sacc = __builtin_amdgcn_mfma_f32_32x32x16_f16(kf, qf[s8], sacc, 0, 0, 0);
    }
    // online softmax of row q over this tile's positions (16 of them in this lane, 16 in lane ^ 32)
    float sc[16], mx = -INFINITY;
#pragma unroll
    for (int j = 0; j < 16; ++j) {
      const uint32_t pos = tile * kAttnTile + 8u * (j >> 2) + 4u * lh + (j & 3);
      sc[j] = pos <= qpos ? sacc[j] * scale : -INFINITY;
      mx = fmaxf(mx, sc[j]);
    }
    mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
    const float m_new = fmaxf(m_run, mx);
    const float m_use = m_new == -INFINITY ? 0.f : m_new;  // a row that has seen nothing yet
    const float alpha = __expf(m_run - m_use);              // 0 while m_run = -inf
    float psum = 0.f;
    h8 pf[2];  // the probabilities as the second product's B fragments
#pragma unroll
    for (int j = 0; j < 16; ++j) {
      const float pj = __expf(sc[j] - m_use);
      psum += pj;
      pf[j >> 3][j & 7] = (_Float16)pj;
    }
    psum += __shfl_xor(psum, 32, 64);
    l_run = fmaf(l_run, alpha, psum);
    m_run = m_new;
#pragma unroll
    for (int dt = 0; dt < 4; ++dt)
#pragma unroll
      for (int j = 0; j < 16; ++j) o[dt][j] *= alpha;
    // O^T += V^T P^T: K index e of half hh <-> position 16 hh + 8 (e / 4) + 4 h + e % 4 = this lane's score 8 hh + e
#pragma unroll
    for (int hh = 0; hh < 2; ++hh) {
#pragma unroll
      for (int dt = 0; dt < 4; ++dt) {
        const h8 vf = *reinterpret_cast<const h8*>(vt + (dt * 32 + l32) * kAttnVPitch + hh * 16 + lh * 8u);
        o[dt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(vf, pf[hh], o[dt], 0, 0, 0);
      }
    }
  }
  // o[dt][j] = O[q = l32][dim 32 dt + 8 (j / 4) + 4 h + j % 4]
  if (has_head && row0 + l32 < n_rows) {
    const float inv = 1.0f / l_run;
    __half* dst = ctx + ((size_t)my_row * n_heads + head) * kDimH;
#pragma unroll
    for (int dt = 0; dt < 4; ++dt)
#pragma unroll
      for (int a = 0; a < 4; ++a) {
        const __half2 lo = __float22half2_rn(make_float2(o[dt][4 * a] * inv, o[dt][4 * a + 1] * inv));
        const __half2 hi = __float22half2_rn(make_float2(o[dt][4 * a + 2] * inv, o[dt][4 * a + 3] * inv));
        uint2 pk;
        pk.x = *reinterpret_cast<const uint32_t*>(&lo);
        pk.y = *reinterpret_cast<const uint32_t*>(&hi);
        *reinterpret_cast<uint2*>(dst + dt * 32 + 8 * a + 4 * lh) = pk;
      }
  }
}

// Attention of one query position over the cache (model.rs:812-822), split over
// the cache: workgroup (kv head, split) takes a contiguous range of positions
// for all query heads that share the kv head, so every K and V row is fetched
// (and, for the int8 cache, rebuilt) once per group.  The range is walked once:
// sixteen position classes (four per wavefront, 16 lanes x 8 dims each) keep a
// running maximum, a sum of exponentials and a weighted V sum per query head,
// with the K and V rows of four positions requested together; the classes meet
// in LDS and the workgroup leaves an unnormalised partial per query head.  The
// workgroup that arrives last at the kv head's counter merges the partials in
// split order and rounds the context once.  Scores, softmax and sums stay in
// f32.  head_dim <= 128, a multiple of 8; G >= query heads per kv head sizes
// the register arrays.
template <bool Q8, int G>
__global__ __launch_bounds__(kAttnThreads) void attn_decode_kernel(AttnNew nw, const __half* __restrict__ kcache,
                                                                   const __half* __restrict__ vcache, KvQ8 q8,
                                                                   __half* __restrict__ ctx,
                                                                   float* __restrict__ part, uint32_t* __restrict__ counters,
                                                                   uint32_t n_heads, uint32_t n_kv, uint32_t head_dim,
                                                                   uint32_t T, uint32_t max_pos, float scale, uint32_t n_splits,
                                                                   uint32_t merge_inline) {
  extern __shared__ __align__(16) float att_smem[];
  __shared__ uint32_t arrived;
  __shared__ float stage[kAttnWaves][256];  // one head per wavefront while it is normed and rotated
  __shared__ float knew[256], vnew[256];    // the new position's k and v as the cache returns them
  const uint32_t kvh = blockIdx.x / n_splits, split = blockIdx.x % n_splits;
  const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
  const uint32_t groups = n_heads / n_kv;  // <= kAttnMaxGroup (checked by the host)
  const uint32_t chunk = (T + n_splits - 1) / n_splits;
  const uint32_t j0 = min(T, split * chunk), j1 = min(T, j0 + chunk), nj = j1 - j0;
  float* qs = att_smem;                         // [groups][head_dim]
  float* cls = qs + groups * head_dim;          // [16 classes][groups][head_dim + 2]: running max, sum, weighted V sums
  const __half* K = kcache + (size_t)kvh * max_pos * head_dim;
  const __half* V = vcache + (size_t)kvh * max_pos * head_dim;
  const uint32_t kvgroups = head_dim / kKvGroup;
  const uint8_t* Kq = q8.kq + (size_t)kvh * max_pos * head_dim;
  const uint8_t* Vq = q8.vq + (size_t)kvh * max_pos * head_dim;
  const __half* Ks = q8.ks + (size_t)kvh * max_pos * kvgroups;
  const __half* Kb = q8.kb + (size_t)kvh * max_pos * kvgroups;
  const __half* Vs = q8.vs + (size_t)kvh * max_pos * kvgroups;
  const __half* Vb = q8.vb + (size_t)kvh * max_pos * kvgroups;
  const uint32_t stride = head_dim + 2;  // floats per partial: max, sum, head_dim sums

  const uint32_t pos = T - 1;  // the position being decoded
  const bool has_new = nj > 0 && j1 == T;
  const uint32_t newj = has_new ? pos : 0xFFFFFFFFu;
  // Lane (pj, sub) = (lane / 16, lane % 16) of wavefront w holds dims [8 sub, 8 sub + 8) of the
  // positions of class c = 4 w + pj: jj = c, c + 16, ...  U rows of K and of V are requested
  // together.  The loads are unconditional (a lane with no row, or with the row this launch
  // appends, re-reads a valid one and ignores it): a guarded load would be waited for where it
  // is issued, and the first batch is issued here, ahead of the work on the query heads, which
  // then runs beside the cache's latency.
  const uint32_t sub = lane & 15u, pj = lane >> 4, i0 = sub * 8u, c = wave * 4u + pj;
  const bool active = i0 < head_dim;
  const uint32_t i0c = active ? i0 : 0u;
  constexpr int U = 4;
  uint4 kraw[U], vraw[U];
  float ksc[U], kbi[U], vsc[U], vbi[U];
  auto request = [&](uint32_t jb) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const uint32_t j = min(j0 + jb + 16u * u, pos);
      if constexpr (Q8) {
        const uint2 kc = *reinterpret_cast<const uint2*>(Kq + (size_t)j * head_dim + i0c);
        const uint2 vc = *reinterpret_cast<const uint2*>(Vq + (size_t)j * head_dim + i0c);
        const size_t gi = (size_t)j * kvgroups + i0c / kKvGroup;
        kraw[u] = make_uint4(kc.x, kc.y, 0, 0);
        vraw[u] = make_uint4(vc.x, vc.y, 0, 0);
        ksc[u] = __half2float(Ks[gi]); kbi[u] = __half2float(Kb[gi]);
        vsc[u] = __half2float(Vs[gi]); vbi[u] = __half2float(Vb[gi]);
      } else {
        kraw[u] = *reinterpret_cast<const uint4*>(K + (size_t)j * head_dim + i0c);
        vraw[u] = *reinterpret_cast<const uint4*>(V + (size_t)j * head_dim + i0c);
        ksc[u] = kbi[u] = vsc[u] = vbi[u] = 0.f;
      }
    }
  };
  request(c);
  // the query heads of this kv head: norm, rotate, scale
  for (uint32_t g = wave; g < groups; g += kAttnWaves) {
    norm_rope_wave(nw.q_raw + (size_t)(kvh * groups + g) * head_dim, nw.qn, nw.cos_t, nw.sin_t, pos, head_dim, nw.eps,
                   stage[wave], lane);
    for (uint32_t i = lane; i < head_dim; i += 64) qs[g * head_dim + i] = stage[wave][i] * scale;
    wave_lds_sync();  // stage is rewritten by this wavefront's next head
  }
  // The range that ends at the new position owns its k and v: they go to the
  // cache for later positions, and to LDS, in the form the cache gives back,
  // for this one (nothing else reads that cache row during this launch).
  if (has_new && wave == 0) {
    norm_rope_wave(nw.k_raw + (size_t)kvh * head_dim, nw.kn, nw.cos_t, nw.sin_t, pos, head_dim, nw.eps, stage[0], lane);
    const size_t row = (size_t)kvh * max_pos + pos;
    if constexpr (Q8) {
      for (uint32_t g = 0; g < kvgroups; ++g) {
        __half sh, bh;
        const uint8_t code = kv_quantize_group(stage[0][g * kKvGroup + lane], &sh, &bh);
        q8.kq[row * head_dim + g * kKvGroup + lane] = code;
        if (lane == 0) {
          q8.ks[row * kvgroups + g] = sh;
          q8.kb[row * kvgroups + g] = bh;
        }
        knew[g * kKvGroup + lane] = kv_dequant(code, __half2float(sh), __half2float(bh));
      }
    } else {
      for (uint32_t i = lane; i < head_dim; i += 64) {
        nw.kcache[row * head_dim + i] = __float2half_rn(stage[0][i]);
        knew[i] = stage[0][i];
      }
    }
  }
  if (has_new && wave == 1) {
    const size_t row = (size_t)kvh * max_pos + pos;
    if constexpr (Q8) {
      for (uint32_t g = 0; g < kvgroups; ++g) {
        const float x = __half2float(nw.v_raw[(size_t)kvh * head_dim + g * kKvGroup + lane]);
        __half sh, bh;
        const uint8_t code = kv_quantize_group(x, &sh, &bh);
        q8.vq[row * head_dim + g * kKvGroup + lane] = code;
        if (lane == 0) {
          q8.vs[row * kvgroups + g] = sh;
          q8.vb[row * kvgroups + g] = bh;
        }
        vnew[g * kKvGroup + lane] = kv_dequant(code, __half2float(sh), __half2float(bh));
      }
    } else {
      for (uint32_t i = lane; i < head_dim; i += 64) {
        const __half x = nw.v_raw[(size_t)kvh * head_dim + i];
        nw.vcache[row * head_dim + i] = x;
        vnew[i] = __half2float(x);
      }
    }
  }
  __syncthreads();

  // ---- one pass over the range: scores, running maxima and weighted V sums together ----
  // Each position class keeps its own running maximum, sum of exponentials and weighted V sum
  // (f32); the scores of a batch are formed first (independent cross-lane sums), then folded in
  // order, with the next batch's rows already requested.
  float qv[G][8], acc[G][8], m[G], l[G];
#pragma unroll
  for (int g = 0; g < G; ++g) {
    m[g] = -INFINITY;
    l[g] = 0.f;
#pragma unroll
    for (int t = 0; t < 8; ++t) {
      acc[g][t] = 0.f;
      qv[g][t] = ((uint32_t)g < groups && active) ? qs[g * head_dim + i0 + t] : 0.f;
    }
  }
  for (uint32_t jb = c; jb < nj; jb += 16u * U) {
    float sc[U][G], vfs[U][8];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const uint32_t jj = jb + 16u * u;
      float kf[8];
      if (j0 + jj == newj) {  // the row appended by this launch: from LDS, as the cache returns it
#pragma unroll
        for (int t = 0; t < 8; ++t) {
          kf[t] = active ? knew[i0 + t] : 0.f;
          vfs[u][t] = active ? vnew[i0 + t] : 0.f;
        }
      } else if constexpr (Q8) {
#pragma unroll
        for (int t = 0; t < 4; ++t) {
          kf[t] = kv_dequant((kraw[u].x >> (8 * t)) & 0xFFu, ksc[u], kbi[u]);
          kf[4 + t] = kv_dequant((kraw[u].y >> (8 * t)) & 0xFFu, ksc[u], kbi[u]);
          vfs[u][t] = kv_dequant((vraw[u].x >> (8 * t)) & 0xFFu, vsc[u], vbi[u]);
          vfs[u][4 + t] = kv_dequant((vraw[u].y >> (8 * t)) & 0xFFu, vsc[u], vbi[u]);
        }
      } else {
        const uint32_t kw[4] = {kraw[u].x, kraw[u].y, kraw[u].z, kraw[u].w}, vw[4] = {vraw[u].x, vraw[u].y, vraw[u].z, vraw[u].w};
#pragma unroll
        for (int t = 0; t < 4; ++t) {
          kf[2 * t] = __half2float(__ushort_as_half((unsigned short)(kw[t] & 0xFFFFu)));
          kf[2 * t + 1] = __half2float(__ushort_as_half((unsigned short)(kw[t] >> 16)));
          vfs[u][2 * t] = __half2float(__ushort_as_half((unsigned short)(vw[t] & 0xFFFFu)));
          vfs[u][2 * t + 1] = __half2float(__ushort_as_half((unsigned short)(vw[t] >> 16)));
        }
      }
#pragma unroll
      for (int g = 0; g < G; ++g) {
        float d = 0.f;
#pragma unroll
        for (int t = 0; t < 8; ++t) d = fmaf(qv[g][t], kf[t], d);
        sc[u][g] = row16_sum(d);
      }
    }
    if (jb + 16u * U < nj) request(jb + 16u * U);
#pragma unroll
    for (int u = 0; u < U; ++u)
      if (jb + 16u * u < nj) {
#pragma unroll
        for (int g = 0; g < G; ++g)
          if ((uint32_t)g < groups) {
            const float d = sc[u][g];
            const float mn = fmaxf(m[g], d);
            const float e0 = __expf(m[g] - mn), p = __expf(d - mn);  // e0 = 0 on the first position (m = -inf)
            l[g] = fmaf(l[g], e0, p);
#pragma unroll
            for (int t = 0; t < 8; ++t) acc[g][t] = fmaf(acc[g][t], e0, p * vfs[u][t]);
            m[g] = mn;
          }
      }
  }
  // the classes' results meet in LDS
#pragma unroll
  for (int g = 0; g < G; ++g)
    if ((uint32_t)g < groups) {
      float* dst = cls + ((size_t)c * groups + g) * stride;
      if (sub == 0) {
        dst[0] = m[g];
        dst[1] = l[g];
      }
      if (active) {
#pragma unroll
        for (int t = 0; t < 8; ++t) dst[2 + i0 + t] = acc[g][t];
      }
    }
  __syncthreads();
  // ---- this workgroup's partial: the sixteen classes merged in class order ----
  // per query head: the maximum over the classes, then each class's weight, once, into its slot for the maximum
  if (tid < groups) {
    float M = -INFINITY;
#pragma unroll
    for (int cc = 0; cc < 16; ++cc) M = fmaxf(M, cls[((size_t)cc * groups + tid) * stride]);
    float Lsum = 0.f;
#pragma unroll
    for (int cc = 0; cc < 16; ++cc) {
      float* src = cls + ((size_t)cc * groups + tid) * stride;
      const float wgt = src[0] == -INFINITY ? 0.f : __expf(src[0] - M);  // a class with no position
      Lsum = fmaf(src[1], wgt, Lsum);
      src[0] = wgt;
    }
    float* dst = part + ((size_t)(kvh * groups + tid) * n_splits + split) * stride;
    dst[0] = M;  // -inf for an empty range
    dst[1] = Lsum;
  }
  __syncthreads();
  for (uint32_t o = tid; o < groups * head_dim; o += kAttnThreads) {
    const uint32_t g = o / head_dim, i = o - g * head_dim;
    float A = 0.f;
#pragma unroll
    for (int cc = 0; cc < 16; ++cc) {
      const float* src = cls + ((size_t)cc * groups + g) * stride;
      A = fmaf(src[2 + i], src[0], A);
    }
    part[((size_t)(kvh * groups + g) * n_splits + split) * stride + 2 + i] = A;
  }
  if (!merge_inline) return;  // attn_merge_kernel finishes (long caches: many partials, merged chip-wide)
  // publish, and let the last workgroup of this kv head merge (one lane's
  // device-scope release / acquire stands for the workgroup, ordered by the barriers)
  __syncthreads();
  if (tid == 0) arrived = __hip_atomic_fetch_add(&counters[kvh], 1u, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_AGENT);
  __syncthreads();
  if (arrived != n_splits - 1) return;
  // Merge (at most kAttnInlineSplits ranges).  The partials come from the other XCDs' writes,
  // i.e. from memory, so latency is what matters: the (max, sum) pairs and the first partial
  // vectors are requested together, every load unconditional (a lane past the end re-reads a
  // valid element and gives it weight zero).  Each lane then forms its head's weights from
  // the pairs in LDS for itself; sums run in range order.
  float* mx = att_smem;                // [groups][n_splits] running maxima (the staging of this launch is dead)
  float* sm = mx + groups * n_splits;  // [groups][n_splits] sums of exponentials
  const uint32_t n_pairs = groups * n_splits, n_out = groups * head_dim;
  auto fetch = [&](uint32_t o, float (&v)[kAttnInlineSplits]) {
    o = min(o, n_out - 1u);
    const uint32_t g = o / head_dim, i = o - g * head_dim;
    const float* src = part + (size_t)(kvh * groups + g) * n_splits * stride + 2 + i;
#pragma unroll
    for (int u = 0; u < kAttnInlineSplits; ++u) v[u] = src[(size_t)min((uint32_t)u, n_splits - 1u) * stride];
  };
  float v[kAttnInlineSplits], vn[kAttnInlineSplits];
  float2 pair[(kAttnMaxGroup * kAttnInlineSplits + kAttnThreads - 1) / kAttnThreads];
#pragma unroll
  for (uint32_t r = 0; r < sizeof(pair) / sizeof(pair[0]); ++r) {
    const uint32_t o = min(tid + r * kAttnThreads, n_pairs - 1u);
    const uint32_t g = o / n_splits, sp = o - g * n_splits;
    pair[r] = *reinterpret_cast<const float2*>(part + ((size_t)(kvh * groups + g) * n_splits + sp) * stride);
  }
  fetch(tid, v);
#pragma unroll
  for (uint32_t r = 0; r < sizeof(pair) / sizeof(pair[0]); ++r) {
    const uint32_t o = tid + r * kAttnThreads;
    if (o < n_pairs) {
      mx[o] = pair[r].x;
      sm[o] = pair[r].y;
    }
  }
  __syncthreads();
  for (uint32_t o = tid; o < n_out; o += kAttnThreads) {
    fetch(o + kAttnThreads, vn);
    const uint32_t g = o / head_dim, i = o - g * head_dim;
    float w[kAttnInlineSplits], M = -INFINITY;
#pragma unroll
    for (int u = 0; u < kAttnInlineSplits; ++u) {
      w[u] = mx[g * n_splits + min((uint32_t)u, n_splits - 1u)];
      M = fmaxf(M, w[u]);
    }
    float L = 0.f, A = 0.f;
#pragma unroll
    for (int u = 0; u < kAttnInlineSplits; ++u) {
      w[u] = (uint32_t)u < n_splits ? __expf(w[u] - M) : 0.f;  // 0 for an empty range too
      L = fmaf(sm[g * n_splits + min((uint32_t)u, n_splits - 1u)], w[u], L);
      A = fmaf(v[u], w[u], A);
    }
    ctx[(size_t)(kvh * groups + g) * head_dim + i] = __float2half_rn(A / L);
#pragma unroll
    for (int u = 0; u < kAttnInlineSplits; ++u) v[u] = vn[u];
  }
  if (tid == 0) counters[kvh] = 0;  // ready for the next launch
}

// Merge of the attention partials as a kernel of its own: one workgroup per query
// head, one lane per output dimension, the partial vectors read eight splits at a
// time.  Same arithmetic and order as the in-kernel merge.
__global__ __launch_bounds__(128) void attn_merge_kernel(const float* __restrict__ part, __half* __restrict__ ctx,
                                                         uint32_t head_dim, uint32_t n_splits) {
  __shared__ float wts[kAttnMaxSplits], ls[kAttnMaxSplits];
  __shared__ float Lsum;
  static_assert(kAttnMaxSplits <= 128, "one lane per range fetches its maximum and its sum");
  const uint32_t head = blockIdx.x, tid = threadIdx.x;
  const uint32_t stride = head_dim + 2;
  const float* src = part + (size_t)head * n_splits * stride;
  if (tid < n_splits) {
    wts[tid] = src[(size_t)tid * stride];
    ls[tid] = src[(size_t)tid * stride + 1];
  }
  __syncthreads();
  float M = -INFINITY;
  for (uint32_t s = 0; s < n_splits; ++s) M = fmaxf(M, wts[s]);
  __syncthreads();
  if (tid < n_splits) wts[tid] = __expf(wts[tid] - M);
  __syncthreads();
  if (tid == 0) {
    float L = 0.f;
    for (uint32_t s = 0; s < n_splits; ++s) L = fmaf(ls[s], wts[s], L);  // range order
    Lsum = L;
  }
  __syncthreads();
  for (uint32_t i = tid; i < head_dim; i += 128) {
    float A = 0.f;
    uint32_t sp = 0;
    for (; sp + 8 <= n_splits; sp += 8) {
      float v[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) v[u] = src[(size_t)(sp + u) * stride + 2 + i];
#pragma unroll
      for (int u = 0; u < 8; ++u) A = fmaf(v[u], wts[sp + u], A);
    }
    for (; sp < n_splits; ++sp) A = fmaf(src[(size_t)sp * stride + 2 + i], wts[sp], A);
    ctx[(size_t)head * head_dim + i] = __float2half_rn(A / Lsum);
  }
}

// act = f16(f16(silu(gate)) * up)   (model.rs:831: gu[0].apply(act).mul(gu[1]))
__global__ __launch_bounds__(256) void silu_mul_kernel(const __half* __restrict__ gate, const __half* __restrict__ up,
                                                       __half* __restrict__ out, uint32_t n) {
  for (uint32_t i = blockIdx.x * blockDim.x + threadIdx.x; i < n; i += gridDim.x * blockDim.x) {
    const float g = __half2float(gate[i]);
    const float s = __half2float(__float2half_rn(g / (1.0f + __expf(-g))));
    out[i] = __float2half_rn(s * __half2float(up[i]));
  }
}

// logits = f16(E h) for a dense binary16 head (Head::project, model.rs:578-587);
// one wavefront per row at a time, 16-byte loads, f32 accumulate.  Every
// wavefront also leaves its best (value, row), lowest row on ties.
constexpr int kHeadThreads = 256;
__global__ __launch_bounds__(kHeadThreads) void lm_head_kernel(const __half* __restrict__ E, const __half* __restrict__ h,
                                                               uint32_t vocab, uint32_t hidden, float* __restrict__ logits,
                                                               float* __restrict__ best_val, uint32_t* __restrict__ best_idx) {
  extern __shared__ __align__(16) float hs[];  // [hidden]
  for (uint32_t i = threadIdx.x; i < hidden; i += kHeadThreads) hs[i] = __half2float(h[i]);
  __syncthreads();
  const uint32_t lane = threadIdx.x & 63u;
  const uint32_t gw = blockIdx.x * (kHeadThreads / 64) + (threadIdx.x >> 6), nw = gridDim.x * (kHeadThreads / 64);
  const uint32_t chunks = hidden >> 3;  // 16-byte units per row
  float bv = -INFINITY;
  uint32_t bi = 0xFFFFFFFFu;
  for (uint32_t r = gw; r < vocab; r += nw) {
    const uint4* row = reinterpret_cast<const uint4*>(E + (size_t)r * hidden);
    float a = 0.f;
    for (uint32_t c = lane; c < chunks; c += 64) {
      const uint4 u = row[c];
      const uint32_t wv[4] = {u.x, u.y, u.z, u.w};
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        a = fmaf(__half2float(__ushort_as_half((unsigned short)(wv[j] & 0xFFFFu))), hs[8 * c + 2 * j], a);
        a = fmaf(__half2float(__ushort_as_half((unsigned short)(wv[j] >> 16))), hs[8 * c + 2 * j + 1], a);
      }
    }
    a = wave_sum(a);
    const float l = __half2float(__float2half_rn(a));
    if (lane == 0) logits[r] = l;
    if (l > bv) {  // rows ascend inside a wavefront, so '>' keeps the lowest row of a tie
      bv = l;
      bi = r;
    }
  }
  if (lane == 0) {
    best_val[gw] = bv;
    best_idx[gw] = bi;
  }
}

// ---- int8 embedding / head (llvq-llm/kernels/emb_q8.cu) --------------------------------
// One byte per weight, binary16 scale and bias per group of 64 along the row
// (llvq-artifact/src/sealed.rs:64-78): weight = f32(s * q) + b.
constexpr uint32_t kEmbedGroup = 64;
struct QuantRows {
  const uint8_t* q;      // [rows, d]
  const __half* scales;  // [rows, ceil(d / 64)]
  const __half* biases;
};

__device__ __forceinline__ float q8_weight(uint32_t q, float s, float b) {
  return __fadd_rn(__fmul_rn(s, (float)q), b);
}

// h = f16(embedding row of *token)   (emb_q8_gather)
__global__ __launch_bounds__(256) void embed_q8_kernel(QuantRows e, const uint32_t* __restrict__ token, uint32_t vocab,
                                                       uint32_t hidden, __half* __restrict__ h) {
  const uint32_t t = min(token[blockIdx.y], vocab - 1u);
  h += (size_t)blockIdx.y * hidden;
  const uint32_t gpr = (hidden + kEmbedGroup - 1) / kEmbedGroup;
  for (uint32_t c = blockIdx.x * blockDim.x + threadIdx.x; c < hidden; c += gridDim.x * blockDim.x) {
    const size_t g = (size_t)t * gpr + c / kEmbedGroup;
    h[c] = __float2half_rn(q8_weight(e.q[(size_t)t * hidden + c], __half2float(e.scales[g]), __half2float(e.biases[g])));
  }
}

// logits = f16(E h) for the int8 head (tv_q8_h): one wavefront per row at a time,
// 16 codes per lane and load (a 16-byte run never straddles a group of 64).
__global__ __launch_bounds__(kHeadThreads) void lm_head_q8_kernel(QuantRows e, const __half* __restrict__ h, uint32_t vocab,
                                                                  uint32_t hidden, float* __restrict__ logits,
                                                                  float* __restrict__ best_val, uint32_t* __restrict__ best_idx) {
  extern __shared__ __align__(16) float hs[];  // [hidden]
  for (uint32_t i = threadIdx.x; i < hidden; i += kHeadThreads) hs[i] = __half2float(h[i]);
  __syncthreads();
  const uint32_t lane = threadIdx.x & 63u;
  const uint32_t gw = blockIdx.x * (kHeadThreads / 64) + (threadIdx.x >> 6), nw = gridDim.x * (kHeadThreads / 64);
  const uint32_t chunks = hidden >> 4, gpr = (hidden + kEmbedGroup - 1) / kEmbedGroup;
  float bv = -INFINITY;
  uint32_t bi = 0xFFFFFFFFu;
  for (uint32_t r = gw; r < vocab; r += nw) {
    const uint4* row = reinterpret_cast<const uint4*>(e.q + (size_t)r * hidden);
    float a = 0.f;
    for (uint32_t c = lane; c < chunks; c += 64) {
      const uint4 u = row[c];
      const float s = __half2float(e.scales[(size_t)r * gpr + (c >> 2)]), b = __half2float(e.biases[(size_t)r * gpr + (c >> 2)]);
      const uint32_t wv[4] = {u.x, u.y, u.z, u.w};
#pragma unroll
      for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int t = 0; t < 4; ++t) a = fmaf(q8_weight((wv[j] >> (8 * t)) & 0xFFu, s, b), hs[16 * c + 4 * j + t], a);
    }
    a = wave_sum(a);
    const float l = __half2float(__float2half_rn(a));
    if (lane == 0) logits[r] = l;
    if (l > bv) {
      bv = l;
      bi = r;
    }
  }
  if (lane == 0) {
    best_val[gw] = bv;
    best_idx[gw] = bi;
  }
}

// token = argmax over the wavefront winners; lowest row on ties
__global__ __launch_bounds__(1024) void argmax_final_kernel(const float* __restrict__ best_val, const uint32_t* __restrict__ best_idx,
                                                            uint32_t n, uint32_t* __restrict__ token_out,
                                                            uint32_t* __restrict__ history, uint32_t slot) {
  __shared__ float sv[1024];
  __shared__ uint32_t si[1024];
  float bv = -INFINITY;
  uint32_t bi = 0xFFFFFFFFu;
  for (uint32_t i = threadIdx.x; i < n; i += 1024) {
    const float v = best_val[i];
    const uint32_t id = best_idx[i];
    if (v > bv || (v == bv && id < bi)) {
      bv = v;
      bi = id;
    }
  }
  sv[threadIdx.x] = bv;
  si[threadIdx.x] = bi;
  __syncthreads();
  for (uint32_t s = 512; s >= 1; s >>= 1) {
    if (threadIdx.x < s) {
      const float v = sv[threadIdx.x + s];
      const uint32_t id = si[threadIdx.x + s];
      if (v > sv[threadIdx.x] || (v == sv[threadIdx.x] && id < si[threadIdx.x])) {
        sv[threadIdx.x] = v;
        si[threadIdx.x] = id;
      }
    }
    __syncthreads();
  }
  if (threadIdx.x == 0) {
    *token_out = si[0];
    if (history) history[slot] = si[0];
  }
}

__global__ void set_token_kernel(uint32_t* token, uint32_t value) { *token = value; }

}  // namespace llvq
