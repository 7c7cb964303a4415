// C ABI and gfx950 kernels of the fused Leech-lattice dequant-GEMV.
//
// Data layout in HBM, per matrix: the packed code stream exactly as the file
// holds it (6 bytes per block, big-endian (idx << 1) | gain, rows
// back to back), f32 row scales, f32 tail columns, two f32 gain centroids.
// Per runtime: one 45 KB table image (Golay words, class records, class ends,
// reciprocals) that every workgroup copies into LDS.
#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstring>
#include <string>
#include <vector>

#include "../../include/llvq_hip.h"
#include "artifact.hpp"
#include "codebook.hpp"
#include "decode_core.h"

namespace llvq {

// ---- table image --------------------------------------------------------------
struct TableImage {
  uint32_t golay[4096];
  DevClass cls[kClassSlots];
  uint64_t ends[kEndsPadded];
  double rcp[32];
};
static_assert(sizeof(TableImage) % 16 == 0, "table image is copied in 16-byte units");

__device__ __forceinline__ DecodeTables stage_tables(uint8_t* smem, const TableImage* g) {
  const uint4* src = reinterpret_cast<const uint4*>(g);
  uint4* dst = reinterpret_cast<uint4*>(smem);
  for (uint32_t i = threadIdx.x; i < sizeof(TableImage) / 16; i += blockDim.x) dst[i] = src[i];
  const TableImage* s = reinterpret_cast<const TableImage*>(smem);
  return DecodeTables{s->golay, s->cls, s->ends, s->rcp};
}

__device__ __forceinline__ uint64_t load_record(const uint8_t* codes, size_t block) {
  // 6-byte big-endian record; the stream is 2-byte aligned at every block.
  const uint16_t* p = reinterpret_cast<const uint16_t*>(codes + 6 * block);
  auto be16 = [](uint32_t h) { return ((h & 0xFFu) << 8) | (h >> 8); };
  return ((uint64_t)be16(p[0]) << 32) | ((uint64_t)be16(p[1]) << 16) | (uint64_t)be16(p[2]);
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) v += __shfl_xor(v, off, 64);
  return v;
}

// ---- parity probe: unrank records to points -----------------------------------
__global__ __launch_bounds__(256) void decode_blocks_kernel(const TableImage* __restrict__ tables,
                                                            const uint8_t* __restrict__ codes,
                                                            size_t nblocks, int8_t* __restrict__ points,
                                                            uint8_t* __restrict__ gains,
                                                            uint8_t* __restrict__ shells) {
  extern __shared__ __align__(16) uint8_t smem[];
  const DecodeTables T = stage_tables(smem, tables);
  __syncthreads();
  for (size_t b = (size_t)blockIdx.x * blockDim.x + threadIdx.x; b < nblocks;
       b += (size_t)gridDim.x * blockDim.x) {
    const uint64_t rec = load_record(codes, b);
    int8_t* out = points + b * kDim;
    const int ci = decode_index(T, rec >> 1, [&](int p, int v) { out[p] = (int8_t)v; });
    if (gains) gains[b] = (uint8_t)(rec & 1);
    if (shells) shells[b] = ci >= 0 ? (uint8_t)T.cls[ci].shell : (ci == -1 ? 0 : 0xFF);
  }
}

// ---- fused dequant-GEMV, one wavefront per output row -------------------------
struct GemvArgs {
  const TableImage* tables;
  const uint8_t* codes;
  const float* rscale;
  const float* tail;
  float g0, g1;
  uint32_t d_out, nblocks, tail_w;
};

template <typename OutT>
__device__ __forceinline__ void store_out(OutT* y, uint32_t r, float v);
template <>
__device__ __forceinline__ void store_out<float>(float* y, uint32_t r, float v) { y[r] = v; }
template <>
__device__ __forceinline__ void store_out<__half>(__half* y, uint32_t r, float v) { y[r] = __float2half_rn(v); }

template <typename OutT>
__global__ __launch_bounds__(256) void gemv_rows_kernel(GemvArgs a, const __half* __restrict__ x,
                                                        OutT* __restrict__ y) {
  extern __shared__ __align__(16) uint8_t smem[];
  const DecodeTables T = stage_tables(smem, a.tables);
  float* xs = reinterpret_cast<float*>(smem + sizeof(TableImage));
  const uint32_t d_in = a.nblocks * kDim + a.tail_w;
  for (uint32_t i = threadIdx.x; i < d_in; i += blockDim.x) xs[i] = __half2float(x[i]);
  __syncthreads();

  const uint32_t lane = threadIdx.x & 63u;
  const uint32_t wave = threadIdx.x >> 6;
  const uint32_t waves = (blockDim.x >> 6) * gridDim.x;
  for (uint32_t row = blockIdx.x * (blockDim.x >> 6) + wave; row < a.d_out; row += waves) {
    float acc = 0.f;
    for (uint32_t b = lane; b < a.nblocks; b += 64u) {
      const uint64_t rec = load_record(a.codes, (size_t)row * a.nblocks + b);
      const float* xb = xs + b * kDim;
      float dot = 0.f;
      const int ci = decode_index(T, rec >> 1, [&](int p, int v) { dot = fmaf((float)v, xb[p], dot); });
      const float g = (rec & 1) ? a.g1 : a.g0;
      const float s = ci >= 0 ? T.cls[ci].inv_norm * g : 0.f;
      acc = fmaf(dot, s, acc);
    }
    float v = acc * a.rscale[row];
    if (lane < a.tail_w) v = fmaf(a.tail[(size_t)row * a.tail_w + lane], xs[a.nblocks * kDim + lane], v);
    v = wave_sum(v);
    if (lane == 0) store_out<OutT>(y, row, v);
  }
}

}  // namespace llvq

// =================================================================================
// C ABI
// =================================================================================
using namespace llvq;

struct llvq_rt {
  int device = 0;
  hipStream_t stream = nullptr;
  TableImage* tables = nullptr;  // device
  int cu_count = 0;
};

struct llvq_mat {
  std::string name;
  uint32_t d_out = 0, d_in = 0, nblocks = 0, tail_w = 0;
  float g[2] = {0, 0};
  uint8_t* codes = nullptr;  // device
  float* rscale = nullptr;   // device
  float* tail = nullptr;     // device
  uint64_t device_bytes = 0;
  uint64_t encoded_bytes = 0;
};

static thread_local std::string g_last_error;

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
  std::vector<uint8_t> host(sizeof(TableImage));
  auto* img = reinterpret_cast<TableImage*>(host.data());
  std::memcpy(img->golay, cb.golay, sizeof img->golay);
  std::memcpy(img->cls, cb.dev_classes, sizeof img->cls);
  std::memcpy(img->ends, cb.ends, sizeof img->ends);
  std::memcpy(img->rcp, cb.rcp, sizeof img->rcp);
  e = hipMalloc(reinterpret_cast<void**>(&rt->tables), sizeof(TableImage));
  if (e != hipSuccess) { delete rt; return hip_fail(e, "hipMalloc(tables)"); }
  e = hipMemcpy(rt->tables, host.data(), sizeof(TableImage), hipMemcpyHostToDevice);
  if (e != hipSuccess) { (void)hipFree(rt->tables); delete rt; return hip_fail(e, "hipMemcpy(tables)"); }
  // the activation tile of a wide matrix pushes dynamic LDS past the 64 KB default
  const int max_lds = 160 * 1024;
  (void)hipFuncSetAttribute(reinterpret_cast<const void*>(gemv_rows_kernel<float>), hipFuncAttributeMaxDynamicSharedMemorySize, max_lds);
  (void)hipFuncSetAttribute(reinterpret_cast<const void*>(gemv_rows_kernel<__half>), hipFuncAttributeMaxDynamicSharedMemorySize, max_lds);
  *out = rt;
  return LLVQ_OK;
}

void llvq_hip_runtime_destroy(llvq_rt* rt) {
  if (!rt) return;
  (void)hipSetDevice(rt->device);
  (void)hipFree(rt->tables);
  delete rt;
}

int llvq_hip_synchronize(llvq_rt* rt) {
  if (!rt) return fail(LLVQ_ERR_INVALID_ARGUMENT, "synchronize: runtime is null");
  HIP_TRY(hipStreamSynchronize(rt->stream));
  return LLVQ_OK;
}

static int upload_impl(llvq_rt* rt, const std::string& name, uint32_t d_out, uint32_t d_in,
                       uint32_t shell_cap, uint32_t n_centroids, const double* centroids,
                       const double* row_scales, const float* tail, const uint8_t* codes,
                       size_t code_bytes, bool has_rotation, llvq_mat** out) {
  if (shell_cap > (uint32_t)kMaxShell)
    return fail(LLVQ_ERR_INCONSISTENT, name + ": shell cap " + std::to_string(shell_cap) +
                                           " exceeds the supported ball (m <= 13)");
  // one gain bit is compiled into the kernels (llvq-llm/src/fused.rs:1168-1177)
  if (n_centroids != 2)
    return fail(LLVQ_ERR_UNSUPPORTED, name + ": " + std::to_string(n_centroids) +
                                          " centroids, but the kernels hard-code 1 gain bit");
  const int ib = index_bits(shell_cap);
  if (ib + 1 != 48)
    return fail(LLVQ_ERR_UNSUPPORTED, name + ": shell cap " + std::to_string(shell_cap) + " packs " +
                                          std::to_string(ib + 1) +
                                          " bits per block; the kernels read 6-byte records (cap 12)");
  if (has_rotation)
    return fail(LLVQ_ERR_UNSUPPORTED, name + ": stored in a rotated basis; activation rotation is not built yet");
  const uint32_t nblocks = d_in / kDim, tail_w = d_in % kDim;
  const uint64_t total_blocks = (uint64_t)d_out * nblocks;
  if ((unsigned __int128)total_blocks * 48 > (unsigned __int128)code_bytes * 8)
    return fail(LLVQ_ERR_TRUNCATED, "file ends mid-code stream");
  if (d_out == 0 || d_in == 0) return fail(LLVQ_ERR_INVALID_ARGUMENT, name + ": empty matrix");
  if ((total_blocks && !codes) || !centroids || !row_scales || (tail_w && !tail))
    return fail(LLVQ_ERR_INVALID_ARGUMENT, name + ": a required array is null");
  // Index range (format.rs:389-392).  The bound is N(13) whatever the cap; a
  // 47-bit field cannot exceed it (2^47 < N(13)), so at cap 12 this never fires.
  if (ib < 64 && ((1ULL << ib) - 1) > kN13) {
    for (uint64_t b = 0; b < total_blocks; ++b) {
      const uint8_t* p = codes + 6 * b;
      const uint64_t v = ((uint64_t)p[0] << 40) | ((uint64_t)p[1] << 32) | ((uint64_t)p[2] << 24) |
                         ((uint64_t)p[3] << 16) | ((uint64_t)p[4] << 8) | p[5];
      if ((v >> 1) > kN13)
        return fail(LLVQ_ERR_INDEX_OUT_OF_RANGE,
                    name + ": index " + std::to_string(v >> 1) + " is not a codebook member");
    }
  }

  HIP_TRY(hipSetDevice(rt->device));
  auto* m = new llvq_mat();
  m->name = name;
  m->d_out = d_out;
  m->d_in = d_in;
  m->nblocks = nblocks;
  m->tail_w = tail_w;
  m->g[0] = (float)centroids[0];  // fused.rs:1209
  m->g[1] = (float)centroids[1];
  std::vector<float> rs(d_out);
  for (uint32_t r = 0; r < d_out; ++r) rs[r] = (float)row_scales[r];  // fused.rs:1210
  const size_t code_len = (size_t)total_blocks * 6;
  const size_t code_alloc = code_len + 64;  // slack so wide loads may run past the last record
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
  if ((e = hipMalloc(reinterpret_cast<void**>(&m->rscale), d_out * sizeof(float))) != hipSuccess) return cleanup(e, "hipMalloc(rscale)");
  if ((e = hipMemcpy(m->rscale, rs.data(), d_out * sizeof(float), hipMemcpyHostToDevice)) != hipSuccess) return cleanup(e, "hipMemcpy(rscale)");
  // zero-length arrays become one-element dummies (fused_cuda.rs:1084-1098)
  if ((e = hipMalloc(reinterpret_cast<void**>(&m->tail), tail_len ? tail_len : sizeof(float))) != hipSuccess) return cleanup(e, "hipMalloc(tail)");
  if (tail_len && (e = hipMemcpy(m->tail, tail, tail_len, hipMemcpyHostToDevice)) != hipSuccess) return cleanup(e, "hipMemcpy(tail)");
  m->device_bytes = code_alloc + d_out * sizeof(float) + (tail_len ? tail_len : sizeof(float));
  m->encoded_bytes = code_len + (uint64_t)d_out * 8 + tail_len + 16;
  *out = m;
  return LLVQ_OK;
}

int llvq_hip_matrix_upload(llvq_rt* rt, const llvq_matrix_desc* d, llvq_mat** out) {
  if (!rt || !d || !out) return fail(LLVQ_ERR_INVALID_ARGUMENT, "matrix_upload: null argument");
  *out = nullptr;
  return upload_impl(rt, d->name ? d->name : "", d->d_out, d->d_in, d->shell_cap, d->n_centroids,
                     d->centroids, d->row_scales, d->tail, d->codes, d->code_bytes,
                     d->has_rotation != 0, out);
}

int llvq_hip_read_header(const uint8_t* buf, size_t len, size_t* pos, uint32_t* version,
                         uint32_t* n_matrices) {
  if (!buf || !pos || !version || !n_matrices || *pos > len)
    return fail(LLVQ_ERR_INVALID_ARGUMENT, "read_header: bad argument");
  std::string err;
  const int rc = parse_header(buf, len, pos, version, n_matrices, &err);
  return rc ? fail(rc, err) : LLVQ_OK;
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
                   r.row_scales.data(), r.tail.data(), r.codes, r.code_bytes, r.has_rotation, out);
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

static int launch_gemv(llvq_rt* rt, const llvq_mat* m, const void* x, void* y, int y_dtype) {
  GemvArgs a{rt->tables, m->codes, m->rscale, m->tail, m->g[0], m->g[1], m->d_out, m->nblocks, m->tail_w};
  const size_t lds = sizeof(TableImage) + (size_t)m->d_in * sizeof(float);
  if (lds > 160 * 1024)
    return fail(LLVQ_ERR_UNSUPPORTED, m->name + ": d_in " + std::to_string(m->d_in) + " does not fit the LDS activation tile");
  const uint32_t waves_per_wg = 4;
  uint32_t grid = (m->d_out + waves_per_wg - 1) / waves_per_wg;
  const uint32_t cap = (uint32_t)(rt->cu_count > 0 ? rt->cu_count : 256) * 2;
  if (grid > cap) grid = cap;
  if (y_dtype == LLVQ_F32) {
    hipLaunchKernelGGL(gemv_rows_kernel<float>, dim3(grid), dim3(256), lds, rt->stream, a,
                       reinterpret_cast<const __half*>(x), reinterpret_cast<float*>(y));
  } else if (y_dtype == LLVQ_F16) {
    hipLaunchKernelGGL(gemv_rows_kernel<__half>, dim3(grid), dim3(256), lds, rt->stream, a,
                       reinterpret_cast<const __half*>(x), reinterpret_cast<__half*>(y));
  } else {
    return fail(LLVQ_ERR_INVALID_ARGUMENT, "gemv: unknown output dtype");
  }
  HIP_TRY(hipGetLastError());
  return LLVQ_OK;
}

int llvq_hip_gemv(llvq_rt* rt, const llvq_mat* m, const void* x, void* y, int y_dtype) {
  if (!rt || !m || !x || !y) return fail(LLVQ_ERR_INVALID_ARGUMENT, "gemv: null argument");
  HIP_TRY(hipSetDevice(rt->device));
  return launch_gemv(rt, m, x, y, y_dtype);
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
  for (int i = 0; i < n; ++i) {
    const int rc = launch_gemv(rt, mats[i], x, y[i], y_dtype);
    if (rc) return rc;
  }
  return LLVQ_OK;
}

int llvq_hip_gemm(llvq_rt* rt, const llvq_mat* m, const void* x, int M, void* y, int y_dtype) {
  if (!rt || !m || !x || !y || M < 0) return fail(LLVQ_ERR_INVALID_ARGUMENT, "gemm: bad argument");
  HIP_TRY(hipSetDevice(rt->device));
  const size_t esz = y_dtype == LLVQ_F32 ? 4 : 2;
  if (y_dtype != LLVQ_F32 && y_dtype != LLVQ_F16) return fail(LLVQ_ERR_INVALID_ARGUMENT, "gemm: unknown output dtype");
  for (int r = 0; r < M; ++r) {
    const int rc = launch_gemv(rt, m, reinterpret_cast<const uint8_t*>(x) + (size_t)r * m->d_in * 2,
                               reinterpret_cast<uint8_t*>(y) + (size_t)r * m->d_out * esz, y_dtype);
    if (rc) return rc;
  }
  return LLVQ_OK;
}

int llvq_hip_decode_blocks(llvq_rt* rt, const uint8_t* codes_dev, size_t nblocks, int8_t* points_dev,
                           uint8_t* gains_dev, uint8_t* shells_dev) {
  if (!rt) return fail(LLVQ_ERR_INVALID_ARGUMENT, "decode_blocks: runtime is null");
  if (nblocks == 0) return LLVQ_OK;  // an empty stream is valid and writes nothing
  if (!points_dev || !codes_dev) return fail(LLVQ_ERR_INVALID_ARGUMENT, "decode_blocks: null argument");
  HIP_TRY(hipSetDevice(rt->device));
  size_t grid = (nblocks + 255) / 256;
  const size_t cap = (size_t)(rt->cu_count > 0 ? rt->cu_count : 256) * 2;
  if (grid > cap) grid = cap;
  hipLaunchKernelGGL(decode_blocks_kernel, dim3((uint32_t)grid), dim3(256), sizeof(TableImage), rt->stream,
                     rt->tables, codes_dev, nblocks, points_dev, gains_dev, shells_dev);
  HIP_TRY(hipGetLastError());
  return LLVQ_OK;
}

}  // extern "C"
