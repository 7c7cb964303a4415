/* A caller of the C ABI with no Python and no C++ in it: what the llvq-hip crate does through
 * its extern block, written in C so that it builds where Rust is not installed.
 *
 * It makes a small LLVQ matrix (random cap-12 ranks and gain bits, two centroids, a row scale
 * per row, f32 tail columns), uploads it, and runs the single-row product, the batched product
 * and the batched product that allocates nothing; every output is checked against a plain loop
 * over the library's own host decoder (llvq_hip_host_decode: the same index map, no GPU).
 *
 *   gcc -std=c11 -I include -I /opt/rocm/include llvq-hip/examples/c_caller.c \
 *       -L llvq_amd/csrc -lllvq_hip -L /opt/rocm/lib -lamdhip64 -lm -o c_caller
 *
 * Exit status 0 and "ok" on success; a message and a non-zero status otherwise. */
#define __HIP_PLATFORM_AMD__ 1
#include <hip/hip_runtime_api.h>
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "llvq_hip.h"

static uint64_t state = 0x9E3779B97F4A7C15ULL;
static uint64_t next_u64(void) { /* SplitMix64 */
  uint64_t z = (state += 0x9E3779B97F4A7C15ULL);
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ULL;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBULL;
  return z ^ (z >> 31);
}

/* binary16 bits of k / 8 for a small integer k (every such value is exact in binary16) */
static uint16_t half_of_eighths(int k) {
  if (k == 0) return 0;
  int e = 0;
  const double fr = frexp(fabs(k / 8.0), &e); /* |k| / 8 = fr * 2^e, fr in [0.5, 1) */
  const unsigned mant = (unsigned)((fr * 2.0 - 1.0) * 1024.0);
  return (uint16_t)((k < 0 ? 0x8000u : 0u) | ((unsigned)(e - 1 + 15) << 10) | mant);
}

#define CHECK(call)                                                                 \
  do {                                                                              \
    int rc_ = (call);                                                               \
    if (rc_ != 0) { fprintf(stderr, "%s: %d: %s\n", #call, rc_, llvq_hip_last_error()); return 2; } \
  } while (0)
#define HIPCHECK(call)                                                              \
  do {                                                                              \
    hipError_t e_ = (call);                                                         \
    if (e_ != hipSuccess) { fprintf(stderr, "%s: %s\n", #call, hipGetErrorString(e_)); return 2; } \
  } while (0)

enum { D_OUT = 96, NB = 21, TAIL = 8, D_IN = NB * 24 + TAIL, M = 40 };

int main(void) {
  static uint8_t codes[D_OUT * NB * 6];
  static uint64_t index_of[D_OUT * NB];
  static uint8_t gain_of[D_OUT * NB];
  static double row_scale[D_OUT];
  static float tail[D_OUT * TAIL];
  static uint16_t x16[M * D_IN];
  static double x[M * D_IN];
  static double want[M * D_OUT], norm[M * D_OUT]; /* the product, and sum |w x| of the same terms */
  static float got[M * D_OUT];
  const double centroids[2] = {0.8, 1.25};

  if (llvq_hip_codebook_fingerprint() != 0x338f420f11866319ULL) { fprintf(stderr, "codebook fingerprint\n"); return 1; }
  for (int b = 0; b < D_OUT * NB; ++b) {
    /* any index below N(12) = 111 043 117 458 000 is a member of the cap-12 ball; 0 is the origin */
    const uint64_t idx = b % 17 == 0 ? 0 : next_u64() % 111043117458000ULL;
    const unsigned gain = (unsigned)(next_u64() & 1);
    const uint64_t rec = (idx << 1) | gain; /* 47-bit index, then the gain bit, most significant bit first */
    for (int k = 0; k < 6; ++k) codes[6 * b + k] = (uint8_t)(rec >> (8 * (5 - k)));
    index_of[b] = idx;
    gain_of[b] = (uint8_t)gain;
  }
  for (int r = 0; r < D_OUT; ++r) row_scale[r] = 0.01 + (double)(next_u64() % 1000) / 20000.0;
  for (int i = 0; i < D_OUT * TAIL; ++i) tail[i] = (float)((int)(next_u64() % 65) - 32) / 1024.0f;
  for (int i = 0; i < M * D_IN; ++i) {
    const int k = (int)(next_u64() % 49) - 24; /* eighths in [-3, 3] */
    x16[i] = half_of_eighths(k);
    x[i] = k / 8.0;
  }
  /* the reference result: reconstruct = point * centroid[gain] * row_scale / sqrt(16 shell) (llvq-core), tail in f32 */
  for (int r = 0; r < D_OUT; ++r) {
    static double w[D_IN];
    for (int b = 0; b < NB; ++b) {
      int8_t pt[24];
      int shell = 0;
      if (llvq_hip_host_decode(index_of[r * NB + b], pt, &shell) != 1) { fprintf(stderr, "host decode refused a valid index\n"); return 1; }
      const double s = shell ? centroids[gain_of[r * NB + b]] / sqrt(16.0 * shell) : 0.0;
      for (int j = 0; j < 24; ++j) w[24 * b + j] = pt[j] * s * (double)(float)row_scale[r];
    }
    for (int t = 0; t < TAIL; ++t) w[24 * NB + t] = tail[r * TAIL + t];
    for (int m = 0; m < M; ++m) {
      double acc = 0, mag = 0;
      for (int c = 0; c < D_IN; ++c) {
        acc += w[c] * x[m * D_IN + c];
        mag += fabs(w[c] * x[m * D_IN + c]);
      }
      want[m * D_OUT + r] = acc;
      norm[m * D_OUT + r] = mag;
    }
  }

  llvq_rt* rt = NULL;
  llvq_mat* mat = NULL;
  CHECK(llvq_hip_runtime_create(0, NULL, &rt));
  llvq_matrix_desc desc;
  memset(&desc, 0, sizeof desc);
  desc.name = "model.layers.0.c_caller.weight";
  desc.d_out = D_OUT;
  desc.d_in = D_IN;
  desc.shell_cap = 12;
  desc.n_centroids = 2;
  desc.centroids = centroids;
  desc.row_scales = row_scale;
  desc.tail = tail;
  desc.codes = codes;
  desc.code_bytes = sizeof codes;
  CHECK(llvq_hip_matrix_upload(rt, &desc, &mat));

  void *xd = NULL, *yd = NULL;
  HIPCHECK(hipMalloc(&xd, sizeof x16));
  HIPCHECK(hipMalloc(&yd, sizeof got));
  HIPCHECK(hipMemcpy(xd, x16, sizeof x16, hipMemcpyHostToDevice));

  double worst[3] = {0, 0, 0};
  for (int pass = 0; pass < 3; ++pass) {
    HIPCHECK(hipMemset(yd, 0xFF, sizeof got));
    if (pass == 0) {
      for (int m = 0; m < M; ++m)
        CHECK(llvq_hip_gemv(rt, mat, (const uint16_t*)xd + (size_t)m * D_IN, (float*)yd + (size_t)m * D_OUT, LLVQ_F32));
    } else if (pass == 1) {
      CHECK(llvq_hip_gemm(rt, mat, xd, M, yd, LLVQ_F32));
    } else {
      CHECK(llvq_hip_gemm_static(rt, mat, xd, M, yd, LLVQ_F32));
    }
    CHECK(llvq_hip_synchronize(rt));
    HIPCHECK(hipMemcpy(got, yd, sizeof got, hipMemcpyDeviceToHost));
    for (int i = 0; i < M * D_OUT; ++i) {
      const double err = fabs((double)got[i] - want[i]) / (norm[i] + 1e-30); /* the norm the library's tests state their bars in */
      if (!(err <= worst[pass])) worst[pass] = err;                          /* written so that a NaN counts */
    }
  }
  printf("max |dy| / sum|w x|: gemv %.3e  gemm %.3e  gemm_static %.3e\n", worst[0], worst[1], worst[2]);
  /* the single-row kernel is exact in the weights (bar 1e-5 in the tests' norm); the batched ones round them to binary16 */
  const int ok = worst[0] < 1e-5 && worst[1] < 1e-3 && worst[2] < 1e-3;

  (void)hipFree(xd);
  (void)hipFree(yd);
  llvq_hip_matrix_free(rt, mat);
  llvq_hip_runtime_destroy(rt);
  if (!ok) { fprintf(stderr, "outputs differ from the host decoder's\n"); return 1; }
  printf("ok\n");
  return 0;
}
