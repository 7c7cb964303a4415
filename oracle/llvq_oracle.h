/* CPU oracle for the LLVQ fused dequant-GEMV path.  TEST INFRASTRUCTURE ONLY.
 *
 * A plain-C restatement of the reference's CPU algorithm, used as the checker
 * in tests, in the smoke test and as the timed CPU baseline of the benchmark.
 * Nothing in the shipped library links, loads or calls this file; the product
 * has its own table builder and its own decoder.
 *
 * Each function cites the reference file:line it restates (paths relative to
 * the reference checkout).  How each one is pinned is listed beside it in
 * llvq_oracle.c.
 */
#ifndef LLVQ_ORACLE_H
#define LLVQ_ORACLE_H
#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define ORC_DIM 24
#define ORC_N13 280974212784720ULL /* llvq-core/src/leech.rs:54 */

/* llvq-artifact/src/error.rs:11-45 — one code per variant. */
enum orc_err {
  ORC_OK = 0,
  ORC_NOT_AN_ARTIFACT = 1,
  ORC_TRUNCATED = 2,
  ORC_BAD_NAME = 3,
  ORC_UNEXPECTED_NAME = 4,
  ORC_INCONSISTENT = 5,
  ORC_POINT_OUTSIDE_CODEBOOK = 6,
  ORC_INDEX_TOO_WIDE = 7,
  ORC_INDEX_OUT_OF_RANGE = 8,
  ORC_BAD_RAW_ENCODING = 9,
  ORC_CODEBOOK_MISMATCH = 10,
  ORC_UNKNOWN_VERSION = 11,
  ORC_IO = 12
};

/* ---- llvq-core ---------------------------------------------------------- */
uint64_t orc_clmul(uint64_t a, uint64_t b);          /* golay.rs:32-42 */
const uint32_t* orc_golay_codewords(void);           /* golay.rs:62-81, :99 — 4096 words */
int orc_golay_of_weight(int w, const uint32_t** out); /* golay.rs:106-111 — returns count */
int orc_golay_contains(uint32_t word);               /* golay.rs:86-95 */
int orc_leech_contains(const int32_t p[ORC_DIM]);    /* leech.rs:76-99 */
int64_t orc_shell_index(const int32_t p[ORC_DIM]);   /* leech.rs:132-142; -1 when 16 does not divide the norm */
/* shells.rs:66-143 — every point of shell 2 or 3 exactly once; returns count,
 * 0 for an unsupported shell.  `out` may be NULL (count only). */
size_t orc_enumerate_shell(int m, int32_t* out /* count*24 */, size_t cap_points);
/* llvq-search/tests/g3_index.rs:41-60 on every stride-th point of shell 2 or 3:
 * count of enumerated points, or a negative failure code. */
long long orc_shell_roundtrip_check(int m, size_t stride, uint64_t lo, uint64_t hi);

/* rng.rs:21-40 */
uint64_t orc_splitmix_next(uint64_t* state);
double orc_splitmix_f64(uint64_t* state);
double orc_splitmix_gaussian(uint64_t* state);

/* ---- llvq-search -------------------------------------------------------- */
int orc_n_classes(void);                             /* 383 */
/* classes.rs:144-254 + index.rs:125-176 layout.  Any out pointer may be NULL. */
void orc_class_info(int ci, uint64_t* lo, uint64_t* hi, int* shell, int* odd,
                    int* w, int* n_levels);
uint64_t orc_shell_cardinality(int m);               /* classes.rs:259-273 */
int orc_index_bits(uint32_t cap);                    /* llvq-quant/src/quantizer.rs:572-576 */

/* index.rs:334-435 (u128, factorial multinomials).  Returns 1, or 0 for idx > N13. */
int orc_index_decode(uint64_t idx, int32_t out[ORC_DIM]);
/* index.rs:190-330.  Returns 1 and *idx, or 0 for a point outside the ball. */
int orc_index_encode(const int32_t p[ORC_DIM], uint64_t* idx);
/* fastdec.rs:321-399 (u64 recurrence).  Same contract as orc_index_decode. */
int orc_fast_decode(uint64_t idx, int32_t out[ORC_DIM]);
/* n indices -> n*24 int8 coordinates with either decoder; ORC_INDEX_OUT_OF_RANGE on a bad index. */
int orc_decode_batch(const uint64_t* idx, size_t n, int8_t* out, int fast);
int orc_class_of(uint64_t idx);                      /* fastdec.rs:293-298; -1 for 0 and > N13 */
/* fastdec.rs:402-433 — canonical level table of a class. */
void orc_class_levels(int ci, int32_t values[5], uint8_t counts[5], int* len,
                      int* nonzero);

/* pack.rs:48-137 — MSB-first dense bit stream. */
typedef struct orc_bitw orc_bitw;
orc_bitw* orc_bitw_new(void);
int orc_bitw_push(orc_bitw*, uint64_t value, uint32_t width); /* 0, or -1 when value does not fit */
size_t orc_bitw_finish(orc_bitw*, uint8_t** bytes);           /* frees the writer; caller frees *bytes with orc_free */
uint64_t orc_bitr_read(const uint8_t* buf, uint64_t* bitpos, uint32_t width);
void orc_free(void* p);

/* ---- llvq-artifact ------------------------------------------------------ */
uint64_t orc_codebook_fingerprint(void);             /* codebook.rs:129-185 */

typedef struct {
  char* name;
  uint32_t d_out, d_in, shell_cap, n_centroids;
  uint64_t rot_seed;
  uint32_t has_rot;
  double* centroids;   /* n_centroids */
  double* row_scales;  /* d_out */
  double* tail;        /* d_out * (d_in % 24), widened from the stored f32 */
  uint64_t* indices;   /* d_out * (d_in / 24) */
  uint32_t* gains;
  size_t nblocks_total;
  /* byte range of the packed code stream inside the buffer that was parsed */
  size_t code_off, code_len;
} orc_raw_matrix;

/* format.rs:563-619.  version and matrix count out; checks the fingerprint for v4. */
int orc_read_header(const uint8_t* buf, size_t len, size_t* pos, uint32_t* version,
                    uint32_t* n_matrices, const char** what);
size_t orc_write_header(uint8_t* out /* >= 16 bytes */, uint32_t version, uint32_t n_matrices);
/* format.rs:301-382 */
int orc_read_matrix_raw(const uint8_t* buf, size_t len, size_t* pos, orc_raw_matrix* m,
                        const char** what);
void orc_raw_matrix_free(orc_raw_matrix* m);
/* format.rs:238-298.  Returns an orc_err; *out is malloc'd (orc_free). */
int orc_write_matrix_raw(const orc_raw_matrix* m, uint8_t** out, size_t* out_len);

/* ---- llvq-quant/src/rotation.rs: the incoherence rotation Q ------------- */
/* Q = (S (x) I_m) (I_k (x) H_m / sqrt m) D, n = m k with m the power-of-two part of n:
 * signs D from the seed's Gaussian stream (rotation.rs:66-69), one Walsh-Hadamard
 * transform per group of m (:201-222), a k x k orthonormal S by Gram-Schmidt on
 * Gaussian rows, applied across groups (:119-143, :226-247). */
typedef struct {
  size_t n, m, k;
  double* signs; /* n, +1 / -1 */
  double* small; /* k * k, row-major */
} orc_rotation;
int orc_rotation_new(size_t n, uint64_t seed, orc_rotation* r); /* rotation.rs:60-79 */
void orc_rotation_free(orc_rotation* r);
void orc_rotation_apply(const orc_rotation* r, double* v);           /* v <- Q v,   :97-105 */
void orc_rotation_apply_transpose(const orc_rotation* r, double* v); /* v <- Q^T v, :108-117 */

/* llvq-quant/src/quantizer.rs:354-367 */
void orc_reconstruct(const int32_t p[ORC_DIM], uint32_t gain, const double* centroids,
                     double row_scale, double out[ORC_DIM]);
/* format.rs:385-439: decode every index (Indexer::decode) then rebuild the
 * d_out x d_in weights in f64, un-rotate every row when the record carries a
 * rotation seed (format.rs:435-437), then narrow to f32. */
int orc_decode_matrix(const orc_raw_matrix* m, float* w /* d_out*d_in */);
/* llvq-artifact/tests/fused_path_matches_dense.rs:96-136: the activation is
 * rotated first when the record carries a rotation seed (:110-115), then
 * y_r = sum_b k_b sum_j p_bj xr_j + tail.xr, all f64.  abs_out (may be NULL)
 * receives sum |w_i x_i| per row, the error normaliser of
 * llvq-cuda/src/bin/matvec.rs:114-120. */
int orc_fused_product(const orc_raw_matrix* m, const double* x, double* y, double* abs_out);
/* f64 GEMV over the f32 weights of orc_decode_matrix
 * (fused_path_matches_dense.rs:149-151). */
void orc_dense_matvec(const float* w, size_t d_out, size_t d_in, const double* x, double* y);

/* sealed.rs:47-62 */
float orc_f16_to_f32(uint16_t h);
/* llvq-cuda/src/lib.rs:60-96 — round-to-nearest-even narrow */
uint16_t orc_f32_to_f16(float f);

/* ---- timed CPU baseline ------------------------------------------------- */
/* FastDecoder decode + reconstruct scale + f32 dot against an f16 activation,
 * rows split over `threads` pthreads.  codes = packed 6-byte records
 * (cap 12, one gain bit).  Returns 0, or an orc_err. */
int orc_cpu_gemv(const uint8_t* codes, size_t d_out, size_t d_in, const double* centroids,
                 const double* row_scales, const float* tail, const uint16_t* x_f16,
                 float* y, int threads);
/* decode-only loop over packed 6-byte records, single thread; returns a
 * checksum so the work cannot be optimised away. */
uint64_t orc_cpu_decode_only(const uint8_t* codes, size_t nblocks);

#ifdef __cplusplus
}
#endif
#endif
