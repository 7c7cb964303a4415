/* llvq_hip.h — C ABI of the MI355X (gfx950) fused Leech-lattice dequant-GEMV/GEMM.
 *
 * This is the boundary a host program binds in place of the reference's
 * quantized-linear operator (llvq-llm/src/fused.rs + fused_cuda.rs).  Plain
 * pointers and sizes only.  Every call returns LLVQ_OK or an llvq_status; the
 * text of the last failure on the calling thread is llvq_hip_last_error().
 *
 * Conventions kept from the reference operator:
 *   - never abort on data: a malformed record is a status code
 *     (llvq-artifact/src/error.rs:11-45, tests/hostile_files.rs);
 *   - exactly two gain centroids / one gain bit (llvq-llm/src/fused.rs:1168-1177);
 *   - every output row is stored, nothing is accumulated into
 *     (llvq-llm/src/fused_cuda.rs:789-797);
 *   - work is enqueued on the runtime's stream and the call returns without
 *     synchronising (fused_cuda.rs:28-34);
 *   - runtime and matrices are immutable after construction; launches are
 *     issued from one thread at a time.
 * Device pointers passed in are caller-owned; llvq_rt and llvq_mat are owned
 * by the library.
 */
#ifndef LLVQ_HIP_H
#define LLVQ_HIP_H
#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Mirrors llvq_artifact::Error (llvq-artifact/src/error.rs:11-45) for the
 * variants that can arise on this path, plus device-side failures. */
typedef enum llvq_status {
  LLVQ_OK = 0,
  LLVQ_ERR_NOT_AN_ARTIFACT = 1,   /* Error::NotAnArtifact */
  LLVQ_ERR_TRUNCATED = 2,         /* Error::Truncated { reading } */
  LLVQ_ERR_BAD_NAME = 3,          /* Error::BadName */
  LLVQ_ERR_INCONSISTENT = 5,      /* Error::Inconsistent */
  LLVQ_ERR_INDEX_TOO_WIDE = 7,    /* Error::IndexTooWide */
  LLVQ_ERR_INDEX_OUT_OF_RANGE = 8,/* Error::IndexOutOfRange */
  LLVQ_ERR_BAD_RAW_ENCODING = 9,  /* Error::BadRawEncoding { tag } */
  LLVQ_ERR_CODEBOOK_MISMATCH = 10,/* Error::CodebookMismatch */
  LLVQ_ERR_UNKNOWN_VERSION = 11,  /* Error::UnknownVersion */
  LLVQ_ERR_INVALID_ARGUMENT = 32, /* null pointer, wrong shape, unsupported dtype */
  LLVQ_ERR_UNSUPPORTED = 33,      /* e.g. centroid count != 2, rotation with an odd factor above 32 */
  LLVQ_ERR_DEVICE = 34            /* a HIP call failed; message carries hipGetErrorString */
} llvq_status;

typedef enum llvq_dtype { LLVQ_F32 = 0, LLVQ_F16 = 1 } llvq_dtype;

typedef struct llvq_rt llvq_rt;   /* replaces FusedRuntime  (fused_cuda.rs:145-180) */
typedef struct llvq_mat llvq_mat; /* replaces FusedProj     (fused_cuda.rs:119-134) */

/* One projection as the file stores it: the fields of RawMatrix
 * (llvq-artifact/src/format.rs:215-229) with the code stream left packed
 * (format.rs:185-203: per block index_bits(cap) bits of index then the gain
 * bit, MSB first — 6 bytes per block at cap 12, 49 bits per block in a dense
 * stream at cap 13, format.rs:87-89). All pointers are host memory.
 * Cap 12 and cap 13 are accepted; other caps are refused by name
 * (LLVQ_ERR_UNSUPPORTED).  A cap-13 matrix is served by llvq_hip_gemv,
 * llvq_hip_gemv_group (a call may mix caps: one launch per cap), llvq_hip_rotate /
 * llvq_hip_gemv_rotated, llvq_hip_sequence_* (the matrices of one sequence share
 * their cap), the decode loop and, as a loop over its rows, by llvq_hip_gemm /
 * llvq_hip_gemm_group and the batched prompt path. */
typedef struct llvq_matrix_desc {
  const char* name;          /* may be NULL */
  uint32_t d_out, d_in;
  uint32_t shell_cap;        /* 12 (6-byte records) or 13 (49-bit blocks, dense) */
  uint32_t n_centroids;      /* must be 2 */
  const double* centroids;   /* [n_centroids] */
  const double* row_scales;  /* [d_out] */
  const float* tail;         /* [d_out * (d_in % 24)], row-major; may be NULL when d_in % 24 == 0 */
  const uint8_t* codes;      /* packed stream, >= ceil(bits per block * d_out * (d_in / 24) / 8) bytes */
  size_t code_bytes;
  uint64_t rotation_seed;
  uint32_t has_rotation;     /* stored as W Q^T: the activation is rotated by Q(d_in, rotation_seed) first */
} llvq_matrix_desc;

/* FusedRuntime::new (fused_cuda.rs:182): builds the Golay / class tables on the
 * host, checks them against the pinned codebook fingerprint, uploads them.
 * `hip_stream` is a hipStream_t (NULL = the device's default stream). */
int llvq_hip_runtime_create(int device, void* hip_stream, llvq_rt** out);
void llvq_hip_runtime_destroy(llvq_rt* rt);

/* codebook_fingerprint (llvq-artifact/src/codebook.rs:182), computed from this
 * library's own tables and host decoder.  Needs no GPU.
 * The published value is 0x338f420f11866319. */
uint64_t llvq_hip_codebook_fingerprint(void);

/* Host-side decode of one index with the library's own tables (the same
 * arithmetic the kernels run).  Returns 1, or 0 for idx > N(13).  Needs no GPU. */
int llvq_hip_host_decode(uint64_t idx, int8_t point[24], int* shell);

/* upload_matrix (fused_cuda.rs:1058): validates, range-checks every index
 * (IndexOutOfRange, format.rs:389-392) and copies the record to the device. */
int llvq_hip_matrix_upload(llvq_rt* rt, const llvq_matrix_desc* desc, llvq_mat** out);

/* read_header (format.rs:588): parses magic, count and, for LVQ4, the
 * fingerprint.  *pos is advanced past the header. */
int llvq_hip_read_header(const uint8_t* buf, size_t len, size_t* pos, uint32_t* version,
                         uint32_t* n_matrices);
/* read_matrix_raw (format.rs:301) without decoding or uploading anything: the
 * shape and byte ranges of the record at buf[*pos..], *pos advanced past it.
 * Needs no GPU.  Offsets are relative to buf. */
typedef struct llvq_record_info {
  char name[256];            /* truncated to 255 bytes, NUL-terminated */
  uint32_t d_out, d_in, shell_cap, n_centroids;
  uint64_t rotation_seed;
  uint32_t has_rotation;
  size_t centroids_off, row_scales_off, tail_off, codes_off;
  size_t code_bytes;
} llvq_record_info;
int llvq_hip_parse_matrix_record(const uint8_t* buf, size_t len, size_t* pos, llvq_record_info* out);

/* read_matrix_raw (format.rs:301) fused with upload: parses one on-disk matrix
 * record at buf[*pos..] and uploads it; the code stream is copied verbatim.
 * *pos is advanced past the record. */
int llvq_hip_matrix_from_record(llvq_rt* rt, const uint8_t* buf, size_t len, size_t* pos,
                                llvq_mat** out);
void llvq_hip_matrix_free(llvq_rt* rt, llvq_mat* m);

/* read_raw (llvq-artifact/src/sealed.rs:277-326): one raw tensor record of the
 * sealed sections that follow the matrices (embedding, norms), as byte ranges
 * of buf; *pos is advanced past it.  version is the file's (records below v3
 * carry no tag and are binary16).  Needs no GPU. */
typedef struct llvq_raw_info {
  char name[256];            /* truncated to 255 bytes, NUL-terminated */
  uint32_t rank;
  uint64_t dims[8];          /* the first 8 */
  uint32_t tag;              /* 0: binary16; 1: int4 / int8 codes + binary16 scale and bias per group */
  uint32_t bits, group;      /* quant only */
  uint64_t count;            /* binary16: values; quant: groups */
  size_t data_off, data_len; /* values, or packed codes */
  size_t scales_off, biases_off;
} llvq_raw_info;
int llvq_hip_parse_raw_tensor(const uint8_t* buf, size_t len, size_t* pos, uint32_t version, llvq_raw_info* out);
/* read_blob (sealed.rs:336-341): config.json, tokenizer.json, ... */
typedef struct llvq_blob_info {
  char name[256];
  size_t data_off, data_len;
} llvq_blob_info;
int llvq_hip_parse_blob(const uint8_t* buf, size_t len, size_t* pos, llvq_blob_info* out);

/* Shape and accounting of an uploaded matrix (FusedMatrix fields, fused.rs:566-588). */
int llvq_hip_matrix_info(const llvq_mat* m, uint32_t* d_out, uint32_t* d_in, uint32_t* nblocks,
                         uint32_t* tail_w, uint64_t* device_bytes);
const char* llvq_hip_matrix_name(const llvq_mat* m);

/* Proj::forward (model.rs:337-345) = rotate + forward_rotated for one activation:
 * y = W x in the natural basis, whatever basis the matrix is stored in.
 * x: d_in binary16 values on the device; y: d_out values of y_dtype. */
int llvq_hip_gemv(llvq_rt* rt, const llvq_mat* m, const void* x_f16_dev, void* y_dev, int y_dtype);

/* FusedRuntime::rotate (fused_cuda.rs:362): one binary16 activation into the
 * basis the matrix was quantized in, x' = Q x with Q = Rotation::new(d_in, seed)
 * (llvq-quant/src/rotation.rs:60-105), as d_in f32 values.  A natural-basis
 * matrix widens the activation unchanged.  Odd factors of d_in above 32 are
 * refused at upload (fused.rs:698-704). */
int llvq_hip_rotate(llvq_rt* rt, const llvq_mat* m, const void* x_f16_dev, float* xr_f32_dev);
/* FusedRuntime::forward_rotated (fused_cuda.rs:384): y = W' xr for an activation
 * already in the matrix's basis (llvq_hip_rotate's output). */
int llvq_hip_gemv_rotated(llvq_rt* rt, const llvq_mat* m, const float* xr_f32_dev, void* y_dev, int y_dtype);
/* The same rotation on the host, from the tables the kernels are handed (sign
 * bitmap, f32 mixing block, f32 1/sqrt m) with f64 arithmetic: v <- Q v.  The
 * check of fused.rs:1272-1331 ("the tables describe the rotation").  Needs no GPU. */
int llvq_hip_host_rotate(uint32_t n, uint64_t seed, double* v);
/* RotKey of a matrix (fused.rs:672-674): whether it is stored rotated, and the seed. */
int llvq_hip_matrix_rotation(const llvq_mat* m, uint32_t* has_rotation, uint64_t* seed);

/* group_forward (llvq-llm/src/model.rs:497-536) for projections that share an
 * activation (q/k/v, gate/up): one launch over the concatenated rows of
 * consecutive matrices that share a basis; the activation is rotated once per basis. */
int llvq_hip_gemv_group(llvq_rt* rt, const llvq_mat* const* mats, int n, const void* x_f16_dev,
                        void* const* y_dev, int y_dtype);

/* A token's worth of group products as ONE launch.  The reference's FusedOp::cuda_fwd
 * (llvq-llm/src/fused_cuda.rs:758-900) launches per projection, and group_forward
 * (model.rs:497-536) calls it once per activation site, so a decode token is hundreds of
 * launches whose latency the reference puts at about half the token (fused_cuda.rs:789-795).
 * A sequence binds a list of items — each item is what one llvq_hip_gemv_group call would
 * be: projections that share d_in, one activation, their outputs — once, and
 * llvq_hip_sequence_run enqueues them all as one persistent kernel on the runtime's stream.
 * Results are those of the separate calls, bit for bit.
 *   after_previous = 0: the item's activation is complete before the run is enqueued.
 *   after_previous = 1: the activation is (or depends on) an output of the item before it in
 *     the list; the kernel orders the two on the device: a workgroup waits, a bounded time,
 *     for the workgroups that store what it is about to read.  That needs every workgroup of the
 *     launch resident at once (one per CU), which holds while nothing else occupies the device's
 *     CUs for long; otherwise the run gives up and llvq_hip_sequence_status reports it.
 * Matrices stored in a rotated basis, and rows wider than 24 576 columns, are refused with
 * LLVQ_ERR_UNSUPPORTED (use the per-call entry points).  The pointers are captured at
 * creation; the matrices and buffers must outlive the sequence.  Runs of one sequence must
 * not overlap (they share its device-side counters). */
typedef struct llvq_seq llvq_seq;
typedef struct llvq_seq_item {
  const llvq_mat* const* mats;
  int n_mats;
  const void* x_f16_dev;
  void* const* y_dev;
  int y_dtype;
  int after_previous;
} llvq_seq_item;
int llvq_hip_sequence_create(llvq_rt* rt, const llvq_seq_item* items, int n_items, llvq_seq** out);
int llvq_hip_sequence_run(llvq_rt* rt, llvq_seq* seq);
/* Waits for the stream, then LLVQ_OK, or LLVQ_ERR_DEVICE if a workgroup of an earlier run gave
 * up waiting for an item (its outputs are then incomplete). */
int llvq_hip_sequence_status(llvq_rt* rt, llvq_seq* seq);
void llvq_hip_sequence_destroy(llvq_rt* rt, llvq_seq* seq);
/* How long an ordered item waits for the one before it: `spin_limit` polls (0: the default, about
 * a second).  hold_item >= 0 makes the NEXT run treat that item as never complete, so that the
 * items behind it give up after spin_limit polls and llvq_hip_sequence_status reports it: how
 * the give-up path is tested without a kernel that hangs.  No counterpart in the reference. */
int llvq_hip_sequence_tune(llvq_seq* seq, uint32_t spin_limit, int hold_item);

/* The row loop of group_forward (model.rs:521-529) as one batched product:
 * Y[M, d_out] = X[M, d_in] W^T, X row-major binary16. */
int llvq_hip_gemm(llvq_rt* rt, const llvq_mat* m, const void* x_f16_dev, int M, void* y_dev,
                  int y_dtype);

/* The same for the projections of one group (model.rs:497-536: q/k/v, gate/up share their
 * activation rows): y_dev[i] = X W_i^T, [M, d_out_i] each.  Consecutive matrices that share a
 * basis go through one launch (up to four at a time), so the activations are prepared once
 * and small matrices fill the chip together with their neighbours. */
int llvq_hip_gemm_group(llvq_rt* rt, const llvq_mat* const* mats, int n, const void* x_f16_dev, int M,
                        void* const* y_dev, int y_dtype);

/* llvq_hip_gemm / llvq_hip_gemm_group keep their partial sums, a tiled copy of the activations and
 * (rotated matrices) the rotated rows in buffers of the runtime, which they grow on first use of a
 * larger shape — a hipFree + hipMalloc, i.e. a device-wide wait inside a call that otherwise only
 * enqueues.  This sizes those buffers ahead of time for calls over `mats` (one group, as
 * llvq_hip_gemm_group takes it) with up to max_rows rows; later calls within that bound allocate
 * nothing and return without synchronising.  llvq_hip_decoder_create does the same for its
 * projections when prefill_rows > 0.  No counterpart in the reference, whose l > 1 path is a row
 * loop of matrix-vector launches (model.rs:521-529). */
int llvq_hip_reserve_batched(llvq_rt* rt, const llvq_mat* const* mats, int n, int max_rows);

/* llvq_hip_gemm for callers that cannot allocate device memory (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc).  It has no counterpart
 * in the reference.  Same kernels and results as llvq_hip_gemm; the partial sums, the tiled
 * copy of the activations and (rotated matrices) the rotated rows live in one static device
 * array of LLVQ_STATIC_SCRATCH_BYTES per GPU instead of buffers the runtime grows, and the
 * call makes no hipMalloc / hipFree.  A shape whose workspaces do not fit is refused with
 * LLVQ_ERR_UNSUPPORTED (the message names the bytes needed).  Every call on a GPU shares that
 * GPU's array: calls that overlap on one GPU (two streams, two runtimes) race. */
#define LLVQ_STATIC_SCRATCH_BYTES (64u << 20)
int llvq_hip_gemm_static(llvq_rt* rt, const llvq_mat* m, const void* x_f16_dev, int M, void* y_dev,
                         int y_dtype);

/* Parity probe (the role of decode_probe, llvq-cuda/kernels/preflight.cu:39):
 * unrank packed 6-byte records on the device.  points: 24 int8 per block;
 * gains: one byte per block; shells (may be NULL): one byte per block.
 * codes_dev holds exactly 6 * nblocks bytes and needs no slack behind them: no byte past
 * the last record is read (that record is fetched byte by byte).  codes_dev starts on a
 * 4-byte boundary (records are read as dwords); LLVQ_ERR_INVALID_ARGUMENT otherwise. */
int llvq_hip_decode_blocks(llvq_rt* rt, const uint8_t* codes_dev, size_t nblocks,
                           int8_t* points_dev, uint8_t* gains_dev, uint8_t* shells_dev);
/* The same for the code stream of a matrix of any accepted shell cap (pack.rs:48-82): cap 12 is
 * llvq_hip_decode_blocks; at cap 13 block b is the 49 bits from bit 49 b on, codes_dev holds
 * ceil(49 * nblocks / 8) bytes, no byte past them is read and no alignment is asked.  An index
 * past N(13) decodes to zeros with shell 0xFF. */
int llvq_hip_decode_stream(llvq_rt* rt, const uint8_t* codes_dev, size_t nblocks, uint32_t shell_cap,
                           int8_t* points_dev, uint8_t* gains_dev, uint8_t* shells_dev);

/* ---- batch-1 decode loop ---------------------------------------------------
 * Replaces Qwen3 / Block at l = 1 (llvq-llm/src/model.rs:589-623, :839-862):
 * a Qwen3-architecture decoder whose projections are uploaded LLVQ matrices and
 * whose other tensors are dense binary16.  Host pointers; everything is copied. */
typedef struct llvq_decoder llvq_decoder;
/* KvMode (llvq-llm/src/kvq.rs:10-34): binary16 cache, or 8-bit codes per group of
 * 64 along head_dim with binary16 scale and bias (kvq.rs:110-165), chosen from
 * the token alone and rebuilt to the same binary16 value on every read. */
typedef enum llvq_kv_mode { LLVQ_KV_F16 = 0, LLVQ_KV_Q8 = 1 } llvq_kv_mode;
/* An int8 tensor of the sealed sections (QuantData, sealed.rs:64-78; the q8
 * embedding of fused_cuda.rs:408-470): one code per weight, binary16 scale and
 * bias per group along the row, weight = scale * code + bias.  Host pointers. */
typedef struct llvq_quant_rows {
  const uint8_t* codes;     /* [rows, row_len]; NULL = absent */
  const uint16_t* scales;   /* [rows, ceil(row_len / group)] */
  const uint16_t* biases;
  uint32_t bits, group;     /* the kernels take 8 and 64 */
} llvq_quant_rows;
/* How llvq_hip_decoder_* launches the projection groups of a decoded position.  The results are the same bit for bit;
 * the speed is not: a decode position is a chain of dependent products, and an ordered item of a sequence pays about
 * what a launch boundary costs (measured on the Qwen3-4B shape: 251 / 235 / 227 tokens/s in the order below).
 * Models a sequence cannot take (matrices in a rotated basis or of mixed shell caps, hidden > 6144) use LLVQ_LAUNCH_PER_GROUP
 * whatever is asked. */
typedef enum llvq_launch_mode {
  LLVQ_LAUNCH_PER_GROUP = 0,  /* one llvq_hip_gemv_group launch per group */
  LLVQ_LAUNCH_SINGLE = 1,     /* one single-item sequence (llvq_hip_sequence_*) per group: the sequence kernel's tile loop */
  LLVQ_LAUNCH_CHAINED = 2     /* o_proj, gate/up, down_proj and the next layer's q/k/v as one sequence of ordered items
                                 between two attention launches */
} llvq_launch_mode;

typedef struct llvq_decoder_desc {
  uint32_t n_layers, hidden, n_heads, n_kv_heads, head_dim, intermediate, vocab;
  uint32_t max_positions;               /* KV-cache length, <= 8192 */
  double rope_theta, rms_eps;
  const llvq_mat* const* projections;   /* [n_layers * 7]: q, k, v, o, gate, up, down per layer */
  const uint16_t* input_norm;           /* [n_layers, hidden]   binary16 bit patterns */
  const uint16_t* post_norm;            /* [n_layers, hidden] */
  const uint16_t* q_norm;               /* [n_layers, head_dim] */
  const uint16_t* k_norm;               /* [n_layers, head_dim] */
  const uint16_t* final_norm;           /* [hidden] */
  const uint16_t* embed;                /* [vocab, hidden]; NULL when embed_q8 is given */
  const uint16_t* lm_head;              /* [vocab, hidden]; NULL = tied to embed */
  uint32_t kv_mode;                     /* llvq_kv_mode; q8 needs head_dim % 64 == 0 */
  llvq_quant_rows embed_q8;             /* int8 embedding instead of `embed` (Embed::Q8, model.rs:546-551) */
  llvq_quant_rows lm_head_q8;           /* int8 head (Head::Q8, model.rs:569-575); absent and lm_head NULL = tied */
  uint32_t prefill_rows;                /* positions llvq_hip_decoder_prefill takes per pass (buffers for that many
                                           rows are allocated); 0 = the batched prompt path is not used */
  uint32_t launch_mode;                 /* llvq_launch_mode: how a decoded position's projection groups are launched */
} llvq_decoder_desc;
/* Qwen3::new_with (model.rs:869): checks every projection's shape against the architecture. */
int llvq_hip_decoder_create(llvq_rt* rt, const llvq_decoder_desc* desc, llvq_decoder** out);
void llvq_hip_decoder_destroy(llvq_decoder* dec);
/* fresh_caches (model.rs:963): the next token is position 0 again. */
int llvq_hip_decoder_reset(llvq_decoder* dec);
int llvq_hip_decoder_position(const llvq_decoder* dec);
/* Measurement aid with no counterpart in the reference: makes `position` the next
 * position without feeding the tokens before it, so the attention cost of a long
 * context can be timed without a long prefill.  Cache entries that were never
 * written hold zeros (a valid key/value), so the results are well defined but
 * are not those of any real prompt. */
int llvq_hip_decoder_seek(llvq_decoder* dec, uint32_t position);
/* hidden_cached at l = 1 followed by Head::project (model.rs:968-982, :578-587):
 * feeds one token at the current position, advances it, and returns the
 * logits (vocab f32 values, each already rounded to binary16 as the reference's
 * f16 matmul leaves them) and their argmax (lowest index on ties).  Either
 * output may be NULL.  Synchronises. */
int llvq_hip_decoder_forward_token(llvq_decoder* dec, uint32_t token, float* logits_host, uint32_t* argmax_host);
/* Qwen3::generate (model.rs:1041-1073): resets, feeds the prompt, then decodes
 * greedily; out receives max_new tokens.  max_new = 0 returns at once.
 * The loop never waits on the host between tokens.  Synchronises at the end. */
int llvq_hip_decoder_generate(llvq_decoder* dec, const uint32_t* prompt, size_t n_prompt, size_t max_new,
                              uint32_t* out);

/* The l > 1 arm of hidden_cached (model.rs:968-982, row loop of :521-529) with the rows of a
 * pass going through the batched product (llvq_hip_gemm) instead of one product per row:
 * feeds n tokens at the positions that follow the current one, prefill_rows at a time,
 * advances the position by n and returns the last token's logits and argmax as
 * llvq_hip_decoder_forward_token does (either may be NULL).  The weights of these products
 * are rounded to binary16 once (see llvq_hip_gemm), so logits differ from the
 * token-by-token path by a few 1e-3 of the largest one; the KV cache it leaves is read by
 * the token-by-token calls that follow.  head_dim <= 128.  Synchronises. */
int llvq_hip_decoder_prefill(llvq_decoder* dec, const uint32_t* tokens, size_t n, float* logits_host,
                             uint32_t* argmax_host);
/* llvq_hip_decoder_generate with the prompt taken through llvq_hip_decoder_prefill. */
int llvq_hip_decoder_generate_prefilled(llvq_decoder* dec, const uint32_t* prompt, size_t n_prompt, size_t max_new,
                                        uint32_t* out);

/* Qwen3::generate_phased (model.rs:1116-1163, behind LLVQ_TIME_PHASES=1 in bin/fusedrun): the tokens
 * of llvq_hip_decoder_generate, with every decode step's phases timed — phase_ms[4 * t + k] for
 * token t, k = 0 final norm + head, 1 argmax, 2 embedding of that token, 3 the layers over it (2 and
 * 3 are zero for the last token, which is not fed back).  The prompt is not phased.  Where the
 * reference fences the device after each phase, this records events on the stream: the phases are
 * device time and the run is not serialised by them.  A diagnostic, not the published rate. */
int llvq_hip_decoder_generate_phased(llvq_decoder* dec, const uint32_t* prompt, size_t n_prompt, size_t max_new,
                                     uint32_t* out, double* phase_ms);

int llvq_hip_synchronize(llvq_rt* rt);
const char* llvq_hip_last_error(void);
const char* llvq_hip_version(void);

#ifdef __cplusplus
}
#endif
#endif
