// Host-side reader of the on-disk .llvq header and matrix record
// (llvq-artifact/src/format.rs:301-382, :588-619).  The code stream is not
// unpacked: the record is parsed into views over the caller's buffer.
#pragma once
#include <cstddef>
#include <cstdint>
#include <string>
#include <vector>

namespace llvq {

struct RecordView {
  std::string name;
  uint32_t d_out = 0, d_in = 0, shell_cap = 0, n_centroids = 0;
  uint64_t rotation_seed = 0;
  bool has_rotation = false;
  std::vector<double> centroids;
  std::vector<double> row_scales;
  std::vector<float> tail;      // d_out * (d_in % 24), as stored (f32)
  const uint8_t* codes = nullptr;
  size_t code_bytes = 0;
  size_t centroids_off = 0, row_scales_off = 0, tail_off = 0, codes_off = 0;  // relative to the buffer
};

// Status codes are the llvq_status values of include/llvq_hip.h.
int parse_header(const uint8_t* buf, size_t len, size_t* pos, uint32_t* version,
                 uint32_t* n_matrices, std::string* err);
int parse_matrix_record(const uint8_t* buf, size_t len, size_t* pos, RecordView* out,
                        std::string* err);

// A raw tensor record (llvq-artifact/src/sealed.rs:80-92, :277-326) as byte
// ranges of the caller's buffer; nothing is copied.
struct RawTensorView {
  std::string name;
  std::vector<uint64_t> dims;
  uint32_t tag = 0;        // 0: binary16 values; 1: int4 / int8 codes with binary16 scale and bias per group
  uint32_t bits = 0, group = 0;
  size_t data_off = 0, data_len = 0;      // f16: values (2 bytes each); quant: packed codes
  size_t scales_off = 0, biases_off = 0;  // quant only
  uint64_t count = 0;                     // f16: values; quant: groups
};
struct BlobView {
  std::string name;
  size_t data_off = 0, data_len = 0;
};
// version < 3 records carry no tag and are binary16 (sealed.rs:278-282).
int parse_raw_tensor(const uint8_t* buf, size_t len, size_t* pos, uint32_t version, RawTensorView* out,
                     std::string* err);
int parse_blob(const uint8_t* buf, size_t len, size_t* pos, BlobView* out, std::string* err);

}  // namespace llvq
