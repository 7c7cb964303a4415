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

}  // namespace llvq
