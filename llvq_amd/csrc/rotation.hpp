// Host-side construction of the incoherence rotation's device tables
// (llvq-quant/src/rotation.rs:60-79 for the draw order and the Gram-Schmidt
// block; llvq-llm/src/fused.rs:672-721 for what a kernel is handed).
// Q = (S (x) I_m) (I_k (x) H_m / sqrt m) D with n = m k, m the power-of-two
// part of n.  An artifact stores W' = W Q^T, so the activation owes x' = Q x.
#pragma once
#include <cstddef>
#include <cstdint>
#include <string>
#include <vector>

namespace llvq {

constexpr uint32_t kRotKMax = 32;  // widest odd factor the kernels take (fused.rs:501)

struct RotationTables {
  uint32_t n = 0, m = 0, k = 0;
  std::vector<uint32_t> signbits;  // bit i set: coordinate i is negated
  std::vector<float> small;        // k x k, row-major (not padded)
  float inv = 1.f;                 // 1 / sqrt(m), narrowed once on the host
};

// Returns false (and says why) when the odd factor of n exceeds kRotKMax.
bool build_rotation(uint32_t n, uint64_t seed, RotationTables* out, std::string* err);

// Reference arithmetic of the rotation in f64 on the host (used by tests of the tables).
void host_rotate(const RotationTables& t, std::vector<double>* v);

}  // namespace llvq
