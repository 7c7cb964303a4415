#include "rotation.hpp"

#include <cmath>

namespace llvq {

namespace {

// llvq-core/src/rng.rs:21-40
struct SplitMix64 {
  uint64_t s;
  uint64_t next() {
    s += 0x9E3779B97F4A7C15ULL;
    uint64_t z = s;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ULL;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBULL;
    return z ^ (z >> 31);
  }
  double gaussian() {  // Box-Muller, cosine branch; u1 in (0, 1]
    const double u1 = ((double)(next() >> 11) + 1.0) * (1.0 / 9007199254740993.0);
    const double u2 = (double)(next() >> 11) * (1.0 / 9007199254740992.0);
    return std::sqrt(-2.0 * std::log(u1)) * std::cos(6.283185307179586476925286766559 * u2);
  }
};

}  // namespace

bool build_rotation(uint32_t n, uint64_t seed, RotationTables* out, std::string* err) {
  if (n == 0) {
    if (err) *err = "rotation of width 0";
    return false;
  }
  RotationTables t;
  t.n = n;
  t.m = n & (~n + 1u);  // lowest set bit = 2^trailing_zeros
  t.k = n / t.m;
  if (t.k > kRotKMax) {
    if (err)
      *err = "width " + std::to_string(n) + ": odd factor " + std::to_string(t.k) + " exceeds " +
             std::to_string(kRotKMax) + ", which the rotation kernel does not take";
    return false;
  }
  SplitMix64 rng{seed};
  t.signbits.assign((n + 31) / 32, 0u);
  for (uint32_t i = 0; i < n; ++i)
    if (rng.gaussian() < 0.0) t.signbits[i >> 5] |= 1u << (i & 31);
  // k Gaussian rows, each made orthogonal to the rows before it, then normalised
  std::vector<double> q((size_t)t.k * t.k, 0.0), row(t.k);
  for (uint32_t i = 0; i < t.k; ++i) {
    for (uint32_t c = 0; c < t.k; ++c) row[c] = rng.gaussian();
    for (uint32_t p = 0; p < i; ++p) {
      double d = 0.0;
      for (uint32_t c = 0; c < t.k; ++c) d += row[c] * q[(size_t)p * t.k + c];
      for (uint32_t c = 0; c < t.k; ++c) row[c] -= d * q[(size_t)p * t.k + c];
    }
    double nrm = 0.0;
    for (uint32_t c = 0; c < t.k; ++c) nrm += row[c] * row[c];
    nrm = std::sqrt(nrm);
    if (!(nrm > 1e-9)) {
      if (err) *err = "degenerate Gram-Schmidt for seed " + std::to_string(seed);
      return false;
    }
    for (uint32_t c = 0; c < t.k; ++c) q[(size_t)i * t.k + c] = row[c] / nrm;
  }
  t.small.resize(q.size());
  for (size_t i = 0; i < q.size(); ++i) t.small[i] = (float)q[i];
  t.inv = (float)(1.0 / std::sqrt((double)t.m));
  *out = std::move(t);
  return true;
}

void host_rotate(const RotationTables& t, std::vector<double>* vp) {
  std::vector<double>& v = *vp;
  for (uint32_t i = 0; i < t.n; ++i)
    if ((t.signbits[i >> 5] >> (i & 31)) & 1u) v[i] = -v[i];
  for (uint32_t g = 0; g < t.k; ++g) {
    double* s = v.data() + (size_t)g * t.m;
    for (uint32_t len = 1; len < t.m; len <<= 1)
      for (uint32_t i = 0; i < t.m; i += len << 1)
        for (uint32_t j = i; j < i + len; ++j) {
          const double a = s[j], b = s[j + len];
          s[j] = a + b;
          s[j + len] = a - b;
        }
  }
  const double inv = (double)t.inv;
  if (t.k == 1) {
    for (auto& x : v) x *= inv;
    return;
  }
  std::vector<double> col(t.k);
  for (uint32_t j = 0; j < t.m; ++j) {
    for (uint32_t c = 0; c < t.k; ++c) col[c] = v[(size_t)c * t.m + j] * inv;
    for (uint32_t g = 0; g < t.k; ++g) {
      double acc = 0.0;
      for (uint32_t c = 0; c < t.k; ++c) acc += (double)t.small[(size_t)g * t.k + c] * col[c];
      v[(size_t)g * t.m + j] = acc;
    }
  }
}

}  // namespace llvq
