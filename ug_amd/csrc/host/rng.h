// Counter-based generator for synthetic inputs and weights: splitmix64 stream -> U[0,1) ->
// Box-Muller.  ug_amd/rng.py implements the same functions with numpy.
#pragma once
#include <cmath>
#include <cstdint>
#include <string>

namespace ugrng {

inline uint64_t mix(uint64_t z) {
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}

// i-th output (0-based) of splitmix64 started from `seed`.
inline uint64_t u64_at(uint64_t seed, uint64_t i) { return mix(seed + (i + 1) * 0x9E3779B97F4A7C15ull); }

// U[0,1) with 53 random bits.
inline double u01_at(uint64_t seed, uint64_t i) { return (double)(u64_at(seed, i) >> 11) * (1.0 / 9007199254740992.0); }

// U(-1,1) as f32.
inline float uniform_pm1_at(uint64_t seed, uint64_t i) { return (float)(2.0 * u01_at(seed, i) - 1.0); }

// Pair p of standard normals: outputs 2p and 2p+1 of the stream feed one Box-Muller transform.
inline void normal_pair(uint64_t seed, uint64_t p, double* z0, double* z1) {
  double u1 = u01_at(seed, 2 * p), u2 = u01_at(seed, 2 * p + 1);
  double r = std::sqrt(-2.0 * std::log(1.0 - u1));
  double a = 6.283185307179586476925286766559 * u2;
  *z0 = r * std::cos(a);
  *z1 = r * std::sin(a);
}

// Per-tensor stream: FNV-1a of the name folded into the seed.
inline uint64_t tensor_seed(uint64_t seed, const std::string& name) {
  uint64_t h = 0xcbf29ce484222325ull;
  for (unsigned char c : name) {
    h ^= c;
    h *= 0x100000001b3ull;
  }
  return mix(seed ^ h);
}

}  // namespace ugrng
