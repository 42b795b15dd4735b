// XXH64 (the public algorithm, scalar form) and the chained page hash built on it:
// hash of page i = xxh64(token bytes of page i, seed = hash of page i-1), root seed 0.
// The reference hashes pages the same way (src/core/hash.h:29-73).
#pragma once
#include <cstddef>
#include <cstdint>
#include <cstring>

namespace kvcm {

class XXH64 {
 public:
  static uint64_t digest(const void* data, size_t len, uint64_t seed) {
    const unsigned char* p = static_cast<const unsigned char*>(data);
    const unsigned char* const stop = p + len;
    uint64_t acc;
    if (len >= 32) {
      uint64_t lane[4] = {seed + kA + kB, seed + kB, seed, seed - kA};
      for (; stop - p >= 32; p += 32)
        for (int i = 0; i < 4; ++i) lane[i] = step(lane[i], word64(p + 8 * i));
      acc = rot(lane[0], 1) + rot(lane[1], 7) + rot(lane[2], 12) + rot(lane[3], 18);
      for (int i = 0; i < 4; ++i) acc = (acc ^ step(0, lane[i])) * kA + kD;
    } else {
      acc = seed + kE;
    }
    acc += static_cast<uint64_t>(len);
    for (; stop - p >= 8; p += 8) acc = rot(acc ^ step(0, word64(p)), 27) * kA + kD;
    if (stop - p >= 4) {
      acc = rot(acc ^ (static_cast<uint64_t>(word32(p)) * kA), 23) * kB + kC;
      p += 4;
    }
    for (; p < stop; ++p) acc = rot(acc ^ (static_cast<uint64_t>(*p) * kE), 11) * kA;
    acc = (acc ^ (acc >> 33)) * kB;
    acc = (acc ^ (acc >> 29)) * kC;
    return acc ^ (acc >> 32);
  }

 private:
  static constexpr uint64_t kA = 0x9E3779B185EBCA87ULL;
  static constexpr uint64_t kB = 0xC2B2AE3D27D4EB4FULL;
  static constexpr uint64_t kC = 0x165667B19E3779F9ULL;
  static constexpr uint64_t kD = 0x85EBCA77C2B2AE63ULL;
  static constexpr uint64_t kE = 0x27D4EB2F165667C5ULL;
  static uint64_t rot(uint64_t v, int s) { return (v << s) | (v >> (64 - s)); }
  static uint64_t step(uint64_t acc, uint64_t in) { return rot(acc + in * kB, 31) * kA; }
  static uint64_t word64(const unsigned char* p) { uint64_t v; std::memcpy(&v, p, 8); return v; }
  static uint32_t word32(const unsigned char* p) { uint32_t v; std::memcpy(&v, p, 4); return v; }
};

inline uint64_t chain_hash(uint64_t parent, const int32_t* tokens, int n) {
  return XXH64::digest(tokens, sizeof(int32_t) * static_cast<size_t>(n), parent);
}

}  // namespace kvcm
