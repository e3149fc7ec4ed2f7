// Philox4x32-10 counter-based generator (Salmon et al., "Parallel random
// numbers: as easy as 1, 2, 3", SC'11), usable from host and device code.
// The sampler keys it by (rng seed) and counts by (node id, draw index,
// stream id), so a draw never depends on which lane or launch produced it.
#pragma once
#include <stdint.h>

#if defined(__HIPCC__)
#define SHMT_HD __host__ __device__ __forceinline__
#else
#define SHMT_HD inline
#endif

namespace shmt {

struct Philox4 {
  uint32_t v[4];
};

SHMT_HD void philox_mulhilo(uint32_t a, uint32_t b, uint32_t *hi, uint32_t *lo) {
  uint64_t p = static_cast<uint64_t>(a) * b;
  *hi = static_cast<uint32_t>(p >> 32);
  *lo = static_cast<uint32_t>(p);
}

SHMT_HD Philox4 philox4x32_10(uint32_t c0, uint32_t c1, uint32_t c2, uint32_t c3, uint32_t k0,
                              uint32_t k1) {
#pragma unroll
  for (int r = 0; r < 10; ++r) {
    uint32_t hi0, lo0, hi1, lo1;
    philox_mulhilo(0xD2511F53u, c0, &hi0, &lo0);
    philox_mulhilo(0xCD9E8D57u, c2, &hi1, &lo1);
    uint32_t n0 = hi1 ^ c1 ^ k0;
    uint32_t n2 = hi0 ^ c3 ^ k1;
    c0 = n0;
    c1 = lo1;
    c2 = n2;
    c3 = lo0;
    k0 += 0x9E3779B9u;
    k1 += 0xBB67AE85u;
  }
  Philox4 out;
  out.v[0] = c0;
  out.v[1] = c1;
  out.v[2] = c2;
  out.v[3] = c3;
  return out;
}

// High 64 bits of a 64x64-bit product.
SHMT_HD uint64_t mulhi64(uint64_t a, uint64_t b) {
#if defined(__HIP_DEVICE_COMPILE__)
  return __umul64hi(a, b);
#else
  return static_cast<uint64_t>((static_cast<unsigned __int128>(a) * b) >> 64);
#endif
}

// Uniform integer in [0, range) for the `draw`-th draw of node `node`:
// 64 random bits scaled by multiply-high (bias <= range / 2^64).
SHMT_HD uint64_t sample_draw(uint64_t rng_seed, uint32_t rng_stream, int64_t node, uint32_t draw,
                             uint64_t range) {
  const uint64_t n = static_cast<uint64_t>(node);
  Philox4 r = philox4x32_10(static_cast<uint32_t>(n), static_cast<uint32_t>(n >> 32), draw,
                            rng_stream, static_cast<uint32_t>(rng_seed),
                            static_cast<uint32_t>(rng_seed >> 32));
  const uint64_t bits = (static_cast<uint64_t>(r.v[1]) << 32) | r.v[0];
  return mulhi64(bits, range);
}

// The same draw for a range that fits 32 bits: floor(bits * range / 2^64) from
// two 32-bit products instead of a 64 x 64-bit one (identical value).
SHMT_HD uint32_t sample_draw32(uint64_t rng_seed, uint32_t rng_stream, int64_t node, uint32_t draw,
                               uint32_t range) {
  const uint64_t n = static_cast<uint64_t>(node);
  Philox4 r = philox4x32_10(static_cast<uint32_t>(n), static_cast<uint32_t>(n >> 32), draw,
                            rng_stream, static_cast<uint32_t>(rng_seed),
                            static_cast<uint32_t>(rng_seed >> 32));
  const uint64_t low = (static_cast<uint64_t>(r.v[0]) * range) >> 32;
  return static_cast<uint32_t>((static_cast<uint64_t>(r.v[1]) * range + low) >> 32);
}

}  // namespace shmt
