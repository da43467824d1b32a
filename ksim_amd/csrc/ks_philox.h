// Philox-4x32-10 counter-based generator (Salmon et al., SC'11): four 32-bit words per call,
// keyed by (seed) and counted by (env, step, purpose, block) so that any draw can be
// regenerated independently of launch geometry.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace ks {

struct Philox4 {
  uint32_t x, y, z, w;
};

__host__ __device__ inline Philox4 philox4x32_10(uint32_t c0, uint32_t c1, uint32_t c2, uint32_t c3, uint32_t k0,
                                                 uint32_t k1) {
  const uint32_t M0 = 0xD2511F53u, M1 = 0xCD9E8D57u, W0 = 0x9E3779B9u, W1 = 0xBB67AE85u;
  for (int r = 0; r < 10; ++r) {
    const uint64_t p0 = (uint64_t)M0 * c0, p1 = (uint64_t)M1 * c2;
    const uint32_t hi0 = (uint32_t)(p0 >> 32), lo0 = (uint32_t)p0, hi1 = (uint32_t)(p1 >> 32), lo1 = (uint32_t)p1;
    const uint32_t n0 = hi1 ^ c1 ^ k0, n2 = hi0 ^ c3 ^ k1;
    c0 = n0; c1 = lo1; c2 = n2; c3 = lo0;
    k0 += W0; k1 += W1;
  }
  return {c0, c1, c2, c3};
}

// U[0, 1) with 24 random bits
__host__ __device__ inline float u01(uint32_t x) { return (float)(x >> 8) * (1.0f / 16777216.0f); }

// one standard normal from two words (Box-Muller)
__device__ inline float normal_from(uint32_t a, uint32_t b) {
  const float u1 = ((float)(a >> 8) + 1.0f) * (1.0f / 16777216.0f);  // (0, 1]
  const float u2 = u01(b);
  return sqrtf(-2.0f * logf(u1)) * cosf(6.28318530717958647692f * u2);
}

enum { kRngObsNoise = 1, kRngReset = 2, kRngAction = 3, kRngEvent = 4, kRngObsCarry = 5, kRngCommand = 6, kRngObsBias = 7, kRngEpisode = 8 };

// draw for (env, element) of a purpose at a step: counter = (env lo, env hi ^ purpose<<24, step lo, element)
__device__ inline Philox4 draw(uint64_t seed, uint64_t step, int purpose, uint64_t env, uint32_t element) {
  return philox4x32_10((uint32_t)env, (uint32_t)(env >> 32) ^ ((uint32_t)purpose << 24), (uint32_t)step, element,
                       (uint32_t)seed, (uint32_t)(seed >> 32) ^ (uint32_t)(step >> 32));
}

}  // namespace ks
