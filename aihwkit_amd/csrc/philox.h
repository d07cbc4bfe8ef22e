// Counter-based Philox4x32-10 generator (Salmon, Moraes, Dror, Shaw: "Parallel random numbers: as easy
// as 1, 2, 3", SC'11) usable from host and device code.  Every random draw of the library is a pure
// function of (tile seed, call index, purpose, element index), so results do not depend on grid
// shape, tiling or launch order.  It takes the place of the per-thread cuRAND XORWOW states of the
// reference (src/rpucuda/cuda/cuda_util.cu:163-176).
#pragma once
#include <stdint.h>

#if defined(__HIPCC__)
#include <hip/hip_runtime.h>
#define RPU_HD __host__ __device__ __forceinline__
#else
#define RPU_HD inline
#endif

namespace rpu_amd {

struct PhiloxKey {
  uint32_t k0, k1;
};

struct Philox4 {
  uint32_t v[4];
};

RPU_HD uint32_t philox_mulhi(uint32_t a, uint32_t b) {
#if defined(__HIP_DEVICE_COMPILE__)
  return __umulhi(a, b);
#else
  return (uint32_t)(((uint64_t)a * (uint64_t)b) >> 32);
#endif
}

RPU_HD Philox4 philox4x32_10(uint32_t c0, uint32_t c1, uint32_t c2, uint32_t c3, uint32_t k0,
                             uint32_t k1) {
  const uint32_t M0 = 0xD2511F53u, M1 = 0xCD9E8D57u, W0 = 0x9E3779B9u, W1 = 0xBB67AE85u;
#pragma unroll
  for (int r = 0; r < 10; ++r) {
    const uint32_t hi0 = philox_mulhi(M0, c0), lo0 = M0 * c0;
    const uint32_t hi1 = philox_mulhi(M1, c2), lo1 = M1 * c2;
    const uint32_t n0 = hi1 ^ c1 ^ k0;
    const uint32_t n2 = hi0 ^ c3 ^ k1;
    c0 = n0;
    c1 = lo1;
    c2 = n2;
    c3 = lo0;
    k0 += W0;
    k1 += W1;
  }
  Philox4 out;
  out.v[0] = c0;
  out.v[1] = c1;
  out.v[2] = c2;
  out.v[3] = c3;
  return out;
}

// what a draw is used for; part of the counter so that streams never overlap
enum RngPurpose : uint32_t {
  RNG_OUT_NOISE = 1,  // ADC output noise
  RNG_INP_NOISE = 2,  // DAC input noise
  RNG_INP_SR = 3,     // DAC stochastic rounding
  RNG_OUT_SR = 4,     // ADC stochastic rounding
  RNG_PULSE_X = 5,    // x bit lines
  RNG_PULSE_D = 6,    // d bit lines
  RNG_CTOC = 7,       // cycle-to-cycle update noise
  RNG_UPDATE_SR = 8   // stochastic rounding of pulse probabilities
};

// uniform in [0, 1) with 24 bits
RPU_HD float u32_to_uniform(uint32_t r) { return (float)(r >> 8) * (1.0f / 16777216.0f); }

#if defined(__HIPCC__)
// Box-Muller on two 32-bit words: two independent N(0,1).
__device__ __forceinline__ void box_muller(uint32_t r0, uint32_t r1, float &n0, float &n1) {
  // u in (0, 1]: never log(0)
  const float u = ((float)(r0 >> 8) + 1.0f) * (1.0f / 16777216.0f);
  const float t = (float)(r1 >> 8) * (1.0f / 16777216.0f); // turns
  const float rad = __fsqrt_rn(-2.0f * __logf(u));
  float s, c;
  __sincosf(6.283185307179586f * t, &s, &c);
  n0 = rad * c;
  n1 = rad * s;
}

__device__ __forceinline__ void philox_normal4(uint32_t c0, uint32_t c1, uint32_t c2, uint32_t c3,
                                               PhiloxKey key, float out[4]) {
  const Philox4 r = philox4x32_10(c0, c1, c2, c3, key.k0, key.k1);
  box_muller(r.v[0], r.v[1], out[0], out[1]);
  box_muller(r.v[2], r.v[3], out[2], out[3]);
}
#endif

} // namespace rpu_amd
