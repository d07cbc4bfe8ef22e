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

RPU_HD Philox4 philox4x32_10(uint32_t c0, uint32_t c1, uint32_t c2, uint32_t c3, uint32_t k0,
                             uint32_t k1) {
  const uint32_t M0 = 0xD2511F53u, M1 = 0xCD9E8D57u, W0 = 0x9E3779B9u, W1 = 0xBB67AE85u;
#pragma unroll
  for (int r = 0; r < 10; ++r) {
    // one 32 x 32 -> 64 bit product per multiplier (v_mad_u64_u32 on gfx950)
    const uint64_t p0 = (uint64_t)M0 * (uint64_t)c0;
    const uint64_t p1 = (uint64_t)M1 * (uint64_t)c2;
    const uint32_t hi0 = (uint32_t)(p0 >> 32), lo0 = (uint32_t)p0;
    const uint32_t hi1 = (uint32_t)(p1 >> 32), lo1 = (uint32_t)p1;
#if defined(__HIP_DEVICE_COMPILE__)
    // three-input xor in one instruction (v_bitop3_b32, truth table 0x96)
    const uint32_t n0 = __builtin_amdgcn_bitop3_b32(hi1, c1, k0, 0x96);
    const uint32_t n2 = __builtin_amdgcn_bitop3_b32(hi0, c3, k1, 0x96);
#else
    const uint32_t n0 = hi1 ^ c1 ^ k0;
    const uint32_t n2 = hi0 ^ c3 ^ k1;
#endif
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
  RNG_UPDATE_SR = 8,  // stochastic rounding of pulse probabilities
  RNG_PCM_PROGRAM = 9, // programming noise and drift coefficients of the inference weight pipeline
  RNG_PCM_DRIFT = 10,  // accumulated read noise at inference time
  RNG_DIFFUSE = 11,    // weight diffusion
  RNG_RESET = 12,      // column reset (noise, and with round 1 the reset lottery)
  RNG_DEVICE_DRIFT = 13, // power-law drift of a training tile: nu variation and read noise
  RNG_MODIFIER = 14,     // weight modifier: noise, stochastic rounding, drop connections
  RNG_W_NOISE = 15,      // output-referred weight noise of the analog MVM
  RNG_WRITE_NOISE = 16,  // write noise on the shown weights (round 0: after an update, 1: refresh of all)
  RNG_TRANSFER = 17      // transfer compound, drawn on the host: word 0 random selection of the slice, word 1 reset lottery
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

// Box-Muller on one 32-bit word: radius from the high 16 bits (mid-point rule, so the discrete
// radius distribution keeps E[r^2] = 2 to O(2^-32)), angle from the low 16 bits.  Two N(0,1) whose
// resolution (2^-16 of the radius range, 2^16 angles) is finer than the fp32 rounding of a weight update
// that adds step * (1 + std * n) to a weight; |n| <= 4.9.
__device__ __forceinline__ void box_muller16(uint32_t r, float &n0, float &n1) {
  const float u = ((float)(r >> 16) + 0.5f) * (1.0f / 65536.0f);
  const float t = (float)(r & 0xffffu) * (1.0f / 65536.0f); // turns
  // -2 ln(u) = -2 ln(2) log2(u)
  const float rad = __builtin_amdgcn_sqrtf(-1.3862943611198906f * __builtin_amdgcn_logf(u));
  n0 = rad * __builtin_amdgcn_cosf(t);
  n1 = rad * __builtin_amdgcn_sinf(t);
}

// eight N(0,1) from one Philox call
__device__ __forceinline__ void philox_normal8(uint32_t c0, uint32_t c1, uint32_t c2, uint32_t c3,
                                               PhiloxKey key, float out[8]) {
  const Philox4 r = philox4x32_10(c0, c1, c2, c3, key.k0, key.k1);
  box_muller16(r.v[0], out[0], out[1]);
  box_muller16(r.v[1], out[2], out[3]);
  box_muller16(r.v[2], out[4], out[5]);
  box_muller16(r.v[3], out[6], out[7]);
}

// eight factors 1 + std * N(0,1) from one Philox call: box_muller16 with std folded into the radius
// (std * sqrt(-2 ln u) = sqrt(-2 ln2 std^2 log2 u)) and the final multiply-add fused
__device__ __forceinline__ void philox_factor8(uint32_t c0, uint32_t c1, uint32_t c2, uint32_t c3,
                                               PhiloxKey key, float std_, float out[8]) {
  const Philox4 r = philox4x32_10(c0, c1, c2, c3, key.k0, key.k1);
  const float m = -1.3862943611198906f * std_ * std_;
#pragma unroll
  for (int p = 0; p < 4; ++p) {
    const float u = __builtin_fmaf((float)(r.v[p] >> 16), 1.0f / 65536.0f, 0.5f / 65536.0f);
    const float t = (float)(r.v[p] & 0xffffu) * (1.0f / 65536.0f); // turns
    const float rad = __builtin_amdgcn_sqrtf(m * __builtin_amdgcn_logf(u));
    out[2 * p] = __builtin_fmaf(rad, __builtin_amdgcn_cosf(t), 1.0f);
    out[2 * p + 1] = __builtin_fmaf(rad, __builtin_amdgcn_sinf(t), 1.0f);
  }
}

__device__ __forceinline__ void philox_normal4(uint32_t c0, uint32_t c1, uint32_t c2, uint32_t c3,
                                               PhiloxKey key, float out[4]) {
  const Philox4 r = philox4x32_10(c0, c1, c2, c3, key.k0, key.k1);
  box_muller(r.v[0], r.v[1], out[0], out[1]);
  box_muller(r.v[2], r.v[3], out[2], out[3]);
}
#endif

} // namespace rpu_amd
