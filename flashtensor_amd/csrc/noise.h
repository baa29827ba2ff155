// Counter-based noise stream of the seeded KeyFormer mode (host and device).
//
// The reference feeds KeyFormer a materialised tensor exp_rand[B,H,Sq,Skv] (cases/kernels/kf.py:19,36-37);
// its MLIR snapshot names an in-graph source instead (bench/keyformer.mlir:4,17, asuka.rng UNIT_GUMBEL).
// Here element (bh, i, j) of that tensor is a pure function of (seed, bh, i, j), so the two passes of
// the fused kernels regenerate it instead of reading 4 bytes per logit from HBM:
//   k0 = mix(seed_lo ^ mix(bh + 0x9E3779B9)),  k1 = mix(seed_hi ^ k0 ^ 0x85EBCA6B)
//   a_i = mix(i ^ k0),  b_j = mix(j ^ k1) | 1,  x = a_i * b_j,  x ^= x >> 16
//   u = ((x >> 9) + 0.5) * 2^-23  in (0,1);   E = -ln(u) ~ Exp(1);   gumbel = -ln(E)
// with mix = the lowbias32 integer finaliser.  a_i and b_j are fully mixed per-row / per-column values, so
// the per-element cost is one 32-bit multiply and one xor-shift; the top 23 bits of the product of two
// mixed words pass the uniformity, neighbour-correlation, pair and 2x2 mixed-difference tests that a
// one-round mix of the sum a_i + b_j fails (its additive structure survives one round).
#pragma once
#include <stdint.h>

#if defined(__HIPCC__)
#define FT_HD __host__ __device__ __forceinline__
#else
#define FT_HD inline
#endif

namespace ft {

FT_HD uint32_t mix32(uint32_t x) {
  x ^= x >> 16;
  x *= 0x7FEB352Du;
  x ^= x >> 15;
  x *= 0x846CA68Bu;
  x ^= x >> 16;
  return x;
}

struct NoiseKeys {
  uint32_t k0, k1;
};

FT_HD NoiseKeys noise_keys(uint64_t seed, uint32_t bh) {
  NoiseKeys k;
  k.k0 = mix32((uint32_t)seed ^ mix32(bh + 0x9E3779B9u));
  k.k1 = mix32((uint32_t)(seed >> 32) ^ k.k0 ^ 0x85EBCA6Bu);
  return k;
}

FT_HD uint32_t noise_row(NoiseKeys k, uint32_t i) { return mix32(i ^ k.k0); }
FT_HD uint32_t noise_col(NoiseKeys k, uint32_t j) { return mix32(j ^ k.k1) | 1u; }

// u in (0,1) from the row and column terms; exact in fp32.
FT_HD float noise_uniform(uint32_t a_i, uint32_t b_j) {
  uint32_t x = a_i * b_j;
  x ^= x >> 16;
#if defined(__HIP_DEVICE_COMPILE__)
  // (x >> 9) | 0x3f800000 in one v_alignbit_b32 is 1 + k 2^-23; subtracting 1 - 2^-24 leaves (k + 0.5) 2^-23,
  // exactly, the value the arithmetic form below computes
  return __builtin_bit_cast(float, __builtin_amdgcn_alignbit(0x7Fu, x, 9u)) - 0.99999994f;
#else
  return (float)(x >> 9) * 1.1920928955078125e-07f + 5.9604644775390625e-08f;
#endif
}

// log2(E) of E = -ln(u) = -ln2 * log2(u), as log2(-log2 u) + log2(ln 2): the constant is folded by callers
constexpr float kLog2Ln2 = -0.5287663729448977f;

}  // namespace ft
