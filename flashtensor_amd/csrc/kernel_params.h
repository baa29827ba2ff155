// Launch-time parameter blocks shared by the host dispatcher and the kernels.
#pragma once
#include <stdint.h>

namespace ft {

struct Strides3 {
  int64_t b, s, h;
};

struct AttnKernelParams {
  const uint16_t* q;
  const uint16_t* k;
  const uint16_t* v;
  uint16_t* o;
  Strides3 sq, sk, sv, so;
  float* lse;     // [B,H,Sq] log2-domain normaliser of the plain softmax (may be null)
  float* lse_kf;  // [B,H,Sq] normaliser of the perturbed softmax (KeyFormer modes)
  const float* exp_rand;
  int64_t er_sb, er_sh, er_sr;
  int er_vec4;  // exp_rand rows can be read as aligned float4
  uint64_t seed;
  int B, H, Sq, Skv;
  int off;          // Skv - Sq: query i sees keys j <= i + off when causal
  float logit_mul;  // reference rounding: f16(f16(acc) * logit_mul) == f16(f16(acc) / sqrt(D)); fast: log2e / sqrt(D)
  float inv_tau;
  // packed fp16 form of the same division for D = 128 (two packed ops on element pairs instead of one
  // mixed-precision multiply per element): t8 = fma(h, pk_hi, h * pk_lo) is 8 * f16(h / sqrt(D)) for every
  // fp16 h except where |h / sqrt(D)| < 2.5e-3, and there within 2e-6 of it; both halves hold the constant
  uint32_t pk_hi2, pk_lo2;
  float softcap;    // kKfSoftcap: logits become softcap * tanh(logit / softcap)
  int pair_order;   // block order of the causal attention kernel: heavy half descending, light half ascending
  int group;        // query heads per k/v head: query head h reads k/v head h / group
  int two_blocks;   // 256-row form: a workgroup takes query blocks nMB - 1 - slot and slot (set by the launcher)
  int head_major;   // workgroup order inside an XCD: all blocks of a (b, h) pair before the next pair's (launcher)
};

struct ColstatsKernelParams {
  const uint16_t* q;
  const uint16_t* k;
  Strides3 sq, sk;
  const float* lse;  // [B,H,Sq] normaliser of the distribution being summed
  float* colsum;     // [B,H,Skv]
  float* colsumsq;   // [B,H,Skv] or null
  uint8_t* keep;     // [B,H,Skv] CoRM modes: 1 where some row's probability reaches its threshold
  const float* exp_rand;  // KeyFormer noise [B,H,Sq,Skv]; CoRM tensor mode: thresholds [Sq,Skv] (er_sb = er_sh = 0)
  int64_t er_sb, er_sh, er_sr;
  uint64_t seed;
  int B, H, Sq, Skv;
  int off;
  float logit_mul;
  uint32_t pk_hi2, pk_lo2;  // as in AttnKernelParams
  float inv_tau;
  int group;  // query heads per k head
  int pair_order;  // key-block order for launches of two workgroups per CU: heavy half descending, light half ascending (launcher)
};

// what happens to a logit between the scaled QK^T and the softmax of the attention pass
// kKfSeededTau1 / kKfSeededFast: the seeded KeyFormer stream inside the packed fp16 path.  The perturbed
// weight exp((t + g) / tau) with g = -ln E equals exp(t / tau) E^(-1/tau); the in-kernel E lies in
// [6e-8, 16.7], so for tau >= 0.25 the plain softmax's running maximum also stabilises the perturbed sum
// (exponent <= (6 + 24) / tau <= 120) and no second maximum is tracked; tau == 1 needs 1 / E only.
// kKfTensorLds: the noise tensor of kKfTensor, its tiles landing in LDS by direct-to-LDS loads a whole tile ahead
// (16-byte aligned rows, Skv a multiple of 4, a (b, h) slice below 2 GiB; kKfTensor reads any layout into registers)
enum KfMode { kKfNone = 0, kKfTensor = 1, kKfSeeded = 2, kKfSoftcap = 3, kKfSeededTau1 = 4, kKfSeededFast = 5, kKfTensorLds = 6 };
// kStatCormRule: thresholds 1 / (i + 1) per query row i; kStatCormTensor: thresholds read from a tensor
enum StatMode {
  kStatSum = 0, kStatSumSq = 1, kStatKfTensor = 2, kStatKfSeeded = 3, kStatCormRule = 4, kStatCormTensor = 5,
  kStatKfSeededTau1 = 6, kStatKfSeededFast = 7  // seeded KeyFormer inside the packed fp16 path (see KfMode)
};

}  // namespace ft
