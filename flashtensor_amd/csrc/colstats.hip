// Per-key column statistics of the attention probabilities for gfx950 (pass B of H2O / RoCo / KeyFormer).
//
// Replaces the column-reduction kernels the reference would emit for h2o_score = probs.sum(dim=2)
// (cases/kernels/h2o.py:35-36), roco_score / roco_sq_score (cases/kernels/roco.py:42-46) and
// kf_score (cases/kernels/kf.py:36-40): sum over query rows i of p_ij, p_ij^2, or of the
// Gumbel-perturbed softmax, with p_ij = exp2(logit2_ij - lse2_i) recomputed from Q, K and the per-row
// normaliser written by the attention pass.  No S x S tensor is written or read (KeyFormer's tensor mode
// reads the noise input once more, as the reference's definition requires).
//
// Mapping.  Key-stationary: one workgroup owns 128 key columns of one (b, h), 4 waves x 32 keys, holds
// their K fragment in registers as the MFMA B operand and streams 64-row Q tiles through double-buffered
// LDS.  S = Q K^T as 16x16 blocks (v_mfma_f32_16x16x32: the same rate as the 32x32x16 shape for a quarter of
// the accumulator traffic per instruction, which on a power-limited chip is clock): a lane owns two key
// columns (l % 16 and 16 + l % 16 of the wave's 32) and 4 of the 16 query rows of each block, so the
// reduction over query rows is a chain of in-lane adds carried across the whole loop; the four quarter-columns
// are combined across lanes l ^ 16, l ^ 32 at the very end.  The modes that read an S x S tensor keep the
// 32x32x16 shape (a lane owns one key column and 16 rows of each 32x32 block: 32 lanes then read 128
// contiguous bytes of a tensor row).  Each output element has exactly one writer: deterministic, no atomics.
#include "device_common.hpp"
#include "kernel_params.h"
#include "noise.h"

#include <type_traits>

namespace ft {

constexpr int kColBK = 128;  // keys per workgroup
constexpr int kColBQ = 64;   // query rows per tile
constexpr int kColThreads = 256;

// waves per SIMD the register budget is sized for: the sum / sum-of-squares variants with a short logit chain
// (packed rounding, or logits kept in fp32) fit three
template <typename T, bool CAUSAL, bool EMU, int MODE>
constexpr int colstats_waves_per_simd() {
  return (MODE == kStatSum || MODE == kStatSumSq) ? 3 : 2;
}

template <typename T, int D, bool CAUSAL, bool EMU, int MODE>
__global__ void __launch_bounds__(kColThreads, (colstats_waves_per_simd<T, CAUSAL, EMU, MODE>())) colstats_kernel(const ColstatsKernelParams p) {
  constexpr int BK = kColBK, BQ = kColBQ, NT = kColThreads;
  constexpr int KSTEPS = D / 16;
  typedef TileGeom<D> G;
  typedef typename T::vec8 vec8;
  constexpr int TILE_BYTES = BQ * G::RB;
  constexpr bool KFM = (MODE == kStatKfTensor || MODE == kStatKfSeeded);                 // generic KeyFormer modes
  constexpr bool KFP = (MODE == kStatKfSeededTau1 || MODE == kStatKfSeededFast);         // seeded noise in the packed path
  constexpr bool kSeeded = MODE == kStatKfSeeded || KFP;
  constexpr bool CORM = (MODE == kStatCormRule || MODE == kStatCormTensor);
  constexpr bool kPacked = __is_same(typename T::elem, _Float16) && EMU;  // packed-fp16 rounding chain
  constexpr bool kPlainF32 = !EMU;                                        // logits stay in fp32: one fma per element
  constexpr bool kTensor = MODE == kStatKfTensor || MODE == kStatCormTensor;
  constexpr bool k16 = !kTensor;            // 16x16x32 blocks; the tensor modes stay on 32x32x16
  constexpr int NKEY = k16 ? 2 : 1;         // key columns per lane
  constexpr int NBLK = k16 ? 4 : 8;         // groups of 4 query rows per lane and key in a tile
  constexpr int KS16 = D / 32;
  // one LDS object per buffer: reads of one do not wait for the direct-to-LDS loads in flight into the other
  __shared__ __align__(16) char ldsQ0[TILE_BYTES];
  __shared__ __align__(16) char ldsQ1[TILE_BYTES];
  __shared__ __align__(16) char ldsQ2[TILE_BYTES];  // tile t lives in buffer t % 3: two tiles in flight behind the one being read
  __shared__ __align__(16) float ldsLse[2 * BQ];     // row normalisers of the current / next tile
  __shared__ __align__(16) uint32_t ldsRow[2 * BQ];  // noise row terms (seeded KeyFormer)

  const int BH = p.B * p.H;
  // Low key blocks see the most rows under the causal mask: heaviest first, every (b, h) pair's block 0 before any
  // pair's block 1.  (Letting an XCD finish one pair's blocks before the next pair's, which pays in the attention
  // pass, loses that balance here: measured 974 against 955 us for the B4 H32 S4096 sum-of-squares call, 267
  // against 239 us at B1.)
  const int bh = blockIdx.x % BH;
  int jb = blockIdx.x / BH;
  if (p.pair_order) {
    // Two workgroups per CU, all resident from the start: nothing is left to hand out as CUs free up, so the heavy half
    // is dealt first, descending, and the light half after it ascending, which puts a heavy and a light block on the
    // same CU (as in the attention pass).
    const int nJB = gridDim.x / BH, half = (nJB + 1) / 2;
    jb = jb < half ? jb : nJB - 1 - (jb - half);
  }
  const int b = bh / p.H, h = bh % p.H;
  const int j0 = jb * BK;
  const int lane = lane_id(), wave = wave_id();
  const int g = lane >> 5, n = lane & 31;      // 32x32 blocks: half and column
  const int q4l = lane >> 4, n16 = lane & 15;  // 16x16 blocks: quarter and column
  const int rsub = k16 ? 4 * q4l : 4 * g;      // first of the lane's 4 rows inside a group of 16 (8) rows
  int kjs[NKEY], kjs_c[NKEY];                  // the lane's key columns
#pragma unroll
  for (int key = 0; key < NKEY; ++key) {
    kjs[key] = j0 + wave * 32 + (k16 ? 16 * key + n16 : n);
    kjs_c[key] = kjs[key] < p.Skv ? kjs[key] : p.Skv - 1;
  }
  const int kj_c = kjs_c[0];
  const float POS_INF = __builtin_inff();
  const float NEG_INF = -__builtin_inff();

  // stationary B operand.  32x32: kf[t] = key n, channels 16 t + 8 g + [0..7]; 16x16: kf[key * KS16 + t] = key
  // 16 key + n16, channels 32 t + 8 q4l + [0..7]
  vec8 kf[KSTEPS];
  if constexpr (k16) {
#pragma unroll
    for (int key = 0; key < 2; ++key) {
      const uint16_t* kptr = p.k + b * p.sk.b + (int64_t)kjs_c[key] * p.sk.s + (h / p.group) * p.sk.h;
#pragma unroll
      for (int t = 0; t < KS16; ++t) kf[key * KS16 + t] = *reinterpret_cast<const vec8*>(kptr + 32 * t + 8 * q4l);
    }
  } else {
    const uint16_t* kptr = p.k + b * p.sk.b + (int64_t)kj_c * p.sk.s + (h / p.group) * p.sk.h;
#pragma unroll
    for (int t = 0; t < KSTEPS; ++t) kf[t] = *reinterpret_cast<const vec8*>(kptr + 16 * t + 8 * g);
  }

  const uint16_t* qbase = p.q + b * p.sq.b + h * p.sq.h;
  const float* lse_bh = p.lse + (int64_t)bh * p.Sq;

  // first query row that can see key j0 is j0 - off
  int i_begin = 0;
  if (CAUSAL) i_begin = max(0, j0 - p.off) / BQ * BQ;
  const int ntiles = (p.Sq - i_begin + BQ - 1) / BQ;  // <= 0 when no row sees this block
  // leading tiles in which some (row, key) pair of this wave is above the diagonal
  const int wave_key0 = j0 + wave * 32;
  int n_masked = 0;
  if (CAUSAL) n_masked = max(0, min(ntiles, (wave_key0 + 31 - p.off - i_begin + BQ - 1) / BQ));

  NoiseKeys nk = {0, 0};
  uint32_t b_j[NKEY] = {};
  const float* er_col = nullptr;
  if (kSeeded) {
    nk = noise_keys(p.seed, (uint32_t)bh);
#pragma unroll
    for (int key = 0; key < NKEY; ++key) b_j[key] = noise_col(nk, (uint32_t)kjs[key]);
  }
  if (MODE == kStatKfTensor || MODE == kStatCormTensor) er_col = p.exp_rand + b * p.er_sb + h * p.er_sh + kj_c;

  TileStager<D, BQ, NT, kRowSwizzle> stQ;
  stQ.init(qbase, p.sq.s);
  // 32x32: Q row n (and n + 32 via an immediate), chunk 2t + g; 16x16: Q row n16 (+ 16, 32, 48), chunk 4t + q4l
  // (rows 16 apart share their swizzle)
  uint32_t qoff[KSTEPS];
#pragma unroll
  for (int t = 0; t < KSTEPS; ++t)
    qoff[t] = k16 ? n16 * G::RB + (((4 * (t % KS16) + q4l) ^ G::row_swz(n16)) << 4) : n * G::RB + (((2 * t + g) ^ G::row_swz(n)) << 4);

  float sum[NKEY][4] = {}, sumsq[NKEY][4] = {};  // independent chains
  // CoRM: running maximum over the rows of log2(p / threshold) (rule mode) or p - threshold (tensor mode).
  // A probability within kCormSlack (relative) of its threshold counts as reaching it: the cases that sit
  // exactly on the boundary in the reference (p_00 == 1 against 1, equal logits against 1 / (i + 1)) are
  // kept as they are there, whatever the last bit of the normaliser.
  constexpr float kCormSlack = 1e-6f;
  float best[NKEY][4];
#pragma unroll
  for (int key = 0; key < NKEY; ++key)
#pragma unroll
    for (int e = 0; e < 4; ++e) best[key][e] = NEG_INF;

  auto stage_q = [&](int t, char* dst) {
    if (t < ntiles) stQ.issue(i_begin + t * BQ, min(BQ, p.Sq - (i_begin + t * BQ)), dst);
  };
  // Tensor modes: this lane's slice of the S x S noise / threshold tensor for one tile (its key column, the rows
  // of its score registers; 32 lanes read 128 contiguous bytes of a row), fetched one tile ahead of its use:
  // the tensor is the only operand that comes from HBM every time, and a load consumed in the iteration that
  // issues it leaves the memory system idle while the tile is worked on.  Tiles the causal mask hides from the
  // wave are not read, and the loads carry the non-temporal hint: the tensor is read once and should not evict Q.
  float er[2][16], er_nx[2][16];
  auto load_er = [&](float (&dst)[2][16], int t) {
    const int i0 = i_begin + t * BQ;
    // nothing to fetch past the last tile, or when no row of the tile sees a key of this wave
    if (t >= ntiles || (CAUSAL && wave_key0 > i0 + BQ - 1 + p.off)) return;
    const float* row0 = er_col + (int64_t)(i0 + 4 * g) * p.er_sr;
    if (i0 + BQ <= p.Sq && !(CAUSAL && wave_key0 + 31 > i0 + p.off)) {  // every pair of the tile is visible
#pragma unroll
      for (int mbk = 0; mbk < 2; ++mbk)
#pragma unroll
        for (int r = 0; r < 16; ++r)
          dst[mbk][r] = __builtin_nontemporal_load(row0 + (int64_t)(32 * mbk + 8 * (r >> 2) + (r & 3)) * p.er_sr);
    } else {
      // Straddles the diagonal or the end of Q.  No branches and nothing that waits for a load here: a pair that
      // does not exist (hidden by the mask, or past the last row) takes the element of the nearest visible pair of
      // its key instead.  Its probability is zero, so the noise does not matter, and a threshold it could reach
      // (<= 0) is reached by that visible pair as well.
#pragma unroll
      for (int mbk = 0; mbk < 2; ++mbk)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          int i = i0 + 4 * g + 32 * mbk + 8 * (r >> 2) + (r & 3);
          if (CAUSAL) i = max(i, kj_c - p.off);
          i = min(i, p.Sq - 1);
          dst[mbk][r] = __builtin_nontemporal_load(er_col + (int64_t)i * p.er_sr);
        }
    }
  };
  // rows of tile t: negated normaliser (-inf past Sq, so that those rows contribute exp2(-inf) = 0) and noise
  // row term.  The normaliser is fetched one iteration before it is parked in LDS, so that no wave sits
  // out a global-memory round trip inside the loop.
  auto load_rows = [&](int t) -> float {
    const int i = i_begin + t * BQ + threadIdx.x;
    return (t < ntiles && threadIdx.x < BQ && i < p.Sq) ? lse_bh[i] : POS_INF;
  };
  auto store_rows = [&](int t, float lse_i) {
    if (t < ntiles && threadIdx.x < BQ) {
      const int i = i_begin + t * BQ + threadIdx.x;
      float nl = -lse_i;  // negated: one fma per logit
      // CoRM rule: p_ij >= 1 / (i + 1)  <=>  log2 p_ij + log2(i + 1) >= 0, so no exponential is needed
      if (MODE == kStatCormRule) nl += __builtin_amdgcn_logf((float)(i + 1));
      if (MODE == kStatKfSeededFast) nl -= kLog2Ln2 * p.inv_tau;  // the constant part of -log2(E) / tau
      ldsLse[(t & 1) * BQ + threadIdx.x] = nl;
      if (kSeeded) ldsRow[(t & 1) * BQ + threadIdx.x] = noise_row(nk, (uint32_t)i);
    }
  };

  // ---- score registers of one tile: 16x16 blocks [query block][key column] of 4 rows, or 32x32 blocks [query half] of 16
  struct STile {
    float4v q[k16 ? 4 : 1][2];
    float16v h[k16 ? 1 : 2];
  };
  // rows 16 (8) blk' + rsub + [0..3] of the tile, key column `key` of the lane
  auto sval = [&](const STile& s, int blk, int key, int e) __attribute__((always_inline)) -> float {
    if constexpr (k16)
      return s.q[blk][key][e];
    else
      return s.h[blk >> 2][4 * (blk & 3) + e];
  };

  // ---- S = Q K^T : [64 queries] x [32 keys]; 16 LDS reads, 16 MFMAs of 32x32x16 or 32 of 16x16x32
  auto qk = [&](STile& s, const char* tq) __attribute__((always_inline)) {
    // operand ring: reads run kAhead steps ahead of the MFMAs that consume them
    if constexpr (k16) {
#pragma unroll
      for (int qb = 0; qb < 4; ++qb)
#pragma unroll
        for (int key = 0; key < 2; ++key) s.q[qb][key] = float4v{0.f, 0.f, 0.f, 0.f};
      constexpr int NR = 4 * KS16;  // reads per tile: query block r / KS16, k-step r % KS16; each feeds both key columns
      constexpr int kAhead = 3;
      vec8 qa[kAhead + 1];
#pragma unroll
      for (int r = 0; r < kAhead; ++r) qa[r] = *reinterpret_cast<const vec8*>(tq + qoff[r % KS16] + (r / KS16) * 16 * G::RB);
#pragma unroll
      for (int r = 0; r < NR; ++r) {
        if (r + kAhead < NR)
          qa[(r + kAhead) % (kAhead + 1)] = *reinterpret_cast<const vec8*>(tq + qoff[(r + kAhead) % KS16] + ((r + kAhead) / KS16) * 16 * G::RB);
#pragma unroll
        for (int key = 0; key < 2; ++key)
          s.q[r / KS16][key] = T::mfma16(qa[r % (kAhead + 1)], kf[key * KS16 + r % KS16], s.q[r / KS16][key]);
      }
    } else {
#pragma unroll
      for (int mbk = 0; mbk < 2; ++mbk)
#pragma unroll
        for (int r = 0; r < 16; ++r) s.h[mbk][r] = 0.f;
      constexpr int kAhead = 1;  // the registers go to the prefetched tensor slice
      vec8 qa[kAhead + 1][2];
#pragma unroll
      for (int t = 0; t < kAhead; ++t)
#pragma unroll
        for (int mbk = 0; mbk < 2; ++mbk) qa[t][mbk] = *reinterpret_cast<const vec8*>(tq + qoff[t] + mbk * 32 * G::RB);
#pragma unroll
      for (int t = 0; t < KSTEPS; ++t) {
        if (t + kAhead < KSTEPS) {
#pragma unroll
          for (int mbk = 0; mbk < 2; ++mbk)
            qa[(t + kAhead) % (kAhead + 1)][mbk] = *reinterpret_cast<const vec8*>(tq + qoff[t + kAhead] + mbk * 32 * G::RB);
        }
#pragma unroll
        for (int mbk = 0; mbk < 2; ++mbk) s.h[mbk] = T::mfma(qa[t % (kAhead + 1)][mbk], kf[t], s.h[mbk]);
      }
    }
  };

  // ---- probabilities of one tile from its raw scores, summed down the query axis in-lane
  // (one group of rows at a time: blk)
  auto block_row0 = [&](int blk) __attribute__((always_inline)) -> int { return (k16 ? 16 * blk : 32 * (blk >> 2) + 8 * (blk & 3)) + rsub; };
  auto reduce_block = [&](auto masked_tag, const STile& s, int t, int blk, const float4v nlse4, const uint4v row4) __attribute__((always_inline)) {
    constexpr bool MASKED = decltype(masked_tag)::value;
    const int i0 = i_begin + t * BQ;
    const half2v pk_hi = __builtin_bit_cast(half2v, p.pk_hi2), pk_lo = __builtin_bit_cast(half2v, p.pk_lo2);
    // key kj is hidden from row i0 + il when kj > i0 + il + off, i.e. il < kj - i0 - off; il = il0 + rsub + e
    int lim[NKEY];
#pragma unroll
    for (int key = 0; key < NKEY; ++key) lim[key] = kjs[key] - i0 - p.off - rsub;
    {
      const int il0 = k16 ? 16 * blk : 32 * (blk >> 2) + 8 * (blk & 3);  // + rsub + e
#pragma unroll
      for (int key = 0; key < NKEY; ++key) {
        float x[4];
        if (kPlainF32 && !KFM && !KFP) {
#pragma unroll
          for (int e = 0; e < 4; ++e) x[e] = __builtin_fmaf(sval(s, blk, key, e), p.logit_mul, nlse4[e]);
        } else if (EMU && !kPacked && !KFM && !KFP) {
          // bf16: round QK^T, multiply by the tuned constant (== dividing by sqrt(D) in bf16), round again
#pragma unroll
          for (int e = 0; e < 4; e += 2) {
            const uint32_t h2 = T::pack2(sval(s, blk, key, e), sval(s, blk, key, e + 1));
            const uint32_t t2 = T::pack2(T::lo(h2) * p.logit_mul, T::hi(h2) * p.logit_mul);
            x[e] = __builtin_fmaf(T::lo(t2), kLog2e, nlse4[e]);
            x[e + 1] = __builtin_fmaf(T::hi(t2), kLog2e, nlse4[e + 1]);
          }
        } else if (kPacked && !KFM) {
#pragma unroll
          for (int e = 0; e < 4; e += 2) {
            const float2v a2 = {sval(s, blk, key, e), sval(s, blk, key, e + 1)};
            const half2v h2 = __builtin_convertvector(a2, half2v);         // QK^T is an fp16 tensor in the reference
            // ... divided by sqrt(D) in fp16: t2 = 8 * f16(h / sqrt(D)), exact for D = 64, two packed ops for D = 128
            const half2v t2 = D == 64 ? h2 : __builtin_elementwise_fma(h2, pk_hi, h2 * pk_lo);
            if (MODE == kStatKfSeededFast) {
              // ((t log2e - log2 E) / tau) - lse: E = -ln u in [6e-8, 16.7]
              // log2 E = log2(-log2 u) + log2(ln 2); the constant rides in the row normaliser staged in LDS
              const float l0 = __builtin_amdgcn_logf(-__builtin_amdgcn_logf(noise_uniform(row4[e], b_j[key])));
              const float l1 = __builtin_amdgcn_logf(-__builtin_amdgcn_logf(noise_uniform(row4[e + 1], b_j[key])));
              x[e] = __builtin_fmaf(__builtin_fmaf((float)t2[0], kLog2e / 8.f, -l0), p.inv_tau, nlse4[e]);
              x[e + 1] = __builtin_fmaf(__builtin_fmaf((float)t2[1], kLog2e / 8.f, -l1), p.inv_tau, nlse4[e + 1]);
            } else {
              x[e] = __builtin_fmaf((float)t2[0], kLog2e / 8.f, nlse4[e]);
              x[e + 1] = __builtin_fmaf((float)t2[1], kLog2e / 8.f, nlse4[e + 1]);
            }
          }
        } else {
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            float v = sval(s, blk, key, e);
            if (EMU) {
              v = T::to_float(T::from_float(v));
              v = T::to_float(T::from_float(v * p.logit_mul));
              v *= kLog2e;
            } else {
              v *= p.logit_mul;
            }
            if (KFM) {
              float log2E;
              if (MODE == kStatKfTensor) {
                log2E = __builtin_amdgcn_logf(er[blk >> 2][4 * (blk & 3) + e]);
              } else {
                const float u = noise_uniform(row4[e], b_j[key]);
                log2E = __builtin_amdgcn_logf(-kLn2 * __builtin_amdgcn_logf(u));
              }
              v = (v - log2E) * p.inv_tau;
            }
            x[e] = v + nlse4[e];  // rows past Sq carry -inf -> p = 0
          }
        }
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          float xv = x[e];
          if (MASKED) xv = (il0 + e < lim[key]) ? NEG_INF : xv;
          if (MODE == kStatCormRule) {
            best[key][e] = fmaxf(best[key][e], xv);
          } else {
            float pr = __builtin_amdgcn_exp2f(xv);
            if (MODE == kStatKfSeededTau1)  // exp(t - lse) / log2 u = -ln2 exp(t - lse) / E; the factor is applied to the total
              pr *= __builtin_amdgcn_rcpf(__builtin_amdgcn_logf(noise_uniform(row4[e], b_j[key])));
            if (MODE == kStatCormTensor) {
              best[key][e] = fmaxf(best[key][e], pr - er[blk >> 2][4 * (blk & 3) + e] * (1.f - kCormSlack));
            } else {
              sum[key][e] += pr;
              if (MODE == kStatSumSq) sumsq[key][e] = __builtin_fmaf(pr, pr, sumsq[key][e]);
            }
          }
        }
      }
    }
  };
  auto reduce_tile = [&](auto masked_tag, const STile& s, int t) __attribute__((always_inline)) {
#pragma unroll
    for (int blk = 0; blk < NBLK; ++blk) {
      const float4v nlse4 = *reinterpret_cast<const float4v*>(ldsLse + (t & 1) * BQ + block_row0(blk));
      uint4v row4 = {0, 0, 0, 0};
      if (kSeeded) row4 = *reinterpret_cast<const uint4v*>(ldsRow + (t & 1) * BQ + block_row0(blk));
      reduce_block(masked_tag, s, t, blk, nlse4, row4);
    }
  };
  // 16x16 blocks, mask-free tiles: the probabilities of tile t from s, and the scores of the next tile (its Q
  // rows at tq) into the same registers, one query block at a time.  A block's registers are free once its
  // probabilities have been summed, so the MFMAs of block qb of the next tile run beside the vector work of
  // block qb + 1 of this one, and one set of score registers serves both tiles; nothing moves from one stage to
  // another.
  auto reduce_qk = [&](STile& s, const char* tq, int t) __attribute__((always_inline)) {
    constexpr int NR = 4 * KS16, kAhead = 5;  // operand reads in flight ahead of their MFMAs
    vec8 qa[kAhead + 1];
    auto rd = [&](int r) __attribute__((always_inline)) -> vec8 {
      return *reinterpret_cast<const vec8*>(tq + qoff[r % KS16] + (r / KS16) * 16 * G::RB);
    };
#pragma unroll
    for (int r = 0; r < kAhead; ++r) qa[r] = rd(r);
    // the row terms of every block up front: a stage that began with its own LDS read would wait for it
    float4v nl[4];
    uint4v rw[4];
#pragma unroll
    for (int qb = 0; qb < 4; ++qb) {
      nl[qb] = *reinterpret_cast<const float4v*>(ldsLse + (t & 1) * BQ + block_row0(qb));
      rw[qb] = uint4v{0, 0, 0, 0};
      if (kSeeded) rw[qb] = *reinterpret_cast<const uint4v*>(ldsRow + (t & 1) * BQ + block_row0(qb));
    }
    reduce_block(std::false_type{}, s, t, 0, nl[0], rw[0]);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int qb = 0; qb < 4; ++qb) {
#pragma unroll
      for (int key = 0; key < 2; ++key) s.q[qb][key] = float4v{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int r = qb * KS16; r < (qb + 1) * KS16; ++r) {
        if (r + kAhead < NR) qa[(r + kAhead) % (kAhead + 1)] = rd(r + kAhead);
#pragma unroll
        for (int key = 0; key < 2; ++key)
          s.q[qb][key] = T::mfma16(qa[r % (kAhead + 1)], kf[key * KS16 + r % KS16], s.q[qb][key]);
      }
      if (qb < 3) {
        reduce_block(std::false_type{}, s, t, qb + 1, nl[qb + 1], rw[qb + 1]);
#pragma unroll
        for (int i = 0; i < 2 * KS16; ++i) {
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
          __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
          __builtin_amdgcn_sched_group_barrier(0x002, ((KFM || KFP) ? 48 : 24) / KS16, 0);
        }
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    // the running sums are next read in the following tile, in another basic block (the staging branches lie
    // between): without a use here the whole vector chain of this tile is sunk into that block, away from the MFMAs
    // it was meant to run beside
#pragma unroll
    for (int key = 0; key < NKEY; ++key)
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        if (MODE == kStatCormRule) {
          asm volatile("" : "+v"(best[key][e]));
        } else {
          asm volatile("" : "+v"(sum[key][e]));
          if (MODE == kStatSumSq) asm volatile("" : "+v"(sumsq[key][e]));
        }
      }
  };
  STile S0;
  if (ntiles > 0) {
    // ---- prologue: Q[0], Q[1], Q[2] in flight; rows of tile 0; scores of tile 0
    if (kTensor) load_er(er, 0);
    stage_q(0, ldsQ0);
    stage_q(1, ldsQ1);
    stage_q(2, ldsQ2);
    store_rows(0, load_rows(0));
    float lse_next = load_rows(1);  // rows of the tile after the current one, in flight
    wait_vmem();
    __syncthreads();
    qk(S0, ldsQ0);

    // One iteration = one barrier.  On entry to iteration t, S0 holds the scores of tile t, Q[t+1] (read in this
    // iteration) and Q[t+2] have been requested; Q[t+3] is requested into the buffer of tile t.  The wait at the
    // top is for Q[t+1] only: loads complete in order, and the staging loads of Q[t+2] (kStageLoads per thread, the
    // newest in flight) may stay outstanding.  The row normalisers of tile t+2 are fetched before those staging
    // loads, so that waiting for them does not wait for the tile.
    constexpr int kStageLoads = BQ * G::CPR / NT;
    static_assert(kStageLoads == 4 || kStageLoads == 2, "s_waitcnt immediates below");
    auto wait_tile = [&](int t) __attribute__((always_inline)) {
      if (!kTensor && t + 2 < ntiles) {
        // vmcnt(kStageLoads) lgkmcnt(0); a bare barrier: __syncthreads() carries a fence that drains every load
        __builtin_amdgcn_s_waitcnt(kStageLoads == 4 ? 0x0074 : 0x0072);
        __builtin_amdgcn_s_barrier();
      } else {
        wait_vmem();
        __syncthreads();
      }
    };
    char *b0 = ldsQ0, *b1 = ldsQ1, *b2 = ldsQ2;  // buffers of tiles t, t + 1, t + 2
    auto rotate = [&]() __attribute__((always_inline)) {
      char* f = b0;
      b0 = b1, b1 = b2, b2 = f;
    };
    auto take_next_er = [&]() {
      // nothing of the tile may be scheduled below this point: the wait for the prefetched slice (which, loads
      // completing in order, is also a wait for the Q tile queued behind it) belongs at the very end
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int mbk = 0; mbk < 2; ++mbk)
#pragma unroll
        for (int r = 0; r < 16; ++r) er[mbk][r] = er_nx[mbk][r];
    };
    int t = 0;
    for (; t < n_masked; ++t) {
      wait_tile(t);
      if (kTensor) load_er(er_nx, t + 1);  // ahead of the staging loads: waiting for it does not wait for them
      store_rows(t + 1, lse_next);
      lse_next = load_rows(t + 2);
      stage_q(t + 3, b0);
      // every row of this tile above the diagonal for all 32 keys of the wave: nothing to add
      const bool skip = CAUSAL && (wave_key0 > i_begin + t * BQ + BQ - 1 + p.off);
      if (!skip) reduce_tile(std::true_type{}, S0, t);
      qk(S0, b1);
      if (kTensor) take_next_er();
      rotate();
    }
    // Tensor modes are bound by the HBM stream of the tensor: one tile per trip, the registers of the second
    // score buffer hold the prefetched slice instead.
    if (kTensor) {
      for (; t < ntiles; ++t) {
        wait_tile(t);
        load_er(er_nx, t + 1);
        store_rows(t + 1, lse_next);
        lse_next = load_rows(t + 2);
        stage_q(t + 3, b0);
        reduce_tile(std::false_type{}, S0, t);
        qk(S0, b1);
        take_next_er();
        rotate();
      }
    }
    // mask-free tiles (the tensor modes have none left here)
    if constexpr (k16) {
      // While tile t + 3 is a whole tile every load of an iteration is issued unconditionally, so that the waits
      // can be counted: kStageLoads staging loads (Q[t+2]) stay in flight across the barrier.  A clean start
      // (nothing outstanding) keeps the compiler's own wait for the row normalisers at that count as well.
      const int nfull = (p.Sq - i_begin) / BQ;  // whole tiles
      if (t + 3 < nfull) wait_vmem();
      for (; t + 3 < nfull; ++t) {
        // vmcnt(kStageLoads) lgkmcnt(0), then a bare barrier: __syncthreads() carries a fence that drains every load
        __builtin_amdgcn_s_waitcnt(kStageLoads == 4 ? 0x0074 : 0x0072);
        __builtin_amdgcn_s_barrier();
        if (threadIdx.x < BQ) {
          const int i = i_begin + (t + 1) * BQ + threadIdx.x;
          float nl = -lse_next;
          if (MODE == kStatCormRule) nl += __builtin_amdgcn_logf((float)(i + 1));
          if (MODE == kStatKfSeededFast) nl -= kLog2Ln2 * p.inv_tau;
          ldsLse[((t + 1) & 1) * BQ + threadIdx.x] = nl;
          if (kSeeded) ldsRow[((t + 1) & 1) * BQ + threadIdx.x] = noise_row(nk, (uint32_t)i);
        }
        lse_next = lse_bh[i_begin + (t + 2) * BQ + (threadIdx.x & (BQ - 1))];
        __builtin_amdgcn_sched_barrier(0);  // the normalisers first: their wait must not reach into the staging loads
        stQ.issue_full(i_begin + (t + 3) * BQ, b0);
        reduce_qk(S0, b1, t);
        rotate();
      }
      for (; t < ntiles; ++t) {
        wait_tile(t);
        store_rows(t + 1, lse_next);
        lse_next = load_rows(t + 2);
        stage_q(t + 3, b0);
        reduce_qk(S0, b1, t);  // scores of tile t + 1: past the last tile they come from stale LDS and are discarded
        rotate();
      }
    }
  }

  // the lanes that share a key column: l ^ 32 (32x32 blocks), l ^ 16 and l ^ 32 (16x16 blocks)
  auto across = [&](float x, auto op) __attribute__((always_inline)) -> float {
    if constexpr (k16) x = op(x, __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute((lane ^ 16) << 2, __builtin_bit_cast(int, x))));
    return op(x, xchg32(x));
  };
  auto add = [](float a, float c) { return a + c; };
  auto mx = [](float a, float c) { return fmaxf(a, c); };
  const bool writer = k16 ? q4l == 0 : g == 0;
#pragma unroll
  for (int key = 0; key < NKEY; ++key) {
    float tot = across((sum[key][0] + sum[key][1]) + (sum[key][2] + sum[key][3]), add);
    if (MODE == kStatKfSeededTau1) tot *= -kLog2e;
    float totsq = (sumsq[key][0] + sumsq[key][1]) + (sumsq[key][2] + sumsq[key][3]);
    if (MODE == kStatSumSq) totsq = across(totsq, add);
    float top = fmaxf(fmaxf(best[key][0], best[key][1]), fmaxf(best[key][2], best[key][3]));
    if (CORM) top = across(top, mx);
    if (writer && kjs[key] < p.Skv) {
      const int64_t idx = (int64_t)bh * p.Skv + kjs[key];
      if (CORM) {
        p.keep[idx] = top >= (MODE == kStatCormRule ? -kCormSlack * kLog2e : 0.f) ? 1 : 0;
        if (p.colsum) p.colsum[idx] = top;  // optional: distance from the decision boundary
      } else {
        p.colsum[idx] = tot;
        if (MODE == kStatSumSq) p.colsumsq[idx] = totsq;
      }
    }
  }
}

// ---------------------------------------------------------------------------------------------------

int device_cu_count();  // attn_fwd.hip

template <typename T, int D, bool CAUSAL, bool EMU, int MODE>
static hipError_t launch_one(const ColstatsKernelParams& p, hipStream_t stream) {
  const int nJB = (p.Skv + kColBK - 1) / kColBK;
  dim3 grid((unsigned)(nJB * p.B * p.H));
  ColstatsKernelParams pp = p;
  const int64_t cus = device_cu_count();
  pp.pair_order = CAUSAL && (int64_t)grid.x > cus && (int64_t)grid.x <= 2 * cus;
  hipLaunchKernelGGL((colstats_kernel<T, D, CAUSAL, EMU, MODE>), grid, dim3(kColThreads), 0, stream, pp);
  return hipGetLastError();
}

template <typename T, int D>
static hipError_t launch_td(const ColstatsKernelParams& p, bool causal, bool emu, int mode, hipStream_t s) {
#define FT_CASE(C, E, M) \
  if (causal == C && emu == E && mode == M) return launch_one<T, D, C, E, M>(p, s);
#define FT_MODES(C, E)                                                                                       \
  FT_CASE(C, E, kStatSum) FT_CASE(C, E, kStatSumSq) FT_CASE(C, E, kStatKfTensor) FT_CASE(C, E, kStatKfSeeded) \
  FT_CASE(C, E, kStatCormRule) FT_CASE(C, E, kStatCormTensor)
  FT_MODES(true, true) FT_MODES(true, false) FT_MODES(false, true) FT_MODES(false, false)
  if constexpr (std::is_same<T, F16>::value) {  // packed KeyFormer modes: fp16 with reference rounding only
    if (emu) {
      FT_CASE(true, true, kStatKfSeededTau1) FT_CASE(false, true, kStatKfSeededTau1)
      FT_CASE(true, true, kStatKfSeededFast) FT_CASE(false, true, kStatKfSeededFast)
    }
  }
#undef FT_MODES
#undef FT_CASE
  return hipErrorInvalidValue;
}

hipError_t launch_colstats(const ColstatsKernelParams& p, int D, bool bf16, bool causal, bool emu, int mode,
                           hipStream_t s) {
  if (D == 128) return bf16 ? launch_td<BF16, 128>(p, causal, emu, mode, s) : launch_td<F16, 128>(p, causal, emu, mode, s);
  if (D == 64) return bf16 ? launch_td<BF16, 64>(p, causal, emu, mode, s) : launch_td<F16, 64>(p, causal, emu, mode, s);
  return hipErrorInvalidValue;
}

}  // namespace ft
