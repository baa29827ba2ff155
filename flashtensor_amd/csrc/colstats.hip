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
// LDS.  S = Q K^T with v_mfma_f32_32x32x16 leaves a lane with one key column (l % 32) and 16 of the 32
// query rows of each block, so the reduction over query rows is a chain of in-lane adds carried across
// the whole loop; the two half-columns are combined by one exchange with lane l ^ 32 at the very end.
// Each output element has exactly one writer: deterministic, no atomics.
#include "device_common.hpp"
#include "kernel_params.h"
#include "noise.h"

namespace ft {

constexpr int kColBK = 128;  // keys per workgroup
constexpr int kColBQ = 64;   // query rows per tile
constexpr int kColThreads = 256;

template <int D>
constexpr int colstats_lds_bytes() {
  return 2 * kColBQ * 2 * D + 2 * kColBQ * 8;
}

template <typename T, int D, bool CAUSAL, bool EMU, int MODE>
__global__ void __launch_bounds__(kColThreads, 2) colstats_kernel(const ColstatsKernelParams p) {
  constexpr int BK = kColBK, BQ = kColBQ, NT = kColThreads;
  constexpr int KSTEPS = D / 16;
  typedef TileGeom<D> G;
  typedef typename T::vec8 vec8;
  constexpr int TILE_BYTES = BQ * G::RB;
  constexpr bool KFM = (MODE == kStatKfTensor || MODE == kStatKfSeeded);
  extern __shared__ __align__(16) char smem[];
  char* ldsQ = smem;
  float* ldsLse = reinterpret_cast<float*>(smem + 2 * TILE_BYTES);             // [2][BQ]
  uint32_t* ldsRow = reinterpret_cast<uint32_t*>(smem + 2 * TILE_BYTES) + 2 * BQ;  // [2][BQ] noise row terms

  const int BH = p.B * p.H;
  const int bh = blockIdx.x % BH;
  const int jb = blockIdx.x / BH;  // low key blocks see the most rows under the causal mask: heaviest first
  const int b = bh / p.H, h = bh % p.H;
  const int j0 = jb * BK;
  const int lane = lane_id(), wave = wave_id();
  const int g = lane >> 5, n = lane & 31;
  const int kj = j0 + wave * 32 + n;
  const int kj_c = kj < p.Skv ? kj : p.Skv - 1;
  const float POS_INF = __builtin_inff();

  const uint16_t* kptr = p.k + b * p.sk.b + (int64_t)kj_c * p.sk.s + h * p.sk.h;
  vec8 kf[KSTEPS];
#pragma unroll
  for (int t = 0; t < KSTEPS; ++t) kf[t] = *reinterpret_cast<const vec8*>(kptr + 16 * t + 8 * g);

  const uint16_t* qbase = p.q + b * p.sq.b + h * p.sq.h;
  const float* lse_bh = p.lse + (int64_t)bh * p.Sq;

  // first query row that can see key j0 is j0 - off
  int i_begin = 0;
  if (CAUSAL) i_begin = max(0, j0 - p.off) / BQ * BQ;
  const int ntiles = (p.Sq - i_begin + BQ - 1) / BQ;  // <= 0 when no row sees this block

  NoiseKeys nk = {0, 0};
  uint32_t b_j = 0;
  const float* er_col = nullptr;
  if (MODE == kStatKfSeeded) {
    nk = noise_keys(p.seed, (uint32_t)bh);
    b_j = noise_col(nk, (uint32_t)kj);
  }
  if (MODE == kStatKfTensor) er_col = p.exp_rand + b * p.er_sb + h * p.er_sh + kj_c;

  float sum = 0.f, sumsq = 0.f;
  TileStager<D, BQ, NT, kRowSwizzle> stQ;
  stQ.init(qbase, p.sq.s);

  if (ntiles > 0) {
    stQ.issue(i_begin, min(BQ, p.Sq - i_begin), ldsQ);
    if (threadIdx.x < BQ) {
      const int i = i_begin + threadIdx.x;
      ldsLse[threadIdx.x] = i < p.Sq ? lse_bh[i] : POS_INF;
      if (MODE == kStatKfSeeded) ldsRow[threadIdx.x] = noise_row(nk, (uint32_t)i);
    }
  }

  for (int it = 0; it < ntiles; ++it) {
    const int i0 = i_begin + it * BQ;
    const int buf = it & 1;
    wait_vmem();
    __syncthreads();

    // rows of the next tile: normaliser (and noise row term) fetched now, parked in LDS at the end
    float lse_next = POS_INF;
    const bool has_next = it + 1 < ntiles;
    if (has_next) {
      const int in = i0 + BQ;
      if (threadIdx.x < BQ && in + (int)threadIdx.x < p.Sq) lse_next = lse_bh[in + threadIdx.x];
    }

    float er[2][16];
    if (MODE == kStatKfTensor) {
#pragma unroll
      for (int mbk = 0; mbk < 2; ++mbk)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int i = i0 + 32 * mbk + 8 * (r >> 2) + 4 * g + (r & 3);
          er[mbk][r] = (i < p.Sq) ? er_col[(int64_t)i * p.er_sr] : 1.f;
        }
    }

    if (has_next) {
      const int in = i0 + BQ;
      stQ.issue(in, min(BQ, p.Sq - in), ldsQ + (buf ^ 1) * TILE_BYTES);
    }

    const int wave_key0 = j0 + wave * 32;
    // every row of this tile is above the diagonal for all 32 keys of the wave
    const bool skip = CAUSAL && (wave_key0 > i0 + BQ - 1 + p.off);
    if (!skip) {
      const char* tq = ldsQ + buf * TILE_BYTES;
      float16v s_acc[2];
#pragma unroll
      for (int mbk = 0; mbk < 2; ++mbk)
#pragma unroll
        for (int r = 0; r < 16; ++r) s_acc[mbk][r] = 0.f;
#pragma unroll
      for (int t = 0; t < KSTEPS; ++t) {
#pragma unroll
        for (int mbk = 0; mbk < 2; ++mbk) {
          vec8 qa = read_row_chunk<D, vec8>(tq, mbk * 32 + n, 2 * t + g);
          s_acc[mbk] = T::mfma(qa, kf[t], s_acc[mbk]);
        }
      }

      const bool need_mask = CAUSAL && (wave_key0 + 31 > i0 + p.off);
#pragma unroll
      for (int mbk = 0; mbk < 2; ++mbk)
#pragma unroll
        for (int q4 = 0; q4 < 4; ++q4) {
          const int il0 = 32 * mbk + 8 * q4 + 4 * g;
          const float4v lse4 = *reinterpret_cast<const float4v*>(ldsLse + buf * BQ + il0);
          uint4v row4 = {0, 0, 0, 0};
          if (MODE == kStatKfSeeded) row4 = *reinterpret_cast<const uint4v*>(ldsRow + buf * BQ + il0);
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const int r = 4 * q4 + e;
            float x = s_acc[mbk][r];
            if (EMU) {
              x = T::to_float(T::from_float(x));
              x = T::to_float(T::from_float(x * p.logit_mul));
              x *= kLog2e;
            } else {
              x *= p.logit_mul;
            }
            if (KFM) {
              float log2E;
              if (MODE == kStatKfTensor) {
                log2E = __builtin_amdgcn_logf(er[mbk][r]);
              } else {
                const float u = noise_uniform(row4[e], b_j);
                log2E = __builtin_amdgcn_logf(-kLn2 * __builtin_amdgcn_logf(u));
              }
              x = (x - log2E) * p.inv_tau;
            }
            float pr = __builtin_amdgcn_exp2f(x - lse4[e]);  // rows past Sq carry lse = +inf -> 0
            if (need_mask && kj > i0 + il0 + e + p.off) pr = 0.f;
            sum += pr;
            if (MODE == kStatSumSq) sumsq = __builtin_fmaf(pr, pr, sumsq);
          }
        }
    }

    if (has_next && threadIdx.x < BQ) {
      ldsLse[(buf ^ 1) * BQ + threadIdx.x] = lse_next;
      if (MODE == kStatKfSeeded) ldsRow[(buf ^ 1) * BQ + threadIdx.x] = noise_row(nk, (uint32_t)(i0 + BQ + threadIdx.x));
    }
  }

  sum += xchg32(sum);
  if (MODE == kStatSumSq) sumsq += xchg32(sumsq);
  if (g == 0 && kj < p.Skv) {
    const int64_t idx = (int64_t)bh * p.Skv + kj;
    p.colsum[idx] = sum;
    if (MODE == kStatSumSq) p.colsumsq[idx] = sumsq;
  }
}

// ---------------------------------------------------------------------------------------------------

template <typename T, int D, bool CAUSAL, bool EMU, int MODE>
static hipError_t launch_one(const ColstatsKernelParams& p, hipStream_t stream) {
  auto kern = colstats_kernel<T, D, CAUSAL, EMU, MODE>;
  constexpr int lds = colstats_lds_bytes<D>();
  const int nJB = (p.Skv + kColBK - 1) / kColBK;
  dim3 grid((unsigned)(nJB * p.B * p.H));
  hipLaunchKernelGGL(kern, grid, dim3(kColThreads), lds, stream, p);
  return hipGetLastError();
}

template <typename T, int D>
static hipError_t launch_td(const ColstatsKernelParams& p, bool causal, bool emu, int mode, hipStream_t s) {
#define FT_CASE(C, E, M) \
  if (causal == C && emu == E && mode == M) return launch_one<T, D, C, E, M>(p, s);
#define FT_MODES(C, E) FT_CASE(C, E, kStatSum) FT_CASE(C, E, kStatSumSq) FT_CASE(C, E, kStatKfTensor) FT_CASE(C, E, kStatKfSeeded)
  FT_MODES(true, true) FT_MODES(true, false) FT_MODES(false, true) FT_MODES(false, false)
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
