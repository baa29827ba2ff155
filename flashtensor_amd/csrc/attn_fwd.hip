// Fused softmax attention forward for gfx950 (pass A of every softmax workload).
//
// Replaces the attention core the reference emits as a Triton kernel for cases/kernels/attn.py:18-34
// (and the identical prefix of h2o.py, kf.py, roco.py): O = softmax(QK^T / sqrt(D) + causal mask) V,
// never writing an S x S tensor.  Also emits the per-row log2-domain normaliser (max + log2 sum) that the
// column-statistics pass consumes, and in the KeyFormer modes the normaliser of the Gumbel-perturbed
// softmax of kf.py:36-39 instead.
//
// Mapping.  One workgroup = 128 query rows of one (b, h), 4 waves x 32 rows; keys are streamed in tiles
// of 64 through double-buffered LDS (direct global->LDS loads).  Each wave computes the TRANSPOSED score
// block S^T = K Q^T with v_mfma_f32_32x32x16: a lane then owns one query (column l % 32) and 16 of the
// 32 keys of each block, so the online-softmax row max / row sum are in-lane reductions plus a single
// exchange with lane l ^ 32, and the accumulator registers are already the B operand (keys on the
// contraction axis) of O^T += V^T P^T.  V^T is fed by ds_read_b64_tr_b16 from the row-major V tile.
#include "device_common.hpp"
#include "kernel_params.h"
#include "noise.h"

namespace ft {

constexpr int kAttnBM = 128;
constexpr int kAttnBN = 64;
constexpr int kAttnThreads = 256;

template <int D>
constexpr int attn_lds_bytes() {
  return 4 * kAttnBN * 2 * D + 2 * kAttnBN * 4;
}

template <typename T, int D, bool CAUSAL, bool EMU, int KF>
__global__ void __launch_bounds__(kAttnThreads, 2) attn_fwd_kernel(const AttnKernelParams p) {
  constexpr int BM = kAttnBM, BN = kAttnBN, NT = kAttnThreads;
  constexpr int KSTEPS = D / 16;
  constexpr int DB = D / 32;
  typedef TileGeom<D> G;
  typedef typename T::vec8 vec8;
  constexpr int TILE_BYTES = BN * G::RB;
  extern __shared__ __align__(16) char smem[];
  char* ldsK = smem;
  char* ldsV = smem + 2 * TILE_BYTES;
  uint32_t* ldsCol = reinterpret_cast<uint32_t*>(smem + 4 * TILE_BYTES);  // [2][BN] noise column terms

  const int BH = p.B * p.H;
  const int nMB = (p.Sq + BM - 1) / BM;
  const int bh = blockIdx.x % BH;
  const int mb = nMB - 1 - blockIdx.x / BH;  // heaviest (last) query blocks first under the causal mask
  const int b = bh / p.H, h = bh % p.H;
  const int m0 = mb * BM;
  const int lane = lane_id(), wave = wave_id();
  const int g = lane >> 5, n = lane & 31;
  const int qi = m0 + wave * 32 + n;
  const int qi_c = qi < p.Sq ? qi : p.Sq - 1;
  const float NEG_INF = -__builtin_inff();

  const uint16_t* qptr = p.q + b * p.sq.b + (int64_t)qi_c * p.sq.s + h * p.sq.h;
  vec8 qf[KSTEPS];
#pragma unroll
  for (int t = 0; t < KSTEPS; ++t) qf[t] = *reinterpret_cast<const vec8*>(qptr + 16 * t + 8 * g);

  const uint16_t* kbase = p.k + b * p.sk.b + h * p.sk.h;
  const uint16_t* vbase = p.v + b * p.sv.b + h * p.sv.h;

  int n_end = p.Skv;
  if (CAUSAL) n_end = min(p.Skv, m0 + BM + p.off);
  const int ntiles = (n_end + BN - 1) / BN;

  NoiseKeys nk = {0, 0};
  uint32_t a_i = 0;
  const float* er_row = nullptr;
  if (KF == kKfSeeded) {
    nk = noise_keys(p.seed, (uint32_t)bh);
    a_i = noise_row(nk, (uint32_t)qi);
  }
  if (KF == kKfTensor) er_row = p.exp_rand + b * p.er_sb + h * p.er_sh + (int64_t)qi_c * p.er_sr;

  // prologue: stage tile 0
  stage_tile<D, BN, NT, kRowSwizzle>(kbase, p.sk.s, min(BN, p.Skv), ldsK);
  stage_tile<D, BN, NT, kTrSwizzle>(vbase, p.sv.s, min(BN, p.Skv), ldsV);
  if (KF == kKfSeeded && threadIdx.x < BN) ldsCol[threadIdx.x] = noise_col(nk, (uint32_t)threadIdx.x);

  float16v o_acc[DB];
#pragma unroll
  for (int i = 0; i < DB; ++i)
#pragma unroll
    for (int r = 0; r < 16; ++r) o_acc[i][r] = 0.f;
  float m_run = NEG_INF, l_run = 0.f;
  float m_kf = NEG_INF, l_kf = 0.f;

  for (int it = 0; it < ntiles; ++it) {
    const int n0 = it * BN;
    const int buf = it & 1;
    wait_vmem();
    __syncthreads();  // tile `it` is in LDS; every wave is done with the buffer tile it+1 will overwrite

    // KeyFormer, tensor mode: fetch this lane's slice of the noise tile before the next tile's staging
    // loads are queued, so that waiting for it does not wait for them.
    float er[2][16];
    if (KF == kKfTensor) {
#pragma unroll
      for (int mbk = 0; mbk < 2; ++mbk)
#pragma unroll
        for (int q4 = 0; q4 < 4; ++q4) {
          const int j0 = n0 + 32 * mbk + 8 * q4 + 4 * g;
          if (p.er_vec4 && j0 + 3 < p.Skv) {
            float4v e4 = *reinterpret_cast<const float4v*>(er_row + j0);
#pragma unroll
            for (int e = 0; e < 4; ++e) er[mbk][4 * q4 + e] = e4[e];
          } else {
#pragma unroll
            for (int e = 0; e < 4; ++e) er[mbk][4 * q4 + e] = (j0 + e < p.Skv) ? er_row[j0 + e] : 1.f;
          }
        }
    }

    if (it + 1 < ntiles) {
      const int nn = n0 + BN;
      stage_tile<D, BN, NT, kRowSwizzle>(kbase + (int64_t)nn * p.sk.s, p.sk.s, min(BN, p.Skv - nn),
                                         ldsK + (buf ^ 1) * TILE_BYTES);
      stage_tile<D, BN, NT, kTrSwizzle>(vbase + (int64_t)nn * p.sv.s, p.sv.s, min(BN, p.Skv - nn),
                                        ldsV + (buf ^ 1) * TILE_BYTES);
      if (KF == kKfSeeded && threadIdx.x < BN)
        ldsCol[(buf ^ 1) * BN + threadIdx.x] = noise_col(nk, (uint32_t)(nn + threadIdx.x));
    }

    // the whole tile lies above the diagonal for this wave's 32 rows: nothing to add
    const int wave_row0 = m0 + wave * 32;
    if (CAUSAL && n0 > wave_row0 + 31 + p.off) continue;

    const char* tk = ldsK + buf * TILE_BYTES;
    const char* tv = ldsV + buf * TILE_BYTES;

    // ---- S^T = K Q^T : [64 keys] x [32 queries] as two 32x32 blocks
    float16v s_acc[2];
#pragma unroll
    for (int mbk = 0; mbk < 2; ++mbk)
#pragma unroll
      for (int r = 0; r < 16; ++r) s_acc[mbk][r] = 0.f;
#pragma unroll
    for (int t = 0; t < KSTEPS; ++t) {
#pragma unroll
      for (int mbk = 0; mbk < 2; ++mbk) {
        vec8 ka = read_row_chunk<D, vec8>(tk, mbk * 32 + n, 2 * t + g);
        s_acc[mbk] = T::mfma(ka, qf[t], s_acc[mbk]);
      }
    }

    // ---- logits in the log2 domain, with the reference's rounding points when EMU
    const bool need_mask = (CAUSAL && (n0 + BN - 1 > wave_row0 + p.off)) || (n0 + BN > p.Skv);
    float rowmax = NEG_INF;
#pragma unroll
    for (int mbk = 0; mbk < 2; ++mbk)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        float x = s_acc[mbk][r];
        if (EMU) {
          x = T::to_float(T::from_float(x));                // QK^T is an fp16 tensor in the reference
          x = T::to_float(T::from_float(x * p.logit_mul));  // ... divided by sqrt(D) in fp16
          x *= kLog2e;
        } else {
          x *= p.logit_mul;
        }
        if (need_mask) {
          const int j = n0 + 32 * mbk + 8 * (r >> 2) + 4 * g + (r & 3);
          if ((CAUSAL && j > qi + p.off) || j >= p.Skv) x = NEG_INF;
        }
        s_acc[mbk][r] = x;
        rowmax = fmaxf(rowmax, x);
      }
    rowmax = fmaxf(rowmax, xchg32(rowmax));

    // ---- KeyFormer: running normaliser of softmax((logit + gumbel) / tau), gumbel = -ln(E)
    if (KF != kKfNone) {
      float z[2][16];
      float zmax = NEG_INF;
#pragma unroll
      for (int mbk = 0; mbk < 2; ++mbk)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          float log2E;
          if (KF == kKfTensor) {
            log2E = __builtin_amdgcn_logf(er[mbk][r]);
          } else {
            const int jl = 32 * mbk + 8 * (r >> 2) + 4 * g + (r & 3);
            const float u = noise_uniform(a_i, ldsCol[buf * BN + jl]);
            log2E = __builtin_amdgcn_logf(-kLn2 * __builtin_amdgcn_logf(u));
          }
          const float zz = (s_acc[mbk][r] - log2E) * p.inv_tau;
          z[mbk][r] = zz;
          zmax = fmaxf(zmax, zz);
        }
      zmax = fmaxf(zmax, xchg32(zmax));
      const float mk_new = fmaxf(m_kf, zmax);
      float zs = 0.f;
#pragma unroll
      for (int mbk = 0; mbk < 2; ++mbk)
#pragma unroll
        for (int r = 0; r < 16; ++r) zs += __builtin_amdgcn_exp2f(z[mbk][r] - mk_new);
      l_kf = l_kf * __builtin_amdgcn_exp2f(m_kf - mk_new) + zs;
      m_kf = mk_new;
    }

    // ---- online softmax
    const float m_new = fmaxf(m_run, rowmax);
    const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);
    m_run = m_new;
    float psum = 0.f;
    vec8 pb[4];
#pragma unroll
    for (int mbk = 0; mbk < 2; ++mbk)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const float pv = __builtin_amdgcn_exp2f(s_acc[mbk][r] - m_new);
        psum += pv;
        pb[2 * mbk + (r >> 3)][r & 7] = T::to_elem(T::from_float(pv));
      }
    l_run = l_run * alpha + psum;
#pragma unroll
    for (int i = 0; i < DB; ++i)
#pragma unroll
      for (int r = 0; r < 16; ++r) o_acc[i][r] *= alpha;

    // ---- O^T += V^T P^T
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {
#pragma unroll
      for (int db = 0; db < DB; ++db) {
        vec8 va = read_tr_operand<D, vec8>(tv, 16 * ks, 32 * db);
        o_acc[db] = T::mfma(va, pb[ks], o_acc[db]);
      }
    }
  }

  // ---- epilogue
  l_run += xchg32(l_run);
  const float inv_l = 1.f / l_run;
  if (qi < p.Sq) {
    uint16_t* optr = p.o + b * p.so.b + (int64_t)qi * p.so.s + h * p.so.h;
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int q4 = 0; q4 < 4; ++q4) {
        const int d = 32 * db + 8 * q4 + 4 * g;
        uint16_t w[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) w[e] = T::from_float(o_acc[db][4 * q4 + e] * inv_l);
        uint2 pk;
        pk.x = (uint32_t)w[0] | ((uint32_t)w[1] << 16);
        pk.y = (uint32_t)w[2] | ((uint32_t)w[3] << 16);
        *reinterpret_cast<uint2*>(optr + d) = pk;
      }
    if (g == 0 && p.lse) p.lse[(int64_t)bh * p.Sq + qi] = m_run + __builtin_amdgcn_logf(l_run);
  }
  if (KF != kKfNone) {
    l_kf += xchg32(l_kf);
    if (qi < p.Sq && g == 0) p.lse_kf[(int64_t)bh * p.Sq + qi] = m_kf + __builtin_amdgcn_logf(l_kf);
  }
}

// ---------------------------------------------------------------------------------------------------
// host-side launcher

template <typename T, int D, bool CAUSAL, bool EMU, int KF>
static hipError_t launch_one(const AttnKernelParams& p, hipStream_t stream) {
  auto kern = attn_fwd_kernel<T, D, CAUSAL, EMU, KF>;
  constexpr int lds = attn_lds_bytes<D>();
  static bool configured = false;  // benign race: the attribute call is idempotent
  if (!configured) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, lds);
    if (e != hipSuccess) return e;
    configured = true;
  }
  const int nMB = (p.Sq + kAttnBM - 1) / kAttnBM;
  dim3 grid((unsigned)(nMB * p.B * p.H));
  hipLaunchKernelGGL(kern, grid, dim3(kAttnThreads), lds, stream, p);
  return hipGetLastError();
}

template <typename T, int D>
static hipError_t launch_td(const AttnKernelParams& p, bool causal, bool emu, int kf, hipStream_t s) {
#define FT_CASE(C, E, K) \
  if (causal == C && emu == E && kf == K) return launch_one<T, D, C, E, K>(p, s);
  FT_CASE(true, true, kKfNone) FT_CASE(true, false, kKfNone) FT_CASE(false, true, kKfNone) FT_CASE(false, false, kKfNone)
  FT_CASE(true, true, kKfTensor) FT_CASE(true, false, kKfTensor) FT_CASE(false, true, kKfTensor) FT_CASE(false, false, kKfTensor)
  FT_CASE(true, true, kKfSeeded) FT_CASE(true, false, kKfSeeded) FT_CASE(false, true, kKfSeeded) FT_CASE(false, false, kKfSeeded)
#undef FT_CASE
  return hipErrorInvalidValue;
}

hipError_t launch_attn_fwd(const AttnKernelParams& p, int D, bool bf16, bool causal, bool emu, int kf, hipStream_t s) {
  if (D == 128) return bf16 ? launch_td<BF16, 128>(p, causal, emu, kf, s) : launch_td<F16, 128>(p, causal, emu, kf, s);
  if (D == 64) return bf16 ? launch_td<BF16, 64>(p, causal, emu, kf, s) : launch_td<F16, 64>(p, causal, emu, kf, s);
  return hipErrorInvalidValue;
}

}  // namespace ft
