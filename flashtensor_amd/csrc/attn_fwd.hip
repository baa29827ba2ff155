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

#include <type_traits>

namespace ft {

constexpr int kAttnBM = 128;
constexpr int kAttnBN = 64;
constexpr int kAttnThreads = 256;

// Rescale threshold of the running maximum in log2 units: the stale maximum is kept (and O, l are not
// rescaled) while the new row maximum exceeds it by less than this, so unnormalised probabilities stay
// below 2^kRescaleSlack (exact in fp16/fp32; the final division uses the same maximum).
constexpr float kRescaleSlack = 6.f;

enum TileMode { kTileFast = 0, kTileMasked = 1, kTileIdle = 2 };

template <typename T, int D, bool CAUSAL, bool EMU, int KF>
__global__ void __launch_bounds__(kAttnThreads, 2) attn_fwd_kernel(const AttnKernelParams p) {
  constexpr int BM = kAttnBM, BN = kAttnBN, NT = kAttnThreads;
  constexpr int KSTEPS = D / 16;
  constexpr int DB = D / 32;
  typedef TileGeom<D> G;
  typedef typename T::vec8 vec8;
  constexpr int TILE_BYTES = BN * G::RB;
  constexpr bool kIsF16 = __is_same(typename T::elem, _Float16);
  // Software pipeline across tiles: the QK^T MFMAs of tile it+1 are issued in the same iteration as the
  // softmax (VALU) and PV MFMAs of tile it, so the matrix and vector pipes overlap inside one wave.
  // K therefore runs one tile ahead of V in LDS.
  // One LDS object per buffer: the compiler tracks outstanding direct-to-LDS loads per object, so reads
  // of one buffer do not wait for the loads in flight into the others.
  __shared__ __align__(16) char ldsK0[TILE_BYTES];
  __shared__ __align__(16) char ldsK1[TILE_BYTES];
  __shared__ __align__(16) char ldsV0[TILE_BYTES];
  __shared__ __align__(16) char ldsV1[TILE_BYTES];
  __shared__ uint32_t ldsCol[2 * BN];  // noise column terms of the current / next tile

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

  // tiles of the workgroup, of this wave (not entirely above its diagonal), and of this wave's mask-free prefix
  const int wave_row0 = m0 + wave * 32;
  int n_end = p.Skv;
  if (CAUSAL) n_end = min(p.Skv, m0 + BM + p.off);
  const int ntiles = (n_end + BN - 1) / BN;
  int nw = ntiles, n_fast = p.Skv / BN;
  if (CAUSAL) {
    nw = min(ntiles, (wave_row0 + 31 + p.off) / BN + 1);
    n_fast = min(n_fast, (wave_row0 + p.off + 1) / BN);  // tiles with n0 + BN - 1 <= wave_row0 + off
  }
  if (KF != kKfNone || !(kIsF16 && EMU)) n_fast = 0;  // only the fp16 reference-rounding path has a mask-free instance
  n_fast = min(n_fast, nw);

  NoiseKeys nk = {0, 0};
  uint32_t a_i = 0;
  const float* er_row = nullptr;
  if (KF == kKfSeeded) {
    nk = noise_keys(p.seed, (uint32_t)bh);
    a_i = noise_row(nk, (uint32_t)qi);
  }
  if (KF == kKfTensor) er_row = p.exp_rand + b * p.er_sb + h * p.er_sh + (int64_t)qi_c * p.er_sr;

  TileStager<D, BN, NT, kRowSwizzle> stK;
  TileStager<D, BN, NT, kTrSwizzle> stV;
  stK.init(p.sk.s);
  stV.init(p.sv.s);
  auto stage_k = [&](int t, char* dst) {
    if (t < ntiles) stK.issue(kbase + (int64_t)t * BN * p.sk.s, p.sk.s, min(BN, p.Skv - t * BN), dst);
  };
  auto stage_v = [&](int t, char* dst) {
    if (t < ntiles) stV.issue(vbase + (int64_t)t * BN * p.sv.s, p.sv.s, min(BN, p.Skv - t * BN), dst);
    if (KF == kKfSeeded && t < ntiles && threadIdx.x < BN)
      ldsCol[(t & 1) * BN + threadIdx.x] = noise_col(nk, (uint32_t)(t * BN + threadIdx.x));
  };

  float16v o_acc[DB];
#pragma unroll
  for (int i = 0; i < DB; ++i)
#pragma unroll
    for (int r = 0; r < 16; ++r) o_acc[i][r] = 0.f;
  float m_run = NEG_INF, l_run = 0.f;  // running max (log2 domain) and this lane's share of the row sum
  float m_kf = NEG_INF, l_kf = 0.f;
  float16v S0[2], S1[2];  // score accumulators of the current / next tile (they swap every tile)

  // ---- S^T = K Q^T : [64 keys] x [32 queries] as two 32x32 blocks, operand reads one step ahead
  auto qk = [&](float16v (&s)[2], const char* tk) {
#pragma unroll
    for (int mbk = 0; mbk < 2; ++mbk)
#pragma unroll
      for (int r = 0; r < 16; ++r) s[mbk][r] = 0.f;
    vec8 ka[2][2];
#pragma unroll
    for (int mbk = 0; mbk < 2; ++mbk) ka[0][mbk] = read_row_chunk<D, vec8>(tk, mbk * 32 + n, g);
#pragma unroll
    for (int t = 0; t < KSTEPS; ++t) {
      if (t + 1 < KSTEPS) {
#pragma unroll
        for (int mbk = 0; mbk < 2; ++mbk) ka[(t + 1) & 1][mbk] = read_row_chunk<D, vec8>(tk, mbk * 32 + n, 2 * (t + 1) + g);
      }
#pragma unroll
      for (int mbk = 0; mbk < 2; ++mbk) s[mbk] = T::mfma(ka[t & 1][mbk], qf[t], s[mbk]);
    }
  };

  auto rescale = [&](float rowmax) {
    const bool grow = rowmax > m_run + kRescaleSlack;  // identical in both lanes of a row
    if (__any(grow)) {
      const float m_new = grow ? rowmax : m_run;
      const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);
      m_run = m_new;
      l_run *= alpha;
#pragma unroll
      for (int i = 0; i < DB; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) o_acc[i][r] *= alpha;
    }
  };

  // ---- softmax of one tile: s (raw accumulators) -> pb (16-bit unnormalised probabilities)
  auto softmax = [&](auto masked_tag, float16v (&s)[2], vec8 (&pb)[4], int n0, int buf, const float (&er)[2][16]) {
    constexpr bool MASKED = decltype(masked_tag)::value;
    if constexpr (kIsF16 && EMU && !MASKED && KF == kKfNone) {
      // Fast path.  Rounding is monotonic, so the row maximum of the rounded logits is the rounded
      // maximum of the raw accumulators.
      float amax = max3(s[0][0], s[0][1], s[1][0]);
#pragma unroll
      for (int mbk = 0; mbk < 2; ++mbk)
#pragma unroll
        for (int r = 0; r < 16; r += 2) amax = max3(amax, s[mbk][r], s[mbk][r + 1]);
      amax = fmaxf(amax, xchg32(amax));
      rescale((float)(_Float16)((float)(_Float16)amax * p.logit_mul) * kLog2e);
      const float neg_m = -m_run;
      const half2v ones = {(_Float16)1.f, (_Float16)1.f};
      uint4v pw[4];
#pragma unroll
      for (int mbk = 0; mbk < 2; ++mbk)
#pragma unroll
        for (int r = 0; r < 16; r += 2) {
          const float2v a2 = {s[mbk][r], s[mbk][r + 1]};
          const half2v h2 = __builtin_convertvector(a2, half2v);       // QK^T is an fp16 tensor in the reference
          const _Float16 t0 = (_Float16)((float)h2[0] * p.logit_mul);  // ... divided by sqrt(D) in fp16
          const _Float16 t1 = (_Float16)((float)h2[1] * p.logit_mul);
          const float p0 = __builtin_amdgcn_exp2f(__builtin_fmaf((float)t0, kLog2e, neg_m));
          const float p1 = __builtin_amdgcn_exp2f(__builtin_fmaf((float)t1, kLog2e, neg_m));
          const float2v p2 = {p0, p1};
          const half2v ph = __builtin_convertvector(p2, half2v);
          l_run = __builtin_amdgcn_fdot2(ph, ones, l_run, false);  // row sum of the fp16 P the MFMA consumes
          pw[2 * mbk + (r >> 3)][(r & 7) >> 1] = __builtin_bit_cast(uint32_t, ph);  // whole 32-bit words: no 16-bit shuffles
        }
#pragma unroll
      for (int i = 0; i < 4; ++i) pb[i] = __builtin_bit_cast(vec8, pw[i]);
    } else {
      // ---- logits in the log2 domain, with the reference's rounding points when EMU
      float rowmax = NEG_INF;
#pragma unroll
      for (int mbk = 0; mbk < 2; ++mbk)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          float x = s[mbk][r];
          if (EMU) {
            x = T::to_float(T::from_float(x));
            x = T::to_float(T::from_float(x * p.logit_mul));
            x *= kLog2e;
          } else {
            x *= p.logit_mul;
          }
          if (MASKED) {
            const int j = n0 + 32 * mbk + 8 * (r >> 2) + 4 * g + (r & 3);
            if ((CAUSAL && j > qi + p.off) || j >= p.Skv) x = NEG_INF;
          }
          s[mbk][r] = x;
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
            const float zz = (s[mbk][r] - log2E) * p.inv_tau;
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

      rescale(rowmax);
      uint4v pw[4];
#pragma unroll
      for (int mbk = 0; mbk < 2; ++mbk)
#pragma unroll
        for (int r = 0; r < 16; r += 2) {
          const uint16_t b0 = T::from_float(__builtin_amdgcn_exp2f(s[mbk][r] - m_run));
          const uint16_t b1 = T::from_float(__builtin_amdgcn_exp2f(s[mbk][r + 1] - m_run));
          l_run += T::to_float(b0) + T::to_float(b1);
          pw[2 * mbk + (r >> 3)][(r & 7) >> 1] = (uint32_t)b0 | ((uint32_t)b1 << 16);
        }
#pragma unroll
      for (int i = 0; i < 4; ++i) pb[i] = __builtin_bit_cast(vec8, pw[i]);
    }
  };

  // ---- O^T += V^T P^T (operand reads one step ahead of the MFMAs)
  auto pv = [&](const vec8 (&pb)[4], const char* tv) {
    vec8 va[2][DB];
#pragma unroll
    for (int db = 0; db < DB; ++db) va[0][db] = read_tr_operand<D, vec8>(tv, 0, 32 * db);
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {
      if (ks + 1 < 4) {
#pragma unroll
        for (int db = 0; db < DB; ++db) va[(ks + 1) & 1][db] = read_tr_operand<D, vec8>(tv, 16 * (ks + 1), 32 * db);
      }
#pragma unroll
      for (int db = 0; db < DB; ++db) o_acc[db] = T::mfma(va[ks & 1][db], pb[ks], o_acc[db]);
    }
  };

  // One iteration = one barrier.  On entry K[it+1] and V[it] have been requested; K[it+2] and V[it+1] are
  // requested here, into the buffers every wave has finished reading.
  float er[2][16];
  auto sync_and_stage = [&](int it, bool active, char* k_dst, char* v_dst) {
    wait_vmem();
    __syncthreads();
    // KeyFormer, tensor mode: fetch this lane's slice of the noise tile before the next tiles' staging
    // loads are queued, so that waiting for it does not wait for them.
    if (KF == kKfTensor && active) {
      const int n0 = it * BN;
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
    stage_k(it + 2, k_dst);
    stage_v(it + 1, v_dst);
  };

  // ---- prologue: K[0], V[0], K[1] in flight; scores of tile 0
  stage_k(0, ldsK0);
  stage_v(0, ldsV0);
  stage_k(1, ldsK1);
  wait_vmem();
  __syncthreads();
  qk(S0, ldsK0);

  int it = 0;
  // ---- mask-free tiles, two per trip so that the two score buffers swap roles without copies
  const int nf2 = n_fast & ~1;
  for (; it < nf2; it += 2) {
    vec8 pb[4];
    sync_and_stage(it, true, ldsK0, ldsV1);      // K[it+2], V[it+1]
    qk(S1, ldsK1);                               // tile it+1
    softmax(std::false_type{}, S0, pb, it * BN, 0, er);
    pv(pb, ldsV0);
    sync_and_stage(it + 1, true, ldsK1, ldsV0);  // K[it+3], V[it+2]
    qk(S0, ldsK0);  // tile it+2; past the last tile this reads stale LDS and is discarded
    softmax(std::false_type{}, S1, pb, (it + 1) * BN, 1, er);
    pv(pb, ldsV1);
  }
  // ---- tiles that straddle the diagonal or the end of K (and every tile of the KeyFormer variants)
  for (; it < nw; ++it) {
    vec8 pb[4];
    const bool odd = it & 1;
    sync_and_stage(it, true, odd ? ldsK1 : ldsK0, odd ? ldsV0 : ldsV1);
    softmax(std::true_type{}, S0, pb, it * BN, it & 1, er);
    pv(pb, odd ? ldsV1 : ldsV0);
    qk(S0, odd ? ldsK0 : ldsK1);
  }
  // ---- tiles entirely above this wave's diagonal: keep the workgroup's barriers and staging in step
  for (; it < ntiles; ++it) sync_and_stage(it, false, (it & 1) ? ldsK1 : ldsK0, (it & 1) ? ldsV0 : ldsV1);

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
  const int nMB = (p.Sq + kAttnBM - 1) / kAttnBM;
  dim3 grid((unsigned)(nMB * p.B * p.H));
  hipLaunchKernelGGL(kern, grid, dim3(kAttnThreads), 0, stream, p);
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
