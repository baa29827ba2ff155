// Linear-attention cores EA and SimA for gfx950, head_dim 64, fp16.
//
// Replaces the fused kernels the reference would emit for bench/ea.mlir:13-17 and bench/sima.mlir:13-17
// (asuka.softmax / asuka.normalize semantics: lib/Dialect/Asuka/Transforms/LowerComplexReduce.cpp:21-69):
//   EA  : O = softmax(Q, dim=D) . (softmax(K, dim=S)^T V)
//   SimA: O = (Q / sum_s|Q|) . ((K / sum_s|K|)^T V)          (per (b, h, channel) L1 norms over S)
// Both are HBM-bound (32 FLOP/byte): the design reads K and V once, Q twice (once for SimA's norm, once
// for the output product; EA reads it once) and writes O once.
//
// Three launches:
//   1. kv_partial: a workgroup streams a chunk of tokens of one (b, h) in 128-token tiles through
//      double-buffered LDS and accumulates the 64x64 matrix sum_s f(K[s,d]) V[s,e] with MFMA (both operands
//      have the contraction axis = tokens strided in memory, so both come from ds_read_b64_tr_b16), plus
//      the per-channel normalisers: EA an online (max, sum of exp) pair, SimA sum|K| and sum|Q|.
//   2. merge: combines the chunks of one (b, h), folds every normaliser into the 64x64 matrix (the deferred
//      division the reference's EquivalentTransform pass performs, EquivalentTransform.cpp:303-341) and
//      stores it transposed as an fp16 hi/lo pair with a power-of-two scale, so that SimA's tiny values
//      (~1e-6) neither underflow nor lose precision in fp16.
//   3. out: O^T = W^T f(Q)^T per 32-token wave tile, with EA's per-token softmax over the 64 channels done
//      in registers (a lane owns half a token row; one exchange with lane l ^ 32).
#include "device_common.hpp"
#include "kernel_params.h"
#include "../../include/ft_abi.h"

namespace ft {

constexpr int kLinD = 64;
constexpr int kLinTile = 128;     // tokens per staged tile
constexpr int kLinThreads = 256;
constexpr int kPartStride = kLinD * kLinD + 2 * kLinD;  // floats per (bh, chunk) partial

struct LinParams {
  const uint16_t* q;
  const uint16_t* k;
  const uint16_t* v;
  void* o;
  Strides3 sq, sk, sv, so;
  float* part;      // [BH][nch][kPartStride]
  uint16_t* w;      // [BH][2][64 e][64 d] fp16: hi, lo * 2^11
  float* winv;      // [BH] 1 / scale
  int B, H, S;
  int nch;              // chunks per (b, h)
  int tiles_per_chunk;  // 128-token tiles per chunk
  int normalize_q;
  int out_f32;
};

static void lin_plan(const FtAttnArgs& a, int* nch, int* tpc) {
  const int ntiles = (a.Sq + kLinTile - 1) / kLinTile;
  const int64_t bh = (int64_t)a.B * a.H;
  int want = (int)((1024 + bh - 1) / bh);  // aim for >= ~1024 workgroups
  if (want < 1) want = 1;
  int t = (ntiles + want - 1) / want;
  if (t < 1) t = 1;
  if (t > 16) t = 16;
  *tpc = t;
  *nch = (ntiles + t - 1) / t;
}

size_t linattn_workspace_bytes(const FtAttnArgs& a, int) {
  int nch, tpc;
  lin_plan(a, &nch, &tpc);
  const size_t bh = (size_t)a.B * a.H;
  size_t bytes = bh * nch * kPartStride * sizeof(float);
  bytes += bh * 2 * kLinD * kLinD * sizeof(uint16_t);
  bytes += bh * sizeof(float);
  return (bytes + 255) & ~(size_t)255;
}

// ---------------------------------------------------------------------------------------------------
template <bool EA>
__global__ void __launch_bounds__(kLinThreads, 2) linattn_kv_kernel(const LinParams p) {
  constexpr int D = kLinD, NT = kLinThreads, TILE = kLinTile;
  typedef TileGeom<D> G;
  constexpr int TILE_BYTES = TILE * G::RB;  // 16 KB
  extern __shared__ __align__(16) char smem[];
  char* ldsK = smem;
  char* ldsV = smem + 2 * TILE_BYTES;
  float* ldsScratch = reinterpret_cast<float*>(smem + 4 * TILE_BYTES);  // [4 waves][32]

  const int BH = p.B * p.H;
  const int bh = blockIdx.x % BH;
  const int ch = blockIdx.x / BH;
  const int b = bh / p.H, h = bh % p.H;
  const int lane = lane_id(), wave = wave_id();
  const int g = lane >> 5, n = lane & 31;
  const int dblock = wave >> 1, eblock = wave & 1;
  const float NEG_INF = -__builtin_inff();

  const uint16_t* kbase = p.k + b * p.sk.b + h * p.sk.h;
  const uint16_t* vbase = p.v + b * p.sv.b + h * p.sv.h;
  const uint16_t* qbase = p.q + b * p.sq.b + h * p.sq.h;

  const int tok_begin = ch * p.tiles_per_chunk * TILE;
  const int tok_end = min(p.S, tok_begin + p.tiles_per_chunk * TILE);
  const int ntiles = (tok_end - tok_begin + TILE - 1) / TILE;

  float16v acc;
#pragma unroll
  for (int r = 0; r < 16; ++r) acc[r] = 0.f;
  float m_run = NEG_INF;  // EA: running max of K[:, d] for this lane's channel d = 32 dblock + n
  float l_run = 0.f;      // EA: sum of exp; SimA: sum |K|   (partial: this lane's token slots only)
  float qabs[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) qabs[e] = 0.f;

  TileStager<D, TILE, NT, kTrSwizzle> stK, stV;
  stK.init(kbase, p.sk.s);
  stV.init(vbase, p.sv.s);
  stK.issue(tok_begin, min(TILE, p.S - tok_begin), ldsK);
  stV.issue(tok_begin, min(TILE, p.S - tok_begin), ldsV);

  for (int it = 0; it < ntiles; ++it) {
    const int t0 = tok_begin + it * TILE;
    const int buf = it & 1;
    wait_vmem();
    __syncthreads();

    // SimA: |Q| partial sums straight from global memory (Q is not needed in LDS here)
    if (!EA && p.normalize_q) {
      const int c = threadIdx.x & 7;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int tok = t0 + (threadIdx.x >> 3) + 32 * i;
        if (tok < p.S) {
          half8 qv = *reinterpret_cast<const half8*>(qbase + (int64_t)tok * p.sq.s + c * 8);
#pragma unroll
          for (int e = 0; e < 8; ++e) qabs[e] += __builtin_fabsf((float)qv[e]);
        }
      }
    }

    if (it + 1 < ntiles) {
      const int tn = t0 + TILE;
      stK.issue(tn, min(TILE, p.S - tn), ldsK + (buf ^ 1) * TILE_BYTES);
      stV.issue(tn, min(TILE, p.S - tn), ldsV + (buf ^ 1) * TILE_BYTES);
    }

    const char* tk = ldsK + buf * TILE_BYTES;
    const char* tv = ldsV + buf * TILE_BYTES;
    const bool tail = t0 + TILE > p.S;

    half8 ka[TILE / 16];
#pragma unroll
    for (int ks = 0; ks < TILE / 16; ++ks) ka[ks] = read_tr_operand<D, half8>(tk, 16 * ks, 32 * dblock);

    if (EA) {
      float tmax = NEG_INF;
#pragma unroll
      for (int ks = 0; ks < TILE / 16; ++ks)
#pragma unroll
        for (int s = 0; s < 8; ++s) {
          const int tok = t0 + 16 * ks + 4 * g + (s & 3) + ((s >> 2) << 3);
          const float x = (float)ka[ks][s];
          tmax = fmaxf(tmax, (tail && tok >= p.S) ? NEG_INF : x);
        }
      tmax = fmaxf(tmax, xchg32(tmax));
      const float m_new = fmaxf(m_run, tmax);
      if (__any(m_new > m_run)) {
        const float f = __builtin_amdgcn_exp2f((m_run - m_new) * kLog2e);
        l_run *= f;
        // move the per-channel factor from "lane = channel" to the accumulator's "register = channel"
        float* sc = ldsScratch + wave * 32;
        if (g == 0) sc[n] = f;
#pragma unroll
        for (int q4 = 0; q4 < 4; ++q4) {
          const float4v f4 = *reinterpret_cast<const float4v*>(sc + 8 * q4 + 4 * g);
#pragma unroll
          for (int e = 0; e < 4; ++e) acc[4 * q4 + e] *= f4[e];
        }
      }
      m_run = m_new;
      const float mb = m_new * kLog2e;
#pragma unroll
      for (int ks = 0; ks < TILE / 16; ++ks)
#pragma unroll
        for (int s = 0; s < 8; ++s) {
          const int tok = t0 + 16 * ks + 4 * g + (s & 3) + ((s >> 2) << 3);
          float pe = __builtin_amdgcn_exp2f(__builtin_fmaf((float)ka[ks][s], kLog2e, -mb));
          if (tail && tok >= p.S) pe = 0.f;
          const _Float16 ph = (_Float16)pe;
          ka[ks][s] = ph;
          l_run += (float)ph;
        }
    } else {
#pragma unroll
      for (int ks = 0; ks < TILE / 16; ++ks)
#pragma unroll
        for (int s = 0; s < 8; ++s) {
          const int tok = t0 + 16 * ks + 4 * g + (s & 3) + ((s >> 2) << 3);
          if (tail && tok >= p.S) ka[ks][s] = (_Float16)0.f;
          l_run += __builtin_fabsf((float)ka[ks][s]);
        }
    }

#pragma unroll
    for (int ks = 0; ks < TILE / 16; ++ks) {
      half8 vb = read_tr_operand<D, half8>(tv, 16 * ks, 32 * eblock);
      acc = F16::mfma(ka[ks], vb, acc);
    }
  }

  // ---- write the partial
  float* part = p.part + ((int64_t)bh * p.nch + ch) * kPartStride;
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    const int d = 32 * dblock + 8 * (r >> 2) + 4 * g + (r & 3);
    part[d * D + 32 * eblock + n] = acc[r];
  }
  l_run += xchg32(l_run);
  if (eblock == 0 && g == 0) {
    const int d = 32 * dblock + n;
    part[D * D + d] = EA ? m_run : l_run;
    if (EA) part[D * D + D + d] = l_run;
  }
  if (!EA) {
    __syncthreads();  // tiles are dead: reuse LDS for the |Q| reduction
    float* red = reinterpret_cast<float*>(smem);  // [32 row groups][64 channels]
    const int c = threadIdx.x & 7, rg = threadIdx.x >> 3;
#pragma unroll
    for (int e = 0; e < 8; ++e) red[rg * D + c * 8 + e] = qabs[e];
    __syncthreads();
    if (threadIdx.x < D) {
      float s = 0.f;
      for (int i = 0; i < 32; ++i) s += red[i * D + threadIdx.x];
      part[D * D + D + threadIdx.x] = s;
    }
  }
}

// ---------------------------------------------------------------------------------------------------
template <bool EA>
__global__ void __launch_bounds__(kLinThreads) linattn_merge_kernel(const LinParams p) {
  constexpr int D = kLinD;
  __shared__ float s_scale[D];   // per-channel factor applied to the summed matrix
  __shared__ float s_w[16][D];   // EA: per-chunk weights exp(m_c - M), up to 16 chunks at a time
  __shared__ float s_red[kLinThreads];
  const int bh = blockIdx.x;
  const float* part = p.part + (int64_t)bh * p.nch * kPartStride;
  const int t = threadIdx.x;

  float accv[16];
#pragma unroll
  for (int i = 0; i < 16; ++i) accv[i] = 0.f;
  float gmax = -__builtin_inff();

  if (EA) {
    if (t < D) {
      float M = -__builtin_inff();
      for (int c = 0; c < p.nch; ++c) M = fmaxf(M, part[c * kPartStride + D * D + t]);
      float L = 0.f;
      for (int c = 0; c < p.nch; ++c)
        L += __builtin_amdgcn_exp2f((part[c * kPartStride + D * D + t] - M) * kLog2e) * part[c * kPartStride + D * D + D + t];
      s_scale[t] = 1.f / L;
      s_red[t] = M;
    }
    __syncthreads();
    for (int c0 = 0; c0 < p.nch; c0 += 16) {
      const int cn = min(16, p.nch - c0);
      for (int i = t; i < cn * D; i += kLinThreads) {
        const int c = i / D, d = i % D;
        s_w[c][d] = __builtin_amdgcn_exp2f((part[(c0 + c) * kPartStride + D * D + d] - s_red[d]) * kLog2e);
      }
      __syncthreads();
      for (int c = 0; c < cn; ++c)
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          const int idx = t + i * kLinThreads;  // d = idx / 64, e = idx % 64
          accv[i] += s_w[c][idx / D] * part[(c0 + c) * kPartStride + idx];
        }
      __syncthreads();
    }
  } else {
    if (t < D) {
      float nk = 0.f, nq = 0.f;
      for (int c = 0; c < p.nch; ++c) {
        nk += part[c * kPartStride + D * D + t];
        nq += part[c * kPartStride + D * D + D + t];
      }
      s_scale[t] = 1.f / (p.normalize_q ? nk * nq : nk);
    }
    __syncthreads();
    for (int c = 0; c < p.nch; ++c)
#pragma unroll
      for (int i = 0; i < 16; ++i) accv[i] += part[c * kPartStride + t + i * kLinThreads];
  }
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    accv[i] *= s_scale[(t + i * kLinThreads) / D];
    gmax = fmaxf(gmax, __builtin_fabsf(accv[i]));
  }
  __syncthreads();
  s_red[t] = gmax;
  __syncthreads();
  for (int s = kLinThreads / 2; s > 0; s >>= 1) {
    if (t < s) s_red[t] = fmaxf(s_red[t], s_red[t + s]);
    __syncthreads();
  }
  gmax = s_red[0];
  // power-of-two scale that puts the largest entry in [2^13, 2^14)
  int ex = 0;
  if (gmax > 0.f && gmax < __builtin_inff()) ex = 13 - (int)__builtin_floorf(__builtin_log2f(gmax));
  ex = max(-100, min(100, ex));
  const float scale = __builtin_ldexpf(1.f, ex);
  if (t == 0) p.winv[bh] = __builtin_ldexpf(1.f, -ex);
  uint16_t* w = p.w + (int64_t)bh * 2 * D * D;
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const int idx = t + i * kLinThreads;
    const int d = idx / D, e = idx % D;
    const float x = accv[i] * scale;
    const _Float16 hi = (_Float16)x;
    const _Float16 lo = (_Float16)((x - (float)hi) * 2048.f);
    w[e * D + d] = __builtin_bit_cast(uint16_t, hi);
    w[D * D + e * D + d] = __builtin_bit_cast(uint16_t, lo);
  }
}

// ---------------------------------------------------------------------------------------------------
template <bool EA, bool F32OUT>
__global__ void __launch_bounds__(kLinThreads, 2) linattn_out_kernel(const LinParams p) {
  constexpr int D = kLinD;
  const int BH = p.B * p.H;
  const int bh = blockIdx.x % BH;
  const int tb = blockIdx.x / BH;
  const int b = bh / p.H, h = bh % p.H;
  const int lane = lane_id(), wave = wave_id();
  const int g = lane >> 5, n = lane & 31;
  const int tok = tb * 128 + wave * 32 + n;
  const int tok_c = tok < p.S ? tok : p.S - 1;

  // A operand: W^T[e][d], hi and lo, rows e = 32 eb + n, contraction slots d = 16 t + 8 g + [0..7]
  const uint16_t* w = p.w + (int64_t)bh * 2 * D * D;
  half8 whi[2][4], wlo[2][4];
#pragma unroll
  for (int eb = 0; eb < 2; ++eb)
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      whi[eb][t] = *reinterpret_cast<const half8*>(w + (32 * eb + n) * D + 16 * t + 8 * g);
      wlo[eb][t] = *reinterpret_cast<const half8*>(w + D * D + (32 * eb + n) * D + 16 * t + 8 * g);
    }
  const float winv = p.winv[bh];

  // B operand: f(Q)^T, column = token n, same contraction slots
  const uint16_t* qrow = p.q + b * p.sq.b + (int64_t)tok_c * p.sq.s + h * p.sq.h;
  half8 qf[4];
#pragma unroll
  for (int t = 0; t < 4; ++t) qf[t] = *reinterpret_cast<const half8*>(qrow + 16 * t + 8 * g);

  if (EA) {
    float x[4][8];
    float mx = -__builtin_inff();
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
      for (int s = 0; s < 8; ++s) {
        x[t][s] = (float)qf[t][s] * kLog2e;
        mx = fmaxf(mx, x[t][s]);
      }
    mx = fmaxf(mx, xchg32(mx));
    float sum = 0.f;
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
      for (int s = 0; s < 8; ++s) {
        x[t][s] = __builtin_amdgcn_exp2f(x[t][s] - mx);
        sum += x[t][s];
      }
    sum += xchg32(sum);
    const float inv = 1.f / sum;
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
      for (int s = 0; s < 8; ++s) qf[t][s] = (_Float16)(x[t][s] * inv);
  }

  float16v ahi[2], alo[2];
#pragma unroll
  for (int eb = 0; eb < 2; ++eb)
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      ahi[eb][r] = 0.f;
      alo[eb][r] = 0.f;
    }
#pragma unroll
  for (int t = 0; t < 4; ++t)
#pragma unroll
    for (int eb = 0; eb < 2; ++eb) {
      ahi[eb] = F16::mfma(whi[eb][t], qf[t], ahi[eb]);
      alo[eb] = F16::mfma(wlo[eb][t], qf[t], alo[eb]);
    }

  if (tok < p.S) {
    const int64_t off = b * p.so.b + (int64_t)tok * p.so.s + h * p.so.h;
#pragma unroll
    for (int eb = 0; eb < 2; ++eb)
#pragma unroll
      for (int q4 = 0; q4 < 4; ++q4) {
        const int e0 = 32 * eb + 8 * q4 + 4 * g;
        float y[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) y[e] = (ahi[eb][4 * q4 + e] + alo[eb][4 * q4 + e] * (1.f / 2048.f)) * winv;
        if (F32OUT) {
          float4v o4 = {y[0], y[1], y[2], y[3]};
          *reinterpret_cast<float4v*>(static_cast<float*>(p.o) + off + e0) = o4;
        } else {
          uint2 pk;
          pk.x = (uint32_t)F16::from_float(y[0]) | ((uint32_t)F16::from_float(y[1]) << 16);
          pk.y = (uint32_t)F16::from_float(y[2]) | ((uint32_t)F16::from_float(y[3]) << 16);
          *reinterpret_cast<uint2*>(static_cast<uint16_t*>(p.o) + off + e0) = pk;
        }
      }
  }
}

// ---------------------------------------------------------------------------------------------------
hipError_t launch_linattn(const FtAttnArgs& a, int kind, int normalize_q, int out_dtype, void* ws, hipStream_t s) {
  LinParams p;
  p.q = (const uint16_t*)a.q;
  p.k = (const uint16_t*)a.k;
  p.v = (const uint16_t*)a.v;
  p.o = a.o;
  p.sq = Strides3{a.sq.b, a.sq.s, a.sq.h};
  p.sk = Strides3{a.sk.b, a.sk.s, a.sk.h};
  p.sv = Strides3{a.sv.b, a.sv.s, a.sv.h};
  p.so = Strides3{a.so.b, a.so.s, a.so.h};
  p.B = a.B;
  p.H = a.H;
  p.S = a.Sq;
  lin_plan(a, &p.nch, &p.tiles_per_chunk);
  const bool ea = kind == FT_OP_EA;
  p.normalize_q = ea ? 0 : normalize_q;
  p.out_f32 = out_dtype == FT_F32;
  const size_t bh = (size_t)a.B * a.H;
  char* base = static_cast<char*>(ws);
  p.part = reinterpret_cast<float*>(base);
  base += bh * p.nch * kPartStride * sizeof(float);
  p.w = reinterpret_cast<uint16_t*>(base);
  base += bh * 2 * kLinD * kLinD * sizeof(uint16_t);
  p.winv = reinterpret_cast<float*>(base);

  constexpr int lds1 = 4 * kLinTile * 2 * kLinD + 4 * 32 * 4;
  static bool configured = false;
  if (!configured) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(linattn_kv_kernel<true>), hipFuncAttributeMaxDynamicSharedMemorySize, lds1);
    if (e == hipSuccess)
      e = hipFuncSetAttribute(reinterpret_cast<const void*>(linattn_kv_kernel<false>), hipFuncAttributeMaxDynamicSharedMemorySize, lds1);
    if (e != hipSuccess) return e;
    configured = true;
  }
  const dim3 grid1((unsigned)(bh * p.nch)), blk(kLinThreads);
  if (ea)
    hipLaunchKernelGGL(linattn_kv_kernel<true>, grid1, blk, lds1, s, p);
  else
    hipLaunchKernelGGL(linattn_kv_kernel<false>, grid1, blk, lds1, s, p);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return e;
  if (ea)
    hipLaunchKernelGGL(linattn_merge_kernel<true>, dim3((unsigned)bh), blk, 0, s, p);
  else
    hipLaunchKernelGGL(linattn_merge_kernel<false>, dim3((unsigned)bh), blk, 0, s, p);
  e = hipGetLastError();
  if (e != hipSuccess) return e;
  const dim3 grid3((unsigned)(bh * ((a.Sq + 127) / 128)));
  if (ea) {
    if (p.out_f32)
      hipLaunchKernelGGL((linattn_out_kernel<true, true>), grid3, blk, 0, s, p);
    else
      hipLaunchKernelGGL((linattn_out_kernel<true, false>), grid3, blk, 0, s, p);
  } else {
    if (p.out_f32)
      hipLaunchKernelGGL((linattn_out_kernel<false, true>), grid3, blk, 0, s, p);
    else
      hipLaunchKernelGGL((linattn_out_kernel<false, false>), grid3, blk, 0, s, p);
  }
  return hipGetLastError();
}

}  // namespace ft
