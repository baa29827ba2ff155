// Fused softmax attention forward for gfx950 (pass A of every softmax workload): the kernel template and its
// launch-shape selection.  Instantiated per element type and head size by attn_fwd_{f16,bf16}_{d64,d128}.hip (one
// translation unit each, so that they compile in parallel); attn_fwd.hip holds the dispatcher.
//
// Replaces the attention core the reference emits as a Triton kernel for cases/kernels/attn.py:18-34
// (and the identical prefix of h2o.py, kf.py, roco.py): O = softmax(QK^T / sqrt(D) + causal mask) V,
// never writing an S x S tensor.  Also emits the per-row log2-domain normaliser (max + log2 sum) that the
// column-statistics pass consumes, and in the KeyFormer modes the normaliser of the Gumbel-perturbed
// softmax of kf.py:36-39 instead.
//
// Mapping.  One workgroup = 32 WAVES query rows of one (b, h), one wave per 32 rows (4 waves and two
// workgroups per CU, or 8 waves and one: the same two waves per SIMD, but a staged K/V tile then serves
// twice as many rows); keys are streamed in tiles
// of 64 through double-buffered LDS (direct global->LDS loads).  Each wave computes the TRANSPOSED score
// block S^T = K Q^T with v_mfma_f32_32x32x16: a lane then owns one query (column l % 32) and 16 of the
// 32 keys of each block, so the online-softmax row max / row sum are in-lane reductions plus a single
// exchange with lane l ^ 32, and the accumulator registers are already the B operand (keys on the
// contraction axis) of O^T += V^T P^T.  V^T is fed by ds_read_b64_tr_b16 from the row-major V tile.
#pragma once
#include "device_common.hpp"
#include "kernel_params.h"
#include "noise.h"

#include <type_traits>

namespace ft {

constexpr int kAttnBN = 64;
constexpr bool kAttnTwoBlocks = true;

// Rescale threshold of the running maximum in log2 units: the stale maximum is kept (and O, l are not
// rescaled) while the new row maximum exceeds it by less than this, so unnormalised probabilities stay
// below 2^kRescaleSlack (exact in fp16/fp32; the final division uses the same maximum).
constexpr float kRescaleSlack = 6.f;

template <typename T, int D, bool CAUSAL, bool EMU, int KF, int WAVES>
__global__ void __launch_bounds__(64 * WAVES, (KF == kKfTensorLds ? 1 : 8 / WAVES)) attn_fwd_kernel(const AttnKernelParams p) {
  constexpr int BM = 32 * WAVES, BN = kAttnBN, NT = 64 * WAVES;
  constexpr int KSTEPS = D / 16;
  constexpr int DB = D / 32;
  typedef TileGeom<D> G;
  typedef typename T::vec8 vec8;
  constexpr int TILE_BYTES = BN * G::RB;
  constexpr bool kIsF16 = __is_same(typename T::elem, _Float16);
  constexpr bool kKfFast = KF == kKfSeededTau1 || KF == kKfSeededFast;           // seeded noise inside the packed path
  constexpr bool kSeeded = KF == kKfSeeded || kKfFast;
  // variants served by the pipelined fast path: the plain softmax in either type with either treatment of the
  // logits, and the packed seeded KeyFormer modes (fp16)
  constexpr bool kFastMasked = (kIsF16 && EMU && kKfFast) || KF == kKfNone || KF == kKfSoftcap;
  constexpr bool kCap = KF == kKfSoftcap;
  constexpr bool kErLds = KF == kKfTensorLds;               // noise tensor staged through LDS
  constexpr bool kTensor = KF == kKfTensor || kErLds;
  static_assert(!kKfFast || (kIsF16 && EMU), "the packed KeyFormer modes exist for fp16 with reference rounding only");
  // Software pipeline across tiles: the QK^T MFMAs of tile it+1 are issued in the same iteration as the
  // softmax (VALU) and PV MFMAs of tile it, so the matrix and vector pipes overlap inside one wave.
  // K therefore runs one tile ahead of V in LDS.
  // One LDS object per buffer: the compiler tracks outstanding direct-to-LDS loads per object, so reads
  // of one buffer do not wait for the loads in flight into the others.
  __shared__ __align__(16) char ldsK0[TILE_BYTES];
  __shared__ __align__(16) char ldsK1[TILE_BYTES];
  __shared__ __align__(16) char ldsV0[TILE_BYTES];
  __shared__ __align__(16) char ldsV1[TILE_BYTES];
  __shared__ __align__(16) uint32_t ldsCol[2 * BN];  // noise column terms of the current / next tile
  // kKfTensorLds: every wave's slice of the next noise tile (32 rows x 64 keys fp32), one 16-byte slot per lane and
  // load instruction: a lane reads back exactly the slots it filled
  constexpr int kErWaveBytes = 32 * BN * 4;
  __shared__ __align__(16) char ldsEr[kErLds ? WAVES * kErWaveBytes : 16];

  const int BH = p.B * p.H;
  const int nMB = (p.Sq + BM - 1) / BM;
  // (b, h) pair and rank among that pair's workgroups.  Workgroups are dealt round-robin to the 8 XCDs and, inside
  // an XCD, start in index order.  head_major: the workgroups of an XCD walk through that XCD's pairs one after
  // the other (all ranks of a pair are neighbours in the XCD's order), so that the workgroups resident on an XCD
  // at one time share the K/V of a few pairs in its L2; otherwise rank-major (every pair's rank 0 first).
  int bh = blockIdx.x % BH, rank = blockIdx.x / BH;
  if (p.head_major) {
    const int li = blockIdx.x >> 3, nrank = gridDim.x / BH;
    bh = (blockIdx.x & 7) + 8 * (li / nrank);
    rank = li % nrank;
  }
  // Heaviest (last) query blocks of every head first: longest-processing-time order keeps the causal
  // triangle balanced over the CUs.  Workgroups are dealt round-robin to the 8 XCDs, so with B*H a
  // multiple of 8 a head stays on one XCD and its K/V are shared through that XCD's L2.  (Walking an XCD
  // through its heads one at a time cuts the K/V re-reads from 1.6x to 1.1x of the operand size but
  // loses the balance: measured 15% slower.)
  int mb = nMB - 1 - rank;
  if (p.pair_order) {
    // Every workgroup is resident from the start (no more of them than slots), so nothing is left to hand out
    // as CUs free up: the heavy half is dealt first, descending, then the light half ascending, which tends to
    // put a heavy and a light block on the same CU (measured 50 -> 47 us at B1 H32 S2048; with more
    // workgroups than slots the descending order wins: 144 vs 164 us at S4096).
    const int half = (nMB + 1) / 2;
    mb = rank < half ? nMB - 1 - rank : rank - half;
  }
  const int b = bh / p.H, h = bh % p.H;
  const int lane = lane_id(), wave = wave_id();
  const int g = lane >> 5, n = lane & 31;
  // two_blocks (causal, set by the launcher when the pairs fill the chip evenly): the workgroup takes query
  // block nMB - 1 - slot and then block slot, the heaviest with the lightest, so that every workgroup walks the
  // same number of key tiles and no workgroup is launched into a half-empty chip at the end
  // (compiled in only where the second pass costs no registers: with it the 4-wave form and the packed KeyFormer
  // modes spill, and a spilled register's reload waits for the tile loads in flight: both count in vmcnt)
  constexpr bool kTwoPass = WAVES == 8 && (KF == kKfNone || KF == kKfSoftcap);
  const int npass = (kTwoPass && p.two_blocks && 2 * rank != nMB - 1) ? 2 : 1;
  for (int pass = 0; pass < npass; ++pass) {
  if (kTwoPass && p.two_blocks) mb = pass == 0 ? nMB - 1 - rank : rank;
  if (pass) __syncthreads();  // every wave has left the first block's K/V tiles
  const int m0 = mb * BM;
  const int qi = m0 + wave * 32 + n;
  const int qi_c = qi < p.Sq ? qi : p.Sq - 1;
  const float NEG_INF = -__builtin_inff();

  const uint16_t* qptr = p.q + b * p.sq.b + (int64_t)qi_c * p.sq.s + h * p.sq.h;
  vec8 qf[KSTEPS];
#pragma unroll
  for (int t = 0; t < KSTEPS; ++t) qf[t] = *reinterpret_cast<const vec8*>(qptr + 16 * t + 8 * g);

  const uint16_t* kbase = p.k + b * p.sk.b + (h / p.group) * p.sk.h;
  const uint16_t* vbase = p.v + b * p.sv.b + (h / p.group) * p.sv.h;

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
  n_fast = min(n_fast, nw);
  const int n_free = n_fast;             // leading tiles of which this wave sees every key
  if (!kFastMasked) n_fast = 0;          // the pipelined loop (and its mask-free instance) is not used

  NoiseKeys nk = {0, 0};
  uint32_t a_i = 0;
  const float* er_row = nullptr;
  if (kSeeded) {
    nk = noise_keys(p.seed, (uint32_t)bh);
    a_i = noise_row(nk, (uint32_t)qi);
  }
  if (KF == kKfTensor) er_row = p.exp_rand + b * p.er_sb + h * p.er_sh + (int64_t)qi_c * p.er_sr;
  // kKfTensorLds: the wave's slice of a noise tile is 32 rows x 256 bytes.  Load r8 of a tile brings rows
  // 4 r8 + [0..3] whole (a load instruction then touches 8 cache lines; with a lane fetching its own row's chunks
  // it touched 32, and the address path, not HBM, bounded the pass): lane l fills slot l % 16 of row 4 r8 + l / 16
  // with global chunk (l % 16) ^ (row % 16), the XOR placement that lets 32 rows be read back one chunk column at
  // a time without bank conflicts.  Chunks past the end of a row re-read its last chunk (those keys are masked),
  // rows past Sq the last row.
  rsrc_t er_rsrc = make_rsrc(kErLds ? p.exp_rand + b * p.er_sb + h * p.er_sh : nullptr);
  char* er_lds = ldsEr + (kErLds ? wave * kErWaveBytes : 0);
  // per-lane state of those loads: two registers (the offsets of the eight loads are rebuilt from them for every
  // tile: kept in registers across the loop they would cost eight, and this path has none to spare)
  const int er_cs = (lane & 15) ^ (lane >> 4);  // slot ^ (row % 4); the row's bits 2..3 are those of r8
  const uint32_t er_row_bytes = (uint32_t)p.er_sr * 4u;
  const uint32_t er_off0 = kErLds ? (uint32_t)(m0 + wave * 32 + (lane >> 4)) * er_row_bytes : 0u;
  const uint32_t er_off_last = kErLds ? (uint32_t)(p.Sq - 1) * er_row_bytes : 0u;
  auto issue_er = [&](int t) __attribute__((always_inline)) {
    const int last_chunk = p.Skv / 4 - 1;
    int cs = er_cs;
    uint32_t off0 = er_off0;
    asm volatile("" : "+v"(cs), "+v"(off0));  // not loop-invariant as far as the compiler can tell
#pragma unroll
    for (int r8 = 0; r8 < 8; ++r8) {
      const int c = min(t * (BN / 4) + (cs ^ (4 * (r8 & 3))), last_chunk);
      const uint32_t row_off = min(off0 + (uint32_t)(4 * r8) * er_row_bytes, er_off_last);
      load_lds16(er_rsrc, er_lds + r8 * 1024, row_off + (uint32_t)c * 16u, 0);
    }
  };
  // the lane's query row n, chunks 2 k8 + g (keys 8 k8 + 4 g + [0..3] of the tile: score registers 4 (k8 % 4) + [0..3]
  // of half k8 / 4)
  // (slot (2 k8 + g) ^ (n % 16) of row n: byte offset ((g ^ n % 16) << 4) ^ (k8 << 5) inside the row, so one
  // register and one xor with a constant per read)
  const uint32_t er_rd0 = (uint32_t)(n * 256) | (uint32_t)((g ^ (n & 15)) << 4);
  auto read_er = [&](float (&dst)[2][16]) __attribute__((always_inline)) {
    uint32_t rd0 = er_rd0;
    asm volatile("" : "+v"(rd0));
#pragma unroll
    for (int k8 = 0; k8 < 8; ++k8) {
      const float4v e4 = *reinterpret_cast<const float4v*>(er_lds + (rd0 ^ (uint32_t)(k8 << 5)));
#pragma unroll
      for (int e = 0; e < 4; ++e) dst[k8 >> 2][4 * (k8 & 3) + e] = e4[e];
    }
  };

  TileStager<D, BN, NT, kRowSwizzle> stK;
  TileStager<D, BN, NT, kTrSwizzle> stV;
  stK.init(kbase, p.sk.s);
  stV.init(vbase, p.sv.s);
  auto stage_k = [&](int t, char* dst) __attribute__((always_inline)) {
    if (t < ntiles) stK.issue(t * BN, min(BN, p.Skv - t * BN), dst);
  };
  auto stage_v = [&](int t, char* dst) __attribute__((always_inline)) {
    if (t < ntiles) stV.issue(t * BN, min(BN, p.Skv - t * BN), dst);
    if (kSeeded && t < ntiles && threadIdx.x < BN)
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

  // Per-lane LDS byte offsets of the MFMA operand reads inside a tile (the XOR swizzles make them
  // lane-dependent, so they are computed once instead of per read).
  uint32_t koff[KSTEPS];  // K row n (and n + 32 via an immediate), chunk 2t + g
#pragma unroll
  for (int t = 0; t < KSTEPS; ++t) koff[t] = n * G::RB + (((2 * t + g) ^ G::row_swz(n)) << 4);
  uint32_t voff[DB];  // V^T operand: rows 4g + (l%16)/4 (+ 16 ks, + 8 via immediates), columns 32 db + ...
  {
    const int j16 = lane & 15, dhalf = (lane >> 4) & 1;
    const int r0 = 4 * g + (j16 >> 2);
#pragma unroll
    for (int db = 0; db < DB; ++db) {
      const int d0 = 32 * db + 16 * dhalf + 4 * (j16 & 3);
      voff[db] = r0 * G::RB + (((d0 >> 3) ^ G::tr_swz(r0)) << 4) + (d0 & 7) * 2;
    }
  }

  // ---- S^T = K Q^T : [64 keys] x [32 queries] as two 32x32 blocks (16 LDS reads, 16 MFMAs), optionally
  // in two halves over the head dimension so that other work can sit between them
  auto qk_part = [&](float16v (&s)[2], const char* tk, auto t0_tag, auto t1_tag) __attribute__((always_inline)) {
    constexpr int T0 = decltype(t0_tag)::value, T1 = decltype(t1_tag)::value;
    if (T0 == 0) {
#pragma unroll
      for (int mbk = 0; mbk < 2; ++mbk)
#pragma unroll
        for (int r = 0; r < 16; ++r) s[mbk][r] = 0.f;
    }
    vec8 ka[KSTEPS][2];
#pragma unroll
    for (int t = T0; t < T1; ++t)
#pragma unroll
      for (int mbk = 0; mbk < 2; ++mbk) ka[t][mbk] = *reinterpret_cast<const vec8*>(tk + koff[t] + mbk * 32 * G::RB);
#pragma unroll
    for (int t = T0; t < T1; ++t)
#pragma unroll
      for (int mbk = 0; mbk < 2; ++mbk) s[mbk] = T::mfma(ka[t][mbk], qf[t], s[mbk]);
  };
  auto qk = [&](float16v (&s)[2], const char* tk) __attribute__((always_inline)) {
    qk_part(s, tk, std::integral_constant<int, 0>{}, std::integral_constant<int, KSTEPS>{});
  };
  // LDS latency is far longer than an MFMA, so operand reads must run several MFMAs ahead of their
  // consumers; sched_group_barrier sequences pin that order (the scheduler would otherwise sink each
  // read next to its use to save registers).  Masks: 0x008 MFMA, 0x100 LDS read, 0x002 VALU.
  auto sched_qk_alone = [&]() __attribute__((always_inline)) {
    __builtin_amdgcn_sched_group_barrier(0x100, 6, 0);
#pragma unroll
    for (int t = 0; t < KSTEPS - 3; ++t) {
      __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
    }
    __builtin_amdgcn_sched_group_barrier(0x008, 6, 0);
  };

  auto rescale = [&](float rowmax) __attribute__((always_inline)) {
    const bool grow = rowmax > m_run + kRescaleSlack;  // identical in both lanes of a row
    if (__any(grow)) {
      const float m_new = grow ? rowmax : m_run;
      const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);
      if (KF == kKfSeededTau1) l_kf *= alpha;
      if (KF == kKfSeededFast) l_kf *= __builtin_amdgcn_exp2f((m_run - m_new) * p.inv_tau);
      m_run = m_new;
      l_run *= alpha;
#pragma unroll
      for (int i = 0; i < DB; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) o_acc[i][r] *= alpha;
    }
  };

  // ---- softmax of the pipelined path, in two parts so that the rescale branch sits between them.
  // Rounding is monotonic, so the row maximum of the rounded logits is the rounded maximum of the raw
  // accumulators.
  // MASKED (tiles that straddle the diagonal or the end of K): hidden keys are left out of the maximum, so
  // that a row whose largest visible logit defines the stabiliser gets exp2(0) = 1 for it exactly (row 0
  // of a causal problem then has the normaliser of the reference, bit for bit).
  const float rcp_cap = kCap ? 1.f / p.softcap : 0.f;
  // row maximum of one tile's logits in the log2 domain (what rescale() compares with the running maximum)
  auto tile_max = [&](auto masked_tag, const float16v (&s)[2], int n0) __attribute__((always_inline)) -> float {
    constexpr bool MASKED = decltype(masked_tag)::value;
    const int lim = (CAUSAL ? min(qi + p.off, p.Skv - 1) : p.Skv - 1) - n0 - 4 * g;
    auto at = [&](int mbk, int r) __attribute__((always_inline)) -> float {
      if (!MASKED) return s[mbk][r];
      const int jl = 32 * mbk + 8 * (r >> 2) + (r & 3);
      return jl > lim ? NEG_INF : s[mbk][r];
    };
    // four independent chains, then a short tree: the reduction is latency-, not throughput-bound.  Three-operand
    // maxima throughout (v_max3_f32; this translation unit is built without NaN honouring, so none of them is
    // preceded by quieting moves of the MFMA results).
    float m4[4];
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      const int mbk = c >> 1, r0 = (c & 1) * 8;
      m4[c] = max3(at(mbk, r0), at(mbk, r0 + 1), at(mbk, r0 + 2));
      m4[c] = max3(m4[c], at(mbk, r0 + 3), at(mbk, r0 + 4));
      m4[c] = max3(m4[c], at(mbk, r0 + 5), at(mbk, r0 + 6));
    }
    const float t0 = max3(m4[0], at(0, 7), at(0, 15)), t1 = max3(m4[1], at(1, 7), at(1, 15));
    float amax = max3(max3(t0, t1, m4[2]), m4[3], m4[3]);
    const float other = xchg32(amax);
    amax = max3(amax, other, other);
    // soft-cap: the cap is monotonic as well (a product with a positive constant, tanh, roundings), so the
    // maximum of the capped logits is the capped maximum
    auto r16 = [](float x) { return T::to_float(T::from_float(x)); };
    if (EMU) {
      float t = r16(r16(amax) * p.logit_mul);
      if (kCap) t = r16(r16(tanh_exp_form(r16(t * rcp_cap))) * p.softcap);
      return t * kLog2e;
    } else if (kCap) {
      return p.softcap * tanh_exp_form(amax * (p.logit_mul * (1.f / kLog2e)) * rcp_cap) * kLog2e;
    }
    return amax * p.logit_mul;  // logit_mul = log2e / sqrt(D) when the logits stay in fp32
  };
  // MASKED: key j of the tile is hidden from this lane's query when j > qi + off or j >= Skv.
  auto fast_exp = [&](auto masked_tag, const float16v (&s)[2], vec8 (&pb)[4], int n0, int buf) __attribute__((always_inline)) {
    constexpr bool MASKED = decltype(masked_tag)::value;
    const float neg_m = -m_run;
    const half2v pk_hi = __builtin_bit_cast(half2v, p.pk_hi2), pk_lo = __builtin_bit_cast(half2v, p.pk_lo2);
    // local key index of register r is 32 mbk + 8 (r / 4) + 4 g + r % 4; it is visible iff <= lim + 4 g
    const int lim = (CAUSAL ? min(qi + p.off, p.Skv - 1) : p.Skv - 1) - n0 - 4 * g;
    uint4v pw[4];
    // Eight elements (one MFMA operand) at a time, stage by stage, so that consecutive instructions are
    // independent: every stage's result is needed only four instructions later.
#pragma unroll
    for (int blk = 0; blk < 4; ++blk) {
      const int mbk = blk >> 1, rb = (blk & 1) * 8;
      float x[8];
      if constexpr (EMU && kIsF16) {
        half2v t2[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const float2v a2 = {s[mbk][rb + 2 * i], s[mbk][rb + 2 * i + 1]};
          const half2v h2 = __builtin_convertvector(a2, half2v);  // QK^T is an fp16 tensor in the reference
          // ... divided by sqrt(D) in fp16: t2 = 8 * f16(h / sqrt(D)), exact for D = 64, two packed ops for D = 128
          t2[i] = D == 64 ? h2 : __builtin_elementwise_fma(h2, pk_hi, h2 * pk_lo);
        }
#pragma unroll
        for (int i = 0; i < 8; ++i)
          x[i] = kCap ? (float)t2[i >> 1][i & 1] * (rcp_cap * 0.125f)  // logit / cap, rounded below
                      : __builtin_fmaf((float)t2[i >> 1][i & 1], kLog2e / 8.f, neg_m);
      } else if constexpr (EMU) {
        // bf16: round QK^T, multiply by the tuned constant (== dividing by sqrt(D) in bf16), round again; the
        // conversions handle two elements each, unpacking a half is a shift or a mask
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const uint32_t h2 = T::pack2(s[mbk][rb + 2 * i], s[mbk][rb + 2 * i + 1]);
          const uint32_t t2 = T::pack2(T::lo(h2) * p.logit_mul, T::hi(h2) * p.logit_mul);
          x[2 * i] = kCap ? T::lo(t2) * rcp_cap : __builtin_fmaf(T::lo(t2), kLog2e, neg_m);
          x[2 * i + 1] = kCap ? T::hi(t2) * rcp_cap : __builtin_fmaf(T::hi(t2), kLog2e, neg_m);
        }
      } else {
#pragma unroll
        for (int i = 0; i < 8; ++i)
          x[i] = kCap ? s[mbk][rb + i] * (p.logit_mul * (1.f / kLog2e) * rcp_cap) : __builtin_fmaf(s[mbk][rb + i], p.logit_mul, neg_m);
      }
      if constexpr (kCap) {
        // Gemma2's soft-cap, cap * tanh(logit / cap): three 16-bit tensor ops in the reference
        // (cases/kernels/gemma2.py:31-33), each rounded when the reference's rounding is reproduced
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          float y0 = x[2 * i], y1 = x[2 * i + 1];
          if (EMU) {
            const uint32_t w = T::pack2(y0, y1);
            y0 = T::lo(w), y1 = T::hi(w);
          }
          float z0 = tanh_exp_form(y0), z1 = tanh_exp_form(y1);
          if (EMU) {
            const uint32_t w = T::pack2(z0, z1);
            const uint32_t c = T::pack2(T::lo(w) * p.softcap, T::hi(w) * p.softcap);
            x[2 * i] = __builtin_fmaf(T::lo(c), kLog2e, neg_m);
            x[2 * i + 1] = __builtin_fmaf(T::hi(c), kLog2e, neg_m);
          } else {
            x[2 * i] = __builtin_fmaf(z0 * p.softcap, kLog2e, neg_m);
            x[2 * i + 1] = __builtin_fmaf(z1 * p.softcap, kLog2e, neg_m);
          }
        }
      }
      if (MASKED) {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          const int jl = 32 * mbk + 8 * ((rb + i) >> 2) + ((rb + i) & 3);
          x[i] = (jl > lim) ? NEG_INF : x[i];
        }
      }
      // KeyFormer, seeded: E = -ln u of the 8 (query, key) pairs; the column terms of keys
      // 32 mbk + 8 (rb / 4 [+ 1]) + 4 g + [0..3] are two aligned groups of four in LDS
      float ee[8];
      if constexpr (kKfFast) {
        const uint32_t* col = ldsCol + buf * BN + 32 * mbk + 2 * rb + 4 * g;
        const uint4v c0 = *reinterpret_cast<const uint4v*>(col), c1 = *reinterpret_cast<const uint4v*>(col + 8);
#pragma unroll
        for (int i = 0; i < 8; ++i)  // log2 u = -E / ln 2 (negative): the constant factor is applied once, at the end
          ee[i] = __builtin_amdgcn_logf(noise_uniform(a_i, i < 4 ? c0[i] : c1[i - 4]));
        if constexpr (KF == kKfSeededFast) {
          const float shift = -kLog2Ln2 * p.inv_tau;
#pragma unroll
          for (int i = 0; i < 8; ++i)  // exp2(((t - m) log2e - log2 E) / tau); hidden keys carry x = -inf
            l_kf += __builtin_amdgcn_exp2f(__builtin_fmaf(x[i] - __builtin_amdgcn_logf(-ee[i]), p.inv_tau, shift));
        }
      }
#pragma unroll
      for (int i = 0; i < 8; ++i) x[i] = __builtin_amdgcn_exp2f(x[i]);
      if constexpr (KF == kKfSeededTau1) {
#pragma unroll
        for (int i = 0; i < 8; ++i) l_kf = __builtin_fmaf(x[i], __builtin_amdgcn_rcpf(ee[i]), l_kf);  // -ln2 exp(t - m) / E
      }
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        pw[blk][i] = T::pack2(x[2 * i], x[2 * i + 1]);  // whole 32-bit words: no 16-bit shuffles
        l_run = T::add2(pw[blk][i], l_run);             // row sum of the 16-bit P the MFMA consumes
      }
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) pb[i] = __builtin_bit_cast(vec8, pw[i]);
  };

  // ---- generic path (tensor-noise KeyFormer, and the seeded modes outside the packed form): softmax of one
  // 32-key half of a tile, s (raw accumulators of one 32x32 block) -> pb (two MFMA operands of 16-bit
  // unnormalised probabilities).  Half a tile at a time keeps the live set small enough for the noise slice
  // of the next tile to be in flight beside the accumulators.
  // MASKED: some key of the half is hidden from some query of the wave (the diagonal, the end of K).
  auto softmax_half = [&](auto masked_tag, const float16v& s, vec8 (&pb)[2], int n0h, int buf, int mbk, const float (&er)[16]) __attribute__((always_inline)) {
    constexpr bool MASKED = decltype(masked_tag)::value;
    // ---- logits in the log2 domain, with the reference's rounding points when EMU (the same chains as the
    // pipelined path: two elements per conversion)
    float x[16];
    if constexpr (EMU && kIsF16) {
      const half2v pk_hi = __builtin_bit_cast(half2v, p.pk_hi2), pk_lo = __builtin_bit_cast(half2v, p.pk_lo2);
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const float2v a2 = {s[2 * i], s[2 * i + 1]};
        const half2v h2 = __builtin_convertvector(a2, half2v);  // QK^T is an fp16 tensor in the reference
        // ... divided by sqrt(D) in fp16: t2 = 8 * f16(h / sqrt(D)), exact for D = 64, two packed ops for D = 128
        const half2v t2 = D == 64 ? h2 : __builtin_elementwise_fma(h2, pk_hi, h2 * pk_lo);
        x[2 * i] = (float)t2[0] * (kLog2e / 8.f);
        x[2 * i + 1] = (float)t2[1] * (kLog2e / 8.f);
      }
    } else if constexpr (EMU) {
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const uint32_t h2 = T::pack2(s[2 * i], s[2 * i + 1]);
        const uint32_t t2 = T::pack2(T::lo(h2) * p.logit_mul, T::hi(h2) * p.logit_mul);
        x[2 * i] = T::lo(t2) * kLog2e;
        x[2 * i + 1] = T::hi(t2) * kLog2e;
      }
    } else {
#pragma unroll
      for (int r = 0; r < 16; ++r) x[r] = s[r] * p.logit_mul;
    }
    if (MASKED) {
      // local key index of register r is 8 (r / 4) + 4 g + r % 4; it is visible iff <= lim + 4 g
      const int lim = (CAUSAL ? min(qi + p.off, p.Skv - 1) : p.Skv - 1) - n0h - 4 * g;
#pragma unroll
      for (int r = 0; r < 16; ++r) x[r] = (8 * (r >> 2) + (r & 3) > lim) ? NEG_INF : x[r];
    }
    float rowmax = max3(x[0], x[1], x[2]);
#pragma unroll
    for (int r = 3; r < 15; r += 2) rowmax = max3(rowmax, x[r], x[r + 1]);
    rowmax = fmaxf(rowmax, x[15]);
    rowmax = fmaxf(rowmax, xchg32(rowmax));

    // ---- KeyFormer: running normaliser of softmax((logit + gumbel) / tau), gumbel = -ln(E)
    {
      float z[16];
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        float log2E;
        if (kTensor) {
          log2E = __builtin_amdgcn_logf(er[r]);
        } else {
          const int jl = 32 * mbk + 8 * (r >> 2) + 4 * g + (r & 3);
          const float u = noise_uniform(a_i, ldsCol[buf * BN + jl]);
          log2E = __builtin_amdgcn_logf(-kLn2 * __builtin_amdgcn_logf(u));
        }
        z[r] = (x[r] - log2E) * p.inv_tau;
      }
      float zmax = max3(z[0], z[1], z[2]);
#pragma unroll
      for (int r = 3; r < 15; r += 2) zmax = max3(zmax, z[r], z[r + 1]);
      zmax = fmaxf(zmax, z[15]);
      zmax = fmaxf(zmax, xchg32(zmax));
      // finite from the first half on: key 0 is visible to every row, so a later half that is hidden
      // entirely (zmax = -inf) adds exp2(-inf) = 0
      const float mk_new = fmaxf(m_kf, zmax);
      float zs = 0.f;
#pragma unroll
      for (int r = 0; r < 16; ++r) zs += __builtin_amdgcn_exp2f(z[r] - mk_new);
      l_kf = l_kf * __builtin_amdgcn_exp2f(m_kf - mk_new) + zs;
      m_kf = mk_new;
    }

    rescale(rowmax);
    uint4v pw[2];
#pragma unroll
    for (int r = 0; r < 16; r += 2) {
      const uint32_t w = T::pack2(__builtin_amdgcn_exp2f(x[r] - m_run), __builtin_amdgcn_exp2f(x[r + 1] - m_run));
      l_run = T::add2(w, l_run);  // row sum of the 16-bit P the MFMA consumes
      pw[r >> 3][(r & 7) >> 1] = w;
    }
#pragma unroll
    for (int i = 0; i < 2; ++i) pb[i] = __builtin_bit_cast(vec8, pw[i]);
  };

  // ---- O^T += V^T P^T (32 transposed LDS reads, 16 MFMAs)
  auto read_vt = [&](const char* tv, int ks, int db) __attribute__((always_inline)) -> vec8 {
    const char* p0 = tv + voff[db] + ks * 16 * G::RB;
    short4v lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(FT_LDS(short4v, p0));
    short4v hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(FT_LDS(short4v, p0 + 8 * G::RB));
    short8v both = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
    return __builtin_bit_cast(vec8, both);
  };
  auto pv = [&](const vec8 (&pb)[4], const char* tv) __attribute__((always_inline)) {
    vec8 va[4][DB];
#pragma unroll
    for (int ks = 0; ks < 4; ++ks)
#pragma unroll
      for (int db = 0; db < DB; ++db) va[ks][db] = read_vt(tv, ks, db);
#pragma unroll
    for (int ks = 0; ks < 4; ++ks)
#pragma unroll
      for (int db = 0; db < DB; ++db) o_acc[db] = T::mfma(va[ks][db], pb[ks], o_acc[db]);
  };
  auto sched_pv_alone = [&]() __attribute__((always_inline)) {
    __builtin_amdgcn_sched_group_barrier(0x100, 8, 1);
#pragma unroll
    for (int i = 0; i < 4 * DB - 4; ++i) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 1);
      __builtin_amdgcn_sched_group_barrier(0x100, 2, 1);
    }
    __builtin_amdgcn_sched_group_barrier(0x008, 4, 1);
  };

  // One tile of the pipelined loop.  Three things overlap inside a wave: the QK^T MFMAs of the NEXT tile, the
  // softmax VALU chain of this tile (whose stabiliser was settled before the tile began) and this tile's PV
  // MFMAs; the row maximum of the next tile is taken at the end, under the PV MFMAs, so that its long dependent
  // chain (32 values -> 1, one lane exchange, the 16-bit roundings) never stands alone.  The only branch, the
  // rare rescale of the running maximum, sits at the very start of the tile.
  //   pend_max: log2-domain row maximum of the tile about to be processed (from the previous tile, or the prologue)
  float pend_max = NEG_INF;
  auto fast_tile = [&](auto masked_tag, auto next_masked_tag, auto stage_tag, float16v (&s_cur)[2], float16v (&s_next)[2],
                       const char* tk_next, const char* tv, int n0, int it, char* k_dst, char* v_dst) __attribute__((always_inline)) {
    constexpr bool STAGE = decltype(stage_tag)::value;
    constexpr int kValuGroup = kKfFast ? 12 : kCap ? 11 : 6;  // vector instructions placed after each MFMA
    vec8 pb[4];
    rescale(pend_max);
    // STAGE: the direct-to-LDS loads of K[it+2] and V[it+1] (both full tiles) are issued from inside this
    // block, one every few MFMAs.  Issued back to back they fill the texture-address queue (one 1 KB load
    // per 16 cycles per CU) and the wave stalls at issue for about a sixth of the tile time.
    if (STAGE) {  // after the rescale branch, so that the loads share a basic block with the MFMAs
      stK.issue_full((it + 2) * BN, k_dst);
      stV.issue_full((it + 1) * BN, v_dst);
    }
    qk(s_next, tk_next);
    if (kKfFast && STAGE && threadIdx.x < BN)  // column terms of tile it + 1 (the other half of ldsCol)
      ldsCol[((it + 1) & 1) * BN + threadIdx.x] = noise_col(nk, (uint32_t)((it + 1) * BN + threadIdx.x));
    fast_exp(masked_tag, s_cur, pb, n0, it & 1);
    pv(pb, tv);
    pend_max = tile_max(next_masked_tag, s_next, n0 + BN);
    __builtin_amdgcn_sched_group_barrier(0x100, 6, 2);
#pragma unroll
    for (int i = 0; i < 2 * KSTEPS; ++i) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 2);
      __builtin_amdgcn_sched_group_barrier(0x100, 2, 2);
      if (STAGE && (i & 3) == 1) __builtin_amdgcn_sched_group_barrier(0x020, 1, 2);
      __builtin_amdgcn_sched_group_barrier(0x002, kValuGroup, 2);
    }
#pragma unroll
    for (int i = 0; i < 4 * DB; ++i) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 2);
      __builtin_amdgcn_sched_group_barrier(0x100, 2, 2);
      if (STAGE && (i & 3) == 1) __builtin_amdgcn_sched_group_barrier(0x020, 1, 2);
      __builtin_amdgcn_sched_group_barrier(0x002, kValuGroup, 2);
    }
  };

  // One iteration = one barrier.  On entry K[it+1] and V[it] have been requested; K[it+2] and V[it+1] are
  // requested here, into the buffers every wave has finished reading.
  auto sync_and_stage = [&](int it, char* k_dst, char* v_dst) __attribute__((always_inline)) {
    wait_vmem();
    __syncthreads();
    stage_k(it + 2, k_dst);
    stage_v(it + 1, v_dst);
  };

  if constexpr (kFastMasked) {
  // ---- prologue: K[0], V[0], K[1] in flight; scores of tile 0
  stage_k(0, ldsK0);
  stage_v(0, ldsV0);
  stage_k(1, ldsK1);
  wait_vmem();
  __syncthreads();
  qk(S0, ldsK0);
  sched_qk_alone();

  int it = 0;
  // ---- mask-free tiles, two per trip so that the two score buffers swap roles without copies
  // pairs (it, it+1) of mask-free tiles whose staged tiles K[it+2], K[it+3], V[it+1], V[it+2] are whole tiles
  const int nf2 = max(0, min(n_fast, p.Skv / BN - 2)) & ~1;
  // tiles from nf2 on go through the masked instance (which is exact for a tile that needs no mask as well); so
  // does tile 0, which may be one of them.
  pend_max = tile_max(std::true_type{}, S0, 0);
  for (; it < nf2 - 2; it += 2) {
    wait_vmem();
    __syncthreads();
    fast_tile(std::false_type{}, std::false_type{}, std::true_type{}, S0, S1, ldsK1, ldsV0, 0, it, ldsK0, ldsV1);      // stages K[it+2], V[it+1]
    wait_vmem();
    __syncthreads();
    fast_tile(std::false_type{}, std::false_type{}, std::true_type{}, S1, S0, ldsK0, ldsV1, 0, it + 1, ldsK1, ldsV0);  // stages K[it+3], V[it+2]
  }
  if (it < nf2) {  // the last mask-free pair: the tile after it takes its maximum over visible keys
    wait_vmem();
    __syncthreads();
    fast_tile(std::false_type{}, std::false_type{}, std::true_type{}, S0, S1, ldsK1, ldsV0, 0, it, ldsK0, ldsV1);
    wait_vmem();
    __syncthreads();
    fast_tile(std::false_type{}, std::true_type{}, std::true_type{}, S1, S0, ldsK0, ldsV1, (it + 1) * BN, it + 1, ldsK1, ldsV0);
    it += 2;
  }
  // ---- tiles that straddle the diagonal or the end of K
  // Two per trip where the registers allow it (`it` is even here), so that the LDS buffers are named at compile
  // time: with a buffer chosen at run time the compiler cannot tell the tile being read from the tile being
  // loaded, and the first operand read of the tile waits for the K / V tiles requested a few instructions earlier.
  constexpr bool kTailPairs = KF == kKfNone || KF == kKfSoftcap;
  if constexpr (kTailPairs) {
    auto tail_tile = [&](int it, auto odd_tag) __attribute__((always_inline)) {
      constexpr bool odd = decltype(odd_tag)::value;
      sync_and_stage(it, odd ? ldsK1 : ldsK0, odd ? ldsV0 : ldsV1);
      fast_tile(std::true_type{}, std::true_type{}, std::false_type{}, S0, S1, odd ? ldsK0 : ldsK1, odd ? ldsV1 : ldsV0, it * BN, it, nullptr, nullptr);
#pragma unroll
      for (int mbk = 0; mbk < 2; ++mbk) S0[mbk] = S1[mbk];
    };
    for (; it + 1 < nw; it += 2) {
      tail_tile(it, std::false_type{});
      tail_tile(it + 1, std::true_type{});
    }
    if (it < nw) {
      tail_tile(it, std::false_type{});
      ++it;
    }
  }
  for (; it < nw; ++it) {
    const bool odd = it & 1;
    sync_and_stage(it, odd ? ldsK1 : ldsK0, odd ? ldsV0 : ldsV1);
    fast_tile(std::true_type{}, std::true_type{}, std::false_type{}, S0, S1, odd ? ldsK0 : ldsK1, odd ? ldsV1 : ldsV0, it * BN, it, nullptr, nullptr);
#pragma unroll
    for (int mbk = 0; mbk < 2; ++mbk) S0[mbk] = S1[mbk];
  }
  // ---- tiles entirely above this wave's diagonal: keep the workgroup's barriers and staging in step
  for (; it < ntiles; ++it) sync_and_stage(it, (it & 1) ? ldsK1 : ldsK0, (it & 1) ? ldsV0 : ldsV1);
  } else {
  // ---- generic path: not pipelined across tiles.  K and V of tile it are read while those of tile it + 1 are
  // loaded; a tile is worked on as two halves of 32 keys (8 + 8 MFMAs each), every key masked by comparison.
  // Two tiles per trip, so that every LDS buffer is named at compile time: with a buffer chosen at run time
  // the compiler cannot tell the tile being read from the tile being loaded, and drains every load in flight
  // before the first LDS read of the tile.
  // KeyFormer, tensor mode: er[mbk] is this lane's slice of the noise tile (its query row, the 16 keys of its
  // score registers in half mbk).  The S x S tensor is the one operand that comes from HBM every time, so the
  // slice of the next tile is requested as soon as the softmax has consumed this tile's (same registers) and is
  // in flight for the rest of the tile: a load consumed in the iteration that issues it leaves the memory
  // system idle while the tile is worked on.  (Ordinary loads: the four 16-byte pieces a lane pair takes from
  // one 128-byte line arrive in four instructions, and with the non-temporal hint each went to HBM.)
  float er[2][16];
  auto load_er_half = [&](float (&dst)[16], int it, int mbk) __attribute__((always_inline)) {
    const int c0 = it * BN + 32 * mbk;
    if (p.er_vec4 && c0 + 32 <= p.Skv) {  // the whole half lies inside the tensor: four 16-byte loads
#pragma unroll
      for (int q4 = 0; q4 < 4; ++q4) {
        const float4v e4 = *reinterpret_cast<const float4v*>(er_row + c0 + 8 * q4 + 4 * g);
#pragma unroll
        for (int e = 0; e < 4; ++e) dst[4 * q4 + e] = e4[e];
      }
    } else {  // keys past the end read the last one instead (no branches); they are masked
#pragma unroll
      for (int r = 0; r < 16; ++r) dst[r] = er_row[min(c0 + 8 * (r >> 2) + 4 * g + (r & 3), p.Skv - 1)];
    }
  };
  auto qk_half = [&](float16v& s, const char* tk, int mbk) __attribute__((always_inline)) {
#pragma unroll
    for (int r = 0; r < 16; ++r) s[r] = 0.f;
#pragma unroll
    for (int t = 0; t < KSTEPS; ++t)
      s = T::mfma(*reinterpret_cast<const vec8*>(tk + koff[t] + mbk * 32 * G::RB), qf[t], s);
  };
  auto pv_half = [&](const vec8 (&pb)[2], const char* tv, int mbk) __attribute__((always_inline)) {
#pragma unroll
    for (int ksl = 0; ksl < 2; ++ksl)
#pragma unroll
      for (int db = 0; db < DB; ++db) o_acc[db] = T::mfma(read_vt(tv, 2 * mbk + ksl, db), pb[ksl], o_acc[db]);
  };
  auto slow_tile = [&](int it, auto odd_tag) __attribute__((always_inline)) {
    constexpr bool odd = decltype(odd_tag)::value;
    wait_vmem();
    __syncthreads();
    if (kErLds && it < nw) {
      // this tile's slice from LDS to registers; the next tile's is requested into the same slots further down.  The
      // reads must have returned before those loads may overwrite their slots (nothing in the hardware orders an LDS
      // read against a later direct-to-LDS load).
      read_er(er);
      __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0)
    }
    stage_k(it + 1, odd ? ldsK0 : ldsK1);
    stage_v(it + 1, odd ? ldsV0 : ldsV1);
    if (it < nw) {  // not entirely above this wave's diagonal
#pragma unroll
      for (int mbk = 0; mbk < 2; ++mbk) {
        float16v s;
        vec8 pb[2];
        qk_half(s, odd ? ldsK1 : ldsK0, mbk);
        if (it < n_free)
          softmax_half(std::false_type{}, s, pb, it * BN + 32 * mbk, odd ? 1 : 0, mbk, er[mbk]);
        else
          softmax_half(std::true_type{}, s, pb, it * BN + 32 * mbk, odd ? 1 : 0, mbk, er[mbk]);
        if (KF == kKfTensor && it + 1 < nw) load_er_half(er[mbk], it + 1, mbk);
        // The next tile's noise, in flight for the rest of the tile without holding a register.  Requested here, behind
        // the first half's contraction and softmax, rather than at the top of the tile in front of the K / V staging
        // loads: the eight loads no longer queue up with the staging at the moment every wave leaves the barrier
        // (B1 H32 S4096, same process: 538 -> 512 us per call; before the softmax 523, after the first half's PV 516,
        // four loads behind each half's softmax 524).
        if (kErLds && mbk == 0 && it + 1 < nw) issue_er(it + 1);
        pv_half(pb, odd ? ldsV1 : ldsV0, mbk);
      }
    }
  };
  if (KF == kKfTensor) {
    load_er_half(er[0], 0, 0);
    load_er_half(er[1], 0, 1);
  }
  if (kErLds && nw > 0) issue_er(0);
  stage_k(0, ldsK0);
  stage_v(0, ldsV0);
  int it = 0;
  for (; it + 1 < ntiles; it += 2) {
    slow_tile(it, std::false_type{});
    slow_tile(it + 1, std::true_type{});
  }
  if (it < ntiles) slow_tile(it, std::false_type{});
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
  if (kTensor || kSeeded) {
    l_kf += xchg32(l_kf);
    if (KF == kKfSeededTau1) l_kf *= -kLog2e;  // the sum was taken over 1 / log2 u = -ln2 / E
    // packed modes: the perturbed sum shares the plain softmax's stabiliser, scaled by 1 / tau
    const float base = KF == kKfSeededTau1 ? m_run : KF == kKfSeededFast ? m_run * p.inv_tau : m_kf;
    if (qi < p.Sq && g == 0) p.lse_kf[(int64_t)bh * p.Sq + qi] = base + __builtin_amdgcn_logf(l_kf);
  }
  }  // pass
}

// ---------------------------------------------------------------------------------------------------
// launch-shape selection (host)

int device_cu_count();     // attn_fwd.hip
int attn_form_override();  // attn_fwd.hip: 0, or (1: 4 waves, 2: 8 waves, 3: 8 waves and two blocks) | 8: head-major order

template <typename T, int D, bool CAUSAL, bool EMU, int KF>
hipError_t launch_one(const AttnKernelParams& p0, hipStream_t stream) {
  AttnKernelParams p = p0;
  p.pair_order = 0;
  p.two_blocks = 0;
  p.head_major = 0;
  const int forced = attn_form_override();
  const int64_t BH = (int64_t)p.B * p.H;
  // 256-row workgroups (8 waves) halve the K/V staging per row (measured 148 vs 158 us at B1 H32 S4096), but
  // there are half as many of them: used on the pipelined paths once they still fill the chip twice
  // (kKfTensorLds: the noise slices in flight through LDS leave room for one workgroup per CU in either form, so the
  // 256-row one is used as soon as there is a workgroup for every CU)
  constexpr bool kHas8 = KF == kKfNone || KF == kKfSoftcap || KF == kKfSeededTau1 || KF == kKfSeededFast || KF == kKfTensorLds;
  if constexpr (kHas8) {
    const int nMB8 = (p.Sq + 255) / 256;
    const int64_t n8 = (int64_t)nMB8 * BH;
    const int64_t cus = device_cu_count();
    if ((forced & 7) ? (forced & 7) >= 2 : n8 >= (KF == kKfTensorLds ? cus : 2 * cus)) {
      // causal: pair the heaviest block with the lightest inside one workgroup when the pairs come out as whole
      // rounds of the chip (or as many rounds that a ragged last one does not matter)
      const int64_t pairs = (int64_t)((nMB8 + 1) / 2) * BH;
      constexpr bool kCanPair = kAttnTwoBlocks && (KF == kKfNone || KF == kKfSoftcap) && CAUSAL;
      p.two_blocks = kCanPair && nMB8 >= 2 && ((forced & 7) ? (forced & 7) == 3 : (pairs % cus == 0 || pairs >= 8 * cus));
      const int64_t grid = p.two_blocks ? pairs : n8;
      // equal workgroups in several rounds: let an XCD finish a pair's blocks before it starts the next pair's
      p.head_major = BH % 8 == 0 && (forced ? (forced & 8) != 0 : (p.two_blocks && grid >= 3 * cus));
      hipLaunchKernelGGL((attn_fwd_kernel<T, D, CAUSAL, EMU, KF, 8>), dim3((unsigned)grid), dim3(512), 0, stream, p);
      return hipGetLastError();
    }
  }
  const int nMB = (p.Sq + 127) / 128;
  dim3 grid((unsigned)(nMB * BH));
  p.pair_order = CAUSAL && (int64_t)grid.x <= 2 * (int64_t)device_cu_count();  // two workgroups of this form per CU
  p.head_major = BH % 8 == 0 && (forced & 8) != 0 && !p.pair_order;
  hipLaunchKernelGGL((attn_fwd_kernel<T, D, CAUSAL, EMU, KF, 4>), grid, dim3(256), 0, stream, p);
  return hipGetLastError();
}

template <typename T, int D>
hipError_t launch_td(const AttnKernelParams& p, bool causal, bool emu, int kf, hipStream_t s) {
#define FT_CASE(C, E, K) \
  if (causal == C && emu == E && kf == K) return launch_one<T, D, C, E, K>(p, s);
  FT_CASE(true, true, kKfNone) FT_CASE(true, false, kKfNone) FT_CASE(false, true, kKfNone) FT_CASE(false, false, kKfNone)
  FT_CASE(true, true, kKfTensor) FT_CASE(true, false, kKfTensor) FT_CASE(false, true, kKfTensor) FT_CASE(false, false, kKfTensor)
  FT_CASE(true, true, kKfTensorLds) FT_CASE(true, false, kKfTensorLds) FT_CASE(false, true, kKfTensorLds) FT_CASE(false, false, kKfTensorLds)
  FT_CASE(true, true, kKfSeeded) FT_CASE(true, false, kKfSeeded) FT_CASE(false, true, kKfSeeded) FT_CASE(false, false, kKfSeeded)
  FT_CASE(true, true, kKfSoftcap) FT_CASE(true, false, kKfSoftcap) FT_CASE(false, true, kKfSoftcap) FT_CASE(false, false, kKfSoftcap)
  if constexpr (std::is_same<T, F16>::value) {  // packed KeyFormer modes: fp16 with reference rounding only
    if (emu) {
      FT_CASE(true, true, kKfSeededTau1) FT_CASE(false, true, kKfSeededTau1)
      FT_CASE(true, true, kKfSeededFast) FT_CASE(false, true, kKfSeededFast)
    }
  }
#undef FT_CASE
  return hipErrorInvalidValue;
}

}  // namespace ft
