// Linear-attention cores EA and SimA for gfx950, head_dim 64 (head_dim 32 as pairs of adjacent heads: the merge
// step drops the two cross-head blocks of the 64x64 matrix, the output step keeps EA's softmax per half).
// fp16 or bf16 tensors (the harness's type switch, cases/attn.py:90,97) with MFMA operands of the same type, or
// fp32 tensors (the type of bench/ea.mlir:2, bench/sima.mlir:2), rounded to fp16 as they are loaded.
//
// Replaces the fused kernels the reference would emit for bench/ea.mlir:13-17 and bench/sima.mlir:13-17
// (asuka.softmax / asuka.normalize semantics: lib/Dialect/Asuka/Transforms/LowerComplexReduce.cpp:21-69):
//   EA  : O = softmax(Q, dim=D) . (softmax(K, dim=S)^T V)
//   SimA: O = (Q / sum_s|Q|) . ((K / sum_s|K|)^T V)          (per (b, h, channel) L1 norms over S)
// Both are HBM-bound (32 FLOP/byte): the design reads K and V once, Q twice (once for SimA's norm, once
// for the output product; EA reads it once) and writes O once.
//
// Three launches:
//   1. kv_partial: a workgroup owns a chunk of tokens of one (b, h); each of its four waves streams its
//      own 16-token strips of K and V (and Q for SimA's norm) independently of the others: global loads
//      into a rotating set of registers keep several strips in flight, a landed strip is written to a
//      wave-private LDS buffer and read back transposed, so the loop has no workgroup barrier.  Per strip
//      a wave accumulates the whole 64x64 matrix sum_s f(K[s,d]) V[s,e] with four MFMAs (both operands
//      have the contraction axis = tokens strided in memory, so both come from ds_read_b64_tr_b16), plus
//      the per-channel normalisers: EA an online (max, sum of exp) pair, SimA sum|K| and sum|Q|.  The
//      four waves are combined through LDS at the end and one partial per chunk is written.
//   2. merge: combines the chunks of one (b, h), folds every normaliser into the 64x64 matrix (the deferred
//      division the reference's EquivalentTransform pass performs, EquivalentTransform.cpp:303-341) and
//      stores it transposed as an fp16 hi/lo pair with a power-of-two scale per block of 16 output
//      channels, so that SimA's tiny values (~1e-6) neither underflow nor lose precision in fp16.
//   3. out: O^T = W^T f(Q)^T per 32-token wave tile.  A wave keeps W in registers for its whole chunk,
//      streams Q strips the same way, does EA's per-token softmax over the 64 channels in registers (a
//      lane owns half a token row; one exchange with lane l ^ 32) and turns the accumulator (lane =
//      token) into full 128-byte output rows through a small LDS transpose.
//
// Direct-to-LDS loads are not used here on purpose: the compiler orders every LDS read after all
// direct-to-LDS loads in flight unless it can prove they touch another LDS object, which drains a
// multi-strip prefetch at each step; plain loads into registers are tracked exactly.
#include "device_common.hpp"
#include "kernel_params.h"
#include <type_traits>
#include "../../include/ft_abi.h"

namespace ft {

constexpr int kLinD = 64;
constexpr int kLinTile = 128;     // chunk granularity in tokens
constexpr int kLinThreads = 256;
constexpr int kLinWaves = kLinThreads / 64;
constexpr int kPartStride = kLinD * kLinD + 2 * kLinD;  // floats per (bh, chunk) partial
constexpr int kNoSwizzle = 2;

struct LinParams {
  const uint16_t* q;
  const uint16_t* k;
  const uint16_t* v;
  void* o;
  Strides3 sq, sk, sv, so;
  float* part;      // [BH][nch][kPartStride]
  uint16_t* w;      // [BH][2][64 e][64 d] fp16: hi, lo * 2^11
  float* winv;      // [BH][4] 1 / scale of each block of 16 output channels
  int B, H, S;
  int nch;              // chunks per (b, h) of the K/V pass
  int tiles_per_chunk;  // 128-token tiles per chunk of the K/V pass
  int out_nch;              // the same for the output pass (its chunks are independent of the K/V pass's)
  int out_tiles_per_chunk;
  int half_heads;           // every 64-channel "head" is two adjacent heads of 32 channels (head_dim 32)
  int out_wave_heads;       // output pass: a workgroup takes four adjacent heads, one per wave
};

// Splits the sequence of every (b, h) into chunks so that about `workgroups` workgroups exist.  The K/V pass
// keeps two workgroups per CU and pays a pipeline fill, a four-wave fold and a partial-result write per
// workgroup, so it wants one round of them (512); the output pass runs more workgroups per CU and has no
// epilogue, so more, shorter ones balance better (measured in one process at B8 H16 S8192, EA / SimA:
// 1024 + 1024 workgroups 148 / 147 us, 512 + 1024 136 / 139, 512 + 2048 135 / 137, 512 + 4096 143 / 141).
constexpr int kKvWorkgroups = 512, kOutWorkgroups = 2048;

static void lin_plan(const FtAttnArgs& a, int workgroups, int* nch, int* tpc) {
  const int ntiles = (a.Sq + kLinTile - 1) / kLinTile;
  const int64_t bh = (int64_t)a.B * a.H > 0 ? (int64_t)a.B * a.H : 1;
  int want = (int)((workgroups + bh - 1) / bh);
  if (want < 1) want = 1;
  int t = (ntiles + want - 1) / want;
  if (t < 1) t = 1;
  if (t > 16) t = 16;
  *tpc = t;
  *nch = (ntiles + t - 1) / t;
}

// head_dim 32 runs as head_dim 64 over pairs of adjacent heads (the caller has checked that H is even and that
// the heads are 32 elements apart): the kernels see H / 2 heads of 64 channels and drop the cross-head blocks.
static FtAttnArgs lin_effective(const FtAttnArgs& a0, int* half_heads) {
  FtAttnArgs a = a0;
  *half_heads = a0.D == 32;
  if (*half_heads) {
    a.H = a0.H / 2 > 0 ? a0.H / 2 : 1;  // sizes a workspace even for arguments the entry point will refuse
    a.D = 64;
    a.sq.h = a.sk.h = a.sv.h = a.so.h = 64;
  }
  return a;
}

size_t linattn_workspace_bytes(const FtAttnArgs& a0, int) {
  int half;
  const FtAttnArgs a = lin_effective(a0, &half);
  int nch, tpc;
  lin_plan(a, kKvWorkgroups, &nch, &tpc);
  const size_t bh = (size_t)a.B * a.H;
  size_t bytes = bh * nch * kPartStride * sizeof(float);
  bytes += bh * 2 * kLinD * kLinD * sizeof(uint16_t);
  bytes += bh * 4 * sizeof(float);
  return (bytes + 255) & ~(size_t)255;
}

// One wave's private strip of ROWS tokens x 64 channels (128-byte rows): lane l moves the 16-byte chunk
// l % 8 of rows l / 8 + 8 i, global -> registers -> LDS, so every load instruction covers 8 whole rows.
// Rows past the end of the sequence re-read the last token (callers mask them).
// IN32: the tensor holds fp32 (256-byte rows); a lane then loads the 32 bytes behind its chunk and rounds them to
// eight fp16 values when the strip is parked in LDS, so that everything downstream sees the 16-bit layout.
template <int ROWS, int SWZ, bool IN32 = false>
struct StripMover {
  typedef TileGeom<kLinD> G;
  static constexpr int ROUNDS = ROWS / 8;
  static constexpr int LOADS = IN32 ? 2 * ROUNDS : ROUNDS;  // 16-byte loads per lane and strip
  typedef uint4v Regs[LOADS];
  const char* base;
  int64_t row_bytes;
  int last_row;
  int r_lane;
  int c16;
  int lds_off[ROUNDS];

  __device__ __forceinline__ void init(const uint16_t* base_, int64_t row_stride, int rows_total) {
    base = reinterpret_cast<const char*>(base_);
    row_bytes = row_stride * (IN32 ? 4 : 2);
    last_row = rows_total - 1;
    const int lane = lane_id();
    r_lane = lane >> 3;
    c16 = (lane & 7) * (IN32 ? 32 : 16);
#pragma unroll
    for (int it = 0; it < ROUNDS; ++it) {
      const int r = it * 8 + r_lane;
      const int cs = lane & 7;
      const int c = SWZ == kRowSwizzle ? (cs ^ G::row_swz(r)) : SWZ == kTrSwizzle ? (cs ^ G::tr_swz(r)) : cs;
      lds_off[it] = r * G::RB + c * 16;
    }
  }
  // rows past `last` are read as row `last`: a wave that limits itself to its own share can issue every
  // prefetch unconditionally (a fixed number of loads in flight, which the compiler can count: with loads that
  // may or may not have been issued it waits for all of them) without touching another wave's rows
  __device__ __forceinline__ void limit_rows(int last) { last_row = max(0, min(last_row, last)); }
  __device__ __forceinline__ void load(int row0, Regs& regs) const {
#pragma unroll
    for (int it = 0; it < ROUNDS; ++it) {
      const int r = min(row0 + it * 8 + r_lane, last_row);
      if (IN32) {
        regs[2 * it] = *reinterpret_cast<const uint4v*>(base + r * row_bytes + c16);
        regs[2 * it + 1] = *reinterpret_cast<const uint4v*>(base + r * row_bytes + c16 + 16);
      } else {
        regs[it] = *reinterpret_cast<const uint4v*>(base + r * row_bytes + c16);
      }
    }
  }
  // the lane's eight 16-bit elements of round `it`
  __device__ __forceinline__ uint4v chunk16(const Regs& regs, int it) const {
    if (!IN32) return regs[it];
    // (whole vectors are reinterpreted, then indexed: a bit cast applied to one element of a vector lvalue read
    // element 0 whatever the index)
    const float4v lo = __builtin_bit_cast(float4v, regs[2 * it]), hi = __builtin_bit_cast(float4v, regs[2 * it + 1]);
    const uint4v out = {F16::pack2(lo[0], lo[1]), F16::pack2(lo[2], lo[3]), F16::pack2(hi[0], hi[1]), F16::pack2(hi[2], hi[3])};
    return out;
  }
  __device__ __forceinline__ void to_lds(const Regs& regs, char* lds_strip) const {
#pragma unroll
    for (int it = 0; it < ROUNDS; ++it) *reinterpret_cast<uint4v*>(lds_strip + lds_off[it]) = chunk16(regs, it);
  }
};

// fp16-only packed maximum of the 8 elements of an operand, or the same through fp32 for bf16
template <typename T>
__device__ __forceinline__ float max8(typename T::vec8 v) {
  if constexpr (__is_same(typename T::elem, _Float16)) {
    half2v hm = __builtin_elementwise_max(__builtin_shufflevector(v, v, 0, 1), __builtin_shufflevector(v, v, 2, 3));
    hm = __builtin_elementwise_max(hm, __builtin_shufflevector(v, v, 4, 5));
    hm = __builtin_elementwise_max(hm, __builtin_shufflevector(v, v, 6, 7));
    return fmaxf((float)hm[0], (float)hm[1]);
  } else {
    float m = (float)v[0];
#pragma unroll
    for (int s = 1; s < 8; ++s) m = fmaxf(m, (float)v[s]);
    return m;
  }
}

// ---------------------------------------------------------------------------------------------------
// NQ: also accumulate sum_s |Q| (SimA with normalised queries).
// T: element type of the MFMA operands (F16 or BF16); IN32: the tensors hold fp32 and are rounded to fp16 on the way.
template <typename T, bool IN32, bool EA, bool NQ>
// (fp32 tensors with the |Q| sums keep three fp32 strips of two slots in flight: one workgroup per CU, so that the wave
// has the accumulation registers as well and nothing spills)
__global__ void __launch_bounds__(kLinThreads, (IN32 && NQ) ? 1 : 2) linattn_kv_kernel(const LinParams p) {
  static_assert(!IN32 || __is_same(typename T::elem, _Float16), "fp32 tensors are rounded to fp16 operands");
  typedef typename T::vec8 vec8;
  constexpr int D = kLinD, STEP = 16;
  // strips in flight per wave (three tensors at three strips each do not fit in registers, nor do fp32 strips)
  constexpr int P = (NQ || IN32) ? 2 : 3;
  constexpr int STRIP = STEP * 2 * D;         // 2 KB
  constexpr int R = STEP / 8;                 // 16-byte loads per lane, strip and tensor
  __shared__ __align__(16) char s_kv[kLinWaves][2 * STRIP];  // wave-private K and V strips
  __shared__ __align__(16) float s_x[2][D * D];              // end-of-kernel combine buffers
  __shared__ float s_m[kLinWaves * D];
  __shared__ float s_l[kLinWaves * D];
  __shared__ float s_f[kLinWaves * D];

  const int BH = p.B * p.H;
  const int bh = blockIdx.x % BH;
  const int ch = blockIdx.x / BH;
  const int b = bh / p.H, h = bh % p.H;
  const int lane = lane_id(), wave = wave_id();
  const int g = lane >> 5, n = lane & 31;
  const float NEG_INF = -__builtin_inff();
  float* fac = s_f + wave * D;
  char* tk = s_kv[wave];
  char* tv = tk + STRIP;

  const int tok_begin = ch * p.tiles_per_chunk * kLinTile;
  const int tok_end = min(p.S, tok_begin + p.tiles_per_chunk * kLinTile);
  const int nsteps = (tok_end - tok_begin + STEP - 1) / STEP;
  const int nmine = nsteps > wave ? (nsteps - wave + kLinWaves - 1) / kLinWaves : 0;  // steps wave, wave + 4, ...

  float16v acc[2][2];  // [channel block of K][channel block of V]
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[i >> 1][i & 1][r] = 0.f;
  float m_run[2] = {NEG_INF, NEG_INF};  // EA: running max of K[:, d], d = 32 db + n
  float l_run[2] = {0.f, 0.f};          // EA: sum of exp; SimA: sum |K|   (this lane's token slots only)
  float qabs[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) qabs[e] = 0.f;

  StripMover<STEP, kTrSwizzle, IN32> mvK, mvV;
  StripMover<STEP, kNoSwizzle, IN32> mvQ;
  constexpr int RL = IN32 ? 2 * R : R;  // 16-byte loads per lane, strip and tensor
  constexpr int ES = IN32 ? 2 : 1;  // tensor element size in units of the 16-bit pointer type
  mvK.init(p.k + (b * p.sk.b + h * p.sk.h) * ES, p.sk.s, p.S);
  mvV.init(p.v + (b * p.sv.b + h * p.sv.h) * ES, p.sv.s, p.S);
  if (NQ) mvQ.init(p.q + (b * p.sq.b + h * p.sq.h) * ES, p.sq.s, p.S);

  uint4v rk[P][RL], rv[P][RL], rq[P][RL];  // strips in flight, indexed by compile-time slot
  auto strip_row0 = [&](int i) { return tok_begin + (wave + kLinWaves * i) * STEP; };
  {
    const int last_mine = nmine > 0 ? strip_row0(nmine - 1) + STEP - 1 : tok_begin;
    mvK.limit_rows(last_mine);
    mvV.limit_rows(last_mine);
    if (NQ) mvQ.limit_rows(last_mine);
  }
  auto fetch = [&](int i, auto slot_tag) {
    constexpr int SLOT = decltype(slot_tag)::value;
    const int row0 = strip_row0(i);
    mvK.load(row0, rk[SLOT]);
    mvV.load(row0, rv[SLOT]);
    if (NQ) mvQ.load(row0, rq[SLOT]);
  };

  // one strip, already in the wave's LDS buffer: TAIL = some of its tokens lie past the end
  auto compute = [&](auto tail_tag, int t0) {
    constexpr bool TAIL = decltype(tail_tag)::value;
    vec8 ka[2];
#pragma unroll
    for (int db = 0; db < 2; ++db) ka[db] = read_tr_operand<D, vec8>(tk, 0, 32 * db);
    vec8 vb[2];
#pragma unroll
    for (int eb = 0; eb < 2; ++eb) vb[eb] = read_tr_operand<D, vec8>(tv, 0, 32 * eb);
    bool dead[8];  // token slot s of this lane is past the end
#pragma unroll
    for (int s = 0; s < 8; ++s) dead[s] = TAIL && t0 + 4 * g + (s & 3) + ((s >> 2) << 3) >= p.S;

    if (EA) {
      float m_new[2];
#pragma unroll
      for (int db = 0; db < 2; ++db) {
        float mx;
        if (TAIL) {
          mx = NEG_INF;
#pragma unroll
          for (int s = 0; s < 8; ++s) mx = fmaxf(mx, dead[s] ? NEG_INF : (float)ka[db][s]);
        } else {
          mx = max8<T>(ka[db]);
        }
        mx = fmaxf(mx, xchg32(mx));
        m_new[db] = fmaxf(m_run[db], mx);
      }
      // Lazy: the stale maximum is kept while no channel has outgrown it by more than kStaleMax (the operand
      // exp(k - m) then stays below e^4 = 55, exact enough in fp16 and far from its range; sums and matrix are
      // fp32 and the merge step works with whatever maximum a chunk reports).  Without the slack some of the
      // 64 channels moves its maximum in almost every strip and the whole 64x64 matrix is rescaled each time.
      constexpr float kStaleMax = 4.f;
      if (__any(m_new[0] > m_run[0] + kStaleMax || m_new[1] > m_run[1] + kStaleMax)) {
        // move the per-channel factor from "lane = channel" to the accumulator's "register = channel"
#pragma unroll
        for (int db = 0; db < 2; ++db) {
          // only the channels that outgrew their maximum move (factor exactly 1 for the others), so a channel's
          // arithmetic depends on its own column of K alone
          const float mt = m_new[db] > m_run[db] + kStaleMax ? m_new[db] : m_run[db];
          const float f = __builtin_amdgcn_exp2f((m_run[db] - mt) * kLog2e);
          l_run[db] *= f;
          if (g == 0) fac[32 * db + n] = f;
          m_run[db] = mt;
        }
        wave_lds_order();
#pragma unroll
        for (int db = 0; db < 2; ++db)
#pragma unroll
          for (int q4 = 0; q4 < 4; ++q4) {
            const float4v f4 = *reinterpret_cast<const float4v*>(fac + 32 * db + 8 * q4 + 4 * g);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              acc[db][0][4 * q4 + e] *= f4[e];
              acc[db][1][4 * q4 + e] *= f4[e];
            }
          }
        wave_lds_order();
      }
#pragma unroll
      for (int db = 0; db < 2; ++db) {
        const float mb = m_run[db] * kLog2e;
        uint4v pw;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          float e0 = __builtin_amdgcn_exp2f(__builtin_fmaf((float)ka[db][2 * j], kLog2e, -mb));
          float e1 = __builtin_amdgcn_exp2f(__builtin_fmaf((float)ka[db][2 * j + 1], kLog2e, -mb));
          if (dead[2 * j]) e0 = 0.f;
          if (dead[2 * j + 1]) e1 = 0.f;
          pw[j] = T::pack2(e0, e1);
          l_run[db] = T::add2(pw[j], l_run[db]);  // sum of the 16-bit values the MFMA consumes
        }
        ka[db] = __builtin_bit_cast(vec8, pw);
      }
    } else {
#pragma unroll
      for (int db = 0; db < 2; ++db)
#pragma unroll
        for (int s = 0; s < 8; ++s) {
          if (dead[s]) ka[db][s] = (typename T::elem)0.f;
          l_run[db] += __builtin_fabsf((float)ka[db][s]);
        }
    }
#pragma unroll
    for (int db = 0; db < 2; ++db)
#pragma unroll
      for (int eb = 0; eb < 2; ++eb) acc[db][eb] = T::mfma(ka[db], vb[eb], acc[db][eb]);
  };

  // strip i has been fetched into register slot SLOT: park it in LDS, refill the slot with strip i + P (past
  // the wave's share that re-reads its last row: see StripMover::limit_rows), then consume the parked strip
  auto step = [&](int i, auto slot_tag) {
    constexpr int SLOT = decltype(slot_tag)::value;
    const int t0 = strip_row0(i);
    const bool tail = t0 + STEP > p.S;
    wave_lds_order();
    mvK.to_lds(rk[SLOT], tk);
    mvV.to_lds(rv[SLOT], tv);
    if (NQ) {
      // a lane holds channels 8 (lane % 8) + [0..7] of rows lane / 8 (+ 8) of the strip
#pragma unroll
      for (int it = 0; it < R; ++it) {
        const vec8 qv = __builtin_bit_cast(vec8, mvQ.chunk16(rq[SLOT], it));
        const bool live = i < nmine && (!tail || t0 + it * 8 + (lane >> 3) < p.S);  // not a re-read row past the share
#pragma unroll
        for (int e = 0; e < 8; ++e) qabs[e] += live ? __builtin_fabsf((float)qv[e]) : 0.f;
      }
    }
    fetch(i + P, slot_tag);
    wave_lds_order();
    if (i < nmine) {
      if (tail)
        compute(std::true_type{}, t0);
      else
        compute(std::false_type{}, t0);
    }
  };

  // in this order (the scheduler is free to issue independent loads last-first, and loads complete in order: the
  // first step would then wait for all three strips, and so would, after the compiler merges the two ways into
  // the loop, every later one)
  fetch(0, std::integral_constant<int, 0>{});
  __builtin_amdgcn_sched_barrier(0);
  fetch(1, std::integral_constant<int, 1>{});
  __builtin_amdgcn_sched_barrier(0);
  if constexpr (P == 3) {
    fetch(2, std::integral_constant<int, 2>{});
    __builtin_amdgcn_sched_barrier(0);
  }
  // Whole trips of P steps (a step past the wave's share moves its re-read row and computes nothing): one
  // entry, one back edge and the same loads on every path, so that the compiler knows how many are in flight at
  // each step and waits for the oldest strip only.
  static_assert(P == 2 || P == 3, "the strip loop is unrolled over the register slots");
  for (int i = 0; i < nmine; i += P) {
    step(i, std::integral_constant<int, 0>{});
    step(i + 1, std::integral_constant<int, 1>{});
    if constexpr (P == 3) step(i + 2, std::integral_constant<int, 2>{});
  }

  // ---- combine the four waves
#pragma unroll
  for (int db = 0; db < 2; ++db) {
    l_run[db] += xchg32(l_run[db]);
    if (g == 0) {
      s_m[wave * D + 32 * db + n] = m_run[db];
      s_l[wave * D + 32 * db + n] = l_run[db];
    }
  }
  if (NQ) {
    // |Q| column sums: a lane holds channels 8 (lane % 8) + [0..7] of its row group; fold the 8 row groups
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      float s = qabs[e];
      s += __shfl_xor(s, 8);
      s += __shfl_xor(s, 16);
      s += __shfl_xor(s, 32);
      qabs[e] = s;
    }
    if (lane < 8) {
#pragma unroll
      for (int e = 0; e < 8; ++e) fac[lane * 8 + e] = qabs[e];
    }
  }
  __syncthreads();
  if (EA) {
    // bring every wave's matrix to the common per-channel maximum
#pragma unroll
    for (int db = 0; db < 2; ++db)
#pragma unroll
      for (int q4 = 0; q4 < 4; ++q4) {
        const int d0 = 32 * db + 8 * q4 + 4 * g;
        float4v mall = *reinterpret_cast<const float4v*>(s_m + d0);
#pragma unroll
        for (int w = 1; w < kLinWaves; ++w) {
          const float4v mw = *reinterpret_cast<const float4v*>(s_m + w * D + d0);
#pragma unroll
          for (int e = 0; e < 4; ++e) mall[e] = fmaxf(mall[e], mw[e]);
        }
        const float4v mine = *reinterpret_cast<const float4v*>(s_m + wave * D + d0);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const float f = __builtin_amdgcn_exp2f((mine[e] - mall[e]) * kLog2e);
          acc[db][0][4 * q4 + e] *= f;
          acc[db][1][4 * q4 + e] *= f;
        }
      }
  }
  // pairwise tree: waves 2, 3 -> waves 0, 1, then wave 1 -> wave 0
  float* xa = s_x[0];
  float* xb = s_x[1];
  auto put = [&](float* dst) {
#pragma unroll
    for (int db = 0; db < 2; ++db)
#pragma unroll
      for (int eb = 0; eb < 2; ++eb)
#pragma unroll
        for (int r = 0; r < 16; ++r) dst[((2 * db + eb) * 16 + r) * 64 + lane] = acc[db][eb][r];
  };
  auto add = [&](const float* src) {
#pragma unroll
    for (int db = 0; db < 2; ++db)
#pragma unroll
      for (int eb = 0; eb < 2; ++eb)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[db][eb][r] += src[((2 * db + eb) * 16 + r) * 64 + lane];
  };
  if (wave == 2) put(xa);
  if (wave == 3) put(xb);
  __syncthreads();
  if (wave == 0) add(xa);
  if (wave == 1) add(xb);
  __syncthreads();
  if (wave == 1) put(xa);
  __syncthreads();

  float* part = p.part + ((int64_t)bh * p.nch + ch) * kPartStride;
  if (wave == 0) {
    add(xa);
#pragma unroll
    for (int db = 0; db < 2; ++db)
#pragma unroll
      for (int eb = 0; eb < 2; ++eb)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int d = 32 * db + 8 * (r >> 2) + 4 * g + (r & 3);
          part[d * D + 32 * eb + n] = acc[db][eb][r];
        }
  } else if (wave == 1) {
    const int d = lane;
    if (EA) {
      float M = s_m[d];
#pragma unroll
      for (int w = 1; w < kLinWaves; ++w) M = fmaxf(M, s_m[w * D + d]);
      float L = 0.f;
#pragma unroll
      for (int w = 0; w < kLinWaves; ++w) L += __builtin_amdgcn_exp2f((s_m[w * D + d] - M) * kLog2e) * s_l[w * D + d];
      part[D * D + d] = M;
      part[D * D + D + d] = L;
    } else {
      float nk = 0.f, nq = 0.f;
#pragma unroll
      for (int w = 0; w < kLinWaves; ++w) {
        nk += s_l[w * D + d];
        if (NQ) nq += s_f[w * D + d];
      }
      part[D * D + d] = nk;
      part[D * D + D + d] = nq;
    }
  }
}

// ---------------------------------------------------------------------------------------------------
// One workgroup per (b, h, block of 16 output channels).
// T: type of the W operand pair written for the output pass: hi = T(x), lo = T((x - hi) 2^kLoShift), i.e. 22
// significant bits as fp16 + fp16 and 16 as bf16 + bf16
template <typename T> constexpr int kLoShift = __is_same(typename T::elem, _Float16) ? 11 : 8;

template <typename T, bool EA>
__global__ void __launch_bounds__(kLinThreads) linattn_merge_kernel(const LinParams p, int normalize_q) {
  constexpr int D = kLinD, EB = 16, TS = D + 8;
  __shared__ float s_scale[D];   // per-channel factor applied to the summed matrix
  __shared__ float s_big[D];     // EA: global max per channel
  __shared__ float s_w[16][D];   // EA: per-chunk weights exp(m_c - M), up to 16 chunks at a time
  __shared__ float s_red[kLinThreads];
  __shared__ __align__(16) uint16_t s_t[2][EB][TS];  // hi / lo, transposed for 16-byte row stores
  const int bh = blockIdx.x >> 2;
  const int qr = blockIdx.x & 3;
  const float* part = p.part + (int64_t)bh * p.nch * kPartStride;
  const int t = threadIdx.x;

  float accv[4] = {0.f, 0.f, 0.f, 0.f};
  int pidx[4], drow[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int idx = t + i * kLinThreads;  // d = idx / 16, e = 16 qr + idx % 16
    drow[i] = idx / EB;
    pidx[i] = drow[i] * D + EB * qr + idx % EB;
  }

  // per-channel statistics: four thread groups split the chunks, then fold through LDS
  const int sd = t & (D - 1), cg = t >> 6;
  const float* stat = part + D * D + sd;
  if (EA) {
    float M = -__builtin_inff();
    for (int c = cg; c < p.nch; c += 4) M = fmaxf(M, stat[c * kPartStride]);
    s_red[t] = M;
    __syncthreads();
    M = fmaxf(fmaxf(s_red[sd], s_red[D + sd]), fmaxf(s_red[2 * D + sd], s_red[3 * D + sd]));
    float L = 0.f;
    for (int c = cg; c < p.nch; c += 4)
      L += __builtin_amdgcn_exp2f((stat[c * kPartStride] - M) * kLog2e) * stat[c * kPartStride + D];
    __syncthreads();
    s_red[t] = L;
    __syncthreads();
    if (t < D) {
      s_scale[t] = 1.f / (s_red[t] + s_red[D + t] + s_red[2 * D + t] + s_red[3 * D + t]);
      s_big[t] = M;
    }
    __syncthreads();
  } else {
    float nk = 0.f, nq = 0.f;
    for (int c = cg; c < p.nch; c += 4) {
      nk += stat[c * kPartStride];
      nq += stat[c * kPartStride + D];
    }
    s_red[t] = nk;
    s_w[cg][sd] = nq;
    __syncthreads();
    if (t < D) {
      nk = s_red[t] + s_red[D + t] + s_red[2 * D + t] + s_red[3 * D + t];
      nq = s_w[0][t] + s_w[1][t] + s_w[2][t] + s_w[3][t];
      s_scale[t] = 1.f / (normalize_q ? nk * nq : nk);
    }
    __syncthreads();
  }
  // weighted sum of the chunk matrices, four chunks (16 independent loads per thread) at a time
  for (int c0 = 0; c0 < p.nch; c0 += 16) {
    const int cn = min(16, p.nch - c0);
    if (EA) {
      for (int i = t; i < cn * D; i += kLinThreads) {
        const int c = i / D, d = i % D;
        s_w[c][d] = __builtin_amdgcn_exp2f((part[(c0 + c) * kPartStride + D * D + d] - s_big[d]) * kLog2e);
      }
      __syncthreads();
    }
    for (int c = 0; c < cn; c += 4) {
      float v[4][4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int cc = c0 + min(c + u, cn - 1);
#pragma unroll
        for (int i = 0; i < 4; ++i) v[u][i] = part[cc * kPartStride + pidx[i]];
      }
#pragma unroll
      for (int u = 0; u < 4; ++u)
        if (c + u < cn) {
#pragma unroll
          for (int i = 0; i < 4; ++i) accv[i] += (EA ? s_w[c + u][drow[i]] : 1.f) * v[u][i];
        }
    }
    if (EA) __syncthreads();
  }
  float gmax = 0.f;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    // two heads of 32 channels side by side: the products between a channel of one and a channel of the other
    // are not part of either head's matrix
    if (p.half_heads && (drow[i] >> 5) != (qr >> 1)) accv[i] = 0.f;
    accv[i] *= s_scale[drow[i]];
    gmax = fmaxf(gmax, __builtin_fabsf(accv[i]));
  }
  // the block's maximum: inside each wave by lane exchanges, then one value per wave through LDS
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) gmax = fmaxf(gmax, __shfl_xor(gmax, o));
  __syncthreads();  // every use of s_red above is over
  if ((t & 63) == 0) s_red[t >> 6] = gmax;
  __syncthreads();
  gmax = fmaxf(fmaxf(s_red[0], s_red[1]), fmaxf(s_red[2], s_red[3]));
  static_assert(kLinThreads == 256, "four waves");
  // power-of-two scale that puts the largest entry of the block in [2^13, 2^14)
  int ex = 0;
  if (gmax > 0.f && gmax < __builtin_inff()) ex = 13 - (int)__builtin_floorf(__builtin_log2f(gmax));
  ex = max(-100, min(100, ex));
  const float scale = __builtin_ldexpf(1.f, ex);
  if (t == 0) p.winv[bh * 4 + qr] = __builtin_ldexpf(1.f, -ex);
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int idx = t + i * kLinThreads;
    const float x = accv[i] * scale;
    const uint16_t hi = T::from_float(x);
    const uint16_t lo = T::from_float((x - T::to_float(hi)) * (float)(1 << kLoShift<T>));
    s_t[0][idx % EB][drow[i]] = hi;
    s_t[1][idx % EB][drow[i]] = lo;
  }
  __syncthreads();
  {
    const int hl = t >> 7, e = (t & 127) >> 3, c = t & 7;
    uint16_t* w = p.w + (int64_t)bh * 2 * D * D + hl * D * D + (EB * qr + e) * D + c * 8;
    *reinterpret_cast<uint4v*>(w) = *reinterpret_cast<const uint4v*>(&s_t[hl][e][c * 8]);
  }
}

// ---------------------------------------------------------------------------------------------------
template <typename T, bool IN32, bool EA, bool F32OUT>
__global__ void __launch_bounds__(kLinThreads, 2) linattn_out_kernel(const LinParams p) {
  static_assert(!IN32 || __is_same(typename T::elem, _Float16), "fp32 tensors are rounded to fp16 operands");
  typedef typename T::vec8 vec8;
  constexpr int D = kLinD, SUB = 32;
  constexpr int P = 2;                           // Q strips in flight per wave
  constexpr int STRIP = SUB * 2 * D;             // 4 KB
  constexpr int R = SUB / 8;                     // 16-byte loads per lane and strip
  constexpr int OROW = F32OUT ? 272 : 144;       // padded output row in the transpose buffer (bytes)
  constexpr int SL = SUB * D * (F32OUT ? 4 : 2) / 1024;  // 16-byte row stores per strip and lane
  __shared__ __align__(16) char s_q[kLinWaves][STRIP];       // wave-private Q strip
  __shared__ __align__(16) char otr[kLinWaves * SUB * OROW]; // wave-private output transpose buffers

  const int lane = lane_id(), wave = wave_id();
  const int g = lane >> 5, n = lane & 31;
  char* ost = otr + wave * SUB * OROW;
  char* tq = s_q[wave];

  // Two ways to share the work.  out_wave_heads: a workgroup takes four adjacent heads of one token chunk, one
  // head per wave, every wave walking all strips of the chunk: with heads adjacent in memory the workgroup
  // then reads and writes 512 contiguous bytes per token instead of 128 (the DRAM pages of a token row are
  // touched by one workgroup at one time, not by sixteen at sixteen times).  Otherwise one head per
  // workgroup, the strips of the chunk dealt round-robin to the waves.
  int bh, ch, strip0, strip_step;
  if (p.out_wave_heads) {
    const int hq = p.H / kLinWaves, groups = p.B * hq;
    const int bg = blockIdx.x % groups;
    ch = blockIdx.x / groups;
    bh = (bg / hq) * p.H + (bg % hq) * kLinWaves + wave;
    strip0 = 0;
    strip_step = 1;
  } else {
    const int BH = p.B * p.H;
    bh = blockIdx.x % BH;
    ch = blockIdx.x / BH;
    strip0 = wave;
    strip_step = kLinWaves;
  }
  const int b = bh / p.H, h = bh % p.H;

  const int tok_begin = ch * p.out_tiles_per_chunk * kLinTile;
  const int tok_end = min(p.S, tok_begin + p.out_tiles_per_chunk * kLinTile);
  const int nsub = (tok_end - tok_begin + SUB - 1) / SUB;
  const int nmine = nsub > strip0 ? (nsub - strip0 + strip_step - 1) / strip_step : 0;

  float winv[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) winv[i] = p.winv[bh * 4 + i];
  // A operand: W^T[e][d], hi and lo, rows e = 32 eb + n, contraction slots d = 16 t + 8 g + [0..7]
  const uint16_t* w = p.w + (int64_t)bh * 2 * D * D;
  vec8 whi[2][4], wlo[2][4];
#pragma unroll
  for (int eb = 0; eb < 2; ++eb)
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      whi[eb][t] = *reinterpret_cast<const vec8*>(w + (32 * eb + n) * D + 16 * t + 8 * g);
      if (F32OUT) wlo[eb][t] = *reinterpret_cast<const vec8*>(w + D * D + (32 * eb + n) * D + 16 * t + 8 * g);
    }

  StripMover<SUB, kRowSwizzle, IN32> mvQ;
  mvQ.init(p.q + (b * p.sq.b + h * p.sq.h) * (IN32 ? 2 : 1), p.sq.s, p.S);
  constexpr int RL = IN32 ? 2 * R : R;
  uint4v rq[P][RL];  // strips in flight, indexed by compile-time slot
  auto strip_row0 = [&](int i) { return tok_begin + (strip0 + strip_step * i) * SUB; };
  mvQ.limit_rows(nmine > 0 ? strip_row0(nmine - 1) + SUB - 1 : tok_begin);
  __builtin_amdgcn_sched_barrier(0);  // scales and W, then strip 0, then strip 1: loads complete in the order they are issued
  mvQ.load(strip_row0(0), rq[0]);
  __builtin_amdgcn_sched_barrier(0);
  mvQ.load(strip_row0(1), rq[1]);
  // W has landed before the loop starts, the two strips (the 2 R loads issued after it) stay in flight.  Left to
  // the compiler, the wait for W sits inside the loop, in front of the MFMAs, where on every later trip it
  // waits for the strip requested a few instructions earlier instead.
  static_assert(P * R == 8, "the wait below counts the loads of the two strips");
  if (IN32)
    __builtin_amdgcn_s_waitcnt(0x4F70);  // vmcnt(16): fp32 strips take twice the loads
  else
    __builtin_amdgcn_s_waitcnt(0x0F78);  // vmcnt(8), every other counter at its maximum

  char* obase = static_cast<char*>(p.o) + (b * p.so.b + h * p.so.h) * (int64_t)(F32OUT ? 4 : 2);
  const int64_t orow_bytes = p.so.s * (int64_t)(F32OUT ? 4 : 2);

  // strip i has been fetched into register slot SLOT: park it in LDS, refill the slot with strip i + P (past
  // the wave's share that re-reads its last row: see StripMover::limit_rows), then consume the parked strip
  auto step = [&](int i, auto slot_tag) {
    constexpr int SLOT = decltype(slot_tag)::value;
    const int t0 = strip_row0(i);
    wave_lds_order();
    mvQ.to_lds(rq[SLOT], tq);
    mvQ.load(strip_row0(i + P), rq[SLOT]);
    wave_lds_order();
    if (i >= nmine) return;  // past the wave's share: the slot has been moved and refilled, nothing to compute

    // B operand: f(Q)^T, column = token n, same contraction slots
    vec8 qf[4];
#pragma unroll
    for (int t = 0; t < 4; ++t) qf[t] = read_row_chunk<D, vec8>(tq, n, 2 * t + g);

    // EA: softmax over the 64 channels of the token.  The operand is the fp16 value of exp(q - max); the
    // division by the row sum (taken over those rounded values) is applied to the fp32 result.
    // A lane holds channels 16 t + 8 g + [0..7]: t = 0, 1 lie in the first 32 channels, t = 2, 3 in the last 32.
    // With head_dim 32 those are two heads, each with its own maximum and sum.
    float inv[2] = {1.f, 1.f};
    if (EA) {
      float mx[2], sum[2] = {0.f, 0.f};
#pragma unroll
      for (int hf = 0; hf < 2; ++hf) mx[hf] = fmaxf(max8<T>(qf[2 * hf]), max8<T>(qf[2 * hf + 1]));
      if (!p.half_heads) mx[0] = mx[1] = fmaxf(mx[0], mx[1]);
      mx[0] = fmaxf(mx[0], xchg32(mx[0]));
      mx[1] = fmaxf(mx[1], xchg32(mx[1]));
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        const float mb = mx[t >> 1] * kLog2e;
        uint4v pw;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          pw[j] = T::pack2(__builtin_amdgcn_exp2f(__builtin_fmaf((float)qf[t][2 * j], kLog2e, -mb)),
                           __builtin_amdgcn_exp2f(__builtin_fmaf((float)qf[t][2 * j + 1], kLog2e, -mb)));
          sum[t >> 1] = T::add2(pw[j], sum[t >> 1]);
        }
        qf[t] = __builtin_bit_cast(vec8, pw);
      }
      if (!p.half_heads) sum[0] = sum[1] = sum[0] + sum[1];
      sum[0] += xchg32(sum[0]);
      sum[1] += xchg32(sum[1]);
      inv[0] = 1.f / sum[0];
      inv[1] = 1.f / sum[1];
    }

    // W as hi + lo / 2^11 only where the output can show the difference (fp32)
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
        ahi[eb] = T::mfma(whi[eb][t], qf[t], ahi[eb]);
        if (F32OUT) alo[eb] = T::mfma(wlo[eb][t], qf[t], alo[eb]);
      }
    float osc[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) osc[i] = winv[i] * inv[i >> 1];

    // accumulator (lane = token, registers = channels) -> padded [token][channel] rows in LDS
#pragma unroll
    for (int eb = 0; eb < 2; ++eb)
#pragma unroll
      for (int q4 = 0; q4 < 4; ++q4) {
        const int e0 = 32 * eb + 8 * q4 + 4 * g;
        float y[4];
#pragma unroll
        for (int e = 0; e < 4; ++e)
          y[e] = (F32OUT ? ahi[eb][4 * q4 + e] + alo[eb][4 * q4 + e] * (1.f / (float)(1 << kLoShift<T>)) : ahi[eb][4 * q4 + e]) * osc[2 * eb + (q4 >> 1)];
        if (F32OUT) {
          float4v o4 = {y[0], y[1], y[2], y[3]};
          *reinterpret_cast<float4v*>(ost + n * OROW + e0 * 4) = o4;
        } else {
          uint2 pk;
          pk.x = T::pack2(y[0], y[1]);
          pk.y = T::pack2(y[2], y[3]);
          *reinterpret_cast<uint2*>(ost + n * OROW + e0 * 2) = pk;
        }
      }
    wave_lds_order();
    // whole rows back out: 16 bytes per lane, 8 (fp16) or 16 (fp32) lanes per token
    constexpr int LPR = F32OUT ? 16 : 8;
#pragma unroll
    for (int j = 0; j < SL; ++j) {
      const int r = j * (64 / LPR) + lane / LPR;
      const int c = lane % LPR;
      const uint4v val = *reinterpret_cast<const uint4v*>(ost + r * OROW + c * 16);
      // streamed out once and not read again here: non-temporal, so that the lines do not linger dirty in
      // the caches and get written back under the next kernel's reads
      if (t0 + r < p.S) __builtin_nontemporal_store(val, reinterpret_cast<uint4v*>(obase + (int64_t)(t0 + r) * orow_bytes + c * 16));
    }
    wave_lds_order();
  };

  static_assert(P == 2, "the strip loop is unrolled over two register slots");
  for (int i = 0; i < nmine; i += 2) {  // whole trips, as in the K/V pass
    step(i, std::integral_constant<int, 0>{});
    step(i + 1, std::integral_constant<int, 1>{});
  }
}

template <typename T>
struct TypeTag {
  typedef T type;
};

// ---------------------------------------------------------------------------------------------------
hipError_t launch_linattn(const FtAttnArgs& a0, int kind, int normalize_q, int out_dtype, void* ws, hipStream_t s) {
  LinParams p;
  const FtAttnArgs a = lin_effective(a0, &p.half_heads);
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
  lin_plan(a, kKvWorkgroups, &p.nch, &p.tiles_per_chunk);
  lin_plan(a, kOutWorkgroups, &p.out_nch, &p.out_tiles_per_chunk);
  const bool ea = kind == FT_OP_EA;
  const bool nq = !ea && normalize_q;
  // Four heads per workgroup in the output pass (see the kernel) where Q comes from HBM: B8 H16 S8192, EA
  // 127.4 -> 121.2 us per call.  SimA with normalised queries has just read Q in its K/V pass and finds much of it
  // in the memory-side cache; there the one-head form is the faster by 1 us (126.6 vs 127.7) and stays.
  p.out_wave_heads = a.H % kLinWaves == 0 && !nq;
  if (p.out_wave_heads) {  // the same number of workgroups over a quarter as many (b, head group) pairs
    FtAttnArgs quarter = a;
    quarter.H = a.H / kLinWaves;
    lin_plan(quarter, kOutWorkgroups, &p.out_nch, &p.out_tiles_per_chunk);
  }
  const bool f32 = out_dtype == FT_F32;
  const size_t bh = (size_t)a.B * a.H;
  char* base = static_cast<char*>(ws);
  p.part = reinterpret_cast<float*>(base);
  base += bh * p.nch * kPartStride * sizeof(float);
  p.w = reinterpret_cast<uint16_t*>(base);
  base += bh * 2 * kLinD * kLinD * sizeof(uint16_t);
  p.winv = reinterpret_cast<float*>(base);

  const dim3 grid1((unsigned)(bh * p.nch)), grid3((unsigned)((p.out_wave_heads ? bh / kLinWaves : bh) * p.out_nch)), blk(kLinThreads);
  const dim3 grid2((unsigned)(bh * 4));
  hipError_t e = hipErrorInvalidValue;
  // T: operand type; IN32: fp32 tensors (fp32 output only)
  auto run = [&](auto t_tag, auto in32_tag) {
    typedef typename decltype(t_tag)::type T;
    constexpr bool IN32 = decltype(in32_tag)::value;
    if (ea)
      hipLaunchKernelGGL((linattn_kv_kernel<T, IN32, true, false>), grid1, blk, 0, s, p);
    else if (nq)
      hipLaunchKernelGGL((linattn_kv_kernel<T, IN32, false, true>), grid1, blk, 0, s, p);
    else
      hipLaunchKernelGGL((linattn_kv_kernel<T, IN32, false, false>), grid1, blk, 0, s, p);
    e = hipGetLastError();
    if (e != hipSuccess) return;
    if (ea)
      hipLaunchKernelGGL((linattn_merge_kernel<T, true>), grid2, blk, 0, s, p, 0);
    else
      hipLaunchKernelGGL((linattn_merge_kernel<T, false>), grid2, blk, 0, s, p, nq ? 1 : 0);
    e = hipGetLastError();
    if (e != hipSuccess) return;
    if constexpr (IN32) {
      if (ea)
        hipLaunchKernelGGL((linattn_out_kernel<T, true, true, true>), grid3, blk, 0, s, p);
      else
        hipLaunchKernelGGL((linattn_out_kernel<T, true, false, true>), grid3, blk, 0, s, p);
    } else if (ea) {
      if (f32)
        hipLaunchKernelGGL((linattn_out_kernel<T, false, true, true>), grid3, blk, 0, s, p);
      else
        hipLaunchKernelGGL((linattn_out_kernel<T, false, true, false>), grid3, blk, 0, s, p);
    } else {
      if (f32)
        hipLaunchKernelGGL((linattn_out_kernel<T, false, false, true>), grid3, blk, 0, s, p);
      else
        hipLaunchKernelGGL((linattn_out_kernel<T, false, false, false>), grid3, blk, 0, s, p);
    }
    e = hipGetLastError();
  };
  if (a.dtype == FT_F32)
    run(TypeTag<F16>{}, std::true_type{});
  else if (a.dtype == FT_BF16)
    run(TypeTag<BF16>{}, std::false_type{});
  else
    run(TypeTag<F16>{}, std::false_type{});
  return e;
}

}  // namespace ft
