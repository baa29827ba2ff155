// The whole block of bench/ea.mlir / bench/sima.mlir (q/k/v Linear :3-5, heads :6-12, core :13-17, output Linear
// :20-22) in two launches for narrow models: C = H * 32 <= 128 channels, the geometry of the .mlir itself
// (x [64,784,128], 4 heads of 32).  With so few channels the projection weights fit in LDS and a token's q, k, v never
// leave the registers they are computed in, so x is read twice and y written once; nothing else touches HBM but a
// few MB of per-chunk partial matrices.  x and y pass through a wave-private LDS tile on the way in and out, so that
// every load and store instruction covers whole 128- or 256-byte row segments.
//
//   pass 1 (linblk_kv_kernel), one workgroup per (batch, token chunk), a wave per strip of 32 tokens:
//     K = x Wk^T + bk and V = x Wv^T + bv with the tokens as MFMA rows, so that a lane ends up holding one channel
//     and 16 tokens of each: exactly the operand form of the next contraction, whose sum runs over tokens.
//     KV^T[e][d] += sum_t V[t][e] Ks[t][d]: the lane of the result holds column d, so EA's running maximum of
//     K[:, d] (softmax over the tokens) rescales the lane's own registers, nothing crosses lanes.
//     The waves are folded through LDS and the chunk's matrix, maxima and sums go to the workspace.
//   pass 2 (linblk_out_kernel), same grid: every workgroup first merges its batch's chunk matrices (a wave per head)
//     into normalised hi + lo 16-bit operand pairs, then per strip: Q^T = Wq x^T + bq with the tokens as MFMA
//     columns (a lane holds one token and 16 channels of a head: EA's softmax over the head's channels is in-lane
//     plus one exchange), O^T = KVn^T Qs^T, y^T = Wo O^T + bo, again feeding accumulators straight back as operands.
//
// Operand convention (v_mfma_f32_32x32x16): a lane supplies row / column l % 32 and contraction slots 8 g + i,
// g = l / 32, i < 8.  Registers 8 s + i of a 32x32 accumulator (rows 16 s + 8 (i / 4) + 4 g + i % 4 of the lane's
// column) become the slots of step s of the next product; the other operand is built in the same order (from an
// accumulator of the same shape, or by permuting the columns of Wo when it is staged).
#include <hip/hip_runtime.h>

#include <algorithm>
#include <type_traits>

#include "../../include/ft_abi.h"
#include "device_common.hpp"

namespace ft {

constexpr int kSbThreads = 512, kSbWaves = 8, kSbStrip = 32;
constexpr int kSbPart = 32 * 32 + 3 * 32;  // per (batch, chunk, head): KV [d][e], then m or unused, l or sum|K|, sum|Q|
constexpr int kSbMaxChunks = 4;

struct SmallBlockParams {
  const void* x;
  const void* w_qkv;
  const void* b_qkv;
  const void* w_out;
  const void* b_out;
  void* y;
  float* part;
  int B, S, nch, strips_per_chunk, normalize_q;
};

namespace {

template <typename T> constexpr int kSbLoShift = __is_same(typename T::elem, _Float16) ? 11 : 8;

template <typename T, bool IN32>
__device__ __forceinline__ uint4v load8(const void* base, int64_t elem) {
  if constexpr (IN32) {
    const float4v* p = reinterpret_cast<const float4v*>(static_cast<const float*>(base) + elem);
    const float4v lo = p[0], hi = p[1];
    const uint4v out = {T::pack2(lo[0], lo[1]), T::pack2(lo[2], lo[3]), T::pack2(hi[0], hi[1]), T::pack2(hi[2], hi[3])};
    return out;
  } else {
    return *reinterpret_cast<const uint4v*>(static_cast<const uint16_t*>(base) + elem);
  }
}

// A 32-token strip of x on its way to a wave: requested one strip ahead with loads that cover whole rows (lane l takes
// a 16-byte chunk of row l / CPR + RPI i: an instruction touches 8 cache lines; with every lane reading its own
// token's row it touched 32, and the address path showed), parked in the wave's LDS tile when the strip's turn comes
// (16-bit elements, the chunk placement of TileGeom's kRowSwizzle) and read back as MFMA operands: token l % 32,
// channels 16 s + 8 g + [0..7] for step s.
template <typename T, bool IN32, int C>
struct XStrip {
  typedef TileGeom<C> G;
  static constexpr int CPR = C * (IN32 ? 4 : 2) / 16;  // 16-byte chunks per row in memory
  static constexpr int RPI = 64 / CPR;                 // rows per load instruction
  static constexpr int N = kSbStrip / RPI;
  static constexpr int kTileBytes = kSbStrip * G::RB;
  uint4v raw[N];
  // tok0: first token of the strip; rows past `last` (the batch's last token) re-read it
  __device__ __forceinline__ void load(const void* x, int64_t batch_row0, int tok0, int last) {
    const int lane = lane_id();
#pragma unroll
    for (int i = 0; i < N; ++i) {
      const int64_t r = batch_row0 + min(tok0 + lane / CPR + RPI * i, last);
      raw[i] = *reinterpret_cast<const uint4v*>(static_cast<const char*>(x) + (r * CPR + lane % CPR) * 16);
    }
  }
  __device__ __forceinline__ void to_lds(char* tile) const {
    const int lane = lane_id();
#pragma unroll
    for (int i = 0; i < N; ++i) {
      const int r = lane / CPR + RPI * i, c = lane % CPR;
      if constexpr (IN32) {  // 4 floats -> half a 16-byte chunk of 16-bit elements
        const float4v v = __builtin_bit_cast(float4v, raw[i]);
        *reinterpret_cast<uint2*>(tile + r * G::RB + (((c >> 1) ^ G::row_swz(r)) << 4) + 8 * (c & 1)) =
            make_uint2(T::pack2(v[0], v[1]), T::pack2(v[2], v[3]));
      } else {
        *reinterpret_cast<uint4v*>(tile + r * G::RB + ((c ^ G::row_swz(r)) << 4)) = raw[i];
      }
    }
  }
  __device__ __forceinline__ typename T::vec8 operand(const char* tile, int s) const {
    const int lane = lane_id();
    return read_row_chunk<C, typename T::vec8>(tile, lane & 31, 2 * s + (lane >> 5));
  }
};

// The same without the LDS tile, for the one kernel whose weights leave no room for it (three matrices of 128 rows):
// every lane reads its own token's row and keeps it.
template <typename T, bool IN32, int C>
struct XStripLane {
  static constexpr int KS = C / 16;
  static constexpr int N = IN32 ? 2 * KS : KS;
  static constexpr int kTileBytes = 0;
  uint4v raw[N];
  __device__ __forceinline__ void load(const void* x, int64_t batch_row0, int tok0, int last) {
    const int lane = lane_id();
    const int64_t elem0 = (batch_row0 + min(tok0 + (lane & 31), last)) * C + 8 * (lane >> 5);
#pragma unroll
    for (int i = 0; i < N; ++i) {
      if (IN32)
        raw[i] = *reinterpret_cast<const uint4v*>(static_cast<const float*>(x) + elem0 + 16 * (i >> 1) + 4 * (i & 1));
      else
        raw[i] = *reinterpret_cast<const uint4v*>(static_cast<const uint16_t*>(x) + elem0 + 16 * i);
    }
  }
  __device__ __forceinline__ void to_lds(char*) const {}
  __device__ __forceinline__ typename T::vec8 operand(const char*, int s) const {
    if constexpr (IN32) {
      const float4v lo = __builtin_bit_cast(float4v, raw[2 * s]), hi = __builtin_bit_cast(float4v, raw[2 * s + 1]);
      const uint4v v = {T::pack2(lo[0], lo[1]), T::pack2(lo[2], lo[3]), T::pack2(hi[0], hi[1]), T::pack2(hi[2], hi[3])};
      return __builtin_bit_cast(typename T::vec8, v);
    } else {
      return __builtin_bit_cast(typename T::vec8, raw[s]);
    }
  }
};

// rows [row0, row0 + nrows) of a row-major [*, C] matrix into LDS rows of WS bytes (16-bit elements); PERM: the four
// 4-column quads of every 16 columns in the order 0, 2, 1, 3 (the slot order of an accumulator used as operand)
template <typename T, bool IN32, int C, int WS, bool PERM>
__device__ __forceinline__ void stage_rows(char* dst, const void* src, int row0, int nrows) {
  constexpr int CH = C / 8;  // 16-byte chunks per row
  constexpr int U = 16;      // loads in flight per thread: the copy is a chain of L2 latencies otherwise
  const int total = nrows * CH;
  for (int i0 = threadIdx.x; i0 < total; i0 += U * kSbThreads) {
    uint4v v[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int i = min(i0 + u * kSbThreads, total - 1);
      v[u] = load8<T, IN32>(src, (int64_t)(row0 + i / CH) * C + 8 * (i % CH));
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int i = i0 + u * kSbThreads;
      if (i >= total) break;
      const int r = i / CH, c = i % CH;
      if (PERM) {
        // chunk c holds quads 2 (c % 2), 2 (c % 2) + 1 of its 16-column group; quad q goes to place (q % 2) * 2 + q / 2
        const int grp = c >> 1, q0 = 2 * (c & 1);
        char* row = dst + r * WS + grp * 32;
        *reinterpret_cast<uint2*>(row + 8 * ((q0 & 1) * 2 + (q0 >> 1))) = make_uint2(v[u][0], v[u][1]);
        *reinterpret_cast<uint2*>(row + 8 * (((q0 + 1) & 1) * 2 + ((q0 + 1) >> 1))) = make_uint2(v[u][2], v[u][3]);
      } else {
        *reinterpret_cast<uint4v*>(dst + r * WS + 16 * c) = v[u];
      }
    }
  }
}

template <typename T, bool IN32>
__device__ __forceinline__ void stage_bias(float* dst, const void* src, int i0, int n) {
  for (int i = threadIdx.x; i < n; i += kSbThreads) {
    float v = 0.f;
    if (src) v = IN32 ? static_cast<const float*>(src)[i0 + i] : T::to_float(static_cast<const uint16_t*>(src)[i0 + i]);
    dst[i] = v;
  }
}

// value as the 16-bit tensor between two stages of the block would hold it (fp32 tensors: unchanged)
template <typename T, bool IN32>
__device__ __forceinline__ float stage_round(float x) {
  return IN32 ? x : T::to_float(T::from_float(x));
}

template <typename T>
__device__ __forceinline__ typename T::vec8 as_operand(const uint32_t (&w)[8], int s) {
  const uint4v v = {w[4 * s], w[4 * s + 1], w[4 * s + 2], w[4 * s + 3]};
  return __builtin_bit_cast(typename T::vec8, v);
}

}  // namespace

// ---------------------------------------------------------------------------------------------------
template <typename T, bool IN32, int H, bool EA, bool NQ>
__global__ void __launch_bounds__(kSbThreads) linblk_kv_kernel(const SmallBlockParams p) {
  typedef typename T::vec8 vec8;
  constexpr int C = 32 * H, KS = C / 16, WS = 2 * C + 16;
  constexpr int NW = NQ ? 3 : 2;  // matrices staged: [Wq,] Wk, Wv (rows of w_qkv in that order)
  typedef typename std::conditional<NQ && H == 4, XStripLane<T, IN32, C>, XStrip<T, IN32, C>>::type XS;
  constexpr int kFoldBytes = kSbWaves * H * 16 * 64 * 4;
  constexpr int kWBytes = NW * C * WS, kXBytes = kSbWaves * XS::kTileBytes;
  // weights, then the waves' x tiles; the fold at the end reuses all of it
  __shared__ __align__(16) char s_w[kWBytes + kXBytes > kFoldBytes ? kWBytes + kXBytes : kFoldBytes];
  __shared__ float s_b[NW * C];
  __shared__ float s_stat[kSbWaves][H][3][32];

  const int b = blockIdx.x % p.B, ch = blockIdx.x / p.B;
  const int lane = lane_id(), wave = wave_id();
  const int g = lane >> 5, n = lane & 31;
  const float NEG_INF = -__builtin_inff();

  // the wave's strips: chunk's first + wave, + kSbWaves, ...; the first one is requested before anything else
  const int nstrips = (p.S + kSbStrip - 1) / kSbStrip;
  const int strip_end = min(nstrips, (ch + 1) * p.strips_per_chunk);
  int strip = ch * p.strips_per_chunk + wave;
  XS xs;
  char* xtile = s_w + kWBytes + wave * XS::kTileBytes;
  xs.load(p.x, (int64_t)b * p.S, min(strip, nstrips - 1) * kSbStrip, p.S - 1);

  stage_rows<T, IN32, C, WS, false>(s_w, p.w_qkv, NQ ? 0 : C, NW * C);
  stage_bias<T, IN32>(s_b, p.b_qkv, NQ ? 0 : C, NW * C);
  __syncthreads();
  const char* wq = s_w;                         // NQ only
  const char* wk = s_w + (NQ ? C * WS : 0);
  const char* wv = wk + C * WS;
  const float* bq = s_b;
  const float* bk = s_b + (NQ ? C : 0);
  const float* bv = bk + C;

  float16v acc[H];  // KV^T of head h: column d = 32 h + n, rows e in register order
  float m_run[H], l_run[H], nq_run[H];
#pragma unroll
  for (int h = 0; h < H; ++h) {
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[h][r] = 0.f;
    m_run[h] = NEG_INF;
    l_run[h] = 0.f;
    nq_run[h] = 0.f;
  }

  for (; strip < strip_end; strip += kSbWaves) {
    const int t0 = strip * kSbStrip;
    vec8 xa[KS];
    xs.to_lds(xtile);
    wave_lds_order();
#pragma unroll
    for (int s = 0; s < KS; ++s) xa[s] = xs.operand(xtile, s);
    wave_lds_order();
    // the next strip (past the wave's share: any valid rows, unused); fp32 rows take twice the registers while they
    // are in flight and are requested after the strip's work instead, where fewer are live
    if (!IN32) xs.load(p.x, (int64_t)b * p.S, min(strip + kSbWaves, nstrips - 1) * kSbStrip, p.S - 1);
    bool dead[16];  // token of register r lies past the end
#pragma unroll
    for (int r = 0; r < 16; ++r) dead[r] = t0 + 8 * (r >> 2) + 4 * g + (r & 3) >= p.S;

#pragma unroll
    for (int h = 0; h < H; ++h) {
      // (the weights never change, and the compiler would lift every fragment of every head out of the strip loop
      // into registers it does not have: the row offset is made opaque once per strip and head)
      int wrow = (32 * h + n) * WS + 16 * g;
      asm volatile("" : "+v"(wrow));
      if (NQ) {
        float16v qacc;
#pragma unroll
        for (int r = 0; r < 16; ++r) qacc[r] = 0.f;
#pragma unroll
        for (int s = 0; s < KS; ++s)
          qacc = T::mfma(xa[s], *reinterpret_cast<const vec8*>(wq + wrow + 32 * s), qacc);
        const float bqn = bq[32 * h + n];
        float sum = 0.f;
#pragma unroll
        for (int r = 0; r < 16; ++r) sum += dead[r] ? 0.f : __builtin_fabsf(stage_round<T, IN32>(qacc[r] + bqn));
        nq_run[h] += sum;
      }
      float16v kacc, vacc;
#pragma unroll
      for (int r = 0; r < 16; ++r) kacc[r] = vacc[r] = 0.f;
#pragma unroll
      for (int s = 0; s < KS; ++s) {
        kacc = T::mfma(xa[s], *reinterpret_cast<const vec8*>(wk + wrow + 32 * s), kacc);
        vacc = T::mfma(xa[s], *reinterpret_cast<const vec8*>(wv + wrow + 32 * s), vacc);
      }
      const float bkn = bk[32 * h + n], bvn = bv[32 * h + n];
      float kf[16];
      uint32_t kw[8], vw[8];
#pragma unroll
      for (int r = 0; r < 16; ++r) kf[r] = stage_round<T, IN32>(kacc[r] + bkn);
#pragma unroll
      for (int j = 0; j < 8; ++j) vw[j] = T::pack2(vacc[2 * j] + bvn, vacc[2 * j + 1] + bvn);
      if (EA) {
        float mx = NEG_INF;
#pragma unroll
        for (int r = 0; r < 16; ++r) mx = fmaxf(mx, dead[r] ? NEG_INF : kf[r]);
        mx = fmaxf(mx, xchg32(mx));  // the other 16 tokens of the channel
        const float m_new = fmaxf(m_run[h], mx);
        const float f = __builtin_amdgcn_exp2f((m_run[h] - m_new) * kLog2e);
        m_run[h] = m_new;
        l_run[h] *= f;
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[h][r] *= f;
        const float mb = m_new * kLog2e;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          float e0 = __builtin_amdgcn_exp2f(__builtin_fmaf(kf[2 * j], kLog2e, -mb));
          float e1 = __builtin_amdgcn_exp2f(__builtin_fmaf(kf[2 * j + 1], kLog2e, -mb));
          if (dead[2 * j]) e0 = 0.f;
          if (dead[2 * j + 1]) e1 = 0.f;
          kw[j] = T::pack2(e0, e1);
          l_run[h] = T::add2(kw[j], l_run[h]);  // the sum of what the MFMA consumes
        }
      } else {
        float sum = 0.f;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          if (dead[r]) kf[r] = 0.f;
          sum += __builtin_fabsf(kf[r]);
        }
        l_run[h] += sum;
#pragma unroll
        for (int j = 0; j < 8; ++j) kw[j] = T::pack2(kf[2 * j], kf[2 * j + 1]);
      }
#pragma unroll
      for (int s = 0; s < 2; ++s) acc[h] = T::mfma(as_operand<T>(vw, s), as_operand<T>(kw, s), acc[h]);
    }
    if (IN32) xs.load(p.x, (int64_t)b * p.S, min(strip + kSbWaves, nstrips - 1) * kSbStrip, p.S - 1);
  }

  // ---- fold the waves (wave h merges head h), write the chunk's partial
  __syncthreads();  // every wave is done with the weights
  float* fold = reinterpret_cast<float*>(s_w);
#pragma unroll
  for (int h = 0; h < H; ++h) {
    l_run[h] += xchg32(l_run[h]);
    nq_run[h] += xchg32(nq_run[h]);
#pragma unroll
    for (int r = 0; r < 16; ++r) fold[((wave * H + h) * 16 + r) * 64 + lane] = acc[h][r];
    if (g == 0) {
      s_stat[wave][h][0][n] = m_run[h];
      s_stat[wave][h][1][n] = l_run[h];
      s_stat[wave][h][2][n] = nq_run[h];
    }
  }
  __syncthreads();
  if (wave < H) {
    const int h = wave;
    float M = NEG_INF, L = 0.f, NQs = 0.f;
    float wgt[kSbWaves];
    if (EA) {
#pragma unroll
      for (int w = 0; w < kSbWaves; ++w) M = fmaxf(M, s_stat[w][h][0][n]);
    }
#pragma unroll
    for (int w = 0; w < kSbWaves; ++w) {
      // a wave that had no strip reports -inf and zeros; M is finite as soon as one wave had one
      wgt[w] = EA ? (s_stat[w][h][0][n] == NEG_INF ? 0.f : __builtin_amdgcn_exp2f((s_stat[w][h][0][n] - M) * kLog2e)) : 1.f;
      L += wgt[w] * s_stat[w][h][1][n];
      NQs += s_stat[w][h][2][n];
    }
    float16v sum;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      float v = 0.f;
#pragma unroll
      for (int w = 0; w < kSbWaves; ++w) v += wgt[w] * fold[((w * H + h) * 16 + r) * 64 + lane];
      sum[r] = v;
    }
    float* part = p.part + (((int64_t)b * p.nch + ch) * H + h) * kSbPart;
    // row d = n of KV [d][e]; registers 4 q + [0..3] are e = 8 q + 4 g + [0..3]
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const float4v v = {sum[4 * q], sum[4 * q + 1], sum[4 * q + 2], sum[4 * q + 3]};
      *reinterpret_cast<float4v*>(part + n * 32 + 8 * q + 4 * g) = v;
    }
    if (g == 0) {
      part[1024 + n] = M;
      part[1024 + 32 + n] = L;
      part[1024 + 64 + n] = NQs;
    }
  }
}

// ---------------------------------------------------------------------------------------------------
template <typename T, bool IN32, int H, bool EA>
__global__ void __launch_bounds__(kSbThreads) linblk_out_kernel(const SmallBlockParams p) {
  typedef typename T::vec8 vec8;
  constexpr int C = 32 * H, KS = C / 16, WS = 2 * C + 16;
  typedef XStrip<T, IN32, C> XS;
  constexpr int ES = IN32 ? 4 : 2;        // bytes per element of y
  constexpr int YCH = 128 / ES;           // output channels per store round: 128 bytes of every token's row
  constexpr int YROW = 144;               // row of the transposition buffer (bytes)
  constexpr int kXTile = XS::kTileBytes > kSbStrip * YROW ? XS::kTileBytes : kSbStrip * YROW;  // the y rounds reuse the wave's x tile
  __shared__ __align__(16) char s_wq[C * WS];
  __shared__ __align__(16) char s_wo[C * WS];             // columns in operand slot order
  __shared__ __align__(16) char s_x[kSbWaves * kXTile];
  __shared__ __align__(16) float s_bq[C];
  __shared__ __align__(16) float s_bo[C];
  __shared__ __align__(16) uint4v s_kv[H][2][2][64];      // [head][hi, lo][step][lane]: operand of O^T = KVn^T Qs^T
  __shared__ float s_wgt[H][kSbMaxChunks][32];           // weight of chunk c in row d of the merged matrix
  __shared__ float s_winv[H];

  const int b = blockIdx.x % p.B, ch = blockIdx.x / p.B;
  const int lane = lane_id(), wave = wave_id();
  const int g = lane >> 5, n = lane & 31;
  const float NEG_INF = -__builtin_inff();

  const int nstrips = (p.S + kSbStrip - 1) / kSbStrip;
  const int strip_end = min(nstrips, (ch + 1) * p.strips_per_chunk);
  int strip = ch * p.strips_per_chunk + wave;
  XS xs;
  char* xtile = s_x + wave * kXTile;
  xs.load(p.x, (int64_t)b * p.S, min(strip, nstrips - 1) * kSbStrip, p.S - 1);

  stage_rows<T, IN32, C, WS, false>(s_wq, p.w_qkv, 0, C);
  stage_rows<T, IN32, C, WS, true>(s_wo, p.w_out, 0, C);
  stage_bias<T, IN32>(s_bq, p.b_qkv, 0, C);
  stage_bias<T, IN32>(s_bo, p.b_out, 0, C);

  // ---- merge this batch's chunk matrices: wave h takes head h
  if (wave < H) {
    const int h = wave;
    const float* part = p.part + ((int64_t)b * p.nch * H + h) * kSbPart;  // chunk c: + c * H * kSbPart
    const int64_t cstride = (int64_t)H * kSbPart;
    // (loops over all kSbMaxChunks slots, the ones past nch re-reading the last chunk with weight 0: every load of
    // the merge is then independent of the others, and the matrix entries are requested before the statistics that
    // weigh them are worked on: one memory latency for the whole merge)
    // lane (e = n, g): slots i of step s are rows d = 16 s + 8 (i / 4) + 4 g + i % 4
    float raw[16][kSbMaxChunks];
#pragma unroll
    for (int k = 0; k < 16; ++k) {
      const int d = 16 * (k >> 3) + 8 * ((k >> 2) & 1) + 4 * g + (k & 3);
#pragma unroll
      for (int c = 0; c < kSbMaxChunks; ++c) raw[k][c] = part[min(c, p.nch - 1) * cstride + d * 32 + n];
    }
    if (g == 0) {  // row d = n: weights of the chunks
      float mc[kSbMaxChunks], lc[kSbMaxChunks], qc[kSbMaxChunks];
#pragma unroll
      for (int c = 0; c < kSbMaxChunks; ++c) {
        const float* st = part + min(c, p.nch - 1) * cstride + 1024 + n;
        mc[c] = st[0];
        lc[c] = st[32];
        qc[c] = st[64];
      }
      float M = NEG_INF, L = 0.f, NQs = 0.f;
#pragma unroll
      for (int c = 0; c < kSbMaxChunks; ++c)
        if (EA && c < p.nch) M = fmaxf(M, mc[c]);
      float w[kSbMaxChunks];
#pragma unroll
      for (int c = 0; c < kSbMaxChunks; ++c) {
        w[c] = c >= p.nch ? 0.f : EA ? (mc[c] == NEG_INF ? 0.f : __builtin_amdgcn_exp2f((mc[c] - M) * kLog2e)) : 1.f;
        L += w[c] * lc[c];
        NQs += c < p.nch ? qc[c] : 0.f;
      }
      const float inv = 1.f / (!EA && p.normalize_q ? L * NQs : L);
#pragma unroll
      for (int c = 0; c < kSbMaxChunks; ++c) s_wgt[h][c][n] = w[c] * inv;
    }
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_s_waitcnt(0xC07F);  // the wave's own LDS writes have landed (lgkmcnt(0))
    float val[16];
    float gmax = 0.f;
#pragma unroll
    for (int k = 0; k < 16; ++k) {
      const int d = 16 * (k >> 3) + 8 * ((k >> 2) & 1) + 4 * g + (k & 3);
      float v = 0.f;
#pragma unroll
      for (int c = 0; c < kSbMaxChunks; ++c) v += s_wgt[h][c][d] * raw[k][c];
      val[k] = v;
      gmax = fmaxf(gmax, __builtin_fabsf(v));
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) gmax = fmaxf(gmax, __shfl_xor(gmax, o));
    // power-of-two scale that puts the largest entry in [2^13, 2^14): SimA's entries are ~1 / S^2
    int ex = 0;
    if (gmax > 0.f && gmax < __builtin_inff()) ex = 13 - (int)__builtin_floorf(__builtin_log2f(gmax));
    ex = max(-100, min(100, ex));
    const float scale = __builtin_ldexpf(1.f, ex);
    uint32_t hi[8], lo[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const float a0 = val[2 * j] * scale, a1 = val[2 * j + 1] * scale;
      hi[j] = T::pack2(a0, a1);
      lo[j] = T::pack2((a0 - T::lo(hi[j])) * (float)(1 << kSbLoShift<T>), (a1 - T::hi(hi[j])) * (float)(1 << kSbLoShift<T>));
    }
#pragma unroll
    for (int s = 0; s < 2; ++s) {
      s_kv[h][0][s][lane] = uint4v{hi[4 * s], hi[4 * s + 1], hi[4 * s + 2], hi[4 * s + 3]};
      s_kv[h][1][s][lane] = uint4v{lo[4 * s], lo[4 * s + 1], lo[4 * s + 2], lo[4 * s + 3]};
    }
    if (lane == 0) s_winv[h] = __builtin_ldexpf(1.f, -ex);
  }
  __syncthreads();

  for (; strip < strip_end; strip += kSbWaves) {
    const int t0 = strip * kSbStrip;
    const int tok = t0 + n;
    vec8 xb[KS];
    xs.to_lds(xtile);
    wave_lds_order();
#pragma unroll
    for (int s = 0; s < KS; ++s) xb[s] = xs.operand(xtile, s);
    wave_lds_order();
    xs.load(p.x, (int64_t)b * p.S, min(strip + kSbWaves, nstrips - 1) * kSbStrip, p.S - 1);

    vec8 of[H][2];  // O^T of head h as operand of the output projection
#pragma unroll
    for (int h = 0; h < H; ++h) {
      float16v qacc;
#pragma unroll
      for (int r = 0; r < 16; ++r) qacc[r] = 0.f;
      int wrow = (32 * h + n) * WS + 16 * g;  // opaque per strip and head: see the K/V pass
      asm volatile("" : "+v"(wrow));
#pragma unroll
      for (int s = 0; s < KS; ++s) qacc = T::mfma(*reinterpret_cast<const vec8*>(s_wq + wrow + 32 * s), xb[s], qacc);
      float qf[16];
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const float4v b4 = *reinterpret_cast<const float4v*>(s_bq + 32 * h + 8 * q + 4 * g);
#pragma unroll
        for (int e = 0; e < 4; ++e) qf[4 * q + e] = stage_round<T, IN32>(qacc[4 * q + e] + b4[e]);
      }
      if (EA) {  // softmax over the head's 32 channels: 16 here, 16 in the partner lane
        float mx = qf[0];
#pragma unroll
        for (int r = 1; r < 16; ++r) mx = fmaxf(mx, qf[r]);
        mx = fmaxf(mx, xchg32(mx));
        float sum = 0.f;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          qf[r] = __builtin_amdgcn_exp2f((qf[r] - mx) * kLog2e);
          sum += qf[r];
        }
        sum += xchg32(sum);
        const float inv = 1.f / sum;
#pragma unroll
        for (int r = 0; r < 16; ++r) qf[r] *= inv;
      }
      uint32_t qw[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) qw[j] = T::pack2(qf[2 * j], qf[2 * j + 1]);
      float16v ohi, olo;
#pragma unroll
      for (int r = 0; r < 16; ++r) ohi[r] = olo[r] = 0.f;
      int kvl = lane;
      asm volatile("" : "+v"(kvl));
#pragma unroll
      for (int s = 0; s < 2; ++s) {
        ohi = T::mfma(__builtin_bit_cast(vec8, s_kv[h][0][s][kvl]), as_operand<T>(qw, s), ohi);
        olo = T::mfma(__builtin_bit_cast(vec8, s_kv[h][1][s][kvl]), as_operand<T>(qw, s), olo);
      }
      const float winv = s_winv[h];
      uint32_t ow[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const float o0 = (ohi[2 * j] + olo[2 * j] * (1.f / (float)(1 << kSbLoShift<T>))) * winv;
        const float o1 = (ohi[2 * j + 1] + olo[2 * j + 1] * (1.f / (float)(1 << kSbLoShift<T>))) * winv;
        ow[j] = T::pack2(o0, o1);
      }
      of[h][0] = as_operand<T>(ow, 0);
      of[h][1] = as_operand<T>(ow, 1);
    }

    // y^T block cb: rows = output channels 32 cb + [0..32), column = this lane's token.  The blocks of 128 bytes of
    // every token's row are turned round in the wave's LDS tile (x is in registers by now) and leave as 16-byte
    // pieces of whole 128-byte row segments, 8 rows per store instruction.
#pragma unroll
    for (int cb = 0; cb < H; ++cb) {
      float16v yacc;
#pragma unroll
      for (int r = 0; r < 16; ++r) yacc[r] = 0.f;
      int orow = (32 * cb + n) * WS + 16 * g;
      asm volatile("" : "+v"(orow));
#pragma unroll
      for (int h = 0; h < H; ++h)
#pragma unroll
        for (int s = 0; s < 2; ++s)
          yacc = T::mfma(*reinterpret_cast<const vec8*>(s_wo + orow + 64 * h + 32 * s), of[h][s], yacc);
      const int cin = (32 * cb) % YCH;  // first channel of the block inside its round
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const float4v b4 = *reinterpret_cast<const float4v*>(s_bo + 32 * cb + 8 * q + 4 * g);
        char* at = xtile + n * YROW + (cin + 8 * q + 4 * g) * ES;
        if constexpr (IN32) {
          const float4v v = {yacc[4 * q] + b4[0], yacc[4 * q + 1] + b4[1], yacc[4 * q + 2] + b4[2], yacc[4 * q + 3] + b4[3]};
          *reinterpret_cast<float4v*>(at) = v;
        } else {
          *reinterpret_cast<uint2*>(at) = make_uint2(T::pack2(yacc[4 * q] + b4[0], yacc[4 * q + 1] + b4[1]),
                                                    T::pack2(yacc[4 * q + 2] + b4[2], yacc[4 * q + 3] + b4[3]));
        }
      }
      if ((32 * cb + 32) % YCH == 0) {  // a round is complete
        const int c0 = 32 * cb + 32 - YCH;  // its first channel
        wave_lds_order();
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int r = 8 * i + (lane >> 3);
          const uint4v v = *reinterpret_cast<const uint4v*>(xtile + r * YROW + 16 * (lane & 7));
          if (t0 + r < p.S)
            *reinterpret_cast<uint4v*>(static_cast<char*>(p.y) + (((int64_t)b * p.S + t0 + r) * C + c0) * ES + 16 * (lane & 7)) = v;
        }
        wave_lds_order();
      }
    }
  }
}

// ---------------------------------------------------------------------------------------------------
int device_cu_count();  // attn_fwd.hip

// Chunking of the token axis, or nch = 0 where this path does not apply: heads of 32 channels, 2 or 4 of them, in at
// most kSbMaxChunks chunks per batch (every workgroup of pass 2 merges all chunks of its batch, holding one entry per
// chunk and matrix row in registers).
void small_block_plan(const FtLinBlockArgs& a, int* nch, int* strips_per_chunk) {
  *nch = 0;
  *strips_per_chunk = 0;
  if (a.D != 32 || (a.H != 2 && a.H != 4)) return;
  const int nstrips = (a.S + kSbStrip - 1) / kSbStrip;
  const int cus = device_cu_count();
  const int want = (int)std::min<int64_t>(std::min(nstrips, kSbMaxChunks), std::max<int64_t>(1, ((int64_t)cus + a.B - 1) / a.B));
  const int spc = (nstrips + want - 1) / want;
  const int n = (nstrips + spc - 1) / spc;
  // Short calls are launch-bound and two launches beat the library form's five whatever the size (B1 S784: 21 against
  // 33 us); with more than two strips per wave the workgroups must also cover a good part of the chip, or the
  // library GEMMs, which spread any token count over all of it, do better (B4 S4096: 55 against 44 us; B16: 57
  // against 68).
  const int strips_per_wave = (spc + kSbWaves - 1) / kSbWaves;
  if (strips_per_wave > 2 && (int64_t)a.B * n * 4 < cus) return;
  *nch = n;
  *strips_per_chunk = spc;
}

size_t small_block_workspace_bytes(const FtLinBlockArgs& a) {
  int nch, spc;
  small_block_plan(a, &nch, &spc);
  return (size_t)a.B * nch * a.H * kSbPart * sizeof(float);
}

template <typename T, bool IN32, int H>
static hipError_t launch_small_th(const SmallBlockParams& p, bool ea, bool nq, hipStream_t s) {
  const dim3 grid((unsigned)(p.B * p.nch)), blk(kSbThreads);
  if (ea)
    hipLaunchKernelGGL((linblk_kv_kernel<T, IN32, H, true, false>), grid, blk, 0, s, p);
  else if (nq)
    hipLaunchKernelGGL((linblk_kv_kernel<T, IN32, H, false, true>), grid, blk, 0, s, p);
  else
    hipLaunchKernelGGL((linblk_kv_kernel<T, IN32, H, false, false>), grid, blk, 0, s, p);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return e;
  if (ea)
    hipLaunchKernelGGL((linblk_out_kernel<T, IN32, H, true>), grid, blk, 0, s, p);
  else
    hipLaunchKernelGGL((linblk_out_kernel<T, IN32, H, false>), grid, blk, 0, s, p);
  return hipGetLastError();
}

// the caller has checked small_block_plan() and the size of the workspace
hipError_t launch_small_block(const FtLinBlockArgs& a, int kind, int normalize_q, void* ws, hipStream_t s) {
  SmallBlockParams p{};
  p.x = a.x;
  p.w_qkv = a.w_qkv;
  p.b_qkv = a.b_qkv;
  p.w_out = a.w_out;
  p.b_out = a.b_out;
  p.y = a.y;
  p.part = static_cast<float*>(ws);
  p.B = a.B;
  p.S = a.S;
  p.normalize_q = normalize_q;
  small_block_plan(a, &p.nch, &p.strips_per_chunk);
  if (p.nch == 0) return hipErrorInvalidValue;
  const bool ea = kind == FT_OP_EA, nq = !ea && normalize_q;
  if (a.H == 4) {
    if (a.dtype == FT_F32) return launch_small_th<F16, true, 4>(p, ea, nq, s);
    if (a.dtype == FT_BF16) return launch_small_th<BF16, false, 4>(p, ea, nq, s);
    return launch_small_th<F16, false, 4>(p, ea, nq, s);
  }
  if (a.dtype == FT_F32) return launch_small_th<F16, true, 2>(p, ea, nq, s);
  if (a.dtype == FT_BF16) return launch_small_th<BF16, false, 2>(p, ea, nq, s);
  return launch_small_th<F16, false, 2>(p, ea, nq, s);
}

}  // namespace ft
