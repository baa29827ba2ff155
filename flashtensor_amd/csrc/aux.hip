// Small epilogue kernels: heavy-hitter selection (top-k of a per-key score row) and materialisation of
// the seeded KeyFormer noise tensor.  Neither exists in the reference: its H2O case ends at the score
// (cases/kernels/h2o.py:34-38) and its KeyFormer case receives the noise as an input (kf.py:48).
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "device_common.hpp"
#include "noise.h"

namespace ft {

// One workgroup of NT threads sorts one row: (score, index) pairs packed into 64-bit keys whose unsigned
// order is "score descending, index ascending", bitonic network over N = NT E keys, first k indices written
// out.  Thread t keeps keys t E .. t E + E - 1 in registers, so a compare-exchange at distance < E stays inside
// the thread, one at distance < 64 E is a lane exchange inside the wave (no barrier), and only the few
// steps at distance >= 64 E go through LDS (3 with 256 threads, 6 with 512) instead of one barrier per
// network step.  E <= 16 keeps the fully unrolled network's keys in registers.

__device__ __forceinline__ uint32_t float_order_desc(float x) {
  uint32_t u = __builtin_bit_cast(uint32_t, x);
  u = (u & 0x80000000u) ? ~u : (u | 0x80000000u);  // ascending unsigned order == ascending float order
  return ~u;                                       // flipped: larger scores first
}

// Value of lane l ^ M for a compile-time M < 64, without the LDS crossbar a generic shuffle goes through (the sort is
// a chain of ~60 dependent exchanges per row, so their latency is its run time): quad permutes for 1 and 2, half-row
// mirror + quad reversal for 4 ((l ^ 7) ^ 3), a rotation by half a row for 8, v_permlane16_swap / v_permlane32_swap
// for 16 and 32.
template <int M>
__device__ __forceinline__ uint32_t lane_xor_u32(uint32_t v) {
#if defined(__HIP_DEVICE_COMPILE__)
  static_assert(M == 1 || M == 2 || M == 4 || M == 8 || M == 16 || M == 32, "one bit of the lane index");
  const int x = (int)v;
  if constexpr (M == 1) return (uint32_t)__builtin_amdgcn_update_dpp(x, x, 0xB1, 0xF, 0xF, false);  // quad_perm [1,0,3,2]
  if constexpr (M == 2) return (uint32_t)__builtin_amdgcn_update_dpp(x, x, 0x4E, 0xF, 0xF, false);  // quad_perm [2,3,0,1]
  if constexpr (M == 4) {
    const int h = __builtin_amdgcn_update_dpp(x, x, 0x141, 0xF, 0xF, false);                         // row_half_mirror
    return (uint32_t)__builtin_amdgcn_update_dpp(h, h, 0x1B, 0xF, 0xF, false);                       // quad_perm [3,2,1,0]
  }
  if constexpr (M == 8) return (uint32_t)__builtin_amdgcn_update_dpp(x, x, 0x128, 0xF, 0xF, false);  // row_ror:8
  if constexpr (M == 16) {
    const auto r = __builtin_amdgcn_permlane16_swap(v, v, false, false);  // {rows 0,0,2,2}, {rows 1,1,3,3}
    return (threadIdx.x & 16) ? (uint32_t)r[0] : (uint32_t)r[1];
  }
  if constexpr (M == 32) {
    const auto r = __builtin_amdgcn_permlane32_swap(v, v, false, false);  // {lower half twice}, {upper half twice}
    return (threadIdx.x & 32) ? (uint32_t)r[0] : (uint32_t)r[1];
  }
#endif
  return v;
}

template <int M>
__device__ __forceinline__ uint64_t lane_xor_u64(uint64_t v) {
  const uint32_t lo = lane_xor_u32<M>((uint32_t)v), hi = lane_xor_u32<M>((uint32_t)(v >> 32));
  return ((uint64_t)hi << 32) | lo;
}

// one compare-exchange step of the bitonic network at distance STRIDE inside runs of SIZE keys
template <int E, int NT, int SIZE, int STRIDE>
__device__ __forceinline__ void bitonic_step(uint64_t (&key)[E], uint64_t* xch, int t) {
  if constexpr (STRIDE < E) {
#pragma unroll
    for (int e = 0; e < E; ++e) {
      if ((e & STRIDE) == 0) {
        const bool up = ((t * E + e) & SIZE) == 0;
        const uint64_t a = key[e], b = key[e | STRIDE];
        const bool swap = (a > b) == up;
        key[e] = swap ? b : a;
        key[e | STRIDE] = swap ? a : b;
      }
    }
  } else {
    constexpr int M = STRIDE / E;  // partner thread t ^ M holds the partner of every key of this thread
    const bool lower = (t & M) == 0;
    if constexpr (M >= 64) {
#pragma unroll
      for (int e = 0; e < E; ++e) xch[e * NT + t] = key[e];
      __syncthreads();
    }
#pragma unroll
    for (int e = 0; e < E; ++e) {
      const uint64_t a = key[e];
      uint64_t b;
      if constexpr (M >= 64)
        b = xch[e * NT + (t ^ M)];
      else
        b = lane_xor_u64<M>(a);
      const bool up = ((t * E + e) & SIZE) == 0;
      const bool want_min = lower == up;
      key[e] = ((a < b) == want_min) ? a : b;
    }
    if constexpr (M >= 64) __syncthreads();
  }
}
template <int E, int NT, int SIZE, int STRIDE>
__device__ __forceinline__ void bitonic_merge(uint64_t (&key)[E], uint64_t* xch, int t) {
  bitonic_step<E, NT, SIZE, STRIDE>(key, xch, t);
  if constexpr (STRIDE > 1) bitonic_merge<E, NT, SIZE, STRIDE / 2>(key, xch, t);
}
template <int E, int NT, int SIZE>
__device__ __forceinline__ void bitonic_sort(uint64_t (&key)[E], uint64_t* xch, int t) {
  bitonic_merge<E, NT, SIZE, SIZE / 2>(key, xch, t);
  if constexpr (SIZE < E * NT) bitonic_sort<E, NT, SIZE * 2>(key, xch, t);
}

template <int E, int NT>
__global__ void __launch_bounds__(NT) topk_kernel(const float* __restrict__ score, int S, int k, int64_t* __restrict__ idx) {
  constexpr int N = NT * E;
  __shared__ uint64_t xch[N];  // slot-major: key e of thread t at [e * NT + t]
  const int t = threadIdx.x;
  const float* row = score + (int64_t)blockIdx.x * S;
  uint64_t key[E];
#pragma unroll
  for (int e = 0; e < E; ++e) {
    const int i = t * E + e;
    key[e] = i < S ? (((uint64_t)float_order_desc(row[i]) << 32) | (uint32_t)i) : ~0ull;  // padding sorts last
  }
  bitonic_sort<E, NT, 2>(key, xch, t);
  int64_t* out = idx + (int64_t)blockIdx.x * k;
#pragma unroll
  for (int e = 0; e < E; ++e) {
    const int i = t * E + e;
    if (i < k) out[i] = (int64_t)(uint32_t)key[e];
  }
}

// Rows longer than the register sort holds (S > 8192), k <= kTopkSelectMax: one workgroup per row
//   1. radix select over the 32-bit order keys, most significant byte first (four passes over the row, a 256-bin
//      histogram in LDS each): the key T of the k-th entry and the number of entries that sort before it;
//   2. one more pass gathers the winners into LDS as the 64-bit (order key, index) words of the register sort: every
//      entry before T, and of the entries equal to T the ones with the smallest indices (a workgroup-wide prefix count
//      in index order), as the full sort would have ranked them;
//   3. a bitonic network over those <= 16384 words in LDS, and the indices go out in rank order.
// The same answers as the register sort, ties and NaNs included (a NaN of positive sign has the largest order key and
// sorts first, as in torch.topk).
constexpr int kTopkSelectMax = 16384;  // 128 KB of LDS for the winners: k = S / 8 up to S = 131072
constexpr int kTopkSelectThreads = 1024;

__global__ void __launch_bounds__(kTopkSelectThreads) topk_select_kernel(const float* __restrict__ score, int S, int k,
                                                                         int64_t* __restrict__ idx) {
  constexpr int NT = kTopkSelectThreads, NW = NT / 64;
  __shared__ uint64_t win[kTopkSelectMax];
  __shared__ uint32_t hist[256];
  __shared__ uint32_t wave_cnt[NW];
  __shared__ uint32_t s_prefix, s_before, s_slot;
  const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
  const float* row = score + (int64_t)blockIdx.x * S;

  // ---- 1. the order key of rank k
  uint32_t prefix = 0, before = 0;  // high bytes fixed so far; entries whose key is below every key with this prefix
#pragma unroll 1
  for (int shift = 24; shift >= 0; shift -= 8) {
    if (t < 256) hist[t] = 0;
    __syncthreads();
    const uint32_t mask = shift == 24 ? 0u : ~0u << (shift + 8);
    for (int i = t; i < S; i += NT) {
      const uint32_t h = float_order_desc(row[i]);
      if ((h & mask) == prefix) atomicAdd(&hist[(h >> shift) & 255u], 1u);
    }
    __syncthreads();
    if (t == 0) {
      uint32_t cum = before, d = 0;
      for (; d < 255; ++d) {
        if (cum + hist[d] >= (uint32_t)k) break;
        cum += hist[d];
      }
      s_prefix = prefix | (d << shift);
      s_before = cum;
    }
    __syncthreads();
    prefix = s_prefix;
    before = s_before;
  }
  const uint32_t T = prefix;
  const uint32_t need_eq = (uint32_t)k - before;  // entries equal to T that make the cut: those of smallest index

  // ---- 2. gather
  if (t == 0) s_slot = 0;
  __syncthreads();
  uint32_t eq_seen = 0;  // entries equal to T in the tiles before this one (the same in every thread)
#pragma unroll 1
  for (int i0 = 0; i0 < S; i0 += NT) {
    const int i = i0 + t;
    const uint32_t h = i < S ? float_order_desc(row[i]) : ~0u;
    const bool lt = i < S && h < T, eq = i < S && h == T;
    const uint64_t bal = __ballot(eq);
    if (lane == 0) wave_cnt[wave] = (uint32_t)__popcll(bal);
    __syncthreads();
    uint32_t rank = eq_seen + (uint32_t)__popcll(bal & ((1ull << lane) - 1ull)), tile_eq = 0;
#pragma unroll
    for (int w = 0; w < NW; ++w) {
      if (w < wave) rank += wave_cnt[w];
      tile_eq += wave_cnt[w];
    }
    if (lt || (eq && rank < need_eq)) win[atomicAdd(&s_slot, 1u)] = ((uint64_t)h << 32) | (uint32_t)i;
    eq_seen += tile_eq;
    __syncthreads();
  }
  // ---- 3. sort the k winners (padding sorts last)
  int n2 = 2;
  while (n2 < k) n2 <<= 1;
  for (int i = k + t; i < n2; i += NT) win[i] = ~0ull;
  __syncthreads();
#pragma unroll 1
  for (int size = 2; size <= n2; size <<= 1)
#pragma unroll 1
    for (int stride = size >> 1; stride > 0; stride >>= 1) {
      for (int p = t; p < (n2 >> 1); p += NT) {
        const int lo = ((p & ~(stride - 1)) << 1) | (p & (stride - 1)), hi = lo | stride;
        const bool up = (lo & size) == 0;
        const uint64_t a = win[lo], b = win[hi];
        if ((a > b) == up) {
          win[lo] = b;
          win[hi] = a;
        }
      }
      __syncthreads();
    }
  int64_t* out = idx + (int64_t)blockIdx.x * k;
  for (int i = t; i < k; i += NT) out[i] = (int64_t)(uint32_t)win[i];
}

hipError_t launch_topk(const float* score, int64_t rows, int S, int k, int64_t* idx, hipStream_t s) {
  const dim3 grid((unsigned)rows);
  if (S > 8192) {
    if (k > kTopkSelectMax) return hipErrorInvalidValue;
    hipLaunchKernelGGL(topk_select_kernel, grid, dim3(kTopkSelectThreads), 0, s, score, S, k, idx);
    return hipGetLastError();
  }
  if (S <= 512)
    hipLaunchKernelGGL((topk_kernel<2, 256>), grid, dim3(256), 0, s, score, S, k, idx);
  else if (S <= 1024)
    hipLaunchKernelGGL((topk_kernel<4, 256>), grid, dim3(256), 0, s, score, S, k, idx);
  else if (S <= 2048)  // more threads with fewer keys each beat fewer, fuller ones: 10.9 vs 12.9 us (8 keys x 256)
    hipLaunchKernelGGL((topk_kernel<4, 512>), grid, dim3(512), 0, s, score, S, k, idx);
  else if (S <= 4096)  // 21.3 vs 25.8 us (16 keys x 256)
    hipLaunchKernelGGL((topk_kernel<8, 512>), grid, dim3(512), 0, s, score, S, k, idx);
  else
    hipLaunchKernelGGL((topk_kernel<16, 512>), grid, dim3(512), 0, s, score, S, k, idx);
  return hipGetLastError();
}

__global__ void __launch_bounds__(256) noise_fill_kernel(float* __restrict__ dst, int Sq, int Skv, uint64_t seed) {
  const int bh = blockIdx.z;
  const int i = blockIdx.y;
  const NoiseKeys nk = noise_keys(seed, (uint32_t)bh);
  const uint32_t a_i = noise_row(nk, (uint32_t)i);
  float* row = dst + ((int64_t)bh * Sq + i) * Skv;
  for (int j = blockIdx.x * blockDim.x + threadIdx.x; j < Skv; j += gridDim.x * blockDim.x) {
    const float u = noise_uniform(a_i, noise_col(nk, (uint32_t)j));
    row[j] = -0.6931471805599453f * __builtin_amdgcn_logf(u);
  }
}

hipError_t launch_noise_fill(float* dst, int B, int H, int Sq, int Skv, uint64_t seed, hipStream_t s) {
  if ((int64_t)B * H > 65535 || Sq > 65535) return hipErrorInvalidValue;
  dim3 grid((unsigned)((Skv + 1023) / 1024 < 1 ? 1 : (Skv + 1023) / 1024), (unsigned)Sq, (unsigned)(B * H));
  hipLaunchKernelGGL(noise_fill_kernel, grid, dim3(256), 0, s, dst, Sq, Skv, seed);
  return hipGetLastError();
}

// Stride-1 window mean along rows of length S with kernel / 2 zeros on both sides, divisor = kernel: the
// SnapKV smoothing of the per-key scores, F.avg_pool1d(score, kernel, padding = kernel // 2, stride = 1)
// (cases/kernels/snapkv.py:39).  The window is summed left to right like the library routine.
__global__ void __launch_bounds__(256) avgpool1d_kernel(const float* __restrict__ src, float* __restrict__ dst, int S, int kernel) {
  const int64_t row = blockIdx.y;
  const int j = blockIdx.x * blockDim.x + threadIdx.x;
  if (j >= S) return;
  const float* r = src + row * S;
  const int pad = kernel / 2;
  float acc = 0.f;
  for (int t = -pad; t <= pad; ++t) {
    const int jj = j + t;
    if (jj >= 0 && jj < S) acc += r[jj];
  }
  dst[row * S + j] = acc / (float)kernel;
}

hipError_t launch_avgpool1d(const float* src, int64_t rows, int S, int kernel, float* dst, hipStream_t s) {
  if (rows > 65535) return hipErrorInvalidValue;
  dim3 grid((unsigned)((S + 255) / 256), (unsigned)rows);
  hipLaunchKernelGGL(avgpool1d_kernel, grid, dim3(256), 0, s, src, dst, S, kernel);
  return hipGetLastError();
}

// Mean over the `group` consecutive rows of each group: src [groups, group, S] -> dst [groups, S]
// (grouped-query H2O score, cases/attn_h2o.py:42-47; the mean over heads commutes with the sum over rows).
__global__ void __launch_bounds__(256) group_mean_kernel(const float* __restrict__ src, float* __restrict__ dst, int S, int group) {
  const int64_t grp = blockIdx.y;
  const int j = blockIdx.x * blockDim.x + threadIdx.x;
  if (j >= S) return;
  const float* r = src + grp * group * S + j;
  float acc = 0.f;
  for (int t = 0; t < group; ++t) acc += r[(int64_t)t * S];
  dst[grp * S + j] = acc / (float)group;
}

hipError_t launch_group_mean(const float* src, int64_t groups, int group, int S, float* dst, hipStream_t s) {
  if (groups > 65535) return hipErrorInvalidValue;
  dim3 grid((unsigned)((S + 255) / 256), (unsigned)groups);
  hipLaunchKernelGGL(group_mean_kernel, grid, dim3(256), 0, s, src, dst, S, group);
  return hipGetLastError();
}

}  // namespace ft
