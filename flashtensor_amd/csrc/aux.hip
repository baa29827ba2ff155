// Small epilogue kernels: heavy-hitter selection (top-k of a per-key score row) and materialisation of
// the seeded KeyFormer noise tensor.  Neither exists in the reference: its H2O case ends at the score
// (cases/kernels/h2o.py:34-38) and its KeyFormer case receives the noise as an input (kf.py:48).
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "noise.h"

namespace ft {

// One workgroup sorts one row: (score, index) pairs packed into 64-bit keys whose unsigned order is
// "score descending, index ascending", bitonic sort in LDS, first k indices written out.
constexpr int kTopkThreads = 1024;

__device__ __forceinline__ uint32_t float_order_desc(float x) {
  uint32_t u = __builtin_bit_cast(uint32_t, x);
  u = (u & 0x80000000u) ? ~u : (u | 0x80000000u);  // ascending unsigned order == ascending float order
  return ~u;                                       // flipped: larger scores first
}

__global__ void __launch_bounds__(kTopkThreads) topk_kernel(const float* __restrict__ score, int S, int N /*pow2 >= S*/, int k,
                                                            int64_t* __restrict__ idx) {
  extern __shared__ __align__(16) char smem_raw[];
  uint64_t* keys = reinterpret_cast<uint64_t*>(smem_raw);
  const float* row = score + (int64_t)blockIdx.x * S;
  for (int i = threadIdx.x; i < N; i += blockDim.x) {
    uint64_t key = ~0ull;  // padding sorts last
    if (i < S) key = ((uint64_t)float_order_desc(row[i]) << 32) | (uint32_t)i;
    keys[i] = key;
  }
  __syncthreads();
  for (int size = 2; size <= N; size <<= 1) {
    for (int stride = size >> 1; stride > 0; stride >>= 1) {
      for (int t = threadIdx.x; t < N / 2; t += blockDim.x) {
        const int lo = 2 * t - (t & (stride - 1));
        const int hi = lo + stride;
        const bool ascending = (lo & size) == 0;
        const uint64_t a = keys[lo], b = keys[hi];
        if ((a > b) == ascending) {
          keys[lo] = b;
          keys[hi] = a;
        }
      }
      __syncthreads();
    }
  }
  int64_t* out = idx + (int64_t)blockIdx.x * k;
  for (int i = threadIdx.x; i < k; i += blockDim.x) out[i] = (int64_t)(uint32_t)keys[i];
}

hipError_t launch_topk(const float* score, int64_t rows, int S, int k, int64_t* idx, hipStream_t s) {
  int N = 2;
  while (N < S) N <<= 1;
  const int lds = N * 8;
  static bool configured = false;
  if (!configured) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(topk_kernel), hipFuncAttributeMaxDynamicSharedMemorySize, 8192 * 8);
    if (e != hipSuccess) return e;
    configured = true;
  }
  const int threads = N / 2 < kTopkThreads ? (N / 2 < 64 ? 64 : N / 2) : kTopkThreads;
  hipLaunchKernelGGL(topk_kernel, dim3((unsigned)rows), dim3(threads), lds, s, score, S, N, k, idx);
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
