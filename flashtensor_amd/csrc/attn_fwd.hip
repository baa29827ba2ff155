// Dispatcher of the fused softmax attention forward: picks the instantiation of attn_fwd_kernel.hpp built by
// attn_fwd_{f16,bf16}_{d64,d128}.hip for the element type and head size of the call.
#include <hip/hip_runtime.h>

#include <atomic>
#include <cstdlib>

#include "kernel_params.h"

namespace ft {

int device_cu_count() {
  static std::atomic<int> cus[16];  // zero-initialised; a racing first call stores the same value twice
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 16) return 256;
  int n = cus[dev].load(std::memory_order_relaxed);
  if (n == 0) {
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
    cus[dev].store(n, std::memory_order_relaxed);
  }
  return n;
}

// Test hook: FT_ATTN_FORM in the environment overrides the launch shape the dispatcher would pick for the
// problem size ("4": 128-row workgroups; "8": 256-row workgroups, one query block each; "8x2": 256-row workgroups
// that take the heaviest and the lightest remaining block; an "h" appended: head-major workgroup order), so that
// every form can be checked on every shape whatever the CU count of the device.  Read on every launch.
int attn_form_override() {
  const char* e = getenv("FT_ATTN_FORM");
  if (!e || !*e) return 0;
  int form = 0;
  if (e[0] == '4') form = 1;
  else if (e[0] == '8') form = (e[1] == 'x' && e[2] == '2') ? 3 : 2;
  for (const char* c = e; *c; ++c)
    if (*c == 'h') form |= 8;
  return form;
}

hipError_t launch_attn_f16_d64(const AttnKernelParams& p, bool causal, bool emu, int kf, hipStream_t s);
hipError_t launch_attn_f16_d128(const AttnKernelParams& p, bool causal, bool emu, int kf, hipStream_t s);
hipError_t launch_attn_bf16_d64(const AttnKernelParams& p, bool causal, bool emu, int kf, hipStream_t s);
hipError_t launch_attn_bf16_d128(const AttnKernelParams& p, bool causal, bool emu, int kf, hipStream_t s);

hipError_t launch_attn_fwd(const AttnKernelParams& p, int D, bool bf16, bool causal, bool emu, int kf, hipStream_t s) {
  if (D == 128) return bf16 ? launch_attn_bf16_d128(p, causal, emu, kf, s) : launch_attn_f16_d128(p, causal, emu, kf, s);
  if (D == 64) return bf16 ? launch_attn_bf16_d64(p, causal, emu, kf, s) : launch_attn_f16_d64(p, causal, emu, kf, s);
  return hipErrorInvalidValue;
}

}  // namespace ft
