// attn_fwd_kernel.hpp instantiated for bf16, head size 64.
#include "attn_fwd_kernel.hpp"

namespace ft {
hipError_t launch_attn_bf16_d64(const AttnKernelParams& p, bool causal, bool emu, int kf, hipStream_t s) {
  return launch_td<BF16, 64>(p, causal, emu, kf, s);
}
}  // namespace ft
