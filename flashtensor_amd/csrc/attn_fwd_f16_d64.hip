// attn_fwd_kernel.hpp instantiated for f16, head size 64.
#include "attn_fwd_kernel.hpp"

namespace ft {
hipError_t launch_attn_f16_d64(const AttnKernelParams& p, bool causal, bool emu, int kf, hipStream_t s) {
  return launch_td<F16, 64>(p, causal, emu, kf, s);
}
}  // namespace ft
