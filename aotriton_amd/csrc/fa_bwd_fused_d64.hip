// Backward fused kernel instantiations for head dim 64 (fp16 and bf16).
#include "fa_bwd_impl.h"

namespace fa {
hipError_t run_bwd_fused_d64(int dtype, const BwdArgs& a, bool windowed, bool bias, bool dropout, hipStream_t s) {
  if (dtype == kDtypeBF16) return launch_bwd_fused<bf16_t, 64>(a, windowed, bias, dropout, s);
  return launch_bwd_fused<f16_t, 64>(a, windowed, bias, dropout, s);
}
}  // namespace fa
