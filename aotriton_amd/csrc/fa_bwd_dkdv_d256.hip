// Backward dkdv kernel instantiations for head dim 256 (fp16 and bf16).
#include "fa_bwd_impl.h"

namespace fa {
hipError_t run_bwd_dkdv_d256(int dtype, const BwdArgs& a, bool windowed, bool bias, bool dropout, hipStream_t s) {
  if (dtype == kDtypeBF16) return launch_bwd_dkdv<bf16_t, 256>(a, windowed, bias, dropout, s);
  return launch_bwd_dkdv<f16_t, 256>(a, windowed, bias, dropout, s);
}
}  // namespace fa
