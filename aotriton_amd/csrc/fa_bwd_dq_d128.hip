// Backward dq kernel instantiations for head dim 128 (fp16 and bf16).
#include "fa_bwd_impl.h"

namespace fa {
hipError_t run_bwd_dq_d128(int dtype, const BwdArgs& a, bool windowed, bool bias, bool dropout, hipStream_t s) {
  if (dtype == kDtypeBF16) return launch_bwd_dq<bf16_t, 128>(a, windowed, bias, dropout, s);
  return launch_bwd_dq<f16_t, 128>(a, windowed, bias, dropout, s);
}
}  // namespace fa
