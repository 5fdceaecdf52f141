// Forward kernel instantiations for head dim 64 (fp16 and bf16).
#include "fa_fwd_impl.h"
#include "fa_kernels.h"

namespace fa {
hipError_t run_fwd_d64(int dtype, const FwdArgs& a, bool windowed, bool bias, bool dropout, hipStream_t s) {
  if (dtype == kDtypeBF16) return launch_fwd<bf16_t, 64>(a, windowed, bias, dropout, s);
  return launch_fwd<f16_t, 64>(a, windowed, bias, dropout, s);
}
}  // namespace fa
