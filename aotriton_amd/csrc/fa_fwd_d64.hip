// Forward kernel instantiations for head dim 64 (fp16 and bf16).
#include "fa_fwd_impl.h"
#include "fa_kernels.h"

// Compiled twice: as is for tensors whose head dim is 64, and with FA_PADDED=1 for smaller
// head dims (a multiple of 8), where the kernels mask the excess columns.
#ifndef FA_PADDED
#define FA_PADDED 0
#endif
#if FA_PADDED
#define FA_RUN run_fwd_d64_padded
#else
#define FA_RUN run_fwd_d64
#endif

namespace fa {
hipError_t FA_RUN(int dtype, const FwdArgs& a, bool windowed, bool bias, bool dropout, hipStream_t s) {
  if (dtype == kDtypeBF16) return launch_fwd<bf16_t, 64, FA_PADDED != 0>(a, windowed, bias, dropout, s);
  return launch_fwd<f16_t, 64, FA_PADDED != 0>(a, windowed, bias, dropout, s);
}
}  // namespace fa
