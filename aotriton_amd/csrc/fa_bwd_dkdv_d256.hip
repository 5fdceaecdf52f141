// Backward dkdv kernel instantiations for head dim 256 (fp16 and bf16).
#include "fa_bwd_impl.h"

// Compiled twice: as is for tensors whose head dim is 256, and with FA_PADDED=1 for smaller
// head dims (a multiple of 8), where the kernels mask the excess columns.
#ifndef FA_PADDED
#define FA_PADDED 0
#endif
#if FA_PADDED
#define FA_RUN run_bwd_dkdv_d256_padded
#else
#define FA_RUN run_bwd_dkdv_d256
#endif

namespace fa {
hipError_t FA_RUN(int dtype, const BwdArgs& a, bool windowed, bool bias, bool dropout, hipStream_t s) {
  if (dtype == kDtypeBF16) return launch_bwd_dkdv<bf16_t, 256, FA_PADDED != 0>(a, windowed, bias, dropout, s);
  return launch_bwd_dkdv<f16_t, 256, FA_PADDED != 0>(a, windowed, bias, dropout, s);
}
}  // namespace fa
