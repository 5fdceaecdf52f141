#include "fa_kernels.h"
namespace fa {
hipError_t run_bwd_preprocess(int, int, const BwdArgs&, hipStream_t) { return hipErrorNotSupported; }
hipError_t run_bwd_dkdv(int, int, const BwdArgs&, bool, bool, bool, hipStream_t) { return hipErrorNotSupported; }
hipError_t run_bwd_dq(int, int, const BwdArgs&, bool, bool, bool, hipStream_t) { return hipErrorNotSupported; }
hipError_t run_bwd_fused(int, int, const BwdArgs&, bool, bool, bool, hipStream_t) { return hipErrorNotSupported; }
}
