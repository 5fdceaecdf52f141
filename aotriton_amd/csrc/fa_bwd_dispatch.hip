// Head-dim dispatch of the backward launchers and the delta (preprocess) kernel.
#include "fa_bwd_impl.h"

namespace fa {

// Tensors whose head dim is one of the compiled ones take the kernels with a constant head
// dim; smaller head dims take the copies that mask the excess columns.
#define FA_DECL(name)                                                                                   \
  hipError_t name##_d64(int, const BwdArgs&, bool, bool, bool, hipStream_t);                            \
  hipError_t name##_d128(int, const BwdArgs&, bool, bool, bool, hipStream_t);                           \
  hipError_t name##_d256(int, const BwdArgs&, bool, bool, bool, hipStream_t);                           \
  hipError_t name##_d64_padded(int, const BwdArgs&, bool, bool, bool, hipStream_t);                     \
  hipError_t name##_d128_padded(int, const BwdArgs&, bool, bool, bool, hipStream_t);                    \
  hipError_t name##_d256_padded(int, const BwdArgs&, bool, bool, bool, hipStream_t);                    \
  hipError_t name(int dtype, int head_dim, const BwdArgs& a, bool w, bool b, bool p, hipStream_t s) {   \
    const bool padded = a.head_dim != head_dim || a.head_dim_v != head_dim;                             \
    switch (head_dim) {                                                                                 \
      case 64: return padded ? name##_d64_padded(dtype, a, w, b, p, s) : name##_d64(dtype, a, w, b, p, s);    \
      case 128: return padded ? name##_d128_padded(dtype, a, w, b, p, s) : name##_d128(dtype, a, w, b, p, s); \
      case 256: return padded ? name##_d256_padded(dtype, a, w, b, p, s) : name##_d256(dtype, a, w, b, p, s); \
    }                                                                                                   \
    return hipErrorNotSupported;                                                                        \
  }

FA_DECL(run_bwd_dkdv)
FA_DECL(run_bwd_dq)
FA_DECL(run_bwd_fused)
#undef FA_DECL

hipError_t run_bwd_preprocess(int dtype, int head_dim, const BwdArgs& a, hipStream_t s) {
  const bool bf = dtype == kDtypeBF16;
  switch (head_dim) {
    case 64: return bf ? launch_bwd_preprocess<bf16_t, 64>(a, s) : launch_bwd_preprocess<f16_t, 64>(a, s);
    case 128: return bf ? launch_bwd_preprocess<bf16_t, 128>(a, s) : launch_bwd_preprocess<f16_t, 128>(a, s);
    case 256: return bf ? launch_bwd_preprocess<bf16_t, 256>(a, s) : launch_bwd_preprocess<f16_t, 256>(a, s);
  }
  return hipErrorNotSupported;
}

}  // namespace fa
