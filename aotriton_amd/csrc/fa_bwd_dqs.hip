// dQ from stored dS: instantiations for the 64-, 128- and 256-column builds (fp16 and bf16), with and
// without masked excess columns.
#include "fa_bwd_dqs_impl.h"

namespace fa {

template <typename T>
static hipError_t run_dqs_t(int head_dim, const BwdArgs& a, hipStream_t s) {
  const bool padded = a.head_dim != head_dim;
  if (head_dim == 128) return padded ? launch_bwd_dqs<T, 128, true>(a, s) : launch_bwd_dqs<T, 128, false>(a, s);
  if (head_dim == 64) return padded ? launch_bwd_dqs<T, 64, true>(a, s) : launch_bwd_dqs<T, 64, false>(a, s);
  if (head_dim == 256) return padded ? launch_bwd_dqs<T, 256, true>(a, s) : launch_bwd_dqs<T, 256, false>(a, s);
  return hipErrorNotSupported;
}

hipError_t run_bwd_dqs(int dtype, int head_dim, const BwdArgs& a, hipStream_t s) {
  return dtype == kDtypeBF16 ? run_dqs_t<bf16_t>(head_dim, a, s) : run_dqs_t<f16_t>(head_dim, a, s);
}

// tiles of stored dS per (batch element, q-head): key tiles of 128 x query tiles of the dK/dV step
void ds_tile_counts(int dtype, int head_dim, int max_sq, int max_sk, int* ntq, int* ntk, int64_t* tile_bytes) {
  const int bm = head_dim >= 256 ? DsTile<bf16_t, 256>::BM : head_dim <= 64 ? DsTile<bf16_t, 64>::BM : DsTile<bf16_t, 128>::BM;
  (void)dtype;
  *ntq = ((max_sq + bm - 1) / bm) | 1;     // odd: the rows of tiles of different key tiles and heads do not start a power of two apart
  *ntk = (max_sk + 127) / 128;
  *tile_bytes = (int64_t)128 * bm * 2;
}

}  // namespace fa
