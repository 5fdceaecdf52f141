// Small HBM-bound kernels: dropout-mask dump and backward preprocess (delta).
#include "fa_device.h"
#include "fa_kernels.h"

namespace fa {

// R[b,h,m,n] = keep ? +0.5 : -0.5 in R's dtype
// (modules/flash/kernel/dropout_rng.py:86-126).  One thread = 4 columns of one
// row = one Philox counter.
template <typename T>
__global__ void encoded_softmax_kernel(const EncodedSoftmaxArgs a) {
  const int groups = (a.seqlen_k + 3) / 4;
  const int64_t total = (int64_t)a.batch * a.heads * a.seqlen_q * groups;
  const int64_t step = (int64_t)gridDim.x * blockDim.x;
  for (int64_t gid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; gid < total; gid += step) {
    const int g = (int)(gid % groups);
    int64_t t = gid / groups;
    const int m = (int)(t % a.seqlen_q); t /= a.seqlen_q;
    const int h = (int)(t % a.heads);
    const int z = (int)(t / a.heads);
    const DropoutState ds = make_dropout(a.drop, z, h, a.heads, a.seqlen_q, a.seqlen_k);
    const uint32_t keep = dropout_keep4(ds, m, 4 * g);
    T* r = reinterpret_cast<T*>(a.r) + (int64_t)z * a.s_z + (int64_t)h * a.s_h + (int64_t)m * a.s_m + 4 * g;
#pragma unroll
    for (int i = 0; i < 4; ++i)
      if (4 * g + i < a.seqlen_k) r[i] = (T)(((keep >> i) & 1u) ? 0.5f : -0.5f);
  }
}

hipError_t run_encoded_softmax(const EncodedSoftmaxArgs& a, hipStream_t s) {
  const int groups = (a.seqlen_k + 3) / 4;
  const int64_t total = (int64_t)a.batch * a.heads * a.seqlen_q * groups;
  if (total == 0) return hipSuccess;
  const int nt = 256;
  // a launch may not exceed 2^32 - 1 threads: larger masks take several counters per thread
  const int64_t nb_all = (total + nt - 1) / nt;
  const int64_t nb = nb_all < (1 << 22) ? nb_all : (1 << 22);
  dim3 grid((unsigned)nb);
  if (a.dtype == kDtypeBF16) hipLaunchKernelGGL(encoded_softmax_kernel<bf16_t>, grid, dim3(nt), 0, s, a);
  else if (a.dtype == kDtypeF16) hipLaunchKernelGGL(encoded_softmax_kernel<f16_t>, grid, dim3(nt), 0, s, a);
  else hipLaunchKernelGGL(encoded_softmax_kernel<float>, grid, dim3(nt), 0, s, a);
  return hipGetLastError();
}

TileShape fwd_tile_shape(int head_dim);

}  // namespace fa
