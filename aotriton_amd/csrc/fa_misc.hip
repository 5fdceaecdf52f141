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

// Tensors whose rows are not made of aligned 16-byte pieces (a head dim or a stride that is no
// multiple of 8 elements, an unaligned base) reach the MFMA kernels through a packed copy: one
// thread moves one group of 8 columns of one row, element by element on the strided side and as one
// vector on the packed side.  The reference pads such head dims inside its kernels
// (modules/flash/csrc/attn_fwd.cc:76-82,109); here the padding is a copy in HBM, which costs one
// pass over the tensor and keeps the kernels' 16-byte staging.
template <typename E, bool kUnpack>
__global__ void repack_kernel(const RepackArgs a) {
  using V = vec<E, 8>;
  const int groups = a.dp / 8;
  const int64_t total = (int64_t)a.n0 * a.n1 * a.n2 * groups;
  const int64_t step = (int64_t)gridDim.x * blockDim.x;
  for (int64_t gid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; gid < total; gid += step) {
    const int g = (int)(gid % groups);
    const int64_t row = gid / groups;
    int64_t t = row;
    const int i2 = (int)(t % a.n2); t /= a.n2;
    const int i1 = (int)(t % a.n1);
    const int i0 = (int)(t / a.n1);
    E* sp = reinterpret_cast<E*>(a.strided) + i0 * a.s0 + i1 * a.s1 + i2 * a.s2 + 8 * g;
    V* pp = reinterpret_cast<V*>(reinterpret_cast<E*>(a.packed) + row * a.dp + 8 * g);
    if (kUnpack) {
      const V v = *pp;
#pragma unroll
      for (int e = 0; e < 8; ++e)
        if (8 * g + e < a.d) sp[e] = v[e];
    } else {
      V v;
#pragma unroll
      for (int e = 0; e < 8; ++e) v[e] = 8 * g + e < a.d ? sp[e] : (E)0;
      *pp = v;
    }
  }
}

hipError_t run_repack(int elem_bytes, bool unpack, const RepackArgs& a, hipStream_t s) {
  const int64_t total = (int64_t)a.n0 * a.n1 * a.n2 * (a.dp / 8);
  if (total == 0) return hipSuccess;
  const int nt = 256;
  const int64_t nb_all = (total + nt - 1) / nt;
  dim3 grid((unsigned)(nb_all < (1 << 20) ? nb_all : (1 << 20)));
  if (elem_bytes == 2) {
    if (unpack) hipLaunchKernelGGL((repack_kernel<uint16_t, true>), grid, dim3(nt), 0, s, a);
    else hipLaunchKernelGGL((repack_kernel<uint16_t, false>), grid, dim3(nt), 0, s, a);
  } else {
    if (unpack) hipLaunchKernelGGL((repack_kernel<uint32_t, true>), grid, dim3(nt), 0, s, a);
    else hipLaunchKernelGGL((repack_kernel<uint32_t, false>), grid, dim3(nt), 0, s, a);
  }
  return hipGetLastError();
}

// Register-only loop of v_mfma_f32_32x32x16_bf16 (4 independent accumulators per wave, 8 waves
// per CU): what the matrix pipe sustains on this machine, on constant operands or on operands
// with random mantissas (the clock under load depends on the data).  clk[0] = shader cycles,
// clk[1] = 100 MHz reference ticks of workgroup 0.
template <bool kRandom>
__global__ __launch_bounds__(256) void mfma_rate_kernel(float* out, int iters, unsigned long long* clk) {
  using op_t = Traits<bf16_t>::op_t;
  op_t a[8], b[8];
  unsigned s = threadIdx.x * 2654435761u + blockIdx.x * 40503u + 12345u;
  for (int j = 0; j < 8; ++j)
    for (int i = 0; i < 8; ++i) {
      s = s * 1664525u + 1013904223u;
      const float fa = kRandom ? ((int)(s >> 8) % 2001 - 1000) * 1e-3f : 1.0f;
      s = s * 1664525u + 1013904223u;
      const float fb = kRandom ? ((int)(s >> 8) % 2001 - 1000) * 1e-3f : 0.5f;
      a[j][i] = (bf16_t)fa; b[j][i] = (bf16_t)fb;
    }
  f32x16 acc[4];
  for (int n = 0; n < 4; ++n)
    for (int i = 0; i < 16; ++i) acc[n][i] = 0.f;
  const unsigned long long t0 = __builtin_amdgcn_s_memtime(), r0 = __builtin_amdgcn_s_memrealtime();
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int j = 0; j < 8; ++j)
#pragma unroll
      for (int n = 0; n < 4; ++n) acc[n] = Traits<bf16_t>::mfma(a[j], b[(j + n) & 7], acc[n]);
  }
  const unsigned long long t1 = __builtin_amdgcn_s_memtime(), r1 = __builtin_amdgcn_s_memrealtime();
  float r = 0.f;
  for (int n = 0; n < 4; ++n)
    for (int i = 0; i < 16; ++i) r += acc[n][i];
  out[(size_t)blockIdx.x * blockDim.x + threadIdx.x] = r;
  if (blockIdx.x == 0 && threadIdx.x == 0) { clk[0] = t1 - t0; clk[1] = r1 - r0; }
}

// out: grid * 256 floats, clk: 2 x u64.  FLOP of one launch = grid * 4 waves * iters * 32 MFMAs * 32768.
hipError_t run_mfma_rate(bool random_operands, int grid, int iters, float* out, unsigned long long* clk, hipStream_t s) {
  if (random_operands) hipLaunchKernelGGL(mfma_rate_kernel<true>, dim3(grid), dim3(256), 0, s, out, iters, clk);
  else hipLaunchKernelGGL(mfma_rate_kernel<false>, dim3(grid), dim3(256), 0, s, out, iters, clk);
  return hipGetLastError();
}


}  // namespace fa
