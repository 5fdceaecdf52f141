// Plain vector-ALU kernels, one row of Q (or of K) per group of 8 lanes: the functional path
// for what the MFMA kernels do not cover, i.e. tensors whose rows are not made of aligned 16-byte
// pieces (loads and stores element by element), and delta for the fp32 kernels and the kernels
// of head dims above 256.
//
// The reference compiles its Triton kernels for fp32 and for head dim 512 as well
// (modules/flash/aot/_common.py:10-14 lists the head dims, '*fp32:16' is among the tensor
// types).  These kernels compute what the MFMA kernels do, in the same base-2 formulation,
// with all arithmetic in fp32
//   forward   modules/flash/kernel/fwd_kernel.py:83-644, fwd_kernel_inner.py:46-287
//   delta     modules/flash/kernel/bwd_preprocess.py:28-250
//   dK, dV    modules/flash/kernel/bwd_kernel_dk_dv.py:48-417, bwd_inner_dk_dv.py:28-267
//   dQ, dB    modules/flash/kernel/bwd_kernel_dq.py:45-389, bwd_inner_dq.py:28-215
// with the online softmax advancing one key at a time.  A row's D columns are spread over
// 8 lanes in 16-byte pieces (lane g holds columns 4g + 32j .. 4g + 32j + 3), dot products
// are finished with three lane exchanges, K/V (or Q/dO) rows are read straight from
// global memory: the 32 rows of a workgroup read the same row at the same time.
#include "fa_device.h"
#include "fa_intervals.h"
#include "fa_kernels.h"

namespace fa {
namespace {

constexpr int kRowsPerBlock = 32;   // 256 threads, 8 lanes per row

template <int DPL>
struct Row {
  float x[DPL];
};

// four consecutive elements of the tensors' type
template <typename T> struct Quad { using type = typename Traits<T>::q4_t; };
template <> struct Quad<float> { using type = f32x4; };
template <typename T> __device__ __forceinline__ T from_float(float x) { return Traits<T>::cvt(x); }
template <> __device__ __forceinline__ float from_float<float>(float x) { return x; }

// columns [0, cols) of a row of D = 8*DPL elements as floats; the rest reads as zero.  `elem`: the
// row is not made of aligned groups of four (a head dim that is no multiple of 8, odd strides, a
// base that is only element-aligned) and is read element by element.
template <int DPL, typename T>
__device__ __forceinline__ Row<DPL> load_row(const T* p, int sub, int cols, bool ok, bool elem) {
  using quad = typename Quad<T>::type;
  Row<DPL> r;
#pragma unroll
  for (int j = 0; j < DPL / 4; ++j) {
    const int c = 4 * sub + 32 * j;
    if (elem) {
#pragma unroll
      for (int e = 0; e < 4; ++e) r.x[4 * j + e] = ok && c + e < cols ? (float)p[c + e] : 0.f;
    } else if (ok && c < cols) {
      const quad v = *reinterpret_cast<const quad*>(p + c);
#pragma unroll
      for (int e = 0; e < 4; ++e) r.x[4 * j + e] = (float)v[e];
    } else {
#pragma unroll
      for (int e = 0; e < 4; ++e) r.x[4 * j + e] = 0.f;
    }
  }
  return r;
}

template <int DPL, typename T>
__device__ __forceinline__ void store_row(T* p, const Row<DPL>& r, int sub, int cols, float scale, bool elem) {
  using quad = typename Quad<T>::type;
#pragma unroll
  for (int j = 0; j < DPL / 4; ++j) {
    const int c = 4 * sub + 32 * j;
    if (elem) {
#pragma unroll
      for (int e = 0; e < 4; ++e)
        if (c + e < cols) p[c + e] = from_float<T>(r.x[4 * j + e] * scale);
    } else if (c < cols) {
      quad v;
#pragma unroll
      for (int e = 0; e < 4; ++e) v[e] = from_float<T>(r.x[4 * j + e] * scale);
      *reinterpret_cast<quad*>(p + c) = v;
    }
  }
}

template <int DPL>
__device__ __forceinline__ float dot8(const Row<DPL>& a, const Row<DPL>& b) {
  float acc = 0.f;
#pragma unroll
  for (int e = 0; e < DPL; ++e) acc = __builtin_fmaf(a.x[e], b.x[e], acc);
  acc += __shfl_xor(acc, 1, 64);
  acc += __shfl_xor(acc, 2, 64);
  acc += __shfl_xor(acc, 4, 64);
  return acc;
}

struct Vis {
  bool windowed;
  int left, right;
  __device__ __forceinline__ bool operator()(int m, int n) const {
    return !windowed || (n <= m + right && n >= m - left);
  }
};

__device__ __forceinline__ Vis make_vis(const MaskArgs& mk, const SeqInfo& si) {
  Vis v{mk.causal_type != 0, 0, 0};
  if (v.windowed) {
    Window w = parse_window(mk.causal_type, mk.window_left, mk.window_right, si.seqlen_q, si.seqlen_k);
    v.left = w.left > (1 << 30) ? (1 << 30) : (w.left < -(1 << 30) ? -(1 << 30) : w.left);
    v.right = w.right > (1 << 30) ? (1 << 30) : (w.right < -(1 << 30) ? -(1 << 30) : w.right);
  }
  return v;
}

// ---------------------------------------------------------------------------
template <typename T, int DPL>
__global__ void valu_fwd_kernel(const FwdArgs a) {
  const int tid = threadIdx.x, sub = tid & 7;
  const int h = blockIdx.y, z = blockIdx.z;
  const SeqInfo si = get_seq(a.seq, z);
  const int m = blockIdx.x * kRowsPerBlock + (tid >> 3);
  if (blockIdx.x == 0 && h == 0 && z == 0 && tid == 0 && a.drop.p > 0.f) {
    // modules/flash/kernel/fwd_kernel.py:199-207
    uint64_t base = a.drop.offset2;
    if (a.drop.offset1_ptr) base += *a.drop.offset1_ptr;
    if (a.seed_out) *a.seed_out = *a.drop.seed_ptr;
    if (a.offset_out) *a.offset_out = base;
  }
  if ((int)blockIdx.x * kRowsPerBlock >= si.seqlen_q) return;
  const bool row_ok = m < si.seqlen_q;
  const int mc = row_ok ? m : si.seqlen_q - 1;
  const int hk = h / (a.hq / a.hk);
  const Vis vis = make_vis(a.mask, si);
  const bool dropout = a.drop.p > 0.f;
  DropoutState ds{};
  if (dropout) ds = make_dropout(a.drop, z, h, a.hq, a.seq.max_seqlen_q, a.seq.max_seqlen_k);
  const T* qp = reinterpret_cast<const T*>(a.q) + (int64_t)si.batch_index * a.sq.z + (int64_t)h * a.sq.h +
                    (int64_t)(si.q_start + mc) * a.sq.s;
  const T* kb = reinterpret_cast<const T*>(a.k) + (int64_t)si.batch_index * a.sk.z + (int64_t)hk * a.sk.h +
                    (int64_t)si.k_start * a.sk.s;
  const T* vb = reinterpret_cast<const T*>(a.v) + (int64_t)si.batch_index * a.sv.z + (int64_t)hk * a.sv.h +
                    (int64_t)si.k_start * a.sv.s;
  const T* bp = a.bias ? reinterpret_cast<const T*>(a.bias) + (int64_t)si.batch_index * a.sb_z +
                                 (int64_t)h * a.sb_h + (int64_t)mc * a.sb_m
                           : nullptr;
  const Row<DPL> q = load_row<DPL, T>(qp, sub, a.head_dim, true, a.elementwise != 0);
  Row<DPL> o;
#pragma unroll
  for (int e = 0; e < DPL; ++e) o.x[e] = 0.f;
  const float qk_scale = a.sm_scale * kLog2e;
  float mi = -__builtin_inff(), li = 0.f;
  // keys any row of this block can see
  const int m_first = blockIdx.x * kRowsPerBlock;
  const int m_last = (m_first + kRowsPerBlock < si.seqlen_q ? m_first + kRowsPerBlock : si.seqlen_q) - 1;
  int n_lo = 0, n_hi = si.seqlen_k - 1;
  if (vis.windowed) {
    n_lo = m_first - vis.left > 0 ? m_first - vis.left : 0;
    n_hi = m_last + vis.right < n_hi ? m_last + vis.right : n_hi;
  }
  for (int n = n_lo; n <= n_hi; ++n) {
    const Row<DPL> kr = load_row<DPL, T>(kb + (int64_t)n * a.sk.s, sub, a.head_dim, true, a.elementwise != 0);
    float s = dot8<DPL>(q, kr) * qk_scale;                                   // fwd_kernel_inner.py:166
    if (bp) s += (float)bp[(int64_t)n * a.sb_n] * kLog2e;                           // :187
    if (!vis(m, n) || s == -__builtin_inff()) continue;                      // lanes of a row agree
    const float m_new = fmaxf(mi, s);
    const float alpha = fast_exp2(mi - m_new);                               // exp2(-inf) = 0 on the first key
    const float p = fast_exp2(s - m_new);
    li = li * alpha + p;                                                     // the sum is over the undropped p (:213-214)
    mi = m_new;
    const bool keep = !dropout || dropout_keep1(ds, m, n);
    const float pv = keep ? p : 0.f;
    const Row<DPL> vr = load_row<DPL, T>(vb + (int64_t)n * a.sv.s, sub, a.head_dim_v, true, a.elementwise != 0);
#pragma unroll
    for (int e = 0; e < DPL; ++e) o.x[e] = __builtin_fmaf(pv, vr.x[e], o.x[e] * alpha);
  }
  if (!row_ok) return;
  const bool alive = li > 0.f;
  float inv = alive ? 1.0f / li : 0.f;
  if (dropout) inv *= ds.scale;                                              // fwd_kernel.py:573-580
  T* op = reinterpret_cast<T*>(a.out) + (int64_t)si.batch_index * a.so.z + (int64_t)h * a.so.h +
              (int64_t)(si.q_start + m) * a.so.s;
  store_row<DPL, T>(op, o, sub, a.head_dim_v, inv, a.elementwise != 0);
  if (a.lse && sub == 0)
    a.lse[lse_offset(si, h, a.hq) + m] = alive ? (mi + fast_log2(li)) * kLn2 : __builtin_inff();   // :610-612, :327-355
}

// ---------------------------------------------------------------------------
template <typename T, int DPL>
__global__ void valu_delta_kernel(const BwdArgs a) {
  const int tid = threadIdx.x, sub = tid & 7;
  const int h = blockIdx.y, z = blockIdx.z;
  const SeqInfo si = get_seq(a.seq, z);
  const int m = blockIdx.x * kRowsPerBlock + (tid >> 3);
  if ((int)blockIdx.x * kRowsPerBlock >= si.seqlen_q) return;
  const bool row_ok = m < si.seqlen_q;
  const int mc = row_ok ? m : si.seqlen_q - 1;
  const T* op = reinterpret_cast<const T*>(a.out) + (int64_t)si.batch_index * a.so.z + (int64_t)h * a.so.h +
                    (int64_t)(si.q_start + mc) * a.so.s;
  const T* dop = reinterpret_cast<const T*>(a.dout) + (int64_t)si.batch_index * a.sdo.z +
                     (int64_t)h * a.sdo.h + (int64_t)(si.q_start + mc) * a.sdo.s;
  const bool elem = a.elementwise != 0;
  const float d = dot8<DPL>(load_row<DPL, T>(op, sub, a.head_dim_v, true, elem), load_row<DPL, T>(dop, sub, a.head_dim_v, true, elem));
  if (row_ok && sub == 0) a.delta[lse_offset(si, h, a.hq) + m] = d;
}

// One row of Q per lane group, all keys: dQ and dB.
template <typename T, int DPL>
__global__ void valu_dq_kernel(const BwdArgs a) {
  const int tid = threadIdx.x, sub = tid & 7;
  const int h = blockIdx.y, z = blockIdx.z;
  const SeqInfo si = get_seq(a.seq, z);
  const int m = blockIdx.x * kRowsPerBlock + (tid >> 3);
  if ((int)blockIdx.x * kRowsPerBlock >= si.seqlen_q) return;
  const bool row_ok = m < si.seqlen_q;
  const int mc = row_ok ? m : si.seqlen_q - 1;
  const int hk = h / (a.hq / a.hk);
  const Vis vis = make_vis(a.mask, si);
  const bool dropout = a.drop.p > 0.f;
  DropoutState ds{};
  if (dropout) ds = make_dropout(a.drop, z, h, a.hq, a.seq.max_seqlen_q, a.seq.max_seqlen_k);
  const int64_t qoff = (int64_t)si.batch_index * a.sq.z + (int64_t)h * a.sq.h + (int64_t)(si.q_start + mc) * a.sq.s;
  const T* dop = reinterpret_cast<const T*>(a.dout) + (int64_t)si.batch_index * a.sdo.z +
                     (int64_t)h * a.sdo.h + (int64_t)(si.q_start + mc) * a.sdo.s;
  const T* kb = reinterpret_cast<const T*>(a.k) + (int64_t)si.batch_index * a.sk.z + (int64_t)hk * a.sk.h +
                    (int64_t)si.k_start * a.sk.s;
  const T* vb = reinterpret_cast<const T*>(a.v) + (int64_t)si.batch_index * a.sv.z + (int64_t)hk * a.sv.h +
                    (int64_t)si.k_start * a.sv.s;
  const T* bp = a.bias ? reinterpret_cast<const T*>(a.bias) + (int64_t)si.batch_index * a.sb_z +
                                 (int64_t)h * a.sb_h + (int64_t)mc * a.sb_m
                           : nullptr;
  T* dbp = a.db ? reinterpret_cast<T*>(a.db) + (int64_t)si.batch_index * a.sdb_z + (int64_t)h * a.sdb_h +
                          (int64_t)mc * a.sdb_m
                    : nullptr;
  const Row<DPL> q = load_row<DPL, T>(reinterpret_cast<const T*>(a.q) + qoff, sub, a.head_dim, true, a.elementwise != 0);
  const Row<DPL> dout = load_row<DPL, T>(dop, sub, a.head_dim_v, true, a.elementwise != 0);
  const int64_t lo = lse_offset(si, h, a.hq) + mc;
  const float L = a.lse[lo] * kRcpLn2;                                       // bwd_kernel_dq.py:305
  const float delta = a.delta[lo];
  const float qk_scale = a.sm_scale * kLog2e;
  Row<DPL> dq;
#pragma unroll
  for (int e = 0; e < DPL; ++e) dq.x[e] = 0.f;
  for (int n = 0; n < si.seqlen_k; ++n) {
    float dsv = 0.f;
    if (vis(m, n)) {
      const Row<DPL> kr = load_row<DPL, T>(kb + (int64_t)n * a.sk.s, sub, a.head_dim, true, a.elementwise != 0);
      const Row<DPL> vr = load_row<DPL, T>(vb + (int64_t)n * a.sv.s, sub, a.head_dim_v, true, a.elementwise != 0);
      float x = dot8<DPL>(q, kr) * qk_scale;
      if (bp) x += (float)bp[(int64_t)n * a.sb_n] * kLog2e;
      const float p = fast_exp2(x - L);                                      // bwd_inner_dq.py:158-160
      float dp = dot8<DPL>(dout, vr);
      if (dropout) dp = dropout_keep1(ds, m, n) ? dp * ds.scale : 0.f;      // :176-185
      dsv = p * (dp - delta);                                                // :188
#pragma unroll
      for (int e = 0; e < DPL; ++e) dq.x[e] = __builtin_fmaf(dsv, kr.x[e], dq.x[e]);
    }
    if (dbp && row_ok && sub == 0) dbp[(int64_t)n * a.sdb_n] = from_float<T>(dsv);          // :200-204; unvisited entries are zero
  }
  if (!row_ok) return;
  T* dqp = reinterpret_cast<T*>(a.dq) + (int64_t)si.batch_index * a.sdq.z + (int64_t)h * a.sdq.h +
               (int64_t)(si.q_start + m) * a.sdq.s;
  store_row<DPL, T>(dqp, dq, sub, a.head_dim, a.sm_scale, a.elementwise != 0);                      // bwd_kernel_dq.py:374-376
}

// One row of K per lane group, all q-heads of its group and all queries: dK and dV.
template <typename T, int DPL>
__global__ void valu_dkdv_kernel(const BwdArgs a) {
  const int tid = threadIdx.x, sub = tid & 7;
  const int hk = blockIdx.y, z = blockIdx.z;
  const SeqInfo si = get_seq(a.seq, z);
  const int n = blockIdx.x * kRowsPerBlock + (tid >> 3);
  if ((int)blockIdx.x * kRowsPerBlock >= si.seqlen_k) return;
  const bool row_ok = n < si.seqlen_k;
  const int nc = row_ok ? n : si.seqlen_k - 1;
  const Vis vis = make_vis(a.mask, si);
  const bool dropout = a.drop.p > 0.f;
  const int group = a.hq / a.hk;
  const Row<DPL> kr = load_row<DPL, T>(reinterpret_cast<const T*>(a.k) + (int64_t)si.batch_index * a.sk.z +
                                        (int64_t)hk * a.sk.h + (int64_t)(si.k_start + nc) * a.sk.s,
                                    sub, a.head_dim, true, a.elementwise != 0);
  const Row<DPL> vr = load_row<DPL, T>(reinterpret_cast<const T*>(a.v) + (int64_t)si.batch_index * a.sv.z +
                                        (int64_t)hk * a.sv.h + (int64_t)(si.k_start + nc) * a.sv.s,
                                    sub, a.head_dim_v, true, a.elementwise != 0);
  const float qk_scale = a.sm_scale * kLog2e;
  Row<DPL> dk, dv;
#pragma unroll
  for (int e = 0; e < DPL; ++e) { dk.x[e] = 0.f; dv.x[e] = 0.f; }
  for (int g = 0; g < group; ++g) {                                          // bwd_kernel_dk_dv.py:285
    const int h = hk * group + g;
    DropoutState ds{};
    if (dropout) ds = make_dropout(a.drop, z, h, a.hq, a.seq.max_seqlen_q, a.seq.max_seqlen_k);
    const T* qb = reinterpret_cast<const T*>(a.q) + (int64_t)si.batch_index * a.sq.z + (int64_t)h * a.sq.h +
                      (int64_t)si.q_start * a.sq.s;
    const T* dob = reinterpret_cast<const T*>(a.dout) + (int64_t)si.batch_index * a.sdo.z +
                       (int64_t)h * a.sdo.h + (int64_t)si.q_start * a.sdo.s;
    const T* bb = a.bias ? reinterpret_cast<const T*>(a.bias) + (int64_t)si.batch_index * a.sb_z +
                                   (int64_t)h * a.sb_h + (int64_t)nc * a.sb_n
                             : nullptr;
    const int64_t lo = lse_offset(si, h, a.hq);
    for (int m = 0; m < si.seqlen_q; ++m) {
      if (!vis(m, n)) continue;                                              // lanes of a row agree
      const Row<DPL> qr = load_row<DPL, T>(qb + (int64_t)m * a.sq.s, sub, a.head_dim, true, a.elementwise != 0);
      const Row<DPL> dor = load_row<DPL, T>(dob + (int64_t)m * a.sdo.s, sub, a.head_dim_v, true, a.elementwise != 0);
      float x = dot8<DPL>(qr, kr) * qk_scale;
      if (bb) x += (float)bb[(int64_t)m * a.sb_m] * kLog2e;
      const float p = fast_exp2(x - a.lse[lo + m] * kRcpLn2);               // bwd_inner_dk_dv.py:185-188
      const bool keep = !dropout || dropout_keep1(ds, m, n);
      const float pd = dropout ? (keep ? p * ds.scale : 0.f) : p;            // :194-201
      float dp = dot8<DPL>(dor, vr);
      if (dropout) dp = keep ? dp * ds.scale : 0.f;                          // :231-240
      const float dsv = p * (dp - a.delta[lo + m]);                          // :242
#pragma unroll
      for (int e = 0; e < DPL; ++e) {
        dv.x[e] = __builtin_fmaf(pd, dor.x[e], dv.x[e]);
        dk.x[e] = __builtin_fmaf(dsv, qr.x[e], dk.x[e]);
      }
    }
  }
  if (!row_ok) return;
  T* dkp = reinterpret_cast<T*>(a.dk) + (int64_t)si.batch_index * a.sdk.z + (int64_t)hk * a.sdk.h +
               (int64_t)(si.k_start + n) * a.sdk.s;
  T* dvp = reinterpret_cast<T*>(a.dv) + (int64_t)si.batch_index * a.sdv.z + (int64_t)hk * a.sdv.h +
               (int64_t)(si.k_start + n) * a.sdv.s;
  store_row<DPL, T>(dkp, dk, sub, a.head_dim, a.sm_scale, a.elementwise != 0);                      // bwd_kernel_dk_dv.py:387-389
  store_row<DPL, T>(dvp, dv, sub, a.head_dim_v, 1.0f, a.elementwise != 0);
}

// head_dim: 64, 128, 256 or 512, the one that holds the tensors' head dims.  The 16-bit types are
// built for 128, 256 and 512 (the MFMA kernels serve them wherever rows are made of aligned 16-byte
// pieces; what is left are the element-wise cases, and 64 columns run on the 128 build).
template <template <typename, int> class Launch, typename... A>
hipError_t valu_dispatch(int dtype, int head_dim, A&&... args) {
  if (dtype == kDtypeF32) {
    switch (head_dim) {
      case 64: return Launch<float, 8>::run(args...);
      case 128: return Launch<float, 16>::run(args...);
      case 256: return Launch<float, 32>::run(args...);
      case 512: return Launch<float, 64>::run(args...);
    }
    return hipErrorNotSupported;
  }
  if (dtype != kDtypeBF16 && dtype != kDtypeF16) return hipErrorNotSupported;
  const bool bf = dtype == kDtypeBF16;
  switch (head_dim) {
    case 64:
    case 128: return bf ? Launch<bf16_t, 16>::run(args...) : Launch<f16_t, 16>::run(args...);
    case 256: return bf ? Launch<bf16_t, 32>::run(args...) : Launch<f16_t, 32>::run(args...);
    case 512: return bf ? Launch<bf16_t, 64>::run(args...) : Launch<f16_t, 64>::run(args...);
  }
  return hipErrorNotSupported;
}

template <typename T, int DPL> struct LaunchFwd {
  static hipError_t run(const dim3& grid, const FwdArgs& a, hipStream_t s) {
    hipLaunchKernelGGL((valu_fwd_kernel<T, DPL>), grid, dim3(256), 0, s, a);
    return hipGetLastError();
  }
};
template <typename T, int DPL> struct LaunchBwd {
  static hipError_t run(int kernel_slot, const dim3& gq, const dim3& gk, const BwdArgs& a, hipStream_t s) {
    switch (kernel_slot) {
      case 0: hipLaunchKernelGGL((valu_delta_kernel<T, DPL>), gq, dim3(256), 0, s, a); break;
      case 1: hipLaunchKernelGGL((valu_dkdv_kernel<T, DPL>), gk, dim3(256), 0, s, a); break;
      case 2: hipLaunchKernelGGL((valu_dq_kernel<T, DPL>), gq, dim3(256), 0, s, a); break;
      default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
  }
};

}  // namespace

hipError_t run_fwd_valu(int dtype, int head_dim, const FwdArgs& a, hipStream_t s) {
  const dim3 grid((a.seq.max_seqlen_q + kRowsPerBlock - 1) / kRowsPerBlock, a.hq, nseq_of(a.seq, a.batch));
  if (grid.x == 0 || grid.z == 0) return hipSuccess;      // an empty tensor: nothing to write
  return valu_dispatch<LaunchFwd>(dtype, head_dim, grid, a, s);
}

// kernel_slot: 0 delta, 1 dK/dV, 2 dQ (and dB)
hipError_t run_bwd_valu(int dtype, int head_dim, int kernel_slot, const BwdArgs& a, hipStream_t s) {
  const int nseq = nseq_of(a.seq, a.batch);
  const dim3 gq((a.seq.max_seqlen_q + kRowsPerBlock - 1) / kRowsPerBlock, a.hq, nseq);
  const dim3 gk((a.seq.max_seqlen_k + kRowsPerBlock - 1) / kRowsPerBlock, a.hk, nseq);
  const dim3& g = kernel_slot == 1 ? gk : gq;
  if (g.x == 0 || g.z == 0) return hipSuccess;            // an empty tensor: nothing to write
  return valu_dispatch<LaunchBwd>(dtype, head_dim, kernel_slot, gq, gk, a, s);
}

}  // namespace fa
