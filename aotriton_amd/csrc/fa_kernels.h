// Host-visible launchers of the gfx950 kernels (one translation unit per head dim).
#pragma once
#include <hip/hip_runtime.h>

#include "fa_args.h"

namespace fa {

constexpr int kDtypeF32 = 1, kDtypeF16 = 2, kDtypeBF16 = 3;

struct TileShape { int block_m, block_n, num_waves, lds_bytes; };

hipError_t run_fwd_d64(int dtype, const FwdArgs& a, bool windowed, bool bias, bool dropout, hipStream_t s);
hipError_t run_fwd_d128(int dtype, const FwdArgs& a, bool windowed, bool bias, bool dropout, hipStream_t s);
hipError_t run_fwd_d256(int dtype, const FwdArgs& a, bool windowed, bool bias, bool dropout, hipStream_t s);
// the same kernels with the columns past FwdArgs::head_dim masked (head dims rounded up)
hipError_t run_fwd_d64_padded(int dtype, const FwdArgs& a, bool windowed, bool bias, bool dropout, hipStream_t s);
hipError_t run_fwd_d128_padded(int dtype, const FwdArgs& a, bool windowed, bool bias, bool dropout, hipStream_t s);
hipError_t run_fwd_d256_padded(int dtype, const FwdArgs& a, bool windowed, bool bias, bool dropout, hipStream_t s);
// tile table lookups: (element type, head dim, causal / windowed)
TileShape fwd_tile_shape(int dtype, int head_dim, bool windowed);

hipError_t run_encoded_softmax(const EncodedSoftmaxArgs& a, hipStream_t s);
// strided -> packed (unpack false) or packed -> strided (unpack true); elem_bytes 2 or 4
hipError_t run_repack(int elem_bytes, bool unpack, const RepackArgs& a, hipStream_t s);
// register-only MFMA loop: the rate the matrix pipe sustains (benchmark aid)
hipError_t run_mfma_rate(bool random_operands, int grid, int iters, float* out, unsigned long long* clk, hipStream_t s);

// backward: kernel_slot 0 = preprocess (delta), 1 = dK/dV, 2 = dQ, 3 = fused
hipError_t run_bwd_preprocess(int dtype, int head_dim, const BwdArgs& a, hipStream_t s);
hipError_t run_bwd_dkdv(int dtype, int head_dim, const BwdArgs& a, bool windowed, bool bias, bool dropout, hipStream_t s);
hipError_t run_bwd_dq(int dtype, int head_dim, const BwdArgs& a, bool windowed, bool bias, bool dropout, hipStream_t s);
hipError_t run_bwd_fused(int dtype, int head_dim, const BwdArgs& a, bool windowed, bool bias, bool dropout, hipStream_t s);
TileShape bwd_tile_shape(int dtype, int head_dim, bool windowed, int kernel_slot);
// dQ = dS K from the dS tiles that the dK/dV kernel stored (BwdArgs::ds_ws), and their geometry
hipError_t run_bwd_dqs(int dtype, int head_dim, const BwdArgs& a, hipStream_t s);
void ds_tile_counts(int dtype, int head_dim, int max_sq, int max_sk, int* ntq, int* ntk, int64_t* tile_bytes);

// MFMA kernels of the 16-bit types for head dims above 256, rounded up to 512 (the head dim split
// over the waves of a workgroup).  kernel_slot of the backward: 1 dK/dV, 2 dQ and dB.
hipError_t run_fwd_d512(int dtype, const FwdArgs& a, bool windowed, bool bias, bool dropout, hipStream_t s);
hipError_t run_bwd_d512(int dtype, int kernel_slot, const BwdArgs& a, bool windowed, bool bias, bool dropout,
                        hipStream_t s);
TileShape d512_tile_shape(int kernel_slot);

// MFMA kernels for fp32 tensors at head dims up to 256 (compiled for 128 and 256 columns, the head
// dim split over the waves of a workgroup).  kernel_slot of the backward: 1 dK/dV, 2 dQ and dB.
hipError_t run_fwd_f32(int head_dim, const FwdArgs& a, bool windowed, bool bias, bool dropout, hipStream_t s);
hipError_t run_bwd_f32(int head_dim, int kernel_slot, const BwdArgs& a, bool windowed, bool bias, bool dropout,
                       hipStream_t s);
TileShape f32_tile_shape(int head_dim, int kernel_slot);

// Vector-ALU kernels (no MFMA): every type at every compiled head dim; they serve tensors whose
// rows the MFMA kernels cannot load in 16-byte pieces, and delta of the fp32 and split-head-dim families.
// head_dim is the compiled one (64, 128, 256, 512).  kernel_slot of the backward: 0 delta,
// 1 dK/dV, 2 dQ and dB.
hipError_t run_fwd_valu(int dtype, int head_dim, const FwdArgs& a, hipStream_t s);
hipError_t run_bwd_valu(int dtype, int head_dim, int kernel_slot, const BwdArgs& a, hipStream_t s);

}  // namespace fa
