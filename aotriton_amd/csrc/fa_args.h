// Kernel argument blocks shared by the host dispatcher and the gfx950 kernels.
// Strides are in elements; the innermost stride of every tensor is 1.
#pragma once
#include <stdint.h>

namespace fa {

constexpr int kNumXcd = 8;   // MI355X: 8 XCDs x 32 CUs, one L2 each

struct Strides3 {   // batch, head, row
  int64_t z, h, s;
};

struct SeqArgs {
  const int32_t* cu_q;   // null when dense
  const int32_t* cu_k;
  const int32_t* ss_q;   // strided varlen only
  const int32_t* ss_k;
  int32_t num_seqlens;   // >0 compact/strided, <0 padded, 0 dense (attn_fwd.cc:99)
  int32_t max_seqlen_q;
  int32_t max_seqlen_k;
};

struct MaskArgs {
  int32_t causal_type;   // 0 or 3
  int32_t window_left;   // raw (sentinels allowed)
  int32_t window_right;
};

struct DropoutArgs {
  float p;
  const uint64_t* seed_ptr;
  const uint64_t* offset1_ptr;
  uint64_t offset2;
};

struct FwdArgs {
  const void* q; const void* k; const void* v; const void* bias;
  void* out; float* lse;
  Strides3 sq, sk, sv, so;
  int64_t sb_z, sb_h, sb_m, sb_n;
  int32_t batch, hq, hk;
  int32_t head_dim;      // columns of Q and K (<= the compiled head dim; a multiple of 8 unless `elementwise`)
  int32_t head_dim_v;    // columns of V, Out and dOut (same bounds)
  int32_t elementwise;   // rows are not made of aligned 16-byte pieces: the vector-ALU kernels move single elements
  float sm_scale;
  SeqArgs seq;
  MaskArgs mask;
  DropoutArgs drop;
  uint64_t* seed_out; uint64_t* offset_out;
  int32_t* atomic_counter;
  int32_t num_cu;        // CUs of the device (host fills it in)
  int32_t num_m_tiles;
  int32_t num_zh;        // (batch or sequences) x q-heads
  int32_t zh_per_xcd;    // ceil(num_zh / 8)
  int32_t zh_group;      // heads walked together on one XCD
  int32_t items_per_xcd; // Q tiles (incl. padding of the last group) per XCD
};

struct BwdArgs {
  const void* q; const void* k; const void* v; const void* bias;
  const void* out; const void* dout;
  void* dq; void* dk; void* dv; void* db;
  const float* lse; float* delta;
  Strides3 sq, sk, sv, so, sdo, sdq, sdk, sdv;
  int64_t sb_z, sb_h, sb_m, sb_n;
  int64_t sdb_z, sdb_h, sdb_m, sdb_n;
  int32_t batch, hq, hk;
  int32_t head_dim;      // columns of Q and K (<= the compiled head dim; a multiple of 8 unless `elementwise`)
  int32_t head_dim_v;    // columns of V, Out and dOut (same bounds)
  int32_t elementwise;   // rows are not made of aligned 16-byte pieces: the vector-ALU kernels move single elements
  float sm_scale;
  SeqArgs seq;
  MaskArgs mask;
  DropoutArgs drop;
  int32_t num_m_tiles, num_n_tiles;
  int32_t num_zh;        // (batch or sequences) x heads of the launched kernel's grid
  int32_t zh_per_xcd;    // ceil(num_zh / 8)
  int32_t zh_group;      // heads walked together on one XCD
  int32_t num_cu;        // CUs of the device (host fills it in)
  int32_t items_per_xcd; // work items (incl. padding of the last group) per XCD
  // dS kept in HBM between the dK/dV kernel (writes it) and the dQ kernel that only does dQ = dS K:
  // tiles of 128 keys x (the dK/dV step's queries), ds_ntk x ds_ntq of them per (batch element, q-head)
  void* ds_ws;           // null: dS is not stored
  int32_t ds_ntq, ds_ntk;
  // with ds_ws: row statistics as that dK/dV kernel stages them, written by the delta kernel
  const float* lse_scaled;   // L / ln 2
  const float* delta_prep;   // -delta (delta with dropout)
};

// Copy between a rank-4 tensor of any strides and head dim (unit last stride) and its packed
// image: contiguous (n0, n1, n2, dp) with dp the head dim rounded up to a multiple of 8, zeros in
// the excess columns.
struct RepackArgs {
  void* strided; void* packed;
  int64_t s0, s1, s2;     // element strides of the strided tensor
  int32_t n0, n1, n2;
  int32_t d, dp;          // columns of the strided tensor / of the packed one
};

struct EncodedSoftmaxArgs {
  void* r; int64_t s_z, s_h, s_m;
  int32_t batch, heads, seqlen_q, seqlen_k;
  int32_t dtype;
  DropoutArgs drop;
};

}  // namespace fa
