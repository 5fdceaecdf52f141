// Backward flash-attention kernels for gfx950 (wave64, MFMA 32x32x16).
//
// What is computed follows the reference's split backward
//   delta   modules/flash/kernel/bwd_preprocess.py:28-250
//   dK, dV  modules/flash/kernel/bwd_kernel_dk_dv.py:48-417, bwd_inner_dk_dv.py:28-267
//   dQ, dB  modules/flash/kernel/bwd_kernel_dq.py:45-389, bwd_inner_dq.py:28-215
// and its single-launch variant modules/flash/kernel/bwd_kernel_fuse.py:49-665
// (grid.y split into dK/dV items and dQ items, delta recomputed inline).
// No atomics anywhere: every dK/dV tile and every dQ tile has exactly one owner.
//
// dK/dV item: a wave owns 32 keys (lane%32 = key), loops over Q tiles and over the
// q-heads of its GQA group:
//   S  (queries x keys) = Q_tile . K^T     A = Q rows from LDS,     B = K in registers
//   dP (queries x keys) = dO_tile . V^T    A = dO rows from LDS,    B = V in registers
//   dV^T (d x keys) += dO_tile^T . P       A = dO^T rows from LDS,  B = P from accumulators
//   dK^T (d x keys) += Q_tile^T . dS       A = Q^T rows from LDS,   B = dS from accumulators
// dQ item: a wave owns 32 queries (lane%32 = query), loops over K tiles:
//   S^T  (keys x queries) = K_tile . Q^T   A = K rows from LDS,     B = Q in registers
//   dP^T (keys x queries) = V_tile . dO^T  A = V rows from LDS,     B = dO in registers
//   dQ^T (d x queries) += K_tile^T . dS^T  A = K^T rows from LDS,   B = dS^T from accumulators
#pragma once
#include <type_traits>

#include "fa_device.h"
#include "fa_kernels.h"

namespace fa {

// ---------------------------------------------------------------------------
// delta = rowsum(O * dO) in fp32, same layout as LSE.
// ---------------------------------------------------------------------------
// kPrep: also writes what the dK/dV kernel that stores dS stages without touching it: L in base 2
// (BwdArgs::lse_scaled) and the initial value of its dP accumulators (delta_prep: -delta, or delta
// itself when dropout comes between dP and the subtraction).
template <typename T, int D, bool kPrep = false>
__global__ void bwd_preprocess_kernel(const BwdArgs a) {
  using op_t = typename Traits<T>::op_t;
  constexpr int LPR = D / 8;               // lanes per row
  constexpr int ROWS = 256 / LPR;
  const int tid = threadIdx.x;
  const int h = blockIdx.y, z = blockIdx.z;
  const SeqInfo si = get_seq(a.seq, z);
  const int row = blockIdx.x * ROWS + tid / LPR;
  const int cc = tid % LPR;
  float acc = 0.f;
  if (row < si.seqlen_q && cc * 8 < a.head_dim_v) {   // columns past the head dim of Out and dOut do not exist
    const int64_t ro = (int64_t)si.batch_index * a.so.z + (int64_t)h * a.so.h + (int64_t)(si.q_start + row) * a.so.s;
    const int64_t rd = (int64_t)si.batch_index * a.sdo.z + (int64_t)h * a.sdo.h + (int64_t)(si.q_start + row) * a.sdo.s;
    // (O is read here and nowhere else in the backward: a streaming load; dO stays cached for the dK/dV kernel)
    const op_t o = __builtin_nontemporal_load(reinterpret_cast<const op_t*>(reinterpret_cast<const T*>(a.out) + ro + cc * 8));
    const op_t d = *reinterpret_cast<const op_t*>(reinterpret_cast<const T*>(a.dout) + rd + cc * 8);
#pragma unroll
    for (int e = 0; e < 8; ++e) acc += (float)o[e] * (float)d[e];
  }
#pragma unroll
  for (int off = LPR / 2; off > 0; off >>= 1) acc += __shfl_xor(acc, off, 64);
  if (row < si.seqlen_q && cc == 0) {
    const int64_t at = lse_offset(si, h, a.hq) + row;
    a.delta[at] = acc;
    if constexpr (kPrep) {
      const_cast<float*>(a.lse_scaled)[at] = a.lse[at] * kRcpLn2;          // bwd_inner_dk_dv.py:185-186
      const_cast<float*>(a.delta_prep)[at] = a.drop.p > 0.f ? acc : -acc;
    }
  }
}

// ---------------------------------------------------------------------------
// Shared-memory plans
// ---------------------------------------------------------------------------
// Every staged tile is row-major, unpadded and swizzled (Swz in fa_device.h): the same
// copy serves the 16-byte row reads of the GEMMs that contract over the head dim and
// the transposing reads of the GEMMs that contract over the tile's rows, both free
// of bank conflicts.  Q and dO (dK/dV item) and K (dQ item) are read both ways.
template <int D, int BM>
struct DkDvSmem {   // per stage: Q, dO (swizzled, one copy each); L, delta; bias tile (BM x 128 keys)
  static constexpr int TILE_BYTES = BM * D * 2;
  static constexpr int BIAS_STR = 128 * 2 + 16;       // bytes per bias row: rows 4 apart land 16 banks apart
  static constexpr int BIAS_BYTES = BM * BIAS_STR;
  static constexpr int STAGE_BYTES = 2 * TILE_BYTES + 2 * BM * 4 + BIAS_BYTES;
  static constexpr int STAGES = 2;
  // D = 256: the registers cannot hold both K and V of the wave's keys next to the dK and dV
  // accumulators, so the workgroup's V tile (128 keys) stays in LDS for the whole item
  static constexpr int V_OFF = STAGES * STAGE_BYTES;
  static constexpr int V_BYTES = D >= 256 ? 128 * D * 2 : 0;
  static constexpr int BYTES = V_OFF + V_BYTES;
};

template <int D, int BN>
struct DqSmem {     // per stage: K, V (swizzled); then one bias / dB tile per wave (32 rows, +16 B per row)
  static constexpr int TILE_BYTES = BN * D * 2;
  static constexpr int STAGE_BYTES = 2 * TILE_BYTES;
  static constexpr int STAGES = 2;
  static constexpr int BIAS_OFF = STAGES * STAGE_BYTES;
  static constexpr int BIAS_ROW = BN * 2 + 16;
  static constexpr int BYTES = BIAS_OFF + 4 * 32 * BIAS_ROW;
};

// Tile table of the backward kernels, keyed on (element type, head dim, causal / windowed).  NW
// waves; dK/dV: 32*NW keys per workgroup, DKDV_BM queries per step; dQ: 32*NW queries per
// workgroup, DQ_BN keys per step.  The reference keeps separate tuned tiles for causal and
// non-causal shapes (its database has 64x16 / 64x32 for dK/dV and 64x64 / 64x32 for dQ at the
// headline shape); here the same tile wins on both sides of every key (same-box A/B at D = 128,
// bf16: 32-query / 32-key steps lose 6 % causal and 7-10 % non-causal on each kernel).
template <typename T, int D, bool kWindowed> struct BwdTile;
template <typename T, bool kWindowed> struct BwdTile<T, 64, kWindowed>  { static constexpr int NW = 4, DKDV_BM = 128, DQ_BN = 128; };
template <typename T, bool kWindowed> struct BwdTile<T, 128, kWindowed> { static constexpr int NW = 4, DKDV_BM = 64, DQ_BN = 64; };
template <typename T, bool kWindowed> struct BwdTile<T, 256, kWindowed> { static constexpr int NW = 4, DKDV_BM = 32, DQ_BN = 32; };

// Stored dS (BwdArgs::ds_ws): one tile per (batch element, q-head, key tile of 128, query tile of the
// dK/dV step) holds 128 x BM values of the 16-bit type as [32-query block][32-key block][half of the
// query block][64 pieces of 16 bytes].  A piece is what one lane of the dK/dV item holds as the MFMA
// operand of its 16-query step t (query block t / 2, half t % 2): its key c (lane % 32) against the
// queries 16 t + 4 hi + {0..3} and 16 t + 8 + 4 hi + {0..3} (hi = lane / 32); it sits at piece position
// (2 c + hi) ^ 8 (t & 1), where the transposing LDS reads of the kernel that consumes the tiles want
// it.  A wave of that kernel owns one query block: what it needs of a tile is contiguous.
template <typename T, int D> struct DsTile {
  static_assert(BwdTile<T, D, false>::DKDV_BM == BwdTile<T, D, true>::DKDV_BM, "one tile shape per head dim");
  static constexpr int BM = BwdTile<T, D, false>::DKDV_BM;   // queries per stored tile
  static constexpr int BN = 128;                             // keys per stored tile
  static constexpr int TS = BM / 16;                         // 1 KB pieces per 32-key block
  static constexpr int BYTES = BN * BM * 2;
  static constexpr int QBLOCK_BYTES = BN * 32 * 2;           // one 32-query block against the tile's keys
  // byte offset of the piece of 32-key block kw and 16-query step t
  static constexpr int piece(int kw, int t) { return (t >> 1) * QBLOCK_BYTES + kw * 2048 + (t & 1) * 1024; }
};

// ---------------------------------------------------------------------------
// dK / dV work item
// ---------------------------------------------------------------------------
// kStoreDs: dS of every visited tile pair is also written to BwdArgs::ds_ws, and the row statistics
// come prepared (BwdArgs::lse_scaled, delta_prep) so that they can travel straight into LDS.
template <typename T, int D, int NW, int BM, bool kWindowed, bool kBias, bool kDropout, bool kInlineDelta, bool kPad,
          bool kStoreDs = false>
__device__ __forceinline__ void dkdv_item(const BwdArgs& a, const int hk, const int nt, const int z,
                                          char* smem_raw) {
  using Tr = Traits<T>;
  using op_t = typename Tr::op_t;
  using q4_t = typename Tr::q4_t;
  using SM = DkDvSmem<D, BM>;
  constexpr int NT = NW * 64;
  constexpr int BN = NW * 32;
  constexpr int KS = D / 16, MB = BM / 32, DB = D / 32, TS = BM / 16;
  constexpr int NCH = BM * D / 8;                // 16-byte chunks per tile, per tensor
  constexpr int CH = (NCH + NT - 1) / NT;        // chunks per thread, per tensor
  constexpr int LPR = D / 8;                     // lanes that share one row

  const int tid = threadIdx.x;
  const int wave = tid >> 6, lane = tid & 63, c = lane & 31, hi = lane >> 5;
  const int wave_u = __builtin_amdgcn_readfirstlane(tid >> 6);
  // columns of Q/K/dQ/dK and of V/Out/dOut/dV: <= D, multiples of 8; constants unless a head dim is rounded up
  const int d_qk = kPad ? a.head_dim : D, d_v = kPad ? a.head_dim_v : D;

  const SeqInfo si = get_seq(a.seq, z);
  const int n0 = nt * BN;
  if (n0 >= si.seqlen_k) return;

  Window w{0, 0};
  if (kWindowed) w = parse_window(a.mask.causal_type, a.mask.window_left, a.mask.window_right,
                                  si.seqlen_q, si.seqlen_k);
  w.left = w.left > (1 << 30) ? (1 << 30) : (w.left < -(1 << 30) ? -(1 << 30) : w.left);
  w.right = w.right > (1 << 30) ? (1 << 30) : (w.right < -(1 << 30) ? -(1 << 30) : w.right);
  // Rows are keys here, columns are queries: key n sees query m iff n - right <= m <= n + left
  // (bwd_kernel_dk_dv.py:268-279 passes the window transposed in the same way).
  const BlockRanges br = block_ranges(kWindowed, w.right, w.left, n0, si.seqlen_k, si.seqlen_q, BN, BM);

  const int key = n0 + wave * 32 + c;
  const bool key_ok = key < si.seqlen_k;
  const int key_c = key_ok ? key : si.seqlen_k - 1;
  T* dkptr = reinterpret_cast<T*>(a.dk) + (int64_t)si.batch_index * a.sdk.z + (int64_t)hk * a.sdk.h +
             (int64_t)(si.k_start + key_c) * a.sdk.s;
  T* dvptr = reinterpret_cast<T*>(a.dv) + (int64_t)si.batch_index * a.sdv.z + (int64_t)hk * a.sdv.h +
             (int64_t)(si.k_start + key_c) * a.sdv.s;

  if (br.lo > br.hi) {   // no query sees these keys
    if (key_ok) {
      q4_t zero4 = {0, 0, 0, 0};
#pragma unroll
      for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          if (32 * db + 8 * g + 4 * hi < d_qk) *reinterpret_cast<q4_t*>(dkptr + 32 * db + 8 * g + 4 * hi) = zero4;
          if (32 * db + 8 * g + 4 * hi < d_v) *reinterpret_cast<q4_t*>(dvptr + 32 * db + 8 * g + 4 * hi) = zero4;
        }
    }
    return;
  }

  // Queries that see this lane's key form one range [q_lo, q_lo + q_rng] (none: q_none): a masked
  // tile then tests an element with one unsigned comparison (fwd_kernel_inner.py:140-160 states the
  // predicate per element: key <= m + right, key >= m - left, both inside their sequences).
  int q_lo = 0, q_hi = si.seqlen_q - 1;
  if (kWindowed) {
    q_lo = key - w.right > 0 ? key - w.right : 0;
    q_hi = key + w.left < q_hi ? key + w.left : q_hi;
  }
  const bool q_none = !key_ok || q_hi < q_lo;
  const unsigned q_rng = q_none ? 0u : (unsigned)(q_hi - q_lo);

  // K and V rows of this lane's key as B operands (k = head dim)
  const T* kptr = reinterpret_cast<const T*>(a.k) + (int64_t)si.batch_index * a.sk.z + (int64_t)hk * a.sk.h +
                  (int64_t)(si.k_start + key_c) * a.sk.s;
  const T* vptr = reinterpret_cast<const T*>(a.v) + (int64_t)si.batch_index * a.sv.z + (int64_t)hk * a.sv.h +
                  (int64_t)(si.k_start + key_c) * a.sv.s;
  constexpr bool kVLds = SM::V_BYTES > 0;       // V operands come from LDS instead of registers
  op_t kreg[KS], vreg[kVLds ? 1 : KS];
#pragma unroll
  for (int k = 0; k < KS; ++k) {
    // columns past the tensors' head dim are zero (head dims are rounded up to D)
    const op_t zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
    kreg[k] = 16 * k + 8 * hi < d_qk ? *reinterpret_cast<const op_t*>(kptr + 16 * k + 8 * hi) : zero8;
    if (!kVLds) vreg[k] = 16 * k + 8 * hi < d_v ? *reinterpret_cast<const op_t*>(vptr + 16 * k + 8 * hi) : zero8;
  }

  f32x16 dk[DB], dv[DB];
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int i = 0; i < 16; ++i) { dk[db][i] = 0.f; dv[db][i] = 0.f; }

  const int group = a.hq / a.hk;
  const int ntq = br.hi - br.lo + 1;
  const int total = group * ntq;
  const float qk_scale = a.sm_scale * kLog2e;
  // lane constants of the two LDS access patterns
  const int row_a = Swz<D>::row_base(lane), tr_a0 = Swz<D>::tr_base(lane, 0), tr_a1 = Swz<D>::tr_base(lane, 1);

  auto stage_ptr = [&](int stage) { return smem_raw + stage * SM::STAGE_BYTES; };

  // dS of every visited (key tile, query tile) pair goes out to HBM for the kernel that forms dQ from
  // it: the operand registers of the dK GEMM as they are, 1 KB per wave instruction.  A store counts
  // in vmcnt until the L2 has taken it, which takes 1700-1900 cycles for a line that misses; loads
  // and stores complete out of order with respect to each other, so the next wait for a load is a
  // wait for every store before it.  The tile therefore has ONE wait for vector memory, in its
  // middle (where the compiler makes the first transposing read wait for the direct-to-LDS pieces
  // anyway), and the pieces leave in the half tile after it, as their operands get complete: the
  // youngest store is more than half a tile old at the next wait.
  using DT = DsTile<T, D>;
  static_assert(!kStoreDs || (!kInlineDelta && BM == DT::BM && BN == DT::BN), "stored tiles have the item's shape");
  const int ds_pos[2] = {((c << 1) | hi) << 4, (((c << 1) | hi) ^ 8) << 4};
  op_t sb[TS];                         // dS operands of the dK GEMM; with kStoreDs they outlive their tile
  char* ds_tile = nullptr;             // stored tile of the running (q-head, Q tile) step
  constexpr int kDsSlots = 4;
  // cache policy bits of the stores: non-temporal (the tile is read once, by another kernel) at agent scope;
  // measured against the other combinations of sc0 / sc1 / nt on one box: 1-2 % of the kernel
  constexpr int kDsStorePolicy = 2 | 16;
  auto ds_slot_of = [](int t) { return TS >= kDsSlots ? t * kDsSlots / TS : 2 * t + 1; };
  auto store_ds_slot = [&](char* tile, int slot) {
    if constexpr (kStoreDs) {
      const auto rs = wave_rsrc(tile, tile != nullptr ? DT::BYTES : 0);
#pragma unroll
      for (int t = 0; t < TS; ++t)
        if (ds_slot_of(t) == slot)
          __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4_t, sb[t]), rs, ds_pos[t & 1],
                                                 DT::piece(0, t) + wave_u * 2048, kDsStorePolicy);
    }
  };

  // ---- staging -----------------------------------------------------------------
  // Q and dO tiles travel global -> registers -> LDS in 16-byte pieces.  The pieces
  // are issued between the MFMAs of the running tile (loads behind S = Q K^T, LDS
  // writes behind dK^T += Q^T dS), so staging costs no issue time of its own.
  // Buffer loads with a descriptor rebased on every tile: rows past the end of the
  // sequence read as zero, and a descriptor of zero records turns the fetch after
  // the last tile into a no-op.
  static_assert(NCH % NT == 0, "threads must cover the tile evenly");
  constexpr int RPI = NT / LPR;                  // rows between two pieces of one thread
  // The Q and dO pieces go from global memory straight into the LDS stage (no staging registers
  // and no LDS write instructions: 3-5 % at D = 64 and 128; at D = 256 the staging registers,
  // next to 256 accumulators, the K operands and the softmax state, were what pushed the K
  // operands out to scratch, and a scratch reload waits for every load in flight).  A wave
  // instruction fills 1 KB of consecutive LDS, 64 / LPR rows; the swizzle is applied on the
  // global side: the lane at chunk position p of row r fetches chunk p ^ f(r).  Lanes outside the
  // descriptor's range deliver zeros.  The pieces count in vmcnt like any load; the compiler makes
  // the first transposing LDS read after them wait for all of them (mid-tile: they have landed).
  // The fused kernel computes delta from the staged O and dO registers and keeps them.
  constexpr bool kDirect = !kInlineDelta;
  constexpr int RWI = 64 / LPR;                  // rows one wave instruction covers
  op_t qch[kDirect ? 1 : CH], doch[kDirect ? 1 : CH], och[kInlineDelta ? CH : 1];
  float l_stage = 0.f, d_stage = 0.f;
  const int r0 = tid / LPR, cc0 = tid % LPR;
  int f_stage = 0;                               // stage the running fetch fills
  // f(r0 + k RPI) takes at most two values, for even and odd k (RPI is a multiple of 8, f has period 16)
  int q_voff_d[2] = {0, 0}, do_voff_d[2] = {0, 0};
  if (kDirect) {
    static_assert(!kDirect || RPI % 8 == 0, "the swizzle must repeat every two pieces");
#pragma unroll
    for (int k = 0; k < 2; ++k) {
      const int gch = cc0 ^ Swz<D>::f(r0 + k * RPI);
      q_voff_d[k] = gch * 8 < d_qk ? r0 * (int)a.sq.s * 2 + gch * 16 : kVoffOutOfRange;
      do_voff_d[k] = gch * 8 < d_v ? r0 * (int)a.sdo.s * 2 + gch * 16 : kVoffOutOfRange;
    }
  }
  using lds_ptr_t = __attribute__((address_space(3))) void*;
  const int q_voff = cc0 * 8 < d_qk ? r0 * (int)a.sq.s * 2 + cc0 * 16 : kVoffOutOfRange,       // bytes inside a tile
            do_voff = cc0 * 8 < d_v ? r0 * (int)a.sdo.s * 2 + cc0 * 16 : kVoffOutOfRange,
            o_voff = cc0 * 8 < d_v ? r0 * (int)a.so.s * 2 + cc0 * 16 : kVoffOutOfRange;
  const int q_soff = RPI * (int)a.sq.s * 2, do_soff = RPI * (int)a.sdo.s * 2, o_soff = RPI * (int)a.so.s * 2;
  int lds_off[CH];                                                        // bytes inside a tile
#pragma unroll
  for (int k = 0; k < CH; ++k) lds_off[k] = Swz<D>::addr(r0 + k * RPI, cc0);

  // Tile base pointers advance incrementally (one 64-bit add per tensor and tile);
  // with one wave per SIMD a chain of scalar multiplies per tile is not hidden.
  const int64_t q_tile_step = (int64_t)BM * a.sq.s, do_tile_step = (int64_t)BM * a.sdo.s,
                o_tile_step = (int64_t)BM * a.so.s;
  const T* qb = nullptr; const T* dob = nullptr; const T* ob = nullptr;
  const float* lse_b = nullptr; const float* delta_b = nullptr;
  auto set_head = [&](int g) {
    const int hq = hk * group + g;
    const int64_t row0 = (int64_t)si.q_start + (int64_t)br.lo * BM;
    qb = reinterpret_cast<const T*>(a.q) + (int64_t)si.batch_index * a.sq.z + (int64_t)hq * a.sq.h + row0 * a.sq.s;
    dob = reinterpret_cast<const T*>(a.dout) + (int64_t)si.batch_index * a.sdo.z + (int64_t)hq * a.sdo.h +
          row0 * a.sdo.s;
    if (kInlineDelta)
      ob = reinterpret_cast<const T*>(a.out) + (int64_t)si.batch_index * a.so.z + (int64_t)hq * a.so.h +
           row0 * a.so.s;
    lse_b = (kStoreDs ? a.lse_scaled : a.lse) + lse_offset(si, hq, a.hq) + (int64_t)br.lo * BM;
    if (!kInlineDelta) delta_b = (kStoreDs ? a.delta_prep : a.delta) + lse_offset(si, hq, a.hq) + (int64_t)br.lo * BM;
  };
  __amdgpu_buffer_rsrc_t q_rs, do_rs, o_rs, b_rs;
  // The bias tile (BM queries x the workgroup's 128 keys) is staged through LDS like Q
  // and dO when its layout allows 16-byte loads; otherwise elements are loaded directly.
  static_assert(BN == 128, "bias staging assumes 128 keys per workgroup");
  constexpr int CHB = kBias ? (BM * 16) / NT : 0;        // 16-byte bias pieces per thread
  const bool bias_lds = kBias && a.sb_n == 1 && ((a.sb_m | a.sb_h | a.sb_z) & 7) == 0 &&
                        (reinterpret_cast<uintptr_t>(a.bias) & 15) == 0;
  op_t bch[CHB > 0 ? CHB : 1];
  const int b_voff = (tid / 16) * (int)a.sb_m * 2 + (tid % 16) * 16;   // bytes inside a bias tile
  const int b_soff = (NT / 16) * (int)a.sb_m * 2;
  const int b_lds = (tid / 16) * SM::BIAS_STR + (tid % 16) * 16;
  const T* bb = nullptr;
  const T* bb_tile = nullptr;     // bias tile being fetched, its valid rows
  int b_rows = 0;
  const int b_cols = si.seqlen_k - n0 < BN ? si.seqlen_k - n0 : BN;      // valid keys of this item
  const bool bias_plain = bias_lds && (b_cols & 7) == 0;                 // no piece straddles the end of a row
  // (g, e) = (q-head inside the GQA group, Q tile inside the range) of the tile to fetch;
  // called for consecutive tiles only; `live` false: nothing is fetched
  auto fetch_begin = [&](bool live, int g, int e) {
    if (live && e == 0) set_head(g);
    const int m0 = (br.lo + e) * BM;
    int rows = si.seqlen_q - m0 < BM ? si.seqlen_q - m0 : BM;
    rows = live ? rows : 0;
    const bool any = rows > 0;
    if (kBias) {
      if (live && e == 0)
        bb = reinterpret_cast<const T*>(a.bias) + (int64_t)si.batch_index * a.sb_z +
             (int64_t)(hk * group + g) * a.sb_h + (int64_t)br.lo * BM * a.sb_m + (int64_t)n0 * a.sb_n;
      bb_tile = bb;
      b_rows = rows;
      b_rs = wave_rsrc(bb, any && bias_lds ? ((rows - 1) * (int)a.sb_m + b_cols) * 2 : 0);
      if (live) bb += (int64_t)BM * a.sb_m;
    }
    q_rs = wave_rsrc(qb, any ? ((rows - 1) * (int)a.sq.s + d_qk) * 2 : 0);
    do_rs = wave_rsrc(dob, any ? ((rows - 1) * (int)a.sdo.s + d_v) * 2 : 0);
    if (kInlineDelta)
      o_rs = wave_rsrc(ob, any ? ((rows - 1) * (int)a.so.s + d_v) * 2 : 0);
    if constexpr (kStoreDs) {
      // the prepared statistics (L log2e; -delta, or delta with dropout) go straight into the stage:
      // no register load in the loop, hence no wait of the compiler's for one at the end of a tile
      // (16 bytes per lane: BM / 4 lanes of wave 0 fetch each array)
      if (tid < BM / 4) {
        const auto l_rs = wave_rsrc(lse_b, rows * 4);
        const auto d_rs = wave_rsrc(delta_b, rows * 4);
        char* st = stage_ptr(f_stage) + 2 * SM::TILE_BYTES;
        __builtin_amdgcn_raw_ptr_buffer_load_lds(l_rs, (lds_ptr_t)st, 16, lane * 16, 0, 0, 0);
        __builtin_amdgcn_raw_ptr_buffer_load_lds(d_rs, (lds_ptr_t)(st + BM * 4), 16, lane * 16, 0, 0, 0);
      }
    } else if (tid < BM) {
      const bool ok = tid < rows;
      l_stage = ok ? lse_b[tid] : 0.f;
      if (!kInlineDelta) d_stage = ok ? delta_b[tid] : 0.f;
    }
    if (live) {
      qb += q_tile_step; dob += do_tile_step; lse_b += BM;
      if (kInlineDelta) ob += o_tile_step; else delta_b += BM;
    }
  };
  constexpr int FETCH_PIECES = 2 * CH + CHB;
  auto fetch_piece = [&](int i) {        // Q pieces first, then dO (and O), then bias
    if (i >= 2 * CH) {
      const int k = i - 2 * CH;
      if (bias_plain) {
        // (the usual case behind one scalar branch: the two below test per lane)
        bch[k] = __builtin_bit_cast(op_t, __builtin_amdgcn_raw_buffer_load_b128(b_rs, b_voff, k * b_soff, 0));
      } else if (bias_lds) {
        bch[k] = __builtin_bit_cast(op_t, __builtin_amdgcn_raw_buffer_load_b128(b_rs, b_voff, k * b_soff, 0));
        // The descriptor ends at the last valid element of the tile's last row.  When that is
        // not at a 16-byte boundary the piece that straddles the end loses its valid elements
        // to the range check too (a dword that holds the last of an odd number of columns reads
        // as zero): that one piece is gathered element by element.
        const int row = tid / 16 + k * (NT / 16), col = (tid % 16) * 8;
        if ((b_cols & 7) != 0 && row == b_rows - 1 && col < b_cols && col + 8 > b_cols) {
          op_t x;
#pragma unroll
          for (int e = 0; e < 8; ++e)
            x[e] = col + e < b_cols ? bb_tile[(int64_t)row * a.sb_m + col + e] : Tr::cvt(0.f);
          bch[k] = x;
        }
      } else {
        // any other layout: the piece is gathered element by element
        const int row = tid / 16 + k * (NT / 16), col = (tid % 16) * 8;
        op_t x;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const bool ok = row < b_rows && n0 + col + e < si.seqlen_k;
          x[e] = ok ? bb_tile[(int64_t)row * a.sb_m + (int64_t)(col + e) * a.sb_n] : Tr::cvt(0.f);
        }
        bch[k] = x;
      }
    } else if (i < CH) {
      if constexpr (kDirect) {
        __builtin_amdgcn_raw_ptr_buffer_load_lds(
            q_rs, (lds_ptr_t)(stage_ptr(f_stage) + (i * RPI + RWI * wave_u) * Swz<D>::ROWB), 16, q_voff_d[i & 1],
            i * q_soff, 0, 0);
      } else {
        qch[i] = __builtin_bit_cast(op_t, __builtin_amdgcn_raw_buffer_load_b128(q_rs, q_voff, i * q_soff, 0));
      }
    } else {
      const int k = i - CH;
      if constexpr (kDirect) {
        __builtin_amdgcn_raw_ptr_buffer_load_lds(
            do_rs, (lds_ptr_t)(stage_ptr(f_stage) + SM::TILE_BYTES + (k * RPI + RWI * wave_u) * Swz<D>::ROWB), 16,
            do_voff_d[k & 1], k * do_soff, 0, 0);
      } else {
        doch[k] = __builtin_bit_cast(op_t, __builtin_amdgcn_raw_buffer_load_b128(do_rs, do_voff, k * do_soff, 0));
      }
      if (kInlineDelta)
        och[k] = __builtin_bit_cast(op_t, __builtin_amdgcn_raw_buffer_load_b128(o_rs, o_voff, k * o_soff, 0));
    }
  };
  // all of this wave's direct pieces have landed (vmcnt 0; the other counters stay as they are)
  auto direct_landed = [&]() {
    if constexpr (kDirect) __builtin_amdgcn_s_waitcnt(0x0F70);
  };
  constexpr int STORE_PIECES = 2 * CH + CHB;
  auto store_piece = [&](int i, int stage) {   // same order as the fetches
    char* sp = stage_ptr(stage);
    if (i >= 2 * CH)
      *reinterpret_cast<op_t*>(sp + 2 * SM::TILE_BYTES + 2 * BM * 4 + b_lds + (i - 2 * CH) * (NT / 16) * SM::BIAS_STR) =
          bch[i - 2 * CH];
    else if (kDirect) return;
    else if (i < CH) *reinterpret_cast<op_t*>(sp + lds_off[i]) = qch[i];
    else *reinterpret_cast<op_t*>(sp + SM::TILE_BYTES + lds_off[i - CH]) = doch[i - CH];
  };
  auto store_stats = [&](int stage) {
    char* sp = stage_ptr(stage);
    float* Ls = reinterpret_cast<float*>(sp + 2 * SM::TILE_BYTES);
    float* Ds = Ls + BM;
    if (kInlineDelta) {
      // delta recomputed from O and dO (bwd_kernel_fuse.py:307-310); the LPR threads
      // that share a row are consecutive lanes
#pragma unroll
      for (int k = 0; k < CH; ++k) {
        float acc = 0.f;
#pragma unroll
        for (int e = 0; e < 8; ++e) acc += (float)och[k][e] * (float)doch[k][e];
#pragma unroll
        for (int off = LPR / 2; off > 0; off >>= 1) acc += __shfl_xor(acc, off, 64);
        if (cc0 == 0) Ds[r0 + k * RPI] = kDropout ? acc : -acc;
      }
    }
    if (!kStoreDs && tid < BM) {
      Ls[tid] = l_stage * kRcpLn2;                          // bwd_inner_dk_dv.py:185-186
      // without dropout -delta is staged: it is the initial value of the dP accumulators
      if (!kInlineDelta) Ds[tid] = kDropout ? d_stage : -d_stage;
    }
  };

  // seed and offset of the dropout mask: read once per item, not once per tile
  DropoutState drop0{};
  if (kDropout) drop0 = make_dropout_base(a.drop, a.seq.max_seqlen_k);

  // ---- one (q-head, Q tile) step -----------------------------------------------
  auto compute = [&](auto masked_tag, int g, int e, int stage, bool live, int g_nxt, int e_nxt) {
    constexpr bool masked = decltype(masked_tag)::value;
    constexpr int G1 = KS * MB, G4 = TS * DB;
    const int hq = hk * group + g;
    const int m0 = (br.lo + e) * BM;
    char* sp = stage_ptr(stage);
    const char* Qb = sp;
    const char* dOb = sp + SM::TILE_BYTES;
    const float* Ls = reinterpret_cast<const float*>(sp + 2 * SM::TILE_BYTES);
    const float* Ds = Ls + BM;
    // The staged bias tile is row-major (queries x keys) and a lane needs its key's column: a
    // transposing read hands each lane four consecutive queries of its key (lane i of a group of
    // 16 gets, in slot j, element i % 4 of the 8 bytes addressed by lane 4 j + i / 4).
    const char* Bt = sp + 2 * SM::TILE_BYTES + 2 * BM * 4 + (4 * hi + (lane & 15) / 4) * SM::BIAS_STR +
                     (wave * 32 + 16 * ((lane >> 4) & 1) + 4 * (lane & 3)) * 2;

    f32x16 s[MB], dp[MB];
    const f32x16 zero16 = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};

    DropoutState dst{};
    if (kDropout) dst = dropout_for_head(drop0, z, hq, a.hq, a.seq.max_seqlen_q);
    if constexpr (kStoreDs) {
      // (the tiles of a q-head follow each other)
      ds_tile = e == 0 ? reinterpret_cast<char*>(a.ds_ws) +
                             ((((int64_t)z * a.hq + hq) * a.ds_ntk + nt) * a.ds_ntq + br.lo) * DT::BYTES
                       : ds_tile + DT::BYTES;
    }

    // The vector ALU work is spread over the MFMAs of the GEMMs that do not depend on
    // it: p = exp2(...) of S runs behind the MFMAs of dP, ds = p (dP - delta) behind
    // those of dV.  Fences keep the hand-made order.
    constexpr int kAhead = D >= 256 ? 1 : 2;
    op_t xa[kAhead + 1][MB];
    op_t pb[TS];
    uint32_t kw[kDropout ? MB : 1][4];
    // row statistics are read four rows at a time, one read ahead of their use
    f32x4 l4[2], d4[2];
    auto stat_ptr = [&](const float* base, int q) { return base + 32 * (q / 4) + 8 * (q % 4) + 4 * hi; };

    // ---- S = Q K^T ---------------------------------------------------------------
#pragma unroll
    for (int k = 0; k < kAhead; ++k)
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) xa[k][mb] = swz_read_row<T, D>(Qb, row_a, k, mb);
    if (!kDropout) {
      // dP starts at -delta of its query rows, so dP - delta leaves the matrix pipe; with
      // dropout the mask and the scale come between the two and the subtraction stays in ds_el
#pragma unroll
      for (int mb = 0; mb < MB; ++mb)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          const f32x4 t4 = *reinterpret_cast<const f32x4*>(stat_ptr(Ds, 4 * mb + g));
#pragma unroll
          for (int r = 0; r < 4; ++r) dp[mb][4 * g + r] = t4[r];
        }
    }
#pragma unroll
    // (the operand ring runs on from the Q rows of S into the dO rows of dP: the first dO operands are
    // requested behind the last MFMAs of S instead of in front of the first ones of dP)
    for (int k = 0; k < KS; ++k) {
#pragma unroll
      for (int mb = 0; mb < MB; ++mb)
        xa[(k + kAhead) % (kAhead + 1)][mb] = k + kAhead < KS ? swz_read_row<T, D>(Qb, row_a, k + kAhead, mb)
                                                              : swz_read_row<T, D>(dOb, row_a, k + kAhead - KS, mb);
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) {
        s[mb] = Tr::mfma(xa[k % (kAhead + 1)][mb], kreg[k], k == 0 ? zero16 : s[mb]);
        // the next tile's descriptors and global loads ride behind these MFMAs
        constexpr int every = G1 / FETCH_PIECES > 0 ? G1 / FETCH_PIECES : 1;
        const int gidx = k * MB + mb;
        if (gidx == 0) { f_stage = stage ^ 1; fetch_begin(live, g_nxt, e_nxt); }
        if (kDropout) {
          // One Philox call yields the keep bits of 4 consecutive keys, i.e. of the 4
          // lanes of a quad, for one row: quad lane q runs the calls of the rows with
          // m % 4 == q (8 per tile of 64 rows instead of 32) and the bits are exchanged
          // with quad broadcasts when they are used.
          constexpr int calls = 4 * MB, stride = G1 / calls > 0 ? G1 / calls : 1;
          if (gidx % stride == 0 && gidx / stride < calls) {
            const int cidx = gidx / stride;
            kw[cidx / 4][cidx % 4] =
                dropout_keep4(dst, m0 + 32 * (cidx / 4) + 8 * (cidx % 4) + 4 * hi + (lane & 3), key & ~3);
          }
        }
        if (gidx % every == every - 1) {
#pragma unroll
          for (int q = 0; q < (FETCH_PIECES + G1 - 1) / G1; ++q) {
            const int piece = gidx / every * ((FETCH_PIECES + G1 - 1) / G1) + q;
            if (piece < FETCH_PIECES) fetch_piece(piece);
          }
        }
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    // row statistics of the tile's queries and the first dO operands
    l4[0] = *reinterpret_cast<const f32x4*>(stat_ptr(Ls, 0));
    // D = 256 has no registers for the whole column: there the reads run one ahead of their use
    constexpr bool kBiasRing = D >= 256;
    typename Tr::q4_t bias4[kBias ? (kBiasRing ? 2 : 4 * MB) : 1];
    auto bias_read = [&](int q) {
      return Tr::lds_read_tr(reinterpret_cast<const T*>(Bt + (32 * (q / 4) + 8 * (q % 4)) * SM::BIAS_STR));
    };
    if (kBias) {
      if (kBiasRing) {
        bias4[0] = bias_read(0);
      } else {
#pragma unroll
        for (int q = 0; q < 4 * MB; ++q) bias4[q] = bias_read(q);
      }
    }
    const char* Vt = smem_raw + SM::V_OFF;
    op_t vl[3];          // ring of V operands when they come from LDS
    if (kVLds) {
      vl[0] = swz_read_row<T, D>(Vt, row_a, 0, wave);
      vl[1] = swz_read_row<T, D>(Vt, row_a, 1, wave);
    }

    // element E = 16*mb + i of the tile: p (kept in s, undropped) and its operand form
    const unsigned q_d = q_none ? 0x40000000u : (unsigned)(m0 + 4 * hi - q_lo);
    auto p_el = [&](int E) {
      const int mb = E / 16, i = E % 16, g = i / 4, r = i % 4;
      if (E % 4 == 0 && E + 4 < 16 * MB) l4[(E / 4 + 1) & 1] = *reinterpret_cast<const f32x4*>(stat_ptr(Ls, E / 4 + 1));
      // p = exp2(s*c + bias*log2e - L*log2e), one fma per element (bwd_inner_dk_dv.py:187-188)
      float x;
      if (kBias) {
        if (kBiasRing && E % 4 == 0 && E + 4 < 16 * MB) bias4[(E / 4 + 1) & 1] = bias_read(E / 4 + 1);
        const float bv = (float)bias4[kBiasRing ? (E / 4) & 1 : E / 4][r];
        x = __builtin_fmaf(s[mb][i], qk_scale, bv * kLog2e) - l4[(E / 4) & 1][r];
      } else {
        x = __builtin_fmaf(s[mb][i], qk_scale, -l4[(E / 4) & 1][r]);
      }
      if (masked) {
        // query m sees this lane's key iff q_lo <= m <= q_lo + q_rng; an empty range fails every element
        const bool vis = q_d + (unsigned)(32 * mb + 8 * g + r) <= q_rng;
        x = vis ? x : -__builtin_inff();
      }
      s[mb][i] = fast_exp2(x);
    };
    // keep bit of element E: held by the quad lane that ran the Philox call of its row
    auto keep_of = [&](int E) -> bool {
      const int mb = E / 16, g = (E % 16) / 4, r = E % 4;
      const int w = (int)kw[mb][g];
      int w4;
      switch (r) {       // quad_perm: [r, r, r, r]
        case 0: w4 = __builtin_amdgcn_mov_dpp(w, 0x00, 0xf, 0xf, true); break;
        case 1: w4 = __builtin_amdgcn_mov_dpp(w, 0x55, 0xf, 0xf, true); break;
        case 2: w4 = __builtin_amdgcn_mov_dpp(w, 0xaa, 0xf, 0xf, true); break;
        default: w4 = __builtin_amdgcn_mov_dpp(w, 0xff, 0xf, 0xf, true); break;
      }
      return ((uint32_t)w4 >> (lane & 3)) & 1u;
    };
    bool keep_bit[kDropout ? 16 * MB : 1];
    auto p_pair = [&](int E) {   // E odd: operand form of (E-1, E); dropout applies to the operand only
      float p0 = s[E / 16][E % 16 - 1], p1 = s[E / 16][E % 16];
      if (kDropout) {
        keep_bit[E - 1] = keep_of(E - 1);
        keep_bit[E] = keep_of(E);
        p0 = keep_bit[E - 1] ? p0 * dst.scale : 0.f;              // :200-201
        p1 = keep_bit[E] ? p1 * dst.scale : 0.f;
      }
      const typename Tr::p2_t p2 = Tr::cvt2(p0, p1);     // p cast to dO's dtype (composed_tensors.py:191-193)
      pb[E / 8][E % 8 - 1] = p2[0];
      pb[E / 8][E % 8] = p2[1];
    };
    auto ds_el = [&](int E) {
      const int mb = E / 16, i = E % 16, r = i % 4;
      if (!kDropout) {
        dp[mb][i] = s[mb][i] * dp[mb][i];                         // dp already holds dP - delta
        return;
      }
      if (E % 4 == 0 && E + 4 < 16 * MB) d4[(E / 4 + 1) & 1] = *reinterpret_cast<const f32x4*>(stat_ptr(Ds, E / 4 + 1));
      float dpv = dp[mb][i];
      dpv = keep_bit[E] ? dpv * dst.scale : 0.f;                  // :239-240
      dp[mb][i] = s[mb][i] * (dpv - d4[(E / 4) & 1][r]);          // ds uses the undropped p (:242)
    };
    auto ds_pair = [&](int E) {  // E odd: ds cast to Q's dtype
      const typename Tr::p2_t s2 = Tr::cvt2(dp[E / 16][E % 16 - 1], dp[E / 16][E % 16]);
      sb[E / 8][E % 8 - 1] = s2[0];
      sb[E / 8][E % 8] = s2[1];
    };

    // ---- dP = dO V^T, with p behind its MFMAs ------------------------------------
    constexpr int EPG1 = 16 * MB / (KS * MB);    // elements per MFMA (D = 128: 2)
    static_assert(16 * MB % (KS * MB) == 0 || KS * MB > 16 * MB, "element split");
#pragma unroll
    for (int k = 0; k < KS; ++k) {
      if (k + kAhead < KS) {
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
          xa[(KS + k + kAhead) % (kAhead + 1)][mb] = swz_read_row<T, D>(dOb, row_a, k + kAhead, mb);
      }
      if (kVLds && k + 2 < KS) vl[(k + 2) % 3] = swz_read_row<T, D>(Vt, row_a, k + 2, wave);
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) {
        dp[mb] = Tr::mfma(xa[(KS + k) % (kAhead + 1)][mb], kVLds ? vl[k % 3] : vreg[kVLds ? 0 : k],
                          k == 0 && kDropout ? zero16 : dp[mb]);
        const int gidx = k * MB + mb;
        if constexpr (EPG1 >= 1) {
#pragma unroll
          for (int e = 0; e < (EPG1 >= 1 ? EPG1 : 1); ++e) {
            const int E = gidx * EPG1 + e;
            p_el(E);
            if (E & 1) p_pair(E);
          }
        } else {
          // more MFMAs than elements (D = 256): one element every other MFMA
          constexpr int every = (KS * MB) / (16 * MB);
          if (gidx % every == 0) {
            const int E = gidx / every;
            p_el(E);
            if (E & 1) p_pair(E);
          }
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    // With stored dS this is the tile's only wait for vector memory: everything the S phase requested
    // for the next tile has arrived (the compiler makes the first transposing read below wait for
    // the direct-to-LDS pieces anyway), and the stores issued since the last wait are at least a
    // phase and a half old.
    if constexpr (kStoreDs) direct_landed();
    // delta of the tile's queries, first transposed dO operands
    if (kDropout) d4[0] = *reinterpret_cast<const f32x4*>(stat_ptr(Ds, 0));
    // Transposed operands are read ahead of their MFMAs: a whole 16-query step ahead, or,
    // where that would take too many registers (D = 256), through a ring of kRing operands.
    constexpr bool kRingTa = DB >= 8;
    constexpr int kRing = 4;
    op_t ta[kRingTa ? 1 : 2][kRingTa ? kRing : DB];
    auto ta_read = [&](const char* tile, int gidx) { return swz_read_tr<T, D>(tile, tr_a0, tr_a1, gidx / DB, gidx % DB); };
    if (kRingTa) {
#pragma unroll
      for (int gi = 0; gi < kRing - 1; ++gi) ta[0][gi] = ta_read(dOb, gi);
    } else {
#pragma unroll
      for (int db = 0; db < DB; ++db) ta[0][db] = swz_read_tr<T, D>(dOb, tr_a0, tr_a1, 0, db);
    }

    // ---- dV^T += dO^T P, with ds behind its MFMAs --------------------------------
    constexpr int G3 = TS * DB;
    constexpr int EPG3 = 16 * MB / G3;           // D = 128: 2
    static_assert(16 * MB % G3 == 0 || G3 > 16 * MB, "element split");
#pragma unroll
    for (int t = 0; t < TS; ++t) {
#pragma unroll
      for (int db = 0; db < DB; ++db) {
        const int gidx = t * DB + db;
        if (kRingTa) {
          if (gidx + kRing - 1 < TS * DB) ta[0][(gidx + kRing - 1) % kRing] = ta_read(dOb, gidx + kRing - 1);
          dv[db] = Tr::mfma(ta[0][gidx % kRing], pb[t], dv[db]);
        } else {
          // (the last step requests the first Q^T operands of the dK phase: TS is even, they land in ta[0])
          ta[(t + 1) & 1 & (kRingTa ? 0 : 1)][db] = t + 1 < TS ? swz_read_tr<T, D>(dOb, tr_a0, tr_a1, t + 1, db)
                                                               : swz_read_tr<T, D>(Qb, tr_a0, tr_a1, 0, db);
          dv[db] = Tr::mfma(ta[t & 1 & (kRingTa ? 0 : 1)][db], pb[t], dv[db]);
        }
        if constexpr (EPG3 >= 1) {
#pragma unroll
          for (int e = 0; e < (EPG3 >= 1 ? EPG3 : 1); ++e) {
            const int E = gidx * EPG3 + e;
            ds_el(E);
            if (E & 1) ds_pair(E);
          }
        } else {
          constexpr int every = G3 / (16 * MB);
          if (gidx % every == 0) {
            const int E = gidx / every;
            ds_el(E);
            if (E & 1) ds_pair(E);
          }
        }
        if (kStoreDs && TS >= kDsSlots && gidx == G3 / 2) store_ds_slot(ds_tile, 0);
        if (kStoreDs && gidx == 3 * G3 / 4) store_ds_slot(ds_tile, 1);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    if constexpr (kStoreDs && TS >= kDsSlots) store_ds_slot(ds_tile, 2);
    // ---- dK^T += Q^T dS ----------------------------------------------------------
    static_assert(TS % 2 == 0, "the dV phase leaves the first operands of this one in ta[0]");
    if (kRingTa) {
#pragma unroll
      for (int gi = 0; gi < kRing - 1; ++gi) ta[0][gi] = ta_read(Qb, gi);
    }
#pragma unroll
    for (int t = 0; t < TS; ++t) {
      if (!kRingTa && t + 1 < TS) {
#pragma unroll
        for (int db = 0; db < DB; ++db)
          ta[(t + 1) & 1 & (kRingTa ? 0 : 1)][db] = swz_read_tr<T, D>(Qb, tr_a0, tr_a1, t + 1, db);
      }
#pragma unroll
      for (int db = 0; db < DB; ++db) {
        if (kRingTa) {
          const int gidx = t * DB + db;
          if (gidx + kRing - 1 < TS * DB) ta[0][(gidx + kRing - 1) % kRing] = ta_read(Qb, gidx + kRing - 1);
          dk[db] = Tr::mfma(ta[0][gidx % kRing], sb[t], dk[db]);
        } else {
          dk[db] = Tr::mfma(ta[t & 1 & (kRingTa ? 0 : 1)][db], sb[t], dk[db]);
        }
        if (kStoreDs && t * DB + db == 2) store_ds_slot(ds_tile, 3);
        // the next tile's LDS writes ride behind these MFMAs
        constexpr int per = (STORE_PIECES + G4 - 1) / G4;
#pragma unroll
        for (int q = 0; q < per; ++q) {
          const int piece = (t * DB + db) * per + q;
          if (piece < STORE_PIECES) store_piece(piece, stage ^ 1);
        }
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    store_stats(stage ^ 1);
    if constexpr (!kStoreDs) direct_landed();
  };

  if (kVLds) {
    // the workgroup's V tile, rows past the sequence and columns past the head dim zero
    const T* vt = reinterpret_cast<const T*>(a.v) + (int64_t)si.batch_index * a.sv.z + (int64_t)hk * a.sv.h +
                  (int64_t)(si.k_start + n0) * a.sv.s;
    const int rows = si.seqlen_k - n0 < BN ? si.seqlen_k - n0 : BN;
    const auto v_rs = wave_rsrc(vt, ((rows - 1) * (int)a.sv.s + d_v) * 2);
    constexpr int VCH = BN * D / 8 / NT;
#pragma unroll
    for (int i = 0; i < VCH; ++i) {
      const int row = r0 + i * RPI;
      const int voff = cc0 * 8 < d_v ? row * (int)a.sv.s * 2 + cc0 * 16 : kVoffOutOfRange;
      const op_t x = __builtin_bit_cast(op_t, __builtin_amdgcn_raw_buffer_load_b128(v_rs, voff, 0, 0));
      *reinterpret_cast<op_t*>(smem_raw + SM::V_OFF + Swz<D>::addr(row, cc0)) = x;
    }
  }
  fetch_begin(true, 0, 0);
#pragma unroll
  for (int i = 0; i < FETCH_PIECES; ++i) fetch_piece(i);
#pragma unroll
  for (int i = 0; i < STORE_PIECES; ++i) store_piece(i, 0);
  store_stats(0);
  direct_landed();
  __syncthreads();
  // Per q-head the Q tiles come as [masked | full | masked]; each run has its own
  // loop so that the loop bodies are straight-line code.
  const int n_lb = br.fb_lo <= br.fb_hi ? br.fb_lo - br.lo : ntq;
  const int n_fb = br.fb_lo <= br.fb_hi ? br.fb_hi - br.fb_lo + 1 : 0;
  int it = 0;
  int g_cur = 0, e_cur = 0;
  auto step = [&](auto masked_tag) {
    const int stage = it & 1;
    int g_nxt = g_cur, e_nxt = e_cur + 1;
    if (e_nxt == ntq) { e_nxt = 0; ++g_nxt; }
    compute(masked_tag, g_cur, e_cur, stage, it + 1 < total, g_nxt, e_nxt);
    __syncthreads();
    ++it;
    g_cur = g_nxt; e_cur = e_nxt;
  };
  for (int g = 0; g < group; ++g) {
    for (int e = 0; e < n_lb; ++e) step(std::true_type{});
    for (int e = 0; e < n_fb; ++e) step(std::false_type{});
    for (int e = n_lb + n_fb; e < ntq; ++e) step(std::true_type{});
  }

  if (key_ok) {
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        q4_t k4, v4;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          k4[r] = Tr::cvt(dk[db][4 * g + r] * a.sm_scale);   // bwd_kernel_dk_dv.py:387-389
          v4[r] = Tr::cvt(dv[db][4 * g + r]);
        }
        if (32 * db + 8 * g + 4 * hi < d_qk) *reinterpret_cast<q4_t*>(dkptr + 32 * db + 8 * g + 4 * hi) = k4;
        if (32 * db + 8 * g + 4 * hi < d_v) *reinterpret_cast<q4_t*>(dvptr + 32 * db + 8 * g + 4 * hi) = v4;
      }
  }
}

// ---------------------------------------------------------------------------
// dQ (+dB) work item
// ---------------------------------------------------------------------------
// kInlineDelta: delta = rowsum(O dO) of the item's rows is computed here, from the rows the lanes
// load anyway (dO) and their O rows, instead of being read.  kStoreDelta: it is also written out:
// the split backward has no preprocess launch, the dK/dV kernel runs after this one and reads it.
template <typename T, int D, int NW, int BN, bool kWindowed, bool kBias, bool kDropout, bool kInlineDelta, bool kPad,
          bool kStoreDelta = false>
__device__ __forceinline__ void dq_item(const BwdArgs& a, const int h, const int mt, const int z,
                                        char* smem_raw) {
  using Tr = Traits<T>;
  using op_t = typename Tr::op_t;
  using q4_t = typename Tr::q4_t;
  using SM = DqSmem<D, BN>;
  constexpr int NT = NW * 64;
  constexpr int BM = NW * 32;
  constexpr int KS = D / 16, MB = BN / 32, DB = D / 32, TS = BN / 16;
  constexpr int CH = (BN * D / 8) / NT;          // 16-byte chunks per thread, per tensor
  static_assert((BN * D / 8) % NT == 0, "tile must split evenly");

  const int tid = threadIdx.x;
  const int wave = tid >> 6, lane = tid & 63, c = lane & 31, hi = lane >> 5;
  // columns of Q/K/dQ/dK and of V/Out/dOut/dV: <= D, multiples of 8; constants unless a head dim is rounded up
  const int d_qk = kPad ? a.head_dim : D, d_v = kPad ? a.head_dim_v : D;

  const SeqInfo si = get_seq(a.seq, z);
  const int q0 = mt * BM;
  if (q0 >= si.seqlen_q) return;

  Window w{0, 0};
  if (kWindowed) w = parse_window(a.mask.causal_type, a.mask.window_left, a.mask.window_right,
                                  si.seqlen_q, si.seqlen_k);
  w.left = w.left > (1 << 30) ? (1 << 30) : (w.left < -(1 << 30) ? -(1 << 30) : w.left);
  w.right = w.right > (1 << 30) ? (1 << 30) : (w.right < -(1 << 30) ? -(1 << 30) : w.right);
  const BlockRanges br = block_ranges(kWindowed, w.left, w.right, q0, si.seqlen_q, si.seqlen_k, BM, BN);

  const int hk = h / (a.hq / a.hk);
  const int row = q0 + wave * 32 + c;
  const bool row_ok = row < si.seqlen_q;
  const int row_c = row_ok ? row : si.seqlen_q - 1;

  // keys visible to this lane's query form one range [m_lo, m_lo + m_rng] (none: m_none)
  int m_lo = 0, m_hi = si.seqlen_k - 1;
  if (kWindowed) {
    m_lo = row - w.left > 0 ? row - w.left : 0;
    m_hi = row + w.right < m_hi ? row + w.right : m_hi;
  }
  const bool m_none = m_hi < m_lo;
  const unsigned m_rng = m_none ? 0u : (unsigned)(m_hi - m_lo);

  T* dqptr = reinterpret_cast<T*>(a.dq) + (int64_t)si.batch_index * a.sdq.z + (int64_t)h * a.sdq.h +
             (int64_t)(si.q_start + row_c) * a.sdq.s;
  T* dbptr = nullptr;
  if (kBias && a.db != nullptr)
    dbptr = reinterpret_cast<T*>(a.db) + (int64_t)si.batch_index * a.sdb_z + (int64_t)h * a.sdb_h +
            (int64_t)row_c * a.sdb_m;
  const int nkt = (si.seqlen_k + BN - 1) / BN;

  // dB of K tiles that are never visited is zero.  The wave sweeps its 32 rows; along a
  // row the 64 lanes write 16 bytes each when the layout allows it.
  auto zero_db = [&](int j_from, int j_to) {
    if (!(kBias && a.db != nullptr)) return;
    const int c0 = j_from * BN, c1 = j_to * BN < si.seqlen_k ? j_to * BN : si.seqlen_k;
    if (c0 >= c1) return;
    T* dbase = reinterpret_cast<T*>(a.db) + (int64_t)si.batch_index * a.sdb_z + (int64_t)h * a.sdb_h;
    const bool vec = a.sdb_n == 1 && ((a.sdb_m | a.sdb_h | a.sdb_z) & 7) == 0 &&
                     (reinterpret_cast<uintptr_t>(a.db) & 15) == 0;
    const op_t zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
    for (int rr = 0; rr < 32; ++rr) {
      const int m = q0 + wave * 32 + rr;
      if (m >= si.seqlen_q) break;
      T* rowp = dbase + (int64_t)m * a.sdb_m;
      if (vec) {
        const int v0 = (c0 + 7) & ~7, v1 = c1 & ~7;      // 16-byte aligned body (c0 is a multiple of BN)
        for (int n = v0 + lane * 8; n < v1; n += 64 * 8) *reinterpret_cast<op_t*>(rowp + n) = zero8;
        for (int n = (v1 > v0 ? v1 : c0) + lane; n < c1; n += 64) rowp[n] = Tr::cvt(0.f);
      } else {
        for (int n = c0 + lane; n < c1; n += 64) rowp[(int64_t)n * a.sdb_n] = Tr::cvt(0.f);
      }
    }
  };

  if (br.lo > br.hi) {
    if (row_ok) {
      q4_t zero4 = {0, 0, 0, 0};
#pragma unroll
      for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int g = 0; g < 4; ++g)
          if (32 * db + 8 * g + 4 * hi < d_qk) *reinterpret_cast<q4_t*>(dqptr + 32 * db + 8 * g + 4 * hi) = zero4;
    }
    if (kStoreDelta) {
      // no key sees these rows and nobody reads their delta; it is written all the same, as the
      // preprocess kernel would (bwd_preprocess.py:28-250)
      const T* optr = reinterpret_cast<const T*>(a.out) + (int64_t)si.batch_index * a.so.z +
                      (int64_t)h * a.so.h + (int64_t)(si.q_start + row_c) * a.so.s;
      const T* doptr = reinterpret_cast<const T*>(a.dout) + (int64_t)si.batch_index * a.sdo.z +
                       (int64_t)h * a.sdo.h + (int64_t)(si.q_start + row_c) * a.sdo.s;
      float acc = 0.f;
      for (int k = 0; k < KS; ++k) {
        if (16 * k + 8 * hi >= d_v) continue;
        const op_t o8 = *reinterpret_cast<const op_t*>(optr + 16 * k + 8 * hi);
        const op_t d8 = *reinterpret_cast<const op_t*>(doptr + 16 * k + 8 * hi);
#pragma unroll
        for (int e = 0; e < 8; ++e) acc += (float)o8[e] * (float)d8[e];
      }
      acc = cross_sum(acc);
      if (row_ok && hi == 0) a.delta[lse_offset(si, h, a.hq) + row] = acc;
    }
    zero_db(0, nkt);
    return;
  }

  const T* qptr = reinterpret_cast<const T*>(a.q) + (int64_t)si.batch_index * a.sq.z + (int64_t)h * a.sq.h +
                  (int64_t)(si.q_start + row_c) * a.sq.s;
  const T* doptr = reinterpret_cast<const T*>(a.dout) + (int64_t)si.batch_index * a.sdo.z +
                   (int64_t)h * a.sdo.h + (int64_t)(si.q_start + row_c) * a.sdo.s;
  op_t qreg[KS], doreg[KS];
#pragma unroll
  for (int k = 0; k < KS; ++k) {
    // columns past the tensors' head dim are zero (head dims are rounded up to D)
    const op_t zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
    qreg[k] = 16 * k + 8 * hi < d_qk ? *reinterpret_cast<const op_t*>(qptr + 16 * k + 8 * hi) : zero8;
    doreg[k] = 16 * k + 8 * hi < d_v ? *reinterpret_cast<const op_t*>(doptr + 16 * k + 8 * hi) : zero8;
  }
  const int64_t lo = lse_offset(si, h, a.hq) + row_c;
  const float l_row = a.lse[lo] * kRcpLn2;               // bwd_kernel_dq.py:305
  float d_row;
  if (kInlineDelta) {
    const T* optr = reinterpret_cast<const T*>(a.out) + (int64_t)si.batch_index * a.so.z +
                    (int64_t)h * a.so.h + (int64_t)(si.q_start + row_c) * a.so.s;
    float acc = 0.f;
#pragma unroll
    for (int k = 0; k < KS; ++k) {
      if (16 * k + 8 * hi >= d_v) continue;
      const op_t o8 = *reinterpret_cast<const op_t*>(optr + 16 * k + 8 * hi);
#pragma unroll
      for (int e = 0; e < 8; ++e) acc += (float)o8[e] * (float)doreg[k][e];
    }
    d_row = cross_sum(acc);
    if (kStoreDelta && row_ok && hi == 0) a.delta[lo] = d_row;
  } else {
    d_row = a.delta[lo];
  }
  // The resident Q / dO operands live in accumulation registers: an MFMA takes its B operand
  // from there directly.  Left to itself the register allocator parks them there as well (the
  // kernel needs more than 256 registers) but copies each one back before every use: 32-44
  // copies per key tile at D = 128, a quarter of the loop's vector instructions.  Not at
  // D = 256, where the allocation gets worse with the constraint.
  if constexpr (D <= 128) {
#pragma unroll
    for (int k = 0; k < KS; ++k) {
      asm volatile("" : "+a"(qreg[k]));
      asm volatile("" : "+a"(doreg[k]));
    }
  }

  // Without dropout (the mask and the scale come between dP and the subtraction) dP starts at
  // -delta.  Not in the dQ kernel at D = 64: with 128-key tiles its register allocation gets
  // worse with the extra tuple (20-50 % slower); the single-launch kernel at D = 64 gains.
  constexpr bool kFoldDelta = !kDropout && (D >= 128 || (kInlineDelta && !kStoreDelta));
  f32x16 negd16;      // -delta of this lane's query in every element: the initial value of dP
#pragma unroll
  for (int i = 0; i < 16; ++i) negd16[i] = -d_row;

  const T* kbase = reinterpret_cast<const T*>(a.k) + (int64_t)si.batch_index * a.sk.z + (int64_t)hk * a.sk.h +
                   (int64_t)si.k_start * a.sk.s;
  const T* vbase = reinterpret_cast<const T*>(a.v) + (int64_t)si.batch_index * a.sv.z + (int64_t)hk * a.sv.h +
                   (int64_t)si.k_start * a.sv.s;
  const T* bptr = nullptr;
  if (kBias)
    bptr = reinterpret_cast<const T*>(a.bias) + (int64_t)si.batch_index * a.sb_z + (int64_t)h * a.sb_h +
           (int64_t)row_c * a.sb_m;
  // 8-byte bias loads / dB stores need unit column stride and 8-byte aligned rows
  const bool bias_vec = kBias && a.sb_n == 1 && ((a.sb_m | a.sb_h | a.sb_z) & 3) == 0 &&
                        (reinterpret_cast<uintptr_t>(a.bias) & 7) == 0;
  const bool db_vec = kBias && a.sdb_n == 1 && ((a.sdb_m | a.sdb_h | a.sdb_z) & 3) == 0 &&
                      (reinterpret_cast<uintptr_t>(a.db) & 7) == 0;
  // Whole tiles of bias and dB travel as row-contiguous 16-byte pieces (consecutive lanes along a
  // row: a wave-wide access touches 64 / (BN / 8) rows) and change to the one-row-per-lane layout
  // of the MFMA results in a 32-row LDS area of the wave.  One 8-byte access per lane and 4 keys
  // touches 32 cache lines for 16 bytes each, and the vector memory pipe's line rate then makes a
  // bias cost more than all the MFMAs of the kernel (dQ with bias 4.4 ms against 1.6 ms without).
  constexpr int BLPR = BN / 8;            // 16-byte pieces per tile row
  constexpr int BRPI = 64 / BLPR;         // rows per wave-wide access
  constexpr int BNI = 32 / BRPI;          // accesses per tile
  char* bw = smem_raw + SM::BIAS_OFF + wave * 32 * SM::BIAS_ROW;
  const int brow = lane / BLPR, bch = lane % BLPR;
  const bool bias_co = kBias && a.sb_n == 1 && ((a.sb_m | a.sb_h | a.sb_z) & 7) == 0 &&
                       (reinterpret_cast<uintptr_t>(a.bias) & 15) == 0;
  const bool db_co = kBias && a.db != nullptr && a.sdb_n == 1 && ((a.sdb_m | a.sdb_h | a.sdb_z) & 7) == 0 &&
                     (reinterpret_cast<uintptr_t>(a.db) & 15) == 0;
  // an item's tiles take the vector code when the bias can be read as vectors and dB (if wanted)
  // written through the LDS area
  const bool want_db = kBias && a.db != nullptr;
  const bool item_fast = !kBias || (bias_vec && (!want_db || (db_co && db_vec)));
  const T* bias_head = kBias ? reinterpret_cast<const T*>(a.bias) + (int64_t)si.batch_index * a.sb_z +
                                   (int64_t)h * a.sb_h : nullptr;
  T* db_head = kBias && a.db != nullptr ? reinterpret_cast<T*>(a.db) + (int64_t)si.batch_index * a.sdb_z +
                                              (int64_t)h * a.sdb_h : nullptr;
  DropoutState dst{};
  if (kDropout) dst = make_dropout(a.drop, z, h, a.hq, a.seq.max_seqlen_q, a.seq.max_seqlen_k);

  f32x16 dq[DB];
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int i = 0; i < 16; ++i) dq[db][i] = 0.f;
  const float qk_scale = a.sm_scale * kLog2e;

  // K and V tiles travel global -> registers -> LDS in 16-byte pieces that are issued
  // between the MFMAs of the running tile (loads behind S^T = K Q^T, LDS writes behind
  // dQ^T += K^T dS^T).  Buffer loads with a descriptor rebased on every tile: rows past
  // the end of the sequence read as zero (dS is 0 there), and a descriptor of zero
  // records turns the fetch after the last tile into a no-op.
  constexpr int LPR = D / 8;                     // 16-byte pieces per row
  constexpr int RPI = NT / LPR;                  // rows between two pieces of one thread
  static_assert((BN * D / 8) % NT == 0 && NT % LPR == 0, "threads must cover the tile evenly");
  // (the pieces go straight into the LDS stage, as in the dK/dV item: lane at chunk position p of
  // row r fetches chunk p ^ f(r), a wave instruction fills 64 / LPR consecutive rows)
  constexpr bool kDirect = true;
  constexpr int RWI = 64 / LPR;
  static_assert(!kDirect || RPI % 8 == 0, "the swizzle must repeat every two pieces");
  op_t kch[kDirect ? 1 : CH], vch[kDirect ? 1 : CH];
  const int r0 = tid / LPR, cc0 = tid % LPR;
  const int wave_u = __builtin_amdgcn_readfirstlane(tid >> 6);
  int f_stage = 0;                               // stage the running fetch fills
  int k_voff_d[2] = {0, 0}, v_voff_d[2] = {0, 0};
  if (kDirect) {
#pragma unroll
    for (int k = 0; k < 2; ++k) {
      const int gch = cc0 ^ Swz<D>::f(r0 + k * RPI);
      k_voff_d[k] = gch * 8 < d_qk ? r0 * (int)a.sk.s * 2 + gch * 16 : kVoffOutOfRange;
      v_voff_d[k] = gch * 8 < d_v ? r0 * (int)a.sv.s * 2 + gch * 16 : kVoffOutOfRange;
    }
  }
  using lds_ptr_t = __attribute__((address_space(3))) void*;
  const int k_voff = cc0 * 8 < d_qk ? r0 * (int)a.sk.s * 2 + cc0 * 16 : kVoffOutOfRange,
            v_voff = cc0 * 8 < d_v ? r0 * (int)a.sv.s * 2 + cc0 * 16 : kVoffOutOfRange;
  const int k_soff = RPI * (int)a.sk.s * 2, v_soff = RPI * (int)a.sv.s * 2;
  int lds_off[CH];                                                        // bytes inside a tile
#pragma unroll
  for (int k = 0; k < CH; ++k) lds_off[k] = Swz<D>::addr(r0 + k * RPI, cc0);
  // lane constants of the two LDS access patterns
  const int row_a = Swz<D>::row_base(lane), tr_a0 = Swz<D>::tr_base(lane, 0), tr_a1 = Swz<D>::tr_base(lane, 1);

  const T* kt = kbase + (int64_t)br.lo * BN * a.sk.s;
  const T* vt = vbase + (int64_t)br.lo * BN * a.sv.s;
  const int64_t k_step = (int64_t)BN * a.sk.s, v_step = (int64_t)BN * a.sv.s;
  int rows_left = si.seqlen_k - br.lo * BN;      // > 0
  __amdgpu_buffer_rsrc_t k_rs, v_rs;
  // tiles are fetched in ascending order; `live` false: nothing is fetched
  auto fetch_begin = [&](bool live) {
    int rows = rows_left < BN ? rows_left : BN;
    rows = live ? rows : 0;
    const bool any = rows > 0;
    k_rs = wave_rsrc(kt, any ? ((rows - 1) * (int)a.sk.s + d_qk) * 2 : 0);
    v_rs = wave_rsrc(vt, any ? ((rows - 1) * (int)a.sv.s + d_v) * 2 : 0);
    if (live) { kt += k_step; vt += v_step; rows_left -= BN; }
  };
  constexpr int FETCH_PIECES = 2 * CH;
  auto fetch_piece = [&](int i) {        // K pieces first, then V
    if constexpr (kDirect) {
      char* sp = smem_raw + f_stage * SM::STAGE_BYTES;
      if (i < CH)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(k_rs, (lds_ptr_t)(sp + (i * RPI + RWI * wave_u) * Swz<D>::ROWB), 16,
                                                 k_voff_d[i & 1], i * k_soff, 0, 0);
      else
        __builtin_amdgcn_raw_ptr_buffer_load_lds(
            v_rs, (lds_ptr_t)(sp + SM::TILE_BYTES + ((i - CH) * RPI + RWI * wave_u) * Swz<D>::ROWB), 16,
            v_voff_d[(i - CH) & 1], (i - CH) * v_soff, 0, 0);
    } else {
      if (i < CH)
        kch[i] = __builtin_bit_cast(op_t, __builtin_amdgcn_raw_buffer_load_b128(k_rs, k_voff, i * k_soff, 0));
      else
        vch[i - CH] =
            __builtin_bit_cast(op_t, __builtin_amdgcn_raw_buffer_load_b128(v_rs, v_voff, (i - CH) * v_soff, 0));
    }
  };
  // all of this wave's direct pieces have landed (vmcnt 0; the other counters stay as they are)
  auto direct_landed = [&]() {
    if constexpr (kDirect) __builtin_amdgcn_s_waitcnt(0x0F70);
  };
  constexpr int STORE_PIECES = 2 * CH;
  auto store_piece = [&](int i, int stage) {   // same order as the fetches
    char* sp = smem_raw + stage * SM::STAGE_BYTES;
    if (kDirect) return;
    if (i < CH) *reinterpret_cast<op_t*>(sp + lds_off[i]) = kch[i];
    else *reinterpret_cast<op_t*>(sp + SM::TILE_BYTES + lds_off[i - CH]) = vch[i - CH];
  };

  // kFast (bias only): the tile lies inside the key range and bias and dB can travel as vectors; the
  // element code then has no run-time branch.  Other tiles of a bias run take the general code, in a
  // loop of their own: one loop body holding both would branch around every element and move the
  // accumulators between the two copies of its MFMAs.
  auto compute = [&](auto masked_tag, auto fast_tag, int j, int stage, bool live) __attribute__((always_inline)) {
    constexpr bool masked = decltype(masked_tag)::value;
    constexpr bool kFast = decltype(fast_tag)::value;
    constexpr int G1 = KS * MB, G4 = TS * DB;
    const char* Kb = smem_raw + stage * SM::STAGE_BYTES;
    const char* Vb = Kb + SM::TILE_BYTES;
    f32x16 s[MB], dp[MB];
    const f32x16 zero16 = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    // The vector ALU work is spread over MFMAs that do not depend on it: p = exp2(...)
    // of S runs behind the MFMAs of dP, ds = p (dP - delta) of one 16-key step behind
    // the dQ MFMAs of the step before.  Fences keep the hand-made order.
    constexpr int kAhead = D >= 256 ? 1 : 2;
    op_t xa[kAhead + 1][MB];
    op_t sb[TS];
    uint32_t keep[kDropout ? 4 * MB : 1];
    const bool tile_vec = kFast;
    // the tile's bias, requested before the S MFMAs and used behind the dP MFMAs: with one wave per
    // SIMD a load that is used where it is issued costs its whole latency
    q4_t bias4[kBias ? 4 * MB : 1];
    const bool tile_co = kFast && bias_co;                     // bias through the wave's LDS area
    const bool tile_dbco = kFast && want_db;                   // dB through it
    op_t bco[kBias ? BNI : 1];
    if (kBias && tile_co) {
#pragma unroll
      for (int i = 0; i < BNI; ++i) {
        int m = q0 + wave * 32 + brow + BRPI * i;
        m = m < si.seqlen_q ? m : si.seqlen_q - 1;
        bco[i] = *reinterpret_cast<const op_t*>(bias_head + (int64_t)m * a.sb_m + j * BN + bch * 8);
      }
    } else if (kBias && tile_vec) {
#pragma unroll
      for (int q = 0; q < 4 * MB; ++q)
        bias4[q] = *reinterpret_cast<const q4_t*>(bptr + j * BN + 32 * (q / 4) + 8 * (q % 4) + 4 * hi);
    }

    // ---- S^T = K Q^T -------------------------------------------------------------
#pragma unroll
    for (int k = 0; k < kAhead; ++k)
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) xa[k][mb] = swz_read_row<T, D>(Kb, row_a, k, mb);
#pragma unroll
    // (the operand ring runs on from the K rows of S into the V rows of dP: the first V operands are
    // requested behind the last MFMAs of S instead of in front of the first ones of dP)
    for (int k = 0; k < KS; ++k) {
#pragma unroll
      for (int mb = 0; mb < MB; ++mb)
        xa[(k + kAhead) % (kAhead + 1)][mb] = k + kAhead < KS ? swz_read_row<T, D>(Kb, row_a, k + kAhead, mb)
                                                              : swz_read_row<T, D>(Vb, row_a, k + kAhead - KS, mb);
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) {
        s[mb] = Tr::mfma(xa[k % (kAhead + 1)][mb], qreg[k], k == 0 ? zero16 : s[mb]);
        // the next tile's descriptors and global loads ride behind these MFMAs
        constexpr int every = G1 / FETCH_PIECES > 0 ? G1 / FETCH_PIECES : 1;
        constexpr int per = (FETCH_PIECES + G1 - 1) / G1;
        const int gidx = k * MB + mb;
        if (gidx == 0) { f_stage = stage ^ 1; fetch_begin(live); }
        if (gidx % every == every - 1) {
#pragma unroll
          for (int q = 0; q < per; ++q) {
            const int piece = gidx / every * per + q;
            if (piece < FETCH_PIECES) fetch_piece(piece);
          }
        }
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    if (kBias && tile_co) {
      // (the wave's LDS operations run in order: the previous tile's dB pieces have left the area)
#pragma unroll
      for (int i = 0; i < BNI; ++i)
        *reinterpret_cast<op_t*>(bw + (brow + BRPI * i) * SM::BIAS_ROW + bch * 16) = bco[i];
#pragma unroll
      for (int q = 0; q < 4 * MB; ++q)
        bias4[q] = *reinterpret_cast<const q4_t*>(bw + c * SM::BIAS_ROW + (32 * (q / 4) + 8 * (q % 4) + 4 * hi) * 2);
    }

    // element E = 16*mb + i of the tile: p, kept in s
    const unsigned m_d = m_none ? 0x40000000u : (unsigned)(j * BN + 4 * hi - m_lo);
    auto p_el = [&](int E) {
      const int mb = E / 16, i = E % 16, g = i / 4, r = i % 4;
      const int n = j * BN + 32 * mb + 8 * g + 4 * hi + r;
      float x;
      if (kBias) {
        float bv;
        if constexpr (kFast) {
          bv = (float)bias4[E / 4][r];
        } else {
          const int nn = n < si.seqlen_k ? n : si.seqlen_k - 1;
          bv = (float)bptr[(int64_t)nn * a.sb_n];
        }
        x = __builtin_fmaf(s[mb][i], qk_scale, bv * kLog2e) - l_row;
      } else {
        x = __builtin_fmaf(s[mb][i], qk_scale, -l_row);
      }
      if (masked) {
        // one unsigned comparison of n - m_lo against the length of the visible range
        const bool vis = m_d + (unsigned)(32 * mb + 8 * g + r) <= m_rng;
        x = vis ? x : -__builtin_inff();
      }
      s[mb][i] = fast_exp2(x);
    };
    auto ds_el = [&](int E) {
      const int mb = E / 16, i = E % 16, g = i / 4, r = i % 4;
      const int n = j * BN + 32 * mb + 8 * g + 4 * hi + r;
      if (kDropout && r == 0) keep[E / 4] = dropout_keep4(dst, row, n);
      float dpv = dp[mb][i];
      if (kDropout) dpv = ((keep[E / 4] >> r) & 1u) ? dpv * dst.scale : 0.f;   // bwd_inner_dq.py:176-185
      // where the dP accumulators start at -delta, dP - delta leaves the matrix pipe
      const float dsv = kFoldDelta ? s[mb][i] * dpv : s[mb][i] * (dpv - d_row);
      dp[mb][i] = dsv;
      if constexpr (kBias && kFast) {                                            // bwd_inner_dq.py:200-204
        // (rows past the sequence write their part of the area too; it is never stored)
        if (r == 3 && tile_dbco) {
          q4_t d4v;
#pragma unroll
          for (int q = 0; q < 4; ++q) d4v[q] = Tr::cvt(dp[mb][i - 3 + q]);
          *reinterpret_cast<q4_t*>(bw + c * SM::BIAS_ROW + (32 * mb + 8 * g + 4 * hi) * 2) = d4v;
        }
      } else if (kBias && dbptr != nullptr && row_ok) {
        if (n < si.seqlen_k) dbptr[(int64_t)n * a.sdb_n] = Tr::cvt(dsv);
      }
      if (E & 1) {   // ds cast to K's dtype, pair by pair
        const typename Tr::p2_t s2 = Tr::cvt2(dp[mb][i - 1], dsv);
        sb[E / 8][E % 8 - 1] = s2[0];
        sb[E / 8][E % 8] = s2[1];
      }
    };

    // ---- dP^T = V dO^T, with p behind its MFMAs -----------------------------------
    constexpr int EPG1 = 16 / KS;          // elements per MFMA
    static_assert(16 % KS == 0, "element split");
#pragma unroll
    for (int k = 0; k < KS; ++k) {
      if (k + kAhead < KS) {
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
          xa[(KS + k + kAhead) % (kAhead + 1)][mb] = swz_read_row<T, D>(Vb, row_a, k + kAhead, mb);
      }
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) {
        dp[mb] = Tr::mfma(xa[(KS + k) % (kAhead + 1)][mb], doreg[k], k == 0 ? (kFoldDelta ? negd16 : zero16) : dp[mb]);
#pragma unroll
        for (int e = 0; e < EPG1; ++e) p_el((k * MB + mb) * EPG1 + e);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    op_t ta[2][DB];
#pragma unroll
    for (int db = 0; db < DB; ++db) ta[0][db] = swz_read_tr<T, D>(Kb, tr_a0, tr_a1, 0, db);
    // ds of the first 16-key step has nothing to hide behind
#pragma unroll
    for (int E = 0; E < 8; ++E) ds_el(E);
    __builtin_amdgcn_sched_barrier(0);

    // ---- dQ^T += K^T dS^T, with the next step's ds and the LDS writes behind its MFMAs ----
    constexpr int EPG3 = 8 / DB;
    static_assert(8 % DB == 0, "element split");
#pragma unroll
    for (int t = 0; t < TS; ++t) {
#pragma unroll
      for (int db = 0; db < DB; ++db) {
        if (t + 1 < TS) ta[(t + 1) & 1][db] = swz_read_tr<T, D>(Kb, tr_a0, tr_a1, t + 1, db);
        dq[db] = Tr::mfma(ta[t & 1][db], sb[t], dq[db]);
        if (t + 1 < TS) {
#pragma unroll
          for (int e = 0; e < EPG3; ++e) ds_el(8 * (t + 1) + db * EPG3 + e);
        }
        constexpr int per = (STORE_PIECES + G4 - 1) / G4;
#pragma unroll
        for (int q = 0; q < per; ++q) {
          const int piece = (t * DB + db) * per + q;
          if (piece < STORE_PIECES) store_piece(piece, stage ^ 1);
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    if (kBias && tile_dbco) {
      // the wave's dB tile leaves as whole 16-byte pieces of its rows
#pragma unroll
      for (int i = 0; i < BNI; ++i) {
        const int m = q0 + wave * 32 + brow + BRPI * i;
        const op_t x = *reinterpret_cast<const op_t*>(bw + (brow + BRPI * i) * SM::BIAS_ROW + bch * 16);
        if (m < si.seqlen_q) *reinterpret_cast<op_t*>(db_head + (int64_t)m * a.sdb_m + j * BN + bch * 8) = x;
      }
    }
    direct_landed();
  };

  fetch_begin(true);
#pragma unroll
  for (int i = 0; i < FETCH_PIECES; ++i) fetch_piece(i);
#pragma unroll
  for (int i = 0; i < STORE_PIECES; ++i) store_piece(i, 0);
  direct_landed();
  __syncthreads();
  // K tiles come as [masked | full | masked]; one straight-line loop per run
  {
    int j = br.lo;
    auto step = [&](auto masked_tag, auto fast_tag) __attribute__((always_inline)) {
      const int stage = (j - br.lo) & 1;
      compute(masked_tag, fast_tag, j, stage, j < br.hi);
      __syncthreads();
      ++j;
    };
    const int full_lo = br.fb_lo <= br.fb_hi ? br.fb_lo : br.hi + 1;
    const int full_hi = br.fb_lo <= br.fb_hi ? br.fb_hi : br.hi;
    // last tile that lies inside the key range (the vector code of a bias run ends there)
    const int j_in = item_fast ? si.seqlen_k / BN - 1 : br.lo - 1;
    // (a closure left out of line keeps its captures in memory: every use becomes a flat load)
    auto run = [&](auto masked_tag, int upto) __attribute__((always_inline)) {
      if constexpr (kBias) {
        const int fast_to = upto < j_in ? upto : j_in;
        while (j <= fast_to) step(masked_tag, std::true_type{});
        while (j <= upto) step(masked_tag, std::false_type{});
      } else {
        while (j <= upto) step(masked_tag, std::true_type{});
      }
    };
    run(std::true_type{}, full_lo - 1);
    run(std::false_type{}, full_hi);
    run(std::true_type{}, br.hi);
  }

  if (row_ok) {
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        q4_t t4;
#pragma unroll
        for (int r = 0; r < 4; ++r) t4[r] = Tr::cvt(dq[db][4 * g + r] * a.sm_scale);   // bwd_kernel_dq.py:374-376
        if (32 * db + 8 * g + 4 * hi < d_qk) *reinterpret_cast<q4_t*>(dqptr + 32 * db + 8 * g + 4 * hi) = t4;
      }
  }
  zero_db(0, br.lo);
  zero_db(br.hi + 1, nkt);
}

// ---------------------------------------------------------------------------
// Kernels
// ---------------------------------------------------------------------------
// Whether the dK/dV kernel walks the level list: persistent workgroups over sequences of different
// lengths, few enough (sequence, kv-head) entries per XCD for the table.
template <int D>
__host__ __device__ inline bool dkdv_level_list(const BwdArgs& a) {
  return D < 256 && a.seq.num_seqlens != 0 && a.bias == nullptr && a.zh_per_xcd <= kLevelCap && a.num_n_tiles <= 0xffff;
}

template <typename T, int D, int NW, int BM, bool kWindowed, bool kBias, bool kDropout, bool kPad, bool kStoreDs = false>
__global__ __attribute__((amdgpu_flat_work_group_size(NW * 64, NW * 64)))
void bwd_dkdv_kernel(const BwdArgs a) {
  extern __shared__ __attribute__((aligned(16))) char smem_raw[];
  // Persistent workgroups, one per CU (a relaunch per item costs a dispatch gap of several
  // microseconds on every CU).  Each XCD owns a contiguous range of (batch, kv-head)
  // pairs and walks them in pairs, K tiles in ascending order (the heaviest causal tile
  // first), so the Q/dO stream of the heads in flight stays in that XCD's L2; the
  // workgroups of the XCD take the items in serpentine order (worker p takes p,
  // 2P-1-p, 2P+p, ...), which pairs heavy with light items.
  const int xcd = blockIdx.x % kNumXcd, p = blockIdx.x / kNumXcd, workers = gridDim.x / kNumXcd;
  const int per_group = a.zh_group * a.num_n_tiles;
  // Sequences of different lengths: the valid tiles only, heaviest first (LevelWalk), taken in the
  // same serpentine order.
  const bool ragged = dkdv_level_list<D>(a);
  const int zh_lo = xcd * a.zh_per_xcd;
  LevelWalk walk;
  if (ragged)
    walk.init<NW * 64>(reinterpret_cast<uint32_t*>(smem_raw + DkDvSmem<D, BM>::BYTES), a.seq, zh_lo,
                       zh_lo + a.zh_per_xcd < a.num_zh ? zh_lo + a.zh_per_xcd : a.num_zh, a.num_zh / a.hk, 1, NW * 32, true,
                       threadIdx.x);
  // (D = 256 is launched with one workgroup per item: the loop would cost registers there)
  for (int r = 0; D >= 256 ? r < 1 : r * workers < a.items_per_xcd; ++r) {
    const int li = r * workers + ((r & 1) ? workers - 1 - p : p);
    int zh, nt;
    if (ragged) {
      int e;
      if (!walk.at(li, e, nt)) break;
      zh = zh_lo + e;
    } else {
      if (li >= a.items_per_xcd) continue;
      const int gi = li / per_group, gr = li % per_group;
      const int zl = gi * a.zh_group + gr % a.zh_group;
      zh = zh_lo + zl;
      if (zl >= a.zh_per_xcd || zh >= a.num_zh) continue;
      nt = gr / a.zh_group;
    }
    int z, hk;
    split_zh(zh, a.num_zh / a.hk, 1, z, hk);
    dkdv_item<T, D, NW, BM, kWindowed, kBias, kDropout, false, kPad, kStoreDs>(a, hk, nt, z, smem_raw);
    __syncthreads();     // the next item reuses the LDS stages
  }
}

template <typename T, int D, int NW, int BN, bool kWindowed, bool kBias, bool kDropout, bool kPad>
__global__ __attribute__((amdgpu_flat_work_group_size(NW * 64, NW * 64)))
void bwd_dq_kernel(const BwdArgs a) {
  extern __shared__ __attribute__((aligned(16))) char smem_raw[];
  // persistent workgroups with the same walk as the forward kernel: (batch, q-head) pairs
  // per XCD, heaviest Q tile first, serpentine over the workgroups of the XCD
  const int xcd = blockIdx.x % kNumXcd, p = blockIdx.x / kNumXcd, workers = gridDim.x / kNumXcd;
  const int per_group = a.zh_group * a.num_m_tiles;
  // (D = 256 is launched with one workgroup per item: the loop would cost registers there)
  for (int r = 0; D >= 256 ? r < 1 : r * workers < a.items_per_xcd; ++r) {
    const int li = r * workers + ((r & 1) ? workers - 1 - p : p);
    if (li >= a.items_per_xcd) continue;
    const int gi = li / per_group, gr = li % per_group;
    const int zl = gi * a.zh_group + gr % a.zh_group;
    const int zh = xcd * a.zh_per_xcd + zl;
    if (zl >= a.zh_per_xcd || zh >= a.num_zh) continue;
    const int mt = a.num_m_tiles - 1 - gr / a.zh_group;
    int z, h;
    split_zh(zh, a.num_zh / a.hq, a.hq / a.hk, z, h);
    dq_item<T, D, NW, BN, kWindowed, kBias, kDropout, true, kPad, true>(a, h, mt, z, smem_raw);
    __syncthreads();     // the next item reuses the LDS stages
  }
}

// Per (batch, kv-head): num_n_tiles dK/dV items followed by num_m_tiles*(Hq/Hk) dQ items
// (modules/flash/csrc/attn_bwd_fused.cc:13-22, bwd_kernel_fuse.py:107-118), laid out on
// the same 1-D grid as the split kernels: each XCD owns a contiguous range of (batch,
// kv-head) pairs and walks them in pairs, so the tensors of the heads in flight stay in
// that XCD's L2.
template <typename T, int D, int NW, int BM, int BN, bool kWindowed, bool kBias, bool kDropout, bool kPad>
__global__ __attribute__((amdgpu_flat_work_group_size(NW * 64, NW * 64)))
void bwd_fused_kernel(const BwdArgs a) {
  extern __shared__ __attribute__((aligned(16))) char smem_raw[];
  const int group = a.hq / a.hk;
  const int items = a.num_n_tiles + a.num_m_tiles * group;
  // persistent workgroups with the walk of the split kernels (one workgroup per item with a bias
  // or at D = 256, where the loop runs once)
  const int xcd = blockIdx.x % kNumXcd, p = blockIdx.x / kNumXcd, workers = gridDim.x / kNumXcd;
  const int per_group = a.zh_group * items;
  for (int r = 0; D >= 256 ? r < 1 : r * workers < a.items_per_xcd; ++r) {
    const int li = r * workers + ((r & 1) ? workers - 1 - p : p);
    if (li >= a.items_per_xcd) continue;
    const int gi = li / per_group, gr = li % per_group;
    const int zl = gi * a.zh_group + gr % a.zh_group;
    const int zh = xcd * a.zh_per_xcd + zl;
    if (zl >= a.zh_per_xcd || zh >= a.num_zh) continue;
    int z, hk;
    split_zh(zh, a.num_zh / a.hk, 1, z, hk);
    const int item = gr / a.zh_group;
    if (item < a.num_n_tiles) {
      dkdv_item<T, D, NW, BM, kWindowed, kBias, kDropout, true, kPad>(a, hk, item, z, smem_raw);
    } else {
      const int t = item - a.num_n_tiles;
      const int h = hk * group + t / a.num_m_tiles;
      const int mt = a.num_m_tiles - 1 - t % a.num_m_tiles;
      dq_item<T, D, NW, BN, kWindowed, kBias, kDropout, true, kPad>(a, h, mt, z, smem_raw);
    }
    __syncthreads();     // the next item reuses the LDS stages
  }
}

// ---------------------------------------------------------------------------
// Host launchers
// ---------------------------------------------------------------------------
inline int bwd_nseq(const BwdArgs& a) {
  return a.seq.num_seqlens != 0 ? (a.seq.num_seqlens < 0 ? -a.seq.num_seqlens : a.seq.num_seqlens) : a.batch;
}

// Workgroups per XCD of the dK/dV and dQ kernels: one per CU, at most one per item.  With a
// bias the kernels get one workgroup per item instead (the loop of a workgroup then runs
// once): measured at B2 H16 S8192 D256 with window, bias, dB and dropout the persistent
// grid was 10 % slower, while it gains 1 % at the headline shape and 12 % on packed
// sequences of very different lengths.  D = 256 also gets one workgroup per item: its
// dK/dV kernel has no register to spare for the loop.
template <int D>
inline int persistent_workers(const BwdArgs& a) {
  if (a.bias != nullptr || D >= 256) return a.items_per_xcd;
  int w = (a.num_cu > 0 ? a.num_cu : 256) / kNumXcd;
  if (w < 1) w = 1;
  return w > a.items_per_xcd ? a.items_per_xcd : w;
}

template <auto kern>
hipError_t launch_with_lds(dim3 grid, int nthreads, int smem, hipStream_t stream, const BwdArgs& a) {
  if (grid.x == 0 || grid.y == 0 || grid.z == 0) return hipSuccess;   // an empty tensor: nothing to write
  if (smem > 64 * 1024) {
    static std::atomic<uint64_t> lds_set{0};
    hipError_t e = allow_large_lds(reinterpret_cast<const void*>(kern), smem, lds_set);
    if (e != hipSuccess) return e;
  }
  hipLaunchKernelGGL(kern, grid, dim3(nthreads), smem, stream, a);
  return hipGetLastError();
}

#define FA_BWD_SWITCH(CALL)                                            \
  switch ((windowed ? 4 : 0) | (bias ? 2 : 0) | (dropout ? 1 : 0)) {   \
    case 0: return CALL(false, false, false);                          \
    case 1: return CALL(false, false, true);                           \
    case 2: return CALL(false, true, false);                           \
    case 3: return CALL(false, true, true);                            \
    case 4: return CALL(true, false, false);                           \
    case 5: return CALL(true, false, true);                            \
    case 6: return CALL(true, true, false);                            \
    default: return CALL(true, true, true);                            \
  }

template <typename T, int D>
hipError_t launch_bwd_preprocess(const BwdArgs& a, hipStream_t stream) {
  constexpr int ROWS = 256 / (D / 8);
  dim3 grid((a.seq.max_seqlen_q + ROWS - 1) / ROWS, a.hq, bwd_nseq(a));
  if (grid.x == 0 || grid.z == 0) return hipSuccess;
  if (a.lse_scaled != nullptr)
    hipLaunchKernelGGL((bwd_preprocess_kernel<T, D, true>), grid, dim3(256), 0, stream, a);
  else
    hipLaunchKernelGGL((bwd_preprocess_kernel<T, D, false>), grid, dim3(256), 0, stream, a);
  return hipGetLastError();
}

template <typename T, int D, bool kPad, bool W, bool B, bool P>
hipError_t launch_dkdv_variant(const BwdArgs& a0, hipStream_t stream) {
  using Tile = BwdTile<T, D, W>;
  constexpr int NW = Tile::NW, BM = Tile::DKDV_BM, BN = NW * 32;
  BwdArgs a = a0;
  a.num_n_tiles = (a.seq.max_seqlen_k + BN - 1) / BN;
  a.num_zh = bwd_nseq(a) * a.hk;
  a.zh_per_xcd = (a.num_zh + kNumXcd - 1) / kNumXcd;
  a.zh_group = 2;
  a.items_per_xcd = ((a.zh_per_xcd + a.zh_group - 1) / a.zh_group) * a.zh_group * a.num_n_tiles;
  dim3 grid((unsigned)(kNumXcd * persistent_workers<D>(a)));
  // (the level table's LDS is requested whether or not this launch uses it: the kernel's limit is set once)
  constexpr int smem = DkDvSmem<D, BM>::BYTES + (D < 256 ? kLevelBytes : 0);
  if (a.ds_ws != nullptr) {
    // (every build has the variant that stores dS; the host decides where it pays)
    if constexpr (D == 64 || D == 128 || D == 256)
      return launch_with_lds<bwd_dkdv_kernel<T, D, NW, BM, W, B, P, kPad, true>>(grid, NW * 64, smem, stream, a);
    else
      return hipErrorNotSupported;
  }
  return launch_with_lds<bwd_dkdv_kernel<T, D, NW, BM, W, B, P, kPad>>(grid, NW * 64, smem, stream, a);
}

template <typename T, int D, bool kPad>
hipError_t launch_bwd_dkdv(const BwdArgs& a0, bool windowed, bool bias, bool dropout, hipStream_t stream) {
#define FA_CALL(W, B, P) launch_dkdv_variant<T, D, kPad, W, B, P>(a0, stream)
  FA_BWD_SWITCH(FA_CALL)
#undef FA_CALL
}

template <typename T, int D, bool kPad, bool W, bool B, bool P>
hipError_t launch_dq_variant(const BwdArgs& a0, hipStream_t stream) {
  using Tile = BwdTile<T, D, W>;
  constexpr int NW = Tile::NW, BN = Tile::DQ_BN, BM = NW * 32;
  BwdArgs a = a0;
  a.num_m_tiles = (a.seq.max_seqlen_q + BM - 1) / BM;
  a.num_zh = bwd_nseq(a) * a.hq;
  a.zh_per_xcd = (a.num_zh + kNumXcd - 1) / kNumXcd;
  a.zh_group = a.hq / a.hk > 2 ? (a.hq / a.hk > 8 ? 8 : a.hq / a.hk) : 2;
  a.items_per_xcd = ((a.zh_per_xcd + a.zh_group - 1) / a.zh_group) * a.zh_group * a.num_m_tiles;
  dim3 grid((unsigned)(kNumXcd * persistent_workers<D>(a)));
  return launch_with_lds<bwd_dq_kernel<T, D, NW, BN, W, B, P, kPad>>(grid, NW * 64, DqSmem<D, BN>::BYTES, stream, a);
}

template <typename T, int D, bool kPad>
hipError_t launch_bwd_dq(const BwdArgs& a0, bool windowed, bool bias, bool dropout, hipStream_t stream) {
#define FA_CALL(W, B, P) launch_dq_variant<T, D, kPad, W, B, P>(a0, stream)
  FA_BWD_SWITCH(FA_CALL)
#undef FA_CALL
}

template <typename T, int D, bool kPad, bool W, bool B, bool P>
hipError_t launch_fused_variant(const BwdArgs& a0, hipStream_t stream) {
  using Tile = BwdTile<T, D, W>;
  constexpr int NW = Tile::NW, BM = Tile::DKDV_BM, BN = Tile::DQ_BN;
  constexpr int smem = DkDvSmem<D, BM>::BYTES > DqSmem<D, BN>::BYTES ? DkDvSmem<D, BM>::BYTES : DqSmem<D, BN>::BYTES;
  BwdArgs a = a0;
  a.num_n_tiles = (a.seq.max_seqlen_k + NW * 32 - 1) / (NW * 32);
  a.num_m_tiles = (a.seq.max_seqlen_q + NW * 32 - 1) / (NW * 32);
  a.num_zh = bwd_nseq(a) * a.hk;
  a.zh_per_xcd = (a.num_zh + kNumXcd - 1) / kNumXcd;
  a.zh_group = 2;
  const int items = a.num_n_tiles + a.num_m_tiles * (a.hq / a.hk);
  a.items_per_xcd = ((a.zh_per_xcd + a.zh_group - 1) / a.zh_group) * a.zh_group * items;
  dim3 grid((unsigned)(kNumXcd * persistent_workers<D>(a)));
  return launch_with_lds<bwd_fused_kernel<T, D, NW, BM, BN, W, B, P, kPad>>(grid, NW * 64, smem, stream, a);
}

template <typename T, int D, bool kPad>
hipError_t launch_bwd_fused(const BwdArgs& a0, bool windowed, bool bias, bool dropout, hipStream_t stream) {
#define FA_CALL(W, B, P) launch_fused_variant<T, D, kPad, W, B, P>(a0, stream)
  FA_BWD_SWITCH(FA_CALL)
#undef FA_CALL
}

template <typename T, int D, bool kWindowed> TileShape bwd_shape(int slot) {
  using Tile = BwdTile<T, D, kWindowed>;
  constexpr int NW = Tile::NW, BM = Tile::DKDV_BM, BN = Tile::DQ_BN;
  constexpr int s1 = DkDvSmem<D, BM>::BYTES, s2 = DqSmem<D, BN>::BYTES;
  switch (slot) {
    case 0: return TileShape{256 / (D / 8), 0, 4, 0};
    case 1: return TileShape{BM, NW * 32, NW, s1 + (D < 256 ? kLevelBytes : 0)};
    case 2: return TileShape{NW * 32, BN, NW, s2};
    default: return TileShape{NW * 32, NW * 32, NW, s1 > s2 ? s1 : s2};
  }
}

}  // namespace fa
