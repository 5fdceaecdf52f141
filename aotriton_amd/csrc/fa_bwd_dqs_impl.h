// dQ from stored dS: the second half of the backward that keeps dS in HBM (gfx950, wave64,
// MFMA 32x32x16).
//
// The split backward of the reference recomputes S and dP in its dQ kernel
// (modules/flash/kernel/bwd_kernel_dq.py:45-389): 7 GEMMs for 5 of algorithmic work, the price of a
// dQ path without atomics.  With 288 GB of HBM at 8 TB/s there is a cheaper price: the dK/dV kernel,
// which forms dS = P (dP - delta) anyway, writes it out in the 16-bit type (the very operand values
// both dK and dQ are formed from), and this kernel reads it back once and only does
//   dQ^T (d x queries) += K_tile^T . dS^T      A = K^T from LDS,  B = dS^T from LDS
// i.e. 5 GEMMs in all, no atomics, one owner per dQ tile, at 2 bytes of HBM traffic each way per
// visible (query, key) pair.  The kernel is bound by that stream, not by the matrix pipe.
//
// Layout of the stored tiles (written by dkdv_item, kStoreDs): one tile per (batch element, q-head,
// key tile of 128, query tile of BM = the dK/dV kernel's step) holds 128 x BM values as
// [key block of 32][16-query step t][64 pieces of 16 bytes].  A piece is what one lane of the dK/dV
// kernel holds as the MFMA operand of step t: its key c (lane % 32) against the queries
// 16 t + 4 hi + {0..3} and 16 t + 8 + 4 hi + {0..3} (hi = lane / 32).  It sits at piece position
// ((2 c + hi) ^ 8 (t & 1)), which is where the transposing LDS reads of this kernel want it: a wave
// copies 1 KB of a tile to LDS as it lies and reads bank-conflict free.
#pragma once
#include "fa_bwd_impl.h"

namespace fa {

template <int D, int BN>
struct DqsSmem {     // two stages of the K tile (swizzled), then one dS area per wave
  static constexpr int NW = 8;
  static constexpr int K_BYTES = BN * D * 2;
  static constexpr int DS_WAVE = BN * 32 * 2;
  static constexpr int DS_OFF = 2 * K_BYTES;
  static constexpr int BYTES = DS_OFF + NW * DS_WAVE;
};

// One Q tile of 256 rows (8 waves x 32 queries) of head h against the key tiles that see it.
template <typename T, int D, int BN, bool kPad>
__device__ __forceinline__ void dqs_item(const BwdArgs& a, const int h, const int mt, const int z, char* smem_raw) {
  using Tr = Traits<T>;
  using op_t = typename Tr::op_t;
  using q4_t = typename Tr::q4_t;
  using SM = DqsSmem<D, BN>;
  using DT = DsTile<T, D>;
  constexpr int NW = SM::NW, NT = NW * 64, BM = NW * 32;
  constexpr int DB = D / 32;
  constexpr int SPT = DT::BN / BN;          // steps per stored tile
  constexpr int KWS = BN / 32;              // 32-key blocks per step
  constexpr int NCK = KWS * 2;              // 1 KB pieces of dS per wave and step
  constexpr int PD = 4;                     // steps of dS in flight, in registers
  constexpr int LPR = D / 8;                // 16-byte pieces per K row
  constexpr int RPI = NT / LPR;             // rows between two pieces of one thread
  constexpr int CH = (BN * LPR) / NT;       // K pieces per thread and step
  static_assert((BN * LPR) % NT == 0 && CH >= 1, "threads must cover the K tile evenly");

  const int tid = threadIdx.x;
  const int wave_u = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lane = tid & 63, c = lane & 31, hi = lane >> 5;
  const int d_qk = kPad ? a.head_dim : D;

  const SeqInfo si = get_seq(a.seq, z);
  const int q0 = mt * BM;
  if (q0 >= si.seqlen_q) return;

  const bool windowed = a.mask.causal_type != 0;
  Window w{0, 0};
  if (windowed) w = parse_window(a.mask.causal_type, a.mask.window_left, a.mask.window_right, si.seqlen_q, si.seqlen_k);
  w.left = w.left > (1 << 30) ? (1 << 30) : (w.left < -(1 << 30) ? -(1 << 30) : w.left);
  w.right = w.right > (1 << 30) ? (1 << 30) : (w.right < -(1 << 30) ? -(1 << 30) : w.right);
  // key tiles (of 128) that hold a key visible to some row of the workgroup
  const BlockRanges br = block_ranges(windowed, w.left, w.right, q0, si.seqlen_q, si.seqlen_k, BM, DT::BN);
  // The wave's rows lie in one stored query tile.  The dK/dV item of key tile nt visits that query
  // tile iff the tile pair holds a visible element; seen from the query tile that is the same range
  // arithmetic with rows and columns exchanged, so this range names exactly the tiles that were written.
  const int qblock = (q0 >> 5) + wave_u;                 // 32-row block of the sequence
  const int pm = qblock / (DT::BM / 32), qb = qblock % (DT::BM / 32);
  const BlockRanges bw = block_ranges(windowed, w.left, w.right, pm * DT::BM, si.seqlen_q, si.seqlen_k, DT::BM, DT::BN);

  const int hk = h / (a.hq / a.hk);
  const int row = q0 + wave_u * 32 + c;
  const bool row_ok = row < si.seqlen_q;
  const int row_c = row_ok ? row : si.seqlen_q - 1;
  T* dqptr = reinterpret_cast<T*>(a.dq) + (int64_t)si.batch_index * a.sdq.z + (int64_t)h * a.sdq.h +
             (int64_t)(si.q_start + row_c) * a.sdq.s;

  f32x16 dq[DB];
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int i = 0; i < 16; ++i) dq[db][i] = 0.f;

  if (br.lo <= br.hi) {
    // steps of BN keys; the last one holds the sequence's last key
    const int j0 = br.lo * SPT;
    int j1 = br.hi * SPT + SPT - 1;
    const int j_end = (si.seqlen_k - 1) / BN;
    j1 = j1 < j_end ? j1 : j_end;
    const int jw0 = bw.lo * SPT, jw1 = bw.lo <= bw.hi ? bw.hi * SPT + SPT - 1 : -1;
    auto active = [&](int j) { return j >= jw0 && j <= jw1 && j <= j1; };

    // ---- K tiles: global -> registers -> LDS (swizzled), one step ahead ------------------------
    const T* kbase = reinterpret_cast<const T*>(a.k) + (int64_t)si.batch_index * a.sk.z + (int64_t)hk * a.sk.h +
                     (int64_t)si.k_start * a.sk.s;
    const int r0 = tid / LPR, cc0 = tid % LPR;
    const int k_voff = cc0 * 8 < d_qk ? r0 * (int)a.sk.s * 2 + cc0 * 16 : kVoffOutOfRange;
    const int k_soff = RPI * (int)a.sk.s * 2;
    int lds_off[CH];
#pragma unroll
    for (int k = 0; k < CH; ++k) lds_off[k] = Swz<D>::addr(r0 + k * RPI, cc0);
    op_t kreg[CH];
    auto load_k = [&](int j) {
      int rows = si.seqlen_k - j * BN;
      rows = rows < BN ? rows : BN;
      rows = j <= j1 ? rows : 0;
      const T* kt = kbase + (int64_t)j * BN * a.sk.s;
      const auto k_rs = wave_rsrc(kt, rows > 0 ? ((rows - 1) * (int)a.sk.s + d_qk) * 2 : 0);
#pragma unroll
      for (int k = 0; k < CH; ++k)
        kreg[k] = __builtin_bit_cast(op_t, __builtin_amdgcn_raw_buffer_load_b128(k_rs, k_voff, k * k_soff, 0));
    };
    auto store_k = [&](int stage) {
#pragma unroll
      for (int k = 0; k < CH; ++k) *reinterpret_cast<op_t*>(smem_raw + stage * SM::K_BYTES + lds_off[k]) = kreg[k];
    };

    // ---- dS pieces: global -> registers (PD steps ahead) -> the wave's LDS area -----------------
    const char* ws_head = reinterpret_cast<const char*>(a.ds_ws) +
                          ((int64_t)z * a.hq + h) * a.ds_ntk * (int64_t)a.ds_ntq * DT::BYTES;
    char* ds_area = smem_raw + SM::DS_OFF + wave_u * SM::DS_WAVE;
    const int ds_voff = lane * 16 + qb * DT::QBLOCK_BYTES;
    op_t dsr[PD][NCK];
    auto load_ds = [&](auto ring_tag, int j) {
      constexpr int R = decltype(ring_tag)::value;
      const int nt = j / SPT, kw0 = (j % SPT) * KWS;
      const char* tile = ws_head + ((int64_t)nt * a.ds_ntq + pm) * DT::BYTES;
      // a wave that has nothing to fetch at this step reads through an empty descriptor: zeros, no traffic
      const auto rs = wave_rsrc(tile, active(j) ? DT::BYTES : 0);
#pragma unroll
      for (int i = 0; i < NCK; ++i)
        dsr[R][i] = __builtin_bit_cast(op_t, __builtin_amdgcn_raw_buffer_load_b128(
                                                 rs, ds_voff, kw0 * 2048 + i * 1024, 2));
    };

    // lane constants of the transposing reads: K^T rows of the swizzled tile, dS^T of the wave's area
    const int tr_a0 = Swz<D>::tr_base(lane, 0), tr_a1 = Swz<D>::tr_base(lane, 1);
    const int g16 = (lane >> 4) & 1, il = lane & 15;
    const int ds_rd = g16 * 1024 + ((((4 * hi + (il >> 2)) * 2 + (il & 1)) ^ (g16 << 3)) << 4) + ((il >> 1) & 1) * 8;

    auto step = [&](auto ring_tag, int j) __attribute__((always_inline)) {
      constexpr int R = decltype(ring_tag)::value;
      __syncthreads();          // K(j) is in its stage; everybody has left the other one
      load_k(j + 1);
      const bool act = active(j);
      if (act) {
#pragma unroll
        for (int i = 0; i < NCK; ++i) *reinterpret_cast<op_t*>(ds_area + i * 1024 + lane * 16) = dsr[R][i];
      }
      load_ds(ring_tag, j + PD);
      if (act) {
        const char* Kb = smem_raw + (j & 1) * SM::K_BYTES;
#pragma unroll
        for (int tk = 0; tk < BN / 16; ++tk) {
          const char* p = ds_area + ds_rd + (tk >> 1) * 2048 + (tk & 1) * 512;
          const q4_t lo = Tr::lds_read_tr(reinterpret_cast<const T*>(p));
          const q4_t up = Tr::lds_read_tr(reinterpret_cast<const T*>(p + 256));
          const op_t b = __builtin_shufflevector(lo, up, 0, 1, 2, 3, 4, 5, 6, 7);
#pragma unroll
          for (int db = 0; db < DB; ++db) dq[db] = Tr::mfma(swz_read_tr<T, D>(Kb, tr_a0, tr_a1, tk, db), b, dq[db]);
        }
      }
      store_k((j + 1) & 1);
    };

    load_k(j0);
    load_ds(std::integral_constant<int, 0>{}, j0);
    load_ds(std::integral_constant<int, 1>{}, j0 + 1);
    load_ds(std::integral_constant<int, 2>{}, j0 + 2);
    load_ds(std::integral_constant<int, 3>{}, j0 + 3);
    store_k(j0 & 1);
    // whole groups of PD steps, so that the loop body is one straight sequence (steps past the last
    // one fetch through empty descriptors and compute nothing); with conditional steps the compiler
    // copies the ring and the accumulators at the loop's end and waits for every load in flight there
    for (int j = j0; j <= j1; j += PD) {
      step(std::integral_constant<int, 0>{}, j);
      step(std::integral_constant<int, 1>{}, j + 1);
      step(std::integral_constant<int, 2>{}, j + 2);
      step(std::integral_constant<int, 3>{}, j + 3);
    }
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
}

// One workgroup per Q tile on a 1-D grid: consecutive ids go round the XCDs, an XCD takes its
// (batch, q-head) pairs two at a time, the heaviest (last) tile of a causal mask first.
template <typename T, int D, int BN, bool kPad>
__global__ __attribute__((amdgpu_flat_work_group_size(512, 512))) __attribute__((amdgpu_waves_per_eu(2, 2)))
void bwd_dqs_kernel(const BwdArgs a) {
  extern __shared__ __attribute__((aligned(16))) char smem_raw[];
  const int xcd = blockIdx.x % kNumXcd, li = blockIdx.x / kNumXcd;
  const int per_group = a.zh_group * a.num_m_tiles;
  const int gi = li / per_group, gr = li % per_group;
  const int zl = gi * a.zh_group + gr % a.zh_group;
  const int zh = xcd * a.zh_per_xcd + zl;
  if (zl >= a.zh_per_xcd || zh >= a.num_zh) return;
  const int mt = a.num_m_tiles - 1 - gr / a.zh_group;
  int z, h;
  split_zh(zh, a.num_zh / a.hq, a.hq / a.hk, z, h);
  dqs_item<T, D, BN, kPad>(a, h, mt, z, smem_raw);
}

template <typename T, int D, bool kPad>
hipError_t launch_bwd_dqs(const BwdArgs& a0, hipStream_t stream) {
  constexpr int BN = D >= 256 ? 32 : 64;
  BwdArgs a = a0;
  a.num_m_tiles = (a.seq.max_seqlen_q + 255) / 256;
  a.num_zh = bwd_nseq(a) * a.hq;
  a.zh_per_xcd = (a.num_zh + kNumXcd - 1) / kNumXcd;
  a.zh_group = a.hq / a.hk > 2 ? (a.hq / a.hk > 8 ? 8 : a.hq / a.hk) : 2;
  a.items_per_xcd = ((a.zh_per_xcd + a.zh_group - 1) / a.zh_group) * a.zh_group * a.num_m_tiles;
  dim3 grid((unsigned)(kNumXcd * a.items_per_xcd));
  return launch_with_lds<bwd_dqs_kernel<T, D, BN, kPad>>(grid, 512, DqsSmem<D, BN>::BYTES, stream, a);
}

}  // namespace fa
