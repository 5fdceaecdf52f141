// Forward flash-attention kernel for gfx950 (wave64, MFMA 32x32x16).
//
// Computes what the reference's attn_fwd does
// (modules/flash/kernel/fwd_kernel.py:83-644, fwd_kernel_inner.py:46-287):
// online softmax in base 2, O = softmax(S) V, LSE = (m + log2 l) ln 2.
//
// Work split: one workgroup = NW waves = BM = 32*NW query rows of one head; each
// wave owns 32 rows; a lane owns ONE query row (lane%32) and half of the key
// columns of every 32-key block, so row max / row sum are in-lane plus a single
// cross-half exchange.  Per K/V tile of BN keys:
//   S^T (keys x queries) = K_tile . Q^T        A = K rows from LDS, B = Q in registers
//   O^T (d x queries)   += V_tile^T . P^T      A = V^T from LDS,    B = P from the S^T accumulators
// Both tiles are staged row-major.  K rows are padded by 16 B (conflict-free
// 16-byte row reads); V rows are padded by 64 B so that the transposing LDS reads
// (ds_read_b64_tr_b16: 4 rows x 64 B per half-wave) sweep all banks once.
// Q rows on the way in and O rows on the way out pass through a private LDS area of
// the wave (32 rows, +16 B per row): global memory sees whole rows in 16-byte pieces
// of consecutive lanes, while the MFMA layouts want one row per lane.
#pragma once
#include <type_traits>

#include "fa_device.h"
#include "fa_fwd_pipe.h"

namespace fa {

template <int D, int BN, int NW>
struct FwdSmem {
  static constexpr int KSTR = D + 8;     // +16 B per row
  static constexpr int VSTR = D + 32;    // +64 B per row
  static constexpr int K_ELEMS = BN * KSTR;
  static constexpr int V_ELEMS = BN * VSTR;
  static constexpr int STAGES = 2;
  static constexpr int ROWS_OFF = STAGES * (K_ELEMS + V_ELEMS) * 2;   // the waves' row areas
  static constexpr int ROW_STR = D * 2 + 16;                          // bytes per staged Q / O row
  static constexpr int BYTES = ROWS_OFF + NW * 32 * ROW_STR;
};

// One Q tile (BM rows of head h of sequence z) against all its visible K/V tiles.
template <typename T, int D, int NW, int BN, bool kWindowed, bool kBias, bool kDropout, bool kPad>
__device__ __forceinline__ void fwd_item(const FwdArgs& a, const int z, const int h, const int mt, char* smem_raw) {
  using Tr = Traits<T>;
  using op_t = typename Tr::op_t;
  using q4_t = typename Tr::q4_t;
  using SM = FwdSmem<D, BN, NW>;
  constexpr int NT = NW * 64;
  constexpr int BM = NW * 32;
  constexpr int KS = D / 16;    // k-steps of S^T = K Q^T
  constexpr int MB = BN / 32;   // 32-key blocks per tile
  constexpr int DB = D / 32;    // 32-wide blocks of the head dim
  constexpr int TS = BN / 16;   // k-steps of O^T += V^T P^T
  constexpr int KSTR = SM::KSTR, VSTR = SM::VSTR;
  constexpr int CH = (BN * D / 8) / NT;                   // 16-byte chunks per thread, per tensor
  static_assert((BN * D / 8) % NT == 0, "tile must split evenly");

  T* Ks = reinterpret_cast<T*>(smem_raw);
  T* Vs = Ks + SM::STAGES * SM::K_ELEMS;

  const int tid = threadIdx.x;
  // At D = 256 (one wave per SIMD, accumulators in AGPRs) the wave index is taken as a scalar:
  // the branches on it are then uniform for the compiler too, and it keeps the copies of the 128
  // accumulator registers that the rarely taken full softmax step needs out of the common path
  // (they doubled the vector instructions per tile of the causal kernel: 737 -> 895 TFLOP/s at
  // S = 16384).  At D <= 128 there are no AGPRs and the plain form measures 0-4 % faster.
  const int wave = D >= 256 ? __builtin_amdgcn_readfirstlane(tid >> 6) : tid >> 6;
  const int lane = tid & 63, c = lane & 31, hi = lane >> 5;
  // columns of Q/K and of V/Out: <= D, multiples of 8; constants unless a head dim is rounded up
  const int d_qk = kPad ? a.head_dim : D, d_v = kPad ? a.head_dim_v : D;

  const SeqInfo si = get_seq(a.seq, z);
  const int q0 = mt * BM;
  if (q0 >= si.seqlen_q) return;

  Window w{0, 0};
  if (kWindowed) w = parse_window(a.mask.causal_type, a.mask.window_left, a.mask.window_right,
                                  si.seqlen_q, si.seqlen_k);
  // keep row +/- window inside int32
  w.left = w.left > (1 << 30) ? (1 << 30) : (w.left < -(1 << 30) ? -(1 << 30) : w.left);
  w.right = w.right > (1 << 30) ? (1 << 30) : (w.right < -(1 << 30) ? -(1 << 30) : w.right);
  const BlockRanges br = block_ranges(kWindowed, w.left, w.right, q0, si.seqlen_q, si.seqlen_k, BM, BN);

  const int hk = h / (a.hq / a.hk);                       // fwd_kernel.py:360
  const int row = q0 + wave * 32 + c;                     // this lane's query row
  const bool row_ok = row < si.seqlen_q;
  const int row_c = row_ok ? row : si.seqlen_q - 1;

  T* optr = reinterpret_cast<T*>(a.out) + (int64_t)si.batch_index * a.so.z + (int64_t)h * a.so.h +
            (int64_t)(si.q_start + row_c) * a.so.s;
  float* lse_ptr = a.lse ? a.lse + lse_offset(si, h, a.hq) : nullptr;

  if (br.lo > br.hi) {
    // No visible key for any row of this tile: O = 0, LSE = +inf (fwd_kernel.py:327-355)
    if (row_ok) {
      q4_t zero4 = {0, 0, 0, 0};
#pragma unroll
      for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int g = 0; g < 4; ++g)
          if (32 * db + 8 * g + 4 * hi < d_v) *reinterpret_cast<q4_t*>(optr + 32 * db + 8 * g + 4 * hi) = zero4;
      if (lse_ptr && hi == 0) lse_ptr[row] = __builtin_inff();
    }
    return;
  }

  // ---- Q rows as the B operand, resident for the whole tile ------------------
  // The wave's 32 rows come in as whole rows (16 bytes per lane, consecutive lanes along a
  // row) through its LDS area; rows past the sequence and columns past the tensors' head
  // dim read as zero (head dims are rounded up to D).
  constexpr int LPRQ = D / 8;             // 16-byte pieces per row
  constexpr int RPQ = 64 / LPRQ;          // rows per wave-wide access
  char* rowbuf = smem_raw + SM::ROWS_OFF + wave * 32 * SM::ROW_STR;
  // The descriptors of the wave's Q and O rows are built from a scalar copy of the wave index.
  // With the per-lane one the compiler takes them for divergent and wraps every access in a loop
  // over the distinct descriptors (readfirstlane, compare, masked issue): 8-16 such loops per item,
  // and a register spilled next to one of them was stored while no lane was enabled (the loop
  // leaves exec at zero and the spill landed before exec is restored), so that the fourth Q piece
  // of a D = 64 bias + dropout build was fetched from wherever the slot's old content pointed.
  const int wave_u = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wrows = si.seqlen_q - q0 - wave_u * 32 < 32 ? si.seqlen_q - q0 - wave_u * 32 : 32;   // may be <= 0
  const int rq = lane / LPRQ, cq = lane % LPRQ;
  const T* kbase = reinterpret_cast<const T*>(a.k) + (int64_t)si.batch_index * a.sk.z +
                   (int64_t)hk * a.sk.h + (int64_t)si.k_start * a.sk.s;
  const T* vbase = reinterpret_cast<const T*>(a.v) + (int64_t)si.batch_index * a.sv.z +
                   (int64_t)hk * a.sv.h + (int64_t)si.k_start * a.sv.s;
  const T* bptr = nullptr;
  if (kBias)
    bptr = reinterpret_cast<const T*>(a.bias) + (int64_t)si.batch_index * a.sb_z + (int64_t)h * a.sb_h +
           (int64_t)row_c * a.sb_m;
  // 8-byte bias loads need unit column stride and 8-byte aligned rows
  const bool bias_vec = kBias && a.sb_n == 1 && ((a.sb_m | a.sb_h | a.sb_z) & 3) == 0 &&
                        (reinterpret_cast<uintptr_t>(a.bias) & 7) == 0;

  DropoutState ds{};
  if (kDropout) ds = make_dropout(a.drop, z, h, a.hq, a.seq.max_seqlen_q, a.seq.max_seqlen_k);

  // ---- global -> register -> LDS staging -------------------------------------
  // Buffer loads: the descriptor is rebased on every tile and bounds the tile to its
  // valid rows, so rows past the end of the sequence read as zero (their scores are
  // masked and P is 0 there) and no per-lane address arithmetic is needed: a thread's
  // chunks sit RPI rows apart, which is a scalar offset on the global side and an
  // immediate offset on the LDS side.
  constexpr int LPR = D / 8;              // 16-byte chunks per row
  constexpr int RPI = NT / LPR;           // rows between two chunks of one thread
  static_assert(NT % LPR == 0, "threads must cover whole rows");
  op_t kreg[CH], vreg[CH];
  const int r0 = tid / LPR, cc0 = tid % LPR;
  const int kvoff = cc0 * 8 < d_qk ? r0 * (int)a.sk.s * 2 + cc0 * 16 : kVoffOutOfRange;      // bytes inside a tile
  const int vvoff = cc0 * 8 < d_v ? r0 * (int)a.sv.s * 2 + cc0 * 16 : kVoffOutOfRange;
  const int ksoff = RPI * (int)a.sk.s * 2, vsoff = RPI * (int)a.sv.s * 2;
  const int ldsk0 = r0 * KSTR + cc0 * 8, ldsv0 = r0 * VSTR + cc0 * 8;   // elements

  // tiles are fetched in ascending order: the tile bases and the count of rows left
  // advance by one tile per call
  const T* kt = kbase + (int64_t)br.lo * BN * a.sk.s;
  const T* vt = vbase + (int64_t)br.lo * BN * a.sv.s;
  const int64_t k_step = (int64_t)BN * a.sk.s, v_step = (int64_t)BN * a.sv.s;
  const int k_row_bytes = (int)a.sk.s * 2, v_row_bytes = (int)a.sv.s * 2;
  int rows_left = si.seqlen_k - br.lo * BN;      // > 0
  auto load_next_tile = [&]() {
    const int rows = rows_left < BN ? rows_left : BN;
    const auto krs = wave_rsrc(kt, (rows - 1) * k_row_bytes + d_qk * 2);
    const auto vrs = wave_rsrc(vt, (rows - 1) * v_row_bytes + d_v * 2);
#pragma unroll
    for (int i = 0; i < CH; ++i)
      kreg[i] = __builtin_bit_cast(op_t, __builtin_amdgcn_raw_buffer_load_b128(krs, kvoff, i * ksoff, 0));
#pragma unroll
    for (int i = 0; i < CH; ++i)
      vreg[i] = __builtin_bit_cast(op_t, __builtin_amdgcn_raw_buffer_load_b128(vrs, vvoff, i * vsoff, 0));
    kt += k_step; vt += v_step; rows_left -= BN;
  };

  // the first K/V tile is requested before the Q rows are waited for: both fetches are in flight
  // together
  load_next_tile();

  op_t qreg[KS];
  {
    const T* qw = reinterpret_cast<const T*>(a.q) + (int64_t)si.batch_index * a.sq.z + (int64_t)h * a.sq.h +
                  (int64_t)(si.q_start + q0 + wave_u * 32) * a.sq.s;
    const auto qrs = wave_rsrc(qw, wrows > 0 ? ((wrows - 1) * (int)a.sq.s + d_qk) * 2 : 0);
    const int qvoff = cq * 8 < d_qk ? rq * (int)a.sq.s * 2 + cq * 16 : kVoffOutOfRange;
    op_t qin[32 / RPQ];
#pragma unroll
    for (int i = 0; i < 32 / RPQ; ++i)
      qin[i] = __builtin_bit_cast(op_t, __builtin_amdgcn_raw_buffer_load_b128(qrs, qvoff, i * RPQ * (int)a.sq.s * 2, 2));
#pragma unroll
    for (int i = 0; i < 32 / RPQ; ++i)
      *reinterpret_cast<op_t*>(rowbuf + (i * RPQ + rq) * SM::ROW_STR + cq * 16) = qin[i];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
      qreg[ks] = *reinterpret_cast<const op_t*>(rowbuf + c * SM::ROW_STR + (16 * ks + 8 * hi) * 2);
  }


  auto store_tile = [&](int stage) {
    T* ks = Ks + stage * SM::K_ELEMS + ldsk0;
    T* vs = Vs + stage * SM::V_ELEMS + ldsv0;
#pragma unroll
    for (int i = 0; i < CH; ++i) *reinterpret_cast<op_t*>(ks + i * RPI * KSTR) = kreg[i];
#pragma unroll
    for (int i = 0; i < CH; ++i) *reinterpret_cast<op_t*>(vs + i * RPI * VSTR) = vreg[i];
  };

  // ---- online softmax state --------------------------------------------------
  f32x16 o[DB];
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int i = 0; i < 16; ++i) o[db][i] = 0.f;
  float m_i = kNegBig;   // running max, in the units of `s` below
  float l_i = 0.f;       // per-lane partial row sum (its half of the columns)
  const float qk_scale = a.sm_scale * kLog2e;
  // Fast path: the max is taken on the raw scores and the scale is folded into the
  // exponent, exp2(s*c - m*c), which needs c > 0.  With a bias (added after
  // scaling, fwd_kernel_inner.py:166-187) or c <= 0 the scores are scaled first.
  const bool prescale = kBias || !(qk_scale > 0.f);
  const float sc = prescale ? 1.0f : qk_scale;

  // lane-constant part of the V^T operand address (see lds_read_tr8)
  const int v_lane = (4 * hi + (lane & 15) / 4) * VSTR + 16 * ((lane >> 4) & 1) + 4 * (lane & 3);

  // last K tile this wave needs: on the causal diagonal the upper waves of a tile
  // see nothing in the trailing K tiles and only take part in staging and barriers
  int wave_hi = br.hi;
  if (kWindowed) {
    const int64_t wl = (int64_t)(q0 + wave * 32 + 31 < si.seqlen_q ? q0 + wave * 32 + 31 : si.seqlen_q - 1);
    int64_t cmax = wl + w.right;
    if (cmax > si.seqlen_k - 1) cmax = si.seqlen_k - 1;
    wave_hi = cmax < 0 ? -1 : (int)(cmax / BN);
  }

  // (At D = 256 the extra lane state costs the one-wave-per-SIMD kernel 2-3 %, so it keeps the
  // plain test on every masked tile.)
  constexpr bool kWaveMask = D <= 128;
  // A K tile needs no mask in this wave when every key of it is visible to every (valid) row of
  // the wave: the tile ends inside the sequence, at or before the first row's right bound, and
  // starts at or after the last row's left bound.
  const int w_rmin = q0 + wave * 32;
  const int w_rmax = w_rmin + 31 < si.seqlen_q ? w_rmin + 31 : si.seqlen_q - 1;
  auto wave_sees_all = [&](int j) -> bool {
    const int n_first = j * BN, n_last = j * BN + BN - 1;
    bool all = n_last < si.seqlen_k;
    if (kWindowed) all = all && n_last <= w_rmin + w.right && n_first >= w_rmax - w.left;
    return all;
  };
  // visible columns of this lane's row as one range [m_lo, m_lo + m_rng] (empty: m_rng < 0)
  int m_lo = 0, m_hi = si.seqlen_k - 1;
  if (kWindowed) {
    m_lo = row - w.left > 0 ? row - w.left : 0;
    m_hi = row + w.right < m_hi ? row + w.right : m_hi;
  }
  const bool m_none = m_hi < m_lo;
  const unsigned m_rng = m_none ? 0u : (unsigned)(m_hi - m_lo);

  f32x16 s[MB];   // S^T of the current tile

  // Bias tiles of the wave (32 rows x BN keys) travel as row-contiguous 16-byte pieces, consecutive
  // lanes along a row, and change to the one-row-per-lane layout of S^T in the wave's row area,
  // which is idle between the Q rows at the start and the O rows at the end of an item.  (One
  // 8-byte load per lane and 4 keys touches 32 cache lines for 16 bytes each; the vector memory
  // pipe's line rate then costs more than the bias bytes.)  A row of the area holds D keys, so a
  // tile passes in BN / BCK chunks of BCK keys.  The pieces are requested behind the QK MFMAs, not
  // before them: 16 more live registers across that phase cost the causal kernel more in spills
  // than the exposed latency costs with two waves per SIMD.
  constexpr int BCK = BN < D ? BN : D;    // keys per chunk
  constexpr int BLPR = BCK / 8;           // 16-byte pieces per chunk row
  constexpr int BRPI = 64 / BLPR;         // rows per wave-wide access
  constexpr int BNI = 32 / BRPI;          // accesses per chunk
  const int brow = lane / BLPR, bch = lane % BLPR;
  const bool bias_co = kBias && a.sb_n == 1 && ((a.sb_m | a.sb_h | a.sb_z) & 7) == 0 &&
                       (reinterpret_cast<uintptr_t>(a.bias) & 15) == 0;
  // adds chunk `ck` of tile j's bias to s (the tile lies inside the key range)
  auto bias_chunk = [&](int j, int ck) {
    const T* bh = reinterpret_cast<const T*>(a.bias) + (int64_t)si.batch_index * a.sb_z + (int64_t)h * a.sb_h;
    op_t bco[BNI];
#pragma unroll
    for (int i = 0; i < BNI; ++i) {
      int m = q0 + wave * 32 + brow + BRPI * i;
      m = m < si.seqlen_q ? m : si.seqlen_q - 1;
      bco[i] = *reinterpret_cast<const op_t*>(bh + (int64_t)m * a.sb_m + j * BN + ck * BCK + bch * 8);
    }
#pragma unroll
    for (int i = 0; i < BNI; ++i)
      *reinterpret_cast<op_t*>(rowbuf + (brow + BRPI * i) * SM::ROW_STR + bch * 16) = bco[i];
#pragma unroll
    for (int mbl = 0; mbl < BCK / 32; ++mbl)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const q4_t b4 = *reinterpret_cast<const q4_t*>(rowbuf + c * SM::ROW_STR + (mbl * 32 + 8 * g + 4 * hi) * 2);
#pragma unroll
        for (int r = 0; r < 4; ++r) s[ck * (BCK / 32) + mbl][4 * g + r] += (float)b4[r] * kLog2e;   // fwd_kernel_inner.py:187
      }
  };

  auto qk = [&](int stage) {
    const T* ks = Ks + stage * SM::K_ELEMS + c * KSTR + hi * 8;
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
      for (int i = 0; i < 16; ++i) s[mb][i] = 0.f;
    // S^T = K Q^T with the K operands read kAhead k-steps ahead of their MFMAs
    __builtin_amdgcn_s_setprio(2);
    constexpr int kAhead = 2;
    op_t ka[kAhead + 1][MB];
#pragma unroll
    for (int k = 0; k < kAhead; ++k)
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) ka[k][mb] = *reinterpret_cast<const op_t*>(ks + mb * 32 * KSTR + k * 16);
#pragma unroll
    for (int k = 0; k < KS; ++k) {
      if (k + kAhead < KS) {
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
          ka[(k + kAhead) % (kAhead + 1)][mb] =
              *reinterpret_cast<const op_t*>(ks + mb * 32 * KSTR + (k + kAhead) * 16);
      }
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) s[mb] = Tr::mfma(ka[k % (kAhead + 1)][mb], qreg[k], s[mb]);
      __builtin_amdgcn_sched_barrier(0);
    }
    __builtin_amdgcn_s_setprio(0);
  };

  // scale, bias and mask on the raw scores
  auto prepare = [&](int j, bool masked) {
    if (prescale) {
#pragma unroll
      for (int mb = 0; mb < MB; ++mb)
#pragma unroll
        for (int i = 0; i < 16; ++i) s[mb][i] *= qk_scale;
    }
    if (kBias) {
      if (bias_co && (j + 1) * BN <= si.seqlen_k) {
#pragma unroll
        for (int ck = 0; ck < BN / BCK; ++ck) bias_chunk(j, ck);
      } else if (bias_vec && (j + 1) * BN <= si.seqlen_k) {
        // a lane's four consecutive keys of every 8-key group in one 8-byte load
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
#pragma unroll
          for (int g = 0; g < 4; ++g) {
            const q4_t b4 = *reinterpret_cast<const q4_t*>(bptr + j * BN + mb * 32 + 8 * g + 4 * hi);
#pragma unroll
            for (int r = 0; r < 4; ++r) s[mb][4 * g + r] += (float)b4[r] * kLog2e;   // fwd_kernel_inner.py:187
          }
      } else {
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
#pragma unroll
          for (int i = 0; i < 16; ++i) {
            int n = j * BN + mb * 32 + 8 * (i / 4) + 4 * hi + (i % 4);
            n = n < si.seqlen_k ? n : si.seqlen_k - 1;
            s[mb][i] += (float)bptr[(int64_t)n * a.sb_n] * kLog2e;   // fwd_kernel_inner.py:187
          }
      }
    }
    if (masked && kWaveMask) {
      // column n of element (mb, i) is visible iff m_lo <= n <= m_hi, tested as one unsigned
      // comparison of n - m_lo; an empty range fails every element
      const unsigned d = m_none ? 0x40000000u : (unsigned)(j * BN + 4 * hi - m_lo);
#pragma unroll
      for (int mb = 0; mb < MB; ++mb)
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          const bool vis = d + (unsigned)(mb * 32 + 8 * (i / 4) + (i % 4)) <= m_rng;
          s[mb][i] = vis ? s[mb][i] : -__builtin_inff();
        }
    } else if (masked) {
#pragma unroll
      for (int mb = 0; mb < MB; ++mb)
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          const int n = j * BN + mb * 32 + 8 * (i / 4) + 4 * hi + (i % 4);
          bool vis = n < si.seqlen_k;
          if (kWindowed) vis = vis & (n <= row + w.right) & (n >= row - w.left);
          s[mb][i] = vis ? s[mb][i] : -__builtin_inff();
        }
    }
  };

  // dropout, operand conversion and O^T += V^T P^T on the p's held in s
  op_t va[2][DB];
  auto finish = [&](int j, const T* vs) {
    op_t pb[TS];
    if (kDropout) {
#pragma unroll
      for (int mb = 0; mb < MB; ++mb)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          const uint32_t keep = dropout_keep4(ds, row, j * BN + mb * 32 + 8 * g + 4 * hi);
#pragma unroll
          for (int r = 0; r < 4; ++r) s[mb][4 * g + r] = ((keep >> r) & 1u) ? s[mb][4 * g + r] : 0.f;
        }
    }
    // P is cast to V's dtype for the second GEMM (:274)
#pragma unroll
    for (int t = 0; t < TS; ++t) pb[t] = pack8<T>(s[t / 2], t % 2);
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_setprio(2);
#pragma unroll
    for (int t = 0; t < TS; ++t) {
      if (t + 1 < TS) {
#pragma unroll
        for (int db = 0; db < DB; ++db)
          va[(t + 1) & 1][db] = lds_read_tr8<T>(vs + (t + 1) * 16 * VSTR + db * 32, VSTR);
      }
#pragma unroll
      for (int db = 0; db < DB; ++db) o[db] = Tr::mfma(va[t & 1][db], pb[t], o[db]);
      __builtin_amdgcn_sched_barrier(0);
    }
    __builtin_amdgcn_s_setprio(0);
  };

  // Speculative softmax step: the exponentials are taken against the reference
  // maximum the rows already have, with no row maximum of the new tile.  p may
  // exceed 1 where a row's maximum grew; that is harmless (the final O = acc / l does
  // not depend on the reference) until the values leave the comfortable range of the
  // 16-bit P operand, which the row sum reveals.  Returns false, leaving the state
  // untouched, when some row needs a new reference; the caller then recomputes S and
  // takes the full step.
  bool have_ref = false;     // every row of the wave has a usable reference maximum
  float msc_ref = 0.f;       // m_i * sc
  auto sv_fast = [&](int j, int stage, bool masked) -> bool {
    const T* vs = Vs + stage * SM::V_ELEMS + v_lane;
#pragma unroll
    for (int db = 0; db < DB; ++db) va[0][db] = lds_read_tr8<T>(vs + db * 32, VSTR);
    prepare(j, masked);
    float rs = 0.f;
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        s[mb][i] = fast_exp2(__builtin_fmaf(s[mb][i], sc, -msc_ref));
        rs += s[mb][i];      // the row sum is over the fp32, undropped p (fwd_kernel_inner.py:213-214)
      }
    // also catches inf and NaN
    if (__builtin_amdgcn_ballot_w64(!(rs < 4096.f)) != 0) return false;
    l_i += rs;
    finish(j, vs);
    return true;
  };

  // full online-softmax step with the row maximum of the tile
  auto sv = [&](int j, int stage, bool masked) {
    const T* vs = Vs + stage * SM::V_ELEMS + v_lane;
    // first V^T operands: in flight while the softmax runs
#pragma unroll
    for (int db = 0; db < DB; ++db) va[0][db] = lds_read_tr8<T>(vs + db * 32, VSTR);
    prepare(j, masked);
    float mx = s[0][0];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
      for (int i = 0; i < 16; ++i) mx = fmaxf(mx, s[mb][i]);
    mx = cross_max(mx);
    // Lazy rescaling: a row adopts the new maximum only when it grew by more than
    // 2^8 in the exponent domain; until then p may exceed 1 (at most 256), which
    // fp32 accumulation and the 16-bit P operand absorb, and the final O = acc / l
    // is unchanged because l is accumulated against the same reference.
    const float m_cand = fmaxf(m_i, mx);
    const bool upd = (m_cand - m_i) * sc > 8.0f;
    const float m_new = upd ? m_cand : m_i;
    const float alpha = fast_exp2((m_i - m_new) * sc);
    const float msc = m_new * sc;
    m_i = m_new;
    msc_ref = msc;

    float rs = 0.f;
    // exp2(s*c - m*c) as one fma is exact enough while |m*c| is small; for huge
    // scores the rounding of m*c alone would be amplified by exp2, so the
    // difference is formed first (the trap documented at fwd_kernel_inner.py:197-205).
    const bool big = __builtin_amdgcn_ballot_w64(!(__builtin_fabsf(msc) < 1024.f)) != 0;
    have_ref = !big;         // rows without a visible key so far keep the seed: they fail the fast test
    if (big) {
#pragma unroll
      for (int mb = 0; mb < MB; ++mb)
#pragma unroll
        for (int i = 0; i < 16; ++i) s[mb][i] = fast_exp2((s[mb][i] - m_new) * sc);
    } else {
#pragma unroll
      for (int mb = 0; mb < MB; ++mb)
#pragma unroll
        for (int i = 0; i < 16; ++i) s[mb][i] = fast_exp2(__builtin_fmaf(s[mb][i], sc, -msc));
    }
    // the row sum is over the fp32, undropped p (fwd_kernel_inner.py:213-214)
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
      for (int i = 0; i < 16; ++i) rs += s[mb][i];
    l_i = l_i * alpha + rs;
    // rescale the accumulator only when some row of this wave moved its max
    if (__builtin_amdgcn_ballot_w64(upd) != 0) {
#pragma unroll
      for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int i = 0; i < 16; ++i) o[db][i] *= alpha;
    }
    finish(j, vs);
  };

  // ---- main loop: LDS double buffer, one barrier per tile ---------------------
  store_tile(0);
  __syncthreads();
  for (int j = br.lo; j <= br.hi; ++j) {
    const int stage = (j - br.lo) & 1;
    if (j < br.hi) load_next_tile();
    if (j <= wave_hi) {
      qk(stage);
      // per-element masks only where some row of this wave has a hidden key in the tile
      const bool masked = !br.is_full(j) && !(kWaveMask && wave_sees_all(j));
      if (!(have_ref && sv_fast(j, stage, masked))) {
        if (have_ref) qk(stage);      // the speculative step consumed S
        sv(j, stage, masked);
      }
    }
    if (j < br.hi) store_tile(stage ^ 1);
    __syncthreads();
  }

  // ---- epilogue ----------------------------------------------------------------
  const float l = cross_sum(l_i);
  const bool alive = l > 0.f;
  float inv = alive ? 1.0f / l : 0.f;
  if (kDropout) inv *= ds.scale;          // fwd_kernel.py:573-575
  // O rows leave the way the Q rows came: through the wave's LDS area, as whole rows
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      q4_t t4;
#pragma unroll
      for (int r = 0; r < 4; ++r) t4[r] = Tr::cvt(o[db][4 * g + r] * inv);
      *reinterpret_cast<q4_t*>(rowbuf + c * SM::ROW_STR + (32 * db + 8 * g + 4 * hi) * 2) = t4;
    }
  {
    T* ow = reinterpret_cast<T*>(a.out) + (int64_t)si.batch_index * a.so.z + (int64_t)h * a.so.h +
            (int64_t)(si.q_start + q0 + wave_u * 32) * a.so.s;
    const auto ors = wave_rsrc(ow, wrows > 0 ? ((wrows - 1) * (int)a.so.s + d_v) * 2 : 0);
    const int ovoff = cq * 8 < d_v ? rq * (int)a.so.s * 2 + cq * 16 : kVoffOutOfRange;
#pragma unroll
    for (int i = 0; i < 32 / RPQ; ++i) {
      const op_t x = *reinterpret_cast<const op_t*>(rowbuf + (i * RPQ + rq) * SM::ROW_STR + cq * 16);
      __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4_t, x), ors, ovoff, i * RPQ * (int)a.so.s * 2, 2);
    }
  }
  if (row_ok && lse_ptr && hi == 0)
    lse_ptr[row] = alive ? (m_i * sc + fast_log2(l)) * kLn2 : __builtin_inff();   // fwd_kernel.py:610-612
}

// Persistent workgroups: the grid holds one workgroup per CU.  Consecutive workgroup
// ids round-robin over the 8 XCDs; each XCD owns a contiguous range of (batch, head)
// pairs, so the K/V of a head stay in one L2.  The Q tiles of an XCD are ordered in
// small groups of heads, inside a group heaviest-first (causal) with the heads
// interleaved, and the workgroups of the XCD take them in serpentine order (worker p
// takes p, 2P-1-p, 2P+p, ...), which pairs heavy with light tiles.  A workgroup
// goes from one tile to the next without a relaunch.
// QB = 0: fwd_item, NW waves of 32 rows.  QB > 0: fwd_item_pipe, 4 waves of 32 * QB rows, one wave
// per SIMD.
template <typename T, int D, int NW, int BN, int QB, bool kWindowed, bool kBias, bool kDropout, bool kPad>
__global__ __attribute__((amdgpu_flat_work_group_size(NW * 64, NW * 64)))
__attribute__((amdgpu_waves_per_eu(D <= 128 && QB == 0 ? 2 : 1, D <= 128 && QB == 0 ? 2 : 1)))
void fwd_kernel(const FwdArgs a) {
  extern __shared__ __attribute__((aligned(16))) char smem_raw[];
  if (kDropout && blockIdx.x == 0 && threadIdx.x == 0) {
    // modules/flash/kernel/fwd_kernel.py:199-207
    const uint64_t seed = *a.drop.seed_ptr;
    uint64_t base = a.drop.offset2;
    if (a.drop.offset1_ptr) base += *a.drop.offset1_ptr;
    if (a.seed_out) *a.seed_out = seed;
    if (a.offset_out) *a.offset_out = base;
  }
  const int xcd = blockIdx.x % kNumXcd;
  const int p = blockIdx.x / kNumXcd;
  const int workers = gridDim.x / kNumXcd;
  const int per_group = a.zh_group * a.num_m_tiles;
  const int items = a.items_per_xcd;
  // Sequences of different lengths: the list of the valid tiles only, either all tiles of the XCD's
  // heads by their distance from the start of the sequence, the heaviest first under a causal mask
  // (LevelWalk, up to kLevelCap heads per XCD), or set by set (RaggedWalk); taken in the same
  // serpentine order.
  const bool ragged = a.seq.num_seqlens != 0;
  const int ratio = a.hq / a.hk, nseq = a.num_zh / a.hq;
  const bool levels = ragged && a.zh_per_xcd <= kLevelCap && a.num_m_tiles <= 0xffff;
  constexpr int kRows = NW * 32 * (QB > 0 ? QB : 1);
  constexpr int kSmem = QB > 0 ? FwdPipeSmem<D, BN, (QB > 0 ? QB : 1)>::BYTES : FwdSmem<D, BN, NW>::BYTES;
  const int zh_lo = xcd * a.zh_per_xcd;
  RaggedWalk walk;
  LevelWalk lwalk;
  if (levels)
    lwalk.init<NW * 64>(reinterpret_cast<uint32_t*>(smem_raw + kSmem), a.seq, zh_lo,
                        zh_lo + a.zh_per_xcd < a.num_zh ? zh_lo + a.zh_per_xcd : a.num_zh, nseq, ratio, kRows, false,
                        threadIdx.x);
  else if (ragged) walk.init(a.seq, xcd, a.zh_per_xcd, a.num_zh, ratio, nseq, kRows, false);
  for (int r = 0;; ++r) {
    const int t = r * workers + ((r & 1) ? workers - 1 - p : p);
    int z, h, mt;
    if (levels) {
      int e;
      if (!lwalk.at(t, e, mt)) break;
      split_zh(zh_lo + e, nseq, ratio, z, h);
    } else if (ragged) {
      int zh, tile;
      if (!walk.at(a.seq, t, zh, tile)) break;
      split_zh(zh, nseq, ratio, z, h);
      mt = walk.tiles_of_set() - 1 - tile;
    } else {
      if (r * workers >= items) break;
      if (t >= items) continue;
      const int gi = t / per_group, gr = t % per_group;
      const int zh_local = gi * a.zh_group + gr % a.zh_group;
      const int zh = xcd * a.zh_per_xcd + zh_local;
      if (zh_local >= a.zh_per_xcd || zh >= a.num_zh) continue;
      mt = a.num_m_tiles - 1 - gr / a.zh_group;
      split_zh(zh, nseq, ratio, z, h);
    }
    if constexpr (QB > 0) fwd_item_pipe<T, D, QB, BN, kWindowed, kBias, kDropout, kPad>(a, z, h, mt, smem_raw);
    else fwd_item<T, D, NW, BN, kWindowed, kBias, kDropout, kPad>(a, z, h, mt, smem_raw);
  }
}

// Tile table of the forward kernel, keyed on (element type, head dim, causal / windowed): NW waves
// of 32 queries each, BN keys per K/V tile.  This is what replaces the reference's tuning
// database for attn_fwd (modules/flash/aot/attn_fwd.py:69-80 lists its candidate tiles, which
// differ between causal and non-causal).  Here the measured best tile is the same on both sides
// of every key; the alternatives that lost are noted per entry (same-box A/B, bf16, B*H*D = 16384,
// S = 4096 and 16384).
template <int D_, int NW_, int BN_, int QB_> struct FwdTileOf {
  static constexpr int NW = NW_, BN = BN_, QB = QB_;
  static constexpr int BM = NW * 32 * (QB > 0 ? QB : 1);
  // (the level table of packed sequences sits behind the item's LDS)
  static constexpr int ITEM_LDS = QB > 0 ? FwdPipeSmem<D_, BN, (QB > 0 ? QB : 1)>::BYTES : FwdSmem<D_, BN, NW>::BYTES;
  static constexpr int LDS = ITEM_LDS + kLevelBytes;
};
template <typename T, int D, bool kWindowed> struct FwdTile;
// D = 64: 128-key tiles; 64-key tiles lose 2 % causal and 6 % non-causal at S = 4096.
template <typename T, bool kWindowed> struct FwdTile<T, 64, kWindowed> : FwdTileOf<64, 8, 128, 0> {};
// D = 128: 64-key tiles; 32-key tiles (finer skipping on the causal diagonal, twice the barriers)
// lose 6-7 % causal and 5 % non-causal.  128-key tiles do not fit the LDS next to the row areas.
template <typename T, bool kWindowed> struct FwdTile<T, 128, kWindowed> : FwdTileOf<128, 8, 64, 0> {};
// (The pipelined item with 64 rows per wave, FwdTileOf<128, 4, 64, 2>, halves the LDS operand traffic
// per MFMA but measures 20 % slower than this one at S = 4096 and 16384: one wave per SIMD issues
// its MFMAs, vector and LDS instructions one after the other, and two waves overlap better.)
// D = 256: one wave per SIMD (the accumulators of 32 rows take 128 registers), 32-key tiles, the
// software-pipelined item: level with fwd_item without bias and dropout (B2 H16 S8192 fp16: 903 vs
// 875 TFLOP/s non-causal, 827 vs 835 causal), 15-25 % faster with them (bias: 644 vs 553, causal
// 629 vs 510; bias + dropout + window 1024: 361 vs 333).
template <typename T, bool kWindowed> struct FwdTile<T, 256, kWindowed> : FwdTileOf<256, 4, 32, 1> {};

template <typename T, int D, bool kWindowed, bool kBias, bool kDropout, bool kPad>
hipError_t launch_fwd_variant(const FwdArgs& a, dim3 grid, hipStream_t stream) {
  using Tile = FwdTile<T, D, kWindowed>;
  constexpr int NW = Tile::NW;
  auto kern = fwd_kernel<T, D, NW, Tile::BN, Tile::QB, kWindowed, kBias, kDropout, kPad>;
  constexpr int smem = Tile::LDS;
  if (grid.x == 0) return hipSuccess;      // no batch, no head or no query row: nothing to write
  if (smem > 64 * 1024) {
    static std::atomic<uint64_t> lds_set{0};
    hipError_t e = allow_large_lds(reinterpret_cast<const void*>(kern), smem, lds_set);
    if (e != hipSuccess) return e;
  }
  hipLaunchKernelGGL(kern, grid, dim3(NW * 64), smem, stream, a);
  return hipGetLastError();
}

// kPad: a head dim of the tensors (FwdArgs::head_dim, head_dim_v) is smaller than D and the excess
// columns are masked.
template <typename T, int D, bool kPad>
hipError_t launch_fwd(const FwdArgs& a, bool windowed, bool bias, bool dropout, hipStream_t stream) {
  const int BM = windowed ? FwdTile<T, D, true>::BM : FwdTile<T, D, false>::BM;
  const int nseq = a.seq.num_seqlens != 0 ? (a.seq.num_seqlens < 0 ? -a.seq.num_seqlens : a.seq.num_seqlens)
                                          : a.batch;
  FwdArgs b = a;
  b.num_m_tiles = (a.seq.max_seqlen_q + BM - 1) / BM;
  b.num_zh = nseq * a.hq;
  b.zh_per_xcd = (b.num_zh + kNumXcd - 1) / kNumXcd;
  b.zh_group = a.hq / a.hk > 2 ? (a.hq / a.hk > 8 ? 8 : a.hq / a.hk) : 2;
  const int groups = (b.zh_per_xcd + b.zh_group - 1) / b.zh_group;
  b.items_per_xcd = groups * b.zh_group * b.num_m_tiles;
  int workers = a.num_cu / kNumXcd;          // one workgroup per CU
  if (workers < 1) workers = 1;
  if (workers > b.items_per_xcd) workers = b.items_per_xcd;
  dim3 grid((unsigned)(kNumXcd * workers));
  const int key = (windowed ? 4 : 0) | (bias ? 2 : 0) | (dropout ? 1 : 0);
  switch (key) {
    case 0: return launch_fwd_variant<T, D, false, false, false, kPad>(b, grid, stream);
    case 1: return launch_fwd_variant<T, D, false, false, true, kPad>(b, grid, stream);
    case 2: return launch_fwd_variant<T, D, false, true, false, kPad>(b, grid, stream);
    case 3: return launch_fwd_variant<T, D, false, true, true, kPad>(b, grid, stream);
    case 4: return launch_fwd_variant<T, D, true, false, false, kPad>(b, grid, stream);
    case 5: return launch_fwd_variant<T, D, true, false, true, kPad>(b, grid, stream);
    case 6: return launch_fwd_variant<T, D, true, true, false, kPad>(b, grid, stream);
    default: return launch_fwd_variant<T, D, true, true, true, kPad>(b, grid, stream);
  }
}

}  // namespace fa
