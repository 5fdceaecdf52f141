// Software-pipelined forward work item: one wave per SIMD, 32*QB query rows per wave.
//
// Same arithmetic as fwd_item (fa_fwd_impl.h; modules/flash/kernel/fwd_kernel.py:83-644,
// fwd_kernel_inner.py:46-287 of the reference), other order of work.  A workgroup is 4 waves;
// a wave keeps the whole register file (512 registers), which pays for 128 accumulator registers
// of O^T (QB * D = 256), the resident Q operands, and two units of scores in flight.  With one
// wave per SIMD nothing else hides the vector work of the softmax, so the wave overlaps it with
// its own MFMAs: the keys are cut into units of 32, and in one step the wave issues, interleaved
// in one instruction stream,
//   S^T(g)   = K(g) . Q^T                      matrix pipe, K rows from LDS
//   P(g-1)   = exp2(S^T(g-1) * c - m * c)      vector ALU (speculative step, no row maximum)
//   O^T     += V(g-2)^T . P(g-2)^T             matrix pipe, V^T from LDS
// Every K / V^T operand read from LDS feeds QB MFMAs (one per 32-row block of the wave).
//
// The speculative step takes the exponentials against the reference maximum the rows already have
// and leaves the raw scores untouched; the row sums tell whether a p left the comfortable range of
// the 16-bit operand, in which case the unit is redone from the raw scores with the full
// online-softmax step (row maximum, lazy move of the reference, rescaling of O and l).  Units that
// need a mask, the units at the ends of a wave's range and every unit while some row has no
// reference yet take the plain path: the three stages one after the other, full softmax step.
//
// LDS: two stages of K tiles and two of V tiles (BN keys each); V is staged LV tiles behind K since
// its consumer runs two units behind.  One barrier per tile.
#pragma once
#include <type_traits>

#include "fa_device.h"

namespace fa {

template <int D, int BN, int QB>
struct FwdPipeSmem {
  static constexpr int KSTR = D + 8;     // +16 B per row
  static constexpr int VSTR = D + 32;    // +64 B per row
  static constexpr int K_ELEMS = BN * KSTR;
  static constexpr int V_ELEMS = BN * VSTR;
  static constexpr int STAGES = 2;
  static constexpr int ROWS_OFF = STAGES * (K_ELEMS + V_ELEMS) * 2;   // the waves' row areas
  static constexpr int ROW_STR = D * 2 + 16;                          // bytes per staged Q / O row
  static constexpr int BYTES = ROWS_OFF + 4 * 32 * QB * ROW_STR;
};

// The rescaling of an O^T accumulator tuple (a lane's 16 values times its row's factor) in place in
// the accumulation registers: the tuple never shows up in VGPRs.  The waits cover the hazards that
// nobody checks inside an asm block: an MFMA result read by the vector ALU (up to 19 wait states)
// and a vector write read by an MFMA as its C operand.
#define FA_ACC_OPS(m) m(0) m(1) m(2) m(3) m(4) m(5) m(6) m(7) m(8) m(9) m(10) m(11) m(12) m(13) m(14) m(15)
#define FA_ACC_SCALE1(i) "v_accvgpr_read_b32 %16, %" #i "\n v_mul_f32 %16, %16, %17\n v_accvgpr_write_b32 %" #i ", %16\n"
#define FA_ACC_SPLIT(t) \
  float e0 = t[0], e1 = t[1], e2 = t[2], e3 = t[3], e4 = t[4], e5 = t[5], e6 = t[6], e7 = t[7], e8 = t[8], e9 = t[9], \
        e10 = t[10], e11 = t[11], e12 = t[12], e13 = t[13], e14 = t[14], e15 = t[15]
#define FA_ACC_JOIN(t) \
  t[0] = e0; t[1] = e1; t[2] = e2; t[3] = e3; t[4] = e4; t[5] = e5; t[6] = e6; t[7] = e7; t[8] = e8; t[9] = e9; \
  t[10] = e10; t[11] = e11; t[12] = e12; t[13] = e13; t[14] = e14; t[15] = e15
__device__ __forceinline__ void acc_scale(f32x16& t, float f) {
  float tmp;
  FA_ACC_SPLIT(t);
  asm volatile("s_nop 15\n s_nop 7\n" FA_ACC_OPS(FA_ACC_SCALE1) "s_nop 3\n"
               : "+a"(e0), "+a"(e1), "+a"(e2), "+a"(e3), "+a"(e4), "+a"(e5), "+a"(e6), "+a"(e7), "+a"(e8), "+a"(e9),
                 "+a"(e10), "+a"(e11), "+a"(e12), "+a"(e13), "+a"(e14), "+a"(e15), "=&v"(tmp)
               : "v"(f));
  FA_ACC_JOIN(t);
}

template <typename T, int D, int QB, int BN, bool kWindowed, bool kBias, bool kDropout, bool kPad>
__device__ __forceinline__ void fwd_item_pipe(const FwdArgs& a, const int z, const int h, const int mt, char* smem_raw) {
  using Tr = Traits<T>;
  using op_t = typename Tr::op_t;
  using q4_t = typename Tr::q4_t;
  using SM = FwdPipeSmem<D, BN, QB>;
  constexpr int NW = 4, NT = NW * 64;
  constexpr int RW = 32 * QB;   // rows per wave
  constexpr int BM = NW * RW;
  constexpr int KS = D / 16;    // k-steps of S^T = K Q^T per unit
  constexpr int DB = D / 32;    // 32-wide blocks of the head dim
  constexpr int UPT = BN / 32;  // units per tile
  constexpr int LV = (UPT + 1) / UPT;   // tiles that the V stages lag behind the K stages
  constexpr int NM = KS * QB;   // MFMAs per GEMM and unit (2 * DB * QB as well)
  constexpr int EPS = 16 / KS;  // softmax elements of a block behind each of its QK MFMAs
  constexpr int KSTR = SM::KSTR, VSTR = SM::VSTR;
  constexpr int CH = (BN * D / 8) / NT;
  static_assert(UPT == 1 || UPT == 2, "a step's V unit must lie in one staged tile");
  static_assert((BN * D / 8) % NT == 0, "tile must split evenly");
  static_assert(KS == 2 * DB && 16 % KS == 0, "one PV MFMA per QK MFMA, whole elements behind each");

  T* Ks = reinterpret_cast<T*>(smem_raw);
  T* Vs = Ks + SM::STAGES * SM::K_ELEMS;

  const int tid = threadIdx.x;
  // the wave index as a scalar: branches on it are uniform for the compiler too
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lane = tid & 63, c = lane & 31, hi = lane >> 5;
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
  const int w_rmin = q0 + wave * RW;                      // first row of the wave
  const int wrows = si.seqlen_q - w_rmin < RW ? si.seqlen_q - w_rmin : RW;   // valid rows, may be <= 0
  const int w_rmax = w_rmin + (wrows > 0 ? wrows : 1) - 1;

  // whole rows of Q come in and whole rows of Out leave through the wave's LDS area: 16 bytes per
  // lane, consecutive lanes along a row
  constexpr int LPRQ = D / 8;             // 16-byte pieces per row
  constexpr int RPQ = 64 / LPRQ;          // rows per wave-wide access
  char* rowbuf = smem_raw + SM::ROWS_OFF + wave * RW * SM::ROW_STR;
  const int rq = lane / LPRQ, cq = lane % LPRQ;
  auto store_rows = [&](bool zeros) {
    T* ow = reinterpret_cast<T*>(a.out) + (int64_t)si.batch_index * a.so.z + (int64_t)h * a.so.h +
            (int64_t)(si.q_start + w_rmin) * a.so.s;
    const auto ors = wave_rsrc(ow, wrows > 0 ? ((wrows - 1) * (int)a.so.s + d_v) * 2 : 0);
    const int ovoff = cq * 8 < d_v ? rq * (int)a.so.s * 2 + cq * 16 : kVoffOutOfRange;
#pragma unroll
    for (int i = 0; i < RW / RPQ; ++i) {
      u32x4_t x = {0u, 0u, 0u, 0u};
      if (!zeros) x = *reinterpret_cast<const u32x4_t*>(rowbuf + (i * RPQ + rq) * SM::ROW_STR + cq * 16);
      __builtin_amdgcn_raw_buffer_store_b128(x, ors, ovoff, i * RPQ * (int)a.so.s * 2, 0);
    }
  };
  float* lse_ptr = a.lse ? a.lse + lse_offset(si, h, a.hq) : nullptr;

  if (br.lo > br.hi) {
    // No visible key for any row of this tile: O = 0, LSE = +inf (fwd_kernel.py:327-355)
    store_rows(true);
    if (lse_ptr && hi == 0) {
#pragma unroll
      for (int qb = 0; qb < QB; ++qb)
        if (w_rmin + 32 * qb + c < si.seqlen_q) lse_ptr[w_rmin + 32 * qb + c] = __builtin_inff();
    }
    return;
  }

  // ---- K/V tile fetches: global -> registers -> LDS, whole tiles by the whole workgroup ---------
  // The buffer descriptor is rebased on every tile and bounds it to its valid rows: rows past the
  // end of the sequence read as zero (their scores are masked).
  constexpr int LPR = D / 8;              // 16-byte chunks per row
  constexpr int RPI = NT / LPR;           // rows between two chunks of one thread
  static_assert(NT % LPR == 0, "threads must cover whole rows");
  // One tile of each tensor is in flight: fetched behind one barrier, stored to LDS behind the
  // next.  Stores and fetches are unconditional and always in the same order (a tile past the last
  // one has an empty descriptor and lands in a stage nobody reads): the counts in the waits before
  // the stores then say exactly "the fetch issued one iteration ago", not "everything".
  op_t kreg[CH], vreg[CH];
  const int r0 = tid / LPR, cc0 = tid % LPR;
  const int kvoff = cc0 * 8 < d_qk ? r0 * (int)a.sk.s * 2 + cc0 * 16 : kVoffOutOfRange;      // bytes inside a tile
  const int vvoff = cc0 * 8 < d_v ? r0 * (int)a.sv.s * 2 + cc0 * 16 : kVoffOutOfRange;
  const int ksoff = RPI * (int)a.sk.s * 2, vsoff = RPI * (int)a.sv.s * 2;
  const int ldsk0 = r0 * KSTR + cc0 * 8, ldsv0 = r0 * VSTR + cc0 * 8;   // elements
  const T* kt = reinterpret_cast<const T*>(a.k) + (int64_t)si.batch_index * a.sk.z + (int64_t)hk * a.sk.h +
                (int64_t)(si.k_start + br.lo * BN) * a.sk.s;
  const T* vt = reinterpret_cast<const T*>(a.v) + (int64_t)si.batch_index * a.sv.z + (int64_t)hk * a.sv.h +
                (int64_t)(si.k_start + br.lo * BN) * a.sv.s;
  const int64_t k_step = (int64_t)BN * a.sk.s, v_step = (int64_t)BN * a.sv.s;
  const int k_row_bytes = (int)a.sk.s * 2, v_row_bytes = (int)a.sv.s * 2;
  // rows of the tiles br.lo .. br.hi that are left to fetch (> 0 at first); a fetch past the last
  // tile gets an empty descriptor and touches no memory
  int k_rows_left = (si.seqlen_k < (br.hi + 1) * BN ? si.seqlen_k : (br.hi + 1) * BN) - br.lo * BN;
  int v_rows_left = k_rows_left;
  // tiles are fetched in ascending order, K and V each at its own pace
  auto load_k_tile = [&]() {
    const int rows = k_rows_left < BN ? k_rows_left : BN;
    const auto krs = wave_rsrc(kt, rows > 0 ? (rows - 1) * k_row_bytes + d_qk * 2 : 0);
#pragma unroll
    for (int i = 0; i < CH; ++i)
      kreg[i] = __builtin_bit_cast(op_t, __builtin_amdgcn_raw_buffer_load_b128(krs, kvoff, i * ksoff, 0));
    kt += k_step; k_rows_left -= BN;
  };
  auto load_v_tile = [&]() {
    const int rows = v_rows_left < BN ? v_rows_left : BN;
    const auto vrs = wave_rsrc(vt, rows > 0 ? (rows - 1) * v_row_bytes + d_v * 2 : 0);
#pragma unroll
    for (int i = 0; i < CH; ++i)
      vreg[i] = __builtin_bit_cast(op_t, __builtin_amdgcn_raw_buffer_load_b128(vrs, vvoff, i * vsoff, 0));
    vt += v_step; v_rows_left -= BN;
  };
  auto store_k_tile = [&](int stage) {
    T* ks = Ks + stage * SM::K_ELEMS + ldsk0;
#pragma unroll
    for (int i = 0; i < CH; ++i) *reinterpret_cast<op_t*>(ks + i * RPI * KSTR) = kreg[i];
  };
  auto store_v_tile = [&](int stage) {
    T* vs = Vs + stage * SM::V_ELEMS + ldsv0;
#pragma unroll
    for (int i = 0; i < CH; ++i) *reinterpret_cast<op_t*>(vs + i * RPI * VSTR) = vreg[i];
  };

  // the first K tile is requested before the Q rows are waited for
  load_k_tile();

  // ---- Q rows as the B operand, resident for the whole item ----------------------------------------
  op_t qreg[QB][KS];
  {
    const T* qw = reinterpret_cast<const T*>(a.q) + (int64_t)si.batch_index * a.sq.z + (int64_t)h * a.sq.h +
                  (int64_t)(si.q_start + w_rmin) * a.sq.s;
    const auto qrs = wave_rsrc(qw, wrows > 0 ? ((wrows - 1) * (int)a.sq.s + d_qk) * 2 : 0);
    const int qvoff = cq * 8 < d_qk ? rq * (int)a.sq.s * 2 + cq * 16 : kVoffOutOfRange;
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) {
      op_t qin[32 / RPQ];
#pragma unroll
      for (int i = 0; i < 32 / RPQ; ++i)
        qin[i] = __builtin_bit_cast(op_t, __builtin_amdgcn_raw_buffer_load_b128(
                                              qrs, qvoff, (qb * 32 + i * RPQ) * (int)a.sq.s * 2, 0));
#pragma unroll
      for (int i = 0; i < 32 / RPQ; ++i)
        *reinterpret_cast<op_t*>(rowbuf + (qb * 32 + i * RPQ + rq) * SM::ROW_STR + cq * 16) = qin[i];
    }
#pragma unroll
    for (int qb = 0; qb < QB; ++qb)
#pragma unroll
      for (int ks = 0; ks < KS; ++ks)
        qreg[qb][ks] = *reinterpret_cast<const op_t*>(rowbuf + (qb * 32 + c) * SM::ROW_STR + (16 * ks + 8 * hi) * 2);
    // The resident operands live in accumulation registers, from where an MFMA takes its B operand
    // directly; left to itself the register allocator parks them there too but copies each one
    // back to a VGPR before every use.
#pragma unroll
    for (int qb = 0; qb < QB; ++qb)
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) asm volatile("" : "+a"(qreg[qb][ks]));
  }

  // ---- the units this wave works on ----------------------------------------------------------------
  // unit u = keys [32 u, 32 u + 32).  Every wave starts at the workgroup's first unit (left of a
  // sliding window its first units are masked out completely and contribute p = 0); past its last
  // unit (the causal diagonal) a wave multiplies zeros into O and only stages and waits.
  const int G0 = UPT * br.lo;
  int u1 = (si.seqlen_k - 1) / 32;
  if (u1 > UPT * br.hi + UPT - 1) u1 = UPT * br.hi + UPT - 1;
  if (kWindowed) {
    const int64_t cmax = (int64_t)w_rmax + w.right;
    if (cmax < (int64_t)u1 * 32 + 31) u1 = cmax < 0 ? -1 : (cmax / 32 < u1 ? (int)(cmax / 32) : u1);
  }
  if (wrows <= 0) u1 = G0 - 1;                 // no valid row in this wave
  // every key of the unit is visible to every valid row of the wave
  auto unit_sees_all = [&](int u) -> bool {
    const int n_first = u * 32, n_last = u * 32 + 31;
    bool all = n_last < si.seqlen_k;
    if (kWindowed) all = all && n_last <= w_rmin + w.right && n_first >= w_rmax - w.left;
    return all;
  };

  // ---- state ------------------------------------------------------------------------------------------
  f32x16 o[QB][DB];
#pragma unroll
  for (int qb = 0; qb < QB; ++qb)
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int i = 0; i < 16; ++i) o[qb][db][i] = 0.f;
  f32x16 acc[QB];           // S^T of the unit whose QK MFMAs run in this step
  f32x16 x[QB];             // raw S^T of the unit before it (copied out of acc at the end of a step)
  op_t pin[QB][2];          // P of the unit two back, as the B operands of its two PV k-steps
  op_t pout[QB][2];         // P of the unit before this one, being built
  float m_i[QB], msc_ref[QB], l_i[QB];
  const float qk_scale = a.sm_scale * kLog2e;
  // Fast form: the max is taken on the raw scores and the scale is folded into the exponent,
  // exp2(s*c - m*c), which needs c > 0.  With a bias (added after scaling,
  // fwd_kernel_inner.py:166-187) or c <= 0 the scores are scaled first.
  const bool prescale = kBias || !(qk_scale > 0.f);
  const float sc = prescale ? 1.0f : qk_scale;
#pragma unroll
  for (int qb = 0; qb < QB; ++qb) { m_i[qb] = kNegBig; msc_ref[qb] = kNegBig * sc; l_i[qb] = 0.f; }
  bool have_ref = false;    // every row of the wave has a usable reference maximum

  const T* bptr[QB];
  if (kBias) {
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) {
      const int row = w_rmin + 32 * qb + c;
      const int row_c = row < si.seqlen_q ? row : si.seqlen_q - 1;
      bptr[qb] = reinterpret_cast<const T*>(a.bias) + (int64_t)si.batch_index * a.sb_z + (int64_t)h * a.sb_h +
                 (int64_t)row_c * a.sb_m;
    }
  }
  // 8-byte bias loads need unit column stride and 8-byte aligned rows
  const bool bias_vec = kBias && a.sb_n == 1 && ((a.sb_m | a.sb_h | a.sb_z) & 3) == 0 &&
                        (reinterpret_cast<uintptr_t>(a.bias) & 7) == 0;
  // Bias of a unit: fetched one step ahead as row-contiguous 16-byte pieces (4 lanes along a row of
  // 32 keys, 16 rows per wave-wide access: one 8-byte load per lane and 4 keys would touch 32 cache
  // lines for 16 bytes each), turned into the one-row-per-lane layout in the wave's row area, which
  // is idle between the Q rows at the start and the O rows at the end of an item.
  constexpr int BNI = RW / 16;    // accesses per unit
  q4_t bin[QB][4];                // bias of the unit before this one, in the layout of S^T
  op_t bco[BNI];                  // pieces of this unit's bias on their way in
  const bool bias_co = kBias && a.sb_n == 1 && ((a.sb_m | a.sb_h | a.sb_z) & 7) == 0 &&
                       (reinterpret_cast<uintptr_t>(a.bias) & 15) == 0;

  DropoutState ds{};
  if (kDropout) ds = make_dropout(a.drop, z, h, a.hq, a.seq.max_seqlen_q, a.seq.max_seqlen_k);

  const int k_lane = c * KSTR + hi * 8;
  // lane-constant part of the V^T operand address (see lds_read_tr8)
  const int v_lane = (4 * hi + (lane & 15) / 4) * VSTR + 16 * ((lane >> 4) & 1) + 4 * (lane & 3);
  const f32x16 zero16 = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};

  // dropout and conversion of one pair of p's into its slot of the P operand
  auto put_pair = [&](op_t (&pout)[2], int e, float p0, float p1, uint32_t keep) {
    if (kDropout) {
      p0 = ((keep >> ((e - 1) & 3)) & 1u) ? p0 : 0.f;
      p1 = ((keep >> (e & 3)) & 1u) ? p1 : 0.f;
    }
    pout[e / 8][e % 8 - 1] = Tr::cvt(p0);      // P is cast to V's dtype for the second GEMM (:274)
    pout[e / 8][e % 8] = Tr::cvt(p1);
  };

  // Full online-softmax step on the raw scores x of unit u (modified in place): scale, bias,
  // mask, row maximum, lazy move of the reference, exponentials, row sum; O and l follow the
  // reference.  Everything accumulated in O so far must belong to the old reference.
  auto softmax_full = [&](int u, bool masked) {
    bool any_big = false;
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) {
      const int row = w_rmin + 32 * qb + c;
      if (prescale) {
#pragma unroll
        for (int i = 0; i < 16; ++i) x[qb][i] *= qk_scale;
      }
      if (kBias) {
        if (bias_co && u <= u1 && (u + 1) * 32 <= si.seqlen_k) {
          // the unit's pieces were fetched a step ago and handed over in the layout of S^T (fetch_bias, hand_over)
#pragma unroll
          for (int i = 0; i < 16; ++i) x[qb][i] += (float)bin[qb][i / 4][i % 4] * kLog2e;   // fwd_kernel_inner.py:187
        } else if (bias_vec && (u + 1) * 32 <= si.seqlen_k) {
          // a lane's four consecutive keys of every 8-key group in one 8-byte load
#pragma unroll
          for (int g = 0; g < 4; ++g) {
            const q4_t b4 = *reinterpret_cast<const q4_t*>(bptr[qb] + u * 32 + 8 * g + 4 * hi);
#pragma unroll
            for (int r = 0; r < 4; ++r) x[qb][4 * g + r] += (float)b4[r] * kLog2e;   // fwd_kernel_inner.py:187
          }
        } else {
#pragma unroll
          for (int i = 0; i < 16; ++i) {
            int n = u * 32 + 8 * (i / 4) + 4 * hi + (i % 4);
            n = n < si.seqlen_k ? n : si.seqlen_k - 1;
            x[qb][i] += (float)bptr[qb][(int64_t)n * a.sb_n] * kLog2e;   // fwd_kernel_inner.py:187
          }
        }
      }
      if (masked) {
        // visible columns of this lane's row as one range [m_lo, m_lo + m_rng]; column n of element
        // i is visible iff the unsigned n - m_lo is within it; an empty range fails every element
        int m_lo = 0, m_hi = si.seqlen_k - 1;
        if (kWindowed) {
          m_lo = row - w.left > 0 ? row - w.left : 0;
          m_hi = row + w.right < m_hi ? row + w.right : m_hi;
        }
        const bool m_none = m_hi < m_lo;
        const unsigned m_rng = m_none ? 0u : (unsigned)(m_hi - m_lo);
        const unsigned d = m_none ? 0x40000000u : (unsigned)(u * 32 + 4 * hi - m_lo);
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          const bool vis = d + (unsigned)(8 * (i / 4) + (i % 4)) <= m_rng;
          x[qb][i] = vis ? x[qb][i] : -__builtin_inff();
        }
      }
      float mx = x[qb][0];
#pragma unroll
      for (int i = 1; i < 16; ++i) mx = fmaxf(mx, x[qb][i]);
      mx = cross_max(mx);
      // Lazy rescaling: a row adopts the new maximum only when it grew by more than 2^8 in the
      // exponent domain; until then p may exceed 1 (at most 256), which fp32 accumulation and the
      // 16-bit P operand absorb, and the final O = acc / l is unchanged because l is accumulated
      // against the same reference.
      const float m_cand = fmaxf(m_i[qb], mx);
      const bool upd = (m_cand - m_i[qb]) * sc > 8.0f;
      const float m_new = upd ? m_cand : m_i[qb];
      const float alpha = fast_exp2((m_i[qb] - m_new) * sc);
      const float msc = m_new * sc;
      m_i[qb] = m_new;
      msc_ref[qb] = msc;
      // exp2(s*c - m*c) as one fma is exact enough while |m*c| is small; for huge scores the
      // rounding of m*c alone would be amplified by exp2, so the difference is formed first (the
      // trap documented at fwd_kernel_inner.py:197-205).  Rows without a visible key so far keep
      // the seed and count as big.
      const bool big = __builtin_amdgcn_ballot_w64(!(__builtin_fabsf(msc) < 1024.f)) != 0;
      any_big |= big;
      float rs = 0.f;
      float p[16];
      if (big) {
#pragma unroll
        for (int i = 0; i < 16; ++i) p[i] = fast_exp2((x[qb][i] - m_new) * sc);
      } else {
#pragma unroll
        for (int i = 0; i < 16; ++i) p[i] = fast_exp2(__builtin_fmaf(x[qb][i], sc, -msc));
      }
      // the row sum is over the fp32, undropped p (fwd_kernel_inner.py:213-214)
#pragma unroll
      for (int i = 0; i < 16; ++i) rs += p[i];
      l_i[qb] = l_i[qb] * alpha + rs;
      // rescale the accumulator only when some row of this block moved its max
      if (__builtin_amdgcn_ballot_w64(upd) != 0) {
#pragma unroll
        for (int db = 0; db < DB; ++db) acc_scale(o[qb][db], alpha);
      }
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        uint32_t keep = 0;
        if (kDropout) keep = dropout_keep4(ds, row, u * 32 + 8 * g + 4 * hi);
        put_pair(pout[qb], 4 * g + 1, p[4 * g], p[4 * g + 1], keep);
        put_pair(pout[qb], 4 * g + 3, p[4 * g + 2], p[4 * g + 3], keep);
      }
    }
    have_ref = !any_big;
  };

  // bias of unit g, used by the step after it
  auto fetch_bias = [&](int g) {
    if (kBias && bias_co && g <= u1 && (g + 1) * 32 <= si.seqlen_k) {
      const T* bh = reinterpret_cast<const T*>(a.bias) + (int64_t)si.batch_index * a.sb_z + (int64_t)h * a.sb_h;
#pragma unroll
      for (int i = 0; i < BNI; ++i) {
        int m = w_rmin + lane / 4 + 16 * i;
        m = m < si.seqlen_q ? m : si.seqlen_q - 1;
        bco[i] = *reinterpret_cast<const op_t*>(bh + (int64_t)m * a.sb_m + g * 32 + (lane % 4) * 8);
      }
    }
  };
  // what a step leaves to the next one
  auto hand_over = [&]() {
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) {
      x[qb] = acc[qb];
      pin[qb][0] = pout[qb][0];
      pin[qb][1] = pout[qb][1];
    }
    if (kBias && bias_co) {
      // (pieces that were not fetched carry leftovers; the step that would use them is not speculative)
#pragma unroll
      for (int i = 0; i < BNI; ++i)
        *reinterpret_cast<op_t*>(rowbuf + (lane / 4 + 16 * i) * SM::ROW_STR + (lane % 4) * 16) = bco[i];
#pragma unroll
      for (int qb = 0; qb < QB; ++qb)
#pragma unroll
        for (int q = 0; q < 4; ++q)
          bin[qb][q] = *reinterpret_cast<const q4_t*>(rowbuf + (qb * 32 + c) * SM::ROW_STR + (8 * q + 4 * hi) * 2);
    }
  };
  // a unit past the wave's last one (or no unit at all) contributes P = 0
  auto no_p = [&]() {
    const op_t zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) { pout[qb][0] = zero8; pout[qb][1] = zero8; }
  };

  // ---- the first two steps: nothing to multiply into O yet ---------------------------------------------
  // step G0: S^T(G0); step G0 + 1: S^T(G0 + 1) and the full softmax of unit G0
  auto first_step = [&](int g, const T* ks) {
    fetch_bias(g);
    if (g <= u1) {
      op_t ka[3];
      ka[0] = *reinterpret_cast<const op_t*>(ks);
      ka[1] = *reinterpret_cast<const op_t*>(ks + 16);
#pragma unroll
      for (int k = 0; k < KS; ++k) {
        if (k + 2 < KS) ka[(k + 2) % 3] = *reinterpret_cast<const op_t*>(ks + (k + 2) * 16);
#pragma unroll
        for (int qb = 0; qb < QB; ++qb) acc[qb] = Tr::mfma(ka[k % 3], qreg[qb][k], k == 0 ? zero16 : acc[qb]);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    if (g == G0 + 1) {
      if (G0 <= u1) softmax_full(G0, !unit_sees_all(G0));
      else no_p();
    }
    hand_over();
  };

  // ---- one pipeline step (g >= G0 + 2) -------------------------------------------------------------------
  // S^T(g) into acc; P(g-1) from the raw scores x into pout; O^T += V(g-2)^T P(g-2)^T from pin.
  // Every wave issues all the MFMAs of every step.  Past a wave's last unit the QK MFMAs run on a
  // tile it does not need, or on a stale one, and their result is dropped; the PV MFMAs multiply
  // P = 0.
  //
  // The step exists twice, each in a loop of its own.  The speculative one (kSpec) carries the
  // exponentials of unit g-1 between its MFMAs and touches the O accumulators with MFMAs only, so
  // its loop keeps them in place; it reports when some row needs the full step instead.  The plain
  // one runs the full softmax step after its MFMAs.  Were both in one loop, the rare rescaling of O
  // would make the compiler carry the 128 accumulator registers round the loop in VGPRs and copy
  // them in and out on every step; now they are copied only where the loops change over.
  auto mfma_step = [&](auto spec_tag, int g) -> bool {
    constexpr bool kSpec = decltype(spec_tag)::value;
    const int j = g / UPT, u = g % UPT;
    const T* ks = Ks + ((j - br.lo) & 1) * SM::K_ELEMS + u * 32 * KSTR + k_lane;
    const T* vs = Vs + ((j - LV - br.lo) & 1) * SM::V_ELEMS + u * 32 * VSTR + v_lane;
    fetch_bias(g);
    op_t ka[3], va[3];
    ka[0] = *reinterpret_cast<const op_t*>(ks);
    ka[1] = *reinterpret_cast<const op_t*>(ks + 16);
    va[0] = lds_read_tr8<T>(vs, VSTR);
    va[1] = lds_read_tr8<T>(vs + (1 / DB) * 16 * VSTR + (1 % DB) * 32, VSTR);
    float rs[QB], plast[QB];
    uint32_t keep[QB];
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) { rs[qb] = 0.f; plast[qb] = 0.f; keep[qb] = 0; }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int i = 0; i < NM; ++i) {
      const int k = i / QB, qb = i % QB;      // QK k-step; PV (t, db) = (k / DB, k % DB)
      if (qb == 0 && k + 2 < KS) {
        ka[(k + 2) % 3] = *reinterpret_cast<const op_t*>(ks + (k + 2) * 16);
        va[(k + 2) % 3] = lds_read_tr8<T>(vs + ((k + 2) / DB) * 16 * VSTR + ((k + 2) % DB) * 32, VSTR);
      }
      acc[qb] = Tr::mfma(ka[k % 3], qreg[qb][k], k == 0 ? zero16 : acc[qb]);
      __builtin_amdgcn_sched_barrier(0);
      if (kSpec) {
        // the softmax elements that ride behind this MFMA
#pragma unroll
        for (int q = 0; q < EPS; ++q) {
          const int e = EPS * k + q;
          if (kDropout && e % 4 == 0)
            keep[qb] = dropout_keep4(ds, w_rmin + 32 * qb + c, (g - 1) * 32 + 8 * (e / 4) + 4 * hi);
          float xv = x[qb][e];
          // (without a bias the speculative step is only taken with a positive scale: sc = qk_scale)
          float p;
          if (kBias) p = fast_exp2(__builtin_fmaf(xv, qk_scale, (float)bin[qb][e / 4][e % 4] * kLog2e) - msc_ref[qb]);
          else p = fast_exp2(__builtin_fmaf(xv, qk_scale, -msc_ref[qb]));
          rs[qb] += p;      // the row sum is over the fp32, undropped p (fwd_kernel_inner.py:213-214)
          if (e & 1) put_pair(pout[qb], e, plast[qb], p, keep[qb]);
          else plast[qb] = p;
        }
        __builtin_amdgcn_sched_barrier(0);
      }
      o[qb][k % DB] = Tr::mfma(va[k % 3], pin[qb][k / DB], o[qb][k % DB]);
      __builtin_amdgcn_sched_barrier(0);
    }
    if (!kSpec) return false;
    // a row whose p grew too far (also inf and NaN) takes the full step on the untouched scores
    bool redo = false;
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) redo |= !(rs[qb] < 4096.f);
    if (__builtin_amdgcn_ballot_w64(redo) != 0) return true;
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) l_i[qb] += rs[qb];
    return false;
  };
  // unit g-1 may take the speculative step (given a reference in every row)
  auto spec_ok = [&](int g) -> bool {
    return g <= u1 && unit_sees_all(g - 1) && (kBias ? bias_co : !prescale);
  };

  // ---- main loop ---------------------------------------------------------------------------------------------
  // Tile j is entered behind a barrier: K(j) and V(j - LV) are in LDS then; K(j + 1) and
  // V(j - LV + 1) are stored and the tiles after them requested.
  {
    const op_t zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) { pin[qb][0] = zero8; pin[qb][1] = zero8; pout[qb][0] = zero8; pout[qb][1] = zero8; }
  }
  store_k_tile(0);
  load_k_tile();              // K(lo + 1)
  if (LV == 1) load_v_tile(); // V(lo)
  auto enter_tile = [&](int g) {
    if ((g - G0) % UPT != 0) return;
    const int j = g / UPT;
    __syncthreads();
    // K(j + 1) and V(j - LV + 1) go to LDS, K(j + 2) and V(j - LV + 2) are requested
    const int tv = j - LV + 1 - br.lo;
    store_k_tile((j + 1 - br.lo) & 1);
    if (tv >= 0) store_v_tile(tv & 1);
    load_k_tile();
    if (tv + 1 >= 0) load_v_tile();
  };
  // the first two steps
  enter_tile(G0);
  first_step(G0, Ks + k_lane);
  enter_tile(G0 + 1);
  first_step(G0 + 1, Ks + ((G0 + 1) / UPT - br.lo) * SM::K_ELEMS + ((G0 + 1) % UPT) * 32 * KSTR + k_lane);
  const int g_last = UPT * (br.hi + LV) + UPT - 1;
  int g = G0 + 2;
  while (g <= g_last) {
#pragma nounroll
    while (g <= g_last && !(have_ref && spec_ok(g))) {
      enter_tile(g);
      mfma_step(std::false_type{}, g);
      // O belongs to the old reference up to and including this step's MFMAs
      if (g - 1 <= u1) softmax_full(g - 1, !unit_sees_all(g - 1));
      else no_p();
      hand_over();
      ++g;
    }
    bool redo = false;
#pragma nounroll
    while (g <= g_last && spec_ok(g)) {
      enter_tile(g);
      redo = mfma_step(std::true_type{}, g);
      if (redo) break;
      hand_over();
      ++g;
    }
    if (redo) {
      softmax_full(g - 1, false);
      hand_over();
      ++g;
    }
  }
  __syncthreads();

  // ---- epilogue ------------------------------------------------------------------------------------------------
#pragma unroll
  for (int qb = 0; qb < QB; ++qb) {
    const float l = cross_sum(l_i[qb]);
    const bool alive = l > 0.f;
    float inv = alive ? 1.0f / l : 0.f;
    if (kDropout) inv *= ds.scale;          // fwd_kernel.py:573-575
#pragma unroll
    for (int db = 0; db < DB; ++db) {
#pragma unroll
      for (int g4 = 0; g4 < 4; ++g4) {
        q4_t t4;
#pragma unroll
        for (int r = 0; r < 4; ++r) t4[r] = Tr::cvt(o[qb][db][4 * g4 + r] * inv);
        *reinterpret_cast<q4_t*>(rowbuf + (qb * 32 + c) * SM::ROW_STR + (32 * db + 8 * g4 + 4 * hi) * 2) = t4;
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    const int row = w_rmin + 32 * qb + c;
    if (lse_ptr && row < si.seqlen_q && hi == 0)
      lse_ptr[row] = alive ? (m_i[qb] * sc + fast_log2(l)) * kLn2 : __builtin_inff();   // fwd_kernel.py:610-612
  }
  store_rows(false);
}

}  // namespace fa
