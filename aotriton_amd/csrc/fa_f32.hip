// MFMA kernels for fp32 tensors (v_mfma_f32_32x32x2_f32), head dims up to 512, gfx950.
//
// The reference compiles its kernels for fp32 tensors as well ('*fp32:16' among the tensor types of
// modules/flash/aot/_common.py:10-14); these compute what the 16-bit kernels of this library do
//   forward   modules/flash/kernel/fwd_kernel.py:83-644, fwd_kernel_inner.py:46-287
//   dK, dV    modules/flash/kernel/bwd_kernel_dk_dv.py:48-417, bwd_inner_dk_dv.py:28-267
//   dQ, dB    modules/flash/kernel/bwd_kernel_dq.py:45-389, bwd_inner_dq.py:28-215
// with every product and sum in fp32 (P and dS stay fp32 for the second GEMMs: they are "cast to
// V's type", which is fp32 here).
//
// Layout of the fp32 MFMA (wave64, lane = 32 hi + c): A holds row c, k = hi (one float per lane); B
// holds column c, k = hi; C/D as for the 16-bit shapes (column c, rows 8 (i / 4) + 4 hi + i % 4).
// The contraction index is a dummy, so a lane's 16-byte piece of a row (columns 8 j + 4 hi + e,
// e = 0..3) feeds four MFMAs, and an accumulator element i is, as it stands, the B operand of the
// k-step whose A operand is row 8 (i / 4) + 4 hi + i % 4 of the other tile: no transposing read, no
// repacking.  One MFMA does 4096 FLOP in 64 cycles (157 TFLOP/s on the chip), so these kernels are
// bound by the matrix pipe and everything around it is kept simple.
//
// The structure is that of the kernels for head dims above 256 (fa_d512.hip): the head dim is
// split over four waves that work on the same 32 rows, the GEMMs that contract over the head dim
// exchange 32 x 32 partial blocks through LDS, and in the backward each wave does a quarter of the
// element work and hands P and dS on.  Compiled for 128, 256 and 512 columns (smaller head dims
// zero-filled).  At 512 columns two staged tiles fill 128 KB of the 160 KB of LDS: the forward and
// the dQ kernel then run one 32-row block per workgroup instead of two, and the partial blocks of
// S and dP go through ONE area one after the other (two more barriers per tile, next to 256 MFMAs
// of 64 cycles per wave).
#include "fa_device.h"
#include "fa_kernels.h"

namespace fa {
namespace {

constexpr int kNW = 4;           // waves per 32-row block
constexpr int kBC = 32;          // rows of the streamed tiles per step
constexpr int kNT = kNW * 64;
constexpr int kPartBytes = kNW * 64 * 16 * 4;     // one partial block per wave
constexpr int kOpndBytes = 4 * 64 * 16;           // one block of P or dS: 4 quarters x 64 lanes x 4 floats

template <int D>
struct Cfg {
  static constexpr int DW = D / kNW;      // columns a wave owns
  static constexpr int KJ = DW / 8;       // 16-byte pieces of a lane per row (each feeds four MFMAs)
  static constexpr int DB = DW / 32;      // 32-column blocks a wave owns
  static constexpr int STR = D;           // floats per tile row in LDS (unpadded, pieces swizzled)
  static constexpr int TILE_BYTES = kBC * STR * 4;
  static constexpr int RB = D > 256 ? 1 : 2;      // 32-row blocks per workgroup (forward, dQ)
  static constexpr int BR = 32 * RB;
  static constexpr int NT = RB * kNT;
  static constexpr bool ONE_PART = D > 256;       // S and dP partial blocks share one area
  static constexpr int PARTS = ONE_PART ? 1 : 2;
};

// LDS tiles keep the 16-byte piece q of row r at piece position q ^ swz(r).  Two access patterns must
// sweep the 64 banks once: a quarter-wave reading one piece each of 16 consecutive rows (swz is a
// bijection on r % 16), and a wave reading 32 consecutive floats each of two rows four apart (bit 3 of
// swz is bit 2 of r, so the two rows' eight pieces fall into different halves of the banks).  With
// padded rows instead, one of the two patterns always pairs up lanes on a bank.
__device__ __forceinline__ int swz(int r) { return (r & 3) | (((r >> 2) & 1) << 3) | (((r >> 3) & 1) << 2); }

__device__ __forceinline__ f32x16 mfma32(float a, float b, f32x16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, 0, 0, 0);
}

__device__ __forceinline__ void part_write(float* area, int wave, int lane, const f32x16& x) {
#pragma unroll
  for (int g = 0; g < 4; ++g) {
    const f32x4 t = {x[4 * g], x[4 * g + 1], x[4 * g + 2], x[4 * g + 3]};
    *reinterpret_cast<f32x4*>(area + ((wave * 4 + g) * 64 + lane) * 4) = t;
  }
}
// elements 4 g .. 4 g + 3 of every lane, the waves' partial blocks added in wave order
__device__ __forceinline__ f32x4 part_sum_quarter(const float* area, int g, int lane) {
  f32x4 acc = *reinterpret_cast<const f32x4*>(area + (g * 64 + lane) * 4);
#pragma unroll
  for (int w = 1; w < kNW; ++w) {
    const f32x4 t = *reinterpret_cast<const f32x4*>(area + ((w * 4 + g) * 64 + lane) * 4);
#pragma unroll
    for (int r = 0; r < 4; ++r) acc[r] += t[r];
  }
  return acc;
}
__device__ __forceinline__ f32x16 part_sum(const float* area, int lane) {
  f32x16 x;
#pragma unroll
  for (int g = 0; g < 4; ++g) {
    const f32x4 q = part_sum_quarter(area, g, lane);
#pragma unroll
    for (int r = 0; r < 4; ++r) x[4 * g + r] = q[r];
  }
  return x;
}
__device__ __forceinline__ f32x16 opnd_read(const float* area, int lane) {
  f32x16 x;
#pragma unroll
  for (int g = 0; g < 4; ++g) {
    const f32x4 q = *reinterpret_cast<const f32x4*>(area + (g * 64 + lane) * 4);
#pragma unroll
    for (int r = 0; r < 4; ++r) x[4 * g + r] = q[r];
  }
  return x;
}

// A tile of kBC rows x D floats, global -> registers -> LDS by the whole workgroup of NT threads, in
// 16-byte pieces.  The buffer descriptor bounds the tile to its valid rows and columns; what lies
// outside reads as zero.
template <int D, int NT>
struct TileFetch {
  static constexpr int LPR = D / 4;             // pieces per row
  static constexpr int RPI = NT / LPR;          // rows between two pieces of a thread
  static constexpr int CH = kBC / RPI;          // pieces per thread
  static_assert(NT % LPR == 0 && kBC % RPI == 0, "threads must cover the tile evenly");
  f32x4 reg[CH];
  __device__ __forceinline__ void load(const float* tile, int rows, int64_t row_stride, int cols, int tid) {
    const int r0 = tid / LPR, cc0 = tid % LPR;
    const auto rs = wave_rsrc(tile, rows > 0 ? ((rows - 1) * (int)row_stride + cols) * 4 : 0);
    const int voff = cc0 * 4 < cols ? r0 * (int)row_stride * 4 + cc0 * 16 : kVoffOutOfRange;
#pragma unroll
    for (int i = 0; i < CH; ++i)
      reg[i] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(rs, voff, i * RPI * (int)row_stride * 4, 0));
  }
  __device__ __forceinline__ void store(float* lds, int tid) const {
    const int r0 = tid / LPR, cc0 = tid % LPR;
#pragma unroll
    for (int i = 0; i < CH; ++i)
      *reinterpret_cast<f32x4*>(lds + (r0 + i * RPI) * Cfg<D>::STR + (cc0 ^ swz(r0 + i * RPI)) * 4) = reg[i];
  }
};

// the wave's columns of one row as resident B operands; columns past `cols` read as zero
template <int D>
__device__ __forceinline__ void load_resident(f32x4 (&reg)[Cfg<D>::KJ], const float* rowp, int col0, int hi, int cols) {
  const f32x4 zero4 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int j = 0; j < Cfg<D>::KJ; ++j)
    reg[j] = col0 + 8 * j + 4 * hi < cols ? *reinterpret_cast<const f32x4*>(rowp + col0 + 8 * j + 4 * hi) : zero4;
}
// acc += (rows of an LDS tile) x (resident rows), over the wave's columns
template <int D>
__device__ __forceinline__ f32x16 row_gemm(const float* tile, int c, int hi, int col0,
                                           const f32x4 (&res)[Cfg<D>::KJ], f32x16 acc) {
  const float* p = tile + c * Cfg<D>::STR;
  const int q0 = col0 / 4 + hi, sw = swz(c);
#pragma unroll
  for (int j = 0; j < Cfg<D>::KJ; ++j) {
    const f32x4 a4 = *reinterpret_cast<const f32x4*>(p + ((q0 + 2 * j) ^ sw) * 4);
#pragma unroll
    for (int e = 0; e < 4; ++e) acc = mfma32(a4[e], res[j][e], acc);
    // at 512 columns the registers are full of accumulators and resident operands: keep the
    // scheduler from requesting all sixteen pieces of the row up front
    if (Cfg<D>::KJ > 8 && j % 4 == 3) __builtin_amdgcn_sched_barrier(0);
  }
  return acc;
}
// acc[db] += (tile^T, the wave's columns) x (a 32 x 32 block held as accumulator elements)
template <int D>
__device__ __forceinline__ void col_gemm(const float* tile, int c, int hi, int col0, const f32x16& x,
                                         f32x16 (&acc)[Cfg<D>::DB]) {
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const int r = 8 * (i / 4) + 4 * hi + (i % 4);
    const float* p = tile + r * Cfg<D>::STR + (c & 3);
    const int q0 = (col0 + c) / 4, sw = swz(r);
#pragma unroll
    for (int db = 0; db < Cfg<D>::DB; ++db) acc[db] = mfma32(p[((q0 + 8 * db) ^ sw) * 4], x[i], acc[db]);
    if (Cfg<D>::KJ > 8 && i % 4 == 3) __builtin_amdgcn_sched_barrier(0);
  }
}

// the window of a sequence, kept inside int32 when added to a row or a key
template <bool kWindowed>
__device__ __forceinline__ Window window_of(const MaskArgs& m, int sq, int sk) {
  Window w{0, 0};
  if (kWindowed) w = parse_window(m.causal_type, m.window_left, m.window_right, sq, sk);
  w.left = w.left > (1 << 30) ? (1 << 30) : (w.left < -(1 << 30) ? -(1 << 30) : w.left);
  w.right = w.right > (1 << 30) ? (1 << 30) : (w.right < -(1 << 30) ? -(1 << 30) : w.right);
  return w;
}

// ---------------------------------------------------------------------------------------------
// forward: one workgroup = 64 (at 512 columns: 32) query rows of one head, four waves per 32-row block
// ---------------------------------------------------------------------------------------------
// At 128 columns there are two K stages: K of the next tile is published behind the PV MFMAs of
// the current one (that stage was last read a tile earlier), V of a tile behind the QK MFMAs of the
// same tile (the V stage was released by the barrier that ended the tile before, and is read behind
// the partial-block barrier), so a tile costs two barriers (forward + 2.5-4.5 %: 110 -> 115 TFLOP/s
// at B4 H32 S4096).  At 256 columns the same schedule measures 1 % slower and at 512 a second K
// stage does not fit; there the next tile is published between two barriers of its own.
template <int D>
struct SmemFwd {
  static constexpr int K_STAGES = D > 128 ? 1 : 2;
  static constexpr int V_OFF = K_STAGES * Cfg<D>::TILE_BYTES;
  static constexpr int PART_OFF = V_OFF + Cfg<D>::TILE_BYTES;
  static constexpr int BYTES = PART_OFF + Cfg<D>::RB * kPartBytes;
};

template <int D, bool kWindowed, bool kBias, bool kDropout>
__global__ __launch_bounds__(Cfg<D>::NT) void fwd_f32_kernel(const FwdArgs a) {
  using C = Cfg<D>;
  using SM = SmemFwd<D>;
  extern __shared__ __attribute__((aligned(16))) char smem_raw[];
  float* Ks = reinterpret_cast<float*>(smem_raw);
  float* Vs = reinterpret_cast<float*>(smem_raw + SM::V_OFF);

  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int rb = wave / kNW, cw = wave % kNW;             // row block, column share
  const int lane = tid & 63, c = lane & 31, hi = lane >> 5;
  // one workgroup per (sequence, q-head, Q tile): the tiles of a kv-head's group back to back on one
  // XCD, most visible keys (causal) first
  const int nmt = (a.seq.max_seqlen_q + C::BR - 1) / C::BR, group = a.hq / a.hk;
  int pair, r_item;
  if (!xcd_item(blockIdx.x, nseq_of(a.seq, a.batch) * a.hk, group * nmt, pair, r_item)) return;
  const int z = pair / a.hk, h = (pair % a.hk) * group + r_item % group;
  const int mt = nmt - 1 - r_item / group;
  const int d_qk = a.head_dim, d_v = a.head_dim_v;
  float* part = reinterpret_cast<float*>(smem_raw + SM::PART_OFF) + rb * (kPartBytes / 4);
  if (kDropout && blockIdx.x == 0 && tid == 0) {
    // modules/flash/kernel/fwd_kernel.py:199-207
    uint64_t base = a.drop.offset2;
    if (a.drop.offset1_ptr) base += *a.drop.offset1_ptr;
    if (a.seed_out) *a.seed_out = *a.drop.seed_ptr;
    if (a.offset_out) *a.offset_out = base;
  }

  const SeqInfo si = get_seq(a.seq, z);
  const int q0 = mt * C::BR;
  if (q0 >= si.seqlen_q) return;
  const Window w = window_of<kWindowed>(a.mask, si.seqlen_q, si.seqlen_k);
  const BlockRanges br = block_ranges(kWindowed, w.left, w.right, q0, si.seqlen_q, si.seqlen_k, C::BR, kBC);

  const int hk = h / (a.hq / a.hk);                       // fwd_kernel.py:360
  const int row = q0 + 32 * rb + c;                       // this lane's query row (the same in the four waves of a row block)
  const bool row_ok = row < si.seqlen_q;
  const int row_c = row_ok ? row : si.seqlen_q - 1;
  const int col0 = cw * C::DW;                            // first column of this wave's share

  float* optr = reinterpret_cast<float*>(a.out) + (int64_t)si.batch_index * a.so.z + (int64_t)h * a.so.h +
                (int64_t)(si.q_start + row_c) * a.so.s + col0;
  float* lse_ptr = a.lse ? a.lse + lse_offset(si, h, a.hq) : nullptr;

  if (br.lo > br.hi) {
    // no visible key for any row of this tile: O = 0, LSE = +inf (fwd_kernel.py:327-355)
    if (row_ok) {
      const f32x4 zero4 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int db = 0; db < C::DB; ++db)
#pragma unroll
        for (int g = 0; g < 4; ++g)
          if (col0 + 32 * db + 8 * g + 4 * hi < d_v) *reinterpret_cast<f32x4*>(optr + 32 * db + 8 * g + 4 * hi) = zero4;
      if (lse_ptr && cw == 0 && hi == 0) lse_ptr[row] = __builtin_inff();
    }
    return;
  }

  f32x4 qreg[C::KJ];
  load_resident<D>(qreg, reinterpret_cast<const float*>(a.q) + (int64_t)si.batch_index * a.sq.z + (int64_t)h * a.sq.h +
                             (int64_t)(si.q_start + row_c) * a.sq.s, col0, hi, d_qk);

  const float* kt = reinterpret_cast<const float*>(a.k) + (int64_t)si.batch_index * a.sk.z + (int64_t)hk * a.sk.h +
                    (int64_t)(si.k_start + br.lo * kBC) * a.sk.s;
  const float* vt = reinterpret_cast<const float*>(a.v) + (int64_t)si.batch_index * a.sv.z + (int64_t)hk * a.sv.h +
                    (int64_t)(si.k_start + br.lo * kBC) * a.sv.s;
  int rows_left = si.seqlen_k - br.lo * kBC;      // > 0
  TileFetch<D, C::NT> kf, vf;
  auto fetch = [&]() {
    const int rows = rows_left < kBC ? rows_left : kBC;
    kf.load(kt, rows, a.sk.s, d_qk, tid);
    vf.load(vt, rows, a.sv.s, d_v, tid);
    kt += (int64_t)kBC * a.sk.s; vt += (int64_t)kBC * a.sv.s; rows_left -= kBC;
  };
  constexpr bool kTwoK = SM::K_STAGES == 2;
  auto publish_k = [&](int stage) { kf.store(Ks + stage * (C::TILE_BYTES / 4), tid); };
  auto publish_v = [&]() { vf.store(Vs, tid); };

  const float* bptr = nullptr;
  if (kBias)
    bptr = reinterpret_cast<const float*>(a.bias) + (int64_t)si.batch_index * a.sb_z + (int64_t)h * a.sb_h +
           (int64_t)row_c * a.sb_m;
  DropoutState ds{};
  if (kDropout) ds = make_dropout(a.drop, z, h, a.hq, a.seq.max_seqlen_q, a.seq.max_seqlen_k);

  f32x16 o[C::DB];
#pragma unroll
  for (int db = 0; db < C::DB; ++db)
#pragma unroll
    for (int i = 0; i < 16; ++i) o[db][i] = 0.f;
  float m_i = kNegBig;   // running max, in the units of the scores below
  float l_i = 0.f;       // per-lane partial row sum (its half of the columns)
  const float qk_scale = a.sm_scale * kLog2e;
  // the scale is folded into the exponent, exp2((s - m) c), which needs c > 0; with a bias (added
  // after scaling, fwd_kernel_inner.py:166-187) or c <= 0 the scores are scaled first
  const bool prescale = kBias || !(qk_scale > 0.f);
  const float sc = prescale ? 1.0f : qk_scale;

  // visible columns of this lane's row as one range [m_lo, m_lo + m_rng]
  int m_lo = 0, m_hi = si.seqlen_k - 1;
  if (kWindowed) {
    m_lo = row - w.left > 0 ? row - w.left : 0;
    m_hi = row + w.right < m_hi ? row + w.right : m_hi;
  }
  const bool m_none = m_hi < m_lo;
  const unsigned m_rng = m_none ? 0u : (unsigned)(m_hi - m_lo);

  fetch();
  publish_k(0);
  publish_v();
  __syncthreads();
  for (int j = br.lo; j <= br.hi; ++j) {
    const int stage = kTwoK ? (j - br.lo) & 1 : 0;
    if (!kTwoK && j < br.hi) fetch();
    // this wave's share of S^T = K Q^T
    f32x16 s;
#pragma unroll
    for (int i = 0; i < 16; ++i) s[i] = 0.f;
    s = row_gemm<D>(Ks + stage * (C::TILE_BYTES / 4), c, hi, col0, qreg, s);
    if (kTwoK) {
      // behind the MFMAs: V of this tile goes to its stage, then the staging registers take the next tile
      if (j > br.lo) publish_v();
      if (j < br.hi) fetch();
    }
    part_write(part, cw, lane, s);
    __syncthreads();
    s = part_sum(part, lane);

    // scale, bias and mask on the raw scores
    if (prescale) {
#pragma unroll
      for (int i = 0; i < 16; ++i) s[i] *= qk_scale;
    }
    if (kBias) {
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        int n = j * kBC + 8 * (i / 4) + 4 * hi + (i % 4);
        n = n < si.seqlen_k ? n : si.seqlen_k - 1;
        s[i] += bptr[(int64_t)n * a.sb_n] * kLog2e;   // fwd_kernel_inner.py:187
      }
    }
    if (!br.is_full(j)) {
      // column n of element i is visible iff m_lo <= n <= m_hi, one unsigned comparison of n - m_lo
      const unsigned d = m_none ? 0x40000000u : (unsigned)(j * kBC + 4 * hi - m_lo);
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const bool vis = d + (unsigned)(8 * (i / 4) + (i % 4)) <= m_rng;
        s[i] = vis ? s[i] : -__builtin_inff();
      }
    }
    // online softmax (fwd_kernel_inner.py:189-232); the difference s - m is formed before the
    // scale so that huge scores lose nothing to the rounding of m c
    float mx = s[0];
#pragma unroll
    for (int i = 1; i < 16; ++i) mx = fmaxf(mx, s[i]);
    mx = cross_max(mx);
    const float m_new = fmaxf(m_i, mx);
    const float alpha = fast_exp2((m_i - m_new) * sc);
    m_i = m_new;
    float rs = 0.f;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      s[i] = fast_exp2((s[i] - m_new) * sc);
      rs += s[i];                       // the row sum is over the undropped p (:213-214)
    }
    l_i = l_i * alpha + rs;
    if (__builtin_amdgcn_ballot_w64(alpha != 1.0f) != 0) {   // some row of the wave moved its maximum
#pragma unroll
      for (int db = 0; db < C::DB; ++db)
#pragma unroll
        for (int i = 0; i < 16; ++i) o[db][i] *= alpha;
    }
    if (kDropout) {
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const uint32_t keep = dropout_keep4(ds, row, j * kBC + 8 * g + 4 * hi);
#pragma unroll
        for (int r = 0; r < 4; ++r) s[4 * g + r] = ((keep >> r) & 1u) ? s[4 * g + r] : 0.f;
      }
    }
    // O^T += V^T P^T on this wave's columns
    col_gemm<D>(Vs, c, hi, col0, s, o);
    if (kTwoK) {
      if (j < br.hi) publish_k(stage ^ 1);
      __syncthreads();               // V and the partial blocks have been read, the next K is in place
    } else {
      __syncthreads();               // the tile and the partial blocks have been read
      if (j < br.hi) {
        publish_k(0);
        publish_v();
        __syncthreads();
      }
    }
  }

  const float l = cross_sum(l_i);
  const bool alive = l > 0.f;
  float inv = alive ? 1.0f / l : 0.f;
  if (kDropout) inv *= ds.scale;          // fwd_kernel.py:573-575
  if (row_ok) {
#pragma unroll
    for (int db = 0; db < C::DB; ++db)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        f32x4 t4;
#pragma unroll
        for (int r = 0; r < 4; ++r) t4[r] = o[db][4 * g + r] * inv;
        if (col0 + 32 * db + 8 * g + 4 * hi < d_v) *reinterpret_cast<f32x4*>(optr + 32 * db + 8 * g + 4 * hi) = t4;
      }
    if (lse_ptr && cw == 0 && hi == 0)
      lse_ptr[row] = alive ? (m_i * sc + fast_log2(l)) * kLn2 : __builtin_inff();   // fwd_kernel.py:610-612
  }
}

// ---------------------------------------------------------------------------------------------
// dK, dV: one workgroup = 32 keys of one kv-head on 4 waves; the lane's key is lane % 32, the
// queries of a tile are spread over the accumulator elements
// ---------------------------------------------------------------------------------------------
template <int D>
struct SmemDkDv {
  static constexpr int STAT_OFF = 2 * Cfg<D>::TILE_BYTES;
  static constexpr int PART_OFF = STAT_OFF + 2 * kBC * 4;
  static constexpr int OPND_OFF = PART_OFF + Cfg<D>::PARTS * kPartBytes;
  static constexpr int BYTES = OPND_OFF + 2 * kOpndBytes;
};

template <int D, bool kWindowed, bool kBias, bool kDropout>
__global__ __launch_bounds__(kNT) void bwd_dkdv_f32_kernel(const BwdArgs a) {
  using C = Cfg<D>;
  using SM = SmemDkDv<D>;
  extern __shared__ __attribute__((aligned(16))) char smem_raw[];
  float* Qs = reinterpret_cast<float*>(smem_raw);
  float* dOs = reinterpret_cast<float*>(smem_raw + C::TILE_BYTES);
  float* Ls = reinterpret_cast<float*>(smem_raw + SM::STAT_OFF);
  float* Ds = Ls + kBC;
  float* partS = reinterpret_cast<float*>(smem_raw + SM::PART_OFF);
  float* partD = C::ONE_PART ? partS : partS + kPartBytes / 4;
  float* opP = reinterpret_cast<float*>(smem_raw + SM::OPND_OFF);
  float* opS = opP + kOpndBytes / 4;

  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lane = tid & 63, c = lane & 31, hi = lane >> 5;
  // one workgroup per (sequence, kv-head, key block): the key blocks of a kv-head back to back on
  // one XCD, those that the most queries see (causal) first
  int pair, nt;
  if (!xcd_item(blockIdx.x, nseq_of(a.seq, a.batch) * a.hk, (a.seq.max_seqlen_k + kBC - 1) / kBC, pair, nt)) return;
  const int z = pair / a.hk, hk = pair % a.hk;
  const int d_qk = a.head_dim, d_v = a.head_dim_v;
  const int col0 = wave * C::DW;

  const SeqInfo si = get_seq(a.seq, z);
  const int n0 = nt * kBC;
  if (n0 >= si.seqlen_k) return;
  const Window w = window_of<kWindowed>(a.mask, si.seqlen_q, si.seqlen_k);
  // rows are keys here, columns are queries: key n sees query m iff n - right <= m <= n + left
  // (bwd_kernel_dk_dv.py:268-279 passes the window transposed in the same way)
  const BlockRanges br = block_ranges(kWindowed, w.right, w.left, n0, si.seqlen_k, si.seqlen_q, kBC, kBC);

  const int key = n0 + c;
  const bool key_ok = key < si.seqlen_k;
  const int key_c = key_ok ? key : si.seqlen_k - 1;
  float* dkptr = reinterpret_cast<float*>(a.dk) + (int64_t)si.batch_index * a.sdk.z + (int64_t)hk * a.sdk.h +
                 (int64_t)(si.k_start + key_c) * a.sdk.s + col0;
  float* dvptr = reinterpret_cast<float*>(a.dv) + (int64_t)si.batch_index * a.sdv.z + (int64_t)hk * a.sdv.h +
                 (int64_t)(si.k_start + key_c) * a.sdv.s + col0;

  f32x16 dk[C::DB], dv[C::DB];
#pragma unroll
  for (int db = 0; db < C::DB; ++db)
#pragma unroll
    for (int i = 0; i < 16; ++i) { dk[db][i] = 0.f; dv[db][i] = 0.f; }

  if (br.lo <= br.hi) {
    // queries that see this lane's key: one range [q_lo, q_lo + q_rng]
    int q_lo = 0, q_hi = si.seqlen_q - 1;
    if (kWindowed) {
      q_lo = key - w.right > 0 ? key - w.right : 0;
      q_hi = key + w.left < q_hi ? key + w.left : q_hi;
    }
    const bool q_none = !key_ok || q_hi < q_lo;
    const unsigned q_rng = q_none ? 0u : (unsigned)(q_hi - q_lo);

    f32x4 kreg[C::KJ], vreg[C::KJ];
    load_resident<D>(kreg, reinterpret_cast<const float*>(a.k) + (int64_t)si.batch_index * a.sk.z + (int64_t)hk * a.sk.h +
                               (int64_t)(si.k_start + key_c) * a.sk.s, col0, hi, d_qk);
    load_resident<D>(vreg, reinterpret_cast<const float*>(a.v) + (int64_t)si.batch_index * a.sv.z + (int64_t)hk * a.sv.h +
                               (int64_t)(si.k_start + key_c) * a.sv.s, col0, hi, d_v);
    const int group = a.hq / a.hk;
    const int ntq = br.hi - br.lo + 1;
    const int total = group * ntq;
    const float qk_scale = a.sm_scale * kLog2e;

    TileFetch<D, kNT> qf, dof;
    float l_stage = 0.f, d_stage = 0.f;
    // tile `it` of the walk over (q-head of the group, Q tile)
    auto fetch = [&](int it) {
      const int hq = hk * group + it / ntq;
      const int m0 = (br.lo + it % ntq) * kBC;
      const int rows = si.seqlen_q - m0 < kBC ? si.seqlen_q - m0 : kBC;
      qf.load(reinterpret_cast<const float*>(a.q) + (int64_t)si.batch_index * a.sq.z + (int64_t)hq * a.sq.h +
                  (int64_t)(si.q_start + m0) * a.sq.s, rows, a.sq.s, d_qk, tid);
      dof.load(reinterpret_cast<const float*>(a.dout) + (int64_t)si.batch_index * a.sdo.z + (int64_t)hq * a.sdo.h +
                   (int64_t)(si.q_start + m0) * a.sdo.s, rows, a.sdo.s, d_v, tid);
      if (tid < kBC) {
        const bool ok = tid < rows;
        const int64_t lo = lse_offset(si, hq, a.hq) + m0 + tid;
        l_stage = ok ? a.lse[lo] : 0.f;
        d_stage = ok ? a.delta[lo] : 0.f;
      }
    };
    auto publish = [&]() {
      qf.store(Qs, tid);
      dof.store(dOs, tid);
      if (tid < kBC) { Ls[tid] = l_stage * kRcpLn2; Ds[tid] = d_stage; }   // bwd_inner_dk_dv.py:185-186
    };

    fetch(0);
    publish();
    __syncthreads();
    // seed and offset of the dropout mask: read once, not once per tile
    DropoutState drop0{};
    if (kDropout) drop0 = make_dropout_base(a.drop, a.seq.max_seqlen_k);
    for (int it = 0; it < total; ++it) {
      const int hq = hk * group + it / ntq;
      const int e = br.lo + it % ntq;
      const int m0 = e * kBC;
      if (it + 1 < total) fetch(it + 1);
      // this wave's share of S = Q K^T and dP = dO V^T (rows: queries, columns: keys)
      f32x16 s, dp;
#pragma unroll
      for (int i = 0; i < 16; ++i) { s[i] = 0.f; dp[i] = 0.f; }
      s = row_gemm<D>(Qs, c, hi, col0, kreg, s);
      dp = row_gemm<D>(dOs, c, hi, col0, vreg, dp);
      // this wave's quarter of the elements: queries m0 + 8 wave + 4 hi + r
      f32x4 s4, dp4;
      part_write(partS, wave, lane, s);
      if constexpr (C::ONE_PART) {
        __syncthreads();
        s4 = part_sum_quarter(partS, wave, lane);
        __syncthreads();               // S has been read: dP goes through the same area
        part_write(partD, wave, lane, dp);
        __syncthreads();
        dp4 = part_sum_quarter(partD, wave, lane);
      } else {
        part_write(partD, wave, lane, dp);
        __syncthreads();
        s4 = part_sum_quarter(partS, wave, lane);
        dp4 = part_sum_quarter(partD, wave, lane);
      }

      DropoutState dst{};
      if (kDropout) dst = dropout_for_head(drop0, z, hq, a.hq, a.seq.max_seqlen_q);
      const float* bptr = nullptr;
      if (kBias)
        bptr = reinterpret_cast<const float*>(a.bias) + (int64_t)si.batch_index * a.sb_z + (int64_t)hq * a.sb_h +
               (int64_t)key_c * a.sb_n;
      const bool masked = !br.is_full(e);
      const unsigned q_d = q_none ? 0x40000000u : (unsigned)(m0 + 8 * wave + 4 * hi - q_lo);
      const f32x4 l4 = *reinterpret_cast<const f32x4*>(Ls + 8 * wave + 4 * hi);
      const f32x4 d4 = *reinterpret_cast<const f32x4*>(Ds + 8 * wave + 4 * hi);
      f32x4 pd, dsv;      // p as the dV GEMM sees it (dropped and scaled), dS
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int m = m0 + 8 * wave + 4 * hi + r;
        // p = exp2(s c + bias log2e - L log2e) (bwd_inner_dk_dv.py:187-188)
        float x = s4[r] * qk_scale - l4[r];
        if (kBias) {
          const int mm = m < si.seqlen_q ? m : si.seqlen_q - 1;
          x = __builtin_fmaf(bptr[(int64_t)mm * a.sb_m], kLog2e, s4[r] * qk_scale) - l4[r];
        }
        if (masked) {
          const bool vis = q_d + (unsigned)r <= q_rng;
          x = vis ? x : -__builtin_inff();
        }
        const float p = fast_exp2(x);
        float pv = p, dpv = dp4[r];
        if (kDropout) {
          const bool keep = dropout_keep1(dst, m, key);
          pv = keep ? p * dst.scale : 0.f;                       // :200-201
          dpv = keep ? dpv * dst.scale : 0.f;                    // :239-240
        }
        pd[r] = pv;
        dsv[r] = p * (dpv - d4[r]);                              // ds uses the undropped p (:242)
      }
      *reinterpret_cast<f32x4*>(opP + (wave * 64 + lane) * 4) = pd;
      *reinterpret_cast<f32x4*>(opS + (wave * 64 + lane) * 4) = dsv;
      __syncthreads();
      // dV^T += dO^T P and dK^T += Q^T dS on this wave's columns
      col_gemm<D>(dOs, c, hi, col0, opnd_read(opP, lane), dv);
      col_gemm<D>(Qs, c, hi, col0, opnd_read(opS, lane), dk);
      __syncthreads();                 // the tiles, the partial blocks and the operands have been read
      if (it + 1 < total) {
        publish();
        __syncthreads();
      }
    }
  }

  if (key_ok) {
#pragma unroll
    for (int db = 0; db < C::DB; ++db)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        f32x4 k4, v4;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          k4[r] = dk[db][4 * g + r] * a.sm_scale;   // bwd_kernel_dk_dv.py:387-389
          v4[r] = dv[db][4 * g + r];
        }
        if (col0 + 32 * db + 8 * g + 4 * hi < d_qk) *reinterpret_cast<f32x4*>(dkptr + 32 * db + 8 * g + 4 * hi) = k4;
        if (col0 + 32 * db + 8 * g + 4 * hi < d_v) *reinterpret_cast<f32x4*>(dvptr + 32 * db + 8 * g + 4 * hi) = v4;
      }
  }
}

// ---------------------------------------------------------------------------------------------
// dQ and dB: one workgroup = 64 (at 512 columns: 32) query rows of one head, four waves per 32-row block; the lane's
// query is lane % 32 of its row block, the keys of a tile are spread over the accumulator elements
// ---------------------------------------------------------------------------------------------
template <int D>
struct SmemDq {
  static constexpr int PART_OFF = 2 * Cfg<D>::TILE_BYTES;
  static constexpr int OPND_OFF = PART_OFF + Cfg<D>::RB * Cfg<D>::PARTS * kPartBytes;
  static constexpr int BYTES = OPND_OFF + Cfg<D>::RB * kOpndBytes;
};

template <int D, bool kWindowed, bool kBias, bool kDropout>
__global__ __launch_bounds__(Cfg<D>::NT) void bwd_dq_f32_kernel(const BwdArgs a) {
  using C = Cfg<D>;
  using SM = SmemDq<D>;
  extern __shared__ __attribute__((aligned(16))) char smem_raw[];
  float* Ks = reinterpret_cast<float*>(smem_raw);
  float* Vs = reinterpret_cast<float*>(smem_raw + C::TILE_BYTES);

  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int rb = wave / kNW, cw = wave % kNW;             // row block, column share
  const int lane = tid & 63, c = lane & 31, hi = lane >> 5;
  // one workgroup per (sequence, q-head, Q tile): the tiles of a kv-head's group back to back on one
  // XCD, most visible keys (causal) first
  const int nmt = (a.seq.max_seqlen_q + C::BR - 1) / C::BR, group = a.hq / a.hk;
  int pair, r_item;
  if (!xcd_item(blockIdx.x, nseq_of(a.seq, a.batch) * a.hk, group * nmt, pair, r_item)) return;
  const int z = pair / a.hk, h = (pair % a.hk) * group + r_item % group;
  const int mt = nmt - 1 - r_item / group;
  const int d_qk = a.head_dim, d_v = a.head_dim_v;
  const int col0 = cw * C::DW;
  float* partS = reinterpret_cast<float*>(smem_raw + SM::PART_OFF) + rb * C::PARTS * (kPartBytes / 4);
  float* partD = C::ONE_PART ? partS : partS + kPartBytes / 4;
  float* opS = reinterpret_cast<float*>(smem_raw + SM::OPND_OFF) + rb * (kOpndBytes / 4);

  const SeqInfo si = get_seq(a.seq, z);
  const int q0 = mt * C::BR;
  if (q0 >= si.seqlen_q) return;
  const Window w = window_of<kWindowed>(a.mask, si.seqlen_q, si.seqlen_k);
  const BlockRanges br = block_ranges(kWindowed, w.left, w.right, q0, si.seqlen_q, si.seqlen_k, C::BR, kBC);

  const int hk = h / (a.hq / a.hk);
  const int row = q0 + 32 * rb + c;
  const bool row_ok = row < si.seqlen_q;
  const int row_c = row_ok ? row : si.seqlen_q - 1;
  const int nkt = (si.seqlen_k + kBC - 1) / kBC;
  float* dqptr = reinterpret_cast<float*>(a.dq) + (int64_t)si.batch_index * a.sdq.z + (int64_t)h * a.sdq.h +
                 (int64_t)(si.q_start + row_c) * a.sdq.s + col0;
  const bool want_db = kBias && a.db != nullptr;
  float* dbhead = want_db ? reinterpret_cast<float*>(a.db) + (int64_t)si.batch_index * a.sdb_z + (int64_t)h * a.sdb_h
                          : nullptr;

  // dB of K tiles that are never visited is zero: wave w sweeps the rows w, w + 8, ...
  auto zero_db = [&](int j_from, int j_to) {
    if (!want_db) return;
    const int c0 = j_from * kBC, c1 = j_to * kBC < si.seqlen_k ? j_to * kBC : si.seqlen_k;
    if (c0 >= c1) return;
    for (int rr = wave; rr < C::BR; rr += C::RB * kNW) {
      const int m = q0 + rr;
      if (m >= si.seqlen_q) break;
      float* rowp = dbhead + (int64_t)m * a.sdb_m;
      for (int n = c0 + lane; n < c1; n += 64) rowp[(int64_t)n * a.sdb_n] = 0.f;
    }
  };

  f32x16 dq[C::DB];
#pragma unroll
  for (int db = 0; db < C::DB; ++db)
#pragma unroll
    for (int i = 0; i < 16; ++i) dq[db][i] = 0.f;

  if (br.lo > br.hi) {
    zero_db(0, nkt);
  } else {
    // visible keys of this lane's query: one range [m_lo, m_lo + m_rng]
    int m_lo = 0, m_hi = si.seqlen_k - 1;
    if (kWindowed) {
      m_lo = row - w.left > 0 ? row - w.left : 0;
      m_hi = row + w.right < m_hi ? row + w.right : m_hi;
    }
    const bool m_none = m_hi < m_lo;
    const unsigned m_rng = m_none ? 0u : (unsigned)(m_hi - m_lo);

    f32x4 qreg[C::KJ], doreg[C::KJ];
    load_resident<D>(qreg, reinterpret_cast<const float*>(a.q) + (int64_t)si.batch_index * a.sq.z + (int64_t)h * a.sq.h +
                               (int64_t)(si.q_start + row_c) * a.sq.s, col0, hi, d_qk);
    load_resident<D>(doreg, reinterpret_cast<const float*>(a.dout) + (int64_t)si.batch_index * a.sdo.z +
                                (int64_t)h * a.sdo.h + (int64_t)(si.q_start + row_c) * a.sdo.s, col0, hi, d_v);
    const int64_t lo = lse_offset(si, h, a.hq) + row_c;
    const float l_row = a.lse[lo] * kRcpLn2;               // bwd_kernel_dq.py:305
    const float d_row = a.delta[lo];
    const float qk_scale = a.sm_scale * kLog2e;
    const float* bptr = nullptr;
    if (kBias)
      bptr = reinterpret_cast<const float*>(a.bias) + (int64_t)si.batch_index * a.sb_z + (int64_t)h * a.sb_h +
             (int64_t)row_c * a.sb_m;
    float* dbptr = want_db ? dbhead + (int64_t)row_c * a.sdb_m : nullptr;
    DropoutState dst{};
    if (kDropout) dst = make_dropout(a.drop, z, h, a.hq, a.seq.max_seqlen_q, a.seq.max_seqlen_k);

    const float* kt = reinterpret_cast<const float*>(a.k) + (int64_t)si.batch_index * a.sk.z + (int64_t)hk * a.sk.h +
                      (int64_t)(si.k_start + br.lo * kBC) * a.sk.s;
    const float* vt = reinterpret_cast<const float*>(a.v) + (int64_t)si.batch_index * a.sv.z + (int64_t)hk * a.sv.h +
                      (int64_t)(si.k_start + br.lo * kBC) * a.sv.s;
    int rows_left = si.seqlen_k - br.lo * kBC;      // > 0
    TileFetch<D, C::NT> kf, vf;
    auto fetch = [&]() {
      const int rows = rows_left < kBC ? rows_left : kBC;
      kf.load(kt, rows, a.sk.s, d_qk, tid);
      vf.load(vt, rows, a.sv.s, d_v, tid);
      kt += (int64_t)kBC * a.sk.s; vt += (int64_t)kBC * a.sv.s; rows_left -= kBC;
    };
    auto publish = [&]() { kf.store(Ks, tid); vf.store(Vs, tid); };

    fetch();
    publish();
    __syncthreads();
    for (int j = br.lo; j <= br.hi; ++j) {
      if (j < br.hi) fetch();
      // this wave's share of S^T = K Q^T and dP^T = V dO^T (rows: keys, columns: queries)
      f32x16 s, dp;
#pragma unroll
      for (int i = 0; i < 16; ++i) { s[i] = 0.f; dp[i] = 0.f; }
      s = row_gemm<D>(Ks, c, hi, col0, qreg, s);
      dp = row_gemm<D>(Vs, c, hi, col0, doreg, dp);
      // this wave's quarter of its row block's elements: keys j kBC + 8 cw + 4 hi + r
      f32x4 s4, dp4;
      part_write(partS, cw, lane, s);
      if constexpr (C::ONE_PART) {
        __syncthreads();
        s4 = part_sum_quarter(partS, cw, lane);
        __syncthreads();               // S has been read: dP goes through the same area
        part_write(partD, cw, lane, dp);
        __syncthreads();
        dp4 = part_sum_quarter(partD, cw, lane);
      } else {
        part_write(partD, cw, lane, dp);
        __syncthreads();
        s4 = part_sum_quarter(partS, cw, lane);
        dp4 = part_sum_quarter(partD, cw, lane);
      }

      const bool masked = !br.is_full(j);
      const unsigned m_d = m_none ? 0x40000000u : (unsigned)(j * kBC + 8 * cw + 4 * hi - m_lo);
      uint32_t keep = 0xfu;
      if (kDropout) keep = dropout_keep4(dst, row, j * kBC + 8 * cw + 4 * hi);
      f32x4 dsv4;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int n = j * kBC + 8 * cw + 4 * hi + r;
        float x = s4[r] * qk_scale - l_row;
        if (kBias) {
          const int nn = n < si.seqlen_k ? n : si.seqlen_k - 1;
          x = __builtin_fmaf(bptr[(int64_t)nn * a.sb_n], kLog2e, s4[r] * qk_scale) - l_row;
        }
        if (masked) {
          const bool vis = m_d + (unsigned)r <= m_rng;
          x = vis ? x : -__builtin_inff();
        }
        const float p = fast_exp2(x);
        float dpv = dp4[r];
        if (kDropout) dpv = ((keep >> r) & 1u) ? dpv * dst.scale : 0.f;   // bwd_inner_dq.py:176-185
        const float dsv = p * (dpv - d_row);
        dsv4[r] = dsv;
        if (want_db && row_ok && n < si.seqlen_k) dbptr[(int64_t)n * a.sdb_n] = dsv;   // :200-204
      }
      *reinterpret_cast<f32x4*>(opS + (cw * 64 + lane) * 4) = dsv4;
      __syncthreads();
      // dQ^T += K^T dS^T on this wave's columns
      col_gemm<D>(Ks, c, hi, col0, opnd_read(opS, lane), dq);
      __syncthreads();                 // the tiles, the partial blocks and the operands have been read
      if (j < br.hi) {
        publish();
        __syncthreads();
      }
    }
    zero_db(0, br.lo);
    zero_db(br.hi + 1, nkt);
  }

  if (row_ok) {
#pragma unroll
    for (int db = 0; db < C::DB; ++db)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        f32x4 t4;
#pragma unroll
        for (int r = 0; r < 4; ++r) t4[r] = dq[db][4 * g + r] * a.sm_scale;   // bwd_kernel_dq.py:374-376
        if (col0 + 32 * db + 8 * g + 4 * hi < d_qk) *reinterpret_cast<f32x4*>(dqptr + 32 * db + 8 * g + 4 * hi) = t4;
      }
  }
}

template <auto kern, int NT, typename Args>
hipError_t launch(dim3 grid, int smem, hipStream_t stream, const Args& a) {
  if (grid.x == 0 || grid.y == 0 || grid.z == 0) return hipSuccess;   // an empty tensor: nothing to write
  if (smem > 64 * 1024) {
    static std::atomic<uint64_t> lds_set{0};
    hipError_t e = allow_large_lds(reinterpret_cast<const void*>(kern), smem, lds_set);
    if (e != hipSuccess) return e;
  }
  hipLaunchKernelGGL(kern, grid, dim3(NT), smem, stream, a);
  return hipGetLastError();
}

#define FA_F32_SWITCH(CALL)                                            \
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

template <int D>
hipError_t run_fwd_d(const FwdArgs& a, bool windowed, bool bias, bool dropout, hipStream_t s) {
  const dim3 grid(xcd_grid(nseq_of(a.seq, a.batch) * a.hk, (a.hq / a.hk) * ((a.seq.max_seqlen_q + Cfg<D>::BR - 1) / Cfg<D>::BR)));
#define FA_CALL(W, B, P) launch<fwd_f32_kernel<D, W, B, P>, Cfg<D>::NT>(grid, SmemFwd<D>::BYTES, s, a)
  FA_F32_SWITCH(FA_CALL)
#undef FA_CALL
}

template <int D>
hipError_t run_bwd_d(int kernel_slot, const BwdArgs& a, bool windowed, bool bias, bool dropout, hipStream_t s) {
  const int nseq = nseq_of(a.seq, a.batch);
  if (kernel_slot == 1) {
    const dim3 grid(xcd_grid(nseq * a.hk, (a.seq.max_seqlen_k + kBC - 1) / kBC));
#define FA_CALL(W, B, P) launch<bwd_dkdv_f32_kernel<D, W, B, P>, kNT>(grid, SmemDkDv<D>::BYTES, s, a)
    FA_F32_SWITCH(FA_CALL)
#undef FA_CALL
  }
  if (kernel_slot == 2) {
    const dim3 grid(xcd_grid(nseq * a.hk, (a.hq / a.hk) * ((a.seq.max_seqlen_q + Cfg<D>::BR - 1) / Cfg<D>::BR)));
#define FA_CALL(W, B, P) launch<bwd_dq_f32_kernel<D, W, B, P>, Cfg<D>::NT>(grid, SmemDq<D>::BYTES, s, a)
    FA_F32_SWITCH(FA_CALL)
#undef FA_CALL
  }
  return hipErrorInvalidValue;
}

}  // namespace

// head_dim: the compiled one that holds the tensors' head dims (64 runs on the 128-column kernels)
hipError_t run_fwd_f32(int head_dim, const FwdArgs& a, bool windowed, bool bias, bool dropout, hipStream_t s) {
  if (head_dim <= 128) return run_fwd_d<128>(a, windowed, bias, dropout, s);
  if (head_dim == 256) return run_fwd_d<256>(a, windowed, bias, dropout, s);
  if (head_dim == 512) return run_fwd_d<512>(a, windowed, bias, dropout, s);
  return hipErrorNotSupported;
}

hipError_t run_bwd_f32(int head_dim, int kernel_slot, const BwdArgs& a, bool windowed, bool bias, bool dropout,
                       hipStream_t s) {
  if (head_dim <= 128) return run_bwd_d<128>(kernel_slot, a, windowed, bias, dropout, s);
  if (head_dim == 256) return run_bwd_d<256>(kernel_slot, a, windowed, bias, dropout, s);
  if (head_dim == 512) return run_bwd_d<512>(kernel_slot, a, windowed, bias, dropout, s);
  return hipErrorNotSupported;
}

template <int D>
static TileShape tile_shape_d(int kernel_slot) {
  // forward (kernel_slot < 0) and dQ: the workgroup's queries against 32 keys per step; dK/dV: 32
  // keys per workgroup against 32 queries per step
  if (kernel_slot < 0) return TileShape{Cfg<D>::BR, kBC, Cfg<D>::RB * kNW, SmemFwd<D>::BYTES};
  if (kernel_slot == 2) return TileShape{Cfg<D>::BR, kBC, Cfg<D>::RB * kNW, SmemDq<D>::BYTES};
  return TileShape{kBC, kBC, kNW, SmemDkDv<D>::BYTES};
}

TileShape f32_tile_shape(int head_dim, int kernel_slot) {
  return head_dim <= 128 ? tile_shape_d<128>(kernel_slot)
         : head_dim <= 256 ? tile_shape_d<256>(kernel_slot) : tile_shape_d<512>(kernel_slot);
}

}  // namespace fa
