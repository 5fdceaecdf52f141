// MFMA kernels for head dims above 256 (up to 512) of the 16-bit types, gfx950.
//
// The reference compiles its kernels for head dim 512 as well (modules/flash/aot/_common.py:10-14);
// these compute what the other MFMA kernels of this library do
//   forward   modules/flash/kernel/fwd_kernel.py:83-644, fwd_kernel_inner.py:46-287
//   dK, dV    modules/flash/kernel/bwd_kernel_dk_dv.py:48-417, bwd_inner_dk_dv.py:28-267
//   dQ, dB    modules/flash/kernel/bwd_kernel_dq.py:45-389, bwd_inner_dq.py:28-215
// for tensors whose head dims are rounded up to 512.
//
// At 512 columns a wave cannot hold a 32-row block of O (or of dK and dV) next to its operands, so
// the head dim is split over the four waves of a workgroup: all four work on the SAME 32 rows and
// wave w owns columns [128 w, 128 w + 128).  A GEMM that contracts over the head dim (S = Q K^T,
// dP = dO V^T) is a sum of four partial products, one per wave: each wave writes its 32 x 32 fp32
// partial block to LDS and, behind a barrier, every wave adds the four in the same order, so all
// of them hold the same S bit for bit and run the same softmax.  The GEMMs whose result has the
// head dim as an outer index (O += P V, dV += P^T dO, dK += dS^T Q, dQ += dS K) need no exchange:
// a wave computes its 128 columns.  No MFMA is executed twice; the price is 4 KB written and 16 KB
// read of LDS per wave and partial block, and two barriers per step.
//
// Register layouts, the transposing LDS reads and the base-2 softmax are those of the kernels for
// the smaller head dims (fa_device.h, fa_fwd_impl.h).
#include "fa_device.h"
#include "fa_kernels.h"

namespace fa {
namespace {

constexpr int kD = 512;          // compiled head dim
constexpr int kNW = 4;           // waves per workgroup
constexpr int kDW = kD / kNW;    // columns of the head dim a wave owns
constexpr int kKS = kDW / 16;    // k-steps of a wave's share of a contraction over the head dim
constexpr int kDB = kDW / 32;    // 32-column blocks a wave owns
constexpr int kBR = 32;          // rows (queries or keys) per workgroup
constexpr int kBC = 32;          // rows of the streamed tiles per step
constexpr int kNT = kNW * 64;

// padded tiles of the forward: one read by rows (+16 B per row), one read transposed (+64 B per row)
struct Smem512 {
  static constexpr int ASTR = kD + 8;
  static constexpr int BSTR = kD + 32;
  static constexpr int A_ELEMS = kBC * ASTR;
  static constexpr int B_ELEMS = kBC * BSTR;
  static constexpr int PART_BYTES = kNW * 64 * 16 * 4;       // one partial block per wave
};

// The waves' partial 32 x 32 blocks (the MFMA result layout, 16 values per lane) summed in wave
// order.  `slot` selects one of the areas; the caller places the barriers.
__device__ __forceinline__ void part_write(float* area, int wave, int lane, const f32x16& x) {
#pragma unroll
  for (int g = 0; g < 4; ++g) {
    const f32x4 t = {x[4 * g], x[4 * g + 1], x[4 * g + 2], x[4 * g + 3]};
    *reinterpret_cast<f32x4*>(area + ((wave * 4 + g) * 64 + lane) * 4) = t;
  }
}
__device__ __forceinline__ f32x16 part_sum(const float* area, int lane) {
  f32x16 x;
#pragma unroll
  for (int g = 0; g < 4; ++g) {
    f32x4 acc = *reinterpret_cast<const f32x4*>(area + (g * 64 + lane) * 4);
#pragma unroll
    for (int w = 1; w < kNW; ++w) {
      const f32x4 t = *reinterpret_cast<const f32x4*>(area + ((w * 4 + g) * 64 + lane) * 4);
#pragma unroll
      for (int r = 0; r < 4; ++r) acc[r] += t[r];
    }
#pragma unroll
    for (int r = 0; r < 4; ++r) x[4 * g + r] = acc[r];
  }
  return x;
}

// The same sum with the wave's own block taken from its registers instead of from LDS (the values
// are the ones it wrote, the order of the additions is unchanged, so the result is the same bit for
// bit in all four waves): a quarter less to read.
template <int W>
__device__ __forceinline__ f32x16 part_sum_own_w(const float* area, int lane, const f32x16& own) {
  f32x16 x;
#pragma unroll
  for (int g = 0; g < 4; ++g) {
    f32x4 acc;
#pragma unroll
    for (int w = 0; w < kNW; ++w) {
      f32x4 t;
      if (w == W) t = f32x4{own[4 * g], own[4 * g + 1], own[4 * g + 2], own[4 * g + 3]};
      else t = *reinterpret_cast<const f32x4*>(area + ((w * 4 + g) * 64 + lane) * 4);
      if (w == 0) acc = t;
      else {
#pragma unroll
        for (int r = 0; r < 4; ++r) acc[r] += t[r];
      }
    }
#pragma unroll
    for (int r = 0; r < 4; ++r) x[4 * g + r] = acc[r];
  }
  return x;
}
__device__ __forceinline__ f32x16 part_sum_own(const float* area, int wave, int lane, const f32x16& own) {
  switch (wave) {      // (the wave index is a scalar)
    case 0: return part_sum_own_w<0>(area, lane, own);
    case 1: return part_sum_own_w<1>(area, lane, own);
    case 2: return part_sum_own_w<2>(area, lane, own);
    default: return part_sum_own_w<3>(area, lane, own);
  }
}

// Backward: the element work on a summed block needs no row reduction, so it is split as well:
// wave g adds only elements 4 g .. 4 g + 3 of every lane (a quarter of each partial block), does the
// exponentials, mask, dropout and dS for those, and hands the two results to all waves as 16-bit
// MFMA operand pieces (8 bytes per lane and quarter); slots 2 t and 2 t + 1 form the operand of
// k-step t.
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
template <typename T>
__device__ __forceinline__ void opnd_write(char* area, int g, int lane, const f32x4& x) {
  typename Traits<T>::q4_t q;
#pragma unroll
  for (int r = 0; r < 4; ++r) q[r] = Traits<T>::cvt(x[r]);
  *reinterpret_cast<typename Traits<T>::q4_t*>(area + (g * 64 + lane) * 8) = q;
}
template <typename T>
__device__ __forceinline__ typename Traits<T>::op_t opnd_read(const char* area, int t, int lane) {
  const auto lo = *reinterpret_cast<const typename Traits<T>::q4_t*>(area + ((2 * t) * 64 + lane) * 8);
  const auto hi = *reinterpret_cast<const typename Traits<T>::q4_t*>(area + ((2 * t + 1) * 64 + lane) * 8);
  return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
}
constexpr int kOpndBytes = 4 * 64 * 8;     // one operand block: 4 quarters x 64 lanes x 8 bytes

// A tile of kBC rows x 512 columns, global -> registers -> LDS by the whole workgroup of NT threads:
// a wave instruction covers one row (64 pieces of 16 bytes), a thread holds its pieces NT / 64
// rows apart.  The buffer descriptor bounds the tile to its valid rows and columns; what lies
// outside reads as zero.
template <typename T, int NT = kNT>
struct TileFetch {
  using op_t = typename Traits<T>::op_t;
  static constexpr int CH = kBC * (kD / 8) / NT;
  static constexpr int RPI = NT / (kD / 8);
  op_t reg[CH];
  __device__ __forceinline__ void load(const T* tile, int rows, int64_t row_stride, int cols, int tid) {
    const int r0 = tid >> 6, cc0 = tid & 63;
    const auto rs = wave_rsrc(tile, rows > 0 ? ((rows - 1) * (int)row_stride + cols) * 2 : 0);
    const int voff = cc0 * 8 < cols ? r0 * (int)row_stride * 2 + cc0 * 16 : kVoffOutOfRange;
#pragma unroll
    for (int i = 0; i < CH; ++i)
      reg[i] = __builtin_bit_cast(op_t, __builtin_amdgcn_raw_buffer_load_b128(rs, voff, i * RPI * (int)row_stride * 2, 0));
  }
  __device__ __forceinline__ void store(T* lds, int stride, int tid) const {
    const int r0 = tid >> 6, cc0 = tid & 63;
#pragma unroll
    for (int i = 0; i < CH; ++i) *reinterpret_cast<op_t*>(lds + (r0 + i * RPI) * stride + cc0 * 8) = reg[i];
  }
};

// ---------------------------------------------------------------------------------------------
// forward: one workgroup = 64 query rows of one head = 8 waves, four per 32-row block
// ---------------------------------------------------------------------------------------------
// A K/V tile of 32 keys is 64 KB; with 32 rows per workgroup that is 32 FLOP per byte streamed and
// the kernel runs at the rate the L2 delivers K/V (about 225 TFLOP/s).  Two row blocks share the
// tile here; each has its own four waves (one per 128 columns), so a SIMD holds two waves and one
// covers the other's waits.  Two K stages and one V stage in LDS, the next tile waits in registers:
// K of the next tile is published behind the PV MFMAs (its stage was last read a tile ago), V behind
// the barrier that ends the tile, where it becomes visible with the next tile's partial blocks; two
// barriers per tile.
constexpr int kFRB = 2;              // 32-row blocks per workgroup
constexpr int kFBR = 32 * kFRB;      // query rows per workgroup
constexpr int kFNT = kFRB * kNT;     // threads per workgroup
struct SmemFwd512 {
  static constexpr int ASTR = Smem512::ASTR, BSTR = Smem512::BSTR;
  static constexpr int K_STAGE = Smem512::A_ELEMS * 2;       // bytes of one K stage; there are two
  static constexpr int V_OFF = 2 * K_STAGE;
  static constexpr int PART_OFF = V_OFF + Smem512::B_ELEMS * 2;
  static constexpr int BYTES = PART_OFF + kFRB * Smem512::PART_BYTES;
};

template <typename T, bool kWindowed, bool kBias, bool kDropout>
__global__ __launch_bounds__(kFNT) void fwd_d512_kernel(const FwdArgs a) {
  using Tr = Traits<T>;
  using op_t = typename Tr::op_t;
  using q4_t = typename Tr::q4_t;
  using SM = SmemFwd512;
  extern __shared__ __attribute__((aligned(16))) char smem_raw[];
  T* Ks = reinterpret_cast<T*>(smem_raw);
  T* Vs = reinterpret_cast<T*>(smem_raw + SM::V_OFF);

  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int rb = wave / kNW, cw = wave % kNW;             // row block, column share
  const int lane = tid & 63, c = lane & 31, hi = lane >> 5;
  // one workgroup per (sequence, q-head, Q tile): the tiles of a kv-head's group back to back on one
  // XCD, most visible keys (causal) first
  const int nmt = (a.seq.max_seqlen_q + kFBR - 1) / kFBR, group = a.hq / a.hk;
  int pair, r_item;
  if (!xcd_item(blockIdx.x, nseq_of(a.seq, a.batch) * a.hk, group * nmt, pair, r_item)) return;
  const int z = pair / a.hk, h = (pair % a.hk) * group + r_item % group;
  const int mt = nmt - 1 - r_item / group;
  const int d_qk = a.head_dim, d_v = a.head_dim_v;
  float* part = reinterpret_cast<float*>(smem_raw + SM::PART_OFF) + rb * (Smem512::PART_BYTES / 4);
  if (kDropout && blockIdx.x == 0 && tid == 0) {
    // modules/flash/kernel/fwd_kernel.py:199-207
    uint64_t base = a.drop.offset2;
    if (a.drop.offset1_ptr) base += *a.drop.offset1_ptr;
    if (a.seed_out) *a.seed_out = *a.drop.seed_ptr;
    if (a.offset_out) *a.offset_out = base;
  }

  const SeqInfo si = get_seq(a.seq, z);
  const int q0 = mt * kFBR;
  if (q0 >= si.seqlen_q) return;

  Window w{0, 0};
  if (kWindowed) w = parse_window(a.mask.causal_type, a.mask.window_left, a.mask.window_right,
                                  si.seqlen_q, si.seqlen_k);
  w.left = w.left > (1 << 30) ? (1 << 30) : (w.left < -(1 << 30) ? -(1 << 30) : w.left);
  w.right = w.right > (1 << 30) ? (1 << 30) : (w.right < -(1 << 30) ? -(1 << 30) : w.right);
  const BlockRanges br = block_ranges(kWindowed, w.left, w.right, q0, si.seqlen_q, si.seqlen_k, kFBR, kBC);

  const int hk = h / (a.hq / a.hk);                       // fwd_kernel.py:360
  const int row = q0 + 32 * rb + c;                       // this lane's query row (the same in the four waves of a row block)
  const bool row_ok = row < si.seqlen_q;
  const int row_c = row_ok ? row : si.seqlen_q - 1;
  const int col0 = cw * kDW;                              // first column of this wave's share

  T* optr = reinterpret_cast<T*>(a.out) + (int64_t)si.batch_index * a.so.z + (int64_t)h * a.so.h +
            (int64_t)(si.q_start + row_c) * a.so.s + col0;
  float* lse_ptr = a.lse ? a.lse + lse_offset(si, h, a.hq) : nullptr;

  if (br.lo > br.hi) {
    // no visible key for any row of this tile: O = 0, LSE = +inf (fwd_kernel.py:327-355)
    if (row_ok) {
      const q4_t zero4 = {0, 0, 0, 0};
#pragma unroll
      for (int db = 0; db < kDB; ++db)
#pragma unroll
        for (int g = 0; g < 4; ++g)
          if (col0 + 32 * db + 8 * g + 4 * hi < d_v) *reinterpret_cast<q4_t*>(optr + 32 * db + 8 * g + 4 * hi) = zero4;
      if (lse_ptr && cw == 0 && hi == 0) lse_ptr[row] = __builtin_inff();
    }
    return;
  }

  // the wave's columns of the Q rows as B operands, resident for the whole tile
  op_t qreg[kKS];
  {
    const T* qptr = reinterpret_cast<const T*>(a.q) + (int64_t)si.batch_index * a.sq.z + (int64_t)h * a.sq.h +
                    (int64_t)(si.q_start + row_c) * a.sq.s + col0;
    const op_t zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
    for (int ks = 0; ks < kKS; ++ks)
      qreg[ks] = col0 + 16 * ks + 8 * hi < d_qk ? *reinterpret_cast<const op_t*>(qptr + 16 * ks + 8 * hi) : zero8;
  }

  const T* kt = reinterpret_cast<const T*>(a.k) + (int64_t)si.batch_index * a.sk.z + (int64_t)hk * a.sk.h +
                (int64_t)(si.k_start + br.lo * kBC) * a.sk.s;
  const T* vt = reinterpret_cast<const T*>(a.v) + (int64_t)si.batch_index * a.sv.z + (int64_t)hk * a.sv.h +
                (int64_t)(si.k_start + br.lo * kBC) * a.sv.s;
  int rows_left = si.seqlen_k - br.lo * kBC;      // > 0
  TileFetch<T, kFNT> kf, vf;
  auto fetch = [&]() {
    const int rows = rows_left < kBC ? rows_left : kBC;
    kf.load(kt, rows, a.sk.s, d_qk, tid);
    vf.load(vt, rows, a.sv.s, d_v, tid);
    kt += (int64_t)kBC * a.sk.s; vt += (int64_t)kBC * a.sv.s; rows_left -= kBC;
  };
  auto publish_k = [&](int stage) { kf.store(Ks + stage * Smem512::A_ELEMS, SM::ASTR, tid); };
  auto publish_v = [&]() { vf.store(Vs, SM::BSTR, tid); };

  const T* bptr = nullptr;
  if (kBias)
    bptr = reinterpret_cast<const T*>(a.bias) + (int64_t)si.batch_index * a.sb_z + (int64_t)h * a.sb_h +
           (int64_t)row_c * a.sb_m;
  DropoutState ds{};
  if (kDropout) ds = make_dropout(a.drop, z, h, a.hq, a.seq.max_seqlen_q, a.seq.max_seqlen_k);

  f32x16 o[kDB];
#pragma unroll
  for (int db = 0; db < kDB; ++db)
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
  // lane-constant part of the V^T operand address (see lds_read_tr8)
  const int v_lane = (4 * hi + (lane & 15) / 4) * SM::BSTR + 16 * ((lane >> 4) & 1) + 4 * (lane & 3) + col0;

  fetch();
  publish_k(0);
  publish_v();
  __syncthreads();
  for (int j = br.lo; j <= br.hi; ++j) {
    const int stage = (j - br.lo) & 1;
    // this wave's share of S^T = K Q^T
    f32x16 s;
#pragma unroll
    for (int i = 0; i < 16; ++i) s[i] = 0.f;
    const T* ks = Ks + stage * Smem512::A_ELEMS + c * SM::ASTR + col0 + hi * 8;
#pragma unroll
    for (int k = 0; k < kKS; ++k) s = Tr::mfma(*reinterpret_cast<const op_t*>(ks + k * 16), qreg[k], s);
    // behind the MFMAs: V of this tile goes to its stage (read behind the next barrier), then the
    // staging registers take the next tile
    if (j > br.lo) publish_v();
    if (j < br.hi) fetch();
    part_write(part, cw, lane, s);
    __syncthreads();
    s = part_sum_own(part, cw, lane, s);

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
        s[i] += (float)bptr[(int64_t)n * a.sb_n] * kLog2e;   // fwd_kernel_inner.py:187
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
      rs += s[i];                       // the row sum is over the fp32, undropped p (:213-214)
    }
    l_i = l_i * alpha + rs;
    if (__builtin_amdgcn_ballot_w64(alpha != 1.0f) != 0) {   // some row of the wave moved its maximum
#pragma unroll
      for (int db = 0; db < kDB; ++db)
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
    // O^T += V^T P^T on this wave's columns; P is cast to V's type (:274)
    const T* vs = Vs + v_lane;
#pragma unroll
    for (int t = 0; t < kBC / 16; ++t) {
      const op_t pb = pack8<T>(s, t);
#pragma unroll
      for (int db = 0; db < kDB; ++db)
        o[db] = Tr::mfma(lds_read_tr8<T>(vs + t * 16 * SM::BSTR + db * 32, SM::BSTR), pb, o[db]);
    }
    if (j < br.hi) publish_k(stage ^ 1);
    __syncthreads();                 // V and the partial blocks have been read, the next K is in place
  }

  const float l = cross_sum(l_i);
  const bool alive = l > 0.f;
  float inv = alive ? 1.0f / l : 0.f;
  if (kDropout) inv *= ds.scale;          // fwd_kernel.py:573-575
  if (row_ok) {
#pragma unroll
    for (int db = 0; db < kDB; ++db)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        q4_t t4;
#pragma unroll
        for (int r = 0; r < 4; ++r) t4[r] = Tr::cvt(o[db][4 * g + r] * inv);
        if (col0 + 32 * db + 8 * g + 4 * hi < d_v) *reinterpret_cast<q4_t*>(optr + 32 * db + 8 * g + 4 * hi) = t4;
      }
    if (lse_ptr && cw == 0 && hi == 0)
      lse_ptr[row] = alive ? (m_i * sc + fast_log2(l)) * kLn2 : __builtin_inff();   // fwd_kernel.py:610-612
  }
}

// ---------------------------------------------------------------------------------------------
// backward
// ---------------------------------------------------------------------------------------------
// One stage of two streamed tiles (32 rows x 512 columns each, stored once with the swizzle of
// fa_device.h: both the row reads of the GEMMs that contract over the head dim and the transposing
// reads of the GEMMs that contract over the tile's rows are free of bank conflicts), the row
// statistics of the tile's queries, and two areas of partial blocks (S and dP).  The next tile
// waits in registers while the current one is worked on.
struct SmemBwd512 {
  static constexpr int TILE_BYTES = kBC * kD * 2;
  static constexpr int STAT_OFF = 2 * TILE_BYTES;
  static constexpr int PART_OFF = STAT_OFF + 2 * kBC * 4;
  static constexpr int OPND_OFF = PART_OFF + 2 * Smem512::PART_BYTES;     // P and dS operand pieces
  static constexpr int BYTES = OPND_OFF + 2 * kOpndBytes;
};

template <typename T, int NT = kNT>
__device__ __forceinline__ void store_swizzled(const TileFetch<T, NT>& f, char* tile, int tid) {
  const int r0 = tid >> 6, cc0 = tid & 63;
#pragma unroll
  for (int i = 0; i < TileFetch<T, NT>::CH; ++i)
    *reinterpret_cast<typename Traits<T>::op_t*>(tile + Swz<kD>::addr(r0 + i * TileFetch<T, NT>::RPI, cc0)) = f.reg[i];
}

// dK, dV: one workgroup = 32 keys of one kv-head; the lane's key is lane % 32 in every wave, the
// queries of a tile are spread over the accumulator elements.
template <typename T, bool kWindowed, bool kBias, bool kDropout>
__global__ __launch_bounds__(kNT) void bwd_dkdv_d512_kernel(const BwdArgs a) {
  using Tr = Traits<T>;
  using op_t = typename Tr::op_t;
  using q4_t = typename Tr::q4_t;
  using SM = SmemBwd512;
  extern __shared__ __attribute__((aligned(16))) char smem_raw[];
  char* Qb = smem_raw;
  char* dOb = smem_raw + SM::TILE_BYTES;
  float* Ls = reinterpret_cast<float*>(smem_raw + SM::STAT_OFF);
  float* Ds = Ls + kBC;
  float* partS = reinterpret_cast<float*>(smem_raw + SM::PART_OFF);
  float* partD = partS + Smem512::PART_BYTES / 4;
  char* opP = smem_raw + SM::OPND_OFF;
  char* opS = opP + kOpndBytes;

  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lane = tid & 63, c = lane & 31, hi = lane >> 5;
  // one workgroup per (sequence, kv-head, key block): the key blocks of a kv-head back to back on
  // one XCD, those that the most queries see (causal) first
  int pair, nt;
  if (!xcd_item(blockIdx.x, nseq_of(a.seq, a.batch) * a.hk, (a.seq.max_seqlen_k + kBR - 1) / kBR, pair, nt)) return;
  const int z = pair / a.hk, hk = pair % a.hk;
  const int d_qk = a.head_dim, d_v = a.head_dim_v;
  const int col0 = wave * kDW;

  const SeqInfo si = get_seq(a.seq, z);
  const int n0 = nt * kBR;
  if (n0 >= si.seqlen_k) return;

  Window w{0, 0};
  if (kWindowed) w = parse_window(a.mask.causal_type, a.mask.window_left, a.mask.window_right,
                                  si.seqlen_q, si.seqlen_k);
  w.left = w.left > (1 << 30) ? (1 << 30) : (w.left < -(1 << 30) ? -(1 << 30) : w.left);
  w.right = w.right > (1 << 30) ? (1 << 30) : (w.right < -(1 << 30) ? -(1 << 30) : w.right);
  // rows are keys here, columns are queries: key n sees query m iff n - right <= m <= n + left
  // (bwd_kernel_dk_dv.py:268-279 passes the window transposed in the same way)
  const BlockRanges br = block_ranges(kWindowed, w.right, w.left, n0, si.seqlen_k, si.seqlen_q, kBR, kBC);

  const int key = n0 + c;
  const bool key_ok = key < si.seqlen_k;
  const int key_c = key_ok ? key : si.seqlen_k - 1;
  T* dkptr = reinterpret_cast<T*>(a.dk) + (int64_t)si.batch_index * a.sdk.z + (int64_t)hk * a.sdk.h +
             (int64_t)(si.k_start + key_c) * a.sdk.s + col0;
  T* dvptr = reinterpret_cast<T*>(a.dv) + (int64_t)si.batch_index * a.sdv.z + (int64_t)hk * a.sdv.h +
             (int64_t)(si.k_start + key_c) * a.sdv.s + col0;

  f32x16 dk[kDB], dv[kDB];
#pragma unroll
  for (int db = 0; db < kDB; ++db)
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

    // the wave's columns of this lane's K and V rows as B operands
    op_t kreg[kKS], vreg[kKS];
    {
      const T* kptr = reinterpret_cast<const T*>(a.k) + (int64_t)si.batch_index * a.sk.z + (int64_t)hk * a.sk.h +
                      (int64_t)(si.k_start + key_c) * a.sk.s + col0;
      const T* vptr = reinterpret_cast<const T*>(a.v) + (int64_t)si.batch_index * a.sv.z + (int64_t)hk * a.sv.h +
                      (int64_t)(si.k_start + key_c) * a.sv.s + col0;
      const op_t zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
      for (int k = 0; k < kKS; ++k) {
        kreg[k] = col0 + 16 * k + 8 * hi < d_qk ? *reinterpret_cast<const op_t*>(kptr + 16 * k + 8 * hi) : zero8;
        vreg[k] = col0 + 16 * k + 8 * hi < d_v ? *reinterpret_cast<const op_t*>(vptr + 16 * k + 8 * hi) : zero8;
      }
    }
    const int group = a.hq / a.hk;
    const int ntq = br.hi - br.lo + 1;
    const int total = group * ntq;
    const float qk_scale = a.sm_scale * kLog2e;
    const int row_a = Swz<kD>::row_base(lane), tr_a0 = Swz<kD>::tr_base(lane, 0), tr_a1 = Swz<kD>::tr_base(lane, 1);

    TileFetch<T> qf, dof;
    float l_stage = 0.f, d_stage = 0.f;
    // tile `it` of the walk over (q-head of the group, Q tile)
    auto fetch = [&](int it) {
      const int hq = hk * group + it / ntq;
      const int m0 = (br.lo + it % ntq) * kBC;
      const int rows = si.seqlen_q - m0 < kBC ? si.seqlen_q - m0 : kBC;
      const T* qt = reinterpret_cast<const T*>(a.q) + (int64_t)si.batch_index * a.sq.z + (int64_t)hq * a.sq.h +
                    (int64_t)(si.q_start + m0) * a.sq.s;
      const T* dot = reinterpret_cast<const T*>(a.dout) + (int64_t)si.batch_index * a.sdo.z + (int64_t)hq * a.sdo.h +
                     (int64_t)(si.q_start + m0) * a.sdo.s;
      qf.load(qt, rows, a.sq.s, d_qk, tid);
      dof.load(dot, rows, a.sdo.s, d_v, tid);
      if (tid < kBC) {
        const bool ok = tid < rows;
        const int64_t lo = lse_offset(si, hq, a.hq) + m0 + tid;
        l_stage = ok ? a.lse[lo] : 0.f;
        d_stage = ok ? a.delta[lo] : 0.f;
      }
    };
    auto publish = [&]() {
      store_swizzled<T>(qf, Qb, tid);
      store_swizzled<T>(dof, dOb, tid);
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
#pragma unroll
      for (int k = 0; k < kKS; ++k) {
        s = Tr::mfma(swz_read_row<T, kD>(Qb, row_a, wave * kKS + k, 0), kreg[k], s);
        dp = Tr::mfma(swz_read_row<T, kD>(dOb, row_a, wave * kKS + k, 0), vreg[k], dp);
      }
      part_write(partS, wave, lane, s);
      part_write(partD, wave, lane, dp);
      __syncthreads();
      // this wave's quarter of the elements: queries m0 + 8 wave + 4 hi + r
      const f32x4 s4 = part_sum_quarter(partS, wave, lane);
      const f32x4 dp4 = part_sum_quarter(partD, wave, lane);

      DropoutState dst{};
      if (kDropout) dst = dropout_for_head(drop0, z, hq, a.hq, a.seq.max_seqlen_q);
      const T* bptr = nullptr;
      if (kBias)
        bptr = reinterpret_cast<const T*>(a.bias) + (int64_t)si.batch_index * a.sb_z + (int64_t)hq * a.sb_h +
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
          x = __builtin_fmaf((float)bptr[(int64_t)mm * a.sb_m], kLog2e, s4[r] * qk_scale) - l4[r];
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
      opnd_write<T>(opP, wave, lane, pd);       // p cast to dO's type (composed_tensors.py:191-193)
      opnd_write<T>(opS, wave, lane, dsv);
      __syncthreads();
      // dV^T += dO^T P and dK^T += Q^T dS on this wave's columns
#pragma unroll
      for (int t = 0; t < kBC / 16; ++t) {
        const op_t pb = opnd_read<T>(opP, t, lane);
        const op_t sb = opnd_read<T>(opS, t, lane);
#pragma unroll
        for (int db = 0; db < kDB; ++db) {
          dv[db] = Tr::mfma(swz_read_tr<T, kD>(dOb, tr_a0, tr_a1, t, wave * kDB + db), pb, dv[db]);
          dk[db] = Tr::mfma(swz_read_tr<T, kD>(Qb, tr_a0, tr_a1, t, wave * kDB + db), sb, dk[db]);
        }
      }
      __syncthreads();                 // the tile and the partial blocks have been read
      if (it + 1 < total) {
        publish();
        __syncthreads();
      }
    }
  }

  if (key_ok) {
#pragma unroll
    for (int db = 0; db < kDB; ++db)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        q4_t k4, v4;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          k4[r] = Tr::cvt(dk[db][4 * g + r] * a.sm_scale);   // bwd_kernel_dk_dv.py:387-389
          v4[r] = Tr::cvt(dv[db][4 * g + r]);
        }
        if (col0 + 32 * db + 8 * g + 4 * hi < d_qk) *reinterpret_cast<q4_t*>(dkptr + 32 * db + 8 * g + 4 * hi) = k4;
        if (col0 + 32 * db + 8 * g + 4 * hi < d_v) *reinterpret_cast<q4_t*>(dvptr + 32 * db + 8 * g + 4 * hi) = v4;
      }
  }
}

// dQ and dB: one workgroup = 64 query rows of one head = 8 waves, four per 32-row block (two row
// blocks share the K/V tiles, two waves per SIMD, as in the forward); the lane's query is
// lane % 32 of its row block, the keys of a tile are spread over the accumulator elements.
struct SmemDq512 {
  static constexpr int TILE_BYTES = SmemBwd512::TILE_BYTES;
  static constexpr int PART_OFF = 2 * TILE_BYTES;
  static constexpr int OPND_OFF = PART_OFF + kFRB * 2 * Smem512::PART_BYTES;   // dS operand pieces per row block
  static constexpr int BYTES = OPND_OFF + kFRB * kOpndBytes;
};

template <typename T, bool kWindowed, bool kBias, bool kDropout>
__global__ __launch_bounds__(kFNT) void bwd_dq_d512_kernel(const BwdArgs a) {
  using Tr = Traits<T>;
  using op_t = typename Tr::op_t;
  using q4_t = typename Tr::q4_t;
  using SM = SmemDq512;
  extern __shared__ __attribute__((aligned(16))) char smem_raw[];
  char* Kb = smem_raw;
  char* Vb = smem_raw + SM::TILE_BYTES;

  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int rb = wave / kNW, cw = wave % kNW;             // row block, column share
  const int lane = tid & 63, c = lane & 31, hi = lane >> 5;
  // one workgroup per (sequence, q-head, Q tile): the tiles of a kv-head's group back to back on one
  // XCD, most visible keys (causal) first
  const int nmt = (a.seq.max_seqlen_q + kFBR - 1) / kFBR, group = a.hq / a.hk;
  int pair, r_item;
  if (!xcd_item(blockIdx.x, nseq_of(a.seq, a.batch) * a.hk, group * nmt, pair, r_item)) return;
  const int z = pair / a.hk, h = (pair % a.hk) * group + r_item % group;
  const int mt = nmt - 1 - r_item / group;
  const int d_qk = a.head_dim, d_v = a.head_dim_v;
  const int col0 = cw * kDW;
  float* partS = reinterpret_cast<float*>(smem_raw + SM::PART_OFF) + rb * 2 * (Smem512::PART_BYTES / 4);
  float* partD = partS + Smem512::PART_BYTES / 4;
  char* opS = smem_raw + SM::OPND_OFF + rb * kOpndBytes;

  const SeqInfo si = get_seq(a.seq, z);
  const int q0 = mt * kFBR;
  if (q0 >= si.seqlen_q) return;

  Window w{0, 0};
  if (kWindowed) w = parse_window(a.mask.causal_type, a.mask.window_left, a.mask.window_right,
                                  si.seqlen_q, si.seqlen_k);
  w.left = w.left > (1 << 30) ? (1 << 30) : (w.left < -(1 << 30) ? -(1 << 30) : w.left);
  w.right = w.right > (1 << 30) ? (1 << 30) : (w.right < -(1 << 30) ? -(1 << 30) : w.right);
  const BlockRanges br = block_ranges(kWindowed, w.left, w.right, q0, si.seqlen_q, si.seqlen_k, kFBR, kBC);

  const int hk = h / (a.hq / a.hk);
  const int row = q0 + 32 * rb + c;
  const bool row_ok = row < si.seqlen_q;
  const int row_c = row_ok ? row : si.seqlen_q - 1;
  const int nkt = (si.seqlen_k + kBC - 1) / kBC;
  T* dqptr = reinterpret_cast<T*>(a.dq) + (int64_t)si.batch_index * a.sdq.z + (int64_t)h * a.sdq.h +
             (int64_t)(si.q_start + row_c) * a.sdq.s + col0;
  const bool want_db = kBias && a.db != nullptr;
  T* dbhead = want_db ? reinterpret_cast<T*>(a.db) + (int64_t)si.batch_index * a.sdb_z + (int64_t)h * a.sdb_h : nullptr;

  // dB of K tiles that are never visited is zero: wave w sweeps the rows w, w + 8, ...
  auto zero_db = [&](int j_from, int j_to) {
    if (!want_db) return;
    const int c0 = j_from * kBC, c1 = j_to * kBC < si.seqlen_k ? j_to * kBC : si.seqlen_k;
    if (c0 >= c1) return;
    for (int rr = wave; rr < kFBR; rr += kFRB * kNW) {
      const int m = q0 + rr;
      if (m >= si.seqlen_q) break;
      T* rowp = dbhead + (int64_t)m * a.sdb_m;
      for (int n = c0 + lane; n < c1; n += 64) rowp[(int64_t)n * a.sdb_n] = Tr::cvt(0.f);
    }
  };

  f32x16 dq[kDB];
#pragma unroll
  for (int db = 0; db < kDB; ++db)
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

    // the wave's columns of this lane's Q and dO rows as B operands
    op_t qreg[kKS], doreg[kKS];
    {
      const T* qptr = reinterpret_cast<const T*>(a.q) + (int64_t)si.batch_index * a.sq.z + (int64_t)h * a.sq.h +
                      (int64_t)(si.q_start + row_c) * a.sq.s + col0;
      const T* doptr = reinterpret_cast<const T*>(a.dout) + (int64_t)si.batch_index * a.sdo.z + (int64_t)h * a.sdo.h +
                       (int64_t)(si.q_start + row_c) * a.sdo.s + col0;
      const op_t zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
      for (int k = 0; k < kKS; ++k) {
        qreg[k] = col0 + 16 * k + 8 * hi < d_qk ? *reinterpret_cast<const op_t*>(qptr + 16 * k + 8 * hi) : zero8;
        doreg[k] = col0 + 16 * k + 8 * hi < d_v ? *reinterpret_cast<const op_t*>(doptr + 16 * k + 8 * hi) : zero8;
      }
    }
    const int64_t lo = lse_offset(si, h, a.hq) + row_c;
    const float l_row = a.lse[lo] * kRcpLn2;               // bwd_kernel_dq.py:305
    const float d_row = a.delta[lo];
    const float qk_scale = a.sm_scale * kLog2e;
    const T* bptr = nullptr;
    if (kBias)
      bptr = reinterpret_cast<const T*>(a.bias) + (int64_t)si.batch_index * a.sb_z + (int64_t)h * a.sb_h +
             (int64_t)row_c * a.sb_m;
    T* dbptr = want_db ? dbhead + (int64_t)row_c * a.sdb_m : nullptr;
    DropoutState dst{};
    if (kDropout) dst = make_dropout(a.drop, z, h, a.hq, a.seq.max_seqlen_q, a.seq.max_seqlen_k);
    const int row_a = Swz<kD>::row_base(lane), tr_a0 = Swz<kD>::tr_base(lane, 0), tr_a1 = Swz<kD>::tr_base(lane, 1);

    const T* kt = reinterpret_cast<const T*>(a.k) + (int64_t)si.batch_index * a.sk.z + (int64_t)hk * a.sk.h +
                  (int64_t)(si.k_start + br.lo * kBC) * a.sk.s;
    const T* vt = reinterpret_cast<const T*>(a.v) + (int64_t)si.batch_index * a.sv.z + (int64_t)hk * a.sv.h +
                  (int64_t)(si.k_start + br.lo * kBC) * a.sv.s;
    int rows_left = si.seqlen_k - br.lo * kBC;      // > 0
    TileFetch<T, kFNT> kf, vf;
    auto fetch = [&]() {
      const int rows = rows_left < kBC ? rows_left : kBC;
      kf.load(kt, rows, a.sk.s, d_qk, tid);
      vf.load(vt, rows, a.sv.s, d_v, tid);
      kt += (int64_t)kBC * a.sk.s; vt += (int64_t)kBC * a.sv.s; rows_left -= kBC;
    };
    auto publish = [&]() {
      store_swizzled<T, kFNT>(kf, Kb, tid);
      store_swizzled<T, kFNT>(vf, Vb, tid);
    };

    fetch();
    publish();
    __syncthreads();
    for (int j = br.lo; j <= br.hi; ++j) {
      if (j < br.hi) fetch();
      // this wave's share of S^T = K Q^T and dP^T = V dO^T (rows: keys, columns: queries)
      f32x16 s, dp;
#pragma unroll
      for (int i = 0; i < 16; ++i) { s[i] = 0.f; dp[i] = 0.f; }
#pragma unroll
      for (int k = 0; k < kKS; ++k) {
        s = Tr::mfma(swz_read_row<T, kD>(Kb, row_a, cw * kKS + k, 0), qreg[k], s);
        dp = Tr::mfma(swz_read_row<T, kD>(Vb, row_a, cw * kKS + k, 0), doreg[k], dp);
      }
      part_write(partS, cw, lane, s);
      part_write(partD, cw, lane, dp);
      __syncthreads();
      // this wave's quarter of its row block's elements: keys j kBC + 8 cw + 4 hi + r
      const f32x4 s4 = part_sum_quarter(partS, cw, lane);
      const f32x4 dp4 = part_sum_quarter(partD, cw, lane);

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
          x = __builtin_fmaf((float)bptr[(int64_t)nn * a.sb_n], kLog2e, s4[r] * qk_scale) - l_row;
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
        if (want_db && row_ok && n < si.seqlen_k) dbptr[(int64_t)n * a.sdb_n] = Tr::cvt(dsv);   // :200-204
      }
      opnd_write<T>(opS, cw, lane, dsv4);       // ds cast to K's type
      __syncthreads();
      // dQ^T += K^T dS^T on this wave's columns
#pragma unroll
      for (int t = 0; t < kBC / 16; ++t) {
        const op_t sb = opnd_read<T>(opS, t, lane);
#pragma unroll
        for (int db = 0; db < kDB; ++db)
          dq[db] = Tr::mfma(swz_read_tr<T, kD>(Kb, tr_a0, tr_a1, t, cw * kDB + db), sb, dq[db]);
      }
      __syncthreads();                 // the tile and the partial blocks have been read
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
    for (int db = 0; db < kDB; ++db)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        q4_t t4;
#pragma unroll
        for (int r = 0; r < 4; ++r) t4[r] = Tr::cvt(dq[db][4 * g + r] * a.sm_scale);   // bwd_kernel_dq.py:374-376
        if (col0 + 32 * db + 8 * g + 4 * hi < d_qk) *reinterpret_cast<q4_t*>(dqptr + 32 * db + 8 * g + 4 * hi) = t4;
      }
  }
}

template <auto kern, int NT = kNT, typename Args>
hipError_t launch512(dim3 grid, int smem, hipStream_t stream, const Args& a) {
  if (grid.x == 0 || grid.y == 0 || grid.z == 0) return hipSuccess;   // an empty tensor: nothing to write
  static std::atomic<uint64_t> lds_set{0};
  hipError_t e = allow_large_lds(reinterpret_cast<const void*>(kern), smem, lds_set);
  if (e != hipSuccess) return e;
  hipLaunchKernelGGL(kern, grid, dim3(NT), smem, stream, a);
  return hipGetLastError();
}

#define FA_D512_SWITCH(CALL)                                           \
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

template <typename T>
hipError_t run_fwd_t(const FwdArgs& a, bool windowed, bool bias, bool dropout, hipStream_t s) {
  const dim3 grid(xcd_grid(nseq_of(a.seq, a.batch) * a.hk, (a.hq / a.hk) * ((a.seq.max_seqlen_q + kFBR - 1) / kFBR)));
  constexpr int smem = SmemFwd512::BYTES;
#define FA_CALL(W, B, P) launch512<fwd_d512_kernel<T, W, B, P>, kFNT>(grid, smem, s, a)
  FA_D512_SWITCH(FA_CALL)
#undef FA_CALL
}

template <typename T>
hipError_t run_bwd_t(int kernel_slot, const BwdArgs& a, bool windowed, bool bias, bool dropout, hipStream_t s) {
  const int nseq = nseq_of(a.seq, a.batch);
  if (kernel_slot == 1) {
    const dim3 grid(xcd_grid(nseq * a.hk, (a.seq.max_seqlen_k + kBR - 1) / kBR));
#define FA_CALL(W, B, P) launch512<bwd_dkdv_d512_kernel<T, W, B, P>>(grid, SmemBwd512::BYTES, s, a)
    FA_D512_SWITCH(FA_CALL)
#undef FA_CALL
  }
  if (kernel_slot == 2) {
    const dim3 grid(xcd_grid(nseq * a.hk, (a.hq / a.hk) * ((a.seq.max_seqlen_q + kFBR - 1) / kFBR)));
#define FA_CALL(W, B, P) launch512<bwd_dq_d512_kernel<T, W, B, P>, kFNT>(grid, SmemDq512::BYTES, s, a)
    FA_D512_SWITCH(FA_CALL)
#undef FA_CALL
  }
  return hipErrorInvalidValue;
}

}  // namespace

hipError_t run_bwd_d512(int dtype, int kernel_slot, const BwdArgs& a, bool windowed, bool bias, bool dropout,
                        hipStream_t s) {
  if (dtype == kDtypeBF16) return run_bwd_t<bf16_t>(kernel_slot, a, windowed, bias, dropout, s);
  if (dtype == kDtypeF16) return run_bwd_t<f16_t>(kernel_slot, a, windowed, bias, dropout, s);
  return hipErrorNotSupported;
}

hipError_t run_fwd_d512(int dtype, const FwdArgs& a, bool windowed, bool bias, bool dropout, hipStream_t s) {
  if (dtype == kDtypeBF16) return run_fwd_t<bf16_t>(a, windowed, bias, dropout, s);
  if (dtype == kDtypeF16) return run_fwd_t<f16_t>(a, windowed, bias, dropout, s);
  return hipErrorNotSupported;
}

TileShape d512_tile_shape(int kernel_slot) {
  // forward (kernel_slot < 0) and dQ: 64 queries per workgroup against 32 keys per step; dK/dV: 32
  // keys per workgroup against 32 queries per step
  if (kernel_slot < 0) return TileShape{kFBR, kBC, kFRB * kNW, SmemFwd512::BYTES};
  if (kernel_slot == 2) return TileShape{kFBR, kBC, kFRB * kNW, SmemDq512::BYTES};
  return TileShape{kBC, kBR, kNW, SmemBwd512::BYTES};
}

}  // namespace fa
