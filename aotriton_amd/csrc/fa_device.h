// Device-side building blocks for the gfx950 flash-attention kernels:
// MFMA wrappers, operand packing, Philox dropout, sequence bookkeeping.
//
// MFMA 32x32x16 register layout (wave64, lane = 32*hi + c):
//   A operand: row  = c, k = 8*hi .. 8*hi+7   (8 x 16-bit per lane)
//   B operand: col  = c, k = 8*hi .. 8*hi+7
//   C/D      : col  = c, row(i) = 8*(i/4) + 4*hi + (i%4), i = 0..15
// The contraction index is a dummy, so any permutation of k that is applied to
// both operands is legal.  All kernels exploit that: an accumulator block is
// re-used as an operand with k-slot (t, hi, j) <-> row 16*t + 8*(j/4) + 4*hi + (j%4),
// and the other operand is fetched from a row-major LDS tile with transposing reads
// that deliver exactly that order.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>

#include "fa_args.h"
#include "fa_intervals.h"

namespace fa {

// Kernels with more than 64 KB of LDS need hipFuncAttributeMaxDynamicSharedMemorySize, which is a
// property of the function on one device: set on the first launch per (kernel, device), `done`
// being the kernel's own bit mask of devices.
inline hipError_t allow_large_lds(const void* kern, int smem, std::atomic<uint64_t>& done) {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return e;
  const uint64_t bit = 1ull << (dev & 63);
  if (done.load(std::memory_order_acquire) & bit) return hipSuccess;
  e = hipFuncSetAttribute(kern, hipFuncAttributeMaxDynamicSharedMemorySize, smem);
  if (e == hipSuccess) done.fetch_or(bit, std::memory_order_release);
  return e;
}

typedef __bf16 bf16_t;
typedef _Float16 f16_t;

template <typename T, int N>
using vec = T __attribute__((ext_vector_type(N)));

using f32x16 = vec<float, 16>;
using f32x4 = vec<float, 4>;
using u32x4_t = vec<unsigned, 4>;   // payload type of the 16-byte buffer loads and stores

constexpr float kLog2e = 1.44269504089f;       // modules/flash/kernel/fwd_kernel.py:422
constexpr float kLn2 = 0.6931471824645996f;    // modules/flash/kernel/fwd_kernel.py:610-612
constexpr float kRcpLn2 = 1.4426950408889634f; // modules/flash/kernel/bwd_inner_dk_dv.py:185
// Running-max seed.  The reference seeds with -3.40282e38 (fwd_kernel.py:417); a
// smaller magnitude keeps max*scale finite so that -inf scores never meet -inf maxima.
constexpr float kNegBig = -1.0e30f;

template <typename T> struct Traits;

// ds_read_b64_tr_b16: 16 lanes x 4 16-bit elements, transposed on the way out of LDS.
typedef short tr_raw_t __attribute__((__vector_size__(4 * sizeof(short))));
__device__ __forceinline__ tr_raw_t lds_read_tr_raw(const void* p) {
  return __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) tr_raw_t*)(p));
}

template <> struct Traits<bf16_t> {
  using op_t = vec<__bf16, 8>;
  using q4_t = vec<__bf16, 4>;
  using p2_t = vec<__bf16, 2>;
  static __device__ __forceinline__ q4_t lds_read_tr(const bf16_t* p) {
    return __builtin_bit_cast(q4_t, lds_read_tr_raw(p));
  }
  static __device__ __forceinline__ f32x16 mfma(op_t a, op_t b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
  }
  static __device__ __forceinline__ bf16_t cvt(float x) { return (bf16_t)x; }
  // two values at once: one v_cvt_pk_bf16_f32
  static __device__ __forceinline__ p2_t cvt2(float x, float y) {
    return __builtin_convertvector((vec<float, 2>){x, y}, p2_t);
  }
};

template <> struct Traits<f16_t> {
  using op_t = vec<_Float16, 8>;
  using q4_t = vec<_Float16, 4>;
  using p2_t = vec<_Float16, 2>;
  static __device__ __forceinline__ q4_t lds_read_tr(const f16_t* p) {
    return __builtin_bit_cast(q4_t, lds_read_tr_raw(p));
  }
  static __device__ __forceinline__ f32x16 mfma(op_t a, op_t b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
  }
  static __device__ __forceinline__ f16_t cvt(float x) { return (f16_t)x; }
  // two values at once: one v_cvt_pk_f16_f32 (from scalar conversions the compiler makes two
  // v_cvt_f16_f32 and a v_pack_b32_f16)
  static __device__ __forceinline__ p2_t cvt2(float x, float y) {
    return __builtin_convertvector((vec<float, 2>){x, y}, p2_t);
  }
};

// Eight accumulator values (i = 8*half .. 8*half+7) -> one MFMA operand.
template <typename T>
__device__ __forceinline__ typename Traits<T>::op_t pack8(const f32x16& s, int half) {
  typename Traits<T>::op_t r;
#pragma unroll
  for (int j = 0; j < 8; j += 2) {
    const typename Traits<T>::p2_t p2 = Traits<T>::cvt2(s[8 * half + j], s[8 * half + j + 1]);
    r[j] = p2[0]; r[j + 1] = p2[1];
  }
  return r;
}

// MFMA operand whose 8 k-slots are rows (kbase + 8*w + 4*hi + j) of a row-major LDS
// tile and whose M/N index (lane%32) is the column: two transposing reads.  `p`
// must already point at row (4*hi + (lane%16)/4), column (16*((lane/16)%2) + 4*(lane%4))
// of the 32-column block; rstr is the row stride in elements.
// Within each group of 16 lanes the hardware returns to lane i, slot j, the element
// (i%4) of the 8 bytes addressed by lane (4*j + i/4).
template <typename T>
__device__ __forceinline__ typename Traits<T>::op_t lds_read_tr8(const T* p, int rstr) {
  const typename Traits<T>::q4_t lo = Traits<T>::lds_read_tr(p);
  const typename Traits<T>::q4_t hi = Traits<T>::lds_read_tr(p + 8 * rstr);
  return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
}

// Swizzled LDS tile of rows of D 16-bit elements, no padding.  The 16-byte chunk `ch`
// of row r lives at chunk position ch ^ f(r) of that row.  f is chosen so that both
// access patterns of the kernels sweep all 64 banks once: the 16-byte row reads of an
// MFMA operand (16 consecutive rows, same chunk) and the transposing reads (4
// consecutive rows x 4 consecutive chunks per half-wave).  A tile can therefore
// serve both as the row operand of one GEMM and as the transposed operand of another.
template <int D>
struct Swz {
  static constexpr int ROWB = D * 2;
  static __device__ __forceinline__ int f(int r) {
    return D == 64 ? ((((r >> 1) & 1) << 2) | ((r >> 2) & 3)) : (((r & 3) << 2) | ((r >> 2) & 3));
  }
  // byte offset of chunk ch of row r
  static __device__ __forceinline__ int addr(int r, int ch) { return r * ROWB + ((ch ^ f(r)) << 4); }
  // lane constant of the row reads: MFMA operand row = lane%32 (+32*mb), k-slots 8*hi..
  static __device__ __forceinline__ int row_base(int lane) { return addr(lane & 31, lane >> 5); }
  // lane constants of the transposing reads (rows 8*w + 4*hi + (lane%16)/4 of a 16-row step)
  static __device__ __forceinline__ int tr_base(int lane, int w) {
    const int r = 8 * w + 4 * (lane >> 5) + (lane & 15) / 4;
    const int ch = 2 * ((lane >> 4) & 1) + ((lane & 3) >> 1);
    return addr(r, ch) + 8 * (lane & 1);
  }
};
// row operand of k-step k, 32-row block mb (f depends on r % 16 only, so the block is a
// plain offset and the k-step flips chunk bits)
template <typename T, int D>
__device__ __forceinline__ typename Traits<T>::op_t swz_read_row(const char* tile, int row_base, int k, int mb) {
  return *reinterpret_cast<const typename Traits<T>::op_t*>(tile + ((row_base ^ (k << 5)) + mb * 32 * Swz<D>::ROWB));
}
// transposed operand: k-slots are rows 16*t + 8*w + 4*hi + j of the tile, M/N index is
// column 32*db + lane%32 (see lds_read_tr8 for the hardware's lane mapping)
template <typename T, int D>
__device__ __forceinline__ typename Traits<T>::op_t swz_read_tr(const char* tile, int tr_base0, int tr_base1,
                                                                int t, int db) {
  const typename Traits<T>::q4_t lo = Traits<T>::lds_read_tr(
      reinterpret_cast<const T*>(tile + ((tr_base0 ^ (db << 6)) + t * 16 * Swz<D>::ROWB)));
  const typename Traits<T>::q4_t hi = Traits<T>::lds_read_tr(
      reinterpret_cast<const T*>(tile + ((tr_base1 ^ (db << 6)) + t * 16 * Swz<D>::ROWB)));
  return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
}

// The one place where a buffer descriptor is built.  Every argument passes through
// v_readfirstlane: the descriptor is then uniform for the compiler whatever it was derived from.
// A descriptor built from a value the compiler takes for divergent (threadIdx.x >> 6, say, which
// is the same in all lanes of a wave without the compiler knowing it) makes it wrap every access
// in a loop over the distinct descriptors, and hipcc 7.2 has placed a register spill into the exit
// block of such a loop, where no lane is enabled: the store is lost and the reload returns what the
// slot held before.  On values that are uniform already the three instructions fold away.
// bytes: length of the range, accesses past it read zero / write nothing.
template <typename P>
__device__ __forceinline__ __amdgpu_buffer_rsrc_t wave_rsrc(P* base, int bytes) {
  const uint64_t a = reinterpret_cast<uint64_t>(base);
  const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)a);
  const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)(a >> 32));
  return __builtin_amdgcn_make_buffer_rsrc(reinterpret_cast<void*>((uint64_t)hi << 32 | lo), 0,
                                           __builtin_amdgcn_readfirstlane(bytes), 0x00020000);
}

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ __forceinline__ float fast_log2(float x) { return __builtin_amdgcn_logf(x); }

// Reductions across the two halves of a wave (lane <-> lane ^ 32) with
// v_permlane32_swap: after the swap one register holds the lower half's value in
// both halves and the other one the upper half's value; no LDS round trip.
__device__ __forceinline__ void wave_halves(float x, float& lower, float& upper) {
  const unsigned u = __builtin_bit_cast(unsigned, x);
  const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  const unsigned r0 = r[0], r1 = r[1];
  lower = __builtin_bit_cast(float, r0);
  upper = __builtin_bit_cast(float, r1);
}
__device__ __forceinline__ float cross_max(float x) {
  float lo, up;
  wave_halves(x, lo, up);
  return fmaxf(lo, up);
}
__device__ __forceinline__ float cross_sum(float x) {
  float lo, up;
  wave_halves(x, lo, up);
  return lo + up;
}

// Philox-4x32-10 with counter (c0, c1, 0, 0); Salmon et al. SC'11.  The
// reference reaches it through Triton's tl.randint4x
// (modules/flash/kernel/dropout.py:19).
__device__ __forceinline__ void philox4x32_10(uint32_t c0, uint32_t c1, uint32_t k0, uint32_t k1,
                                              uint32_t (&w)[4]) {
  uint32_t c2 = 0, c3 = 0;
#pragma unroll
  for (int i = 0; i < 10; ++i) {
    // one 32x32->64 multiply per product (v_mad_u64_u32) instead of a high and a low half
    const uint64_t p0 = (uint64_t)0xD2511F53u * c0, p1 = (uint64_t)0xCD9E8D57u * c2;
    const uint32_t hi0 = (uint32_t)(p0 >> 32), lo0 = (uint32_t)p0;
    const uint32_t hi1 = (uint32_t)(p1 >> 32), lo1 = (uint32_t)p1;
    // (three-input xor: one v_bitop3_b32 with truth table 0x96 instead of two v_xor_b32)
    const uint32_t n0 = __builtin_amdgcn_bitop3_b32(hi1, c1, k0, 0x96), n2 = __builtin_amdgcn_bitop3_b32(hi0, c3, k1, 0x96);
    c0 = n0; c1 = lo1; c2 = n2; c3 = lo0;
    k0 += 0x9E3779B9u; k1 += 0xBB67AE85u;
  }
  w[0] = c0; w[1] = c1; w[2] = c2; w[3] = c3;
}

struct DropoutState {
  uint32_t k0, k1;
  uint64_t base;     // philox_offset2 + *philox_offset1 + int32((z*Hq + h)*max_seqlen_q*stride)
  uint32_t stride;   // cdiv(max_seqlen_k, 4)
  int32_t thr;
  float scale;       // 1/(1-p)
};

// The part that reads memory (seed and offset are device scalars): once per work item.  A kernel
// that walks several heads keeps this and calls dropout_for_head per head; reading the two scalars
// again for every tile costs two L2 round trips that nothing hides.
__device__ __forceinline__ DropoutState make_dropout_base(const DropoutArgs& d, int max_seqlen_k) {
  DropoutState s;
  const uint64_t seed = d.seed_ptr ? *d.seed_ptr : 0ull;
  uint64_t base = d.offset2;
  if (d.offset1_ptr) base += *d.offset1_ptr;
  s.k0 = (uint32_t)seed; s.k1 = (uint32_t)(seed >> 32);
  s.stride = (uint32_t)((max_seqlen_k + 3) / 4);
  s.base = base;
  s.thr = dropout_threshold(d.p);
  s.scale = 1.0f / (1.0f - d.p);
  return s;
}

__device__ __forceinline__ DropoutState dropout_for_head(const DropoutState& s0, int z, int h, int hq,
                                                         int max_seqlen_q) {
  DropoutState s = s0;
  // modules/flash/kernel/fwd_kernel.py:405-407: the per-head term is a product of int32
  // values there, so it wraps modulo 2^32 and is sign-extended into the 64-bit base.
  const uint32_t head_term = (uint32_t)(z * hq + h) * (uint32_t)max_seqlen_q * s.stride;
  s.base = s0.base + (uint64_t)(int64_t)(int32_t)head_term;
  return s;
}

__device__ __forceinline__ DropoutState make_dropout(const DropoutArgs& d, int z, int h, int hq,
                                                     int max_seqlen_q, int max_seqlen_k) {
  return dropout_for_head(make_dropout_base(d, max_seqlen_k), z, h, hq, max_seqlen_q);
}

// Keep bits of columns n0..n0+3 (n0 % 4 == 0) of row m, bit r <-> column n0+r.
// Word order along the row is (w0, w2, w1, w3): modules/flash/kernel/dropout.py:37.
__device__ __forceinline__ uint32_t dropout_keep4(const DropoutState& s, int m, int n0) {
  const uint64_t ctr = s.base + (uint64_t)m * s.stride + (uint64_t)(n0 >> 2);
  uint32_t w[4];
  philox4x32_10((uint32_t)ctr, (uint32_t)(ctr >> 32), s.k0, s.k1, w);
  return ((int32_t)w[0] > s.thr ? 1u : 0u) | ((int32_t)w[2] > s.thr ? 2u : 0u) |
         ((int32_t)w[1] > s.thr ? 4u : 0u) | ((int32_t)w[3] > s.thr ? 8u : 0u);
}

// Keep bit of a single element.
__device__ __forceinline__ bool dropout_keep1(const DropoutState& s, int m, int n) {
  return (dropout_keep4(s, m, n & ~3) >> (n & 3)) & 1u;
}

// Per-sequence bookkeeping: modules/flash/kernel/fwd_kernel.py:243-286.
struct SeqInfo {
  int32_t seqlen_q, seqlen_k;
  int32_t q_start, k_start;   // row offset inside the (packed) tensor
  int32_t batch_index;        // index along the tensors' batch stride
  int64_t lse_stride;         // rows per (batch, head) slab of LSE / delta
};

__device__ __forceinline__ SeqInfo get_seq(const SeqArgs& s, int z) {
  SeqInfo r;
  if (s.num_seqlens > 0) {
    r.seqlen_q = s.cu_q[z + 1] - s.cu_q[z];
    r.seqlen_k = s.cu_k[z + 1] - s.cu_k[z];
    r.batch_index = 0;
    if (s.ss_q != nullptr) {
      r.q_start = s.ss_q[z];
      r.k_start = s.ss_k[z];
      r.lse_stride = s.ss_q[s.num_seqlens];
    } else {
      r.q_start = s.cu_q[z];
      r.k_start = s.cu_k[z];
      r.lse_stride = s.cu_q[s.num_seqlens];
    }
  } else if (s.num_seqlens < 0) {
    r.seqlen_q = s.cu_q[z + 1] - s.cu_q[z];
    r.seqlen_k = s.cu_k[z + 1] - s.cu_k[z];
    r.q_start = 0; r.k_start = 0;
    r.batch_index = z;
    r.lse_stride = s.max_seqlen_q;
  } else {
    r.seqlen_q = s.max_seqlen_q;
    r.seqlen_k = s.max_seqlen_k;
    r.q_start = 0; r.k_start = 0;
    r.batch_index = z;
    r.lse_stride = s.max_seqlen_q;
  }
  return r;
}

// Byte offset that no buffer descriptor of these kernels covers: a lane whose 16-byte
// chunk lies in the padding of a head dim that was rounded up reads zeros with it.
constexpr int kVoffOutOfRange = 0x7fff0000;

// (sequence, head) of the linear work index zh.  The heads of one GQA group are
// adjacent, then come the sequences, then the kv-heads: the contiguous range of zh
// that an XCD owns then holds whole kv-heads across ALL sequences, so XCDs get equal
// work even when the sequences of a varlen batch differ in length, and neighbours in
// zh share K/V.  `group` = q-heads per kv-head when zh counts q-heads, 1 when it counts
// kv-heads.
__device__ __forceinline__ void split_zh(int zh, int nseq, int group, int& z, int& h) {
  const int g = zh % group, t = zh / group;
  z = t % nseq;
  h = (t / nseq) * group + g;
}

// The list of work items of one XCD when the sequences differ in length.  The dense list of the
// persistent kernels has a slot for every tile up to the longest sequence, most of them empty for
// the short ones, and which worker draws the empty slots is systematic (16 packed sequences of
// 256-8192 tokens: the busiest forward worker had 19 % more K tiles than the average).  This list
// holds the valid tiles only: the heads zh of the XCD set by set (a set = the `ratio` heads that
// share K/V, or Q/dO: the q-heads of one kv-head of one sequence), a set's tiles one after the
// other with its heads interleaved.  A worker asks for positions t in increasing order.
struct RaggedWalk {
  int lo, hi, ratio, nseq, rows_per_tile;
  bool keys;                       // tiles count keys (dK/dV) instead of queries
  int set, set_end, base, first, members, tiles;
  __device__ __forceinline__ void open(const SeqArgs& seq) {
    first = lo > set * ratio ? lo : set * ratio;
    members = (hi < (set + 1) * ratio ? hi : (set + 1) * ratio) - first;
    const SeqInfo si = get_seq(seq, set % nseq);
    tiles = ((keys ? si.seqlen_k : si.seqlen_q) + rows_per_tile - 1) / rows_per_tile;
  }
  __device__ __forceinline__ void init(const SeqArgs& seq, int xcd, int zh_per_xcd, int num_zh, int ratio_, int nseq_,
                                       int rows_per_tile_, bool keys_) {
    lo = xcd * zh_per_xcd;
    hi = lo + zh_per_xcd < num_zh ? lo + zh_per_xcd : num_zh;
    ratio = ratio_; nseq = nseq_; rows_per_tile = rows_per_tile_; keys = keys_;
    set = lo / ratio; set_end = (hi + ratio - 1) / ratio;
    base = 0; first = 0; members = 0; tiles = 0;
    if (set < set_end) open(seq);
  }
  // head zh and tile index (counted from the sequence's start) at position t; false past the end
  __device__ __forceinline__ bool at(const SeqArgs& seq, int t, int& zh, int& tile) {
    while (set < set_end && t >= base + members * tiles) {
      base += members * tiles;
      if (++set < set_end) open(seq);
    }
    if (set >= set_end) return false;
    const int off = t - base;
    zh = first + off % members;
    tile = off / members;
    return true;
  }
  __device__ __forceinline__ int tiles_of_set() const { return tiles; }
};

// A second list for sequences of different lengths, in the order of the tiles' distance to the end of
// their sequence: level w holds tile n - w of every (sequence, head) entry that has n >= w tiles, the
// levels run from the longest sequence's n down to 1.  Under a causal mask that distance is the weight
// of a dK/dV item (the queries from the key tile to the end), so the list is sorted heaviest first and
// the serpentine rounds of the workers pair items of nearly equal weight; any other mask only loses
// that property, every valid tile still appears exactly once.  Replaying the schedule of 16 packed
// sequences of 256-8192 tokens on 32 workers: the busiest worker has 1.5 % more work than the average
// against 16 % with the dense list.  The workgroup sorts the entries of its XCD by tile count into
// LDS once (at most kLevelCap entries; the caller keeps the dense list beyond that).
constexpr int kLevelCap = 512;
constexpr int kLevelBytes = 2 * kLevelCap * 4;
struct LevelWalk {
  const uint32_t* tab;             // (tiles << 16 | 0xffff - entry), descending
  int count, w, base, c;           // entries; current level, position of its first item, entries that reach it
  bool keys;                       // tiles count keys and a level is the distance to the END (dK/dV); else queries, from the start
  __device__ __forceinline__ int tiles_at(int i) const { return (int)(__builtin_amdgcn_readfirstlane(tab[i]) >> 16); }
  // all threads of the workgroup (NT of them) call this; entries are the heads lo .. hi-1, `ratio` of
  // them per (sequence, kv-head)
  template <int NT>
  __device__ __forceinline__ void init(uint32_t* lds, const SeqArgs& seq, int lo, int hi, int nseq, int ratio,
                                       int rows_per_tile, bool keys_, int tid) {
    count = hi - lo;
    keys = keys_;
    uint32_t* raw = lds + kLevelCap;
    for (int i = tid; i < count; i += NT) {
      const SeqInfo si = get_seq(seq, ((lo + i) / ratio) % nseq);
      const int n = ((keys ? si.seqlen_k : si.seqlen_q) + rows_per_tile - 1) / rows_per_tile;
      raw[i] = (uint32_t)n << 16 | (uint32_t)(0xffff - i);
    }
    __syncthreads();
    for (int i = tid; i < count; i += NT) {
      const uint32_t key = raw[i];
      int rank = 0;
      for (int j = 0; j < count; ++j) rank += raw[j] > key ? 1 : 0;
      lds[rank] = key;
    }
    __syncthreads();
    tab = lds;
    w = count > 0 ? tiles_at(0) : 0;
    base = 0; c = 0;
    while (c < count && tiles_at(c) >= w) ++c;
  }
  // entry (0 .. count-1) and tile index, counted from the sequence's start, at position t; false past
  // the end.  A worker asks for positions in increasing order.
  __device__ __forceinline__ bool at(int t, int& entry, int& tile) {
    while (w > 0 && t >= base + c) {
      base += c;
      --w;
      while (c < count && tiles_at(c) >= w) ++c;
    }
    if (w <= 0) return false;
    const uint32_t key = __builtin_amdgcn_readfirstlane(tab[t - base]);
    entry = 0xffff - (int)(key & 0xffffu);
    tile = keys ? (int)(key >> 16) - w : w - 1;
    return true;
  }
};

// 1-D grids of the kernels that launch one workgroup per tile.  Consecutive workgroup ids go round
// the 8 XCDs, so XCD x = id % 8 takes the (sequence, kv-head) pairs x, x + 8, ... one after the
// other and the `per` tiles of a pair back to back: what every tile of a pair streams (its K/V, or
// the Q/dO of the group's q-heads) then stays in that XCD's L2.  Handed out tile by tile in grid
// order, the workgroups of one pair landed on all XCDs and drifted apart under a causal mask, and
// each streamed from HBM on its own (head dim 512, S = 4096: causal forward 3.39 ms against 2.31 for
// half of the non-causal one).  Returns false past the last pair.
__device__ __forceinline__ bool xcd_item(int id, int pairs, int per, int& pair, int& r) {
  const int xcd = id % kNumXcd, idx = id / kNumXcd;
  pair = xcd + kNumXcd * (idx / per);
  r = idx % per;
  return pair < pairs;
}
inline int xcd_grid(int pairs, int per) { return kNumXcd * ((pairs + kNumXcd - 1) / kNumXcd) * per; }
__host__ __device__ inline int nseq_of(const SeqArgs& s, int batch) {
  return s.num_seqlens != 0 ? (s.num_seqlens < 0 ? -s.num_seqlens : s.num_seqlens) : batch;
}

// _lse_offset, modules/flash/kernel/fwd_kernel_inner.py:38-43
__device__ __forceinline__ int64_t lse_offset(const SeqInfo& si, int h, int hq) {
  return ((int64_t)si.batch_index * hq + h) * si.lse_stride + si.q_start;
}

}  // namespace fa
