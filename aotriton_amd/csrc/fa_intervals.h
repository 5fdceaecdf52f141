// Window parsing and K-block ranges for one tile of rows; compiled for host and
// device.  Semantics of the element predicate and of the sentinels follow
// modules/flash/kernel/masked_load_store.py:43-63 and
// modules/flash/kernel/fwd_kernel_inner.py:137-148 of the reference; the range
// arithmetic is this library's own (rows past the end of the sequence need no
// mask here because every lane owns whole rows).
#pragma once
#include <stdint.h>

#if defined(__HIPCC__)
#define FA_HD __host__ __device__ inline
#define FA_HD_MEMBER __host__ __device__
#else
#define FA_HD inline
#define FA_HD_MEMBER
#endif

namespace fa {

constexpr int32_t kWindowTopLeft = -2147483647;
constexpr int32_t kWindowBottomRight = -2147483646;

struct Window { int32_t left, right; };

FA_HD Window parse_window(int causal_type, int32_t Wl, int32_t Wr, int32_t seqlen_q, int32_t seqlen_k) {
  Window w;
  if (causal_type == 1 || Wl == kWindowTopLeft) w.left = seqlen_q;
  else if (causal_type == 2 || Wl == kWindowBottomRight) w.left = seqlen_q;
  else w.left = Wl;
  if (causal_type == 1 || Wr == kWindowTopLeft) w.right = 0;
  else if (causal_type == 2 || Wr == kWindowBottomRight) w.right = seqlen_k - seqlen_q;
  else w.right = Wr;
  return w;
}

FA_HD int32_t floor_div(int32_t x, int32_t y) {  // y > 0
  int32_t d = x / y;
  return (d * y > x) ? d - 1 : d;
}

struct BlockRanges {
  // closed ranges of column-block indices; empty when lo > hi
  int32_t lb_lo, lb_hi;  // need per-element masking (left side)
  int32_t fb_lo, fb_hi;  // every element of every real row visible
  int32_t rb_lo, rb_hi;  // need per-element masking (right side / ragged end)
  int32_t lo, hi;        // union of the three ranges
  FA_HD_MEMBER bool is_full(int32_t j) const { return j >= fb_lo && j <= fb_hi; }
};

// Rows [start, min(start+BR, n_rows)), columns blocked by BC over n_cols.
// Row r sees column c iff r - left <= c <= r + right (when windowed) and c < n_cols.
FA_HD BlockRanges block_ranges(bool windowed, int32_t left, int32_t right, int32_t start,
                               int32_t n_rows, int32_t n_cols, int32_t BR, int32_t BC) {
  BlockRanges r;
  r.lb_lo = 0; r.lb_hi = -1; r.fb_lo = 0; r.fb_hi = -1; r.rb_lo = 0; r.rb_hi = -1;
  r.lo = 0; r.hi = -1;
  if (n_cols <= 0 || start >= n_rows) return r;
  int32_t last = (start + BR < n_rows ? start + BR : n_rows) - 1;
  int64_t c_min = 0, c_max = (int64_t)n_cols - 1;
  if (windowed) {
    int64_t lo = (int64_t)start - left, hi = (int64_t)last + right;
    if (lo > c_min) c_min = lo;
    if (hi < c_max) c_max = hi;
  }
  if (c_min > c_max) return r;
  int32_t j_lo = (int32_t)(c_min / BC), j_hi = (int32_t)(c_max / BC);
  r.lo = j_lo; r.hi = j_hi;
  int32_t f_lo = j_lo, f_hi = n_cols / BC - 1;   // block must lie inside n_cols
  if (f_hi > j_hi) f_hi = j_hi;
  if (windowed) {
    // left edge: first column of the block visible to the last row
    int64_t need = (int64_t)last - left;          // c >= need
    if (need > 0) {
      int64_t b = (need + BC - 1) / BC;
      if (b > f_lo) f_lo = (int32_t)(b > 0x3fffffff ? 0x3fffffff : b);
    }
    // right edge: last column of the block visible to the first row
    int64_t lim = (int64_t)start + right + 1;     // (j+1)*BC <= lim
    int64_t b = lim >= 0 ? lim / BC - 1 : -1;
    if (b < f_hi) f_hi = (int32_t)b;
  }
  if (f_lo > f_hi) {
    r.lb_lo = j_lo; r.lb_hi = j_hi;
    return r;
  }
  r.lb_lo = j_lo; r.lb_hi = f_lo - 1;
  r.fb_lo = f_lo; r.fb_hi = f_hi;
  r.rb_lo = f_hi + 1; r.rb_hi = j_hi;
  return r;
}

// int32 keep threshold: fptosi(fp32(fp32(p) - 0.5f) * 2^32), as the reference
// kernels compute it (modules/flash/kernel/fwd_kernel.py:195).
FA_HD int32_t dropout_threshold(float p) {
  float x = (p - 0.5f) * 4294967296.0f;
  if (x >= 2147483648.0f) return 2147483647;
  if (x <= -2147483648.0f) return (int32_t)(-2147483647 - 1);
  return (int32_t)x;
}

}  // namespace fa
