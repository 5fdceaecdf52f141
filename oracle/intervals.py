"""Window parsing and K-block interval algebra (test infrastructure only).

Restates modules/flash/kernel/masked_load_store.py:
  div_rd               :25-27
  closed_interval_isect:9-14
  parse_window         :43-63
  calculate_intervals  :67-210
and the element predicate modules/flash/kernel/fwd_kernel_inner.py:127-150.
Plain Python integers; intended for small brute-force checks.
"""

TOP_LEFT = -2147483647
BOTTOM_RIGHT = -2147483646


def div_rd(x, y):
    # masked_load_store.py:25-27 -- floor division built from a truncating '//'
    d = abs(x) // abs(y)
    if (x < 0) != (y < 0):
        d = -d
    return d - 1 if d * y > x else d


def isect(a_s, a_e, b_s, b_e):
    # masked_load_store.py:9-14
    if (b_s > a_e or a_s > b_e) or (a_s > a_e):
        return -114, -514
    return max(a_s, b_s), min(a_e, b_e)


def parse_window(causal_type, Window_left, Window_right, seqlen_q, seqlen_k):
    # masked_load_store.py:43-63
    if causal_type == 1 or Window_left == TOP_LEFT:
        wl = seqlen_q
    elif causal_type == 2 or Window_left == BOTTOM_RIGHT:
        wl = seqlen_q
    else:
        wl = Window_left
    if causal_type == 1 or Window_right == TOP_LEFT:
        wr = 0
    elif causal_type == 2 or Window_right == BOTTOM_RIGHT:
        wr = seqlen_k - seqlen_q
    else:
        wr = Window_right
    return wl, wr


def visible(m, n, seqlen_q, seqlen_k, is_causal, wl, wr):
    # fwd_kernel_inner.py:137-148
    ok = m < seqlen_q and n < seqlen_k
    if is_causal:
        ok = ok and (m + wr >= n) and (m - wl <= n)
    return ok


def calculate_intervals(is_causal, wl, wr, start_M, seqlen_q, seqlen_k,
                        mask_on_seq_q, BLOCK_M, BLOCK_N):
    # masked_load_store.py:67-210; returns (lb_lo, lb_hi, fb_lo, fb_hi, rb_lo, rb_hi)
    masked_seq_k_block = seqlen_k // BLOCK_N
    if is_causal:
        isec_lo = start_M - wl
        isec_hi = min(start_M + BLOCK_M, seqlen_q) - wl
        lsec_lob = div_rd(isec_lo, BLOCK_N)
        lsec_hib = div_rd(isec_hi - 1, BLOCK_N)
        isec_lo = start_M + wr
        isec_hi = min(start_M + BLOCK_M, seqlen_q) + wr
        rsec_lob = div_rd(isec_lo, BLOCK_N)
        rsec_hib = div_rd(isec_hi - 1, BLOCK_N)
        vb_lo, vb_hi = 0, (seqlen_k - 1) // BLOCK_N
        lb_lo, lb_hi = isect(lsec_lob, lsec_hib, vb_lo, vb_hi)
        rb_lo, rb_hi = isect(rsec_lob, rsec_hib, vb_lo, vb_hi)
        ub_lo, ub_hi = isect(lsec_lob, lsec_hib, rsec_lob, rsec_hib)
        ub_empty = ub_lo > ub_hi
        if ub_empty and not mask_on_seq_q:
            fb_lo, fb_hi = isect(lsec_hib + 1, rsec_lob - 1, vb_lo, vb_hi)
        else:
            lb_lo, lb_hi = isect(lsec_lob, rsec_hib, vb_lo, vb_hi)
            fb_lo, fb_hi = -3, -4
            rb_lo, rb_hi = -3, -4
        if fb_lo * BLOCK_N < seqlen_k and seqlen_k < fb_hi * BLOCK_N + BLOCK_N:
            fb_hi = seqlen_k // BLOCK_N - 1
            rb_lo = masked_seq_k_block
            rb_hi = masked_seq_k_block
    else:
        lb_lo, lb_hi = -1, -2
        n_blocks = (seqlen_k + BLOCK_N - 1) // BLOCK_N
        if mask_on_seq_q:
            lb_lo, lb_hi = 0, n_blocks - 1
            fb_lo, fb_hi = -1, -2
            rb_lo, rb_hi = -1, -2
        else:
            fb_lo, fb_hi = 0, seqlen_k // BLOCK_N
            rb_lo, rb_hi = seqlen_k // BLOCK_N + 1, n_blocks - 1
        if fb_lo * BLOCK_N < seqlen_k and seqlen_k < fb_hi * BLOCK_N + BLOCK_N:
            fb_hi = seqlen_k // BLOCK_N - 1
            rb_lo = masked_seq_k_block
            rb_hi = masked_seq_k_block
    return lb_lo, lb_hi, fb_lo, fb_hi, rb_lo, rb_hi
