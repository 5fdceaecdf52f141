"""The kernels test an element's visibility with one unsigned comparison: the visible keys of a
query row (or the queries that see a key) form one range [lo, lo + rng], and `n` is inside iff
uint32(n - lo) <= rng, with an empty range mapped to an offset no element reaches
(fa_fwd_impl.h: prepare, fa_fwd_pipe.h: softmax_full).  This checks that form against the
element predicate of the reference (modules/flash/kernel/fwd_kernel_inner.py:140-160:
row - left <= key <= row + right, and key < seqlen_k) on the CPU, over window values of both
signs, the clamped sentinels and ragged sequence ends."""
import itertools

M32 = 0xFFFFFFFF


def _range_form(idx, centre, back, fwd, limit, live=True):
    lo = max(centre - back, 0)
    hi = min(centre + fwd, limit - 1)
    none = (not live) or hi < lo
    rng = 0 if none else hi - lo
    base = 0x40000000 if none else (0 - lo) & M32
    return ((base + idx) & M32) <= rng


def test_query_row_sees_key_range():
    wins = [-70, -33, -1, 0, 1, 5, 31, 32, 33, 64, 1 << 30]
    bad = 0
    for sk in (1, 2, 31, 32, 33, 64, 65):
        for left, right in itertools.product(wins, repeat=2):
            for row in range(0, 70, 3):
                for key in range(0, 70):
                    ref = key < sk and row - left <= key <= row + right
                    bad += ref != _range_form(key, row, left, right, sk)
    assert bad == 0


def test_key_seen_by_query_range():
    wins = [-33, -1, 0, 1, 31, 32, 33, 1 << 30]
    bad = 0
    for sq, sk in itertools.product((1, 31, 32, 33, 65), repeat=2):
        for left, right in itertools.product(wins, repeat=2):
            for key in range(0, 70, 3):
                for m in range(0, 70):
                    ref = m < sq and key < sk and m - left <= key <= m + right
                    bad += ref != _range_form(m, key, right, left, sq, live=key < sk)
    assert bad == 0
