"""Pins oracle/intervals.py by brute force on small shapes (no GPU)."""
import random

import torch

from oracle import intervals as iv
from oracle.fa_ref import visible_mask


def _blocks(lo, hi):
    return set(range(lo, hi + 1)) if lo <= hi else set()


def test_worked_examples():
    # causal top-left, BM=BN=128, S=4096, start_M=512
    wl, wr = iv.parse_window(3, iv.TOP_LEFT, iv.TOP_LEFT, 4096, 4096)
    assert (wl, wr) == (4096, 0)
    r = iv.calculate_intervals(True, wl, wr, 512, 4096, 4096, False, 128, 128)
    assert _blocks(r[0], r[1]) == set() and (r[2], r[3]) == (0, 3) and (r[4], r[5]) == (4, 4)
    # sliding window (1024, 0), BM=128 BN=64, S=8192, start_M=2048
    r = iv.calculate_intervals(True, 1024, 0, 2048, 8192, 8192, False, 128, 64)
    assert (r[0], r[1]) == (16, 17) and (r[2], r[3]) == (18, 31) and (r[4], r[5]) == (32, 33)
    # bottom-right sentinel
    assert iv.parse_window(3, iv.BOTTOM_RIGHT, iv.BOTTOM_RIGHT, 5, 9) == (5, 4)


def test_visible_mask_special_cases():
    # top-left causal == tril; bottom-right == tril(diagonal=Sk-Sq)
    for sq, sk in [(5, 5), (4, 9), (9, 4)]:
        tl_ = visible_mask(sq, sk, 3, iv.TOP_LEFT, iv.TOP_LEFT)
        assert torch.equal(tl_, torch.ones(sq, sk, dtype=torch.bool).tril())
        br = visible_mask(sq, sk, 3, iv.BOTTOM_RIGHT, iv.BOTTOM_RIGHT)
        assert torch.equal(br, torch.ones(sq, sk, dtype=torch.bool).tril(diagonal=sk - sq))
    w = visible_mask(8, 8, 3, 2, 1)
    exp = torch.ones(8, 8, dtype=torch.bool).tril(diagonal=1) & torch.ones(8, 8, dtype=torch.bool).triu(diagonal=-2)
    assert torch.equal(w, exp)


def test_intervals_brute_force():
    rnd = random.Random(1234)
    for _ in range(4000):
        BM = rnd.choice([16, 32, 64]); BN = rnd.choice([16, 32, 64])
        sq = rnd.randint(1, 200); sk = rnd.randint(1, 200)
        causal = rnd.random() < 0.8
        wl = rnd.randint(-40, 220); wr = rnd.randint(-40, 220)
        start_M = BM * rnd.randint(0, (sq - 1) // BM)
        mask_q = start_M + BM > sq
        lb_lo, lb_hi, fb_lo, fb_hi, rb_lo, rb_hi = iv.calculate_intervals(
            causal, wl, wr, start_M, sq, sk, mask_q, BM, BN)
        L, F, R = _blocks(lb_lo, lb_hi), _blocks(fb_lo, fb_hi), _blocks(rb_lo, rb_hi)
        assert not (L & F) and not (L & R) and not (F & R)
        assert all(b >= 0 for b in L | F | R)
        nblk = (sk + BN - 1) // BN
        for b in range(nblk + 1):
            vis = [iv.visible(m, n, sq, sk, causal, wl, wr)
                   for m in range(start_M, start_M + BM) for n in range(b * BN, b * BN + BN)]
            if any(vis):
                assert b in (L | F | R), (BM, BN, sq, sk, causal, wl, wr, start_M, b)
            if b in F:
                assert all(vis), (BM, BN, sq, sk, causal, wl, wr, start_M, b)
