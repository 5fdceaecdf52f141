"""Philox-4x32-10 dropout mask, numpy restatement (test infrastructure only).

Follows the reference's call chain:
  fast_dropout_mask  modules/flash/kernel/dropout.py:41-71
  fast_philox        modules/flash/kernel/dropout.py:16-38
  threshold          modules/flash/kernel/fwd_kernel.py:195
  per-head base      modules/flash/kernel/fwd_kernel.py:405-407
Pinned by tests/golden/dropout_mask_reference.npz: masks that the reference's own
debug_simulate_encoded_softmax kernel (dropout_rng.py:86-126) wrote under Triton's CPU
interpreter (tests/golden/make_dropout_fixture.py), including a case where the int32
per-head term wraps.  The row term r * stride is computed exactly here; the reference
forms it from int32 pieces that depend on its tile size, which differs only when
Max_seqlen_q * cdiv(Max_seqlen_k, 4) reaches 2**31.
The generator itself lives in a third-party dependency (Triton
``tl.randint4x`` / ``philox_impl``, submodule third_party/triton, not vendored):
it is the published Philox-4x32 with 10 rounds (Salmon et al., SC'11) with
counter (lo32(ctr), hi32(ctr), 0, 0) and key (lo32(seed), hi32(seed)).
"""
import numpy as np

PHILOX_M0 = np.uint64(0xD2511F53)
PHILOX_M1 = np.uint64(0xCD9E8D57)
PHILOX_W0 = 0x9E3779B9
PHILOX_W1 = 0xBB67AE85
MASK32 = np.uint64(0xFFFFFFFF)


def philox4x32_10(c0, c1, c2, c3, k0, k1):
    """All arguments broadcastable uint32 arrays; returns four uint32 arrays."""
    c0 = np.asarray(c0, dtype=np.uint64) & MASK32
    c1 = np.asarray(c1, dtype=np.uint64) & MASK32
    c2 = np.asarray(c2, dtype=np.uint64) & MASK32
    c3 = np.asarray(c3, dtype=np.uint64) & MASK32
    k0 = int(k0) & 0xFFFFFFFF
    k1 = int(k1) & 0xFFFFFFFF
    for _ in range(10):
        p0 = PHILOX_M0 * c0          # 64-bit product of the 32-bit c0
        p1 = PHILOX_M1 * c2
        hi0, lo0 = p0 >> np.uint64(32), p0 & MASK32
        hi1, lo1 = p1 >> np.uint64(32), p1 & MASK32
        n0 = hi1 ^ c1 ^ np.uint64(k0)
        n1 = lo1
        n2 = hi0 ^ c3 ^ np.uint64(k1)
        n3 = lo0
        c0, c1, c2, c3 = n0, n1, n2, n3
        k0 = (k0 + PHILOX_W0) & 0xFFFFFFFF
        k1 = (k1 + PHILOX_W1) & 0xFFFFFFFF
    return (c0.astype(np.uint32), c1.astype(np.uint32),
            c2.astype(np.uint32), c3.astype(np.uint32))


def idropout_p(dropout_p):
    """int32 keep threshold, fp32 arithmetic as the kernels do it.

    fwd_kernel.py:195 ``((dropout_p - 0.5) * 0xFFFFFFFF).to(tl.int32)``: the
    integer literal is promoted to fp32, where it rounds to 2**32.
    """
    p = np.float32(dropout_p)
    x = np.float32(p - np.float32(0.5)) * np.float32(4294967296.0)
    # fptosi saturates in hardware; values here are always inside int32 range
    # for 0 <= p < 1 (p = 1 gives 2**31 which saturates to INT32_MAX).
    x = float(x)
    if x >= 2147483647.0:
        return 2147483647
    if x <= -2147483648.0:
        return -2147483648
    return int(x)   # truncation toward zero


def philox_words(seed, ctr):
    """Four 32-bit words per 64-bit counter in *column order*.

    ``tl.join(tl.join(r0,r1), tl.join(r2,r3)).reshape(M, 4N)`` (dropout.py:37)
    lays the words out as [r0, r2, r1, r3] along the row.
    Returns uint32 array of shape ctr.shape + (4,).
    """
    ctr = np.asarray(ctr, dtype=np.uint64)
    seed = int(seed) & 0xFFFFFFFFFFFFFFFF
    lo = ctr & MASK32
    hi = ctr >> np.uint64(32)
    w0, w1, w2, w3 = philox4x32_10(lo, hi, 0, 0, seed & 0xFFFFFFFF, seed >> 32)
    return np.stack([w0, w2, w1, w3], axis=-1)


def dropout_keep_mask(batch, num_heads, max_seqlen_q, max_seqlen_k, dropout_p,
                      seed, offset, rows=None, b_sel=None, h_sel=None):
    """Boolean keep mask [B, H, Sq, Sk] (or the selected slices).

    offset = philox_offset2 + *philox_offset1 (u64 wraparound).
    rows: optional (lo, hi) row range; b_sel/h_sel: optional index lists.
    """
    stride = (max_seqlen_k + 3) // 4
    thr = np.int32(idropout_p(dropout_p))
    bs = np.arange(batch) if b_sel is None else np.asarray(b_sel)
    hs = np.arange(num_heads) if h_sel is None else np.asarray(h_sel)
    r_lo, r_hi = (0, max_seqlen_q) if rows is None else rows
    rs = np.arange(r_lo, r_hi, dtype=np.uint64)
    cs = np.arange(stride, dtype=np.uint64)
    zh = (bs[:, None].astype(np.uint64) * np.uint64(num_heads) + hs[None, :].astype(np.uint64))
    with np.errstate(over='ignore'):
        # The per-head term is a product of int32 values in the reference (off_zh *
        # Max_seqlen_q * philox_offset_stride, fwd_kernel.py:405-407, dropout_rng.py:110):
        # it wraps modulo 2**32 and is sign-extended when it meets the uint64 base.
        head = (zh * np.uint64(max_seqlen_q) * np.uint64(stride)) & MASK32
        head = head.astype(np.uint32).view(np.int32).astype(np.int64).view(np.uint64)
        base = np.uint64(int(offset) & 0xFFFFFFFFFFFFFFFF) + head
        ctr = base[:, :, None, None] + rs[None, None, :, None] * np.uint64(stride) + cs[None, None, None, :]
    words = philox_words(seed, ctr)                       # [b,h,r,stride,4]
    words = words.reshape(len(bs), len(hs), len(rs), stride * 4)[..., :max_seqlen_k]
    return words.view(np.int32) > thr
