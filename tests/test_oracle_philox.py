"""Pins oracle/philox.py against known-answer vectors (no GPU)."""
import json
import os

import numpy as np

from oracle import philox

GOLD = json.load(open(os.path.join(os.path.dirname(__file__), 'golden', 'philox_seed1234.json')))


def _h(xs):
    return [int(x, 16) for x in xs]


def test_random123_known_answers():
    for kat in GOLD['random123_kat']:
        c = _h(kat['ctr']); k = _h(kat['key'])
        out = philox.philox4x32_10(c[0], c[1], c[2], c[3], k[0], k[1])
        assert [int(x) for x in out] == _h(kat['out'])


def test_word_order_seed1234():
    raw = philox.philox4x32_10(0, 0, 0, 0, 0x1234, 0)
    assert [int(x) for x in raw] == _h(GOLD['raw_counter0'])
    for ctr, row in GOLD['rows'].items():
        w = philox.philox_words(0x1234, np.uint64(int(ctr)))
        assert [int(x) for x in w] == _h(row), ctr


def test_threshold_fp32():
    for p, v in GOLD['idropout_p'].items():
        assert philox.idropout_p(float(p)) == v
    # the double-precision host helper of the JIT harness gives a different
    # value and must not be what we compute
    assert philox.idropout_p(0.1) != -1717986918


def test_mask_equals_the_reference_kernels_mask():
    """The oracle's whole-tensor mask against what the reference's own
    debug_simulate_encoded_softmax kernel wrote (modules/flash/kernel/dropout_rng.py:86-126,
    run under Triton's CPU interpreter by tests/golden/make_dropout_fixture.py): several batch
    elements and heads, more than one 64-row tile, key counts off the multiples of 4 and 32,
    a seed above 2**32, offset1 and offset2 both non-zero, a counter that carries into its
    high word, and a per-head term that wraps in int32."""
    from tests._util import reference_dropout_fixture
    cases = reference_dropout_fixture()
    assert len(cases) == 5
    for c in cases:
        m = philox.dropout_keep_mask(c['B'], c['H'], c['max_sq'], c['Sk'], c['p'], c['seed'],
                                     c['off1'] + c['off2'], rows=(0, c['Sq']))
        assert np.array_equal(m, c['keep']), (c['B'], c['H'], c['Sq'], c['Sk'])
    # the wrapping case really wraps: exact 64-bit arithmetic gives another mask for heads 1, 2
    c = cases[-1]
    assert c['H'] * c['max_sq'] * ((c['Sk'] + 3) // 4) >= 2 ** 31


def test_mask_matches_per_element_closed_form():
    B, H, Sq, Sk, p, seed, off = 2, 3, 5, 10, 0.1, 0x1234, 7
    mask = philox.dropout_keep_mask(B, H, Sq, Sk, p, seed, off)
    assert mask.shape == (B, H, Sq, Sk)
    thr = philox.idropout_p(p)
    stride = (Sk + 3) // 4
    for b in range(B):
        for h in range(H):
            for r in range(Sq):
                for c in range(Sk):
                    ctr = off + (b * H + h) * Sq * stride + r * stride + c // 4
                    w = philox.philox4x32_10(ctr & 0xFFFFFFFF, ctr >> 32, 0, 0, seed & 0xFFFFFFFF, seed >> 32)
                    word = [w[0], w[2], w[1], w[3]][c % 4]
                    keep = int(np.int32(np.uint32(word))) > thr
                    assert bool(mask[b, h, r, c]) == keep


def test_first_row_of_config5_is_the_probe_words():
    # seed 0x1234, offset 0, b=h=0, row 0, columns 0..7 are counters 0 and 1
    thr = philox.idropout_p(0.1)
    mask = philox.dropout_keep_mask(1, 1, 1, 8, 0.1, 0x1234, 0)[0, 0, 0]
    words = _h(GOLD['rows']['0']) + _h(GOLD['rows']['1'])
    exp = [int(np.int32(np.uint32(w))) > thr for w in words]
    assert mask.tolist() == exp


def test_counter_carry_into_high_word():
    off = (1 << 32) - 2
    m = philox.dropout_keep_mask(1, 1, 1, 16, 0.5, 99, off)[0, 0, 0]
    exp = []
    for c in range(16):
        ctr = off + c // 4
        w = philox.philox4x32_10(ctr & 0xFFFFFFFF, ctr >> 32, 0, 0, 99, 0)
        word = [w[0], w[2], w[1], w[3]][c % 4]
        exp.append(int(np.int32(np.uint32(word))) > 0)
    assert m.tolist() == exp


def test_keep_rate():
    m = philox.dropout_keep_mask(1, 2, 256, 256, 0.1, 0x1234, 0)
    assert abs(m.mean() - 0.9) < 0.01
    m = philox.dropout_keep_mask(1, 2, 256, 256, 0.5, 0x1BF52, 0x1D4000 + 0xB42)
    assert abs(m.mean() - 0.5) < 0.01
