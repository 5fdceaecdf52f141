"""GPU parity tests for the packed-sequence (compact varlen) path, the dropout
mask (bit-exact against the Philox closed form), the reference's known-answer
tests, and size-independent properties at the full benchmark sizes."""
import math

import numpy as np
import pytest
import torch

from _util import FUDGE, LSE_ATOL, check, make_inputs

pytestmark = pytest.mark.gpu
DEV = 'cuda'


def _u64(x):
    return torch.tensor([int(np.uint64(x).astype(np.int64))], dtype=torch.int64, device=DEV).view(torch.uint64)


@pytest.mark.parametrize('dtype', [torch.bfloat16, torch.float16])
@pytest.mark.parametrize('D', [64, 128])
@pytest.mark.parametrize('causal', [False, True])
@pytest.mark.parametrize('backend', [0, 1])
def test_compact_varlen_gqa(dtype, D, causal, backend):
    # seqlens drawn as the reference does (tests/test_varlen.py:34-47)
    from aotriton_amd import flash
    from aotriton_amd.autograd import attention_varlen, AttentionExtraArgs
    from oracle import fa_ref
    np.random.seed(8139)
    lens = np.random.choice([4, 8, 63, 64, 128, 143, 301], size=6)
    T = int(lens.sum())
    Hq, Hk = 8, 2
    cu = [0] + np.cumsum(lens).tolist()
    g = torch.Generator().manual_seed(5)
    # THD storage viewed as (1, H, T, D) (tests/_common_test.py:677-678)
    mk = lambda H: torch.randn(1, T, H, D, generator=g).to(dtype).to(DEV).transpose(1, 2)
    q, k, v, do = mk(Hq), mk(Hk), mk(Hk), mk(Hq)
    sm = 1.0 / math.sqrt(D)
    qg, kg, vg = [t.clone().requires_grad_() for t in (q, k, v)]
    ext = AttentionExtraArgs(return_logsumexp=True, fillnan=True, bwd_backend=backend)
    o, _, L = attention_varlen(qg, kg, vg, lens, lens, causal, sm, 0.0, ext)
    o.backward(do)
    torch.cuda.synchronize()
    assert L.shape == (Hq, T)
    ct, wl, wr = flash.translate_causal(causal)
    f = lambda t: t.float()
    ro, rl = fa_ref.varlen_fwd_ref(f(q), f(k), f(v), cu, cu, sm, ct, wl, wr)
    lo, ll = fa_ref.varlen_fwd_ref(q, k, v, cu, cu, sm, ct, wl, wr)
    check('out', o, ro, lo, FUDGE['out'])
    assert (L - rl).abs().max().item() <= LSE_ATOL
    rg = fa_ref.varlen_bwd_ref(f(q), f(k), f(v), cu, cu, sm, ro, f(do), rl, ct, wl, wr)
    lg = fa_ref.varlen_bwd_ref(q, k, v, cu, cu, sm, lo, do, ll.to(dtype), ct, wl, wr)
    check('dq', qg.grad, rg[0], lg[0], FUDGE['dq'])
    check('dk', kg.grad, rg[1], lg[1], FUDGE['dk'])
    check('dv', vg.grad, rg[2], lg[2], FUDGE['dv'])


def _run_varlen_case(lq, lk, Hq, Hk, D, dtype, causal, backend, p=0.0, seed=11):
    """Packed sequences against the dense oracle, sequence by sequence.  Rows without a key
    give O = 0, LSE = +inf, dQ = 0; keys without a query give dK = dV = 0."""
    from aotriton_amd import flash
    from aotriton_amd.autograd import attention_varlen, AttentionExtraArgs
    from oracle import fa_ref, philox
    lq, lk = np.asarray(lq), np.asarray(lk)
    cq = [0] + np.cumsum(lq).tolist()
    ck = [0] + np.cumsum(lk).tolist()
    g = torch.Generator().manual_seed(seed)
    mk = lambda H, T: torch.randn(1, T, H, D, generator=g).to(dtype).to(DEV).transpose(1, 2)
    q, do = mk(Hq, cq[-1]), mk(Hq, cq[-1])
    k, v = mk(Hk, ck[-1]), mk(Hk, ck[-1])
    sm = 1.0 / math.sqrt(D)
    qg, kg, vg = [t.clone().requires_grad_() for t in (q, k, v)]
    ext = AttentionExtraArgs(return_logsumexp=True, fillnan=True, bwd_backend=backend)
    o, _, L = attention_varlen(qg, kg, vg, lq, lk, causal, sm, p, ext)
    o.backward(do)
    torch.cuda.synchronize()
    ct, wl, wr = flash.translate_causal(causal)
    keep = None
    if p > 0.0:      # counters use the sequence index and the maximal lengths (fwd_kernel.py:405-407)
        keep = philox.dropout_keep_mask(len(lq), Hq, int(lq.max()), int(lk.max()), p, ext.philox_seed,
                                        ext.philox_offset1 + ext.philox_offset2)
    hp = torch.float64 if dtype == torch.float32 else torch.float32
    f = lambda t: t.to(hp)
    for i in range(len(lq)):
        sq, sk = slice(cq[i], cq[i + 1]), slice(ck[i], ck[i + 1])
        if lq[i] == 0:
            assert torch.count_nonzero(kg.grad[:, :, sk]) == 0 and torch.count_nonzero(vg.grad[:, :, sk]) == 0
            continue
        if lk[i] == 0:
            assert torch.count_nonzero(o[:, :, sq]) == 0 and bool(torch.isposinf(L[:, sq]).all())
            assert torch.count_nonzero(qg.grad[:, :, sq]) == 0
            continue
        km = None if keep is None else torch.from_numpy(keep[i:i + 1, :, :lq[i], :lk[i]]).to(DEV)
        ro, rl, _ = fa_ref.attn_fwd_ref(f(q[:, :, sq]), f(k[:, :, sk]), f(v[:, :, sk]), None, sm, ct, wl, wr, p, km)
        lo, ll, _ = fa_ref.attn_fwd_ref(q[:, :, sq], k[:, :, sk], v[:, :, sk], None, sm, ct, wl, wr, p, km)
        check(f'out[{i}]', o[:, :, sq], ro, lo, FUDGE['out'])
        live = torch.isfinite(rl[0])
        assert torch.equal(torch.isinf(L[:, sq]), ~live)
        assert not bool(live.any()) or (L[:, sq][live] - rl[0][live]).abs().max().item() <= LSE_ATOL
        rg = fa_ref.attn_bwd_ref(f(q[:, :, sq]), f(k[:, :, sk]), f(v[:, :, sk]), None, sm, ro, f(do[:, :, sq]), rl,
                                 ct, wl, wr, p, km)
        lg = fa_ref.attn_bwd_ref(q[:, :, sq], k[:, :, sk], v[:, :, sk], None, sm, lo, do[:, :, sq],
                                 ll.to(dtype), ct, wl, wr, p, km)
        check(f'dq[{i}]', qg.grad[:, :, sq], rg[0], lg[0], FUDGE['dq'])
        check(f'dk[{i}]', kg.grad[:, :, sk], rg[1], lg[1], FUDGE['dk'])
        check(f'dv[{i}]', vg.grad[:, :, sk], rg[2], lg[2], FUDGE['dv'])
    for t in (o, qg.grad, kg.grad, vg.grad):
        assert not bool(torch.isnan(t).any())


@pytest.mark.parametrize('dtype', [torch.bfloat16, torch.float32])
@pytest.mark.parametrize('causal', [False, True])
@pytest.mark.parametrize('backend', [0, 1])
def test_compact_varlen_with_empty_sequences(dtype, causal, backend):
    # sequences without queries, without keys and without both among ordinary ones, and
    # query and key lengths that differ
    _run_varlen_case([5, 0, 70, 0, 33, 130], [9, 64, 0, 0, 33, 40], 4, 2, 64, dtype, causal, backend)


@pytest.mark.parametrize('nseq,hk', [(67, 1), (300, 2), (4200, 1)])
@pytest.mark.parametrize('causal', [True, (40, 0)])
def test_many_packed_sequences(nseq, hk, causal):
    # The dK/dV kernel sorts the (sequence, kv-head) entries of an XCD by length into an LDS table of
    # 512 entries and walks the valid key tiles heaviest first; beyond 512 entries per XCD it keeps the
    # dense list.  9, 75 and 525 entries per XCD, lengths from empty to several key tiles, equal
    # lengths among them.
    rng = np.random.default_rng(nseq)
    hi = 700 if nseq < 100 else (300 if nseq < 1000 else 40)
    lens = rng.integers(0, hi, size=nseq)
    lens[::7] = 129
    lens[3] = 0
    _run_varlen_case(lens, lens, 2 * hk, hk, 64, torch.bfloat16, causal, 0)


@pytest.mark.parametrize('D,dtype', [(37, torch.bfloat16), (203, torch.float16), (7, torch.float32)])
def test_compact_varlen_head_dim_no_multiple_of_8(D, dtype, with_and_without_workspace):
    # packed sequences at any head dim (modules/flash/csrc/attn_fwd.cc:76-82): through packed copies on the
    # MFMA kernels, and on the element-wise kernels
    _run_varlen_case([5, 0, 70, 33], [9, 64, 41, 33], 4, 2, D, dtype, True, 0, p=0.1)


def _sampled_varlen_cases(n=40, seed=4242):
    """Seeded packed-sequence cases: 1-6 sequences of 0-300 tokens (the reference draws its
    lengths from a fixed list, tests/test_varlen.py:34-47), key lengths that differ from the
    query lengths in a third of the cases, GQA, head dims of the reference's list, dropout,
    windows and both alignments."""
    import random
    from aotriton_amd.flash import CausalType
    rnd = random.Random(seed)
    cases = []
    for i in range(n):
        ns = rnd.randint(1, 6)
        pick = lambda: rnd.choice([0, 1, 4, 8, 63, 64, 65, 128, 143, 257, 301])
        lq = [pick() for _ in range(ns)]
        lk = [pick() for _ in range(ns)] if rnd.random() < 0.33 else list(lq)
        if sum(lq) == 0: lq[0] = 17
        if sum(lk) == 0: lk[0] = 17
        Hq, Hk = rnd.choice([(4, 4), (8, 2), (6, 1), (2, 2)])
        D = rnd.choice([16, 40, 64, 96, 128, 192, 256, 408])
        dtype = rnd.choice([torch.float16, torch.bfloat16, torch.float32])
        r = rnd.random()
        causal = False if r < 0.3 else (True if r < 0.6 else
                                        ((rnd.randint(-3, 200), rnd.randint(-3, 200)) if r < 0.8 else CausalType.BOTTOM_RIGHT))
        p = rnd.choice([0.0, 0.0, 0.3])
        if p > 0.0:
            # With a single key dS = P (dP - delta) is exactly zero, and the low-precision oracle
            # rounds dP and delta alike, so its error (the yardstick) is ~0, while a kernel that
            # takes delta from the rounded O keeps that rounding in dQ.  Two keys avoid the case.
            lq = [2 if x == 1 else x for x in lq]
            lk = [2 if x == 1 else x for x in lk]
        backend = 0 if (dtype == torch.float32 or D > 256) else rnd.choice([0, 1])
        cases.append((tuple(lq), tuple(lk), Hq, Hk, D, dtype, causal, backend, p))
    return cases


@pytest.mark.parametrize('case', _sampled_varlen_cases(), ids=lambda c: f"n{len(c[0])}-h{c[2]}_{c[3]}-d{c[4]}-{str(c[5])[6:]}-be{c[7]}-p{c[8]}")
def test_sampled_packed_sequences(case):
    lq, lk, Hq, Hk, D, dtype, causal, backend, p = case
    _run_varlen_case(lq, lk, Hq, Hk, D, dtype, causal, backend, p)


def test_compact_varlen_fp32():
    # packed sequences through the fp32 kernels; oracle in fp64 against fp32
    from aotriton_amd import flash
    from aotriton_amd.autograd import attention_varlen, AttentionExtraArgs
    from oracle import fa_ref
    lens = np.array([5, 64, 131, 17])
    T = int(lens.sum())
    Hq, Hk, D = 4, 2, 64
    cu = [0] + np.cumsum(lens).tolist()
    g = torch.Generator().manual_seed(6)
    mk = lambda H: torch.randn(1, T, H, D, generator=g).to(DEV).transpose(1, 2)
    q, k, v, do = mk(Hq), mk(Hk), mk(Hk), mk(Hq)
    sm = 1.0 / math.sqrt(D)
    qg, kg, vg = [t.clone().requires_grad_() for t in (q, k, v)]
    o, _, L = attention_varlen(qg, kg, vg, lens, lens, True, sm, 0.0,
                               AttentionExtraArgs(return_logsumexp=True, fillnan=True, bwd_backend=0))
    o.backward(do)
    torch.cuda.synchronize()
    ct, wl, wr = flash.translate_causal(True)
    f = lambda t: t.double()
    ro, rl = fa_ref.varlen_fwd_ref(f(q), f(k), f(v), cu, cu, sm, ct, wl, wr)
    lo, ll = fa_ref.varlen_fwd_ref(q, k, v, cu, cu, sm, ct, wl, wr)
    check('out', o, ro, lo, FUDGE['out'])
    assert (L - rl).abs().max().item() <= LSE_ATOL
    rg = fa_ref.varlen_bwd_ref(f(q), f(k), f(v), cu, cu, sm, ro, f(do), rl, ct, wl, wr)
    lg = fa_ref.varlen_bwd_ref(q, k, v, cu, cu, sm, lo, do, ll, ct, wl, wr)
    check('dq', qg.grad, rg[0], lg[0], FUDGE['dq'])
    check('dk', kg.grad, rg[1], lg[1], FUDGE['dk'])
    check('dv', vg.grad, rg[2], lg[2], FUDGE['dv'])


def test_varlen_dropout_mask_uses_sequence_index_and_max_seqlens():
    from aotriton_amd.autograd import attention_varlen, AttentionExtraArgs
    from oracle import fa_ref, philox
    lens = np.array([37, 128, 5, 90])
    T = int(lens.sum()); H = 4; D = 64
    cu = [0] + np.cumsum(lens).tolist()
    g = torch.Generator().manual_seed(1)
    mk = lambda: torch.randn(1, H, T, D, generator=g).to(torch.float16).to(DEV)
    q, k, v = mk(), mk(), mk()
    ext = AttentionExtraArgs(return_encoded_softmax=True, return_logsumexp=True)
    p = 0.3
    o, enc, L = attention_varlen(q, k, v, lens, lens, True, 0.125, p, ext)
    torch.cuda.synchronize()
    mq = int(lens.max())
    keep = philox.dropout_keep_mask(len(lens), H, mq, mq, p, ext.philox_seed, ext.philox_offset1 + ext.philox_offset2)
    assert np.array_equal((enc >= 0).cpu().numpy(), keep)
    keeps = [torch.from_numpy(keep[i:i + 1, :, :lens[i], :lens[i]]).to(DEV) for i in range(len(lens))]
    ro, _ = fa_ref.varlen_fwd_ref(q.float(), k.float(), v.float(), cu, cu, 0.125, 3, -2147483647, -2147483647, p, keeps)
    lo, _ = fa_ref.varlen_fwd_ref(q, k, v, cu, cu, 0.125, 3, -2147483647, -2147483647, p, keeps)
    check('out', o, ro, lo, FUDGE['out'])


@pytest.mark.parametrize('dtype', [torch.float16, torch.bfloat16, torch.float32])
@pytest.mark.parametrize('shape', [(2, 3, 70, 131), (1, 2, 64, 32), (1, 1, 1, 5)])
@pytest.mark.parametrize('p', [0.1, 0.5])
@pytest.mark.parametrize('state', [(0x1234, (1 << 32) - 3, 9), (0xDEADBEEF12345678, 0x100000005, (1 << 40) + 7),
                                   ((1 << 64) - 1, (1 << 63) + 11, (1 << 63) - 5)], ids=['carry', 'wide', 'wrap'])
def test_encoded_softmax_is_bit_exact(dtype, shape, p, state):
    # seeds and offsets that use all 64 bits; a counter that carries into its high word, and
    # offset1 + offset2 that wraps around 2^64
    from aotriton_amd import flash
    from oracle import philox
    B, H, Sq, Sk = shape
    sk8 = (Sk + 7) // 8 * 8
    r = torch.zeros(B, H, Sq, sk8, dtype=dtype, device=DEV)[..., :Sk]
    seed, off1, off2 = state
    assert flash.debug_simulate_encoded_softmax(r, p, _u64(seed), _u64(off1), off2) == flash.hipError_t.hipSuccess
    torch.cuda.synchronize()
    keep = philox.dropout_keep_mask(B, H, Sq, Sk, p, seed, off1 + off2)
    assert set(torch.unique(r.float()).tolist()) <= {0.5, -0.5}
    assert np.array_equal((r >= 0).cpu().numpy(), keep)


def test_mask_equals_the_reference_kernels_mask():
    """debug_simulate_encoded_softmax and the forward's own encoded_softmax against the masks
    that the reference's kernel wrote (tests/golden/dropout_mask_reference.npz, see
    tests/golden/make_dropout_fixture.py)."""
    from aotriton_amd import flash
    from aotriton_amd.autograd import attention, AttentionExtraArgs
    from _util import reference_dropout_fixture
    for c in reference_dropout_fixture():
        if c['max_sq'] != c['Sq']:
            continue   # the int32-wrap case needs 2**27 rows: covered at full size below
        B, H, Sq, Sk = c['B'], c['H'], c['Sq'], c['Sk']
        sk8 = (Sk + 7) // 8 * 8
        for dtype in (torch.float16, torch.bfloat16, torch.float32):
            r = torch.zeros(B, H, Sq, sk8, dtype=dtype, device=DEV)[..., :Sk]
            assert flash.debug_simulate_encoded_softmax(r, c['p'], _u64(c['seed']), _u64(c['off1']), c['off2']) == 0
            assert np.array_equal((r >= 0).cpu().numpy(), c['keep'])
        # the mask the forward kernel applies (returned through encoded_softmax)
        q, k, v, _, _ = make_inputs(B, H, H, Sq, Sk, 64, torch.float16, DEV, seed=3)
        ext = AttentionExtraArgs(return_encoded_softmax=True, philox_seed=c['seed'], philox_offset1=c['off1'],
                                 philox_offset2=c['off2'])
        _, enc, _ = attention(q, k, v, None, False, 0.125, c['p'], ext)
        assert np.array_equal((enc >= 0).cpu().numpy(), c['keep'])


def test_per_head_counter_term_wraps_in_int32():
    """B1 H2 Sq 2^20 Sk 8192: head 1's term (1 * 2^20 * 2048 = 2^31) wraps to -2^31 as in the
    reference (fwd_kernel.py:405-407; pinned on the CPU by the fixture's wrapping case)."""
    from aotriton_amd import flash
    from oracle import philox
    H, Sq, Sk = 2, 1 << 20, 8192
    r = torch.empty(1, H, Sq, Sk, dtype=torch.float16, device=DEV)
    off2 = 1 << 40
    assert flash.debug_simulate_encoded_softmax(r, 0.5, _u64(0x1234), _u64(5), off2) == 0
    for h in range(H):
        for m in (0, 1, 4097, Sq - 1):
            exp = philox.dropout_keep_mask(1, H, Sq, Sk, 0.5, 0x1234, 5 + off2, rows=(m, m + 1), h_sel=[h])[0, 0, 0]
            assert np.array_equal((r[0, h, m] >= 0).cpu().numpy(), exp), (h, m)
    # what exact 64-bit arithmetic would have given for head 1 is a different row
    unwrapped = philox.dropout_keep_mask(1, 1, 1, Sk, 0.5, 0x1234, 5 + off2 + (1 << 31))[0, 0, 0]
    assert not np.array_equal((r[0, 1, 0] >= 0).cpu().numpy(), unwrapped)
    del r
    torch.cuda.empty_cache()


def test_config5_mask_first_words_and_popcount():
    """Mask of the benchmark configuration with dropout (seed 0x1234, offset 0, p=0.1, 8192x8192) on sampled
    (b, h) slices: bit-exact rows against the oracle and a keep-rate check."""
    from aotriton_amd import flash
    from oracle import philox
    S = 8192
    B, H = 2, 16
    r = torch.empty(1, 1, S, S, dtype=torch.float16, device=DEV)
    # the (b, h) slice is selected through the offset: base + (b*H + h) * S * S/4
    for (b, h) in [(0, 0), (1, 7)]:
        off = (b * H + h) * S * (S // 4)
        assert flash.debug_simulate_encoded_softmax(r, 0.1, _u64(0x1234), _u64(0), off) == 0
        got = (r[0, 0] >= 0)
        rows = (0, 1, 4095, 8191)
        for m in rows:
            exp = philox.dropout_keep_mask(B, H, S, S, 0.1, 0x1234, 0, rows=(m, m + 1), b_sel=[b], h_sel=[h])[0, 0, 0]
            assert np.array_equal(got[m].cpu().numpy(), exp)
        rate = got.float().mean().item()
        assert abs(rate - 0.9) < 2e-4, rate


@pytest.mark.parametrize('dtype', [torch.float16, torch.bfloat16])
def test_logsumexp_scaling_known_answer(dtype):
    # modules/flash/tests/_core_test_backward.py:333-351, embedded in a built head dim
    from aotriton_amd.autograd import attention, AttentionExtraArgs
    D = 64
    e = torch.zeros(1, 1, 16, D, dtype=dtype, device=DEV)
    e[0, 0, :, :16] = torch.eye(16, dtype=dtype, device=DEV)
    o, _, L = attention(e, e, e, None, False, 1.0 / math.sqrt(16), 0.0, AttentionExtraArgs(return_logsumexp=True))
    assert torch.allclose(L, torch.full_like(L, 2.79018449783325195))


@pytest.mark.parametrize('D', [64, 128, 256])
def test_large_bf16_values_do_not_give_nan(D):
    # modules/flash/tests/_core_test_backward.py:353-374
    from aotriton_amd.autograd import attention
    x = torch.full((1, 1, 1, D), 133120.0, dtype=torch.bfloat16, device=DEV)
    o, _, _ = attention(x, x.clone(), x.clone(), None, False, 0.125, 0.0)
    assert not torch.isnan(o).any()


@pytest.mark.parametrize('causal', [True, (3, 2)])
def test_sm_scale_zero_with_masks(causal):
    # -inf * 0 must not become NaN (fwd_kernel_inner.py:207-211)
    from aotriton_amd import flash
    from aotriton_amd.autograd import attention, AttentionExtraArgs
    from oracle import fa_ref
    q, k, v, _, do = make_inputs(1, 2, 2, 77, 91, 64, torch.float16, DEV)
    qg, kg, vg = [t.clone().requires_grad_() for t in (q, k, v)]
    o, _, L = attention(qg, kg, vg, None, causal, 0.0, 0.0, AttentionExtraArgs(return_logsumexp=True))
    o.backward(do)
    ct, wl, wr = flash.translate_causal(causal)
    ro, rl, _ = fa_ref.attn_fwd_ref(q.float(), k.float(), v.float(), None, 0.0, ct, wl, wr)
    lo, _, _ = fa_ref.attn_fwd_ref(q, k, v, None, 0.0, ct, wl, wr)
    check('out', o, ro, lo, FUDGE['out'])
    for t in (qg.grad, kg.grad, vg.grad):
        assert torch.isfinite(t).all()


def test_headline_size_properties():
    """B4 H32 S4096 D128 bf16 causal: properties that hold at any size.
    (1) row 0 of every head attends only to key 0: O[0] == V[0], LSE[0] == s00;
    (2) a sampled head matches the oracle; (3) the backward's dV column sums:
    sum_n dV[n] == sum_m dO[m] (rows of P sum to one)."""
    from aotriton_amd.autograd import attention, AttentionExtraArgs
    from oracle import fa_ref
    B, H, S, D = 4, 32, 4096, 128
    g = torch.Generator(device='cpu').manual_seed(1234)
    mk = lambda: torch.randn(B, H, S, D, generator=g).to(torch.bfloat16).to(DEV)
    q, k, v, do = mk(), mk(), mk(), mk()
    sm = 1.0 / math.sqrt(D)
    for backend in (0, 1):
        qg, kg, vg = [t.clone().requires_grad_() for t in (q, k, v)]
        o, _, L = attention(qg, kg, vg, None, True, sm, 0.0,
                            AttentionExtraArgs(return_logsumexp=True, fillnan=True, bwd_backend=backend))
        o.backward(do)
        torch.cuda.synchronize()
        assert torch.equal(o[:, :, 0], v[:, :, 0])
        s00 = (q[:, :, 0].float() * k[:, :, 0].float()).sum(-1) * sm
        assert torch.allclose(L.view(B, H, S)[:, :, 0], s00, atol=1e-4, rtol=1e-5)
        assert not torch.isnan(o).any() and not torch.isnan(L).any()
        for (b, h) in [(0, 0), (3, 31)]:
            sl = lambda t: t[b:b + 1, h:h + 1]
            ro, rl, _ = fa_ref.attn_fwd_ref(sl(q).float(), sl(k).float(), sl(v).float(), None, sm, 3, -2147483647, -2147483647)
            lo, ll, _ = fa_ref.attn_fwd_ref(sl(q), sl(k), sl(v), None, sm, 3, -2147483647, -2147483647)
            check('out', sl(o), ro, lo, FUDGE['out'])
            assert (L.view(B, H, S)[b, h] - rl[0, 0]).abs().max().item() <= LSE_ATOL
            rg = fa_ref.attn_bwd_ref(sl(q).float(), sl(k).float(), sl(v).float(), None, sm, ro, sl(do).float(), rl,
                                     3, -2147483647, -2147483647)
            lg = fa_ref.attn_bwd_ref(sl(q), sl(k), sl(v), None, sm, lo, sl(do), ll.to(torch.bfloat16), 3,
                                     -2147483647, -2147483647)
            check('dq', sl(qg.grad), rg[0], lg[0], FUDGE['dq'])
            check('dk', sl(kg.grad), rg[1], lg[1], FUDGE['dk'])
            check('dv', sl(vg.grad), rg[2], lg[2], FUDGE['dv'])
        colsum = vg.grad.float().sum(dim=2)
        dosum = do.float().sum(dim=2)
        assert (colsum - dosum).abs().max().item() < 0.5, (colsum - dosum).abs().max().item()


@pytest.mark.parametrize('backend', [0, 1])
def test_sequence_of_100k_tokens(backend):
    """B1 Hq4 Hkv2 S100003 D128 bf16 causal.  Blocks of query rows are compared with the
    oracle run on those rows against the keys they see (bottom-right aligned causal mask of
    the slice = the rows' causal mask); the last block's dK/dV rows are complete from the
    last block of queries alone; sum_n dV[n] == sum_m dO[m]."""
    from aotriton_amd.autograd import attention, AttentionExtraArgs
    from oracle import fa_ref
    B, Hq, Hk, S, D = 1, 4, 2, 100003, 128
    g = torch.Generator(device=DEV).manual_seed(78)
    mk = lambda H: torch.randn(B, H, S, D, generator=g, device=DEV, dtype=torch.bfloat16)
    q, k, v, do = mk(Hq), mk(Hk), mk(Hk), mk(Hq)
    sm = 1.0 / math.sqrt(D)
    qg, kg, vg = [t.clone().requires_grad_() for t in (q, k, v)]
    o, _, L = attention(qg, kg, vg, None, True, sm, 0.0,
                        AttentionExtraArgs(return_logsumexp=True, fillnan=True, bwd_backend=backend))
    o.backward(do)
    torch.cuda.synchronize()
    for t in (o, L, qg.grad, kg.grad, vg.grad):
        assert not bool(torch.isnan(t).any())
    BR = -2147483646
    for i0, i1 in [(0, 64), (65500, 65600), (S - 64, S)]:
        qs, dos = q[:, :, i0:i1], do[:, :, i0:i1]
        ks, vs = k[:, :, :i1], v[:, :, :i1]
        f = lambda t: t.float()
        ro, rl, _ = fa_ref.attn_fwd_ref(f(qs), f(ks), f(vs), None, sm, 3, BR, BR)
        lo, ll, _ = fa_ref.attn_fwd_ref(qs, ks, vs, None, sm, 3, BR, BR)
        check('out', o[:, :, i0:i1], ro, lo, FUDGE['out'])
        assert (L.view(B, Hq, S)[:, :, i0:i1] - rl).abs().max().item() <= LSE_ATOL
        rg = fa_ref.attn_bwd_ref(f(qs), f(ks), f(vs), None, sm, ro, f(dos), rl, 3, BR, BR)
        lg = fa_ref.attn_bwd_ref(qs, ks, vs, None, sm, lo, dos, ll.to(torch.bfloat16), 3, BR, BR)
        check('dq', qg.grad[:, :, i0:i1], rg[0], lg[0], FUDGE['dq'])
        if i1 == S:
            check('dk', kg.grad[:, :, i0:], rg[1][:, :, i0:], lg[1][:, :, i0:], FUDGE['dk'])
            check('dv', vg.grad[:, :, i0:], rg[2][:, :, i0:], lg[2][:, :, i0:], FUDGE['dv'])
    colsum = vg.grad.float().sum(dim=2)                                  # (B, Hk, D)
    dosum = do.float().view(B, Hk, Hq // Hk, S, D).sum(dim=(2, 3))
    assert (colsum - dosum).abs().max().item() < 1.0, (colsum - dosum).abs().max().item()


def test_tensors_with_more_than_2g_elements():
    """B520 H64 S1024 D64 bf16 causal: 2,181,038,080 elements per tensor, so element offsets
    pass 2^31.  Row 0 of every head attends only to key 0 (O[0] == V[0]); the first, a
    middle and the last head match the oracle; sum_n dV[n] == sum_m dO[m] for every head."""
    from aotriton_amd.autograd import attention, AttentionExtraArgs
    from oracle import fa_ref
    B, H, S, D = 520, 64, 1024, 64
    assert B * H * S * D > 2 ** 31
    g = torch.Generator(device=DEV).manual_seed(77)
    mk = lambda: torch.randn(B, H, S, D, generator=g, device=DEV, dtype=torch.bfloat16)
    q, k, v, do = mk(), mk(), mk(), mk()
    sm = 1.0 / math.sqrt(D)
    for backend in (0, 1):
        q.grad = k.grad = v.grad = None
        q.requires_grad_(); k.requires_grad_(); v.requires_grad_()
        o, _, L = attention(q, k, v, None, True, sm, 0.0,
                            AttentionExtraArgs(return_logsumexp=True, fillnan=True, bwd_backend=backend))
        o.backward(do)
        torch.cuda.synchronize()
        assert torch.equal(o[:, :, 0], v[:, :, 0])
        assert not bool(torch.isnan(o).any()) and not bool(torch.isnan(L).any())
        for t in (q.grad, k.grad, v.grad):
            assert not bool(torch.isnan(t).any())
        for (b, h) in [(0, 0), (263, 31), (B - 1, H - 1)]:
            sl = lambda t: t.detach()[b:b + 1, h:h + 1]
            ro, rl, _ = fa_ref.attn_fwd_ref(sl(q).float(), sl(k).float(), sl(v).float(), None, sm, 3, -2147483647, -2147483647)
            lo, ll, _ = fa_ref.attn_fwd_ref(sl(q), sl(k), sl(v), None, sm, 3, -2147483647, -2147483647)
            check('out', sl(o), ro, lo, FUDGE['out'])
            assert (L.view(B, H, S)[b, h] - rl[0, 0]).abs().max().item() <= LSE_ATOL
            rg = fa_ref.attn_bwd_ref(sl(q).float(), sl(k).float(), sl(v).float(), None, sm, ro, sl(do).float(), rl,
                                     3, -2147483647, -2147483647)
            lg = fa_ref.attn_bwd_ref(sl(q), sl(k), sl(v), None, sm, lo, sl(do), ll.to(torch.bfloat16), 3,
                                     -2147483647, -2147483647)
            check('dq', sl(q.grad), rg[0], lg[0], FUDGE['dq'])
            check('dk', sl(k.grad), rg[1], lg[1], FUDGE['dk'])
            check('dv', sl(v.grad), rg[2], lg[2], FUDGE['dv'])
        colsum = v.grad.float().sum(dim=2)
        dosum = do.float().sum(dim=2)
        assert (colsum - dosum).abs().max().item() < 0.5, (colsum - dosum).abs().max().item()
        del o, L, colsum, dosum
    q.grad = k.grad = v.grad = None
    del q, k, v, do
    torch.cuda.empty_cache()


@pytest.mark.parametrize('layout', ['padded', 'strided'])
@pytest.mark.parametrize('causal', [False, True])
@pytest.mark.parametrize('backend', [0, 1])
def test_padded_and_strided_varlen(layout, causal, backend):
    _run_layout_case(layout, causal, backend, [70, 5, 192, 133], [3, 11, 0, 60], 128, torch.bfloat16, 4, 2)


@pytest.mark.parametrize('layout', ['padded', 'compact'])
@pytest.mark.parametrize('dtype,D', [(torch.bfloat16, 64), (torch.float16, 128), (torch.float32, 64)])
@pytest.mark.parametrize('backend', [0, 1])
def test_varlen_with_bias(layout, dtype, D, backend):
    """The reference's kernels index the bias of a varlen batch by batch index and by rows and columns
    counted from the sequence's start (modules/flash/kernel/fwd_kernel.py:393-395): one (Hq, max, max)
    slab per sequence in the padded layout (dB likewise), one slab shared by all sequences of packed
    tokens (no dB then).  Against the oracle, sequence by sequence."""
    from aotriton_amd import flash
    from oracle import fa_ref
    lens = np.asarray([70, 5, 0, 131, 64])
    n, mx, Hq, Hk = len(lens), int(lens.max()), 4, 2
    g = torch.Generator().manual_seed(21)
    rn = lambda *s, scale=1.0: (torch.randn(*s, generator=g) * scale).to(dtype).to(DEV)
    cu = torch.tensor([0] + np.cumsum(lens).tolist(), dtype=torch.int32, device=DEV)
    padded = layout == 'padded'
    if padded:
        q, k, v, do = rn(n, Hq, mx, D), rn(n, Hk, mx, D), rn(n, Hk, mx, D), rn(n, Hq, mx, D)
        L = torch.zeros(n * Hq, mx, device=DEV, dtype=torch.float32)
        sl = lambda t, i: t[i:i + 1, :, :lens[i]]
        b = rn(n, Hq, mx, (mx + 7) // 8 * 8, scale=0.5)[..., :mx]
        db = torch.full_like(b, float('nan'))
    else:
        T = int(lens.sum())
        starts = cu.tolist()
        q, k, v, do = rn(1, Hq, T, D), rn(1, Hk, T, D), rn(1, Hk, T, D), rn(1, Hq, T, D)
        L = torch.zeros(Hq, T, device=DEV, dtype=torch.float32)
        sl = lambda t, i: t[:, :, starts[i]:starts[i] + lens[i]]
        b = rn(1, Hq, mx, (mx + 7) // 8 * 8, scale=0.5)[..., :mx]
        db = None
    o, dq, dk, dv = torch.empty_like(q), torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    delta = torch.zeros_like(L)
    null = torch.empty([0], device=DEV, dtype=torch.uint64)
    atomic = torch.zeros([1], device=DEV, dtype=torch.int32)
    sm = 1.0 / math.sqrt(D)
    ok = flash.hipError_t.hipSuccess
    causal = True
    assert flash.attn_fwd_varlen(q, k, v, cu, cu, mx, mx, None, None, b, sm, L, o, 0.0, null, null, 0, null, null,
                                 None, causal, atomic, layout) == ok
    ext = flash.attn_options(); ext.force_backend_index = backend
    assert flash.attn_bwd_varlen(q, k, v, cu, cu, mx, mx, None, None, b, sm, o, do, dq, dk, dv, db, None, L, delta,
                                 0.0, null, null, 0, causal, layout, extargs=ext) == ok
    torch.cuda.synchronize()
    if not padded:      # a dB of packed tokens has no owner
        assert flash.attn_bwd_varlen(q, k, v, cu, cu, mx, mx, None, None, b, sm, o, do, dq, dk, dv, torch.empty_like(b),
                                     None, L, delta, 0.0, null, null, 0, causal, layout,
                                     extargs=ext) == flash.hipError_t.hipErrorNotSupported
    ct, wl, wr = flash.translate_causal(causal)
    hp = torch.float64 if dtype == torch.float32 else torch.float32
    f = lambda t: t.to(hp)
    for i in range(n):
        if lens[i] == 0:
            continue
        qi, ki, vi, doi = sl(q, i), sl(k, i), sl(v, i), sl(do, i)
        bi = b[i:i + 1, :, :lens[i], :lens[i]] if padded else b[:, :, :lens[i], :lens[i]]
        ro, rl, _ = fa_ref.attn_fwd_ref(f(qi), f(ki), f(vi), f(bi), sm, ct, wl, wr, 0.0, None)
        lo, ll, _ = fa_ref.attn_fwd_ref(qi, ki, vi, bi, sm, ct, wl, wr, 0.0, None)
        check(f'out[{i}]', sl(o, i), ro, lo, FUDGE['out'])
        rg = fa_ref.attn_bwd_ref(f(qi), f(ki), f(vi), f(bi), sm, ro, f(doi), rl, ct, wl, wr, 0.0, None)
        lg = fa_ref.attn_bwd_ref(qi, ki, vi, bi, sm, lo, doi, ll.to(dtype).float().to(dtype), ct, wl, wr, 0.0, None)
        check(f'dq[{i}]', sl(dq, i), rg[0], lg[0], FUDGE['dq'])
        check(f'dk[{i}]', sl(dk, i), rg[1], lg[1], FUDGE['dk'])
        check(f'dv[{i}]', sl(dv, i), rg[2], lg[2], FUDGE['dv'])
        if padded:
            check(f'db[{i}]', db[i:i + 1, :, :lens[i], :lens[i]], rg[3], lg[3], FUDGE['db'])


def test_packed_sequences_at_full_size_equal_per_sequence_runs(recomputing_backward):
    """16 packed sequences of 256-8192 tokens (GQA 32 / 8, D = 128, bf16, causal: the packed benchmark
    configuration at full size): every sequence's O, LSE, dQ, dK, dV must equal, bit for bit, what the
    dense entry points give for that sequence alone.  The work lists of the packed run (valid tiles of
    all sequences ordered by weight) change the order in which tiles are computed, never a result.
    (Both sides on the recomputing kernels: packed sequences always take them, and the backward that
    keeps dS in HBM forms delta in another kernel, i.e. in another summation order.)"""
    from aotriton_amd import flash
    ok = flash.hipError_t.hipSuccess
    null = torch.empty([0], device=DEV, dtype=torch.uint64)
    rng = np.random.default_rng(1234)
    lens = rng.integers(256, 8193, size=16)
    cu = np.zeros(17, dtype=np.int32)
    cu[1:] = np.cumsum(lens)
    T, Hq, Hk, D = int(cu[-1]), 32, 8, 128
    gg = torch.Generator(device=DEV).manual_seed(1)
    mk = lambda h: torch.randn(1, T, h, D, device=DEV, dtype=torch.float32, generator=gg).to(torch.bfloat16).transpose(1, 2)
    q, k, v, do = mk(Hq), mk(Hk), mk(Hk), mk(Hq)
    o, dq, dk, dv = torch.empty_like(q), torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    L = torch.empty(Hq, T, device=DEV, dtype=torch.float32)
    d = torch.empty_like(L)
    cuq = torch.from_numpy(cu).to(DEV)
    mx, sm = int(lens.max()), 1.0 / math.sqrt(D)
    atomic = torch.zeros([1], device=DEV, dtype=torch.int32)
    assert flash.attn_fwd_compact_varlen(q, k, v, None, cuq, cuq, mx, mx, sm, L, o, 0.0, null, null, 0, null, null, None,
                                         True, atomic) == ok
    assert flash.attn_bwd_compact_varlen(q, k, v, cuq, cuq, mx, mx, None, sm, o, do, dq, dk, dv, None, L, d, 0.0, null,
                                         null, 0, True) == ok
    torch.cuda.synchronize()
    for i in range(len(lens)):
        s, n = slice(int(cu[i]), int(cu[i + 1])), int(lens[i])
        qi, ki, vi, doi = [t[:, :, s].contiguous() for t in (q, k, v, do)]
        oi, dqi, dki, dvi = torch.empty_like(qi), torch.empty_like(qi), torch.empty_like(ki), torch.empty_like(vi)
        Li = torch.empty(Hq, n, device=DEV, dtype=torch.float32)
        di = torch.empty_like(Li)
        assert flash.attn_fwd(qi, ki, vi, None, sm, Li, oi, 0.0, null, null, 0, null, null, None, True, atomic) == ok
        assert flash.attn_bwd(qi, ki, vi, None, sm, oi, doi, dqi, dki, dvi, None, None, Li, di, 0.0, null, null, 0,
                              True) == ok
        torch.cuda.synchronize()
        for name, a, b in (('o', o[:, :, s], oi), ('lse', L[:, s], Li), ('dq', dq[:, :, s], dqi),
                           ('dk', dk[:, :, s], dki), ('dv', dv[:, :, s], dvi)):
            assert torch.equal(a, b), f'sequence {i}: {name} differs from the run of the sequence alone'


def _sampled_layout_cases(n=24, seed=77):
    import random
    rnd = random.Random(seed)
    cases = []
    for i in range(n):
        ns = rnd.randint(1, 5)
        lens = [rnd.choice([0, 2, 5, 31, 64, 70, 129, 192, 260]) for _ in range(ns)]
        if max(lens) == 0: lens[0] = 9
        pads = [rnd.choice([0, 0, 3, 8, 60]) for _ in range(ns)]
        D = rnd.choice([32, 64, 72, 128, 256, 320])
        dtype = rnd.choice([torch.float16, torch.bfloat16, torch.float32])
        Hq, Hk = rnd.choice([(4, 2), (3, 3), (8, 1)])
        causal = rnd.choice([False, True])
        backend = 0 if (dtype == torch.float32 or D > 256) else rnd.choice([0, 1])
        cases.append((['padded', 'strided'][i % 2], causal, backend, tuple(lens), tuple(pads), D, dtype, Hq, Hk))
    return cases


@pytest.mark.parametrize('case', _sampled_layout_cases(),
                         ids=lambda c: f"{c[0]}-{'c' if c[1] else 'n'}-be{c[2]}-n{len(c[3])}-d{c[5]}-{str(c[6])[6:]}-h{c[7]}_{c[8]}")
def test_sampled_padded_and_strided_varlen(case):
    _run_layout_case(*case)


def _run_layout_case(layout, causal, backend, lens, pads, D, dtype, Hq, Hk):
    # varlen_type 2: rank-4 batch tensors padded to the longest sequence, LSE (n*Hq, max_sq);
    # varlen_type 3: packed tokens with gaps, sequence starts from seq_strides, LSE (Hq, total)
    # (modules/flash/kernel/fwd_kernel.py:243-286, tests/varlen_attn_torch_function.py:52-84).
    from aotriton_amd import flash
    from oracle import fa_ref
    lens = np.asarray(lens)
    pads = np.asarray(pads)
    n, mx = len(lens), int(lens.max())
    g = torch.Generator().manual_seed(11)
    rn = lambda *s: torch.randn(*s, generator=g).to(dtype).to(DEV)
    cu = torch.tensor([0] + np.cumsum(lens).tolist(), dtype=torch.int32, device=DEV)
    if layout == 'padded':
        q, k, v, do = rn(n, Hq, mx, D), rn(n, Hk, mx, D), rn(n, Hk, mx, D), rn(n, Hq, mx, D)
        L = torch.zeros(n * Hq, mx, device=DEV, dtype=torch.float32)
        ss = None
        starts = [0] * n
        sl = lambda t, i: t[i:i + 1, :, :lens[i]]
    else:
        T = int((lens + pads).sum())
        q, k, v, do = rn(1, Hq, T, D), rn(1, Hk, T, D), rn(1, Hk, T, D), rn(1, Hq, T, D)
        L = torch.zeros(Hq, T, device=DEV, dtype=torch.float32)
        ss = torch.tensor([0] + np.cumsum(lens + pads).tolist(), dtype=torch.int32, device=DEV)
        starts = ss.tolist()
        sl = lambda t, i: t[:, :, starts[i]:starts[i] + lens[i]]
    nan = float('nan')
    o = torch.full_like(q, nan); dq = torch.full_like(q, nan); dk = torch.full_like(k, nan); dv = torch.full_like(v, nan)
    delta = torch.zeros_like(L)
    null = torch.empty([0], device=DEV, dtype=torch.uint64)
    atomic = torch.zeros([1], device=DEV, dtype=torch.int32)
    sm = 1.0 / math.sqrt(D)
    ok = flash.hipError_t.hipSuccess
    assert flash.attn_fwd_varlen(q, k, v, cu, cu, mx, mx, ss, ss, None, sm, L, o, 0.0, null, null, 0, null, null,
                                 None, causal, atomic, layout) == ok
    ext = flash.attn_options(); ext.force_backend_index = backend
    assert flash.attn_bwd_varlen(q, k, v, cu, cu, mx, mx, ss, ss, None, sm, o, do, dq, dk, dv, None, None, L, delta,
                                 0.0, null, null, 0, causal, layout, extargs=ext) == ok
    torch.cuda.synchronize()
    ct, wl, wr = flash.translate_causal(causal)
    hp = torch.float64 if dtype == torch.float32 else torch.float32
    f = lambda t: t.to(hp)
    for i in range(n):
        if lens[i] == 0:
            continue
        qi, ki, vi, doi = sl(q, i), sl(k, i), sl(v, i), sl(do, i)
        ro, rl, _ = fa_ref.attn_fwd_ref(f(qi), f(ki), f(vi), None, sm, ct, wl, wr, 0.0, None)
        lo, ll, _ = fa_ref.attn_fwd_ref(qi, ki, vi, None, sm, ct, wl, wr, 0.0, None)
        check(f'out[{i}]', sl(o, i), ro, lo, FUDGE['out'])
        Li = L.view(n, Hq, mx)[i:i + 1, :, :lens[i]] if layout == 'padded' else L[None, :, starts[i]:starts[i] + lens[i]]
        assert (Li - rl).abs().max().item() <= LSE_ATOL
        rg = fa_ref.attn_bwd_ref(f(qi), f(ki), f(vi), None, sm, ro, f(doi), rl, ct, wl, wr, 0.0, None)
        lg = fa_ref.attn_bwd_ref(qi, ki, vi, None, sm, lo, doi, ll.to(dtype).float().to(dtype), ct, wl, wr, 0.0, None)
        check(f'dq[{i}]', sl(dq, i), rg[0], lg[0], FUDGE['dq'])
        check(f'dk[{i}]', sl(dk, i), rg[1], lg[1], FUDGE['dk'])
        check(f'dv[{i}]', sl(dv, i), rg[2], lg[2], FUDGE['dv'])
    # rows outside the sequences are never written
    for i in range(n):
        if layout == 'padded':
            assert torch.isnan(o[i, :, lens[i]:]).all() and torch.isnan(dk[i, :, lens[i]:]).all()
            assert torch.isnan(dq[i, :, lens[i]:]).all() and torch.isnan(dv[i, :, lens[i]:]).all()
        else:
            gap = slice(starts[i] + lens[i], starts[i + 1])
            assert torch.isnan(o[:, :, gap]).all() and torch.isnan(dv[:, :, gap]).all()
            assert torch.isnan(dq[:, :, gap]).all() and torch.isnan(dk[:, :, gap]).all()


def test_config4_full_size_properties():
    """GQA varlen at full size: Hq 32, Hkv 8, D 128 bf16 causal, 16 packed sequences of
    256..8192 tokens (~68K in all).  Checked per sequence, so at any size: (1) the first
    row of a sequence attends to its first key only; (2) the shortest and the longest
    sequence match the dense oracle for one kv-head and its four q-heads; (3) the keys'
    dV sums equal the dO sums of the q-heads that share the kv-head."""
    from aotriton_amd.autograd import attention_varlen, AttentionExtraArgs
    from oracle import fa_ref
    rng = np.random.default_rng(1234)
    lens = rng.integers(256, 8193, size=16)
    cu = np.concatenate([[0], np.cumsum(lens)]).astype(np.int64)
    T = int(cu[-1])
    Hq, Hk, D = 32, 8, 128
    dt = torch.bfloat16
    g = torch.Generator(device=DEV).manual_seed(4)
    mk = lambda H: torch.randn(1, T, H, D, device=DEV, generator=g).to(dt).transpose(1, 2)
    q, k, v, do = mk(Hq), mk(Hk), mk(Hk), mk(Hq)
    sm = 1.0 / math.sqrt(D)
    TL = -2147483647
    for backend in (0, 1):
        qg, kg, vg = [t.clone().requires_grad_() for t in (q, k, v)]
        o, _, L = attention_varlen(qg, kg, vg, lens, lens, True, sm, 0.0,
                                   AttentionExtraArgs(return_logsumexp=True, fillnan=True, bwd_backend=backend))
        o.backward(do)
        torch.cuda.synchronize()
        for t in (o, L, qg.grad, kg.grad, vg.grad):
            assert torch.isfinite(t).all()
        first = torch.from_numpy(cu[:-1]).to(DEV)
        assert torch.equal(o[0, :, first], v[0, :, first].repeat_interleave(Hq // Hk, dim=0))
        s00 = (q[0, :, first].float() * k[0, :, first].float().repeat_interleave(Hq // Hk, dim=0)).sum(-1) * sm
        assert torch.allclose(L[:, first], s00, atol=1e-4, rtol=1e-5)
        hk = 5
        hs = slice(hk * 4, hk * 4 + 4)
        for i in (int(np.argmin(lens)), int(np.argmax(lens))):
            a, b = int(cu[i]), int(cu[i + 1])
            qs, ks, vs, dos = q[:, hs, a:b], k[:, hk:hk + 1, a:b], v[:, hk:hk + 1, a:b], do[:, hs, a:b]
            ro, rl, _ = fa_ref.attn_fwd_ref(qs.float(), ks.float(), vs.float(), None, sm, 3, TL, TL)
            lo, ll, _ = fa_ref.attn_fwd_ref(qs, ks, vs, None, sm, 3, TL, TL)
            check('out', o[:, hs, a:b], ro, lo, FUDGE['out'])
            assert (L[hs, a:b] - rl[0]).abs().max().item() <= LSE_ATOL
            rg = fa_ref.attn_bwd_ref(qs.float(), ks.float(), vs.float(), None, sm, ro, dos.float(), rl, 3, TL, TL)
            lg = fa_ref.attn_bwd_ref(qs, ks, vs, None, sm, lo, dos, ll.to(dt), 3, TL, TL)
            check('dq', qg.grad[:, hs, a:b], rg[0], lg[0], FUDGE['dq'])
            check('dk', kg.grad[:, hk:hk + 1, a:b], rg[1], lg[1], FUDGE['dk'])
            check('dv', vg.grad[:, hk:hk + 1, a:b], rg[2], lg[2], FUDGE['dv'])
        for i in range(len(lens)):
            a, b = int(cu[i]), int(cu[i + 1])
            colsum = vg.grad[0, :, a:b].float().sum(dim=1)                            # (Hk, D)
            dosum = do[0, :, a:b].float().sum(dim=1).view(Hk, Hq // Hk, D).sum(dim=1)
            assert (colsum - dosum).abs().max().item() < 1.0, (i, (colsum - dosum).abs().max().item())


def test_config5_full_size_properties():
    """Window (1024, 0) + bias + dropout 0.1 (seed 0x1234, offset 0) at B2 H16 S8192 D256
    fp16: a sampled (batch, head) against the dense oracle with the oracle's own keep
    mask, dB exactly zero outside the band, everything finite."""
    from aotriton_amd.autograd import attention, AttentionExtraArgs
    from oracle import fa_ref, philox
    B, H, S, D = 2, 16, 8192, 256
    dt = torch.float16
    g = torch.Generator(device=DEV).manual_seed(0)
    rn = lambda *s, sc=1.0: (torch.randn(*s, device=DEV, dtype=torch.float32, generator=g) * sc).to(dt)
    q, k, v, do = rn(B, H, S, D), rn(B, H, S, D), rn(B, H, S, D), rn(B, H, S, D)
    bias = torch.empty(B, H, S, S, device=DEV, dtype=dt)
    for i in range(B):
        for h in range(H):
            bias[i, h] = rn(S, S, sc=0.5)
    sm = 1.0 / math.sqrt(D)
    p = 0.1
    qg, kg, vg, bg = [t.requires_grad_() for t in (q, k, v, bias)]
    ext = AttentionExtraArgs(return_logsumexp=True, philox_seed=0x1234, philox_offset1=0, philox_offset2=0)
    o, _, L = attention(qg, kg, vg, bg, (1024, 0), sm, p, ext)
    o.backward(do)
    torch.cuda.synchronize()
    for t in (o, L, qg.grad, kg.grad, vg.grad):
        assert torch.isfinite(t).all()
    bsel, hsel = 1, 7
    sl = lambda t: t.detach()[bsel:bsel + 1, hsel:hsel + 1]
    keep = torch.from_numpy(philox.dropout_keep_mask(B, H, S, S, p, 0x1234, 0, b_sel=[bsel], h_sel=[hsel])).to(DEV)
    f = lambda t: sl(t).float()
    ro, rl, _ = fa_ref.attn_fwd_ref(f(q), f(k), f(v), f(bias), sm, 3, 1024, 0, p, keep)
    lo, ll, _ = fa_ref.attn_fwd_ref(sl(q), sl(k), sl(v), sl(bias), sm, 3, 1024, 0, p, keep)
    check('out', sl(o), ro, lo, FUDGE['out'])
    assert (L.view(B, H, S)[bsel, hsel] - rl[0, 0]).abs().max().item() <= LSE_ATOL
    rg = fa_ref.attn_bwd_ref(f(q), f(k), f(v), f(bias), sm, ro, f(do), rl, 3, 1024, 0, p, keep)
    lg = fa_ref.attn_bwd_ref(sl(q), sl(k), sl(v), sl(bias), sm, lo, sl(do), ll.to(dt), 3, 1024, 0, p, keep)
    check('dq', sl(qg.grad), rg[0], lg[0], FUDGE['dq'])
    check('dk', sl(kg.grad), rg[1], lg[1], FUDGE['dk'])
    check('dv', sl(vg.grad), rg[2], lg[2], FUDGE['dv'])
    check('db', sl(bg.grad), rg[3], lg[3], FUDGE['db'])
    # outside the band dB is exactly zero, for every (batch, head)
    m = torch.arange(S, device=DEV).view(S, 1)
    n = torch.arange(S, device=DEV).view(1, S)
    outside = (n > m) | (n < m - 1024)
    for i in range(B):
        for h in range(0, H, 5):
            assert not bg.grad[i, h][outside].any()
