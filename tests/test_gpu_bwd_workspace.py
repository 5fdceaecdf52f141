"""The split backward that keeps dS in HBM (dK/dV kernel writes it, a dQ = dS K kernel reads it
back; head dims 72 to 256) against the oracle and against the recomputing kernels, through the C ABI.

The reference's split backward always recomputes S and dP in its dQ kernel
(modules/flash/kernel/bwd_kernel_dq.py:45-389); both ways must give its results.  Tolerances are
the reference's model (tests/_util.py); the two ways may differ from each other by the rounding of
delta, which one forms in the dQ kernel and the other in the delta kernel."""
import math

import pytest
import torch

from _util import FUDGE, check, keep_mask_from_oracle, make_inputs

pytestmark = pytest.mark.gpu

DEV = 'cuda'
BIG = 1 << 40


def _lib():
    from aotriton_amd._lib import lib
    return lib


@pytest.fixture(autouse=True)
def _restore_limit():
    yield
    _lib().fa_set_bwd_workspace_limit(-1)


def _backward(q, k, v, b, do, sm, causal, p, limit, seed=(77, 3, 5), stream=None):
    """O, L, dQ, dK, dV of one forward + split backward with the given workspace limit."""
    from aotriton_amd import flash
    ok = flash.hipError_t.hipSuccess
    B, Hq, Sq = q.shape[0], q.shape[1], q.shape[2]
    u64 = lambda x: torch.tensor([x], device=DEV, dtype=torch.uint64)
    sd, o1, so, oo = u64(seed[0]), u64(seed[1]), u64(0), u64(0)
    atomic = torch.zeros([1], device=DEV, dtype=torch.int32)
    o = torch.empty(q.shape[:3] + (v.shape[3],), device=DEV, dtype=q.dtype)
    L = torch.empty(B * Hq, Sq, device=DEV, dtype=torch.float32)
    assert flash.attn_fwd(q, k, v, b, sm, L, o, p, sd, o1, seed[2], so, oo, None, causal, atomic) == ok
    dq = torch.full_like(q, float('nan'))
    dk = torch.full_like(k, float('nan'))
    dv = torch.full_like(v, float('nan'))
    delta = torch.full_like(L, float('nan'))
    _lib().fa_set_bwd_workspace_limit(limit)
    ext = flash.attn_options()
    ext.force_backend_index = 0
    assert flash.attn_bwd(q, k, v, b, sm, o, do, dq, dk, dv, None, None, L, delta, p, so, oo, 0, causal,
                          extargs=ext) == ok
    torch.cuda.synchronize()
    assert flash.hipGetLastError() == ok
    return o, L, dq, dk, dv, delta


def _would_keep_ds(q, k, v, b, do, sm, causal, p):
    """bit 4 of fa_query_bwd_config's flags: the call would keep dS in HBM"""
    from aotriton_amd import flash
    from aotriton_amd.pyaotriton.v3.flash import attn_bwd_params, query_bwd_config
    seed = torch.zeros([1], device=DEV, dtype=torch.uint64)
    o = torch.empty_like(q)
    L = torch.empty(q.shape[0] * q.shape[1], q.shape[2], device=DEV, dtype=torch.float32)
    params = attn_bwd_params()
    flash._fill_bwd(params, q, k, v, b, sm, o, do, torch.empty_like(q), torch.empty_like(k), torch.empty_like(v), None,
                    None, L, torch.empty_like(L), p, seed, seed, 0, causal)
    err, cfg = query_bwd_config(params, 1)
    assert err == flash.hipError_t.hipSuccess
    return bool(cfg.flags & 16)


CASES = [
    # B, Hq, Hk, Sq, Sk, D, dtype, causal, dropout, bias, bshd
    (2, 4, 4, 256, 256, 128, torch.bfloat16, False, 0.0, False, False),
    (2, 4, 2, 200, 264, 128, torch.bfloat16, True, 0.0, False, False),
    (3, 10, 2, 523, 337, 128, torch.float16, True, 0.0, False, True),
    (3, 10, 2, 203, 1063, 128, torch.bfloat16, False, 0.0, False, True),
    (1, 3, 1, 777, 1301, 128, torch.bfloat16, (100, 20), 0.0, False, False),
    (2, 4, 2, 515, 300, 128, torch.float16, True, 0.2, False, False),
    (1, 2, 2, 333, 257, 128, torch.float16, False, 0.1, True, False),
    (1, 2, 1, 300, 431, 128, torch.bfloat16, (64, 0), 0.3, True, False),
    (1, 2, 2, 300, 300, 96, torch.bfloat16, True, 0.0, False, False),
    (2, 2, 1, 129, 65, 72, torch.float16, False, 0.0, False, False),
    (1, 1, 1, 1, 1, 128, torch.bfloat16, True, 0.0, False, False),
    (1, 2, 2, 64, 2048, 128, torch.bfloat16, False, 0.0, False, False),
    (1, 2, 2, 2048, 64, 128, torch.bfloat16, True, 0.0, False, False),
    # the 256-column build (32-query tiles)
    (2, 4, 2, 300, 264, 256, torch.float16, True, 0.0, False, False),
    (1, 3, 3, 523, 337, 256, torch.bfloat16, False, 0.0, False, True),
    (1, 2, 1, 777, 1301, 256, torch.float16, (100, 20), 0.2, False, False),
    (1, 2, 2, 333, 257, 192, torch.bfloat16, True, 0.1, True, False),
    (2, 2, 1, 129, 65, 136, torch.float16, False, 0.0, False, False),
    (1, 1, 1, 1, 1, 256, torch.bfloat16, True, 0.0, False, False),
    # the 64-column build (128-query tiles): with dropout or a bias only
    (2, 4, 2, 300, 264, 64, torch.float16, True, 0.2, False, False),
    (1, 3, 3, 523, 337, 64, torch.bfloat16, False, 0.1, False, True),
    (1, 2, 1, 777, 1301, 40, torch.float16, (100, 20), 0.3, False, False),
    (1, 2, 2, 129, 257, 16, torch.bfloat16, True, 0.5, False, False),
]


@pytest.mark.parametrize('case', CASES, ids=lambda c: '-'.join(str(x).replace('torch.', '') for x in c))
def test_both_backwards_meet_the_oracle(case):
    from aotriton_amd import flash
    from oracle import fa_ref
    B, Hq, Hk, Sq, Sk, D, dtype, causal, p, bias, bshd = case
    q, k, v, b, do = make_inputs(B, Hq, Hk, Sq, Sk, D, dtype, DEV, seed=11, bias=bias, bshd=bshd)
    sm = 1.0 / math.sqrt(D)
    _lib().fa_set_bwd_workspace_limit(BIG)
    assert _would_keep_ds(q, k, v, b, do, sm, causal, p)
    _lib().fa_set_bwd_workspace_limit(0)
    assert not _would_keep_ds(q, k, v, b, do, sm, causal, p)

    ct, wl, wr = flash.translate_causal(causal)
    seed = (77, 3, 5)
    keep = keep_mask_from_oracle(B, Hq, Sq, Sk, p, seed[0], seed[1] + seed[2], DEV)
    f32 = lambda t: None if t is None else t.float()
    ro, rl, _ = fa_ref.attn_fwd_ref(f32(q), f32(k), f32(v), f32(b), sm, ct, wl, wr, p, keep)
    lo, ll, _ = fa_ref.attn_fwd_ref(q, k, v, b, sm, ct, wl, wr, p, keep)
    rg = fa_ref.attn_bwd_ref(f32(q), f32(k), f32(v), f32(b), sm, ro, f32(do), rl, ct, wl, wr, p, keep)
    lg = fa_ref.attn_bwd_ref(q, k, v, b, sm, lo, do, ll.to(q.dtype).float().to(q.dtype), ct, wl, wr, p, keep)
    got = {}
    for mode, limit in (('kept', BIG), ('recomputed', 0)):
        o, L, dq, dk, dv, delta = _backward(q, k, v, b, do, sm, causal, p, limit, seed)
        check(f'dq ({mode})', dq, rg[0], lg[0], FUDGE['dq'])
        check(f'dk ({mode})', dk, rg[1], lg[1], FUDGE['dk'])
        check(f'dv ({mode})', dv, rg[2], lg[2], FUDGE['dv'])
        # delta is an output of both: the row sum of O * dO (modules/flash/kernel/bwd_preprocess.py:63-121)
        want = (o.float() * do.float()).sum(-1).view(B * Hq, Sq)
        assert (delta - want).abs().max().item() <= 1e-3 * max(1.0, want.abs().max().item())
        got[mode] = (dq.float(), dk.float(), dv.float())
    # the two ways use the same operand values; what differs is the summation order of delta
    for name, x, y in zip(('dq', 'dk', 'dv'), got['kept'], got['recomputed']):
        scale = max(y.abs().max().item(), 1e-6)
        assert (x - y).abs().max().item() <= 2.0 ** -6 * scale, f'{name}: the two backwards disagree'


def test_calls_that_do_not_qualify_recompute():
    """head dims up to 64 without dropout and bias (where keeping dS measured slower), head dims above 256, fp32,
    packed sequences and dB keep the recomputing kernels"""
    from aotriton_amd import flash
    _lib().fa_set_bwd_workspace_limit(BIG)
    sm = 0.1
    for D, dtype in ((64, torch.bfloat16), (128, torch.float32), (40, torch.bfloat16), (512, torch.bfloat16)):
        q, k, v, b, do = make_inputs(1, 2, 2, 128, 128, D, dtype, DEV, seed=1)
        assert not _would_keep_ds(q, k, v, None, do, sm, True, 0.0), (D, dtype)
    for D in (72, 256):
        q, k, v, b, do = make_inputs(1, 2, 2, 128, 128, D, torch.float16, DEV, seed=1)
        assert _would_keep_ds(q, k, v, None, do, sm, True, 0.0), D
    q, k, v, b, do = make_inputs(1, 2, 2, 128, 128, 64, torch.float16, DEV, seed=1)
    assert _would_keep_ds(q, k, v, None, do, sm, True, 0.1)
    q, k, v, b, do = make_inputs(1, 2, 2, 128, 128, 128, torch.bfloat16, DEV, seed=1)
    assert _would_keep_ds(q, k, v, None, do, sm, True, 0.0)
    # a limit below the need (2 bytes per (head, query, key) pair, in tiles of 128 x 64, plus the row statistics)
    _lib().fa_set_bwd_workspace_limit(2 * 128 * 128 * 2)
    assert not _would_keep_ds(q, k, v, None, do, sm, True, 0.0)
    _lib().fa_set_bwd_workspace_limit(1 << 20)
    assert _would_keep_ds(q, k, v, None, do, sm, True, 0.0)


def test_scale_zero_and_huge_scores():
    """sm_scale = 0 (every p is 1 / visible keys) and scores far outside exp2's range of the 16-bit
    types (fwd_kernel_inner.py:197-205 documents the trap; there P is one-hot, dP - delta is what the
    rounding of O leaves, and the yardstick is the low-precision oracle's own error)"""
    from aotriton_amd import flash
    from oracle import fa_ref
    ct, wl, wr = flash.translate_causal(True)
    for sm, scale in ((0.0, 1.0), (1.0, 30.0)):
        g = torch.Generator().manual_seed(3)
        mk = lambda *s: (torch.randn(*s, generator=g) * scale).to(torch.bfloat16).to(DEV)
        q, k, v, do = mk(1, 2, 200, 128), mk(1, 2, 264, 128), mk(1, 2, 264, 128), mk(1, 2, 200, 128)
        f32 = lambda t: t.float()
        ro, rl, _ = fa_ref.attn_fwd_ref(f32(q), f32(k), f32(v), None, sm, ct, wl, wr, 0.0, None)
        lo, ll, _ = fa_ref.attn_fwd_ref(q, k, v, None, sm, ct, wl, wr, 0.0, None)
        rg = fa_ref.attn_bwd_ref(f32(q), f32(k), f32(v), None, sm, ro, f32(do), rl, ct, wl, wr, 0.0, None)
        lg = fa_ref.attn_bwd_ref(q, k, v, None, sm, lo, do, ll.to(q.dtype).float().to(q.dtype), ct, wl, wr, 0.0, None)
        for mode, limit in (('kept', BIG), ('recomputed', 0)):
            got = _backward(q, k, v, None, do, sm, True, 0.0, limit)
            check(f'dq ({mode}, sm_scale {sm})', got[2], rg[0], lg[0], FUDGE['dq'])
            check(f'dk ({mode}, sm_scale {sm})', got[3], rg[1], lg[1], FUDGE['dk'])
            check(f'dv ({mode}, sm_scale {sm})', got[4], rg[2], lg[2], FUDGE['dv'])


def test_growing_shrinking_and_trimmed_workspace_on_two_streams():
    """the buffer grows with the largest call, smaller calls reuse it, calls on two streams take
    turns, and after a trim the next call allocates again"""
    lib = _lib()
    shapes = [(1, 2, 2, 256, 256), (2, 4, 2, 1024, 1024), (1, 2, 1, 130, 700), (2, 4, 4, 512, 384)]
    inputs = [make_inputs(B, Hq, Hk, Sq, Sk, 128, torch.bfloat16, DEV, seed=5 + i)
              for i, (B, Hq, Hk, Sq, Sk) in enumerate(shapes)]
    sm = 1.0 / math.sqrt(128)
    want = [_backward(q, k, v, None, do, sm, True, 0.0, 0) for q, k, v, _, do in inputs]
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    for rep in range(3):
        if rep == 2:
            assert lib.fa_trim_workspace() == 0
        for i, (q, k, v, _, do) in enumerate(inputs):
            with torch.cuda.stream(streams[i % 2]):
                got = _backward(q, k, v, None, do, sm, True, 0.0, BIG)
            for name, x, y in zip(('dq', 'dk', 'dv'), got[2:5], want[i][2:5]):
                tol = 2.0 ** -6 * y.float().abs().max().item()
                assert (x.float() - y.float()).abs().max().item() <= tol, f'{name}, shape {shapes[i]}, round {rep}'


def test_two_host_threads_share_the_workspace():
    """Two host threads enqueue backwards of different sizes on a stream each, without synchronising
    between calls: the calls take turns on the one buffer (mutex on the host, event on the GPU) and
    every result equals the recomputing backward's within the rounding of delta."""
    import threading
    from aotriton_amd import flash
    lib = _lib()
    ok = flash.hipError_t.hipSuccess
    shapes = [(1, 4, 2, 1024, 1024), (2, 2, 2, 384, 640)]
    sm = 1.0 / math.sqrt(128)
    jobs = []
    for i, (B, Hq, Hk, Sq, Sk) in enumerate(shapes):
        q, k, v, _, do = make_inputs(B, Hq, Hk, Sq, Sk, 128, torch.bfloat16, DEV, seed=40 + i)
        o, L, dq, dk, dv, _ = _backward(q, k, v, None, do, sm, True, 0.0, 0)
        jobs.append((q, k, v, do, o, L, (dq, dk, dv)))
    lib.fa_set_bwd_workspace_limit(BIG)
    assert lib.fa_trim_workspace() == 0          # the first calls of both threads race for the allocation
    null = torch.empty([0], device=DEV, dtype=torch.uint64)
    results, errors = {}, []

    def worker(i):
        try:
            q, k, v, do, o, L, _ = jobs[i]
            stream = torch.cuda.Stream()
            outs = []
            with torch.cuda.stream(stream):
                for rep in range(6):
                    dq, dk, dv = torch.full_like(q, float('nan')), torch.full_like(k, float('nan')), torch.full_like(v, float('nan'))
                    delta = torch.empty_like(L)
                    ext = flash.attn_options()
                    ext.force_backend_index = 0
                    assert flash.attn_bwd(q, k, v, None, sm, o, do, dq, dk, dv, None, None, L, delta, 0.0, null, null, 0,
                                          True, extargs=ext) == ok
                    outs.append((dq, dk, dv))
            stream.synchronize()
            results[i] = outs
        except Exception as e:      # surfaces in the main thread
            errors.append(repr(e))

    threads = [threading.Thread(target=worker, args=(i,)) for i in range(len(jobs))]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    torch.cuda.synchronize()
    assert not errors, errors
    for i, outs in results.items():
        want = jobs[i][6]
        for rep, got in enumerate(outs):
            for name, x, y in zip(('dq', 'dk', 'dv'), got, want):
                tol = 2.0 ** -6 * y.float().abs().max().item()
                assert (x.float() - y.float()).abs().max().item() <= tol, f'{name}, thread {i}, call {rep}'


def test_headline_size_with_kept_ds():
    """B4 H32 S4096 D128 bf16 causal, the benchmark's shape, needs 4.3 GB of dS tiles: sampled heads
    against the recomputing kernels, and the closed forms that hold at any size (the first query sees
    one key: dQ[0] = 0 up to the rounding of O in delta; sum over keys of dV = sum over queries of dO
    weighted by nothing but the softmax, i.e. column sums agree)."""
    B, H, S, D = 4, 32, 4096, 128
    g = torch.Generator(device=DEV).manual_seed(1234)
    rn = lambda: torch.randn(B, H, S, D, device=DEV, dtype=torch.float32, generator=g).to(torch.bfloat16)
    q, k, v, do = rn(), rn(), rn(), rn()
    sm = 1.0 / math.sqrt(D)
    a = _backward(q, k, v, None, do, sm, True, 0.0, BIG)
    b = _backward(q, k, v, None, do, sm, True, 0.0, 0)
    for name, x, y in zip(('dq', 'dk', 'dv'), a[2:5], b[2:5]):
        assert not torch.isnan(x).any(), name
        for z, h in ((0, 0), (1, 17), (3, 31)):
            xs, ys = x[z, h].float(), y[z, h].float()
            assert (xs - ys).abs().max().item() <= 2.0 ** -6 * ys.abs().max().item(), f'{name}[{z},{h}]'
    # a row of P sums to 1, so the column sums of dV equal those of dO
    dv_sum, do_sum = a[4].float().sum(2), do.float().sum(2)
    assert (dv_sum - do_sum).abs().max().item() <= 2e-2 * do_sum.abs().max().item()
    # query 0 sees key 0 only: P = 1, dS = dP - delta = 0
    assert a[2][:, :, 0].float().abs().max().item() <= 1e-2


def test_no_room_for_the_workspace_means_recomputing():
    """When hipMalloc cannot deliver the workspace (the caller's allocator holds the device's memory) the
    call recomputes instead of failing: same results as with the limit at 0, bit for bit."""
    B, H, S, D = 4, 32, 4096, 128                      # needs 4.4 GB of dS tiles
    g = torch.Generator(device=DEV).manual_seed(99)
    rn = lambda: torch.randn(B, H, S, D, device=DEV, dtype=torch.float32, generator=g).to(torch.bfloat16)
    q, k, v, do = rn(), rn(), rn(), rn()
    sm = 1.0 / math.sqrt(D)
    want = _backward(q, k, v, None, do, sm, True, 0.0, 0)
    assert _lib().fa_trim_workspace() == 0
    torch.cuda.empty_cache()
    free, _ = torch.cuda.mem_get_info()
    if free < (16 << 30):
        pytest.skip('not enough free device memory to stage the case')
    try:
        hog = torch.empty(free - (2 << 30), device=DEV, dtype=torch.int8)      # leaves 2 GiB
    except RuntimeError:
        pytest.skip('could not take the device memory in one piece')
    try:
        got = _backward(q, k, v, None, do, sm, True, 0.0, BIG)
    finally:
        del hog
        torch.cuda.empty_cache()
    for name, x, y in zip(('dq', 'dk', 'dv'), got[2:5], want[2:5]):
        assert torch.equal(x, y), name


def test_packed_copies_take_odd_head_dims_to_the_mfma_kernels():
    """Head dim 113 (one of the reference's, modules/flash/tests/test_forward.py:22): with workspace the
    queries report packed copies (bit 5), with the limit at 0 they do not; both give the oracle's results
    (test_gpu_attention.py) and agree with each other here; the packed way is several times faster."""
    from aotriton_amd import flash
    from aotriton_amd.pyaotriton.v3.flash import attn_bwd_params, attn_fwd_params, query_bwd_config, query_fwd_config
    B, H, S, D = 2, 8, 1024, 113
    q, k, v, _, do = make_inputs(B, H, H, S, S, D, torch.bfloat16, DEV, seed=5)
    sm = 1.0 / math.sqrt(D)
    seed = torch.zeros([1], device=DEV, dtype=torch.uint64)
    o = torch.empty_like(q)
    L = torch.empty(B * H, S, device=DEV, dtype=torch.float32)
    atomic = torch.zeros([1], device=DEV, dtype=torch.int32)

    def flags():
        pf, pb = attn_fwd_params(), attn_bwd_params()
        flash._fill_fwd(pf, q, k, v, None, sm, L, o, 0.0, seed, seed, 0, seed, seed, None, True, atomic)
        flash._fill_bwd(pb, q, k, v, None, sm, o, do, torch.empty_like(q), torch.empty_like(k), torch.empty_like(v),
                        None, None, L, torch.empty_like(L), 0.0, seed, seed, 0, True)
        ef, cf = query_fwd_config(pf)
        eb, cb = query_bwd_config(pb, 1)
        assert ef == eb == flash.hipError_t.hipSuccess
        return bool(cf.flags & 32), bool(cb.flags & 32), bool(cb.flags & 16)

    def timed(limit):
        res = _backward(q, k, v, None, do, sm, True, 0.0, limit)      # warms up, grows the buffer
        t0, t1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        t0.record()
        for _ in range(3):
            _backward(q, k, v, None, do, sm, True, 0.0, limit)
        t1.record()
        torch.cuda.synchronize()
        return res, t0.elapsed_time(t1)

    _lib().fa_set_bwd_workspace_limit(-1)
    assert flags() == (True, True, False)      # dS is kept by the call on the copies, not by this one
    _lib().fa_set_bwd_workspace_limit(0)
    assert flags() == (False, False, False)
    packed, t_packed = timed(-1)
    plain, t_plain = timed(0)
    for name, a, b_ in zip(('out', 'L', 'dq', 'dk', 'dv'), packed, plain):
        assert torch.isfinite(a).all(), name
        assert (a.float() - b_.float()).abs().max().item() <= 2e-2 * max(1.0, b_.float().abs().max().item()), name
    assert t_packed * 3 < t_plain, (t_packed, t_plain)
