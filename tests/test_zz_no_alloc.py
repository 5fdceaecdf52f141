"""fa_attn_bwd_noalloc (delta in the library's own device array, nothing allocated) against
fa_attn_bwd with the split backend, through the C ABI: bit-identical dQ, dK, dV on two calls in
a row, the second with a smaller input, and the size limit.  fa_attn_bwd runs with its dS
workspace switched off here: the entry point that allocates nothing uses the recomputing kernels,
and only the same kernels give the same bits."""
import math

import pytest
import torch

from _util import make_inputs

pytestmark = pytest.mark.gpu
DEV = 'cuda'


def _run_pair(B, Hq, Hk, Sq, Sk, D, dtype, causal, seed):
    from aotriton_amd import flash
    from aotriton_amd.pyaotriton.v3.flash import attn_bwd_noalloc, attn_bwd_params
    q, k, v, _, do = make_inputs(B, Hq, Hk, Sq, Sk, D, dtype, DEV, seed=seed)
    sm = 1.0 / math.sqrt(D)
    o = torch.empty_like(q)
    L = torch.empty(B * Hq, Sq, device=DEV, dtype=torch.float32)
    null = torch.empty([0], device=DEV, dtype=torch.uint64)
    atomic = torch.zeros([1], device=DEV, dtype=torch.int32)
    ok = flash.hipError_t.hipSuccess
    assert flash.attn_fwd(q, k, v, None, sm, L, o, 0.0, null, null, 0, null, null, None, causal, atomic) == ok
    # existing entry point, split backend, caller's delta buffer
    delta = torch.full_like(L, float('nan'))
    ref = [torch.full_like(t, float('nan')) for t in (q, k, v)]
    ext = flash.attn_options()
    ext.force_backend_index = 0
    assert flash.attn_bwd(q, k, v, None, sm, o, do, ref[0], ref[1], ref[2], None, None, L, delta, 0.0, null, null, 0,
                          causal, extargs=ext) == ok
    # new entry point: no delta passed at all
    got = [torch.full_like(t, float('nan')) for t in (q, k, v)]
    params = attn_bwd_params()
    flash._fill_bwd(params, q, k, v, None, sm, o, do, got[0], got[1], got[2], None, None, L, None, 0.0, null, null, 0,
                    causal)
    assert attn_bwd_noalloc(params, attn_bwd_params.kVersion, flash._stream()) == ok      # warm-up: symbol lookup, LDS limits
    torch.cuda.synchronize()
    for t in got:
        t.fill_(float('nan'))
    torch.cuda.synchronize()
    before, free_before = torch.cuda.memory_allocated(), torch.cuda.mem_get_info()[0]
    assert attn_bwd_noalloc(params, attn_bwd_params.kVersion, flash._stream()) == ok
    torch.cuda.synchronize()
    # neither torch's allocator nor the device itself (hipMemGetInfo: a hipMalloc inside the library would show) gave memory
    assert torch.cuda.memory_allocated() == before
    assert torch.cuda.mem_get_info()[0] >= free_before
    for name, g, r in zip(('dq', 'dk', 'dv'), got, ref):
        assert not torch.isnan(g.float()).any(), name
        assert torch.equal(g, r), name


def test_two_calls_in_a_row_second_smaller(recomputing_backward):
    _run_pair(2, 4, 2, 1000, 777, 128, torch.bfloat16, True, seed=11)
    _run_pair(1, 2, 2, 130, 200, 64, torch.float16, False, seed=12)


def test_rejects_more_rows_than_the_array_holds():
    from aotriton_amd import flash
    from aotriton_amd.pyaotriton.v3.flash import attn_bwd_noalloc, attn_bwd_params
    # 4 * 1024 * 1024 delta values are the limit: one batch element, 8 heads, 2^19 + 8 rows
    B, H, S, D = 1, 8, (1 << 19) + 8, 64
    q = torch.zeros(B, H, S, D, device=DEV, dtype=torch.bfloat16)
    L = torch.zeros(B * H, S, device=DEV, dtype=torch.float32)
    null = torch.empty([0], device=DEV, dtype=torch.uint64)
    params = attn_bwd_params()
    flash._fill_bwd(params, q, q, q, None, 0.125, q, q, q, q, q, None, None, L, None, 0.0, null, null, 0, False)
    assert attn_bwd_noalloc(params, attn_bwd_params.kVersion, flash._stream()) == flash.hipError_t.hipErrorOutOfMemory
    assert attn_bwd_noalloc(params, attn_bwd_params.kVersion + 1, flash._stream()) == flash.hipError_t.hipErrorInvalidSymbol
