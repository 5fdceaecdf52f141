"""GPU parity tests: HIP kernels (through the C ABI) against the CPU-restated
oracle run in fp32 on the same seeded inputs.  Tolerances are the reference's
(tests/_util.py).  Case grid mirrors the reference's default `test_fast` grid
(modules/flash/tests/test_backward.py:34-49) at the built head dims: ragged Sq/Sk,
GQA, BSHD strides, causal on/off, dropout on/off, fp16/bf16."""
import math

import numpy as np

import pytest
import torch

from _util import FUDGE, LSE_ATOL, check, keep_mask_from_oracle, make_inputs

pytestmark = pytest.mark.gpu

DEV = 'cuda'


def _run_case(B, Hq, Hk, Sq, Sk, D, dtype, causal, dropout_p=0.0, bias=False, bshd=False,
              bwd_backend=-1, sm_scale=None, seed=0, bias_layout='padded', Dv=None, philox=None):
    from aotriton_amd import flash
    from aotriton_amd.autograd import attention, AttentionExtraArgs
    from oracle import fa_ref
    q, k, v, b, do = make_inputs(B, Hq, Hk, Sq, Sk, D, dtype, DEV, seed=seed, bias=bias, bshd=bshd,
                                 bias_layout=bias_layout, Dv=Dv)
    sm_scale = 1.0 / math.sqrt(D) if sm_scale is None else sm_scale
    ext = AttentionExtraArgs(return_logsumexp=True, fillnan=True, bwd_backend=bwd_backend)
    if philox is not None:
        ext.philox_seed, ext.philox_offset1, ext.philox_offset2 = philox
    qg, kg, vg = [t.clone().requires_grad_() for t in (q, k, v)]
    bg = b.detach().requires_grad_() if b is not None else None      # keeps the strides of b
    o, _, L = attention(qg, kg, vg, bg, causal, sm_scale, dropout_p, ext)
    o.backward(do)
    torch.cuda.synchronize()
    assert flash.hipGetLastError() == flash.hipError_t.hipSuccess

    ct, wl, wr = flash.translate_causal(causal)
    keep = keep_mask_from_oracle(B, Hq, Sq, Sk, dropout_p, ext.philox_seed,
                                 ext.philox_offset1 + ext.philox_offset2, DEV)
    hp = torch.float64 if dtype == torch.float32 else torch.float32      # _common_test.py:347
    f32 = lambda t: None if t is None else t.to(hp)
    ro, rl, _ = fa_ref.attn_fwd_ref(f32(q), f32(k), f32(v), f32(b), sm_scale, ct, wl, wr, dropout_p, keep)
    lo, ll, _ = fa_ref.attn_fwd_ref(q, k, v, b, sm_scale, ct, wl, wr, dropout_p, keep)
    live = torch.isfinite(rl)
    check('out', o, ro, lo, FUDGE['out'])
    Lv = L.view(B, Hq, Sq)
    assert torch.equal(torch.isinf(Lv), ~live), 'LSE must be +inf exactly on rows with no visible key'
    assert not bool(live.any()) or (Lv[live] - rl[live]).abs().max().item() <= LSE_ATOL
    rg = fa_ref.attn_bwd_ref(f32(q), f32(k), f32(v), f32(b), sm_scale, ro, f32(do), rl, ct, wl, wr, dropout_p, keep)
    lg = fa_ref.attn_bwd_ref(q, k, v, b, sm_scale, lo, do, ll.to(q.dtype).float().to(q.dtype), ct, wl, wr,
                             dropout_p, keep)
    check('dq', qg.grad, rg[0], lg[0], FUDGE['dq'])
    check('dk', kg.grad, rg[1], lg[1], FUDGE['dk'])
    check('dv', vg.grad, rg[2], lg[2], FUDGE['dv'])
    if b is not None:
        check('db', bg.grad, rg[3], lg[3], FUDGE['db'])


DTYPES = [torch.bfloat16, torch.float16]


@pytest.mark.parametrize('dtype', DTYPES)
@pytest.mark.parametrize('D', [64, 128, 256])
@pytest.mark.parametrize('causal', [False, True])
@pytest.mark.parametrize('backend', [0, 1])
def test_dense_square(dtype, D, causal, backend):
    _run_case(2, 4, 4, 256, 256, D, dtype, causal, bwd_backend=backend)


@pytest.mark.parametrize('dtype', DTYPES)
@pytest.mark.parametrize('D', [64, 128, 256])
@pytest.mark.parametrize('sq,sk', [(11, 31), (523, 337), (203, 1063), (128, 77)])
@pytest.mark.parametrize('causal', [False, True])
def test_ragged_gqa_bshd(dtype, D, sq, sk, causal):
    # B=3, heads (10,2), BSHD storage: the reference's default grid
    _run_case(3, 10, 2, sq, sk, D, dtype, causal, bshd=True, sm_scale=1.0 / D)


@pytest.mark.parametrize('D', [64, 128])
@pytest.mark.parametrize('causal', [False, True, (17, 5), 2])
@pytest.mark.parametrize('backend', [0, 1])
def test_dropout(D, causal, backend):
    _run_case(2, 5, 5, 197, 223, D, torch.float16, causal, dropout_p=0.5, bwd_backend=backend)


@pytest.mark.parametrize('backend', [0, 1])
def test_dropout_with_64_bit_seed_and_offsets(backend):
    # forward, dK/dV and dQ kernels must draw the same mask from a seed and offsets that use all 64 bits
    _run_case(2, 4, 2, 130, 259, 128, torch.bfloat16, True, dropout_p=0.3, bwd_backend=backend,
              philox=(0xDEADBEEF12345678, (1 << 32) - 2, (1 << 40) + 7))


@pytest.mark.parametrize('D', [64, 128, 256])
@pytest.mark.parametrize('causal', [False, (40, 0), True])
@pytest.mark.parametrize('backend', [0, 1])
def test_bias_and_db(D, causal, backend):
    _run_case(2, 3, 3, 150, 201, D, torch.float16, causal, bias=True, bwd_backend=backend)


@pytest.mark.parametrize('backend', [0, 1])
def test_bias_rows_without_vector_alignment(backend):
    # bias whose rows are not 8- or 16-byte aligned: the kernels fall back to element access
    _run_case(2, 2, 2, 150, 201, 128, torch.float16, (40, 0), bias=True, bwd_backend=backend, bias_layout='odd')


def test_window_bias_dropout_small_config5():
    # the D = 256 benchmark configuration at a size the oracle handles: window (left, 0) + bias + dropout 0.1
    _run_case(1, 2, 2, 384, 384, 256, torch.float16, (100, 0), dropout_p=0.1, bias=True)


@pytest.mark.parametrize('D', [16, 40, 80, 96, 160, 192, 224])
@pytest.mark.parametrize('causal', [False, True])
@pytest.mark.parametrize('backend', [0, 1])
def test_head_dims_rounded_up(D, causal, backend):
    # head dims between the compiled ones run on the next larger kernel with the excess
    # columns masked (the reference's PADDED_HEAD, modules/flash/csrc/attn_fwd.cc:76-82,109)
    _run_case(2, 4, 2, 203, 171, D, torch.bfloat16, causal, bwd_backend=backend, bshd=(D % 32 == 0))


def test_head_dim_rounded_up_with_bias_dropout_varlen_strides():
    _run_case(1, 2, 2, 130, 130, 72, torch.float16, (30, 0), dropout_p=0.3, bias=True)


@pytest.mark.parametrize('D,Dv', [(192, 128), (128, 64), (64, 128), (40, 72), (96, 256), (256, 8)])
@pytest.mark.parametrize('causal', [False, True])
@pytest.mark.parametrize('backend', [0, 1])
def test_head_dims_of_qk_and_v_differ(D, Dv, causal, backend):
    # Q/K with D columns, V/Out/dOut with Dv (hdim_qk != hdim_vo, modules/flash/csrc/attn_fwd.cc:76-82):
    # both run on the compiled head dim that holds the larger one
    _run_case(2, 4, 2, 203, 171, D, torch.float16 if D == 40 else torch.bfloat16, causal, bwd_backend=backend, Dv=Dv)


def test_head_dims_of_qk_and_v_differ_with_bias_and_dropout():
    _run_case(1, 2, 1, 140, 150, 192, torch.bfloat16, (40, 3), dropout_p=0.2, bias=True, Dv=128)


def test_fp32_baseline_config_1():
    # B2 H4 S128 D64 fp32 non-causal: the reference's CPU-runnable configuration, on the GPU
    _run_case(2, 4, 4, 128, 128, 64, torch.float32, False, sm_scale=1.0 / 8)


@pytest.mark.parametrize('case', [
    dict(D=64, causal=True), dict(D=128, causal=(13, 4), Hk=2, sq=203, sk=171, bshd=True),
    dict(D=256, causal=2, sq=90, sk=150), dict(D=128, causal=True, bias=True, dropout_p=0.25, sq=150, sk=150),
    dict(D=40, causal=False, Dv=72, Hk=1, sq=77, sk=129), dict(D=128, causal=1, sq=300, sk=140),
])
def test_fp32_inputs(case):
    # fp32 tensors run on the fp32 MFMA kernels; the oracle is fp64 against fp32
    c = dict(Hk=4, sq=128, sk=128, bias=False, dropout_p=0.0, bshd=False, Dv=None)
    c.update(case)
    _run_case(2, 4, c['Hk'], c['sq'], c['sk'], c['D'], torch.float32, c['causal'], dropout_p=c['dropout_p'],
              bias=c['bias'], bshd=c['bshd'], Dv=c['Dv'], bwd_backend=0)


@pytest.mark.parametrize('causal', [False, True, (70, 33)])
@pytest.mark.parametrize('D,Dv,p,bias', [(128, None, 0.0, False), (256, 200, 0.1, False), (72, 256, 0.0, True),
                                         (192, None, 0.3, True), (512, None, 0.0, False), (384, 272, 0.1, False),
                                         (264, 512, 0.0, True), (448, None, 0.3, True)])
def test_fp32_mfma_kernels(causal, D, Dv, p, bias):
    # several 32-row tiles each way, ragged ends, grouped heads, every combination of mask, bias
    # (with dB) and dropout, on the three compiled widths (128, 256 and 512 columns)
    if bias and causal is True:
        causal = (1000, 0)       # the same mask through the window arguments
    _run_case(2, 6, 2, 203, 261, D, torch.float32, causal, Dv=Dv, dropout_p=p, bias=bias, bwd_backend=0)


@pytest.mark.parametrize('dtype', [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize('D,Dv', [(512, None), (320, 264), (128, 512)])
def test_head_dims_up_to_512(dtype, D, Dv):
    # above 256 the 16-bit types run on the kernels that split the head dim over the waves, fp32 on
    # the 512-column build of its MFMA kernels (the reference compiles head dim 512, modules/flash/aot/_common.py:10-14)
    _run_case(1, 4, 2, 150, 131, D, dtype, (40, 0), Dv=Dv, bwd_backend=0)


@pytest.mark.parametrize('dtype', [torch.bfloat16, torch.float16])
@pytest.mark.parametrize('causal', [False, True, (70, 33)])
@pytest.mark.parametrize('D,Dv,p,bias', [(512, None, 0.0, False), (384, 272, 0.1, False), (264, 512, 0.0, True),
                                         (448, None, 0.3, True)])
def test_split_head_dim_kernels(dtype, causal, D, Dv, p, bias):
    # several tiles of 32 rows each way, ragged ends, grouped heads, every combination of mask,
    # bias (with dB) and dropout
    if bias and causal is True:
        causal = (1000, 0)       # the same mask through the window arguments
    _run_case(2, 6, 2, 203, 261, D, dtype, causal, Dv=Dv, dropout_p=p, bias=bias, bwd_backend=0)


@pytest.mark.parametrize('dtype', [torch.bfloat16, torch.float32])
@pytest.mark.parametrize('sk', [1, 31, 33, 64, 65])
def test_head_dim_512_with_one_to_three_key_tiles(dtype, sk):
    # the kernels of head dims above 256 stream 32-key tiles through two K stages: one tile (nothing to
    # prefetch), two (each stage used once) and three (the first stage reused)
    _run_case(1, 2, 1, 70, sk, 512, dtype, False, bwd_backend=0)
    _run_case(1, 2, 1, 70, sk, 384, dtype, (1000, 5), bwd_backend=0)


def test_head_dim_512_with_bias_and_dropout():
    _run_case(1, 2, 2, 100, 100, 512, torch.bfloat16, True, dropout_p=0.2, bias=True, bwd_backend=0)


@pytest.mark.parametrize('dtype,D', [(torch.float32, 64), (torch.bfloat16, 512), (torch.float32, 300)])
def test_backend_1_where_no_single_launch_kernel_exists(dtype, D):
    """The reference compiles its fused backward for fp32 too (modules/flash/aot/bwd_kernel_fuse.py:25-28).
    Here fp32 tensors and head dims above 256 have split kernels only; a call for backend 1, which brings
    no delta buffer (v2 attn_bwd_fused), runs them with delta in the library's workspace: same results as
    backend 0, bit for bit.  Without workspace the call is refused."""
    from aotriton_amd import flash
    from aotriton_amd._lib import lib
    ok = flash.hipError_t.hipSuccess
    B, H, Sq, Sk = 2, 2, 100, 77
    q, k, v, _, do = make_inputs(B, H, H, Sq, Sk, D, dtype, DEV, seed=3)
    sm = D ** -0.5
    null = torch.empty([0], device=DEV, dtype=torch.uint64)
    atomic = torch.zeros([1], device=DEV, dtype=torch.int32)
    o = torch.empty_like(q)
    L = torch.empty(B * H, Sq, device=DEV, dtype=torch.float32)
    assert flash.attn_fwd(q, k, v, None, sm, L, o, 0.0, null, null, 0, null, null, None, True, atomic) == ok
    want = [torch.empty_like(t) for t in (q, k, v)]
    delta = torch.empty_like(L)
    ext = flash.attn_options()
    ext.force_backend_index = 0
    assert flash.attn_bwd(q, k, v, None, sm, o, do, *want, None, None, L, delta, 0.0, null, null, 0, True,
                          extargs=ext) == ok
    got = [torch.full_like(t, float('nan')) for t in (q, k, v)]
    assert flash.attn_bwd_fused(q, k, v, None, sm, o, do, *got, None, L, 0.0, null, null, 0, True) == ok
    torch.cuda.synchronize()
    for name, x, y in zip(('dq', 'dk', 'dv'), got, want):
        assert torch.equal(x, y), name
    lib.fa_set_bwd_workspace_limit(0)
    try:
        assert flash.attn_bwd_fused(q, k, v, None, sm, o, do, *got, None, L, 0.0, null, null, 0, True) == \
            flash.hipError_t.hipErrorPeerAccessUnsupported
    finally:
        lib.fa_set_bwd_workspace_limit(-1)


@pytest.mark.parametrize('D,dtype', [(113, torch.bfloat16), (71, torch.float16)])
def test_fused_backend_on_a_head_dim_that_is_no_multiple_of_8(D, dtype):
    """The reference's fused backward takes any head dim (modules/flash/csrc/attn_bwd.cc:55-160 with the padding
    of attn_fwd.cc:76-82).  Here it runs on packed copies; a call without workspace is refused when the backend
    is forced (the element-wise kernels have the split backend only)."""
    from aotriton_amd.autograd import attention, AttentionExtraArgs
    from aotriton_amd._lib import lib
    _run_case(2, 4, 2, 150, 131, D, dtype, True, dropout_p=0.1, bwd_backend=1, seed=D)
    lib.fa_set_bwd_workspace_limit(0)
    try:
        q, k, v, _, do = make_inputs(1, 2, 2, 64, 64, D, dtype, DEV)
        qg = q.clone().requires_grad_()
        o, _, _ = attention(qg, k, v, None, False, 0.125, 0.0, AttentionExtraArgs(bwd_backend=1))
        with pytest.raises(NotImplementedError):
            o.backward(do)
    finally:
        lib.fa_set_bwd_workspace_limit(-1)


def _sampled_grid_cases(n=72, seed=2024):
    """A seeded sample of the reference's test grids (tests/test_backward.py:35-142 with the
    lists of tests/_core_test_backward.py:60-89): regular, matrix bias, GQA, irregular
    (prime) sequence lengths and Dqk != Dv, over all dtypes, both storage orders, both
    scales and both backward backends.  Sequence lengths above 2048 are left out and a
    dropout case keeps Sq*Sk small (its mask comes from the CPU oracle)."""
    import random
    rnd = random.Random(seed)
    hd_all = sorted(set([16, 32, 64, 128, 256, 512, 48, 80, 96, 160, 192, 224,
                         8, 24, 40, 56, 72, 88, 96, 120, 152, 184, 216, 248, 408]))
    regular = [8, 16, 32, 64, 128, 256, 512, 1024, 2048]
    prime_q = [11, 17, 37, 67, 157, 257, 523, 1033]
    prime_k = [13, 31, 41, 71, 223, 337, 571, 1063]
    cases = []
    for i in range(n):
        fam = ['regular', 'bias', 'gqa', 'irregular', 'qk_ne_vo'][i % 5]
        dtype = rnd.choice([torch.float16, torch.bfloat16, torch.float32])
        D = rnd.choice(hd_all); Dv = None
        heads = (5, 5); bias = False; flip = rnd.random() < 0.5
        causal = rnd.random() < 0.5
        scale = rnd.choice(['l1', 'l2'])
        if fam == 'regular':
            sq, sk = rnd.choice(regular), rnd.choice(regular)
        elif fam == 'bias':
            sq, sk = rnd.choice(regular), rnd.choice(regular); bias = True; causal = False; scale = 'l1'
        elif fam == 'gqa':
            heads = rnd.choice([(16, 8), (10, 2)]); flip = False
            sq, sk = rnd.choice([4, 143, 2048]), rnd.choice([4, 127, 579, 2048])
        elif fam == 'irregular':
            sq, sk = rnd.choice(prime_q), rnd.choice(prime_k); bias = rnd.random() < 0.5
        else:
            sq, sk = rnd.choice(prime_q[:7]), rnd.choice(prime_k[:7]); bias = rnd.random() < 0.5
            Dv = rnd.choice(hd_all); flip = False; scale = 'l1'
        if bias:
            causal = False          # the reference skips causal with an explicit bias
        p = rnd.choice([0.0, 0.5])
        if p > 0.0 and sq * sk > 600 * 600:
            p = 0.0
        if dtype == torch.float32 and max(D, Dv or 0) > 256 and sq * sk > 1024 * 1024:
            sq, sk = min(sq, 512), min(sk, 512)      # keep the fp64 oracle of the case short
        split_only = dtype == torch.float32 or max(D, Dv or 0) > 256
        backend = 0 if split_only else rnd.choice([0, 1])
        cases.append((fam, heads, D, Dv, sq, sk, causal, p, dtype, flip, bias, scale, backend))
    return cases


def _case_id(c):
    fam, heads, D, Dv, sq, sk, causal, p, dtype, flip, bias, scale, backend = c
    return (f"{fam}-h{heads[0]}_{heads[1]}-d{D}{'_%d' % Dv if Dv else ''}-q{sq}-k{sk}-{'c' if causal else 'n'}"
            f"-p{p}-{str(dtype)[6:]}-{'bshd' if flip else 'bhsd'}-{'bias' if bias else 'nobias'}-{scale}-be{backend}")


@pytest.mark.parametrize('case', _sampled_grid_cases(), ids=_case_id)
def test_sample_of_the_reference_grids(case):
    fam, heads, D, Dv, sq, sk, causal, p, dtype, flip, bias, scale, backend = case
    sm = 1.0 / D if scale == 'l1' else 1.0 / math.sqrt(D)
    _run_case(3, heads[0], heads[1], sq, sk, D, dtype, causal, dropout_p=p, bias=bias, bshd=flip,
              bwd_backend=backend, sm_scale=sm, seed=20, Dv=Dv)


def _layout_case(i, seed=3):
    import random
    from aotriton_amd.flash import CausalType
    rnd = random.Random(seed * 100003 + i)
    c = dict(i=i)
    c['B'] = rnd.choice([1, 2, 3]); c['Hk'] = rnd.choice([1, 2, 3]); c['Hq'] = c['Hk'] * rnd.choice([1, 1, 2, 4])
    c['D'] = rnd.choice([16, 40, 64, 72, 128, 160, 256])
    c['Dv'] = c['D'] if rnd.random() < 0.8 else rnd.choice([32, 64, 128])
    lens = [1, 2, 7, 31, 64, 65, 127, 128, 129, 200, 256, 257, 383, 512, 700]
    c['sq'] = rnd.choice(lens); c['sk'] = rnd.choice(lens)
    c['dtype'] = rnd.choice([torch.float16, torch.bfloat16, torch.float32])
    c['layout'] = rnd.choice(['bhsd', 'bshd', 'qkv', 'gap'])
    c['bias'] = rnd.choice([None, None, 'full', 'odd', 'bcast_b', 'bcast_h', 'bcast_bh', 'bcast_m'])
    r = rnd.random()
    c['causal'] = False if r < 0.3 else (True if r < 0.55 else (
        (rnd.randint(-3, c['sq']), rnd.randint(-3, c['sk'])) if r < 0.8 else CausalType.BOTTOM_RIGHT))
    c['p'] = rnd.choice([0.0, 0.0, 0.2]) if c['sk'] > 1 else 0.0
    split_only = c['dtype'] == torch.float32 or max(c['D'], c['Dv']) > 256
    c['be'] = 0 if split_only else rnd.choice([0, 1])
    c['sm'] = rnd.choice([1.0 / c['D'], c['D'] ** -0.5])
    return c


@pytest.mark.parametrize('i', range(64))
def test_sampled_strides_bias_layouts_and_masks(i):
    """Seeded cases over what the callers' tensors look like: BHSD, BSHD, q/k/v as slices of one
    packed (B, S, 3, H, D) tensor, rows wider than the head dim; bias padded, with odd row
    stride, broadcast along batch, heads, both or the query rows; windows, both causal
    alignments and dropout on top; sequence lengths from 1 to 700."""
    from aotriton_amd import flash
    from aotriton_amd.autograd import attention, AttentionExtraArgs
    from oracle import fa_ref
    c = _layout_case(i)
    B, Hq, Hk, D, Dv, sq, sk, dtype = (c[x] for x in ('B', 'Hq', 'Hk', 'D', 'Dv', 'sq', 'sk', 'dtype'))
    g = torch.Generator().manual_seed(1000 + i)
    rn = lambda *s, scale=1.0: (torch.randn(*s, generator=g) * scale).to(dtype).to(DEV)
    if c['layout'] == 'qkv' and Hq == Hk and D == Dv and sq == sk:
        qkv = rn(B, sq, 3, Hq, D)
        q, k, v = [qkv[:, :, j].transpose(1, 2) for j in range(3)]
    elif c['layout'] == 'bshd':
        q = rn(B, sq, Hq, D).transpose(1, 2); k = rn(B, sk, Hk, D).transpose(1, 2); v = rn(B, sk, Hk, Dv).transpose(1, 2)
    elif c['layout'] == 'gap':
        q = rn(B, Hq, sq, D + 24)[..., 8:8 + D]; k = rn(B, Hk, sk, D + 8)[..., :D]; v = rn(B, Hk, sk, Dv + 16)[..., 16:]
    else:
        q = rn(B, Hq, sq, D); k = rn(B, Hk, sk, D); v = rn(B, Hk, sk, Dv)
    do = rn(B, Hq, sq, Dv)
    kind, b = c['bias'], None
    if kind == 'full': b = rn(B, Hq, sq, (sk + 7) // 8 * 8, scale=0.5)[..., :sk]
    elif kind == 'odd': b = rn(B, Hq, sq, sk + 3, scale=0.5)[..., 1:sk + 1]
    elif kind == 'bcast_b': b = rn(1, Hq, sq, sk, scale=0.5).expand(B, Hq, sq, sk)
    elif kind == 'bcast_h': b = rn(B, 1, sq, sk, scale=0.5).expand(B, Hq, sq, sk)
    elif kind == 'bcast_bh': b = rn(1, 1, sq, sk, scale=0.5).expand(B, Hq, sq, sk)
    elif kind == 'bcast_m': b = rn(B, Hq, 1, sk, scale=0.5).expand(B, Hq, sq, sk)
    need_db = kind in ('full', 'odd')
    causal, p, sm = c['causal'], c['p'], c['sm']
    ext = AttentionExtraArgs(return_logsumexp=True, fillnan=True, bwd_backend=c['be'])
    qg, kg, vg = [t.detach().requires_grad_() for t in (q, k, v)]     # keeps the strides
    bg = b.detach().requires_grad_() if need_db else b
    o, _, L = attention(qg, kg, vg, bg, causal, sm, p, ext)
    o.backward(do)
    torch.cuda.synchronize()
    ct, wl, wr = flash.translate_causal(causal)
    keep = keep_mask_from_oracle(B, Hq, sq, sk, p, ext.philox_seed, ext.philox_offset1 + ext.philox_offset2, DEV)
    hp = torch.float64 if dtype == torch.float32 else torch.float32
    f = lambda t: None if t is None else t.to(hp)
    ro, rl, _ = fa_ref.attn_fwd_ref(f(q), f(k), f(v), f(b), sm, ct, wl, wr, p, keep)
    lo, ll, _ = fa_ref.attn_fwd_ref(q, k, v, b, sm, ct, wl, wr, p, keep)
    live = torch.isfinite(rl)
    check('out', o, ro, lo, FUDGE['out'])
    Lv = L.view(B, Hq, sq)
    assert torch.equal(torch.isinf(Lv), ~live)
    assert not bool(live.any()) or (Lv[live] - rl[live]).abs().max().item() <= LSE_ATOL
    rg = fa_ref.attn_bwd_ref(f(q), f(k), f(v), f(b), sm, ro, f(do), rl, ct, wl, wr, p, keep)
    lg = fa_ref.attn_bwd_ref(q, k, v, b, sm, lo, do, ll.to(q.dtype), ct, wl, wr, p, keep)
    check('dq', qg.grad, rg[0], lg[0], FUDGE['dq'])
    check('dk', kg.grad, rg[1], lg[1], FUDGE['dk'])
    check('dv', vg.grad, rg[2], lg[2], FUDGE['dv'])
    if need_db:
        check('db', bg.grad, rg[3], lg[3], FUDGE['db'])


@pytest.mark.parametrize('D', [7, 23, 37, 53, 67, 73, 89, 113, 149, 179, 211, 241, 203, 300, 509])
def test_head_dims_that_are_no_multiple_of_8(D, with_and_without_workspace):
    """The reference rounds ANY head dim up to a compiled one and masks the excess columns
    (modules/flash/csrc/attn_fwd.cc:76-82,109); its test grid includes the primes below
    (modules/flash/tests/test_forward.py:22,92).  Rows of such tensors are not made of aligned 16-byte
    pieces: they reach the MFMA kernels as packed copies in the library's workspace, or, without
    workspace, run on the kernels that move single elements (split backend)."""
    dtype = [torch.bfloat16, torch.float16, torch.float32][D % 3]
    causal = [False, True, (9, 4)][(D // 3) % 3]
    _run_case(2, 4, 2, 70, 83, D, dtype, causal, dropout_p=0.2 if D % 2 else 0.0, bias=D % 5 == 0, bwd_backend=0, seed=D)


@pytest.mark.parametrize('dtype', [torch.bfloat16, torch.float32])
@pytest.mark.parametrize('how', ['base', 'row_stride', 'head_stride'])
def test_rows_that_are_not_16_byte_aligned(dtype, how, with_and_without_workspace):
    """Head dim 64, but a base address that is only element-aligned, a row stride of 65 or a head stride
    that is no multiple of 8: packed copies or the element-wise kernels, same results as the oracle."""
    from aotriton_amd import flash
    from aotriton_amd.autograd import attention, AttentionExtraArgs
    from oracle import fa_ref
    B, Hq, Hk, Sq, Sk, D = 2, 2, 2, 45, 61, 64
    g = torch.Generator().manual_seed(3)
    def mk(H, S):
        if how == 'base':
            return torch.randn(B * H * S * D + 1, generator=g).to(dtype).to(DEV)[1:].view(B, H, S, D)
        if how == 'row_stride':
            return torch.randn(B, H, S, D + 1, generator=g).to(dtype).to(DEV)[..., :D]
        return torch.randn(B, H, S * D + 3, generator=g).to(dtype).to(DEV)[..., :S * D].view(B, H, S, D)
    q, k, v, do = mk(Hq, Sq), mk(Hk, Sk), mk(Hk, Sk), mk(Hq, Sq)
    sm = D ** -0.5
    ext = AttentionExtraArgs(return_logsumexp=True, fillnan=True, bwd_backend=0)
    qg, kg, vg = [t.detach().requires_grad_() for t in (q, k, v)]
    o, _, L = attention(qg, kg, vg, None, True, sm, 0.0, ext)
    o.backward(do)
    torch.cuda.synchronize()
    ct, wl, wr = flash.translate_causal(True)
    hp = torch.float64 if dtype == torch.float32 else torch.float32
    f = lambda t: t.to(hp)
    ro, rl, _ = fa_ref.attn_fwd_ref(f(q), f(k), f(v), None, sm, ct, wl, wr, 0.0, None)
    lo, ll, _ = fa_ref.attn_fwd_ref(q, k, v, None, sm, ct, wl, wr, 0.0, None)
    check('out', o, ro, lo, FUDGE['out'])
    rg = fa_ref.attn_bwd_ref(f(q), f(k), f(v), None, sm, ro, f(do), rl, ct, wl, wr, 0.0, None)
    lg = fa_ref.attn_bwd_ref(q, k, v, None, sm, lo, do, ll.to(q.dtype), ct, wl, wr, 0.0, None)
    check('dq', qg.grad, rg[0], lg[0], FUDGE['dq'])
    check('dk', kg.grad, rg[1], lg[1], FUDGE['dk'])
    check('dv', vg.grad, rg[2], lg[2], FUDGE['dv'])


@pytest.mark.parametrize('dtype,D', [(torch.bfloat16, 64), (torch.float16, 128), (torch.bfloat16, 256), (torch.bfloat16, 512),
                                     (torch.float32, 128), (torch.float32, 320), (torch.bfloat16, 72)])
@pytest.mark.parametrize('causal', [False, True])
def test_delta_is_the_row_sum_of_o_times_do(dtype, D, causal):
    """bwd_preprocess (modules/flash/kernel/bwd_preprocess.py:28-133): delta[z, h, m] = sum_d fp32(O) fp32(dO),
    laid out like the LSE.  The split backward leaves it in the caller's buffer whichever kernel computes it
    (the dQ kernel at head dims up to 256, the preprocess kernel otherwise), and the preprocess kernel
    launched on its own writes the same.  Closed form, computed here in fp64."""
    from aotriton_amd import flash
    from aotriton_amd.pyaotriton.v3.flash import attn_bwd_kernel, attn_bwd_params
    B, Hq, Hk, Sq, Sk = 2, 4, 2, 203, 261
    q, k, v, _, do = make_inputs(B, Hq, Hk, Sq, Sk, D, dtype, DEV, seed=5)
    sm = 1.0 / math.sqrt(D)
    ok = flash.hipError_t.hipSuccess
    null = torch.empty([0], device=DEV, dtype=torch.uint64)
    o = torch.empty_like(q)
    L = torch.empty(B * Hq, Sq, device=DEV, dtype=torch.float32)
    atomic = torch.zeros([1], device=DEV, dtype=torch.int32)
    assert flash.attn_fwd(q, k, v, None, sm, L, o, 0.0, null, null, 0, null, null, None, causal, atomic) == ok
    want = (o.double() * do.double()).sum(-1).view(B * Hq, Sq)
    tol = 1e-5 * max(1.0, want.abs().max().item())
    dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    delta = torch.full_like(L, float('nan'))
    assert flash.attn_bwd(q, k, v, None, sm, o, do, dq, dk, dv, None, None, L, delta, 0.0, null, null, 0, causal) == ok
    torch.cuda.synchronize()
    assert (delta.double() - want).abs().max().item() <= tol
    alone = torch.full_like(L, float('nan'))
    bp = attn_bwd_params()
    flash._fill_bwd(bp, q, k, v, None, sm, o, do, dq, dk, dv, None, None, L, alone, 0.0, null, null, 0, causal)
    assert attn_bwd_kernel(bp, attn_bwd_params.kVersion, flash._stream(), 0) == ok
    torch.cuda.synchronize()
    assert (alone.double() - want).abs().max().item() <= tol


def test_concurrent_streams_and_threads_give_the_serial_results():
    """Calls are re-entrant and ordered only by the stream they are given: three host threads,
    each on its own stream with its own shape, repeat forward + backward; every result must
    equal the one computed alone on the default stream, bit for bit (both backends are
    deterministic)."""
    import threading
    from aotriton_amd.autograd import attention, AttentionExtraArgs
    shapes = [(2, 8, 4, 1024, 128, torch.bfloat16, True, 0), (1, 6, 6, 777, 64, torch.float16, False, 1),
              (3, 4, 1, 300, 256, torch.bfloat16, (50, 10), 0)]
    g = torch.Generator().manual_seed(9)
    cases = []
    for B, Hq, Hk, S, D, dtype, causal, be in shapes:
        rn = lambda *sh: torch.randn(*sh, generator=g).to(dtype).to(DEV)
        cases.append((rn(B, Hq, S, D), rn(B, Hk, S, D), rn(B, Hk, S, D), rn(B, Hq, S, D), causal, be, D))

    def run(case):
        q, k, v, do, causal, be, D = case
        qg, kg, vg = [t.clone().requires_grad_() for t in (q, k, v)]
        o, _, L = attention(qg, kg, vg, None, causal, D ** -0.5, 0.0,
                            AttentionExtraArgs(return_logsumexp=True, bwd_backend=be))
        o.backward(do)
        return [o.detach(), L, qg.grad, kg.grad, vg.grad]

    serial = [run(c) for c in cases]
    torch.cuda.synchronize()
    results = [None] * len(cases)
    errors = []

    def worker(i):
        try:
            st = torch.cuda.Stream()
            st.wait_stream(torch.cuda.default_stream())
            with torch.cuda.stream(st):
                for _ in range(5):
                    results[i] = run(cases[i])
            st.synchronize()
        except Exception as e:       # surfaces in the main thread
            errors.append(e)

    threads = [threading.Thread(target=worker, args=(i,)) for i in range(len(cases))]
    for t in threads: t.start()
    for t in threads: t.join()
    torch.cuda.synchronize()
    assert not errors, errors
    for a, b in zip(serial, results):
        for x, y in zip(a, b):
            assert torch.equal(x, y)


@pytest.mark.parametrize('causal', [1, 2])
def test_bottom_right_and_top_left_with_sq_gt_sk(causal):
    # rows with no visible key: O = 0, LSE = +inf, gradients finite
    _run_case(2, 2, 2, 300, 140, 128, torch.bfloat16, causal)


@pytest.mark.parametrize('dtype', [torch.bfloat16, torch.float32])
@pytest.mark.parametrize('backend', [0, 1])
@pytest.mark.parametrize('shape', [(0, 16, 16), (2, 0, 16), (2, 16, 0)])
def test_empty_tensors(shape, backend, dtype):
    # no batch element, no query row, no key: the calls succeed; without a key O = 0,
    # LSE = +inf and dQ = 0; without a query dK = dV = 0
    from aotriton_amd.autograd import attention, AttentionExtraArgs
    B, Sq, Sk = shape
    H, D = 2, 64
    q = torch.randn(B, H, Sq, D, device=DEV).to(dtype).requires_grad_()
    k = torch.randn(B, H, Sk, D, device=DEV).to(dtype).requires_grad_()
    v = torch.randn(B, H, Sk, D, device=DEV).to(dtype).requires_grad_()
    for causal in (False, True):
        q.grad = k.grad = v.grad = None
        ext = AttentionExtraArgs(return_logsumexp=True, fillnan=True, bwd_backend=backend)
        o, _, L = attention(q, k, v, None, causal, 0.125, 0.0, ext)
        o.backward(torch.randn(B, H, Sq, D, device=DEV).to(dtype))
        torch.cuda.synchronize()
        assert o.shape == (B, H, Sq, D) and L.shape == (B * H, Sq)
        assert torch.count_nonzero(o) == 0 and bool(torch.isposinf(L).all())
        for g, t in ((q.grad, q), (k.grad, k), (v.grad, v)):
            assert g.shape == t.shape and torch.count_nonzero(g) == 0 and not bool(torch.isnan(g).any())


@pytest.mark.parametrize('dtype', DTYPES)
@pytest.mark.parametrize('causal', [False, True])
def test_row_maximum_grows_along_keys(dtype, causal):
    # The score scale grows ~40x from the first to the last key, so every row's maximum
    # is overtaken again and again by later K tiles: a forward that reuses the maximum
    # of earlier tiles has to notice and renormalise.  Checked against the oracle.
    from aotriton_amd import flash
    from aotriton_amd.autograd import attention, AttentionExtraArgs
    from oracle import fa_ref
    B, H, S, D = 1, 2, 1024, 128
    q, k, v, _, do = make_inputs(B, H, H, S, S, D, dtype, DEV, seed=7)
    ramp = torch.linspace(0.25, 10.0, S, device=DEV).view(1, 1, S, 1)
    k = (k.float() * ramp).to(dtype)
    sm_scale = 1.0 / math.sqrt(D)
    ext = AttentionExtraArgs(return_logsumexp=True, fillnan=True)
    qg, kg, vg = [t.clone().requires_grad_() for t in (q, k, v)]
    o, _, L = attention(qg, kg, vg, None, causal, sm_scale, 0.0, ext)
    o.backward(do)
    torch.cuda.synchronize()
    assert flash.hipGetLastError() == flash.hipError_t.hipSuccess
    ct, wl, wr = flash.translate_causal(causal)
    ro, rl, _ = fa_ref.attn_fwd_ref(q.float(), k.float(), v.float(), None, sm_scale, ct, wl, wr, 0.0, None)
    lo, ll, _ = fa_ref.attn_fwd_ref(q, k, v, None, sm_scale, ct, wl, wr, 0.0, None)
    check('out', o, ro, lo, FUDGE['out'])
    assert (L.view(B, H, S) - rl).abs().max().item() <= LSE_ATOL * max(1.0, rl.abs().max().item() / 8)
    rg = fa_ref.attn_bwd_ref(q.float(), k.float(), v.float(), None, sm_scale, ro, do.float(), rl, ct, wl, wr, 0.0, None)
    lg = fa_ref.attn_bwd_ref(q, k, v, None, sm_scale, lo, do, ll.to(dtype).float().to(dtype), ct, wl, wr, 0.0, None)
    check('dq', qg.grad, rg[0], lg[0], FUDGE['dq'])
    check('dk', kg.grad, rg[1], lg[1], FUDGE['dk'])
    check('dv', vg.grad, rg[2], lg[2], FUDGE['dv'])


@pytest.mark.parametrize('mode', ['plain', 'causal', 'float_mask', 'bool_mask', 'gqa_bshd'])
def test_sdpa_entry_point_matches_torch_math(mode):
    # the F.scaled_dot_product_attention-shaped entry point against PyTorch's math SDPA in fp32
    import torch.nn.functional as F
    from torch.nn.attention import sdpa_kernel, SDPBackend
    from aotriton_amd.sdpa import scaled_dot_product_attention as sdpa
    B, H, L, S, E = 2, 4, 150, 201, 96
    dtype = torch.bfloat16
    g = torch.Generator().manual_seed(3)
    rn = lambda *s: torch.randn(*s, generator=g).to(dtype).to(DEV)
    hk = 2 if mode == 'gqa_bshd' else H
    if mode == 'gqa_bshd':
        q, k, v = rn(B, L, H, E).transpose(1, 2), rn(B, S, hk, E).transpose(1, 2), rn(B, S, hk, E).transpose(1, 2)
    else:
        q, k, v = rn(B, H, L, E), rn(B, hk, S, E), rn(B, hk, S, E)
    kw = {}
    if mode == 'causal':
        kw['is_causal'] = True
    elif mode == 'float_mask':
        kw['attn_mask'] = rn(1, 1, L, S) * 0.5            # broadcast over batch and heads
    elif mode == 'bool_mask':
        keep = torch.rand(B, 1, L, S, generator=g) > 0.3
        keep[..., 0] = True                                # no fully hidden row
        kw['attn_mask'] = keep.to(DEV)
    elif mode == 'gqa_bshd':
        kw['enable_gqa'] = True
    do = rn(*q.shape) if mode != 'gqa_bshd' else rn(B, L, H, E).transpose(1, 2)
    outs, grads = [], []
    for fn, cast in ((sdpa, lambda t: t), (F.scaled_dot_product_attention, lambda t: t.float()),
                     (F.scaled_dot_product_attention, lambda t: t)):
        qq, kk, vv = [cast(t).detach().clone().requires_grad_() for t in (q, k, v)]
        kw2 = dict(kw)
        if 'attn_mask' in kw2 and kw2['attn_mask'].dtype != torch.bool:
            kw2['attn_mask'] = cast(kw2['attn_mask'])
        if fn is sdpa:
            o = fn(qq, kk, vv, **kw2)
        else:
            with sdpa_kernel(SDPBackend.MATH):
                o = fn(qq, kk, vv, **kw2)
        o.backward(cast(do))
        outs.append(o); grads.append((qq.grad, kk.grad, vv.grad))
    check('out', outs[0], outs[1], outs[2], FUDGE['out'])
    for name, i in (('dq', 0), ('dk', 1), ('dv', 2)):
        check(name, grads[0][i], grads[1][i], grads[2][i], FUDGE[name])


@pytest.mark.gpu
def test_v2_positional_c_abi_matches_the_params_entry_points():
    """fa_v2_attn_fwd / attn_bwd / attn_bwd_fused / *_compact_varlen against fa_attn_fwd / fa_attn_bwd
    on the same inputs: bit-identical O, LSE, dQ, dK, dV."""
    from aotriton_amd import flash
    from aotriton_amd.pyaotriton.v2 import flash as v2
    mk = flash.mk_aotensor
    ok = flash.hipError_t.hipSuccess
    s = flash._stream()
    null = torch.empty([0], device=DEV, dtype=torch.uint64)
    B, Hq, Hk, Sq, Sk, D = 2, 4, 2, 300, 421, 128
    q, k, v, _, do = make_inputs(B, Hq, Hk, Sq, Sk, D, torch.bfloat16, DEV, seed=5)
    sm = 1.0 / math.sqrt(D)
    for causal in (False, True):
        o1, o2 = torch.empty_like(q), torch.empty_like(q)
        L1 = torch.empty(B * Hq, Sq, device=DEV, dtype=torch.float32)
        L2 = torch.empty_like(L1)
        atomic = torch.zeros([1], device=DEV, dtype=torch.int32)
        assert flash.attn_fwd(q, k, v, None, sm, L1, o1, 0.0, null, null, 0, null, null, None, causal, atomic) == ok
        assert v2.attn_fwd(mk(q), mk(k), mk(v), None, sm, mk(L2), mk(o2), 0.0, None, None, 0, None, None, None, causal,
                           mk(atomic), s) == ok
        assert torch.equal(o1, o2) and torch.equal(L1, L2)
        for fused in (False, True):
            g1 = [torch.empty_like(t) for t in (q, k, v)]
            g2 = [torch.empty_like(t) for t in (q, k, v)]
            delta = torch.empty_like(L1)
            ext = flash.attn_options()
            ext.force_backend_index = 1 if fused else 0
            assert flash.attn_bwd(q, k, v, None, sm, o1, do, g1[0], g1[1], g1[2], None, None, L1, delta, 0.0, null, null,
                                  0, causal, extargs=ext) == ok
            if fused:
                assert v2.attn_bwd_fused(mk(q), mk(k), mk(v), None, sm, mk(o1), mk(do), mk(g2[0]), mk(g2[1]), mk(g2[2]),
                                         None, mk(L1), 0.0, None, None, 0, causal, s) == ok
            else:
                assert v2.attn_bwd(mk(q), mk(k), mk(v), None, sm, mk(o1), mk(do), mk(g2[0]), mk(g2[1]), mk(g2[2]), None,
                                   mk(L1), mk(delta), 0.0, None, None, 0, causal, s) == ok
            for a, b in zip(g1, g2):
                assert torch.equal(a, b)
    # packed sequences
    lens = [100, 37, 256]
    cu = torch.tensor([0] + list(np.cumsum(lens)), dtype=torch.int32, device=DEV)
    T = sum(lens)
    qv, kv, vv, _, dov = make_inputs(1, Hq, Hk, T, T, D, torch.bfloat16, DEV, seed=6, bshd=True)
    o1, o2 = torch.empty_like(qv), torch.empty_like(qv)
    L1 = torch.empty(Hq, T, device=DEV, dtype=torch.float32)
    L2 = torch.empty_like(L1)
    atomic = torch.zeros([1], device=DEV, dtype=torch.int32)
    mx = max(lens)
    assert flash.attn_fwd_compact_varlen(qv, kv, vv, None, cu, cu, mx, mx, sm, L1, o1, 0.0, null, null, 0, null, null,
                                         None, True, atomic) == ok
    assert v2.attn_fwd_compact_varlen(mk(qv), mk(kv), mk(vv), None, mk(cu), mk(cu), mx, mx, sm, mk(L2), mk(o2), 0.0,
                                      None, None, 0, None, None, None, True, mk(atomic), s) == ok
    assert torch.equal(o1, o2) and torch.equal(L1, L2)
    g1 = [torch.empty_like(t) for t in (qv, kv, vv)]
    g2 = [torch.empty_like(t) for t in (qv, kv, vv)]
    delta = torch.empty_like(L1)
    assert flash.attn_bwd_compact_varlen(qv, kv, vv, cu, cu, mx, mx, None, sm, o1, dov, g1[0], g1[1], g1[2], None, L1,
                                         delta, 0.0, null, null, 0, True) == ok
    assert v2.attn_bwd_compact_varlen(mk(qv), mk(kv), mk(vv), mk(cu), mk(cu), mx, mx, None, sm, mk(o1), mk(dov),
                                      mk(g2[0]), mk(g2[1]), mk(g2[2]), None, mk(L1), mk(delta), 0.0, None, None, 0,
                                      True, s) == ok
    for a, b in zip(g1, g2):
        assert torch.equal(a, b)
