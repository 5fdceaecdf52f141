"""CPU tests of the C ABI: the library loads, exports every declared symbol, and
its pure-host argument checks / tile algebra behave as the header says.  No
compute call is made."""
import ctypes
import os
import random
import re

import pytest
import torch

from oracle import intervals as iv
from oracle import philox

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _lib():
    from aotriton_amd import _lib
    return _lib


def test_exports_every_declared_symbol():
    L = _lib()
    import glob
    hdr = '\n'.join(open(h).read() for h in sorted(glob.glob(os.path.join(ROOT, 'include', 'aotriton_amd', '*.h'))))
    declared = set(re.findall(r'FA_API\s+[\w\s\*]+?\b(fa_\w+)\s*\(', hdr))
    assert declared, 'no declarations parsed'
    assert declared == set(L.SYMBOLS), (declared ^ set(L.SYMBOLS))
    for name in declared:
        assert getattr(L.lib, name) is not None


def test_struct_layout_matches_header_order():
    L = _lib()
    names = [f[0] for f in L.fa_fwd_params._fields_]
    # attn_fwd_params member order, include/aotriton/flash.h:96-126 of the reference
    assert names == ['Q', 'K', 'V', 'B', 'A', 'Sm_scale', 'L', 'Out', 'cu_seqlens_q', 'cu_seqlens_k',
                     'Max_seqlen_q', 'Max_seqlen_k', 'seq_strides_q', 'seq_strides_k', 'dropout_p',
                     'philox_seed_ptr', 'philox_offset1', 'philox_offset2', 'philox_seed_output',
                     'philox_offset_output', 'encoded_softmax', 'persistent_atomic_counter',
                     'causal_type', 'varlen_type', 'window_left', 'window_right']
    assert ctypes.sizeof(L.fa_tensor4) == 80 and ctypes.sizeof(L.fa_tensor0) == 16


def test_suffix_and_threshold():
    from aotriton_amd import flash
    assert flash.get_name_suffix() != ''          # aotriton_flash.py:66-69 requires a suffix
    L = _lib()
    for p in (0.1, 0.2, 0.5, 0.0, 0.999):
        assert L.lib.fa_dropout_threshold(p) == philox.idropout_p(p)
    assert L.lib.fa_dropout_threshold(0.1) == -1717986944


def test_translate_causal_table():
    from aotriton_amd.flash import translate_causal, CausalType, WindowValue
    assert translate_causal(False) == (0, 0, 0)
    assert translate_causal(True) == (3, WindowValue.TOP_LEFT_ALIGNED, WindowValue.TOP_LEFT_ALIGNED)
    assert translate_causal((5, 7)) == (3, 5, 7)
    assert translate_causal(CausalType.TOP_LEFT) == (3, -2147483647, -2147483647)
    assert translate_causal(CausalType.BOTTOM_RIGHT) == (3, -2147483646, -2147483646)
    assert translate_causal(CausalType.NONE) == (0, 0, 0)


def test_mk_aotensor_ranks():
    from aotriton_amd import flash
    from aotriton_amd.pyaotriton import T0, T1, T2, T4, DType
    q = torch.zeros(2, 3, 4, 8, dtype=torch.float16)
    v = flash.mk_aotensor(q)
    assert isinstance(v, T4) and v.sizes == [2, 3, 4, 8] and v.strides == [96, 32, 8, 1] and v.dtype == DType.kFloat16
    assert isinstance(flash.mk_aotensor(torch.zeros(5, dtype=torch.int32)), T1)
    assert isinstance(flash.mk_aotensor(torch.zeros(2, 5)), T2)
    s = flash.mk_aotensor(torch.zeros(1, dtype=torch.uint64))
    assert isinstance(s, T0) and s.dtype == DType.kUInt64
    e = flash.mk_aotensor(torch.empty(0, dtype=torch.int32))
    assert isinstance(e, T0) and not e
    n = flash.mk_aotensor(None, if_empty_then_like=q)
    assert isinstance(n, T4) and not n and n.dtype == DType.kFloat16
    with pytest.raises(AssertionError):
        flash.mk_aotensor(q.transpose(2, 3))
    assert flash.cast_dtype(torch.bfloat16) == DType.kBFloat16
    assert flash.cast_dtype(torch.float32) == DType.kFloat32


def _fwd_params(D=128, dtype=torch.bfloat16, Hq=4, Hk=2, Sq=64, Sk=80, B=2, Dv=None):
    """Views over CPU tensors: fine for the pure-host checks (nothing is launched)."""
    from aotriton_amd import flash
    from aotriton_amd.pyaotriton.v3.flash import attn_fwd_params
    Dv = D if Dv is None else Dv
    keep = dict(q=torch.zeros(B, Hq, Sq, D, dtype=dtype), k=torch.zeros(B, Hk, Sk, D, dtype=dtype),
                v=torch.zeros(B, Hk, Sk, Dv, dtype=dtype), o=torch.zeros(B, Hq, Sq, Dv, dtype=dtype),
                M=torch.zeros(B * Hq, Sq))
    p = attn_fwd_params()
    p.Q = flash.mk_aotensor(keep['q']); p.K = flash.mk_aotensor(keep['k']); p.V = flash.mk_aotensor(keep['v'])
    p.Out = flash.mk_aotensor(keep['o']); p.L = flash.mk_aotensor(keep['M'])
    p.Sm_scale = 0.1
    return p, keep


def test_validate_fwd_error_contract():
    from aotriton_amd.pyaotriton import hipError_t as E, T4, T2, DType
    from aotriton_amd.pyaotriton.v3.flash import validate_fwd, attn_fwd_params, attn_options, query_fwd_config
    from aotriton_amd.flash import mk_aotensor as flash_mk
    p, keep = _fwd_params()
    assert validate_fwd(p, attn_fwd_params.kVersion) == E.hipSuccess
    assert validate_fwd(p, 2) == E.hipErrorInvalidSymbol                       # version gate
    p2, k2 = _fwd_params(D=96)
    assert validate_fwd(p2, 3) == E.hipSuccess                                 # rounded up to 128, columns masked
    err, cfg = query_fwd_config(p2)
    assert err == E.hipSuccess and cfg.head_dim == 128
    p5, k5 = _fwd_params(D=192, Dv=128)                                        # Dqk != Dv: the larger one picks the kernel
    err, cfg = query_fwd_config(p5)
    assert err == E.hipSuccess and cfg.head_dim == 256
    p6, k6 = _fwd_params(D=64, Dv=128)
    p6.Out = flash_mk(k6['q'])                                                 # Out must have V's head dim
    assert validate_fwd(p6, 3) == E.hipErrorInvalidValue
    p7, k7 = _fwd_params(D=512)                                                # above 256: the head dim split over the waves, 64 rows per workgroup
    err, cfg = query_fwd_config(p7)
    assert err == E.hipSuccess and cfg.head_dim == 512 and cfg.block_m == 64 and list(cfg.grid) == [16, 1, 1]
    pb, kb = _fwd_params(D=520)                                                # above 512
    assert validate_fwd(pb, 3) == E.hipErrorNotSupported
    for odd in (100, 7, 203):                                                  # rows that are not made of 16-byte pieces: element-wise kernels
        po, ko = _fwd_params(D=odd)
        err, cfg = query_fwd_config(po)
        assert err == E.hipSuccess and cfg.head_dim == {100: 128, 7: 64, 203: 256}[odd] and cfg.block_m == 32
        assert list(cfg.grid)[1:] == [po.Q.sizes[1], po.Q.sizes[0]]
    p3, k3 = _fwd_params(dtype=torch.float32)
    assert validate_fwd(p3, 3) == E.hipSuccess                                 # fp32: fp32 MFMA kernels
    p4, k4 = _fwd_params(Hq=5, Hk=2)
    assert validate_fwd(p4, 3) == E.hipErrorInvalidValue                       # heads not divisible
    p.Q = T4(0, [0] * 4, [0] * 4, DType.kBFloat16)
    assert validate_fwd(p, 3) == E.hipErrorInvalidValue                        # null Q
    p, keep = _fwd_params()
    p.K = T4(p.K.data_ptr, p.K.sizes, [p.K.stride(0), p.K.stride(1), 1 << 22, 1], p.K.dtype)
    assert validate_fwd(p, 3) == E.hipErrorNotSupported                        # row stride beyond 32-bit tile offsets
    p.K = T4(p.K.data_ptr, p.K.sizes, [p.K.stride(0), p.K.stride(1), -128, 1], p.K.dtype)
    assert validate_fwd(p, 3) == E.hipErrorNotSupported                        # negative stride
    p, keep = _fwd_params()
    bias = torch.zeros(2, 4, 64, 80, dtype=torch.bfloat16)
    p.B = flash_mk(bias)
    assert validate_fwd(p, 3) == E.hipSuccess
    p.B = T4(p.B.data_ptr, p.B.sizes, [p.B.stride(0), p.B.stride(1), (1 << 21) + 8, 1], p.B.dtype)
    assert validate_fwd(p, 3) == E.hipErrorNotSupported                        # bias row stride beyond 32-bit tile offsets
    p, keep = _fwd_params()
    rows, cols = p.L.sizes
    p.L = T2(p.L.data_ptr, [rows - 1, cols], [cols, 1], DType.kFloat32)
    assert validate_fwd(p, 3) == E.hipErrorInvalidValue                        # L too small for B*Hq rows
    p.L = T2(p.L.data_ptr, [rows, cols], [cols + 8, 1], DType.kFloat32)
    assert validate_fwd(p, 3) == E.hipErrorNotSupported                        # L rows not contiguous
    p, keep = _fwd_params()
    p.causal_type = 1
    assert validate_fwd(p, 3) == E.hipErrorNotSupported                        # only 0 and 3 exist
    p.causal_type = 3
    p.dropout_p = 0.5
    assert validate_fwd(p, 3) == E.hipErrorInvalidValue                        # dropout without a seed
    p.dropout_p = 0.0
    opt = attn_options(); opt.force_backend_index = 1
    assert validate_fwd(p, 3, opt) == E.hipErrorPeerAccessUnsupported          # forced unknown backend
    p.A = T2(1234, [1, 1], [1, 1], DType.kFloat32)
    assert validate_fwd(p, 3) == E.hipErrorNotSupported                        # alibi
    p, keep = _fwd_params()
    err, cfg = query_fwd_config(p)
    assert err == E.hipSuccess and cfg.block_m == 256 and cfg.head_dim == 128
    assert list(cfg.grid) == [16, 1, 1]     # persistent workgroups: 8 XCDs x min(CUs per XCD, 2 Q-tile slots per XCD)


def test_validate_bwd_error_contract():
    from aotriton_amd import flash
    from aotriton_amd.pyaotriton import hipError_t as E
    from aotriton_amd.pyaotriton.v3.flash import validate_bwd, attn_bwd_params, attn_options
    B, Hq, Hk, Sq, Sk, D = 2, 4, 2, 64, 80, 128
    dt = torch.float16
    q = torch.zeros(B, Hq, Sq, D, dtype=dt); k = torch.zeros(B, Hk, Sk, D, dtype=dt); v = torch.zeros_like(k)
    o = torch.zeros_like(q); do = torch.zeros_like(q); dq = torch.zeros_like(q)
    dk = torch.zeros_like(k); dv = torch.zeros_like(v)
    L = torch.zeros(B * Hq, Sq); delta = torch.zeros_like(L)
    null = torch.empty(0, dtype=torch.uint64)
    p = attn_bwd_params()
    flash._fill_bwd(p, q, k, v, None, 0.1, o, do, dq, dk, dv, None, None, L, delta, 0.0, null, null, 0, True)
    assert validate_bwd(p, attn_bwd_params.kVersion) == E.hipSuccess
    assert validate_bwd(p, 5) == E.hipErrorInvalidSymbol
    opt = attn_options(); opt.force_backend_index = 2                          # assembly backend of the reference
    assert validate_bwd(p, 6, opt) == E.hipErrorPeerAccessUnsupported
    opt.force_backend_index = 1
    assert validate_bwd(p, 6, opt) == E.hipSuccess
    p.D = None                                                                 # no delta: split cannot run
    opt.force_backend_index = 0
    assert validate_bwd(p, 6, opt) == E.hipErrorInvalidValue
    assert validate_bwd(p, 6) == E.hipSuccess                                  # library falls to fused


def test_tile_intervals_against_brute_force_and_reference_algebra():
    L = _lib()
    rnd = random.Random(99)
    out = (ctypes.c_int32 * 6)()
    for _ in range(3000):
        BM = rnd.choice([16, 32, 64]); BN = rnd.choice([16, 32, 64])
        sq = rnd.randint(1, 160); sk = rnd.randint(1, 160)
        causal = rnd.random() < 0.8
        if rnd.random() < 0.3:
            wl = wr = rnd.choice([iv.TOP_LEFT, iv.BOTTOM_RIGHT])
        else:
            wl = rnd.randint(-30, 180); wr = rnd.randint(-30, 180)
        start = BM * rnd.randint(0, (sq - 1) // BM)
        ct = 3 if causal else 0
        assert L.lib.fa_tile_intervals(ct, wl, wr, start, sq, sk, BM, BN, out) == 0
        lb, fb, rb = [set(range(out[i], out[i + 1] + 1)) if out[i] <= out[i + 1] else set() for i in (0, 2, 4)]
        pwl, pwr = iv.parse_window(ct, wl, wr, sq, sk) if causal else (0, 0)
        rows = range(start, min(start + BM, sq))
        nblk = (sk + BN - 1) // BN
        assert not (lb & fb) and not (lb & rb) and not (fb & rb)
        assert all(0 <= b < nblk for b in lb | fb | rb)
        for b in range(nblk):
            vis = [iv.visible(m, n, sq, sk, causal, pwl, pwr) for m in rows for n in range(b * BN, b * BN + BN)]
            if any(vis):
                assert b in (lb | fb | rb)
            if b in fb:
                assert all(vis)
        # the reference's algebra (oracle restatement) never calls a block "full" that we must mask
        # when the tile is not ragged in q, and its union covers ours
        r = iv.calculate_intervals(causal, pwl, pwr, start, sq, sk, start + BM > sq, BM, BN)
        ref_full = set(range(r[2], r[3] + 1)) if r[2] <= r[3] else set()
        ref_all = ref_full | (set(range(r[0], r[1] + 1)) if r[0] <= r[1] else set()) \
            | (set(range(r[4], r[5] + 1)) if r[4] <= r[5] else set())
        assert ref_full <= fb
        assert {b for b in (lb | fb | rb)} <= {b for b in ref_all} | fb


def test_v2_positional_entry_points_validate_before_any_launch():
    """fa_v2_* fill the v3 params and go through the same host checks (views over CPU tensors,
    every call ends in an argument error before a device is needed)."""
    from aotriton_amd import flash
    from aotriton_amd.pyaotriton import hipError_t as E, Stream
    from aotriton_amd.pyaotriton.v2 import flash as v2
    mk = flash.mk_aotensor
    B, Hq, Hk, Sq, Sk, D = 2, 4, 2, 64, 80, 128
    dt = torch.float16
    q = torch.zeros(B, Hq, Sq, D, dtype=dt); k = torch.zeros(B, Hk, Sk, D, dtype=dt); v = torch.zeros_like(k)
    o = torch.zeros_like(q); L = torch.zeros(B * Hq, Sq); delta = torch.zeros_like(L)
    s = Stream()
    # missing tensors
    assert v2.attn_fwd(None, mk(k), mk(v), None, 0.1, mk(L), mk(o), 0.0, None, None, 0, None, None, None, True,
                       None, s) == E.hipErrorInvalidValue
    assert v2.attn_bwd(mk(q), mk(k), mk(v), None, 0.1, mk(o), mk(o), mk(q), mk(k), mk(v), None, mk(L), None, 0.0,
                       None, None, 0, False, s) == E.hipErrorInvalidValue            # split backend without delta
    # heads of K do not divide those of Q
    k3 = torch.zeros(B, 3, Sk, D, dtype=dt)
    assert v2.attn_fwd(mk(q), mk(k3), mk(k3), None, 0.1, mk(L), mk(o), 0.0, None, None, 0, None, None, None, True,
                       None, s) == E.hipErrorInvalidValue
    # dropout without a seed, and a head dim that is not built
    assert v2.attn_fwd(mk(q), mk(k), mk(v), None, 0.1, mk(L), mk(o), 0.5, None, None, 0, None, None, None, False,
                       None, s) == E.hipErrorInvalidValue
    qb = torch.zeros(B, Hq, Sq, 520, dtype=dt); kb = torch.zeros(B, Hk, Sk, 520, dtype=dt)
    assert v2.attn_bwd_fused(mk(qb), mk(kb), mk(kb), None, 0.1, mk(qb), mk(qb), mk(qb), mk(kb), mk(kb), None, mk(L),
                             0.0, None, None, 0, True, s) == E.hipErrorNotSupported
    # packed sequences need both offset arrays and a batch of one
    cu = torch.tensor([0, 30, 64], dtype=torch.int32)
    assert v2.attn_fwd_compact_varlen(mk(q), mk(k), mk(v), None, mk(cu), None, 40, 40, 0.1, mk(L), mk(o), 0.0, None,
                                      None, 0, None, None, None, True, None, s) == E.hipErrorInvalidValue
    assert v2.attn_fwd_compact_varlen(mk(q), mk(k), mk(v), None, mk(cu), mk(cu), 40, 40, 0.1, mk(L), mk(o), 0.0, None,
                                      None, 0, None, None, None, True, None, s) == E.hipErrorInvalidValue
    assert v2.attn_bwd_compact_varlen(mk(q), mk(k), mk(v), mk(cu), mk(cu), 40, 40, None, 0.1, mk(o), mk(o), mk(q),
                                      mk(k), mk(v), None, mk(L), None, 0.0, None, None, 0, True, s) == E.hipErrorInvalidValue


def test_buffer_descriptors_are_built_in_one_place():
    """Every buffer descriptor of the kernels comes from wave_rsrc (fa_device.h), which makes its
    arguments wave-uniform for the compiler.  A descriptor built anywhere else can be taken for
    divergent; the compiler then loops over the distinct descriptors around every access, and a
    register spilled next to such a loop has been stored with no lane enabled (wrong results now
    and then, no error).  Source check: the builtin appears once, inside the helper."""
    import glob
    import re
    csrc = os.path.join(ROOT, 'aotriton_amd', 'csrc')
    uses = []
    for path in sorted(glob.glob(os.path.join(csrc, '*.h')) + glob.glob(os.path.join(csrc, '*.hip')) +
                       glob.glob(os.path.join(csrc, '*.cpp'))):
        text = open(path).read()
        text = re.sub(r'//[^\n]*', '', text)                    # comments may name the builtin
        for m in re.finditer(r'__builtin_amdgcn_make_buffer_rsrc', text):
            uses.append((os.path.basename(path), text.count('\n', 0, m.start()) + 1))
    assert [u[0] for u in uses] == ['fa_device.h'], f'buffer descriptors built outside wave_rsrc: {uses}'
    dev = open(os.path.join(csrc, 'fa_device.h')).read()
    body = dev[dev.index('wave_rsrc(P* base, int bytes)'):]
    body = body[:body.index('\n}\n')]
    assert body.count('__builtin_amdgcn_readfirstlane') == 3 and '__builtin_amdgcn_make_buffer_rsrc' in body
    # descriptors of other origin would have to be typed somewhere: the type's name appears only where one is held
    for path in glob.glob(os.path.join(csrc, '*')):
        if os.path.isfile(path) and path.endswith(('.h', '.hip', '.cpp')):
            assert 'amdgcn_make_buffer_rsrc(' not in re.sub(r'//[^\n]*', '', open(path).read()) or path.endswith('fa_device.h')
