"""Shared helpers for the GPU parity tests: seeded inputs and the reference's
tolerance model (modules/flash/tests/_common_test.py:459-495):
    max|out - ref_hp| <= max(1e-5, fudge * max|ref_hp - ref_lp|)
with ref_hp the oracle in fp32 and ref_lp the oracle in the input dtype (fp64 and fp32
for fp32 inputs, _common_test.py:347).
Fudge factors: out 3.0, dq 148, dk 48, dv 36, db 17 (_common_test.py:171-180,384-407),
each capped at STRICT_FACTOR here.
"""
import math
import os

import numpy as np
import torch

from oracle import fa_ref, philox

FUDGE = dict(out=3.0, dq=148.0, dk=48.0, dv=36.0, db=17.0)
# the LSE has no entry in the reference's tolerance table (its tests only check
# the known-answer case); fp32 accumulation of 16-bit products, absolute bound
LSE_ATOL = 2e-3
STRICT_FACTOR = 6.0
STRICT_FACTOR_FP32 = 24.0


def make_inputs(B, Hq, Hk, Sq, Sk, D, dtype, device, seed=0, bias=False, bshd=False, bias_layout='padded',
                Dv=None):
    Dv = D if Dv is None else Dv          # head dim of V, Out and dOut
    g = torch.Generator(device='cpu').manual_seed(seed)

    def rn(*shape, scale=1.0):
        return (torch.randn(*shape, generator=g, dtype=torch.float32) * scale).to(dtype).to(device)

    if bshd:   # storage (B, S, H, D) viewed as (B, H, S, D): non-contiguous head stride
        q = rn(B, Sq, Hq, D).transpose(1, 2)
        k = rn(B, Sk, Hk, D).transpose(1, 2)
        v = rn(B, Sk, Hk, Dv).transpose(1, 2)
        do = rn(B, Sq, Hq, Dv).transpose(1, 2)
    else:
        q = rn(B, Hq, Sq, D); k = rn(B, Hk, Sk, D); v = rn(B, Hk, Sk, Dv); do = rn(B, Hq, Sq, Dv)
    b = None
    if bias:
        if bias_layout == 'padded':
            sk8 = (Sk + 7) // 8 * 8      # rows padded to 8 then sliced (_common_test.py:197-199)
            b = rn(B, Hq, Sq, sk8, scale=0.5)[:, :, :, :Sk]
        else:                            # 'odd': odd row stride and a base that is only 2-byte aligned
            b = rn(B, Hq, Sq, Sk + 3, scale=0.5)[:, :, :, 1:Sk + 1]
    return q, k, v, b, do


def keep_mask_from_oracle(B, H, Sq, Sk, p, seed, offset, device):
    if p <= 0:
        return None
    return torch.from_numpy(philox.dropout_keep_mask(B, H, Sq, Sk, p, seed, offset)).to(device)


def ref_fwd(q, k, v, b, sm_scale, ct, wl, wr, p, keep, dtype):
    cast = lambda t: None if t is None else t.to(dtype)
    return fa_ref.attn_fwd_ref(cast(q), cast(k), cast(v), cast(b), sm_scale, ct, wl, wr, p, keep)


def check(name, out, ref_hp, ref_lp, fudge, mask=None):
    strict = STRICT_FACTOR_FP32 if out.dtype == torch.float32 else STRICT_FACTOR
    out = out.double(); ref_hp = ref_hp.double(); ref_lp = ref_lp.double()
    if mask is not None:
        out = out[mask]; ref_hp = ref_hp[mask]; ref_lp = ref_lp[mask]
    assert not torch.isnan(out).any(), f'{name}: NaN in output'
    err = (out - ref_hp).abs().max().item() if out.numel() else 0.0
    ref_err = (ref_lp - ref_hp).abs().max().item() if out.numel() else 0.0
    # The reference's factors are what its own kernels need on their worst shapes; with
    # dk 48, dv 36 or dq 148 a wrong element can hide (a bias value read as zero for one key
    # of one row per tile did, at 8x the 16-bit oracle's error).  These kernels stay within
    # 4.3x of the low-precision oracle's error over the whole suite, so they are held to 6x.
    # For fp32 tensors the "low-precision" oracle is torch's fp32 matmul with its blocked sums,
    # while the fp32 kernels add one term at a time: up to 19x seen on 10240-term dK/dV sums, bar 24x.
    thr = max(1e-5, min(fudge, strict) * ref_err)
    log = os.environ.get('FA_TEST_ERROR_LOG')
    if log:      # one line per checked tensor: error relative to the low-precision oracle's
        with open(log, 'a') as f:
            f.write(f"{os.environ.get('PYTEST_CURRENT_TEST', '?')}\t{name}\t{err:.4e}\t{ref_err:.4e}\n")
    assert err <= thr, f'{name}: max|out-ref|={err:.3e} > {thr:.3e} (ref_lp err {ref_err:.3e}, fudge {fudge})'
    return err, thr


def reference_dropout_fixture():
    """Masks written by the reference's own debug_simulate_encoded_softmax kernel under
    Triton's CPU interpreter (tests/golden/make_dropout_fixture.py).  Yields dicts with
    B, H, Sq (rows stored), max_sq (the Max_seqlen_q the kernel was given), Sk, p, seed,
    off1, off2 and keep[B, H, Sq, Sk] (bool)."""
    z = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), 'golden', 'dropout_mask_reference.npz'))
    out = []
    i = 0
    while f'case{i}_keep' in z:
        B, H, Sq, Sk = (int(x) for x in z[f'case{i}_params'])
        seed, off1, off2 = (int(x) for x in z[f'case{i}_rng'])
        keep = np.unpackbits(z[f'case{i}_keep'])[:B * H * Sq * Sk].reshape(B, H, Sq, Sk).astype(bool)
        out.append(dict(B=B, H=H, Sq=Sq, max_sq=Sq, Sk=Sk, p=float(z[f'case{i}_p'][0]), seed=seed, off1=off1,
                        off2=off2, keep=keep))
        i += 1
    B, H, rows, max_sq, Sk = (int(x) for x in z['wrap_params'])
    seed, off1, off2 = (int(x) for x in z['wrap_rng'])
    keep = np.unpackbits(z['wrap_keep'])[:B * H * rows * Sk].reshape(B, H, rows, Sk).astype(bool)
    out.append(dict(B=B, H=H, Sq=rows, max_sq=max_sq, Sk=Sk, p=float(z['wrap_p'][0]), seed=seed, off1=off1,
                    off2=off2, keep=keep))
    return out
