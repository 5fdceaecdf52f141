"""Pins oracle/fa_ref.py against PyTorch math SDPA (library routine), autograd,
and the reference's known-answer LSE (no GPU)."""
import math

import numpy as np
import pytest
import torch

from oracle import fa_ref, philox
from oracle.intervals import TOP_LEFT, BOTTOM_RIGHT


def _inputs(B, Hq, Hk, Sq, Sk, D, dtype=torch.float64, seed=0, bias=False):
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(B, Hq, Sq, D, generator=g, dtype=dtype)
    k = torch.randn(B, Hk, Sk, D, generator=g, dtype=dtype)
    v = torch.randn(B, Hk, Sk, D, generator=g, dtype=dtype)
    do = torch.randn(B, Hq, Sq, D, generator=g, dtype=dtype)
    b = torch.randn(B, Hq, Sq, Sk, generator=g, dtype=dtype) * 0.5 if bias else None
    return q, k, v, b, do


CASES = [
    # B Hq Hk Sq Sk D causal_type wl wr bias dropout
    (2, 4, 4, 128, 128, 64, 0, 0, 0, False, 0.0),       # the benchmark configuration that runs on the CPU (fp32, D = 64)
    (1, 4, 2, 37, 53, 16, 3, TOP_LEFT, TOP_LEFT, False, 0.0),
    (1, 2, 2, 40, 24, 16, 3, BOTTOM_RIGHT, BOTTOM_RIGHT, False, 0.0),
    (1, 2, 1, 33, 47, 8, 3, 5, 3, False, 0.5),
    (2, 2, 2, 17, 19, 8, 0, 0, 0, True, 0.1),
    (1, 2, 2, 31, 31, 8, 3, 7, 0, True, 0.1),
]


@pytest.mark.parametrize('case', CASES)
def test_closed_forms_match_sdpa_math_and_autograd(case):
    B, Hq, Hk, Sq, Sk, D, ct, wl, wr, use_bias, pdrop = case
    q, k, v, b, do = _inputs(B, Hq, Hk, Sq, Sk, D, bias=use_bias)
    sm_scale = 1.0 / math.sqrt(D)
    keep = None
    if pdrop > 0:
        keep = torch.from_numpy(philox.dropout_keep_mask(B, Hq, Sq, Sk, pdrop, 0x1234, 5))
    o, lse, _ = fa_ref.attn_fwd_ref(q, k, v, b, sm_scale, ct, wl, wr, pdrop, keep)
    tensors = [t.clone().requires_grad_() for t in (q, k, v)]
    bb = b.clone().requires_grad_() if b is not None else None
    o2 = fa_ref.sdpa_math_ref(tensors[0], tensors[1], tensors[2], bb, sm_scale, ct, wl, wr, pdrop, keep)
    vis = fa_ref.visible_mask(Sq, Sk, ct, wl, wr)
    live = vis.any(dim=-1)                     # rows with at least one visible key
    # fully masked rows: math SDPA gives NaN, the kernels give 0 / +inf
    assert torch.allclose(o[:, :, live], o2[:, :, live].detach(), atol=1e-10)
    assert (o[:, :, ~live] == 0).all()
    assert torch.isinf(lse[:, :, ~live]).all() and (lse[:, :, ~live] > 0).all()
    assert torch.allclose(lse, fa_ref.lse_ref(q, k, b, sm_scale, ct, wl, wr))
    if not live.all():
        return
    o2.backward(do)
    dq, dk, dv, db, delta = fa_ref.attn_bwd_ref(q, k, v, b, sm_scale, o, do, lse, ct, wl, wr, pdrop, keep)
    assert torch.allclose(dq, tensors[0].grad, atol=1e-9)
    assert torch.allclose(dk, tensors[1].grad, atol=1e-9)
    assert torch.allclose(dv, tensors[2].grad, atol=1e-9)
    if b is not None:
        assert torch.allclose(db, bb.grad, atol=1e-9)
    assert torch.allclose(delta, (o * do).sum(-1))


def test_bwd_with_fully_masked_rows_is_finite():
    q, k, v, b, do = _inputs(1, 2, 2, 40, 24, 16)
    o, lse, _ = fa_ref.attn_fwd_ref(q, k, v, None, 0.25, 3, BOTTOM_RIGHT, BOTTOM_RIGHT)
    out = fa_ref.attn_bwd_ref(q, k, v, None, 0.25, o, do, lse, 3, BOTTOM_RIGHT, BOTTOM_RIGHT)
    for t in out[:3]:
        assert torch.isfinite(t).all()
    assert (out[0][:, :, :16] == 0).all()      # rows 0..15 see no key


def test_lse_known_answer():
    # modules/flash/tests/_core_test_backward.py:333-351
    for dt in (torch.float32, torch.float64):
        e = torch.eye(16, dtype=dt).reshape(1, 1, 16, 16)
        _, lse, _ = fa_ref.attn_fwd_ref(e, e, e, None, 0.25)
        assert torch.allclose(lse, torch.full_like(lse, 2.79018449783325195))
    assert abs(math.log(math.exp(0.25) + 15) - 2.79018449783325195) < 1e-7


def test_large_bf16_values_no_nan():
    # modules/flash/tests/_core_test_backward.py:353-374
    x = torch.full((1, 1, 1, 64), 133120.0, dtype=torch.bfloat16).float()
    o, lse, _ = fa_ref.attn_fwd_ref(x, x, x, None, 0.125)
    assert torch.isfinite(o).all() and torch.isfinite(lse).all()


def test_varlen_equals_per_sequence_dense():
    rng = np.random.default_rng(3)
    lens = rng.integers(3, 30, size=4)
    cu = [0] + np.cumsum(lens).tolist()
    T = cu[-1]
    q, k, v, _, do = _inputs(1, 4, 2, T, T, 8)
    o, lse = fa_ref.varlen_fwd_ref(q, k, v, cu, cu, 0.3, 3, TOP_LEFT, TOP_LEFT)
    assert o.shape == (1, 4, T, 8) and lse.shape == (4, T)
    i = 2
    sl = slice(cu[i], cu[i + 1])
    oi, lsei, _ = fa_ref.attn_fwd_ref(q[:, :, sl], k[:, :, sl], v[:, :, sl], None, 0.3, 3, TOP_LEFT, TOP_LEFT)
    assert torch.equal(o[:, :, sl], oi) and torch.equal(lse[:, sl], lsei[0])
    dq, dk, dv = fa_ref.varlen_bwd_ref(q, k, v, cu, cu, 0.3, o, do, lse, 3, TOP_LEFT, TOP_LEFT)
    assert dq.shape == q.shape and dk.shape == k.shape and dv.shape == v.shape


def test_sm_scale_zero_with_mask_is_finite():
    q, k, v, _, do = _inputs(1, 1, 1, 9, 9, 8)
    o, lse, p = fa_ref.attn_fwd_ref(q, k, v, None, 0.0, 3, TOP_LEFT, TOP_LEFT)
    assert torch.isfinite(o).all()
    # uniform softmax over the visible prefix
    assert torch.allclose(p[0, 0, 4, :5], torch.full((5,), 0.2, dtype=p.dtype))
