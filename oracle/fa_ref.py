"""Attention forward/backward on the CPU in fp32/fp64 (test infrastructure only).

Restates, element by element, what the reference kernels compute:
  forward   modules/flash/kernel/fwd_kernel.py:83-644, fwd_kernel_inner.py:46-287
  delta     modules/flash/kernel/bwd_preprocess.py:28-133
  dK, dV    modules/flash/kernel/bwd_kernel_dk_dv.py:48-417, bwd_inner_dk_dv.py:28-267
  dQ, dB    modules/flash/kernel/bwd_kernel_dq.py:45-389, bwd_inner_dq.py:28-215
The reference's own tests use torch.ops.aten._scaled_dot_product_attention_math
as their oracle (modules/flash/tests/_common_test.py:61-79); ``sdpa_math_ref``
wraps the same routine and tests/test_oracle_attention.py checks the closed
forms below against it.

Layouts: q [B,Hq,Sq,Dqk], k [B,Hk,Sk,Dqk], v [B,Hk,Sk,Dv], bias [B,Hq,Sq,Sk],
LSE [B,Hq,Sq] (natural log).  Fully masked rows: O = 0, LSE = +inf
(fwd_kernel.py:327-355).
"""
import math
import torch

from .intervals import parse_window


def visible_mask(seqlen_q, seqlen_k, causal_type, window_left, window_right,
                 device='cpu'):
    """Bool [Sq,Sk]; fwd_kernel_inner.py:137-148 with parse_window applied."""
    if causal_type == 0:
        return torch.ones(seqlen_q, seqlen_k, dtype=torch.bool, device=device)
    wl, wr = parse_window(causal_type, window_left, window_right, seqlen_q, seqlen_k)
    m = torch.arange(seqlen_q, device=device)[:, None]
    n = torch.arange(seqlen_k, device=device)[None, :]
    return (m + wr >= n) & (m - wl <= n)


def _expand_kv(x, hq):
    hk = x.shape[1]
    if hk == hq:
        return x
    # off_h_k = off_h_q // (Hq // Hk)  (fwd_kernel.py:360)
    return x.repeat_interleave(hq // hk, dim=1)


def attn_fwd_ref(q, k, v, bias, sm_scale, causal_type=0, window_left=0,
                 window_right=0, dropout_p=0.0, keep_mask=None):
    """Returns (O, LSE, P) in q.dtype; P is the undropped softmax."""
    B, Hq, Sq, _ = q.shape
    Sk = k.shape[2]
    kk = _expand_kv(k, Hq)
    vv = _expand_kv(v, Hq)
    s = torch.matmul(q, kk.transpose(-1, -2)) * sm_scale
    if bias is not None:
        s = s + bias
    vis = visible_mask(Sq, Sk, causal_type, window_left, window_right, q.device)
    s = s.masked_fill(~vis, float('-inf'))
    m = s.max(dim=-1, keepdim=True).values
    dead = torch.isinf(m) & (m < 0)
    m_safe = torch.where(dead, torch.zeros_like(m), m)
    e = torch.exp(s - m_safe)
    l = e.sum(dim=-1, keepdim=True)
    lse = m_safe + torch.log(l)
    lse = torch.where(dead, torch.full_like(lse, float('inf')), lse)
    p = torch.where(dead, torch.zeros_like(e), e / torch.where(dead, torch.ones_like(l), l))
    pd = p
    if dropout_p > 0.0:
        # l sums the undropped p (fwd_kernel_inner.py:213-214); 1/(1-p) applied
        # once to the accumulator (fwd_kernel.py:573-575).
        pd = torch.where(keep_mask, p, torch.zeros_like(p)) / (1.0 - dropout_p)
    o = torch.matmul(pd, vv)
    return o, lse.squeeze(-1), p


def attn_bwd_ref(q, k, v, bias, sm_scale, o, do, lse, causal_type=0,
                 window_left=0, window_right=0, dropout_p=0.0, keep_mask=None):
    """Closed-form gradients.  Returns (dq, dk, dv, db, delta)."""
    B, Hq, Sq, _ = q.shape
    Hk, Sk = k.shape[1], k.shape[2]
    g = Hq // Hk
    kk = _expand_kv(k, Hq)
    vv = _expand_kv(v, Hq)
    s = torch.matmul(q, kk.transpose(-1, -2)) * sm_scale
    if bias is not None:
        s = s + bias
    vis = visible_mask(Sq, Sk, causal_type, window_left, window_right, q.device)
    # p = exp(s - LSE); LSE=+inf rows give 0 (bwd_inner_dk_dv.py:185-188)
    p = torch.exp(s - lse.unsqueeze(-1))
    p = torch.where(vis, p, torch.zeros_like(p))
    p = torch.nan_to_num(p, nan=0.0)
    delta = (o * do).sum(dim=-1)                      # bwd_preprocess.py:28-133
    dp = torch.matmul(do, vv.transpose(-1, -2))       # bwd_inner_dk_dv.py:231-236
    if dropout_p > 0.0:
        scale = 1.0 / (1.0 - dropout_p)
        keepf = keep_mask.to(p.dtype)
        p_dropped = p * keepf * scale                 # :200-201
        dp = dp * keepf * scale                       # :239-240
    else:
        p_dropped = p
    ds = p * (dp - delta.unsqueeze(-1))               # :242 (undropped p)
    dv_full = torch.matmul(p_dropped.transpose(-1, -2), do)
    dk_full = torch.matmul(ds.transpose(-1, -2), q) * sm_scale
    dq = torch.matmul(ds, kk) * sm_scale
    dv = dv_full.reshape(B, Hk, g, Sk, -1).sum(dim=2)
    dk = dk_full.reshape(B, Hk, g, Sk, -1).sum(dim=2)
    db = ds if bias is not None else None             # bwd_inner_dq.py:200-204
    return dq, dk, dv, db, delta


def sdpa_math_ref(q, k, v, bias, sm_scale, causal_type=0, window_left=0,
                  window_right=0, dropout_p=0.0, keep_mask=None):
    """The reference's own oracle (tests/_common_test.py:61-79): PyTorch math SDPA.

    Window/causal visibility is folded into the additive mask so that any
    (left, right) window can be expressed.  Returns O only (autograd-capable).
    """
    B, Hq, Sq, _ = q.shape
    Sk = k.shape[2]
    attn_mask = None
    if causal_type != 0:
        vis = visible_mask(Sq, Sk, causal_type, window_left, window_right, q.device)
        attn_mask = torch.zeros(Sq, Sk, dtype=q.dtype, device=q.device)
        attn_mask = attn_mask.masked_fill(~vis, float('-inf'))
    if bias is not None:
        attn_mask = bias if attn_mask is None else bias + attn_mask
    out, _ = torch.ops.aten._scaled_dot_product_attention_math(
        q, k, v, attn_mask=attn_mask, dropout_p=dropout_p, is_causal=False,
        dropout_mask=keep_mask, scale=sm_scale, enable_gqa=(k.shape[1] != Hq))
    return out


def lse_ref(q, k, bias, sm_scale, causal_type=0, window_left=0, window_right=0):
    """logsumexp of the masked scores (modules/flash/tune/sdpa_math.py:16-41)."""
    Hq = q.shape[1]
    s = torch.matmul(q, _expand_kv(k, Hq).transpose(-1, -2)) * sm_scale
    if bias is not None:
        s = s + bias
    vis = visible_mask(q.shape[2], k.shape[2], causal_type, window_left, window_right, q.device)
    s = s.masked_fill(~vis, float('-inf'))
    out = torch.logsumexp(s, dim=-1)
    return torch.where(torch.isinf(out) & (out < 0), torch.full_like(out, float('inf')), out)


def varlen_fwd_ref(q, k, v, cu_q, cu_k, sm_scale, causal_type=0, window_left=0,
                   window_right=0, dropout_p=0.0, keep_masks=None):
    """Compact varlen: q [1,Hq,Tq,D], k/v [1,Hk,Tk,D]; per-sequence dense loop
    (tests/_common_test.py:729-759).  LSE is [Hq, Tq]
    (varlen_attn_torch_function.py:81-84)."""
    outs, lses = [], []
    for i in range(len(cu_q) - 1):
        qs = q[:, :, cu_q[i]:cu_q[i + 1]]
        ks = k[:, :, cu_k[i]:cu_k[i + 1]]
        vs = v[:, :, cu_k[i]:cu_k[i + 1]]
        km = None if keep_masks is None else keep_masks[i]
        o, lse, _ = attn_fwd_ref(qs, ks, vs, None, sm_scale, causal_type, window_left,
                                 window_right, dropout_p, km)
        outs.append(o)
        lses.append(lse[0])
    return torch.cat(outs, dim=2), torch.cat(lses, dim=1)


def varlen_bwd_ref(q, k, v, cu_q, cu_k, sm_scale, o, do, lse, causal_type=0,
                   window_left=0, window_right=0, dropout_p=0.0, keep_masks=None):
    dqs, dks, dvs = [], [], []
    for i in range(len(cu_q) - 1):
        sq = slice(cu_q[i], cu_q[i + 1])
        sk = slice(cu_k[i], cu_k[i + 1])
        km = None if keep_masks is None else keep_masks[i]
        dq, dk, dv, _, _ = attn_bwd_ref(q[:, :, sq], k[:, :, sk], v[:, :, sk], None, sm_scale,
                                        o[:, :, sq], do[:, :, sq], lse[None, :, sq],
                                        causal_type, window_left, window_right, dropout_p, km)
        dqs.append(dq); dks.append(dk); dvs.append(dv)
    return torch.cat(dqs, dim=2), torch.cat(dks, dim=2), torch.cat(dvs, dim=2)
