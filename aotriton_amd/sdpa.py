"""`torch.nn.functional.scaled_dot_product_attention` routed to the flash operators.

Mirrors how PyTorch's ROCm SDPA fills the operator's arguments: BHSD views of any
storage with unit last stride (BSHD storage included), an additive mask as the bias
operand, top-left causal alignment for `is_causal`, grouped-query attention by head
ratio.  Differences from the PyTorch function are listed in the docstring below.
"""
import math

import torch

from .autograd import attention, AttentionExtraArgs


def prepare(query, key, value, attn_mask, is_causal, scale, enable_gqa):
    """Argument checks and layout fixes shared by the SDPA-shaped entry points: returns
    (q, k, v, bias, sm_scale) with unit last strides and the mask as an additive
    (B, H, L, S) bias (None without a mask)."""
    if query.dim() != 4 or key.dim() != 4 or value.dim() != 4:
        raise ValueError('expected (batch, heads, seq, head_dim) tensors')
    if is_causal and attn_mask is not None:
        raise ValueError('attn_mask and is_causal cannot both be set')          # as torch does
    hq, hk = query.shape[1], key.shape[1]
    if hq != hk and not (enable_gqa and hq % hk == 0 and value.shape[1] == hk):
        raise ValueError('number of heads of query and key/value differ; pass enable_gqa=True for grouped queries')
    sm_scale = 1.0 / math.sqrt(query.shape[-1]) if scale is None else float(scale)
    unit = lambda t: t if t.stride(-1) == 1 else t.contiguous()
    q, k, v = unit(query), unit(key), unit(value)
    bias = None
    if attn_mask is not None:
        m = attn_mask
        if m.dtype == torch.bool:
            m = torch.zeros_like(m, dtype=q.dtype).masked_fill_(~m, float('-inf'))
        m = m.to(q.dtype)
        while m.dim() < 4:
            m = m.unsqueeze(0)
        bias = m.expand(q.shape[0], hq, q.shape[2], k.shape[2])
        if bias.stride(-1) != 1:
            bias = bias.contiguous()
    return q, k, v, bias, sm_scale


def scaled_dot_product_attention(query, key, value, attn_mask=None, dropout_p=0.0, is_causal=False,
                                 scale=None, enable_gqa=False, extra=None):
    """Same signature and semantics as torch.nn.functional.scaled_dot_product_attention for
    4-D fp16/bf16 CUDA tensors (B, H, L, E), with these limits: the head dims (of q/k, and of
    v) are multiples of 8 up to 512 (fp32 and head dims above 256 take slow kernels); a boolean mask is turned into an additive one
    (0 / -inf), and a query row that the mask hides completely yields zeros instead of NaN;
    dropout uses the operators' Philox stream (seed/offsets in `extra`), not torch's generator.
    """
    q, k, v, bias, sm_scale = prepare(query, key, value, attn_mask, is_causal, scale, enable_gqa)
    out, _, _ = attention(q, k, v, bias, bool(is_causal), sm_scale, float(dropout_p),
                          extra or AttentionExtraArgs())
    return out
