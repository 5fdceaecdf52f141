"""torch.autograd Functions over the flash operators.

Counterpart of modules/flash/tests/attn_torch_function.py:87-270 and
varlen_attn_torch_function.py:38-206: same allocation shapes (O (B,Hq,Sq,Dv); LSE
(B*Hq, Sq) dense, (Hq, total_q) compact), philox seed/offset passed as device
uint64[1] tensors with the reference's defaults, the int32 counter zeroed before
every causal forward, and the backward reading the forward's *output* seed/offset
with offset2 = 0.
"""
from dataclasses import dataclass

import numpy as np
import torch

from . import flash
from .flash import hipError_t, attn_options

DEFAULT_PHILOX_SEED = 0x1BF52
DEFAULT_PHILOX_OFFSET_1 = 0x1D4000
DEFAULT_PHILOX_OFFSET_2 = 0x000B42


@dataclass
class AttentionExtraArgs:
    return_encoded_softmax: bool = False
    return_logsumexp: bool = False
    fillnan: bool = False
    bwd_backend: int = -1          # -1 library's choice, 0 split, 1 fused
    philox_seed: int = DEFAULT_PHILOX_SEED
    philox_offset1: int = DEFAULT_PHILOX_OFFSET_1
    philox_offset2: int = DEFAULT_PHILOX_OFFSET_2


def _u64(x, device):
    return torch.tensor([np.int64(np.uint64(x))], device=device, dtype=torch.int64).view(torch.uint64)


def _philox(dropout_p, device, ext):
    null = torch.empty([0], device=device, dtype=torch.uint64)
    if dropout_p > 0.0:
        return (_u64(ext.philox_seed, device), _u64(ext.philox_offset1, device), ext.philox_offset2,
                _u64(0, device), _u64(0, device))
    return null, null, 0, null, null


def _check(ret):
    if ret == hipError_t.hipErrorPeerAccessUnsupported:
        raise NotImplementedError('backend cannot take this input')
    if ret != hipError_t.hipSuccess:
        raise RuntimeError(f'flash operator failed: {ret!r}')


class _attention(torch.autograd.Function):

    @staticmethod
    def forward(ctx, q, k, v, b, causal, sm_scale, dropout_p, ext=None):
        ext = ext or AttentionExtraArgs()
        o = torch.empty((q.shape[0], q.shape[1], q.shape[2], v.shape[3]), device=q.device, dtype=q.dtype)
        M = torch.empty((q.shape[0] * q.shape[1], q.shape[2]), device=q.device, dtype=torch.float32)
        if ext.fillnan:
            o.fill_(float('nan'))
            M.fill_(float('nan'))
        encoded_softmax = None
        if ext.return_encoded_softmax:
            encoded_softmax = torch.zeros((q.shape[0], q.shape[1], q.shape[2], k.shape[2]),
                                          device=q.device, dtype=q.dtype)
        seed, off1, off2, seed_out, off_out = _philox(dropout_p, q.device, ext)
        atomic = (torch.zeros([1], device=q.device, dtype=torch.int32) if causal
                  else torch.empty([0], device=q.device, dtype=torch.int32))
        _check(flash.attn_fwd(q, k, v, b, sm_scale, M, o, dropout_p, seed, off1, off2, seed_out, off_out,
                              encoded_softmax, causal, atomic))
        ctx.save_for_backward(q, k, v, b, o, M)
        ctx.sm_scale = sm_scale
        ctx.causal = causal
        ctx.dropout_p = dropout_p
        ctx.philox_seed = seed_out
        ctx.philox_offset = off_out
        ctx.ext = ext
        return o, encoded_softmax, (M if ext.return_logsumexp else None)

    @staticmethod
    def backward(ctx, do, _, __):
        q, k, v, b, o, L = ctx.saved_tensors
        dq = torch.empty_like(q)
        dk = torch.empty_like(k)
        dv = torch.empty_like(v)
        db = torch.empty_like(b) if b is not None else None
        extargs = None
        if ctx.ext.bwd_backend >= 0:
            extargs = attn_options()
            extargs.force_backend_index = ctx.ext.bwd_backend
        if do.stride(-1) != 1:
            do = do.contiguous()
        _check(flash.attn_bwd(q, k, v, b, ctx.sm_scale, o, do, dq, dk, dv, db, flash.lazy_dq_acc(q), L,
                              flash.lazy_delta(L), ctx.dropout_p, ctx.philox_seed, ctx.philox_offset, 0,
                              ctx.causal, extargs=extargs))
        return dq, dk, dv, db, None, None, None, None


attention = _attention.apply


class _attention_varlen(torch.autograd.Function):
    """Compact varlen: q (1, Hq, total_q, D), k/v (1, Hk, total_k, D)."""

    @staticmethod
    def forward(ctx, q, k, v, seqlens_q, seqlens_k, causal, sm_scale, dropout_p, ext=None):
        ext = ext or AttentionExtraArgs()
        seqlens_q = np.asarray(seqlens_q)
        seqlens_k = np.asarray(seqlens_k)
        total_q = int(seqlens_q.sum())
        num_heads = q.shape[1]
        max_q, max_k = int(seqlens_q.max()), int(seqlens_k.max())
        cu_q = torch.tensor([0] + np.cumsum(seqlens_q).tolist(), dtype=torch.int32, device=q.device)
        cu_k = torch.tensor([0] + np.cumsum(seqlens_k).tolist(), dtype=torch.int32, device=q.device)
        o = torch.empty((q.shape[0], q.shape[1], q.shape[2], v.shape[3]), device=q.device, dtype=q.dtype)
        M = torch.empty((num_heads, total_q), device=q.device, dtype=torch.float32)
        if ext.fillnan:
            o.fill_(float('nan'))
            M.fill_(float('nan'))
        encoded_softmax = None
        if ext.return_encoded_softmax:
            encoded_softmax = torch.zeros((len(seqlens_q), num_heads, max_q, max_k), device=q.device,
                                          dtype=q.dtype)
        seed, off1, off2, seed_out, off_out = _philox(dropout_p, q.device, ext)
        atomic = (torch.zeros([1], device=q.device, dtype=torch.int32) if causal
                  else torch.empty([0], device=q.device, dtype=torch.int32))
        _check(flash.attn_fwd_compact_varlen(q, k, v, None, cu_q, cu_k, max_q, max_k, sm_scale, M, o,
                                             dropout_p, seed, off1, off2, seed_out, off_out,
                                             encoded_softmax, causal, atomic))
        ctx.save_for_backward(q, k, v, o, M, cu_q, cu_k)
        ctx.max_q, ctx.max_k = max_q, max_k
        ctx.sm_scale = sm_scale
        ctx.causal = causal
        ctx.dropout_p = dropout_p
        ctx.philox_seed = seed_out
        ctx.philox_offset = off_out
        ctx.ext = ext
        return o, encoded_softmax, (M if ext.return_logsumexp else None)

    @staticmethod
    def backward(ctx, do, _, __):
        q, k, v, o, L, cu_q, cu_k = ctx.saved_tensors
        dq = torch.empty_like(q)
        dk = torch.empty_like(k)
        dv = torch.empty_like(v)
        extargs = None
        if ctx.ext.bwd_backend >= 0:
            extargs = attn_options()
            extargs.force_backend_index = ctx.ext.bwd_backend
        if do.stride(-1) != 1:
            do = do.contiguous()
        _check(flash.attn_bwd_compact_varlen(q, k, v, cu_q, cu_k, ctx.max_q, ctx.max_k, None, ctx.sm_scale,
                                             o, do, dq, dk, dv, None, L, flash.lazy_delta(L),
                                             ctx.dropout_p, ctx.philox_seed, ctx.philox_offset, 0,
                                             ctx.causal, extargs=extargs))
        return dq, dk, dv, None, None, None, None, None, None


attention_varlen = _attention_varlen.apply
