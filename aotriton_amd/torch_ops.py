"""torch.library registration of the flash operators.

`torch.ops.aotriton_amd.flash_attention_forward / flash_attention_backward` are custom ops
with fake (shape-only) implementations and an autograd formula, so that code using them
can be traced by torch.compile / AOTAutograd.  They take what PyTorch's ROCm SDPA puts
into attn_fwd_params / attn_bwd_params (include/aotriton/flash.h:96-174 of the
reference): (B, H, S, D) tensors with unit last stride, an optional additive bias,
causal type with window sentinels, and the Philox seed / offset as uint64[1] device
tensors.  `philox_state` hands out seed and offset from torch's CUDA generator and
advances it, the way the ROCm SDPA takes them from the generator's philox state.

`scaled_dot_product_attention` here has the signature of
torch.nn.functional.scaled_dot_product_attention and runs on those ops.
"""
from typing import Optional, Tuple

import numpy as np
import torch
from torch import Tensor

from . import flash
from .flash import hipError_t, attn_options, WindowValue
from .sdpa import prepare

__all__ = ['flash_attention_forward', 'flash_attention_backward', 'philox_state', 'scaled_dot_product_attention']


def _check(ret):
    if ret != hipError_t.hipSuccess:
        raise RuntimeError(f'flash operator failed: {ret!r}')


def _causal_arg(causal_type, window_left, window_right):
    return (window_left, window_right) if causal_type != 0 else False


@torch.library.custom_op('aotriton_amd::philox_state', mutates_args=(), device_types='cuda',
                         tags=(torch.Tag.nondeterministic_seeded,))
def philox_state(like: Tensor, increment: int) -> Tuple[Tensor, Tensor]:
    """Seed and offset (uint64[1] tensors on like's device) of the device's default generator;
    the generator's offset moves on by `increment` counters (rounded up to a multiple of 4).

    The op reads and advances host-side generator state, so it is tagged as a seeded random op:
    graph passes must not merge two calls or recompute one.  Under CUDA/HIP graph capture the
    host read happens once, at capture: every replay would reuse the captured seed and offset.
    Callers that replay graphs pass their own seed / offset tensors to flash_attention_forward
    and update them on the device between replays."""
    gen = torch.cuda.default_generators[like.device.index]
    seed, offset = gen.initial_seed(), gen.get_offset()
    gen.set_offset(offset + (increment + 3) // 4 * 4)
    mk = lambda x: torch.tensor([np.int64(np.uint64(x))], device=like.device, dtype=torch.int64).view(torch.uint64)
    return mk(seed), mk(offset)


@philox_state.register_fake
def _(like, increment):
    return (torch.empty([1], device=like.device, dtype=torch.uint64),
            torch.empty([1], device=like.device, dtype=torch.uint64))


@torch.library.custom_op('aotriton_amd::flash_attention_forward', mutates_args=(), device_types='cuda')
def flash_attention_forward(q: Tensor, k: Tensor, v: Tensor, bias: Optional[Tensor], dropout_p: float,
                            causal_type: int, window_left: int, window_right: int, sm_scale: float,
                            philox_seed: Tensor, philox_offset: Tensor) -> Tuple[Tensor, Tensor]:
    """Returns (Out (B, Hq, Sq, Dv), logsumexp (B*Hq, Sq) fp32)."""
    o = torch.empty((q.shape[0], q.shape[1], q.shape[2], v.shape[3]), device=q.device, dtype=q.dtype)
    lse = torch.empty((q.shape[0] * q.shape[1], q.shape[2]), device=q.device, dtype=torch.float32)
    null = torch.empty([0], device=q.device, dtype=torch.uint64)
    drop = dropout_p > 0.0
    atomic = torch.empty([0], device=q.device, dtype=torch.int32)
    if causal_type != 0:
        atomic = torch.zeros([1], device=q.device, dtype=torch.int32)
    _check(flash.attn_fwd(q, k, v, bias, sm_scale, lse, o, dropout_p,
                          philox_seed if drop else null, philox_offset if drop else null, 0, null, null,
                          None, _causal_arg(causal_type, window_left, window_right), atomic))
    return o, lse


@flash_attention_forward.register_fake
def _(q, k, v, bias, dropout_p, causal_type, window_left, window_right, sm_scale, philox_seed, philox_offset):
    o = torch.empty((q.shape[0], q.shape[1], q.shape[2], v.shape[3]), device=q.device, dtype=q.dtype)
    lse = torch.empty((q.shape[0] * q.shape[1], q.shape[2]), device=q.device, dtype=torch.float32)
    return o, lse


@torch.library.custom_op('aotriton_amd::flash_attention_backward', mutates_args=(), device_types='cuda')
def flash_attention_backward(dout: Tensor, q: Tensor, k: Tensor, v: Tensor, bias: Optional[Tensor], out: Tensor,
                             lse: Tensor, dropout_p: float, causal_type: int, window_left: int,
                             window_right: int, sm_scale: float, philox_seed: Tensor, philox_offset: Tensor,
                             need_dbias: bool, backend: int) -> Tuple[Tensor, Tensor, Tensor, Tensor]:
    """Returns (dQ, dK, dV, dB); dB is an empty tensor unless need_dbias.  backend: -1 the
    library's choice, 0 split kernels, 1 fused kernel."""
    dq = torch.empty(q.shape, device=q.device, dtype=q.dtype)
    dk = torch.empty(k.shape, device=q.device, dtype=q.dtype)
    dv = torch.empty(v.shape, device=q.device, dtype=q.dtype)
    want_db = need_dbias and bias is not None
    db = torch.empty(bias.shape if want_db else [0], device=q.device, dtype=q.dtype)
    null = torch.empty([0], device=q.device, dtype=torch.uint64)
    drop = dropout_p > 0.0
    extargs = None
    if backend >= 0:
        extargs = attn_options()
        extargs.force_backend_index = backend
    if dout.stride(-1) != 1:
        dout = dout.contiguous()
    _check(flash.attn_bwd(q, k, v, bias, sm_scale, out, dout, dq, dk, dv, db if want_db else None,
                          flash.lazy_dq_acc(q), lse, flash.lazy_delta(lse), dropout_p,
                          philox_seed if drop else null, philox_offset if drop else null, 0,
                          _causal_arg(causal_type, window_left, window_right), extargs=extargs))
    return dq, dk, dv, db


@flash_attention_backward.register_fake
def _(dout, q, k, v, bias, out, lse, dropout_p, causal_type, window_left, window_right, sm_scale, philox_seed,
      philox_offset, need_dbias, backend):
    mk = lambda t: torch.empty(t.shape, device=q.device, dtype=q.dtype)
    want_db = need_dbias and bias is not None
    return mk(q), mk(k), mk(v), (mk(bias) if want_db else torch.empty([0], device=q.device, dtype=q.dtype))


def _setup_context(ctx, inputs, output):
    q, k, v, bias, dropout_p, causal_type, wl, wr, sm_scale, seed, offset = inputs
    o, lse = output
    ctx.save_for_backward(q, k, v, bias, o, lse, seed, offset)
    ctx.scalars = (dropout_p, causal_type, wl, wr, sm_scale)
    ctx.need_dbias = bias is not None and ctx.needs_input_grad[3]


def _backward(ctx, dout, dlse):
    q, k, v, bias, o, lse, seed, offset = ctx.saved_tensors
    dropout_p, causal_type, wl, wr, sm_scale = ctx.scalars
    dq, dk, dv, db = torch.ops.aotriton_amd.flash_attention_backward(
        dout, q, k, v, bias, o, lse, dropout_p, causal_type, wl, wr, sm_scale, seed, offset, ctx.need_dbias, -1)
    return dq, dk, dv, (db if ctx.need_dbias else None), None, None, None, None, None, None, None


flash_attention_forward.register_autograd(_backward, setup_context=_setup_context)


def scaled_dot_product_attention(query, key, value, attn_mask=None, dropout_p=0.0, is_causal=False,
                                 scale=None, enable_gqa=False):
    """torch.nn.functional.scaled_dot_product_attention on the custom ops above: 4-D fp16/bf16
    CUDA tensors (B, H, L, E), head dims multiples of 8 up to 512.  A boolean mask becomes an
    additive one (0 / -inf); a query row that the mask hides completely yields zeros instead
    of NaN; dropout draws seed and offset from torch's CUDA generator (so torch.manual_seed
    governs it) but uses the operators' Philox stream, not the one of torch's own kernels.
    As in torch, is_causal means the top-left aligned lower triangle.
    """
    q, k, v, bias, sm_scale = prepare(query, key, value, attn_mask, is_causal, scale, enable_gqa)
    hq = q.shape[1]
    if dropout_p > 0.0:
        stride = (k.shape[2] + 3) // 4          # Philox counters per query row
        seed, offset = torch.ops.aotriton_amd.philox_state(q, q.shape[0] * hq * q.shape[2] * stride)
    else:
        seed = offset = torch.zeros([1], device=q.device, dtype=torch.int64).view(torch.uint64)
    ct = 3 if is_causal else 0
    wl = wr = int(WindowValue.TOP_LEFT_ALIGNED) if is_causal else 0
    o, _ = torch.ops.aotriton_amd.flash_attention_forward(q, k, v, bias, float(dropout_p), ct, wl, wr, sm_scale,
                                                          seed, offset)
    return o
