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
    CUDA tensors (B, H, L, E), head dims up to 512 (multiples of 8 for the MFMA kernels).  A boolean mask becomes an
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


# ---- routing torch.nn.functional.scaled_dot_product_attention itself --------------------------
# The consumer the reference names is PyTorch's SDPA on ROCm (README.md:71-75 of the reference):
# callers write F.scaled_dot_product_attention and the dispatcher picks the flash backend.  The
# two hooks below give the same effect without touching callers: `sdpa_router()` is a
# TorchFunctionMode (scoped, composes with torch.compile's tracing of the custom ops), `install()`
# replaces the attribute on torch.nn.functional for code that cannot be wrapped in a `with`.
def _routable(query, key, value, attn_mask, dropout_p, enable_gqa=False):
    ts = (query, key, value)
    if not all(isinstance(t, Tensor) and t.is_cuda and t.dim() == 4 for t in ts):
        return False
    if query.dtype not in (torch.float16, torch.bfloat16, torch.float32):
        return False
    if not (key.dtype == query.dtype and value.dtype == query.dtype):
        return False
    dqk, dv = query.shape[-1], value.shape[-1]
    # (head dims that are no multiple of 8 would run on the element-wise kernels: correct but slow, so the
    # router leaves them to torch; scaled_dot_product_attention above takes them when called directly)
    if dqk % 8 or dv % 8 or dqk > 512 or dv > 512 or key.shape[-1] != dqk:
        return False
    if query.shape[1] % max(key.shape[1], 1) or key.shape[1] != value.shape[1]:
        return False
    # unequal head counts are grouped-query attention only when the caller says so (torch raises otherwise)
    if query.shape[1] != key.shape[1] and not enable_gqa:
        return False
    # what the operators would reject goes to torch, which raises its own error or broadcasts
    if not (query.shape[0] == key.shape[0] == value.shape[0]) or key.shape[2] != value.shape[2]:
        return False
    if not (query.device == key.device == value.device):
        return False
    if attn_mask is not None and (not isinstance(attn_mask, Tensor) or attn_mask.device != query.device):
        return False
    if getattr(query, 'is_nested', False) or getattr(key, 'is_nested', False):
        return False
    return True


_torch_sdpa = torch.nn.functional.scaled_dot_product_attention


def _dispatch(query, key, value, attn_mask=None, dropout_p=0.0, is_causal=False, scale=None, enable_gqa=False):
    if _routable(query, key, value, attn_mask, dropout_p, enable_gqa):
        return scaled_dot_product_attention(query, key, value, attn_mask, dropout_p, is_causal, scale, enable_gqa)
    return _torch_sdpa(query, key, value, attn_mask=attn_mask, dropout_p=dropout_p, is_causal=is_causal,
                       scale=scale, enable_gqa=enable_gqa)


class sdpa_router(torch.overrides.TorchFunctionMode):
    """`with sdpa_router(): ...` sends every F.scaled_dot_product_attention call on 4-D CUDA
    fp16/bf16/fp32 tensors (head dims multiples of 8 up to 512) to this library's operators;
    anything else falls through to PyTorch's own implementation."""

    def __torch_function__(self, func, types, args=(), kwargs=None):
        kwargs = kwargs or {}
        if func is _torch_sdpa:
            with torch._C.DisableTorchFunction():
                return _dispatch(*args, **kwargs)
        return func(*args, **kwargs)


def install():
    """Make torch.nn.functional.scaled_dot_product_attention route here process-wide
    (undo with uninstall()).  Modules that bound the function at import time keep the original;
    for those use the sdpa_router() mode."""
    torch.nn.functional.scaled_dot_product_attention = _dispatch


def uninstall():
    torch.nn.functional.scaled_dot_product_attention = _torch_sdpa
