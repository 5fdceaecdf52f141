"""Host layer over the pyaotriton-shaped bindings.

Counterpart of the reference's Python caller layer
(modules/flash/tests/aotriton_flash.py:38-408): tensor -> view marshalling,
``translate_causal``, the v3 params fill for dense and varlen calls, plus the v2
positional entry points (attn_fwd / attn_bwd / attn_bwd_fused /
attn_fwd_compact_varlen / attn_bwd_compact_varlen) as thin wrappers that fill the
v3 params.  Same names, argument meaning and error behaviour (hipError_t return).
"""
from .pyaotriton import (T0, T1, T2, T4, DType, Stream, hipError_t, get_name_suffix,  # noqa: F401
                         hipGetLastError, hipDeviceSynchronize, lazy_tensor)
from .pyaotriton.v2.flash import debug_simulate_encoded_softmax as fa_debug_simulate_encoded_softmax
from .pyaotriton.v2.flash import check_gpu as fa_check_gpu
from .pyaotriton.v3.flash import (attn_fwd as fa_forward_op, attn_fwd_params as fa_forward_op_params,
                                  attn_bwd as fa_backward_op, attn_bwd_params as fa_backward_op_params,
                                  attn_options)


class CausalType:
    NONE = 0
    TOP_LEFT = 1
    BOTTOM_RIGHT = 2
    WINDOWED = 3


class WindowValue:
    NONE = 0
    TOP_LEFT_ALIGNED = -2147483647      # 0x80000001
    BOTTOM_RIGHT_ALIGNED = -2147483646  # 0x80000002


IVARLEN_TYPE = {'compact': 1, 'padded': 2, 'strided': 3}


_TL = WindowValue.TOP_LEFT_ALIGNED
_BR = WindowValue.BOTTOM_RIGHT_ALIGNED
# what the v3 params carry for each way of saying "causal": (causal_type, window_left, window_right)
_CAUSAL_OF_ENUM = {
    CausalType.NONE: (CausalType.NONE, 0, 0),
    CausalType.TOP_LEFT: (CausalType.WINDOWED, _TL, _TL),
    CausalType.BOTTOM_RIGHT: (CausalType.WINDOWED, _BR, _BR),
}


def translate_causal(causal, v3_api=True):
    """(causal_type, window_left, window_right) of the v3 params for a bool, a (left, right)
    window or a CausalType; same mapping as aotriton_flash.py:38-63.  Only the bool form exists
    in the v2 API."""
    if isinstance(causal, bool):
        return _CAUSAL_OF_ENUM[CausalType.TOP_LEFT if causal else CausalType.NONE]
    assert v3_api, 'windows and alignment enums need the v3 params'
    if isinstance(causal, tuple):
        left, right = causal
        return CausalType.WINDOWED, left, right
    return _CAUSAL_OF_ENUM[causal]


def cast_dtype(dtype):
    """torch dtype -> DType of the bindings (aotriton_flash.py:83-91): k<Float|BFloat|Int|UInt><bits>."""
    import torch
    family = ('BFloat' if dtype == torch.bfloat16 else 'Float') if dtype.is_floating_point else \
             ('Int' if dtype.is_signed else 'UInt')
    assert not dtype.is_complex
    return getattr(DType, f'k{family}{8 * dtype.itemsize}')


_VIEW_OF_RANK = {1: T1, 2: T2, 4: T4}


def mk_aotensor(q, if_empty_then_like=None):
    """Tensor -> view of the bindings (aotriton_flash.py:93-114).  A 1-D tensor with at most one
    element is a device scalar (T0); None is a null view with the rank and dtype of
    ``if_empty_then_like``; other tensors need rank 1, 2 or 4 and a unit last stride."""
    if q is None:
        like = if_empty_then_like
        return _VIEW_OF_RANK[like.dim()](0, [0] * like.dim(), [0] * like.dim(), cast_dtype(like.dtype))
    if q.dim() == 1 and q.numel() <= 1:
        return T0(q.data_ptr(), cast_dtype(q.dtype))
    assert q.dim() in _VIEW_OF_RANK, f'Unsupported tensor rank {q.dim()}'
    assert q.stride(-1) == 1, 'the last stride of tensors must be 1'
    return _VIEW_OF_RANK[q.dim()](q.data_ptr(), tuple(q.size()), q.stride(), cast_dtype(q.dtype))


def _stream():
    """The reference passes Stream() (null stream); with torch on the GPU the
    current torch stream is the one the caller's other work is ordered on."""
    try:
        import torch
        if torch.cuda.is_available():
            return Stream(torch.cuda.current_stream().cuda_stream)
    except Exception:
        pass
    return Stream()


def _fill_fwd(params, q, k, v, b, sm_scale, M, o, dropout_p, philox_seed, philox_offset1, philox_offset2,
              philox_seed_output, philox_offset_output, encoded_softmax, causal, atomic):
    params.Q = mk_aotensor(q)
    params.K = mk_aotensor(k)
    params.V = mk_aotensor(v)
    params.B = mk_aotensor(b if (b is not None and b.numel() > 0) else None, if_empty_then_like=q)
    params.Sm_scale = float(sm_scale)
    params.L = mk_aotensor(M) if M is not None else T2(0, [0, 0], [0, 0], cast_dtype(q.dtype))
    params.Out = mk_aotensor(o)
    params.dropout_p = float(dropout_p)
    params.philox_seed_ptr = mk_aotensor(philox_seed)
    params.philox_offset1 = mk_aotensor(philox_offset1)
    params.philox_offset2 = philox_offset2
    params.philox_seed_output = mk_aotensor(philox_seed_output)
    params.philox_offset_output = mk_aotensor(philox_offset_output)
    params.encoded_softmax = mk_aotensor(encoded_softmax, if_empty_then_like=q)
    params.persistent_atomic_counter = mk_aotensor(atomic)
    params.causal_type, params.window_left, params.window_right = translate_causal(causal)


def attn_fwd(q, k, v, b, sm_scale, M, o, dropout_p, philox_seed, philox_offset1, philox_offset2,
             philox_seed_output, philox_offset_output, encoded_softmax, causal, atomic,
             extargs=None, stream=None):
    """aotriton_flash.py:141-196 (also the v2 positional attn_fwd: is_causal -> windowed
    with top-left sentinels)."""
    params = fa_forward_op_params()
    _fill_fwd(params, q, k, v, b, sm_scale, M, o, dropout_p, philox_seed, philox_offset1, philox_offset2,
              philox_seed_output, philox_offset_output, encoded_softmax, causal, atomic)
    params.varlen_type = 0
    return fa_forward_op(params, fa_forward_op_params.kVersion, stream or _stream(), extargs)


def attn_fwd_varlen(q, k, v, cu_seqlens_q, cu_seqlens_k, max_seqlen_q, max_seqlen_k,
                    seq_strides_q, seq_strides_k, b, sm_scale, M, o, dropout_p, philox_seed,
                    philox_offset1, philox_offset2, philox_seed_output, philox_offset_output,
                    encoded_softmax, causal, atomic, varlen_type, extargs=None, stream=None):
    """aotriton_flash.py:277-335."""
    params = fa_forward_op_params()
    _fill_fwd(params, q, k, v, b, sm_scale, M, o, dropout_p, philox_seed, philox_offset1, philox_offset2,
              philox_seed_output, philox_offset_output, encoded_softmax, causal, atomic)
    params.cu_seqlens_q = mk_aotensor(cu_seqlens_q)
    params.cu_seqlens_k = mk_aotensor(cu_seqlens_k)
    params.Max_seqlen_q = max_seqlen_q
    params.Max_seqlen_k = max_seqlen_k
    params.seq_strides_q = mk_aotensor(seq_strides_q, if_empty_then_like=cu_seqlens_q)
    params.seq_strides_k = mk_aotensor(seq_strides_k, if_empty_then_like=cu_seqlens_k)
    params.varlen_type = IVARLEN_TYPE[varlen_type]
    return fa_forward_op(params, fa_forward_op_params.kVersion, stream or _stream(), extargs)


def attn_fwd_compact_varlen(q, k, v, b, cu_seqlens_q, cu_seqlens_k, max_seqlen_q, max_seqlen_k,
                            sm_scale, M, o, dropout_p, philox_seed, philox_offset1, philox_offset2,
                            philox_seed_output, philox_offset_output, encoded_softmax, is_causal,
                            atomic, extargs=None, stream=None):
    """v2 positional attn_fwd_compact_varlen: q is (1, H, total, D)."""
    return attn_fwd_varlen(q, k, v, cu_seqlens_q, cu_seqlens_k, max_seqlen_q, max_seqlen_k, None, None,
                           b, sm_scale, M, o, dropout_p, philox_seed, philox_offset1, philox_offset2,
                           philox_seed_output, philox_offset_output, encoded_softmax, is_causal, atomic,
                           'compact', extargs=extargs, stream=stream)


def _fill_bwd(params, q, k, v, b, sm_scale, o, dout, dq, dk, dv, db, dq_acc, L, delta, dropout_p,
              philox_seed, philox_offset1, philox_offset2, causal):
    params.Q = mk_aotensor(q)
    params.K = mk_aotensor(k)
    params.V = mk_aotensor(v)
    params.B = mk_aotensor(b if (b is not None and b.numel() > 0) else None, if_empty_then_like=q)
    params.Sm_scale = float(sm_scale)
    params.Out = mk_aotensor(o)
    params.DO = mk_aotensor(dout)
    params.DK = mk_aotensor(dk)
    params.DV = mk_aotensor(dv)
    params.DQ = mk_aotensor(dq)
    params.DB = mk_aotensor(db, if_empty_then_like=q)
    params.DQ_ACC = dq_acc
    params.L = mk_aotensor(L)
    if delta is not None and not hasattr(delta, 'c'):      # a plain tensor: wrap as eager
        delta = lazy_tensor.eager_delta(mk_aotensor(delta))
    params.D = delta
    params.dropout_p = float(dropout_p)
    params.philox_seed_ptr = mk_aotensor(philox_seed)
    params.philox_offset1 = mk_aotensor(philox_offset1)
    params.philox_offset2 = philox_offset2
    params.causal_type, params.window_left, params.window_right = translate_causal(causal)


def attn_bwd(q, k, v, b, sm_scale, o, dout, dq, dk, dv, db, dq_acc, L, delta, dropout_p, philox_seed,
             philox_offset1, philox_offset2, causal, extargs=None, stream=None):
    """aotriton_flash.py:198-263.  ``delta`` is a lazy tensor (lazy_delta) or a
    plain fp32 tensor; ``dq_acc`` may be None."""
    params = fa_backward_op_params()
    _fill_bwd(params, q, k, v, b, sm_scale, o, dout, dq, dk, dv, db, dq_acc, L, delta, dropout_p,
              philox_seed, philox_offset1, philox_offset2, causal)
    params.varlen_type = 0
    return fa_backward_op(params, fa_backward_op_params.kVersion, stream or _stream(), extargs)


def attn_bwd_fused(q, k, v, b, sm_scale, o, dout, dq, dk, dv, db, L, dropout_p, philox_seed,
                   philox_offset1, philox_offset2, causal, stream=None):
    """v2 positional attn_bwd_fused: no delta buffer, single launch (backend 1)."""
    ext = attn_options()
    ext.force_backend_index = 1
    return attn_bwd(q, k, v, b, sm_scale, o, dout, dq, dk, dv, db, None, L, None, dropout_p,
                    philox_seed, philox_offset1, philox_offset2, causal, extargs=ext, stream=stream)


def attn_bwd_varlen(q, k, v, cu_seqlens_q, cu_seqlens_k, max_seqlen_q, max_seqlen_k, seq_strides_q,
                    seq_strides_k, b, sm_scale, o, dout, dq, dk, dv, db, dq_acc, L, delta, dropout_p,
                    philox_seed, philox_offset1, philox_offset2, causal, varlen_type, extargs=None,
                    stream=None):
    """aotriton_flash.py:337-398."""
    params = fa_backward_op_params()
    _fill_bwd(params, q, k, v, b, sm_scale, o, dout, dq, dk, dv, db, dq_acc, L, delta, dropout_p,
              philox_seed, philox_offset1, philox_offset2, causal)
    params.cu_seqlens_q = mk_aotensor(cu_seqlens_q)
    params.cu_seqlens_k = mk_aotensor(cu_seqlens_k)
    params.Max_seqlen_q = max_seqlen_q
    params.Max_seqlen_k = max_seqlen_k
    params.seq_strides_q = mk_aotensor(seq_strides_q, if_empty_then_like=cu_seqlens_q)
    params.seq_strides_k = mk_aotensor(seq_strides_k, if_empty_then_like=cu_seqlens_k)
    params.varlen_type = IVARLEN_TYPE[varlen_type]
    return fa_backward_op(params, fa_backward_op_params.kVersion, stream or _stream(), extargs)


def attn_bwd_compact_varlen(q, k, v, cu_seqlens_q, cu_seqlens_k, max_seqlen_q, max_seqlen_k, b,
                            sm_scale, o, dout, dq, dk, dv, db, L, delta, dropout_p, philox_seed,
                            philox_offset1, philox_offset2, is_causal, extargs=None, stream=None):
    """v2 positional attn_bwd_compact_varlen."""
    return attn_bwd_varlen(q, k, v, cu_seqlens_q, cu_seqlens_k, max_seqlen_q, max_seqlen_k, None, None,
                           b, sm_scale, o, dout, dq, dk, dv, db, None, L, delta, dropout_p, philox_seed,
                           philox_offset1, philox_offset2, is_causal, 'compact', extargs=extargs,
                           stream=stream)


def debug_simulate_encoded_softmax(R, dropout_p, philox_seed, philox_offset1, philox_offset2, stream=None):
    """aotriton_flash.py:265-275."""
    return fa_debug_simulate_encoded_softmax(mk_aotensor(R), dropout_p, mk_aotensor(philox_seed),
                                             mk_aotensor(philox_offset1), philox_offset2,
                                             stream or _stream())


def check_gpu(stream=None):
    return fa_check_gpu(stream or _stream())


def lazy_dq_acc(dq):
    """aotriton_flash.py:400-403."""
    return lazy_tensor.dq_acc(T4(dq.data_ptr(), tuple(dq.size()), dq.stride(), cast_dtype(dq.dtype)),
                              dq.device.index)


def lazy_delta(L):
    """aotriton_flash.py:405-408."""
    return lazy_tensor.delta(T2(L.data_ptr(), tuple(L.size()), L.stride(), cast_dtype(L.dtype)),
                             L.device.index)
