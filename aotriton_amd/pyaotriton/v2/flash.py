"""pyaotriton.v2.flash (modules/flash/bindings/v2.cc:27-37)."""
import ctypes

from ... import _lib
from ..._lib import lib


def check_gpu(stream):
    from .. import hipError_t
    return hipError_t(lib.fa_check_gpu(stream.native() or None))


def debug_simulate_encoded_softmax(r, dropout_p, philox_seed, philox_offset1, philox_offset2, stream):
    from .. import hipError_t
    rc = r.to_c()
    sc = philox_seed.to_c()
    oc = philox_offset1.to_c()
    return hipError_t(lib.fa_debug_simulate_encoded_softmax(
        ctypes.byref(rc), float(dropout_p), ctypes.byref(sc), ctypes.byref(oc),
        int(philox_offset2) & 0xFFFFFFFFFFFFFFFF, stream.native() or None))


# The positional v2 operators (AOTriton 0.11 include/aotriton/v2/flash.h:31-141), bound to the
# fa_v2_* symbols of the C ABI.  Views are T4 / T2 / T1 / T0 objects; None stands for an empty view.
def _ref(view, keep):
    if view is None:
        return None
    c = view.to_c()
    keep.append(c)
    return ctypes.byref(c)


def _call(name, args, stream):
    from .. import hipError_t
    keep = []
    conv = [_ref(a, keep) if (a is None or hasattr(a, 'to_c')) else a for a in args]
    return hipError_t(getattr(lib, name)(*conv, stream.native() or None))


def attn_fwd(q, k, v, b, sm_scale, softmax_lse, out, dropout_p, philox_seed, philox_offset1, philox_offset2,
             philox_seed_output, philox_offset_output, encoded_softmax, is_causal, atomic_for_causal, stream):
    return _call('fa_v2_attn_fwd', [q, k, v, b, float(sm_scale), softmax_lse, out, float(dropout_p), philox_seed,
                                    philox_offset1, int(philox_offset2), philox_seed_output, philox_offset_output,
                                    encoded_softmax, int(bool(is_causal)), atomic_for_causal], stream)


def attn_fwd_compact_varlen(q, k, v, b, cu_seqlens_q, cu_seqlens_k, max_seqlen_q, max_seqlen_k, sm_scale,
                            softmax_lse, out, dropout_p, philox_seed, philox_offset1, philox_offset2,
                            philox_seed_output, philox_offset_output, encoded_softmax, is_causal,
                            atomic_for_causal, stream):
    return _call('fa_v2_attn_fwd_compact_varlen',
                 [q, k, v, b, cu_seqlens_q, cu_seqlens_k, int(max_seqlen_q), int(max_seqlen_k), float(sm_scale),
                  softmax_lse, out, float(dropout_p), philox_seed, philox_offset1, int(philox_offset2),
                  philox_seed_output, philox_offset_output, encoded_softmax, int(bool(is_causal)),
                  atomic_for_causal], stream)


def attn_bwd(q, k, v, b, sm_scale, out, dout, dq, dk, dv, db, softmax_lse, delta, dropout_p, philox_seed,
             philox_offset1, philox_offset2, is_causal, stream):
    return _call('fa_v2_attn_bwd', [q, k, v, b, float(sm_scale), out, dout, dq, dk, dv, db, softmax_lse, delta,
                                    float(dropout_p), philox_seed, philox_offset1, int(philox_offset2),
                                    int(bool(is_causal))], stream)


def attn_bwd_fused(q, k, v, b, sm_scale, out, dout, dq, dk, dv, db, softmax_lse, dropout_p, philox_seed,
                   philox_offset1, philox_offset2, is_causal, stream):
    return _call('fa_v2_attn_bwd_fused', [q, k, v, b, float(sm_scale), out, dout, dq, dk, dv, db, softmax_lse,
                                          float(dropout_p), philox_seed, philox_offset1, int(philox_offset2),
                                          int(bool(is_causal))], stream)


def attn_bwd_compact_varlen(q, k, v, cu_seqlens_q, cu_seqlens_k, max_seqlen_q, max_seqlen_k, b, sm_scale, out,
                            dout, dq, dk, dv, db, softmax_lse, delta, dropout_p, philox_seed, philox_offset1,
                            philox_offset2, is_causal, stream):
    return _call('fa_v2_attn_bwd_compact_varlen',
                 [q, k, v, cu_seqlens_q, cu_seqlens_k, int(max_seqlen_q), int(max_seqlen_k), b, float(sm_scale), out,
                  dout, dq, dk, dv, db, softmax_lse, delta, float(dropout_p), philox_seed, philox_offset1,
                  int(philox_offset2), int(bool(is_causal))], stream)
