"""pyaotriton.v3.flash (modules/flash/bindings/v3.cc:26-128): params structs with
the reference's member names, attn_fwd / attn_bwd taking
(params, params_version, stream, options)."""
import ctypes

from ... import _lib
from ..._lib import lib
from .. import DType, T0, T1, T2, T4, hipError_t    # defined before the parent package imports this module


class attn_options:
    def __init__(self):
        self.force_backend_index = -1
        self.deterministic = False

    def to_c(self):
        c = _lib.fa_options()
        c.force_backend_index = int(self.force_backend_index)
        c.deterministic = 1 if self.deterministic else 0
        return c


def _null(cls_name):
    """A null view of the given rank.  Views are immutable, so one object per rank serves
    every params struct."""
    v = _NULLS.get(cls_name)
    if v is None:
        cls = {'T0': T0, 'T1': T1, 'T2': T2, 'T4': T4}[cls_name]
        v = T0(0, DType.kUnknown) if cls is T0 else cls(0, [0] * cls.RANK, [0] * cls.RANK, DType.kUnknown)
        _NULLS[cls_name] = v
    return v


_NULLS = {}


class attn_fwd_params:
    kVersion = 3

    _T = dict(Q='T4', K='T4', V='T4', B='T4', A='T2', L='T2', Out='T4', cu_seqlens_q='T1',
              cu_seqlens_k='T1', seq_strides_q='T1', seq_strides_k='T1', philox_seed_ptr='T0',
              philox_offset1='T0', philox_seed_output='T0', philox_offset_output='T0',
              encoded_softmax='T4', persistent_atomic_counter='T0')

    def __init__(self):
        for k, t in self._T.items():
            setattr(self, k, _null(t))
        self.Sm_scale = 0.0
        self.Max_seqlen_q = 0
        self.Max_seqlen_k = 0
        self.dropout_p = 0.0
        self.philox_offset2 = 0
        self.causal_type = 0
        self.varlen_type = 0
        self.window_left = 0
        self.window_right = 0

    def to_c(self):
        c = _lib.fa_fwd_params()
        for k in self._T:
            setattr(c, k, getattr(self, k).to_c())
        c.Sm_scale = float(self.Sm_scale)
        c.Max_seqlen_q = int(self.Max_seqlen_q)
        c.Max_seqlen_k = int(self.Max_seqlen_k)
        c.dropout_p = float(self.dropout_p)
        c.philox_offset2 = int(self.philox_offset2) & 0xFFFFFFFFFFFFFFFF
        c.causal_type = int(self.causal_type)
        c.varlen_type = int(self.varlen_type)
        c.window_left = int(self.window_left)
        c.window_right = int(self.window_right)
        return c


class attn_bwd_params:
    kVersion = 6

    _T = dict(Q='T4', K='T4', V='T4', B='T4', Out='T4', DO='T4', DK='T4', DV='T4', DQ='T4', DB='T4',
              L='T2', cu_seqlens_q='T1', cu_seqlens_k='T1', seq_strides_q='T1', seq_strides_k='T1',
              philox_seed_ptr='T0', philox_offset1='T0')

    def __init__(self):
        for k, t in self._T.items():
            setattr(self, k, _null(t))
        self.Sm_scale = 0.0
        self.D = None        # lazy_tensor.delta(...) / eager_delta(...)
        self.DQ_ACC = None   # lazy_tensor.dq_acc(...)
        self.Max_seqlen_q = 0
        self.Max_seqlen_k = 0
        self.dropout_p = 0.0
        self.philox_offset2 = 0
        self.causal_type = 0
        self.varlen_type = 0
        self.window_left = 0
        self.window_right = 0

    def to_c(self):
        c = _lib.fa_bwd_params()
        for k in self._T:
            setattr(c, k, getattr(self, k).to_c())
        c.Sm_scale = float(self.Sm_scale)
        if self.D is not None:
            c.D = self.D.c
        if self.DQ_ACC is not None:
            c.DQ_ACC = self.DQ_ACC.c
        c.Max_seqlen_q = int(self.Max_seqlen_q)
        c.Max_seqlen_k = int(self.Max_seqlen_k)
        c.dropout_p = float(self.dropout_p)
        c.philox_offset2 = int(self.philox_offset2) & 0xFFFFFFFFFFFFFFFF
        c.causal_type = int(self.causal_type)
        c.varlen_type = int(self.varlen_type)
        c.window_left = int(self.window_left)
        c.window_right = int(self.window_right)
        return c




def _opt(options):
    if options is None:
        return None, None
    c = options.to_c()
    return c, ctypes.byref(c)


def attn_fwd(params, params_version, stream, options=None):
    c = params.to_c()
    keep, optp = _opt(options)
    return hipError_t(lib.fa_attn_fwd(ctypes.byref(c), int(params_version), stream.native() or None, optp))


def attn_bwd(params, params_version, stream, options=None):
    c = params.to_c()
    keep, optp = _opt(options)
    return hipError_t(lib.fa_attn_bwd(ctypes.byref(c), int(params_version), stream.native() or None, optp))


def attn_bwd_noalloc(params, params_version, stream):
    """Split backward with delta in the library's own device array: allocates nothing, ignores
    params.D; at most FA_NOALLOC_MAX_ROWS delta values (hipErrorOutOfMemory beyond)."""
    c = params.to_c()
    return hipError_t(lib.fa_attn_bwd_noalloc(ctypes.byref(c), int(params_version), stream.native() or None))


def attn_bwd_kernel(params, params_version, stream, kernel_slot):
    """Launch one backward kernel only (0 delta, 1 dK/dV, 2 dQ, 3 fused)."""
    c = params.to_c()
    return hipError_t(lib.fa_attn_bwd_kernel(ctypes.byref(c), int(params_version),
                                             stream.native() or None, int(kernel_slot)))


def validate_fwd(params, params_version, options=None):
    c = params.to_c()
    keep, optp = _opt(options)
    return hipError_t(lib.fa_validate_fwd(ctypes.byref(c), int(params_version), optp))


def validate_bwd(params, params_version, options=None):
    c = params.to_c()
    keep, optp = _opt(options)
    return hipError_t(lib.fa_validate_bwd(ctypes.byref(c), int(params_version), optp))


def query_fwd_config(params, num_cu=256):
    c = params.to_c()
    out = _lib.fa_kernel_config()
    err = hipError_t(lib.fa_query_fwd_config(ctypes.byref(c), int(num_cu), ctypes.byref(out)))
    return err, out


def query_bwd_config(params, kernel_slot, options=None):
    c = params.to_c()
    keep, optp = _opt(options)
    out = _lib.fa_kernel_config()
    err = hipError_t(lib.fa_query_bwd_config(ctypes.byref(c), optp, int(kernel_slot), ctypes.byref(out)))
    return err, out
