"""ctypes binding of libaotriton_amd.so (the C ABI declared in include/aotriton_amd/flash.h).

The library is the product path; if it is missing this module raises instead of
falling back to anything else.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, 'libaotriton_amd.so')


class fa_tensor4(ctypes.Structure):
    _fields_ = [('ptr', ctypes.c_void_p), ('sizes', ctypes.c_uint64 * 4),
                ('strides', ctypes.c_uint64 * 4), ('dtype', ctypes.c_int32)]


class fa_tensor2(ctypes.Structure):
    _fields_ = [('ptr', ctypes.c_void_p), ('sizes', ctypes.c_uint64 * 2),
                ('strides', ctypes.c_uint64 * 2), ('dtype', ctypes.c_int32)]


class fa_tensor1(ctypes.Structure):
    _fields_ = [('ptr', ctypes.c_void_p), ('sizes', ctypes.c_uint64 * 1),
                ('strides', ctypes.c_uint64 * 1), ('dtype', ctypes.c_int32)]


class fa_tensor0(ctypes.Structure):
    _fields_ = [('ptr', ctypes.c_void_p), ('dtype', ctypes.c_int32)]


class fa_lazy_tensor2(ctypes.Structure):
    pass


ACQUIRE2 = ctypes.CFUNCTYPE(ctypes.c_int, ctypes.POINTER(fa_lazy_tensor2), ctypes.POINTER(fa_tensor2))
DISPOSE2 = ctypes.CFUNCTYPE(None, ctypes.POINTER(fa_lazy_tensor2))
fa_lazy_tensor2._fields_ = [('cookie', ctypes.c_void_p), ('acquire', ACQUIRE2),
                            ('dispose', DISPOSE2), ('eager', fa_tensor2)]


class fa_lazy_tensor4(ctypes.Structure):
    pass


ACQUIRE4 = ctypes.CFUNCTYPE(ctypes.c_int, ctypes.POINTER(fa_lazy_tensor4), ctypes.POINTER(fa_tensor4))
DISPOSE4 = ctypes.CFUNCTYPE(None, ctypes.POINTER(fa_lazy_tensor4))
fa_lazy_tensor4._fields_ = [('cookie', ctypes.c_void_p), ('acquire', ACQUIRE4),
                            ('dispose', DISPOSE4), ('eager', fa_tensor4)]


class fa_options(ctypes.Structure):
    _fields_ = [('force_backend_index', ctypes.c_int32), ('deterministic', ctypes.c_int32)]


class fa_fwd_params(ctypes.Structure):
    _fields_ = [
        ('Q', fa_tensor4), ('K', fa_tensor4), ('V', fa_tensor4), ('B', fa_tensor4), ('A', fa_tensor2),
        ('Sm_scale', ctypes.c_float), ('L', fa_tensor2), ('Out', fa_tensor4),
        ('cu_seqlens_q', fa_tensor1), ('cu_seqlens_k', fa_tensor1),
        ('Max_seqlen_q', ctypes.c_int32), ('Max_seqlen_k', ctypes.c_int32),
        ('seq_strides_q', fa_tensor1), ('seq_strides_k', fa_tensor1),
        ('dropout_p', ctypes.c_float),
        ('philox_seed_ptr', fa_tensor0), ('philox_offset1', fa_tensor0), ('philox_offset2', ctypes.c_uint64),
        ('philox_seed_output', fa_tensor0), ('philox_offset_output', fa_tensor0),
        ('encoded_softmax', fa_tensor4), ('persistent_atomic_counter', fa_tensor0),
        ('causal_type', ctypes.c_int8), ('varlen_type', ctypes.c_int8),
        ('window_left', ctypes.c_int32), ('window_right', ctypes.c_int32),
    ]


class fa_bwd_params(ctypes.Structure):
    _fields_ = [
        ('Q', fa_tensor4), ('K', fa_tensor4), ('V', fa_tensor4), ('B', fa_tensor4),
        ('Sm_scale', ctypes.c_float),
        ('Out', fa_tensor4), ('DO', fa_tensor4), ('DK', fa_tensor4), ('DV', fa_tensor4),
        ('DQ', fa_tensor4), ('DB', fa_tensor4), ('L', fa_tensor2), ('D', fa_lazy_tensor2),
        ('cu_seqlens_q', fa_tensor1), ('cu_seqlens_k', fa_tensor1),
        ('Max_seqlen_q', ctypes.c_int32), ('Max_seqlen_k', ctypes.c_int32),
        ('seq_strides_q', fa_tensor1), ('seq_strides_k', fa_tensor1),
        ('dropout_p', ctypes.c_float),
        ('philox_seed_ptr', fa_tensor0), ('philox_offset1', fa_tensor0), ('philox_offset2', ctypes.c_uint64),
        ('causal_type', ctypes.c_int8), ('varlen_type', ctypes.c_int8),
        ('window_left', ctypes.c_int32), ('window_right', ctypes.c_int32),
        ('DQ_ACC', fa_lazy_tensor4),
    ]


class fa_kernel_config(ctypes.Structure):
    _fields_ = [('block_m', ctypes.c_int32), ('block_n', ctypes.c_int32), ('num_waves', ctypes.c_int32),
                ('lds_bytes', ctypes.c_int32), ('grid', ctypes.c_int32 * 3),
                ('backend_index', ctypes.c_int32), ('head_dim', ctypes.c_int32), ('flags', ctypes.c_int32)]


# every symbol include/aotriton_amd/flash.h declares: name -> (restype, argtypes)
P = ctypes.POINTER
SYMBOLS = {
    'fa_check_gpu': (ctypes.c_int, [ctypes.c_void_p]),
    'fa_attn_fwd': (ctypes.c_int, [P(fa_fwd_params), ctypes.c_int32, ctypes.c_void_p, P(fa_options)]),
    'fa_attn_bwd': (ctypes.c_int, [P(fa_bwd_params), ctypes.c_int32, ctypes.c_void_p, P(fa_options)]),
    'fa_v2_attn_fwd': (ctypes.c_int, [P(fa_tensor4)] * 4 + [ctypes.c_float, P(fa_tensor2), P(fa_tensor4), ctypes.c_float,
                                      P(fa_tensor0), P(fa_tensor0), ctypes.c_int64, P(fa_tensor0), P(fa_tensor0),
                                      P(fa_tensor4), ctypes.c_int32, P(fa_tensor0), ctypes.c_void_p]),
    'fa_v2_attn_fwd_compact_varlen': (ctypes.c_int, [P(fa_tensor4)] * 4 + [P(fa_tensor1), P(fa_tensor1), ctypes.c_int32,
                                                     ctypes.c_int32, ctypes.c_float, P(fa_tensor2), P(fa_tensor4),
                                                     ctypes.c_float, P(fa_tensor0), P(fa_tensor0), ctypes.c_int64,
                                                     P(fa_tensor0), P(fa_tensor0), P(fa_tensor4), ctypes.c_int32,
                                                     P(fa_tensor0), ctypes.c_void_p]),
    'fa_v2_attn_bwd': (ctypes.c_int, [P(fa_tensor4)] * 4 + [ctypes.c_float] + [P(fa_tensor4)] * 6 +
                       [P(fa_tensor2), P(fa_tensor2), ctypes.c_float, P(fa_tensor0), P(fa_tensor0), ctypes.c_int64,
                        ctypes.c_int32, ctypes.c_void_p]),
    'fa_v2_attn_bwd_fused': (ctypes.c_int, [P(fa_tensor4)] * 4 + [ctypes.c_float] + [P(fa_tensor4)] * 6 +
                             [P(fa_tensor2), ctypes.c_float, P(fa_tensor0), P(fa_tensor0), ctypes.c_int64,
                              ctypes.c_int32, ctypes.c_void_p]),
    'fa_v2_attn_bwd_compact_varlen': (ctypes.c_int, [P(fa_tensor4)] * 3 + [P(fa_tensor1), P(fa_tensor1), ctypes.c_int32,
                                                     ctypes.c_int32, P(fa_tensor4), ctypes.c_float] +
                                      [P(fa_tensor4)] * 6 + [P(fa_tensor2), P(fa_tensor2), ctypes.c_float,
                                                             P(fa_tensor0), P(fa_tensor0), ctypes.c_int64,
                                                             ctypes.c_int32, ctypes.c_void_p]),
    'fa_attn_bwd_noalloc': (ctypes.c_int, [P(fa_bwd_params), ctypes.c_int32, ctypes.c_void_p]),
    'fa_set_bwd_workspace_limit': (None, [ctypes.c_int64]),
    'fa_trim_workspace': (ctypes.c_int, []),
    'fa_attn_bwd_kernel': (ctypes.c_int, [P(fa_bwd_params), ctypes.c_int32, ctypes.c_void_p, ctypes.c_int32]),
    'fa_debug_simulate_encoded_softmax': (ctypes.c_int, [P(fa_tensor4), ctypes.c_float, P(fa_tensor0),
                                                         P(fa_tensor0), ctypes.c_uint64, ctypes.c_void_p]),
    'fa_validate_fwd': (ctypes.c_int, [P(fa_fwd_params), ctypes.c_int32, P(fa_options)]),
    'fa_validate_bwd': (ctypes.c_int, [P(fa_bwd_params), ctypes.c_int32, P(fa_options)]),
    'fa_query_fwd_config': (ctypes.c_int, [P(fa_fwd_params), ctypes.c_int32, P(fa_kernel_config)]),
    'fa_query_bwd_config': (ctypes.c_int, [P(fa_bwd_params), P(fa_options), ctypes.c_int32, P(fa_kernel_config)]),
    'fa_tile_intervals': (ctypes.c_int, [ctypes.c_int32] * 8 + [P(ctypes.c_int32)]),
    'fa_dropout_threshold': (ctypes.c_int32, [ctypes.c_float]),
    'fa_get_name_suffix': (ctypes.c_char_p, []),
    'fa_version': (ctypes.c_char_p, []),
    'fa_get_arch': (ctypes.c_int, [ctypes.c_void_p, ctypes.c_char_p, ctypes.c_int32]),
    'fa_get_multiprocessor_count': (ctypes.c_int, [ctypes.c_void_p]),
    'fa_get_clock_rate_khz': (ctypes.c_int, [ctypes.c_void_p]),
    'fa_probe_mfma_rate': (ctypes.c_int, [ctypes.c_int32, ctypes.c_int32, ctypes.c_int32, ctypes.c_void_p,
                                          ctypes.c_void_p, ctypes.c_void_p]),
    'fa_hip_get_last_error': (ctypes.c_int, []),
    'fa_hip_device_synchronize': (ctypes.c_int, []),
}


def _load():
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f'{LIB_PATH} is missing: build it with `python -m aotriton_amd.build` '
            '(hipcc --offload-arch=gfx950). There is no fallback path.')
    lib = ctypes.CDLL(LIB_PATH)
    for name, (res, args) in SYMBOLS.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    return lib


lib = _load()
