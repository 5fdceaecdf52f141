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
