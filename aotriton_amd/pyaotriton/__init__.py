"""Python surface shaped like the reference's ``pyaotriton`` module
(bindings/module.cc:58-113, bindings/hipruntime.cc:11-95, bindings/hipmemory.cc:15-69,
bindings/lazy_tensor/main.cc:25-34), bound to the C ABI with ctypes."""
import ctypes
import enum

from .. import _lib
from .._lib import lib


class DType(enum.IntEnum):
    # include/aotriton/dtypes.h:12-25
    kUnknown = 0
    kFloat32 = 1
    kFloat16 = 2
    kBFloat16 = 3
    kInt8 = 10
    kInt16 = 11
    kInt32 = 12
    kInt64 = 13
    kUInt8 = 20
    kUInt16 = 21
    kUInt32 = 22
    kUInt64 = 23


class hipError_t(enum.IntEnum):
    # subset the bindings expose (bindings/hipruntime.cc) that this library returns
    hipSuccess = 0
    hipErrorInvalidValue = 1
    hipErrorOutOfMemory = 2
    hipErrorProfilerNotInitialized = 6
    hipErrorInvalidSymbol = 13
    hipErrorPriorLaunchFailure = 53
    hipErrorInvalidDevice = 101
    hipErrorInvalidImage = 200
    hipErrorNoBinaryForGpu = 209
    hipErrorPeerAccessUnsupported = 217
    hipErrorSharedObjectSymbolNotFound = 302
    hipErrorIllegalAddress = 700
    hipErrorLaunchFailure = 719
    hipErrorNotSupported = 801
    hipErrorUnknown = 999

    @classmethod
    def _missing_(cls, value):
        obj = int.__new__(cls, value)
        obj._name_ = f'hipError_{value}'
        obj._value_ = value
        return obj


class Stream:
    """include/aotriton/runtime.h:15-31; Stream() is the null stream."""

    def __init__(self, native=None):
        self._native = int(native) if native else 0

    def native(self):
        return self._native


class _TensorView:
    RANK = 0
    CTYPE = None

    def __init__(self, ptr=0, sizes=None, strides=None, dtype=DType.kUnknown):
        rank = self.RANK
        sizes = [0] * rank if sizes is None else list(sizes)
        strides = [0] * rank if strides is None else list(strides)
        assert len(sizes) == rank and len(strides) == rank, f'rank-{rank} view needs {rank} sizes/strides'
        self._ptr = int(ptr)
        self._sizes = [int(x) for x in sizes]
        self._strides = [int(x) for x in strides]
        self._dtype = DType(int(dtype))

    def __bool__(self):
        return self._ptr != 0

    def size(self, i):
        return self._sizes[i]

    def stride(self, i):
        return self._strides[i]

    @property
    def sizes(self):
        return list(self._sizes)

    @property
    def strides(self):
        return list(self._strides)

    @property
    def data_ptr(self):
        return self._ptr

    @property
    def dtype(self):
        return self._dtype

    def to_c(self):
        c = self.CTYPE()
        c.ptr = self._ptr or None
        for i in range(self.RANK):
            c.sizes[i] = self._sizes[i]
            c.strides[i] = self._strides[i]
        c.dtype = int(self._dtype)
        return c

    @classmethod
    def from_c(cls, c):
        return cls(c.ptr or 0, list(c.sizes), list(c.strides), c.dtype)

    def __repr__(self):
        return f'T{self.RANK}(0x{self._ptr:x}, {self._sizes}, {self._strides}, {self._dtype.name})'


class T4(_TensorView):
    RANK = 4
    CTYPE = _lib.fa_tensor4


class T2(_TensorView):
    RANK = 2
    CTYPE = _lib.fa_tensor2


class T1(_TensorView):
    RANK = 1
    CTYPE = _lib.fa_tensor1


class T0:
    """TensorView<0>: a device scalar (include/aotriton/util.h:160-210)."""

    def __init__(self, ptr=0, dtype=DType.kUnknown):
        self._ptr = int(ptr)
        self._dtype = DType(int(dtype))

    def __bool__(self):
        return self._ptr != 0

    def size(self, i):
        return 1 if i == 0 else 0

    def stride(self, i):
        return 1 if i == 0 else 0

    @property
    def sizes(self):
        return []

    @property
    def strides(self):
        return []

    @property
    def data_ptr(self):
        return self._ptr

    @property
    def dtype(self):
        return self._dtype

    def to_c(self):
        c = _lib.fa_tensor0()
        c.ptr = self._ptr or None
        c.dtype = int(self._dtype)
        return c


def get_name_suffix():
    return lib.fa_get_name_suffix().decode()


def hipGetLastError():
    return hipError_t(lib.fa_hip_get_last_error())


def hipDeviceSynchronize():
    return hipError_t(lib.fa_hip_device_synchronize())


class HipMemory:
    """bindings/hipmemory.cc:15-69: a raw device allocation used when torch itself
    stays on the CPU.  Backed by the HIP runtime that the library links."""

    def __init__(self):
        self._hip = ctypes.CDLL('libamdhip64.so')
        self._ptr = ctypes.c_void_p(0)
        self._size = 0

    def alloc(self, nbytes):
        self.free()
        err = self._hip.hipMalloc(ctypes.byref(self._ptr), ctypes.c_size_t(nbytes))
        if err != 0:
            raise MemoryError(f'hipMalloc({nbytes}) -> {err}')
        self._size = nbytes

    def free(self):
        if self._ptr.value:
            self._hip.hipFree(self._ptr)
            self._ptr = ctypes.c_void_p(0)
            self._size = 0

    def get_pointer(self):
        return self._ptr.value or 0

    def load_from_host(self, host_ptr, nbytes):
        return self._hip.hipMemcpy(self._ptr, ctypes.c_void_p(host_ptr), ctypes.c_size_t(nbytes), 1)

    def store_to_host(self, host_ptr, nbytes):
        return self._hip.hipMemcpy(ctypes.c_void_p(host_ptr), self._ptr, ctypes.c_size_t(nbytes), 2)

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


from . import lazy_tensor  # noqa: E402,F401
from . import v2, v3       # noqa: E402,F401
