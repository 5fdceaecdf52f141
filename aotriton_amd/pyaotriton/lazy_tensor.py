"""Lazy tensors backed by torch allocations (bindings/lazy_tensor/main.cc:25-34,
lazy_tensor_template.h:19-98): the buffer is created only if the chosen backend
asks for it and is dropped when the operator returns."""
import ctypes

from .. import _lib


class _Lazy:
    """Owns the ctypes struct plus the Python callbacks that keep it alive."""
    C = None
    ACQ = None
    DISP = None
    VIEW = None

    def __init__(self, like_view, device_index, dtype=None, eager=None):
        import torch
        from . import DType
        self._like = like_view
        self._device = device_index
        self._held = None
        self.c = self.C()
        self.c.cookie = None
        if eager is not None:
            self.c.eager = eager.to_c()
            self._acq = self.ACQ(0)
            self._disp = self.DISP(0)
        else:
            view_c = self.VIEW

            def acquire(self_ptr, out_ptr):
                try:
                    dev = torch.device('cuda', self._device) if self._device is not None else None
                    t = torch.empty(tuple(self._like.sizes), dtype=torch.float32, device=dev)
                    self._held = t
                    out = out_ptr.contents
                    out.ptr = t.data_ptr()
                    for i in range(len(self._like.sizes)):
                        out.sizes[i] = t.size(i)
                        out.strides[i] = t.stride(i)
                    out.dtype = int(DType.kFloat32)
                    self_ptr.contents.cookie = 1
                    return 0
                except Exception:
                    return 1

            def dispose(self_ptr):
                self._held = None
                self_ptr.contents.cookie = None

            self._acq = self.ACQ(acquire)
            self._disp = self.DISP(dispose)
        self.c.acquire = self._acq
        self.c.dispose = self._disp

    def __bool__(self):
        return True


class LazyTensor2(_Lazy):
    C = _lib.fa_lazy_tensor2
    ACQ = _lib.ACQUIRE2
    DISP = _lib.DISPOSE2


class LazyTensor4(_Lazy):
    C = _lib.fa_lazy_tensor4
    ACQ = _lib.ACQUIRE4
    DISP = _lib.DISPOSE4


def delta(L_view, device_index):
    """fp32 tensor shaped like L, allocated on demand."""
    return LazyTensor2(L_view, device_index)


def dq_acc(dq_view, device_index):
    """fp32 tensor shaped like dQ; this library never acquires it."""
    return LazyTensor4(dq_view, device_index)


def eager_delta(delta_view):
    return LazyTensor2(delta_view, None, eager=delta_view)


def eager_null_dq_acc():
    from . import T4, DType
    return LazyTensor4(T4(0, [0] * 4, [0] * 4, DType.kFloat32), None,
                       eager=T4(0, [0] * 4, [0] * 4, DType.kFloat32))
