"""MI355X (gfx950) flash attention behind the AOTriton flash operator API.

Submodules (imported on demand so that ``python -m aotriton_amd.build`` can run
before the shared library exists):
  pyaotriton  pyaotriton-shaped bindings over the C ABI (ctypes)
  flash       host layer: tensor marshalling, v2/v3 operator wrappers
  autograd    torch.autograd Functions
  build       hipcc driver that builds libaotriton_amd.so in-tree
"""
import importlib

__all__ = ['pyaotriton', 'flash', 'autograd', 'build']


def __getattr__(name):
    if name in __all__:
        return importlib.import_module(f'{__name__}.{name}')
    raise AttributeError(name)
