"""MI355X (gfx950) flash attention behind the AOTriton flash operator API."""
from . import pyaotriton  # noqa: F401
from . import flash       # noqa: F401

__all__ = ['pyaotriton', 'flash']
