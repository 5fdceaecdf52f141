from . import flash  # noqa: F401
