from . import bwd, fwd  # noqa: F401
