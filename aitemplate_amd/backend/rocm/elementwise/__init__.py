from . import elementwise  # noqa: F401
