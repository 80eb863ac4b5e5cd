from . import alignment, environ, shape_utils  # noqa: F401
