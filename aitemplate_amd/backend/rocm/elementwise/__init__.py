from . import elementwise, strided_copy  # noqa: F401
