from .detect_target import detect_target  # noqa: F401
from . import test_utils  # noqa: F401
