"""MI355X-native GEMM-family backend behind the AITemplate operator API."""

__version__ = "0.1.0"
