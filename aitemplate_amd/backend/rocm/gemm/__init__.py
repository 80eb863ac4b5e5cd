"""Importing this package registers the ROCm hooks of the GEMM family."""
from . import bmm_rcr, bmm_softmax_bmm_permute, gemm_rcr_family, gemm_rcr_permute  # noqa: F401
