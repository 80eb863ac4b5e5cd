"""Backend: registry, target, code generation, build, profiling.  The ROCm hooks register
themselves when `aitemplate_amd.backend.rocm` is imported (detect_target / compile_model do)."""
from . import registry, target  # noqa: F401
