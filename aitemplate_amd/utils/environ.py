"""Environment switches (names kept from python/aitemplate/utils/environ.py and
backend/target.py:245-297 so existing workflows keep working)."""
import os


def recompile() -> bool:
    """AIT_RECOMPILE=0 makes compile_model() load the existing .so instead of rebuilding."""
    return os.environ.get("AIT_RECOMPILE", "1") != "0"


def force_profile() -> bool:
    return os.environ.get("FORCE_PROFILE", "0") == "1"


def ci_dummy_profiling() -> bool:
    """CI_FLAG=CIRCLECI: no GPU timing, the shape heuristic picks the kernel instance."""
    return os.environ.get("CI_FLAG", "") == "CIRCLECI"


def ndebug() -> bool:
    return os.environ.get("AIT_NDEBUG", "1") != "0"


def compiler_opt_level() -> str:
    return os.environ.get("AIT_COMPILER_OPT", "-O2")


def num_builders() -> int:
    n = os.environ.get("NUM_BUILDERS")
    if n:
        return max(1, int(n))
    return max(1, min(16, os.cpu_count() or 1))
