"""detect_target(): the ROCm / gfx950 target (counterpart of python/aitemplate/testing/detect_target.py:87-133)."""
import os
import subprocess

from ..backend.rocm.target_def import ROCM

_DETECTED = None


def _detect_rocm_arch():
    """gfx arch string reported by rocminfo, or None when no GPU / no driver is present."""
    try:
        out = subprocess.run(["/opt/rocm/bin/rocminfo"], capture_output=True, text=True, timeout=20).stdout
    except Exception:
        return None
    for line in out.splitlines():
        line = line.strip()
        if line.startswith("Name:") and "gfx" in line:
            return line.split()[-1].split(":")[0]
    return None


def detect_target(**kwargs):
    """Return ROCM(arch="gfx950").  A different detected GPU is rejected; with no GPU at all
    (compile-only machines) the gfx950 target is still returned so graphs can be built and
    code generated, with the instance choice falling back to the shape heuristic."""
    global _DETECTED
    if _DETECTED is None:
        _DETECTED = os.environ.get("AIT_ROCM_ARCH") or _detect_rocm_arch() or "gfx950"
    if not _DETECTED.startswith("gfx950"):
        raise RuntimeError(f"Unsupported GPU {_DETECTED}: this backend targets gfx950 (MI355X)")
    return ROCM(arch="gfx950", **kwargs)
