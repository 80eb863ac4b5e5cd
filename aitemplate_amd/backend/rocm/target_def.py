"""The ROCm target for gfx950 (MI355X).

Counterpart of python/aitemplate/backend/rocm/target_def.py:43-234.  Differences
that follow from the design: the kernels are prebuilt in
libaitemplate_amd_kernels.so, so the per-model build is host-only C++ (no CK include
paths, no device code, no rocrand) and the arch gate accepts gfx950 only.
"""
from __future__ import annotations

import os
import re
from typing import List

from ... import _kernels
from ...utils import environ
from ..target import Target

_PKG_ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
STATIC_PATH = os.path.join(_PKG_ROOT, "static")
LIB_PATH = os.path.join(_PKG_ROOT, "lib")
INCLUDE_PATH = os.path.join(os.path.dirname(_PKG_ROOT), "include")


class ROCM(Target):
    SUPPORTED_ARCHS = ("gfx950",)

    def __init__(self, arch: str = "gfx950", **kwargs):
        super().__init__(STATIC_PATH)
        if arch.lower() not in self.SUPPORTED_ARCHS:
            raise RuntimeError(f"Unsupported ROCm arch {arch}: this backend is written for gfx950 (MI355X) only")
        self._arch = arch.lower()
        self._kwargs = kwargs
        self._rocm_path = os.environ.get("ROCM_PATH", "/opt/rocm")

    def name(self) -> str:
        return "rocm"

    def arch(self) -> str:
        return self._arch

    def device_name(self) -> str:
        return f"rocm-{self._arch}"

    def cc(self) -> str:
        return os.environ.get("AIT_HOST_CXX", "g++")

    def dev_select_flag(self) -> str:
        return "HIP_VISIBLE_DEVICES"

    def compile_options(self) -> List[str]:
        opts = [environ.compiler_opt_level(), "-std=c++17", "-fPIC", "-fvisibility=hidden", "-w",
                "-D__HIP_PLATFORM_AMD__", f"-I{self._rocm_path}/include",
                f"-I{os.path.join(STATIC_PATH, 'include')}", f"-I{INCLUDE_PATH}"]
        if environ.ndebug():
            opts.append("-DNDEBUG")
        return opts

    def compile_cmd(self, executable: bool = False) -> str:
        """Command template with {target} and {src} placeholders."""
        opts = " ".join(self.compile_options())
        if executable:
            return f"{self.cc()} {opts} -o {{target}} {{src}} {self.link_options(shared=False)}"
        return f"{self.cc()} {opts} -c -o {{target}} {{src}}"

    def link_options(self, shared: bool = True) -> str:
        """A model library is self-contained: the runtime archive whole, and from the kernel archive the objects
        its op functions refer to (each names the instance table it dispatches through).  Nothing points back
        into this source tree; the only shared libraries it needs are the HIP runtime and the C++ runtime
        (reference: backend/builder.py:398-527, where everything is linked into test.so)."""
        flags = ["-shared"] if shared else []
        flags += [
            f"-L{LIB_PATH}",
            # the runtime archive's C ABI objects are referenced by nobody inside the library: keep all of it
            "-Wl,--whole-archive -laitemplate_amd_runtime -Wl,--no-whole-archive" if shared else "",
            "-l:libaitemplate_amd_kernels_static.a",
            # the kernel entry points stay private to the model library (a process may hold several model
            # libraries and the shared kernel library at once)
            "-Wl,--exclude-libs,libaitemplate_amd_kernels_static.a",
            f"-L{self._rocm_path}/lib", "-lamdhip64", "-lpthread",
            f"-Wl,-rpath,{self._rocm_path}/lib",
        ]
        return " ".join(f for f in flags if f)

    def kernel_library(self):
        """The loaded kernel library (fails loudly when it has not been built)."""
        return _kernels.load()

    def profiler_executable(self) -> str:
        path = os.path.join(LIB_PATH, "aitamd_profiler")
        if not os.access(path, os.X_OK):
            raise RuntimeError(f"profiler executable {path} is missing: run `make -C aitemplate_amd/csrc`")
        return path

    def select_minimal_algo(self, algo_names: List[str]) -> str:
        """Smallest tile by area among `algo_names` (instance names carry `<BM>x<BN>x<BK>`).

        Plays the role of ROCM.select_minimal_algo of the reference
        (backend/rocm/target_def.py:214-234), for this backend's instance names."""
        best, best_area = None, None
        for name in algo_names:
            m = re.search(r"_(\d+)x(\d+)x(\d+)_", name)
            if m is None:
                continue
            area = int(m.group(1)) * int(m.group(2))
            if best is None or area < best_area:
                best, best_area = name, area
        if best is None:
            if not algo_names:
                raise RuntimeError("no kernel instance to choose from")
            best = algo_names[0]
        return best
