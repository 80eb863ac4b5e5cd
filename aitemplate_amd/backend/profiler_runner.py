"""Runs profiler executables as subprocesses, at most one in flight per GPU, and hands the
parsed timings to a post-processing delegate.

Counterpart of python/aitemplate/backend/profiler_runner.py:40-356.  The stdout protocol is the
reference's: one `OP:<instance>,TIME:<ms>,WS:<bytes>` line per timed instance; the device is
selected through the target's dev_select_flag (HIP_VISIBLE_DEVICES)."""
from __future__ import annotations

import logging
import os
import queue
import re
import subprocess
import threading
import time
from collections import namedtuple
from typing import Callable, List, Optional, Tuple, Union

_LOGGER = logging.getLogger(__name__)

PROF_RUNTIME_PATTERN = re.compile(r"OP:([a-zA-Z0-9_]+),TIME:([\d\.]+),WS:([\d]+)")
PROFILER_RUN_MAX_ATTEMPTS = 3
PROFILER_RUN_RETRY_DELAY_SECONDS = 1

ProfileResult = namedtuple("ProfileResult", "op_config duration workspace")


def extract_profile_result(stdout: str, return_ops: Optional[List[str]] = None
                           ) -> Tuple[Union[ProfileResult, List[ProfileResult]], bool]:
    """Parse profiler output.  With `return_ops` every listed instance is returned, otherwise
    the fastest one.  The flag is True when nothing could be parsed."""
    found = PROF_RUNTIME_PATTERN.findall(stdout or "")
    if not found:
        return ProfileResult(op_config="", duration=0, workspace=0), True
    results = [ProfileResult(op_config=n, duration=float(t), workspace=int(w)) for n, t, w in found]
    if return_ops is not None:
        keep = set(return_ops)
        return [r for r in results if r.op_config in keep], False
    return min(results, key=lambda r: r.duration), False


class ProfilerRunner:
    def __init__(self, devices: List[str], postprocessing_delegate, timeout: int = 500):
        if not devices:
            devices = ["0"]
        self._devices = [str(d) for d in devices]
        self._timeout = timeout
        self._postprocessing_delegate = postprocessing_delegate
        self._free_devices: "queue.Queue[str]" = queue.Queue()
        for d in self._devices:
            self._free_devices.put(d)
        self._threads: List[threading.Thread] = []
        self._errors: List[str] = []
        self._lock = threading.Lock()
        try:
            from .target import Target

            self._dev_flag = Target.current().dev_select_flag()
        except Exception:
            self._dev_flag = "HIP_VISIBLE_DEVICES"

    def _run_once(self, cmds: List[str], device: str) -> Tuple[str, str, int]:
        env = dict(os.environ)
        env[self._dev_flag] = device
        proc = subprocess.run([str(c) for c in cmds], capture_output=True, text=True, env=env, timeout=self._timeout)
        return proc.stdout, proc.stderr, proc.returncode

    def _worker(self, cmds, callback: Callable, return_ops, delegate_kwargs):
        device = self._free_devices.get()
        try:
            result, failed, err = None, True, ""
            for attempt in range(PROFILER_RUN_MAX_ATTEMPTS):
                try:
                    out, err, rc = self._run_once(cmds, device)
                except subprocess.TimeoutExpired:
                    out, err, rc = "", f"timed out after {self._timeout}s", None
                result, failed = extract_profile_result(out, return_ops)
                if not failed or rc == 0:
                    break
                if rc is None or rc < 0:
                    # The child hung or was ended by a signal (a GPU memory fault aborts it): running the
                    # same command again would repeat that on the device.  Report it once, do not retry.
                    how = "timed out" if rc is None else f"was killed by signal {-rc}"
                    with self._lock:
                        self._errors.append(
                            f"Profiler {how} (not retried): {' '.join(map(str, cmds))}\n{err}")
                    return
                time.sleep(PROFILER_RUN_RETRY_DELAY_SECONDS)
            if failed and callback is None:
                with self._lock:
                    self._errors.append(f"Profiler failure: {' '.join(map(str, cmds))}\n{err}")
                return
            with self._lock:
                if callback is not None:
                    callback(result, self._postprocessing_delegate)
                else:
                    named = [(r.op_config, r) for r in (result if isinstance(result, list) else [result])]
                    self._postprocessing_delegate.add_instance(named, **delegate_kwargs)
        except Exception as e:  # keep the pool alive; surface at join()
            with self._lock:
                self._errors.append(f"{type(e).__name__}: {e}")
        finally:
            self._free_devices.put(device)

    def push(self, cmds: List[str], process_result_callback: Optional[Callable] = None, return_ops=None,
             **delegate_kwargs) -> None:
        """Schedule one profiler run.  `process_result_callback(result, delegate)` receives the parsed
        result; without it the delegate's add_instance(results, **delegate_kwargs) is called."""
        if return_ops is None and "func_attrs" in delegate_kwargs and process_result_callback is None:
            return_ops = list(delegate_kwargs["func_attrs"].get("op_instance", {}).keys()) or None
        t = threading.Thread(target=self._worker, args=(cmds, process_result_callback, return_ops, delegate_kwargs),
                             daemon=True)
        t.start()
        self._threads.append(t)

    def join(self) -> None:
        for t in self._threads:
            t.join()
        self._threads = []
        if self._errors:
            raise RuntimeError("Profiling failed:\n" + "\n".join(self._errors))
        self._postprocessing_delegate.postprocess_results()
