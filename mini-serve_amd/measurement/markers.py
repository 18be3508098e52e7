"""Range markers for the profiler (ROCTx). The reference wraps the measured part of its harness in
NVTX ranges so that a profile holds those steps and nothing of the set-up
(bench/offline.py:235-241,435,443-445); here the same with the ROCTx library that ships with ROCm:

    rocprofv3 --kernel-trace --marker-trace --stats --selected-regions -- python3 bench.py ...

keeps only what runs inside ``measured_region`` (it calls ``roctxProfilerResume`` on entry and
``roctxProfilerPause`` on exit; without ``--marker-trace`` the profiler does not see these calls and
records nothing); the marker trace also shows the named ranges of ``mark``. Without the library, or
outside a profiler, every call is a no-op."""

from __future__ import annotations

import contextlib
import ctypes

_lib = None
_tried = False


def _roctx():
    global _lib, _tried
    if not _tried:
        _tried = True
        for name in ("librocprofiler-sdk-roctx.so", "libroctx64.so"):
            try:
                lib = ctypes.CDLL(name)
                lib.roctxRangePushA.argtypes = [ctypes.c_char_p]
                lib.roctxRangePushA.restype = ctypes.c_int
                lib.roctxRangePop.restype = ctypes.c_int
                _lib = lib
                break
            except (OSError, AttributeError):
                continue
    return _lib


@contextlib.contextmanager
def mark(name: str):
    """A named range in the profiler's marker trace."""
    lib = _roctx()
    if lib is not None:
        lib.roctxRangePushA(name.encode())
    try:
        yield
    finally:
        if lib is not None:
            lib.roctxRangePop()


@contextlib.contextmanager
def measured_region(name: str = "measure"):
    """The steps a measurement times: a named range, and the only part a profiler started with
    ``--selected-regions`` records."""
    lib = _roctx()
    resume = getattr(lib, "roctxProfilerResume", None) if lib is not None else None
    pause = getattr(lib, "roctxProfilerPause", None) if lib is not None else None
    if resume is not None:
        resume.argtypes = [ctypes.c_uint64]
        resume(0)
    try:
        with mark(name):
            yield
    finally:
        if pause is not None:
            pause.argtypes = [ctypes.c_uint64]
            pause(0)
