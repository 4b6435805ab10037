"""Range timers around parts of a scripted program (the harness of functs/utils/prof.py:40-100).

In a program, `print("label", True)` opens the range `label` and `print("label", False)` closes
it; `functs_amd.jit.build` turns those markers into `prof::Begin` / `prof::End` operators
(fait/passes/profile_ops.cpp:16-30).  A range is bracketed by device synchronisations, shows up as
a roctx range under `rocprofv3 --marker-trace`, and costs nothing while profiling is disabled::

    import functs_amd.prof as prof
    prof.enable_profiling()
    for _ in range(n): fn(*inputs)
    prof.disable_profiling()
    prof.print_profiling_results(n)

The C entry points `enableProfiling`, `disableProfiling` and `printProfilingResults(size_t)` are
exported by `functs_amd/_C.so` for harnesses that load them with ctypes, as the reference's does.
"""
import ctypes

from . import _C

_lib = ctypes.CDLL(_C.__file__)
_lib.printProfilingResults.argtypes = [ctypes.c_size_t]
_lib.metricsEnabled.restype = ctypes.c_bool
_lib.allPassesSubmitted.restype = ctypes.c_bool


def metrics_enabled() -> bool:
    """Counter passes inside the process (functs/utils/prof.py:16-36) have no counterpart here:
    hardware counters are read with rocprofv3 from outside.  Always False."""
    return bool(_lib.metricsEnabled())


def initialize_metrics():
    _lib.initializeMetrics()


def finalize_metrics():
    _lib.finalizeMetrics()


def begin_profiler_pass():
    _lib.beginProfilerPass()


def end_profiler_pass():
    _lib.endProfilerPass()


def all_passes_submitted() -> bool:
    return bool(_lib.allPassesSubmitted())


def enable_profiling():
    _lib.enableProfiling()


def disable_profiling():
    _lib.disableProfiling()


def prof_begin(label: str):
    """Open a range from Python (eager code); inside a scripted program use print(label, True)."""
    _C._prof_begin(label)


def prof_end(label: str):
    _C._prof_end(label)


def profiling_results(count: int) -> str:
    """Launches of region kernels per run and one line per label: count, total, mean, min, max."""
    return _C._prof_results(int(count))


def print_profiling_results(count: int):
    _lib.printProfilingResults(ctypes.c_size_t(int(count)))


def reset():
    _C._prof_reset()
