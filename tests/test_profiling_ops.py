"""Range timers of scripted programs: `print(label, True / False)` markers become prof::Begin /
prof::End (fait/passes/profile_ops.cpp:16-30), timed as in fait/util/profile.cpp:133-245 and
reported by the harness entry points of functs/utils/prof.py:40-100."""
import ctypes
import re

import pytest
import torch
from torch.testing import FileCheck

import functs_amd.jit as fj
import functs_amd.prof as prof
from functs_amd import _C


def staged(x: torch.Tensor, y: torch.Tensor):
    print("first", True)
    a = (x * 2.0 + y).sigmoid()
    print("first", False)
    print("second", True)
    b = a.clone()
    b[0] = b[0] + 1.0
    print("second", False)
    print("not a marker", 3)
    return b


def test_markers_become_operators():
    g = torch.jit.script(staged).graph.copy()
    _C._jit_pass_convert_profiling_instrumentation(g)
    FileCheck().check('prof::Begin').check('prof::End').check('prof::Begin').check('prof::End').check(
        'prim::Print').run(str(g))
    assert str(g).count("prim::Print") == 1   # the print that is no marker stays


def test_disabled_ranges_record_nothing():
    prof.disable_profiling()
    prof.reset()
    prof.prof_begin("idle")
    prof.prof_end("idle")
    assert "idle" not in prof.profiling_results(1)


def test_ranges_are_counted_and_reported():
    prof.reset()
    prof.enable_profiling()
    try:
        for _ in range(3):
            prof.prof_begin("outer")
            prof.prof_begin("inner")
            prof.prof_end("inner")
            prof.prof_end("outer")
        with pytest.raises(RuntimeError, match="without a prof::Begin"):
            prof.prof_end("never opened")
    finally:
        prof.disable_profiling()
    text = prof.profiling_results(3)
    lines = {l.split()[0]: l.split() for l in text.splitlines() if l and l.split()[0] in ("outer", "inner", "Label")}
    assert lines["Label"] == ["Label", "Count", "Total", "Mean", "Min", "Max"]
    assert lines["outer"][1] == "3" and lines["inner"][1] == "3"
    assert all(re.fullmatch(r"[0-9.e+-]+(ns|us|ms|s)", c) for c in lines["outer"][2:])
    assert text.index("outer") < text.index("inner")   # order of first use


def test_c_entry_points_are_exported():
    lib = ctypes.CDLL(_C.__file__)
    for name in ("enableProfiling", "disableProfiling", "printProfilingResults"):
        assert hasattr(lib, name)


def test_scripted_program_with_markers_runs_on_the_cpu_interpreter(capfd):
    # functionalized but not built: the markers are ordinary operators of the graph
    g = torch.jit.script(staged).graph.copy()
    _C._jit_pass_convert_profiling_instrumentation(g)
    fn = _C._create_function_from_graph("staged", g)
    x, y = torch.rand(4, 8), torch.rand(4, 8)
    prof.reset()
    prof.enable_profiling()
    try:
        out = fn(x, y)
    finally:
        prof.disable_profiling()
    assert torch.equal(out, staged(x, y))
    text = prof.profiling_results(1)
    assert "first" in text and "second" in text


@pytest.mark.gpu
def test_ranges_around_fused_regions_on_the_gpu():
    dev = torch.device("cuda:0")
    x, y = torch.rand(64, 256), torch.rand(64, 256)
    fn = fj.build(fj.script(staged), [x, y])
    assert "prof::Begin" in str(fn.graph) and "tssa::ParallelFunctor" in str(fn.graph)
    gx, gy = x.to(dev), y.to(dev)
    fn(gx, gy)
    prof.reset()
    prof.enable_profiling()
    try:
        for _ in range(4):
            out = fn(gx, gy)
    finally:
        prof.disable_profiling()
    ref = staged(x, y)
    torch.testing.assert_close(out.cpu(), ref, rtol=1e-5, atol=1e-6)
    text = prof.profiling_results(4)
    m = re.search(r"Kernel launch: (\d+)", text)
    assert m and 1 <= int(m.group(1)) <= 3
    rows = {l.split()[0]: l.split() for l in text.splitlines() if l.startswith(("first", "second"))}
    assert rows["first"][1] == "4" and rows["second"][1] == "4"
