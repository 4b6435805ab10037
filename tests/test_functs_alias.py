"""A script written against the reference's import names runs unchanged: `import functs._C`,
`functs.jit`, the step-by-step pass calls of the reference's walkthrough
(examples/get_started.py:39-75: the same sequence of calls, on a program of this test's own) and
the entry points functs/csrc/jit/python/init.cpp:45-48 adds (`_jit_pass_fait_shape_infer`,
`_jit_pass_freeze`, `_jit_pass_clone`), plus the metric entry points a harness resolves from the
library (fait/util/metrics.h:6-13, functs/utils/prof.py:19-36)."""
import ctypes

import pytest
import torch

import functs
import functs._C
import functs.jit
import functs.utils.prof as fprof


def rows_plus_one(a: torch.Tensor, b: torch.Tensor, n: int):
    a = a.clone()
    b = b.clone()
    for i in range(n):
        b[i] = b[i] + 1
    return b


def test_walkthrough_pass_by_pass_under_the_reference_names():
    jit_func = torch.jit.script(rows_plus_one)
    g = jit_func.graph.copy()
    info = functs._C.TensorSSAMutateInfo()
    functs._C._jit_pass_rewrite_mutation(g, info)
    assert len(info.mutValues) >= 1 and len(info.mutNodes) >= 1
    assert "immut::select_rev" in str(g) and "tssa::update" in str(g)
    functs._C._jit_pass_block_propagation(g, info)
    functs._C._jit_pass_rename(g)
    functs._C._jit_pass_tensorssa_remove_update(g)
    torch._C._jit_pass_cse(g)
    torch._C._jit_pass_dce(g)
    torch._C._jit_pass_constant_propagation(g)
    assert "tssa::update" not in str(g) and "aten::copy_" not in str(g)
    fn = torch._C._create_function_from_graph("rows_plus_one", g)
    a, b = torch.randn(16, 16), torch.randn(16, 16)
    assert torch.equal(fn(a, b, 3), rows_plus_one(a, b, 3))


def test_script_under_the_reference_name():
    fn = functs.jit.script(rows_plus_one)
    a, b = torch.randn(8, 8), torch.randn(8, 8)
    assert torch.equal(fn(a, b, 8), rows_plus_one(a, b, 8))
    assert functs.jit.build is not None and functs.jit.shape_infer is not None


def bias_rows(a: torch.Tensor, b: torch.Tensor):
    return a + b.sum(0)


def test_fait_shape_infer_refines_inputs_and_propagates():
    g = torch.jit.script(bias_rows).graph.copy()
    hints = [functs.jit.extract_type_hint_from_tensor(torch.rand(3, 4)),
             functs.jit.extract_type_hint_from_tensor(torch.rand(5, 4))]
    functs._C._jit_pass_fait_shape_infer(g, hints, {})
    ins = list(g.inputs())
    assert ins[0].type().sizes() == [3, 4] and ins[1].type().sizes() == [5, 4]
    out = list(g.outputs())[0].type()
    assert out.dtype() == torch.float32 and out.sizes() == [3, 4]


class Scale(torch.nn.Module):
    def __init__(self):
        super().__init__()
        self.w = torch.nn.Parameter(torch.full((3,), 2.0))

    def forward(self, x):
        return x * self.w


def test_freeze_and_clone_of_a_module():
    m = torch.jit.script(Scale().eval())
    c = functs._C._jit_pass_clone(m._c)
    assert "GetAttr" in str(m._c.forward.graph)
    functs._C._jit_pass_freeze(m._c)
    assert "GetAttr" not in str(m._c.forward.graph)       # the parameter is a constant of the graph now
    assert "GetAttr" in str(c.forward.graph)              # the clone was taken before
    x = torch.rand(2, 3)
    assert torch.equal(m._c.forward(x), x * 2.0)


def test_metric_entry_points_resolve_from_the_library():
    lib = ctypes.CDLL(functs._C.__file__)
    for name in ("metricsEnabled", "initializeMetrics", "finalizeMetrics", "beginProfilerPass", "endProfilerPass",
                 "allPassesSubmitted", "enableProfiling", "disableProfiling", "printProfilingResults"):
        assert hasattr(lib, name), name
    assert fprof.metrics_enabled() is False
    fprof.initialize_metrics()
    fprof.begin_profiler_pass()
    fprof.end_profiler_pass()
    assert fprof.all_passes_submitted() is True
    fprof.finalize_metrics()
