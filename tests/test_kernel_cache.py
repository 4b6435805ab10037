"""Kernels compiled at run time.

The reference generates and compiles code for every subgraph when the operator is made
(fait/fuser/graph_builder.cpp:259-712, fait/tensorexpr/cuda_codegen_tssa.cpp:1319-1414).  Here
kernels are generated ahead of time and linked into the library; for a region without linked
kernels ``functs_amd.aot.compile_missing`` / ``functs_amd.jit.build(..., compile_kernels=True)``
does the reference's thing: it generates the region's unit, compiles it with hipcc into a shared
object of its own in the kernel cache and loads it, and later processes load it from there."""
import os
import subprocess
import sys

import pytest
import torch

import functs_amd.aot as aot
from functs_amd import configs
from functs_amd._lib import lib
from tests.util import assert_exact

needs_hipcc = pytest.mark.skipif(aot.hipcc_path() is None, reason="no hipcc on this machine")
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _unlinked_region(batch=3, obj_col=2):
    # a spelling of the detection head that no linked kernel serves: corners by cat, objectness in
    # column 2 (column 1 for the GPU test, whose object stays in the package's cache)
    return configs.build_head_variant(batch=batch, decode="cat", obj_col=obj_col)


def _args(batch=3, n=700, seed=0):
    g = torch.Generator().manual_seed(seed)
    pred = torch.randn(batch, n, 85, generator=g)
    anchors = torch.rand(n, 4, generator=g) * 100
    strides = torch.full((n,), 8.0)
    return pred, anchors, strides


@needs_hipcc
def test_a_region_without_linked_kernels_gets_its_own(tmp_path, monkeypatch):
    monkeypatch.setenv("FUNCTS_AMD_KERNEL_CACHE", str(tmp_path))
    r = _unlinked_region()
    args = _args()
    info = r.rowstream_info(*args)
    if info["active"]:
        pytest.skip("a kernel for this region is loaded already (an earlier test of this process compiled it)")
    assert info["ok"]
    n0 = lib.fx_rowstream_count()
    names = aot.compile_missing(planner=lambda: aot._plan_region(r, *args))
    assert names == ["fx_rs_%016x" % info["key"]]
    assert lib.fx_rowstream_count() == n0 + 1
    assert r.rowstream_info(*args)["active"]
    assert os.path.isfile(os.path.join(aot.kernel_cache_dir(), names[0] + ".so"))
    # nothing left to do the second time
    assert aot.compile_missing(planner=lambda: aot._plan_region(r, *args)) == []
    # a process that starts later finds the kernel in the cache
    code = ("import torch, functs_amd\n"
            "from functs_amd import configs\n"
            "r = configs.build_head_variant(batch=3, decode='cat', obj_col=2)\n"
            "i = r.rowstream_info(torch.rand(3, 700, 85), torch.rand(700, 4), torch.rand(700))\n"
            "print('active' if i['active'] else 'not active')\n")
    env = dict(os.environ, PYTHONPATH=ROOT + os.pathsep + os.environ.get("PYTHONPATH", ""))
    out = subprocess.run([sys.executable, "-c", code], env=env, stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=300)
    assert out.returncode == 0, out.stderr[-2000:]
    assert out.stdout.strip().splitlines()[-1] == "active"


def test_the_cache_is_per_state_of_the_headers():
    d = aot.kernel_cache_dir()
    assert os.path.basename(d) == aot._abi_tag() and len(aot._abi_tag()) == 16


@pytest.mark.gpu
@needs_hipcc
def test_a_kernel_compiled_at_run_time_gives_the_two_passes_rows():
    """(compiled into the package's cache, functs_amd/lib/jit, unless an earlier run left it there)"""
    r = _unlinked_region(batch=5, obj_col=1)
    args = _args(batch=5, n=3000, seed=4)
    aot.compile_missing(planner=lambda: aot._plan_region(r, *args))
    assert r.rowstream_info(*args)["active"]
    dev = torch.device("cuda:0")
    dargs = [a.to(dev) for a in args]
    arr, n, _ = r._flatten(dargs)
    assert lib.fx_plan_launches(r.plan(arr, n).handle) == 1
    one = [[t.cpu() for t in o] for o in r(*dargs)]
    torch.cuda.synchronize()
    lib.fx_set_rowstream(0)
    try:
        two = [[t.cpu() for t in o] for o in r(*dargs)]
        torch.cuda.synchronize()
    finally:
        lib.fx_set_rowstream(1)
    assert_exact(one, two, "kernel compiled at run time vs two passes")
    kept = [int((torch.sigmoid(args[0][t, :, 1]) >= 0.3).sum()) for t in range(5)]
    assert [o.shape[0] for o in one[0]] == kept


def _scripted_variant(pred: torch.Tensor, anchors: torch.Tensor, strides: torch.Tensor):
    """The benchmark's post-processing with the rows kept on the product of objectness and the
    first class score, and the boxes scaled by the stride: a program no linked kernel serves."""
    pred = pred.clone()
    pred[..., :2].sigmoid_()
    obj = pred[..., 4].sigmoid()
    cls = pred[..., 5:].sigmoid()
    p = pred[0]
    xy = (anchors[:, :2] + anchors[:, 2:]) * 0.5 + (p[:, :2] - 0.5) * strides.unsqueeze(-1)
    wh = (anchors[:, 2:] - anchors[:, :2]) * 0.5 * p[:, 2:4].exp()
    boxes = torch.cat([xy - wh, xy + wh], 1) / strides.unsqueeze(-1)
    keep = obj[0] * cls[0][:, 0] >= 0.2
    return boxes[keep], cls[0][keep], obj[0][keep]


@needs_hipcc
def test_build_with_compile_kernels_links_the_row_stream_kernel_of_a_new_program(tmp_path, monkeypatch):
    import functs_amd.jit as fj
    monkeypatch.setenv("FUNCTS_AMD_KERNEL_CACHE", str(tmp_path))
    pred, anchors, strides = _args(batch=1, n=900, seed=2)
    fn = fj.build(fj.script(_scripted_variant), [pred, anchors, strides])
    before = aot.plan(fn)
    assert len(before) == 1 and "row-stream key" in before[0], before
    if "(kernel linked)" in before[0]:
        pytest.skip("a kernel for this program is loaded already")
    fn = fj.build(fj.script(_scripted_variant), [pred, anchors, strides], compile_kernels=True)
    after = aot.plan(fn)
    assert "(kernel linked)" in after[0], after
    assert len([f for f in os.listdir(aot.kernel_cache_dir()) if f.endswith(".so")]) == 1


@needs_hipcc
def test_the_environment_switches_it_on_for_code_that_builds_the_reference_way(tmp_path, monkeypatch):
    import functs_amd.jit as fj
    monkeypatch.setenv("FUNCTS_AMD_KERNEL_CACHE", str(tmp_path))
    pred, anchors, strides = _args(batch=1, n=640, seed=3)

    def other(pred: torch.Tensor, anchors: torch.Tensor, strides: torch.Tensor):
        obj = pred[0][:, 4].sigmoid()
        keep = obj * 2.0 >= 1.1
        return (pred[0].tanh() * strides.unsqueeze(-1))[keep], (anchors[:, 0] + obj)[keep]

    monkeypatch.setenv("FUNCTS_AMD_COMPILE_KERNELS", "0")
    first = aot.plan(fj.build(fj.script(other), [pred, anchors, strides]))
    if len(first) != 1 or "row-stream key" not in first[0] or "(kernel linked)" in first[0]:
        pytest.skip("not a program for this test: %r" % (first,))
    monkeypatch.setenv("FUNCTS_AMD_COMPILE_KERNELS", "1")
    assert "(kernel linked)" in aot.plan(fj.build(fj.script(other), [pred, anchors, strides]))[0]


@pytest.mark.gpu
@needs_hipcc
def test_a_program_built_with_compile_kernels_equals_eager():
    import functs_amd.jit as fj
    from functs_amd import aot as _aot
    from tests.util import assert_close, assert_boxes_close
    dev = torch.device("cuda:0")
    pred, anchors, strides = _args(batch=1, n=5000, seed=6)
    want = _scripted_variant(pred, anchors, strides)
    dargs = [pred.to(dev), anchors.to(dev), strides.to(dev)]
    fn = fj.build(fj.script(_scripted_variant), dargs, compile_kernels=True)
    assert "(kernel linked)" in _aot.plan(fn)[0]
    l0, _ = _aot.launch_stats()
    got = fn(*dargs)
    torch.cuda.synchronize()
    l1, _ = _aot.launch_stats()
    assert l1 - l0 == 1, "launches per call: %d" % (l1 - l0)
    assert got[2].shape == want[2].shape
    assert_close(got[2].cpu(), want[2], "objectness")
    assert_close(got[1].cpu(), want[1], "class scores")
    assert_boxes_close(got[0].cpu(), want[0], "boxes")


@needs_hipcc
def test_a_dense_region_with_a_short_program_gets_compiled_kernels_too(tmp_path, monkeypatch):
    import functs_amd.jit as fj
    monkeypatch.setenv("FUNCTS_AMD_KERNEL_CACHE", str(tmp_path))

    def short(x: torch.Tensor, y: torch.Tensor):
        z = x.clone()
        z[:, 1:3] = (y[:, 1:3] * 1.5 - x[:, 1:3]).tanh()
        return z.relu() + y

    ex = [torch.rand(300, 40), torch.rand(300, 40)]
    first = aot.plan(fj.build(fj.script(short), ex))
    if len(first) != 1 or "interpreted" not in first[0]:
        pytest.skip("not a program for this test: %r" % (first,))
    after = aot.plan(fj.build(fj.script(short), ex, compile_kernels=True))
    assert "compiled" in after[0], after


@pytest.mark.gpu
@needs_hipcc
def test_a_dense_program_built_with_compile_kernels_equals_eager_and_the_interpreter():
    import functs_amd.jit as fj
    dev = torch.device("cuda:0")

    def short(x: torch.Tensor, y: torch.Tensor):
        z = x.clone()
        z[:, 2:5] = (y[:, 2:5] * 0.75 - x[:, 2:5]).tanh()
        return z.relu() + y

    torch.manual_seed(8)
    ex = [torch.randn(1000, 33), torch.randn(1000, 33)]
    want = short(*ex)
    dex = [t.to(dev) for t in ex]
    interpreted = fj.build(fj.script(short), dex, compile_kernels=False)(*dex).cpu()
    fn = fj.build(fj.script(short), dex, compile_kernels=True)
    assert "compiled" in aot.plan(fn)[0], aot.plan(fn)
    got = fn(*dex).cpu()
    assert torch.equal(got, interpreted)
    torch.testing.assert_close(got, want, rtol=1e-5, atol=1e-6)
