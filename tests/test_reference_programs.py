"""Programs with the structure of the reference's own model files, in this build's text
(functs_amd/benchmark/programs.py): the whole YOLOv3 detection head up to the NMS (per-level NCHW
maps permuted and flattened, in-place sigmoid on a slice, anchors generated from the feature-map
sizes, boxes decoded with torch.stack, a zero column behind the class scores, a per-image loop
with a confidence mask: yolov3_bbox.py:12-23, 78-101, 194-243), the attention loop over a growing
key / value cache (simpleops/attention/attention.py:38-58) and the SSD box regression with
in-place clamps on strided slices (ssd_bbox.py:121-154).

CPU: what the pipeline makes of them (functors, their kinds).  GPU: results against eager mode
on the CPU (the way the reference tests itself: test/test_basic.py:50-52), launches per call."""
import pytest
import torch

import functs_amd.aot as aot
import functs_amd.jit as fj
from functs_amd.benchmark import PROGRAMS
from functs_amd.benchmark.inputs import INPUTS
from tests.util import assert_boxes_close, assert_close


def _functors(block, out=None):
    out = [] if out is None else out
    for n in block.nodes():
        if n.kind() == "tssa::ParallelFunctor":
            out.append(n)
        for b in n.blocks():
            _functors(b, out)
    return out


def _kinds(block, out=None):
    out = [] if out is None else out
    for n in block.nodes():
        out.append(n.kind())
        for b in n.blocks():
            _kinds(b, out)
    return out


def _cuda(args):
    def mv(a):
        if isinstance(a, torch.Tensor):
            return a.cuda()
        if isinstance(a, (list, tuple)):
            return type(a)(mv(x) for x in a)
        return a
    return [mv(a) for a in args]


# ---- the whole detection head -----------------------------------------------------------------
def test_the_head_is_two_functors_and_the_second_streams_rows():
    args = INPUTS["yolo_head"](0, batch=4, grids=(4, 8, 16))
    fn = fj.build(fj.script(PROGRAMS["yolo_head"]), list(args))
    fs = _functors(fn.graph.block())
    # the level loop is written out (the levels differ in shape), the lists it filled are list
    # constructions, no loop and no list mutation is left
    kinds = _kinds(fn.graph.block())
    assert "prim::Loop" not in kinds and "aten::append" not in kinds
    # permute / reshape / sigmoid_ / cat / decode for the whole batch, then the per-image map
    assert [(n.i("is_parallel_map"), n.i("compact_rows")) for n in fs] == [(0, 0), (1, 1)]
    assert fs[1].i("parallel_degree") == 4
    sub = _kinds(fs[1].g("Subgraph"))
    assert "aten::sigmoid" in sub and "aten::cat" in sub and "aten::zeros" in sub   # objectness, scores and their padding sank into the map
    report = aot.plan(fn)
    assert len(report) == 2 and "row-stream key" in report[1], report


def test_the_dense_part_of_the_head_runs_the_lean_kernel_at_the_benchmark_shape():
    # (level sizes are constants of the lowered program: compiled kernels are linked for the
    # shape the benchmark uses)
    args = INPUTS["yolo_head"](0)
    report = aot.plan(fj.build(fj.script(PROGRAMS["yolo_head"]), list(args)))
    assert len(report) == 2 and "lean dense kernel" in report[0] and "kernel linked" in report[1], report


@pytest.mark.gpu
@pytest.mark.parametrize("batch,grids", [(2, (4, 8, 16)), (16, (13, 26, 52))])
def test_the_head_equals_eager(batch, grids):
    args = INPUTS["yolo_head"](0, batch=batch, grids=grids)
    want_b, want_s, want_o = PROGRAMS["yolo_head"](*args)
    fn = fj.build(fj.script(PROGRAMS["yolo_head"]), _cuda(args))
    total0, _ = aot.launch_stats()
    got_b, got_s, got_o = fn(*_cuda(args))
    torch.cuda.synchronize()
    total1, _ = aot.launch_stats()
    assert total1 - total0 == 2, "launches of the library per call: %d" % (total1 - total0)
    assert len(got_b) == batch
    for t in range(batch):
        assert got_o[t].shape == want_o[t].shape, (t, got_o[t].shape, want_o[t].shape)
        assert_close(got_o[t].cpu(), want_o[t], "objectness image %d" % t)
        assert_close(got_s[t].cpu(), want_s[t], "scores image %d" % t)
        assert_boxes_close(got_b[t].cpu(), want_b[t], "boxes image %d" % t)
        assert got_s[t].shape[1] == 81 and float(got_s[t][:, 80].abs().max()) == 0.0


# ---- attention over a growing cache ---------------------------------------------------------
def test_the_attention_loop_is_functionalized_around_the_library_products():
    args = INPUTS["attention"](0, length=36, start=32)
    fn = fj.build(fj.script(PROGRAMS["attention"]), list(args))
    kinds = _kinds(fn.graph.block())
    assert "aten::copy_" not in kinds and "tssa::update" not in kinds
    assert kinds.count("aten::matmul") == 6          # the products stay ATen's
    loops = [n for n in fn.graph.nodes() if n.kind() == "prim::Loop"]
    assert len(loops) == 1
    inner = _functors(list(loops[0].blocks())[0])
    assert len(inner) == 2                            # cache row writes + transpose; cache row write + scale + softmax
    assert any("aten::softmax" in _kinds(f.g("Subgraph")) for f in inner)


@pytest.mark.gpu
def test_the_attention_loop_equals_eager():
    args = INPUTS["attention"](0)
    want = PROGRAMS["attention"](*args)
    fn = fj.build(fj.script(PROGRAMS["attention"]), list(args))
    got = fn(*_cuda(args))
    torch.cuda.synchronize()
    for name, g, w in zip(("k", "v", "x"), got, want):
        assert g.shape == w.shape
        # 18 dependent steps of products and a softmax: 1e-4 relative to the largest element
        assert float((g.cpu() - w).abs().max()) <= 1e-4 * float(w.abs().max()) + 1e-6, name


# ---- box regression with in-place clamps on strided slices ----------------------------------
def test_delta2bbox_is_one_region():
    args = INPUTS["delta2bbox"](0, n=100, classes=3)
    fn = fj.build(fj.script(PROGRAMS["delta2bbox"]), list(args))
    fs = _functors(fn.graph.block())
    assert len(fs) == 1 and fs[0].i("is_parallel_map") == 0
    sub = _kinds(fs[0].g("Subgraph"))
    assert sub.count("immut::slice_rev") == 2 and sub.count("aten::clamp") == 3 and "aten::tensor" in sub
    assert "aten::clamp_" not in _kinds(fn.graph.block())


@pytest.mark.gpu
@pytest.mark.parametrize("n,classes", [(100, 3), (8732, 4)])
def test_delta2bbox_equals_eager(n, classes):
    args = INPUTS["delta2bbox"](0, n=n, classes=classes)
    want = PROGRAMS["delta2bbox"](*args)
    fn = fj.build(fj.script(PROGRAMS["delta2bbox"]), list(args))
    total0, _ = aot.launch_stats()
    got = fn(*_cuda(args))
    torch.cuda.synchronize()
    total1, _ = aot.launch_stats()
    assert total1 - total0 == 1
    assert got.shape == want.shape
    assert_boxes_close(got.cpu(), want, "delta2bbox")
