"""The detection tail as TorchScript operators (functs::nms, functs::batched_nms,
functs::multiclass_nms: functs_amd/csrc/ext/detection_ops.cpp) and the pass that joins a
compacting map functor with a per-image loop of functs::multiclass_nms behind it
(FuseDetectionTail): functor[padded_outputs] -> functs::multiclass_nms_batched ->
functs::unbatch_detections, two launches and one wait.
Reference programs: functs/benchmark/ai_model/yolov3/yolov3_bbox.py:104-179, 233-243,
functs/benchmark/ai_model/ssd/ssd_bbox.py:175-214 (torchvision::nms inside ATen glue).

CPU: schemas, what the pass makes of the programs and what it leaves alone.
GPU: the operators and the scripted programs against the oracle (oracle/nms.py, pinned in
tests/test_nms.py): kept candidates and labels bit-exact, boxes and scores bit-exact on the same
compacted rows."""
from typing import List, Tuple

import pytest
import torch
from torch import Tensor

import functs_amd.aot as aot
import functs_amd.jit as fj
from functs_amd import _C
from functs_amd.benchmark import PROGRAMS
from functs_amd.benchmark.inputs import INPUTS
from functs_amd.benchmark.programs import yolov3_postproc
from oracle import nms as onms


def _kinds(block, out=None):
    out = [] if out is None else out
    for n in block.nodes():
        out.append(n.kind())
        for b in n.blocks():
            _kinds(b, out)
    return out


def _functors(graph):
    return [n for n in graph.nodes() if n.kind() == "tssa::ParallelFunctor"]


# ---- CPU: schemas and the pass --------------------------------------------------------------------
def test_the_operators_are_registered_with_the_reference_signatures():
    schemas = {s.name: str(s) for s in torch._C._jit_get_all_schemas() if s.name.startswith("functs::")}
    # torchvision::nms(Tensor dets, Tensor scores, float iou_threshold) -> Tensor
    assert schemas["functs::nms"] == "functs::nms(Tensor dets, Tensor scores, float iou_threshold) -> Tensor"
    assert schemas["functs::multiclass_nms"].startswith("functs::multiclass_nms(Tensor multi_bboxes, Tensor multi_scores, Tensor score_factors")
    assert "functs::batched_nms" in schemas and "functs::multiclass_nms_batched" in schemas and "functs::unbatch_detections" in schemas


def test_host_tensors_are_refused():
    with pytest.raises(RuntimeError, match="GPU only"):
        torch.ops.functs.nms(torch.zeros(3, 4), torch.zeros(3), 0.5)
    with pytest.raises(RuntimeError, match="GPU only"):
        torch.ops.functs.multiclass_nms(torch.zeros(3, 4), torch.zeros(3, 5), torch.zeros(3))


@pytest.mark.parametrize("name,small", [("c5_nms", dict(grids=[2, 3, 4], batch=3)), ("yolo_head_nms", dict(batch=3, grids=(2, 4, 8)))])
def test_the_tail_of_a_compacting_map_becomes_one_batched_launch(name, small):
    args = INPUTS[name](0, **small)
    fn = fj.build(fj.script(PROGRAMS[name]), list(args))
    kinds = _kinds(fn.graph.block())
    assert "functs::multiclass_nms" not in kinds
    # the loop that appended (dets, labels) per image is gone: the list of pairs comes from one operator
    assert kinds.count("functs::multiclass_nms_batched") == 1 and kinds.count("functs::unbatch_detection_pairs") == 1
    assert "prim::Loop" not in kinds and "aten::append" not in kinds
    fs = _functors(fn.graph)
    last = fs[-1]
    assert last.i("padded_outputs") == 1 and last.i("compact_rows") == 1 and last.i("is_parallel_map") == 1
    outs = list(last.outputs())
    assert len(outs) == 4 and all(o.type().kind() == "TensorType" for o in outs)   # three padded results and the counts
    # the counts go from the functor to the batched tail, nothing else reads them
    batched = [n for n in fn.graph.nodes() if n.kind() == "functs::multiclass_nms_batched"][0]
    assert list(batched.inputs())[3].node() == last and len(outs[3].uses()) == 1


def test_a_loop_that_does_more_with_the_detections_stays():
    def scaled(preds: Tensor, anchors: Tensor, strides: Tensor):
        out: List[Tensor] = []
        for i in range(preds.size(0)):
            b, c, o = yolov3_postproc(preds[i:i + 1], anchors, strides)
            dets, labels = torch.ops.functs.multiclass_nms(b, c, o, 0.05, 0.45, 100, False)
            out.append(dets * 0.5)
        return out

    args = INPUTS["c5_nms"](0, grids=[2, 3, 4], batch=3)
    fn = fj.build(fj.script(scaled), list(args))
    kinds = _kinds(fn.graph.block())
    assert kinds.count("functs::multiclass_nms_batched") == 1 and kinds.count("functs::unbatch_detections") == 1
    assert "functs::multiclass_nms" not in kinds and "prim::Loop" in kinds


def test_lists_that_are_read_elsewhere_keep_their_functor():
    """The map's lists are results of the function as well: they keep their sizes (and their wait),
    the tail stays a loop over the images."""
    def both(preds: Tensor, anchors: Tensor, strides: Tensor):
        out_b: List[Tensor] = []
        dets: List[Tuple[Tensor, Tensor]] = []
        for i in range(preds.size(0)):
            b, c, o = yolov3_postproc(preds[i:i + 1], anchors, strides)
            out_b.append(b)
            dets.append(torch.ops.functs.multiclass_nms(b, c, o, 0.05, 0.45, 100, False))
        return out_b, dets

    args = INPUTS["c5_nms"](0, grids=[2, 3, 4], batch=3)
    fn = fj.build(fj.script(both), list(args))
    kinds = _kinds(fn.graph.block())
    assert "functs::multiclass_nms" in kinds and "functs::multiclass_nms_batched" not in kinds
    assert all(not n.hasAttribute("padded_outputs") for n in _functors(fn.graph))


# ---- GPU ---------------------------------------------------------------------------------------
def _boxes(g, n, span=100.0, size=40.0):
    xy = torch.rand(n, 2, generator=g) * span
    wh = torch.rand(n, 2, generator=g) * size + 1.0
    return torch.cat([xy, xy + wh], 1)


@pytest.mark.gpu
@pytest.mark.parametrize("n", [0, 1, 77, 1000, 3000])
def test_nms_and_batched_nms_against_the_oracle(n):
    g = torch.Generator().manual_seed(n + 5)
    b, s = _boxes(g, n, span=100.0 if n <= 1000 else 25.0), torch.rand(n, generator=g)   # (at most 1024 boxes come back)
    lab = torch.randint(0, 5, (n,), generator=g)
    print("functs::nms n=%d" % n, flush=True)
    keep = torch.ops.functs.nms(b.cuda(), s.cuda(), 0.45)
    dets, kept = torch.ops.functs.batched_nms(b.cuda(), s.cuda(), lab.cuda(), 0.45)
    if n == 0:
        assert keep.numel() == 0 and dets.shape == (0, 5) and kept.numel() == 0
        return
    ref = onms.nms(b, s, 0.45)
    assert keep.cpu().tolist() == ref.tolist()[:1024]
    rd, rk = onms.batched_nms(b, s, lab, 0.45)
    assert kept.cpu().tolist() == rk.tolist()[:1024] and torch.equal(dets.cpu(), rd[:1024])


@pytest.mark.gpu
def test_more_kept_boxes_than_one_launch_returns_is_an_error():
    n = 1500
    x = torch.arange(n, dtype=torch.float32) * 20.0          # no two boxes overlap: all are kept
    b = torch.stack([x, torch.zeros(n), x + 10.0, torch.full((n,), 5.0)], 1)
    with pytest.raises(RuntimeError, match="more than 1024 boxes are kept"):
        torch.ops.functs.nms(b.cuda(), torch.rand(n).cuda(), 0.45)


@pytest.mark.gpu
@pytest.mark.parametrize("padded", [True, False])
def test_multiclass_nms_operator_against_the_oracle(padded):
    g = torch.Generator().manual_seed(3)
    K, C = 900, 7
    b = _boxes(g, K, span=60.0, size=50.0)
    u = torch.rand(K, C, generator=g)
    cls = torch.where(u < 0.2, 0.05 + 0.9 * torch.rand(K, C, generator=g), 0.04 * torch.rand(K, C, generator=g))
    obj = torch.rand(K, generator=g)
    scores = torch.cat([cls, torch.full((K, 1), 0.9)], 1) if padded else cls    # whatever the padding column holds, it is no class
    print("functs::multiclass_nms padded=%s" % padded, flush=True)
    dets, labels = torch.ops.functs.multiclass_nms(b.cuda(), scores.cuda(), obj.cuda(), 0.05, 0.45, 100, padded)
    rd, rl, _ = onms.multiclass_nms(b, cls, obj, 0.05, 0.45, 100)
    assert torch.equal(labels.cpu(), rl) and torch.equal(dets.cpu(), rd)


@pytest.mark.gpu
def test_an_image_with_too_many_candidates_is_an_error_and_the_next_call_works():
    """The reference switches to a per-class pass from 10000 candidates on (yolov3_bbox.py:148-166);
    here one pass serves 16384 and more is refused, loudly."""
    from functs_amd._lib import lib
    g = torch.Generator().manual_seed(1)
    K, C = 300, 80                                  # 24000 (row, class) pairs above the threshold
    b, cls, obj = _boxes(g, K), torch.full((K, C), 0.5), torch.ones(K)
    with pytest.raises(RuntimeError, match="more than 16384 candidates"):
        torch.ops.functs.multiclass_nms(b.cuda(), cls.cuda(), obj.cuda(), 0.05, 0.45, 100, False)
    assert lib.fx_async_error(0) == 0               # raised here, not left for the next operator
    cls[:, 8:] = 0.0
    dets, labels = torch.ops.functs.multiclass_nms(b.cuda(), cls.cuda(), obj.cuda(), 0.05, 0.45, 100, False)
    rd, rl, _ = onms.multiclass_nms(b, cls, obj, 0.05, 0.45, 100)
    assert torch.equal(labels.cpu(), rl) and torch.equal(dets.cpu(), rd)


def _cuda(args):
    def mv(a):
        if isinstance(a, torch.Tensor):
            return a.cuda()
        if isinstance(a, (list, tuple)):
            return type(a)(mv(x) for x in a)
        return a
    return [mv(a) for a in args]


@pytest.mark.gpu
@pytest.mark.parametrize("name,small,head,pad", [
    ("c5_nms", dict(grids=[4, 6, 8], batch=5, shift=3.5), "c5", False),
    ("c5_nms", dict(), "c5", False),
    ("yolo_head_nms", dict(batch=4, grids=(4, 8, 16), shift=5.0), "yolo_head", True),
])
def test_scripted_program_with_its_tail_is_two_launches(name, small, head, pad):
    """Expected values: the oracle's multiclass_nms on the rows that the same program WITHOUT the
    tail returns on the GPU (that program's own parity is tests/test_configs.py's and
    tests/test_reference_programs.py's business; a box that differs in its last bit may flip an
    overlap test)."""
    args = INPUTS[name](0, **small)
    fn = fj.build(fj.script(PROGRAMS[name]), list(args))
    head_fn = fj.build(fj.script(PROGRAMS[head]), list(args))
    gargs = _cuda(args)
    print("scripted %s %s" % (name, small), flush=True)
    got = fn(*gargs)
    torch.cuda.synchronize()
    boxes, cls, obj = head_fn(*gargs)
    n_images = len(boxes)
    assert len(got) == n_images
    assert any(0 < b.size(0) for b in boxes)
    for t in range(n_images):
        c = cls[t].cpu()
        rd, rl, _ = onms.multiclass_nms(boxes[t].cpu(), c[:, :-1] if pad else c, obj[t].cpu(), 0.05, 0.45, 100)
        assert torch.equal(got[t][1].cpu(), rl), "image %d: labels" % t
        assert torch.equal(got[t][0].cpu(), rd), "image %d: dets" % t
    assert sum(d.size(0) for d, _ in got) > 0
    # launches of one call: the compaction (after the head's dense region, if any) and the tail
    n_functors = len(_functors(fn.graph))
    l0, _ = aot.launch_stats()
    fn(*gargs)
    torch.cuda.synchronize()
    l1, _ = aot.launch_stats()
    assert l1 - l0 == n_functors + 1
    assert n_functors == (1 if head == "c5" else 2)
