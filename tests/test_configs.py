"""Parity of the five benchmark configurations with the oracle (stock
TorchScript on the CPU, oracle/configs.py) on the same seeded inputs.

Reduced shapes run on the emulator and on the GPU; the benchmark configurations' full shapes
run on the GPU only.  Bars: bit-exact for select/slice/assign/compaction
results (c1, kept-row sets and row order everywhere), 1e-5 relative for fp32
elementwise math (sigmoid/exp/softmax/box decode).

Threshold rule: a mask `f(x) >= thr` computed with a transcendental f can only
differ between CPU and GPU for elements within rounding distance of thr.  The
tests assert that the oracle has no element within 1e-6 of the threshold for
the seeds used (oracle.configs.threshold_margin), so the kept-row SETS must be
identical.
"""
import pytest
import torch

from functs_amd import configs
from oracle import configs as oc
from tests.util import assert_boxes_close, assert_close, assert_exact, run_region

SMALL_GRIDS = [2, 3, 4]


def test_c1_reduced(backend):
    a, b, n = oc.c1_inputs(0, 48, 31)
    (got,) = run_region(backend, configs.build_c1(), b, n)
    assert_exact(got, oc.run("c1", a, b, n), "c1")
    # closed form
    ref = b.clone()
    ref[:n] += 1
    assert_exact(got, ref, "c1 closed form")


@pytest.mark.parametrize("n", [0, 1, 48])
def test_c1_trip_counts(backend, n):
    a, b, _ = oc.c1_inputs(1, 48, 0)
    (got,) = run_region(backend, configs.build_c1(), b, n)
    assert_exact(got, oc.run("c1", a, b, n), "c1 n=%d" % n)


def test_c1_trip_count_past_the_dimension_is_an_error():
    """The oracle raises an index error for b[48] on 48 rows; the collapsed loop says so too instead
    of stopping at the last row."""
    from functs_amd._lib import C, FxError
    from tests.support import emul
    a, b, _ = oc.c1_inputs(1, 48, 0)
    with pytest.raises((IndexError, RuntimeError)):   # TorchScript reports the IndexError as a RuntimeError
        oc.run("c1", a, b, 49)
    with pytest.raises(FxError) as e:
        emul.run(configs.build_c1(), b, 49)
    assert e.value.code == C["FX_E_INVALID"] and "outside a dimension" in str(e.value)


def _check_yolo(got, ref, pred, what):
    boxes, cls, obj = got
    rboxes, rcls, robj = ref
    assert_boxes_close(boxes, rboxes, what + " boxes")
    assert_close(cls, rcls, what + " cls")
    assert_close(obj, robj, what + " obj")


def _yolo_margin(pred):
    return oc.threshold_margin(torch.sigmoid(pred[..., 4]), 0.3)


def test_c2_reduced(backend):
    pred, anchors, strides = oc.c2_inputs(0, SMALL_GRIDS)
    assert _yolo_margin(pred) > 1e-6
    ref = oc.run("c2", pred, anchors, strides)
    got = run_region(backend, configs.build_c2(), pred, anchors, strides)
    _check_yolo(got, ref, pred, "c2")
    keep = torch.sigmoid(pred[0, :, 4]) >= 0.3
    assert got[0].shape[0] == int(keep.sum())


def test_c2_zero_logits_closed_form(backend):
    """Zero logits: sigmoid = 0.5, exp = 1 -> box = anchor centre +- anchor half size
    = the anchor itself; every row is kept (0.5 >= 0.3)."""
    _, anchors, strides = oc.c2_inputs(0, SMALL_GRIDS)
    pred = torch.zeros(1, anchors.size(0), 85)
    boxes, cls, obj = run_region(backend, configs.build_c2(), pred, anchors, strides)
    assert_close(boxes, anchors, "boxes == anchors", rtol=1e-6, atol=1e-4)
    assert_exact(cls, torch.full((anchors.size(0), 80), 0.5))
    assert_exact(obj, torch.full((anchors.size(0),), 0.5))


def test_c2_all_rejected(backend):
    _, anchors, strides = oc.c2_inputs(0, SMALL_GRIDS)
    pred = torch.full((1, anchors.size(0), 85), -20.0)
    boxes, cls, obj = run_region(backend, configs.build_c2(), pred, anchors, strides)
    assert boxes.shape == (0, 4) and cls.shape == (0, 80) and obj.shape == (0,)


def test_c5_reduced(backend):
    preds, anchors, strides = oc.c5_inputs(0, SMALL_GRIDS, 3)
    assert _yolo_margin(preds) > 1e-6
    rb, rc, ro = oc.run("c5", preds, anchors, strides)
    gb, gc, go = run_region(backend, configs.build_c5(3), preds, anchors, strides)
    assert_boxes_close(gb, list(rb), "c5 boxes")
    assert_close(gc, list(rc), "c5 cls")
    assert_close(go, list(ro), "c5 obj")


def test_c5_task_permutation(backend):
    """ParallelMap invariant: permuting the tasks permutes the outputs."""
    preds, anchors, strides = oc.c5_inputs(3, SMALL_GRIDS, 4)
    perm = [2, 0, 3, 1]
    r = configs.build_c5(4)
    a = run_region(backend, r, preds, anchors, strides)
    b = run_region(backend, r, preds[perm].contiguous(), anchors, strides)
    for k in range(3):
        for i, p in enumerate(perm):
            assert_exact(b[k][i], a[k][p], "output %d task %d" % (k, i))


def _run_c3(backend, loc, conf, priors):
    boxes, scores = run_region(backend, configs.build_c3_decode(), loc, conf, priors)
    gb, gs = run_region(backend, configs.build_c3_classes(conf.size(2) - 1), boxes, scores)
    return boxes, scores, gb, gs


def test_c3_reduced(backend):
    loc, conf, priors = oc.c3_inputs(0, 60, 7)
    assert oc.threshold_margin(conf[0].softmax(-1)[:, 1:], 0.05) > 1e-6
    rb, rs = oc.run("c3", loc, conf, priors)
    boxes, scores, gb, gs = _run_c3(backend, loc, conf, priors)
    assert torch.allclose(scores.sum(-1), torch.ones(60), atol=1e-6)  # closed form
    assert_close(gb, list(rb), "c3 boxes", rtol=1e-5, atol=1e-6)
    assert_close(gs, list(rs), "c3 scores")


def test_c3_zero_loc_closed_form(backend):
    """Zero loc: cxcy = prior centre, wh = prior size -> boxes = [c - wh/2, c + wh/2]."""
    _, conf, priors = oc.c3_inputs(0, 60, 7)
    loc = torch.zeros(1, 60, 4)
    boxes, _, _, _ = _run_c3(backend, loc, conf, priors)
    ref = torch.cat([priors[:, :2] - priors[:, 2:] / 2, priors[:, :2] + priors[:, 2:] / 2], 1)
    assert_exact(boxes, ref, "c3 zero loc")


# ---------------------------------------------------------------------------
# the benchmark configurations' full shapes (GPU only)
# ---------------------------------------------------------------------------


@pytest.mark.gpu
def test_c1_full():
    a, b, n = oc.c1_inputs(0)
    (got,) = run_region("hip", configs.build_c1(), b, n)
    assert_exact(got, oc.run("c1", a, b, n), "c1 full")


@pytest.mark.gpu
def test_c2_full():
    pred, anchors, strides = oc.c2_inputs(0)
    assert pred.shape == (1, 10647, 85)
    assert _yolo_margin(pred) > 1e-6
    ref = oc.run("c2", pred, anchors, strides)
    got = run_region("hip", configs.build_c2(), pred, anchors, strides)
    _check_yolo(got, ref, pred, "c2 full")


@pytest.mark.gpu
def test_c3_full():
    loc, conf, priors = oc.c3_inputs(0)
    assert conf.shape == (1, 8732, 81)
    assert oc.threshold_margin(conf[0].softmax(-1)[:, 1:], 0.05) > 1e-7
    rb, rs = oc.run("c3", loc, conf, priors)
    boxes, scores, gb, gs = _run_c3("hip", loc, conf, priors)
    assert len(gb) == 80
    assert_close(gb, list(rb), "c3 full boxes", rtol=1e-5, atol=1e-6)
    assert_close(gs, list(rs), "c3 full scores")


@pytest.mark.gpu
def test_c5_full():
    preds, anchors, strides = oc.c5_inputs(0)
    assert preds.shape == (16, 10647, 85)
    assert _yolo_margin(preds) > 1e-6
    rb, rc, ro = oc.run("c5", preds, anchors, strides)
    gb, gc, go = run_region("hip", configs.build_c5(16), preds, anchors, strides)
    assert_boxes_close(gb, list(rb), "c5 full boxes")
    assert_close(gc, list(rc), "c5 full cls")
    assert_close(go, list(ro), "c5 full obj")
    # size-independent property: compaction keeps source order (obj column equals
    # the oracle's gather of the kept rows, already checked) and total count
    keep = torch.sigmoid(preds[..., 4]) >= 0.3
    assert [int(g.shape[0]) for g in go] == keep.sum(1).tolist()
