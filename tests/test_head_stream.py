"""The hand-written kernel for the decode + score filter of a YOLO-style detection head
(fx_head_stream, yolov3_bbox.py:12-23, 104-130 in the reference): which plans it is chosen for,
and that it gives, bit for bit, what the generic two-pass kernels give (and so the oracle's
result within the tolerance of the build) for any number of rows, images and classes."""
import ctypes

import pytest
import torch

from functs_amd import Region, configs
from functs_amd._lib import lib
from oracle import configs as oc
from tests.util import assert_boxes_close, assert_close, assert_exact, run_region


@pytest.fixture(autouse=True)
def hand_written_kernel_only():
    """These tests are about the hand-written kernel: the generated row-stream kernels, which
    come first where one is linked (tests/test_rowstream.py), are switched off."""
    lib.fx_set_rowstream(0)
    yield
    lib.fx_set_rowstream(1)


def _head(thr=0.3, obj_col=4, half=0.5, batch=None):
    """The region of configs.build_c2 / build_c5 with its constants as parameters."""
    r = Region(parallel_degree=batch, is_parallel_map=True) if batch else Region()
    preds = r.tensor_input(torch.float32, 3)
    anchors = r.tensor_input(torch.float32, 2)
    strides = r.tensor_input(torch.float32, 1)
    if batch:
        i = r.task_index()
        pred = preds.slice(0, i, r.op("INT_ADD", i, 1))
    else:
        pred = preds
    pred1 = pred.slice_rev(pred.slice(2, 0, 2).sigmoid(), 2, 0, 2)
    obj = pred1.select(2, obj_col).sigmoid()
    cls = pred1.slice(2, 5, None).sigmoid()
    p = pred1.select(0, 0)
    xy = (anchors.slice(1, 0, 2) + anchors.slice(1, 2, None)) * 0.5 + (p.slice(1, 0, 2) - 0.5) * strides.unsqueeze(-1)
    wh = (anchors.slice(1, 2, None) - anchors.slice(1, 0, 2)) * half * p.slice(1, 2, 4).exp()
    boxes = r.op("FULL", r.int_list([r.op("SIZE", anchors, 0), 4]), 0.0, dtype=torch.float32)
    boxes = boxes.select_rev(xy.select(1, 0) - wh.select(1, 0), 1, 0)
    boxes = boxes.select_rev(xy.select(1, 1) - wh.select(1, 1), 1, 1)
    boxes = boxes.select_rev(xy.select(1, 0) + wh.select(1, 0), 1, 2)
    boxes = boxes.select_rev(xy.select(1, 1) + wh.select(1, 1), 1, 3)
    obj0 = obj.select(0, 0)
    r.output(boxes)
    r.output(cls.select(0, 0))
    r.output(obj0)
    r.compact_rows(obj0 >= thr)
    return r.finalize()


def _head_folded(thr=0.3, batch=None):
    """The same head after constant propagation has folded anchors that were generated from static
    shapes: box centres [N, 2] and half sizes [N, 2] instead of anchors, strides as [N, 1]."""
    r = Region(parallel_degree=batch, is_parallel_map=True) if batch else Region()
    preds = r.tensor_input(torch.float32, 3)
    strd = r.tensor_input(torch.float32, 2)
    ctr = r.tensor_input(torch.float32, 2)
    half = r.tensor_input(torch.float32, 2)
    if batch:
        i = r.task_index()
        pred = preds.slice(0, i, r.op("INT_ADD", i, 1))
    else:
        pred = preds
    pred1 = pred.slice_rev(pred.slice(2, 0, 2).sigmoid(), 2, 0, 2)
    obj = pred1.select(2, 4).sigmoid()
    cls = pred1.slice(2, 5, None).sigmoid()
    p = pred1.select(0, 0)
    xy = ctr + (p.slice(1, 0, 2) - 0.5) * strd
    wh = half * p.slice(1, 2, 4).exp()
    boxes = r.op("FULL", r.int_list([r.op("SIZE", ctr, 0), 4]), 0.0, dtype=torch.float32)
    boxes = boxes.select_rev(xy.select(1, 0) - wh.select(1, 0), 1, 0)
    boxes = boxes.select_rev(xy.select(1, 1) - wh.select(1, 1), 1, 1)
    boxes = boxes.select_rev(xy.select(1, 0) + wh.select(1, 0), 1, 2)
    boxes = boxes.select_rev(xy.select(1, 1) + wh.select(1, 1), 1, 3)
    obj0 = obj.select(0, 0)
    r.output(boxes)
    r.output(cls.select(0, 0))
    r.output(obj0)
    r.compact_rows(obj0 >= thr)
    return r.finalize()


def _folded(pred, anchors, strides):
    """Arguments of _head_folded from those of _head (the folding is exact: sums and halvings)."""
    return pred, strides.unsqueeze(-1), (anchors[:, :2] + anchors[:, 2:]) * 0.5, (anchors[:, 2:] - anchors[:, :2]) * 0.5


def _inputs(n, classes, batch, seed=0):
    g = torch.Generator().manual_seed(seed)
    pred = torch.randn(batch, n, 5 + classes, generator=g)
    xy = torch.rand(n, 2, generator=g) * 400
    wh = torch.rand(n, 2, generator=g) * 100 + 4
    anchors = torch.cat([xy, xy + wh], 1)
    strides = torch.tensor([8.0, 16.0, 32.0])[torch.randint(0, 3, (n,), generator=g)]
    return pred, anchors, strides


def _info(r, *args):
    arr, n, _ = r._flatten(args)
    p = r.plan(arr, n)
    out = (ctypes.c_int64 * 8)()
    lib.fx_plan_head_info(p.handle, out, 8)
    return list(out), p


def test_the_benchmark_regions_are_recognised():
    for r, args in ((configs.build_c2(), oc.c2_inputs(0)), (configs.build_c5(16), oc.c5_inputs(0))):
        info, p = _info(r, *args)
        assert info[0] == 1 and info[4] == 80 and info[5] == 85 and info[6] == 10647
        assert lib.fx_plan_launches(p.handle) == 1
        lib.fx_set_head_kernel(0)
        try:
            assert lib.fx_plan_launches(p.handle) == 2
        finally:
            lib.fx_set_head_kernel(1)


def test_classes_rows_images_and_threshold_are_parameters():
    for classes, n, batch, thr in ((8, 100, None, 0.3), (4, 1, 3, 0.5), (80, 10647, 2, 0.05), (12, 777, 5, 0.9)):
        info, _ = _info(_head(thr=thr, batch=batch), *_inputs(n, classes, batch or 1))
        assert info[0] == 1 and info[4] == classes and info[6] == n and info[7] == (batch or 1), (classes, n, batch, info)


def test_the_head_with_folded_anchors_is_recognised():
    for classes, n, batch in ((8, 100, None), (80, 10647, 16)):
        info, p = _info(_head_folded(batch=batch), *_folded(*_inputs(n, classes, batch or 1)))
        assert info[0] == 1 and info[1] == 1 and info[4] == classes and info[6] == n and info[7] == (batch or 1)
        assert lib.fx_plan_launches(p.handle) == 1


def test_other_regions_keep_the_generic_kernels():
    # objectness read from another column; another factor in the box size; classes not a multiple of four
    for r, classes in ((_head(obj_col=3), 8), (_head(half=0.25), 8), (_head(), 6)):
        info, p = _info(r, *_inputs(50, classes, 1))
        assert info[0] == 0 and lib.fx_plan_launches(p.handle) == 2
    # a row compaction of another kind
    r = Region()
    x = r.tensor_input(torch.float32, 2)
    r.output(x)
    r.compact_rows(x.select(1, 0) > 0.5)
    r.finalize()
    info, _ = _info(r, torch.rand(40, 8))
    assert info[0] == 0


def _both(r, *args):
    """(head kernel, generic two passes), both on the GPU."""
    one = run_region("hip", r, *args)
    lib.fx_set_head_kernel(0)
    try:
        two = run_region("hip", r, *args)
    finally:
        lib.fx_set_head_kernel(1)
    return one, two


@pytest.mark.gpu
@pytest.mark.parametrize("name", ["c2", "c5"])
def test_benchmark_configurations_bit_exact_and_against_the_oracle(name):
    args = oc.CONFIGS[name][1](0)
    r = configs.build_c2() if name == "c2" else configs.build_c5(16)
    one, two = _both(r, *args)
    assert_exact(one, two, "head kernel vs two passes")
    rb, rc, ro = oc.run(name, *args)
    assert_boxes_close(one[0], rb if name == "c2" else list(rb), "boxes")
    assert_close(one[1], rc if name == "c2" else list(rc), "cls")
    assert_close(one[2], ro if name == "c2" else list(ro), "obj")


@pytest.mark.gpu
@pytest.mark.parametrize("n,classes,batch", [(1, 4, None), (63, 8, None), (64, 8, 3), (65, 80, 2), (399, 80, 5), (1000, 12, 16),
                                              (5000, 160, 2), (2049, 400, 1)])
def test_any_number_of_rows_images_and_classes(n, classes, batch):
    args = _inputs(n, classes, batch or 1, seed=n + classes)
    one, two = _both(_head(batch=batch), *args)
    assert_exact(one, two, "n=%d classes=%d batch=%s" % (n, classes, batch))
    pred = args[0]
    kept = [(torch.sigmoid(pred[t, :, 4]) >= 0.3) for t in range(pred.size(0))]
    objs = one[2] if batch else [one[2]]
    # rows near the threshold may fall on either side of it in float32: the count is bounded, not pinned
    for t, k in enumerate(kept):
        near = int(((torch.sigmoid(pred[t, :, 4]) - 0.3).abs() < 1e-6).sum())
        assert abs(objs[t].shape[0] - int(k.sum())) <= near


@pytest.mark.gpu
@pytest.mark.parametrize("n,classes,batch", [(1, 4, None), (65, 80, 2), (1000, 12, 16), (10647, 80, None), (10647, 80, 16)])
def test_folded_anchors_bit_exact_against_both_other_forms(n, classes, batch):
    args = _inputs(n, classes, batch or 1, seed=n + classes)
    one, two = _both(_head_folded(batch=batch), *_folded(*args))
    assert_exact(one, two, "folded anchors: head kernel vs two passes")
    plain = run_region("hip", _head(batch=batch), *args)
    assert_exact(one, plain, "folded anchors vs anchors")


@pytest.mark.gpu
def test_nothing_kept_and_everything_kept():
    for value in (-20.0, 20.0):
        pred, anchors, strides = _inputs(700, 80, 4)
        pred[..., 4] = value
        one, two = _both(_head(batch=4), pred, anchors, strides)
        assert_exact(one, two, "objectness %g" % value)
        assert [t.shape[0] for t in one[2]] == [0 if value < 0 else 700] * 4


@pytest.mark.gpu
def test_bounded_wait_falls_back_to_counting():
    args = _inputs(3000, 80, 6, seed=5)
    r = _head(batch=6)
    ref = run_region("hip", r, *args)
    lib.fx_set_stream_spin_limit(0)
    try:
        got = run_region("hip", r, *args)
    finally:
        lib.fx_set_stream_spin_limit(4000)
    assert_exact(got, ref, "workgroups that count for themselves")


@pytest.mark.gpu
def test_calls_in_a_row_with_changing_inputs():
    """The status words are never cleared: each call must read only the counts of its own epoch."""
    r = _head(batch=3)
    dev = torch.device("cuda:0")
    for seed in range(5):
        pred, anchors, strides = _inputs(1500, 80, 3, seed=seed)
        if seed == 2:
            pred[..., 4] = -10.0
        got = r(pred.to(dev), anchors.to(dev), strides.to(dev))
        torch.cuda.synchronize()
        for t in range(3):
            keep = torch.sigmoid(pred[t, :, 4]) >= 0.3
            assert_close(got[2][t].cpu(), torch.sigmoid(pred[t, keep, 4]), "obj seed %d image %d" % (seed, t))
            assert_close(got[1][t].cpu(), torch.sigmoid(pred[t, keep, 5:]), "cls seed %d image %d" % (seed, t))


@pytest.mark.gpu
def test_predictions_that_start_at_an_odd_address():
    """A view into a larger tensor: rows that are only 4-byte aligned."""
    n, classes = 500, 80
    pred, anchors, strides = _inputs(n, classes, 1, seed=9)
    dev = torch.device("cuda:0")
    base = torch.zeros(pred.numel() + 7, device=dev)
    base[3:3 + pred.numel()] = pred.flatten().to(dev)
    view = base[3:3 + pred.numel()].view(1, n, 5 + classes)
    r = _head()
    got = r(view, anchors.to(dev), strides.to(dev))
    ref = r(pred.to(dev), anchors.to(dev), strides.to(dev))
    torch.cuda.synchronize()
    assert_exact([t.cpu() for t in got], [t.cpu() for t in ref], "odd start")


@pytest.mark.gpu
@pytest.mark.parametrize("n,classes,batch", [(100000, 4, None), (300000, 4, None), (60000, 8, 16)])
def test_long_images_and_launches_beyond_what_the_device_holds_at_once(n, classes, batch):
    """More than 128 chunks per image (the look-back polls the later words one round at a time) and
    more workgroups than are resident together (later workgroups wait only for earlier ones)."""
    args = _inputs(n, classes, batch or 1, seed=3)
    one, two = _both(_head(batch=batch), *args)
    assert_exact(one, two, "n=%d classes=%d batch=%s" % (n, classes, batch))


@pytest.mark.gpu
def test_replays_of_a_captured_call():
    """A call recorded into a HIP graph takes the two-pass form (the one-launch form's epoch would
    be frozen in the recorded arguments); every replay must follow its inputs."""
    dev = torch.device("cuda:0")
    n, classes, batch = 700, 80, 2
    r = _head(batch=batch)
    pred, anchors, strides = [t.to(dev) for t in _inputs(n, classes, batch, seed=0)]
    bc = r.bind(pred, anchors, strides)
    bc.launch()                       # descriptor upload and allocations happen here, not under capture
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        bc.launch()
    for seed in (1, 2, 3):
        new = _inputs(n, classes, batch, seed=seed)[0]
        if seed == 2:
            new[0, :, 4] = -20.0      # nothing kept in image 0
        pred.copy_(new.to(dev))
        ref = r(pred.clone(), anchors, strides)      # eager work between the replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        got = bc.results()
        assert_exact([[t.cpu() for t in row] for row in got], [[t.cpu() for t in row] for row in ref], "replay %d" % seed)
