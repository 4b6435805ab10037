"""The one-pass (streaming) form of a row compaction (opt-in) against the two-pass form and the oracle:
same rows, same order, same values.  The look-back wait is bounded; with a poll limit of zero every
workgroup takes the path that counts the earlier tiles itself, which must give the same result."""
import ctypes

import pytest
import torch

from functs_amd import Region, configs
from functs_amd._lib import lib
from oracle import configs as oc
from tests.util import assert_boxes_close, assert_close, assert_exact, run_region


@pytest.fixture(autouse=True)
def generic_kernels_only():
    """The detection-head regions used here have a kernel of their own (tests/test_head_stream.py);
    these tests are about the generic one-pass form."""
    lib.fx_set_head_kernel(0)
    lib.fx_set_rowstream(0)
    yield
    lib.fx_set_head_kernel(1)
    lib.fx_set_rowstream(1)


def _stream_info(r, *args):
    arr, n, _ = r._flatten(args)
    p = r.plan(arr, n)
    out = (ctypes.c_int64 * 8)()
    lib.fx_plan_stream_info(p.handle, out, 8)
    return list(out), p


def test_window_input_is_found_for_the_detection_head():
    r = configs.build_c5(16)           # the plan lives as long as its region
    info, p = _stream_info(r, *oc.c5_inputs(0))
    ok, tile_rows, tiles, grid, stride, tcoef, lo, span = info
    assert ok == 1 and stride == 85 and tcoef == 10647 * 85 and lo == 0 and span == 85
    assert tile_rows in (64, 128, 256) and tiles == -(-10647 // tile_rows) and grid == 16 * tiles
    assert lib.fx_plan_launches(p.handle) == 2          # two passes unless streaming is switched on
    lib.fx_set_streaming(1)
    try:
        assert lib.fx_plan_launches(p.handle) == 1
    finally:
        lib.fx_set_streaming(0)


def test_no_window_when_rows_are_read_column_by_column():
    """scores[:, c] reads one element of every row: a window would fetch the whole matrix per task."""
    r = Region(parallel_degree=4, is_parallel_map=True)
    scores = r.tensor_input(torch.float32, 2)
    c = r.op("INT_ADD", r.task_index(), 1)
    sc = scores.select(1, c)
    r.output(sc)
    r.compact_rows(sc > 0.5)
    r.finalize()
    info, p = _stream_info(r, torch.rand(300, 9))
    assert info[0] == 0 and lib.fx_plan_launches(p.handle) == 2


@pytest.fixture
def streaming():
    lib.fx_set_streaming(1)
    yield
    lib.fx_set_streaming(0)


def _both_forms(r, *args):
    lib.fx_set_streaming(1)
    try:
        one = run_region("hip", r, *args)
    finally:
        lib.fx_set_streaming(0)
    two = run_region("hip", r, *args)
    return one, two


@pytest.mark.gpu
@pytest.mark.parametrize("compiled", [True, False])
def test_c5_one_pass_equals_two_pass_and_the_oracle(compiled):
    import functs_amd.aot as aot
    preds, anchors, strides = oc.c5_inputs(0)
    r = configs.build_c5(16)
    aot.enable(compiled)
    try:
        one, two = _both_forms(r, preds, anchors, strides)
    finally:
        aot.enable(True)
    assert_exact(one, two, "one pass vs two passes")
    rb, rc, ro = oc.run("c5", preds, anchors, strides)
    assert_boxes_close(one[0], list(rb), "boxes")
    assert_close(one[1], list(rc), "cls")
    assert_close(one[2], list(ro), "obj")


@pytest.mark.gpu
def test_bounded_wait_falls_back_to_counting(streaming):
    preds, anchors, strides = oc.c5_inputs(3, [4, 6, 9], 5)     # 399 rows per task: several tiles, a ragged last one
    r = configs.build_c5(5)
    ref = run_region("hip", r, preds, anchors, strides)
    lib.fx_set_stream_spin_limit(0)
    try:
        got = run_region("hip", r, preds, anchors, strides)
    finally:
        lib.fx_set_stream_spin_limit(4000)
    assert_exact(got, ref, "workgroups that count for themselves")
    rb, rc, ro = oc.run("c5", preds, anchors, strides)
    assert [t.shape[0] for t in got[2]] == [t.shape[0] for t in ro]


@pytest.mark.gpu
def test_calls_in_a_row_with_changing_inputs(streaming):
    """The status words are never cleared: each call must read only the counts of its own epoch."""
    r = configs.build_c2()
    _, anchors, strides = oc.c2_inputs(0)
    dev = torch.device("cuda:0")
    for seed in range(4):
        pred = torch.randn(1, anchors.size(0), 85, generator=torch.Generator().manual_seed(seed))
        if seed == 2:
            pred[..., 4] = -10.0            # nothing kept
        if seed == 3:
            pred[..., 4] = 10.0             # everything kept
        got = r(pred.to(dev), anchors.to(dev), strides.to(dev))
        torch.cuda.synchronize()
        rb, rc, ro = oc.run("c2", pred, anchors, strides)
        assert got[2].shape[0] == ro.shape[0], "seed %d" % seed
        assert_close(got[2].cpu(), ro, "obj seed %d" % seed)
        assert_close(got[1].cpu(), rc, "cls seed %d" % seed)


@pytest.mark.gpu
@pytest.mark.parametrize("n,width,view", [(1, 8, False), (63, 8, False), (64, 5, False), (1000, 7, True), (5000, 33, False)])
def test_windows_of_any_width_and_alignment(streaming, n, width, view):
    """Row-major input of `width` floats per row, possibly starting at an address that is only
    4-byte aligned (a view into a larger tensor): x[mask] bit-exact, mask computed from column 0."""
    g = torch.Generator().manual_seed(n * 131 + width)
    base = torch.rand(n * width + 3, generator=g)
    x = base[1:1 + n * width].view(n, width) if view else base[:n * width].view(n, width).clone()
    r = Region()
    xi = r.tensor_input(torch.float32, 2)
    r.output(xi)
    r.output(xi.select(1, width - 1) * 2.0)
    r.compact_rows(xi.select(1, 0) > 0.5)
    r.finalize()
    info, _ = _stream_info(r, x)
    assert info[0] == 1 and info[4] == width
    dev = torch.device("cuda:0")
    xg = base.to(dev)[1:1 + n * width].view(n, width) if view else x.to(dev)
    got = r(xg)
    torch.cuda.synchronize()
    m = x[:, 0] > 0.5
    assert_exact([t.cpu() for t in got], [x[m], x[m][:, width - 1] * 2.0], "n=%d width=%d" % (n, width))
