"""The hand-written kernel for the decode + per-class score filter of an SSD-style detection head
(fx_classmap_head; ssd_bbox.py:163-214 in the reference): which plans it is chosen for, and that
it gives, bit for bit, what the generic kernels give for the same computation split in a dense
region (decode + softmax) and a class map over its results, and so the oracle's result within the
tolerance of the build, for any number of priors and classes."""
import ctypes

import pytest
import torch

from functs_amd import Region, configs
from functs_amd._lib import lib
from oracle import configs as oc
from tests.util import assert_close, assert_exact, run_region


def _info(r, *args):
    arr, n, _ = r._flatten(args)
    p = r.plan(arr, n)
    out = (ctypes.c_int64 * 8)()
    lib.fx_plan_head_info(p.handle, out, 8)
    return list(out), p


def _inputs(n, n_cls, seed=0, spread=3.0):
    g = torch.Generator().manual_seed(seed)
    loc = torch.randn(1, n, 4, generator=g)
    conf = torch.randn(1, n, n_cls, generator=g) * spread
    cxcy = torch.rand(n, 2, generator=g)
    wh = torch.rand(n, 2, generator=g) * 0.5 + 0.05
    return loc, conf, torch.cat([cxcy, wh], 1)


def _split(loc, conf, priors, thr=0.05, first=1, n_fg=None):
    """The same computation as two regions through the generic kernels."""
    boxes, scores = run_region("hip", configs.build_c3_decode(), loc, conf, priors)
    n_fg = conf.size(2) - first if n_fg is None else n_fg
    r = Region(parallel_degree=n_fg, is_parallel_map=True)
    b = r.tensor_input(torch.float32, 2)
    s = r.tensor_input(torch.float32, 2)
    sc = s.select(1, r.op("INT_ADD", r.task_index(), first))
    r.output(b)
    r.output(sc)
    r.compact_rows(sc > thr)
    r.finalize()
    return run_region("hip", r, boxes, scores)


def test_the_fused_benchmark_region_is_recognised():
    info, p = _info(configs.build_c3_fused(), *oc.c3_inputs(0))
    assert info[0] == 2 and info[1] == 1 and info[4:] == [80, 81, 8732, 1]
    assert lib.fx_plan_launches(p.handle) == 1
    lib.fx_set_head_kernel(0)
    try:
        assert lib.fx_plan_launches(p.handle) == 2
    finally:
        lib.fx_set_head_kernel(1)


def test_priors_classes_first_class_threshold_and_variances_are_parameters():
    for n, n_cls, n_fg, first, thr, vxy, vwh in ((60, 7, 6, 1, 0.05, 0.1, 0.2), (1, 2, 1, 1, 0.5, 0.1, 0.2),
                                                 (500, 128, 128, 0, 0.01, 0.3, 0.4), (333, 21, 10, 5, 0.2, 1.0, 1.0)):
        info, _ = _info(configs.build_c3_fused(n_fg, thr, vxy, vwh, first), *_inputs(n, n_cls))
        assert info[0] == 2 and info[4:] == [n_fg, n_cls, n, first], (n, n_cls, info)


def test_other_regions_keep_the_generic_kernels():
    # more classes than a half-wave holds; tasks beyond the last class are refused by the lowering itself
    info, p = _info(configs.build_c3_fused(n_fg=129, first=0), *_inputs(40, 129))
    assert info[0] == 0 and lib.fx_plan_launches(p.handle) == 2

    def variant(edit):
        r = Region(parallel_degree=6, is_parallel_map=True)
        loc = r.tensor_input(torch.float32, 3)
        conf = r.tensor_input(torch.float32, 3)
        priors = r.tensor_input(torch.float32, 2)
        l0 = loc.select(0, 0)
        cxcy = priors.slice(1, 0, 2) + l0.slice(1, 0, 2) * 0.1 * priors.slice(1, 2, None)
        wh = priors.slice(1, 2, None) * (l0.slice(1, 2, None) * 0.2).exp()
        if edit == "third":
            half = wh / 3
        else:
            half = wh / 2
        boxes = r.op("FULL", r.int_list([r.op("SIZE", priors, 0), 4]), 0.0, dtype=torch.float32)
        boxes = boxes.slice_rev(cxcy - half, 1, 0, 2)
        boxes = boxes.slice_rev(cxcy + half, 1, 2, None)
        c0 = conf.select(0, 0)
        scores = c0.sigmoid() if edit == "sigmoid" else c0.softmax(-1)
        sc = scores.select(1, r.op("INT_ADD", r.task_index(), 1))
        r.output(boxes)
        r.output(sc)
        r.compact_rows((sc >= 0.05) if edit == "ge" else (sc > 0.05))
        return r.finalize()

    for edit in ("third", "sigmoid", "ge"):
        info, p = _info(variant(edit), *_inputs(40, 7))
        assert info[0] == 0 and lib.fx_plan_launches(p.handle) == 2, edit
    info, _ = _info(variant("none"), *_inputs(40, 7))
    assert info[0] == 2


@pytest.mark.gpu
def test_c3_bit_exact_against_the_split_regions_and_close_to_the_oracle():
    args = oc.c3_inputs(0)
    got = run_region("hip", configs.build_c3_fused(), *args)
    ref = _split(*args)
    assert_exact(got, ref, "one launch vs decode region + class map")
    rb, rs = oc.run("c3", *args)
    assert_close(got[0], list(rb), "c3 boxes", rtol=1e-5, atol=1e-6)
    assert_close(got[1], list(rs), "c3 scores")


@pytest.mark.gpu
@pytest.mark.parametrize("n,n_cls,first,thr", [(1, 2, 1, 0.3), (31, 5, 1, 0.1), (32, 9, 0, 0.05), (33, 81, 1, 0.01),
                                               (64, 128, 0, 0.004), (1000, 21, 1, 0.05), (8732, 81, 1, 0.01),
                                               (20000, 4, 1, 0.2), (3001, 100, 37, 0.02)])
def test_any_number_of_priors_and_classes(n, n_cls, first, thr):
    args = _inputs(n, n_cls, seed=n + n_cls)
    got = run_region("hip", configs.build_c3_fused(n_cls - first, thr, 0.1, 0.2, first), *args)
    ref = _split(*args, thr=thr, first=first)
    assert_exact(got, ref, "n=%d classes=%d first=%d" % (n, n_cls, first))
    scores = torch.softmax(args[1][0].double(), -1)
    for t in range(n_cls - first):
        col = scores[:, first + t]
        near = int(((col - thr).abs() < 1e-6).sum())
        assert abs(got[1][t].shape[0] - int((col > thr).sum())) <= near


@pytest.mark.gpu
def test_nothing_kept_and_everything_kept():
    loc, conf, priors = _inputs(700, 8, seed=1)
    for thr, want in ((2.0, 0), (-1.0, 700)):
        got = run_region("hip", configs.build_c3_fused(7, thr), loc, conf, priors)
        ref = _split(loc, conf, priors, thr=thr)
        assert_exact(got, ref, "threshold %g" % thr)
        assert [t.shape[0] for t in got[1]] == [want] * 7


@pytest.mark.gpu
def test_bounded_wait_falls_back_to_computing_the_earlier_chunks():
    args = _inputs(2000, 40, seed=5)
    r = configs.build_c3_fused(39)
    ref = run_region("hip", r, *args)
    lib.fx_set_stream_spin_limit(0)
    try:
        got = run_region("hip", r, *args)
    finally:
        lib.fx_set_stream_spin_limit(4000)
    assert_exact(got, ref, "workgroups that compute the earlier chunks themselves")


@pytest.mark.gpu
def test_calls_in_a_row_with_changing_inputs():
    """The status words are never cleared: each call must read only the counts of its own epoch."""
    r = configs.build_c3_fused(20)
    for seed in range(6):
        loc, conf, priors = _inputs(1500, 21, seed=seed)
        if seed == 2:
            conf[..., 1:] = -30.0          # nothing but background
        got = run_region("hip", r, loc, conf, priors)
        ref = _split(loc, conf, priors)
        assert_exact(got, ref, "seed %d" % seed)


@pytest.mark.gpu
def test_the_generic_kernels_on_the_fused_region_agree_within_the_tolerance():
    """Without the kernel the fused region still runs (every task redoes the softmax, with a
    serial sum): same rows, values within 1e-6 relative."""
    args = _inputs(900, 12, seed=4)
    r = configs.build_c3_fused(11)
    one = run_region("hip", r, *args)
    lib.fx_set_head_kernel(0)
    try:
        two = run_region("hip", r, *args)
    finally:
        lib.fx_set_head_kernel(1)
    assert_close(one[0], two[0], "boxes", rtol=1e-6)
    assert_close(one[1], two[1], "scores", rtol=1e-6)


@pytest.mark.gpu
def test_scores_that_start_at_an_odd_address():
    n, n_cls = 500, 81
    loc, conf, priors = _inputs(n, n_cls, seed=9)
    dev = torch.device("cuda:0")
    base = torch.zeros(conf.numel() + 7, device=dev)
    base[3:3 + conf.numel()] = conf.flatten().to(dev)
    view = base[3:3 + conf.numel()].view(1, n, n_cls)
    r = configs.build_c3_fused(80)
    got = r(loc.to(dev), view, priors.to(dev))
    ref = r(loc.to(dev), conf.to(dev), priors.to(dev))
    torch.cuda.synchronize()
    assert_exact([[t.cpu() for t in o] for o in got], [[t.cpu() for t in o] for o in ref], "odd start")


@pytest.mark.gpu
def test_the_epoch_of_the_status_words_wraps():
    """The tag of a status word has 16 bits: after 65 534 calls on a stream the library clears the
    words (in stream order) and starts the epochs over.  Calls on either side of the wrap must see
    only their own counts."""
    dev = torch.device("cuda:0")
    loc, conf, priors = [t.to(dev) for t in _inputs(200, 9, seed=2)]
    r = configs.build_c3_fused(8)
    bc = r.bind(loc, conf, priors)
    bc.launch()
    torch.cuda.synchronize()
    ref = [[t.clone() for t in o] for o in bc.results()]
    for i in range(66000):
        bc.launch()
        if i % 256 == 0:
            torch.cuda.synchronize()      # (the pinned count words of a call must not be reused while it is in flight)
        if i % 8192 == 0 or i > 65500 and i % 64 == 0:
            torch.cuda.synchronize()
            got = bc.results()
            assert_exact([[t.cpu() for t in o] for o in got], [[t.cpu() for t in o] for o in ref], "call %d" % i)
    # other inputs right after the wrap
    loc2, conf2, priors2 = _inputs(200, 9, seed=3)
    got = run_region("hip", r, loc2, conf2, priors2)
    assert_exact(got, _split(loc2, conf2, priors2), "new inputs after the wrap")
