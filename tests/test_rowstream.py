"""Generated row-stream kernels (fx_plan_rowstream_source, fx_rowstream.h): a row compaction over
a row-major matrix as ONE launch of a kernel written from the region's own lowered programs.

Where the reference generates CUDA for every subgraph (fait/tensorexpr/cuda_codegen_tssa.cpp:
881-1121) and leaves x[mask] to ATen (convert_to_tensorssa.cpp:422-443).  The programs tested are
the detection head in the spellings of functs_amd.configs.HEAD_VARIANTS: the reference's own
(torch.stack of the four corners, a zero column behind the class scores: yolov3_bbox.py:12-23,
227-228), cat of the corner pairs, objectness in another column, another constant, a filter on a
class score, one joined matrix per image.

CPU: the generator's output is compiled as plain C++ (tests/support/fx_rs_host.cpp) and must equal
the bytecode emulator bit for bit.  GPU: the linked kernels must equal the generic two passes bit
for bit, and the oracle within the tolerance of the build.
"""
import ctypes

import pytest
import torch

from functs_amd import Region, configs
from functs_amd._lib import lib
from oracle import configs as oc
from tests.support import emul
from tests.util import assert_boxes_close, assert_close, assert_exact, run_region

VARIANTS = sorted(configs.HEAD_VARIANTS)


def _inputs(n, classes, batch, seed=0):
    g = torch.Generator().manual_seed(seed)
    pred = torch.randn(batch, n, 5 + classes, generator=g)
    xy = torch.rand(n, 2, generator=g) * 400
    wh = torch.rand(n, 2, generator=g) * 100 + 4
    anchors = torch.cat([xy, xy + wh], 1)
    strides = torch.tensor([8.0, 16.0, 32.0])[torch.randint(0, 3, (n,), generator=g)]
    return pred, anchors, strides


def _flat(outs):
    return [t for o in outs for t in (o if isinstance(o, list) else [o])]


def _eager(name, pred, anchors, strides, thr=0.3):
    """The variant in plain torch (float32 on the CPU): per image the list of outputs."""
    kw = dict(decode="assign", pad=False, obj_col=4, half=0.5, mask_class=None, joined=False)
    kw.update(configs.HEAD_VARIANTS.get(name, {}))
    res = []
    for p in pred:
        box_cols = [c for c in range(5) if c != kw["obj_col"]]
        pxy = torch.sigmoid(p[:, box_cols[:2]])
        pwh = p[:, box_cols[2:]]
        obj = torch.sigmoid(p[:, kw["obj_col"]])
        cls = torch.sigmoid(p[:, 5:])
        xy = (anchors[:, :2] + anchors[:, 2:]) * 0.5 + (pxy - 0.5) * strides.unsqueeze(-1)
        wh = (anchors[:, 2:] - anchors[:, :2]) * kw["half"] * pwh.exp()
        boxes = torch.cat([xy - wh, xy + wh], 1)
        if kw["pad"]:
            cls = torch.cat([cls, torch.zeros(cls.size(0), 1)], 1)
        keep = (cls[:, kw["mask_class"]] if kw["mask_class"] is not None else obj) >= thr
        if kw["joined"]:
            res.append([torch.cat([boxes, obj.unsqueeze(-1), cls], 1)[keep]])
        else:
            res.append([boxes[keep], cls[keep], obj[keep]])
    return res


def _build(name, batch):
    if name == "benchmark":
        return configs.build_c5(batch) if batch else configs.build_c2()
    return configs.build_head_variant(batch=batch, **configs.HEAD_VARIANTS[name])


# ---- host logic (no GPU) ------------------------------------------------------------------
@pytest.mark.parametrize("name", VARIANTS + ["benchmark"])
def test_generated_code_equals_the_emulator(name):
    for batch, n, chunk, sub, threads in ((None, 150, 70, 9, 5), (3, 333, 256, 64, 64), (2, 64, 64, 1, 1)):
        r = _build(name, batch)
        args = _inputs(n, 80, batch or 1, seed=n)
        info = r.rowstream_info(*args)
        assert info["ok"] and info["row_elements"] == 85 and info["rows"] == n and info["tasks"] == (batch or 1), info
        ref = _flat(emul.run(r, *args))
        got = _flat(emul.run_rowstream(r, *args, chunk_rows=chunk, sub_rows=sub, threads=threads))
        assert_exact(got, ref, "%s batch %s" % (name, batch))


def test_one_kernel_serves_rows_tasks_offsets_and_constant_values():
    base = configs.build_head_variant().rowstream_info(*_inputs(50, 80, 1))
    assert base["ok"]
    same = [configs.build_head_variant(batch=7).rowstream_info(*_inputs(999, 80, 7)),          # rows, tasks, per-task offsets
            configs.build_head_variant(thr=0.05).rowstream_info(*_inputs(50, 80, 1)),          # the threshold
            configs.build_head_variant(thr=0.7, half=0.5).rowstream_info(*_inputs(50, 80, 1))]
    assert all(s["ok"] and s["key"] == base["key"] for s in same), (base, same)
    # a threshold that equals another constant of the program (0.5) makes two constants one: a kernel of its own
    assert configs.build_head_variant(thr=0.5).rowstream_info(*_inputs(50, 80, 1))["key"] != base["key"]
    # 0.5 appears in the centre and in the half size: changed in one place only, equal constants
    # are no longer equal, and that is another kernel; so is another number of classes
    other = [configs.build_head_variant(half=0.25).rowstream_info(*_inputs(50, 80, 1)),
             configs.build_head_variant().rowstream_info(*_inputs(50, 20, 1)),
             configs.build_head_variant(decode="stack").rowstream_info(*_inputs(50, 80, 1))]
    assert all(s["ok"] and s["key"] != base["key"] for s in other)
    assert len({s["key"] for s in other}) == 3


def test_the_generated_row_code_shares_what_the_columns_share():
    """The four corners of a box need two exp and two sigmoid (plus the objectness): the generic
    lowering evaluates every column on its own (eight of each)."""
    for decode in ("assign", "stack", "cat"):
        r = configs.build_head_variant(decode=decode)
        src = r.rowstream_source(*_inputs(50, 80, 1))
        row = src[src.index("static FX_RS_FN void row("):src.index("using Vecs")]
        assert row.count("rs_EXP(") == 2 and row.count("rs_SIGMOID(") == 3, (decode, row)
        # what the row reads besides the window is loaded by a part of its own (it leaves ahead of
        # the next sub-tile's requests): the anchor's four corners as one 128-bit load, the stride
        side = src[src.index("static FX_RS_FN void row_side("):src.index("static FX_RS_FN void row(")]
        assert side.count("rs_ld4(") == 1 and side.count("rs_ld<") == 1 and "rs_ld" not in row
        assert "rs_SEL" not in row and "rs_INR" not in row   # every column predicate decided by the generator


def test_regions_without_a_row_stream_form_say_why():
    # reductions (the SSD head's softmax)
    r = configs.build_c3_fused(6)
    info = r.rowstream_info(*oc.c3_inputs(0, 40, 7))
    assert not info["ok"] and "reduction" in info["why"]
    # a class map that reads one column of the scores per task: the scores are not streamed (every
    # task would pull whole rows through LDS for one element), the boxes are
    r = configs.build_c3_classes(6)
    info = r.rowstream_info(torch.rand(40, 4), torch.rand(40, 7))
    assert info["ok"] and info["row_elements"] == 4
    # ... and at the benchmark's size (80 tasks of 8 732 rows) the launch has more chunks than the
    # device holds workgroups, and all tasks stream the same rows: the generic kernels keep it
    r = configs.build_c3_classes(80)
    big = r.rowstream_info(torch.rand(8732, 4), torch.rand(8732, 81))
    assert big["ok"] and not big["active"]
    assert r.rowstream_info(torch.rand(873, 4), torch.rand(873, 81))["active"]
    # a row of which less than half is read
    r = Region()
    x = r.tensor_input(torch.float32, 2)
    r.output(x.slice(1, 0, 3))
    r.compact_rows(x.select(1, 0) > 0.5)
    info = r.finalize().rowstream_info(torch.rand(40, 16))
    assert not info["ok"] and "half" in info["why"]
    # a dense region
    r = Region()
    x = r.tensor_input(torch.float32, 2)
    r.output(x * 2.0)
    info = r.finalize().rowstream_info(torch.rand(8, 8))
    assert not info["ok"] and "compaction" in info["why"]


def test_data_dependent_predicates_and_other_dtypes_on_the_cpu():
    """where on data, an int64 output (two words per element), a uint8 input, rows of 19 elements
    of which a ragged 7-column output is put together in a staging buffer."""
    r = configs.build_row_filter()
    args = [torch.rand(*sh) - 0.5 for sh in configs.ROW_FILTER_SHAPES]
    assert r.rowstream_info(*args)["ok"]
    assert_exact(_flat(emul.run_rowstream(r, *args, chunk_rows=100, sub_rows=17, threads=3)), _flat(emul.run(r, *args)), "row filter")

    r = Region()
    x = r.tensor_input(torch.float32, 2)
    idx = r.tensor_input(torch.int64, 1)
    flag = r.tensor_input(torch.uint8, 1)
    r.output(r.where(x > 0.0, x, x * 0.5))
    r.output(idx)
    r.output(x.select(1, 2).clamp(-0.25, 0.25))
    r.compact_rows((x.select(1, 1) > 0.1) & (flag > 0))
    r.finalize()
    g = torch.Generator().manual_seed(1)
    xs = torch.randn(300, 12, generator=g)
    ids = torch.arange(300) + (1 << 40)
    fl = (torch.rand(300, generator=g) > 0.3).to(torch.uint8)
    info = r.rowstream_info(xs, ids, fl)
    assert info["ok"], info
    got = emul.run_rowstream(r, xs, ids, fl, chunk_rows=77, sub_rows=10, threads=4)
    assert_exact(_flat(got), _flat(emul.run(r, xs, ids, fl)), "where / int64 / uint8")
    keep = (xs[:, 1] > 0.1) & (fl > 0)
    assert_exact(got[1], ids[keep], "int64 rows")
    assert_exact(got[0], torch.where(xs > 0, xs, xs * 0.5)[keep], "where")


# ---- on the GPU ---------------------------------------------------------------------------------
def _three_ways(r, *args, mode=1):
    """(generated kernel, generic two passes), both on the GPU; the generated kernel must be in use."""
    info = r.rowstream_info(*args)
    assert info["ok"] and info["active"], "no generated kernel linked for key %016x: run python -m functs_amd.aot --plan-only and rebuild" % info["key"]
    arr, n, _ = r._flatten(args)
    assert lib.fx_plan_launches(r.plan(arr, n).handle) == 1
    one = run_region("hip", r, *args)
    lib.fx_set_rowstream(0)
    lib.fx_set_head_kernel(0)
    try:
        assert lib.fx_plan_launches(r.plan(arr, n).handle) == 2
        two = run_region("hip", r, *args)
    finally:
        lib.fx_set_rowstream(mode)
        lib.fx_set_head_kernel(1)
    return one, two


@pytest.mark.gpu
@pytest.mark.parametrize("name", VARIANTS + ["benchmark"])
def test_variants_at_the_benchmark_shape_bit_exact_and_against_eager(name):
    pred, anchors, strides = oc.c5_inputs(0)
    r = _build(name, 16)
    one, two = _three_ways(r, pred, anchors, strides)
    assert_exact(_flat(one), _flat(two), "%s: generated kernel vs two passes" % name)
    ref = _eager(name, pred, anchors, strides)
    outs = list(zip(*one)) if len(one) > 1 else [(t,) for t in one[0]]
    for t, (got, want) in enumerate(zip(outs, ref)):
        if len(want) == 1:
            assert got[0].shape == want[0].shape
            assert_boxes_close(got[0][:, :4], want[0][:, :4], "%s boxes image %d" % (name, t))
            assert_close(got[0][:, 4:], want[0][:, 4:], "%s scores image %d" % (name, t))
        else:
            assert_boxes_close(got[0], want[0], "%s boxes image %d" % (name, t))
            assert_close(got[1], want[1], "%s cls image %d" % (name, t))
            assert_close(got[2], want[2], "%s obj image %d" % (name, t))


@pytest.mark.gpu
@pytest.mark.parametrize("n,batch", [(1, None), (63, None), (64, 3), (65, 2), (399, 5), (1000, 16), (5000, 2), (10647, 1)])
@pytest.mark.parametrize("name", ["stack_padded", "one_matrix", "benchmark"])
def test_any_number_of_rows_and_images(name, n, batch):
    args = _inputs(n, 80, batch or 1, seed=n)
    one, two = _three_ways(_build(name, batch), *args)
    assert_exact(_flat(one), _flat(two), "%s n=%d batch=%s" % (name, n, batch))


@pytest.mark.gpu
def test_the_generated_kernel_equals_the_hand_written_one():
    """fx_head_stream stays in the library as the reference the generated kernel is held to."""
    for r, args in ((configs.build_c2(), oc.c2_inputs(0)), (configs.build_c5(16), oc.c5_inputs(0))):
        gen = run_region("hip", r, *args)
        lib.fx_set_rowstream(0)
        try:
            out = (ctypes.c_int64 * 8)()
            arr, n, _ = r._flatten(args)
            lib.fx_plan_head_info(r.plan(arr, n).handle, out, 8)
            assert out[0] == 1 and out[1] == 1
            hand = run_region("hip", r, *args)
        finally:
            lib.fx_set_rowstream(1)
        assert_exact(_flat(gen), _flat(hand), "generated vs hand-written")


@pytest.mark.gpu
def test_nothing_kept_and_everything_kept():
    for name in ("stack_padded", "benchmark"):
        for value in (-20.0, 20.0):
            pred, anchors, strides = _inputs(700, 80, 4)
            pred[..., 4] = value
            one, two = _three_ways(_build(name, 4), pred, anchors, strides)
            assert_exact(_flat(one), _flat(two), "%s objectness %g" % (name, value))
            assert [t.shape[0] for t in one[2]] == [0 if value < 0 else 700] * 4


@pytest.mark.gpu
def test_bounded_wait_falls_back_to_counting():
    args = _inputs(3000, 80, 6, seed=5)
    for name in ("class_score_mask", "one_matrix"):
        r = _build(name, 6)
        ref = run_region("hip", r, *args)
        lib.fx_set_stream_spin_limit(0)
        try:
            got = run_region("hip", r, *args)
        finally:
            lib.fx_set_stream_spin_limit(4000)
        assert_exact(_flat(got), _flat(ref), "%s: workgroups that count for themselves" % name)


@pytest.mark.gpu
def test_calls_in_a_row_with_changing_inputs():
    """The status words are never cleared: each call must read only the counts of its own epoch."""
    r = _build("stack_padded", 3)
    dev = torch.device("cuda:0")
    for seed in range(5):
        pred, anchors, strides = _inputs(1500, 80, 3, seed=seed)
        if seed == 2:
            pred[..., 4] = -10.0
        got = r(pred.to(dev), anchors.to(dev), strides.to(dev))
        torch.cuda.synchronize()
        want = _eager("stack_padded", pred, anchors, strides)
        for t in range(3):
            assert_close(got[2][t].cpu(), want[t][2], "obj seed %d image %d" % (seed, t))
            assert_close(got[1][t].cpu(), want[t][1], "cls seed %d image %d" % (seed, t))


@pytest.mark.gpu
def test_predictions_that_start_at_an_odd_address_and_outputs_of_every_phase():
    """A view into a larger tensor: rows that are only 4-byte aligned; and kept-row counts that put
    the staged runs of the sub-tiles at every phase of a 16-byte group."""
    n = 500
    pred, anchors, strides = _inputs(n, 80, 1, seed=9)
    dev = torch.device("cuda:0")
    base = torch.zeros(pred.numel() + 7, device=dev)
    base[3:3 + pred.numel()] = pred.flatten().to(dev)
    view = base[3:3 + pred.numel()].view(1, n, 85)
    for name in ("one_matrix", "stack_padded"):
        r = _build(name, None)
        got = r(view, anchors.to(dev), strides.to(dev))
        ref = r(pred.to(dev), anchors.to(dev), strides.to(dev))
        torch.cuda.synchronize()
        assert_exact([t.cpu() for t in _flat(got)], [t.cpu() for t in _flat(ref)], name + ": odd start")


@pytest.mark.gpu
@pytest.mark.parametrize("n,batch", [(100000, None), (60000, 16)])
def test_launches_beyond_what_the_device_holds_at_once(n, batch):
    """The workgroups are persistent: with more chunks than the device holds workgroups (16 x 235
    chunks of 256 rows against six workgroups on each of 256 CUs) every workgroup takes chunks in
    turn, and the rows are those of the two passes."""
    args = _inputs(n, 80, batch or 1, seed=3)
    r = _build("stack", batch)
    info = r.rowstream_info(*args)
    assert info["ok"] and info["active"]
    one, two = _three_ways(r, *args)
    assert_exact(_flat(one), _flat(two), "n=%d batch=%s" % (n, batch))


@pytest.mark.gpu
def test_one_task_with_more_chunks_than_the_device_holds_workgroups():
    """450 000 rows are 1 758 chunks of 256 rows for 1 536 workgroups: some take a second chunk."""
    r = configs.build_row_filter()
    torch.manual_seed(11)
    args = [torch.rand(450000, 19) - 0.5, torch.rand(450000, 2) - 0.5]
    one, two = _three_ways(r, *args)
    assert_exact(_flat(one), _flat(two), "row filter, 450 000 rows")


@pytest.mark.gpu
def test_a_map_over_the_same_rows_keeps_the_two_passes_beyond_that_size_unless_forced():
    """80 class tasks over the same 8 732 boxes: by default the generic kernels; forced onto the
    generated kernel (every workgroup takes chunks in turn) the same rows."""
    r = configs.build_c3_classes(80)
    torch.manual_seed(12)
    args = [torch.rand(8732, 4), torch.rand(8732, 81) * 0.1]
    assert not r.rowstream_info(*args)["active"]
    two = run_region("hip", r, *args)
    lib.fx_set_rowstream(2)
    try:
        assert r.rowstream_info(*args)["active"]
        one = run_region("hip", r, *args)
    finally:
        lib.fx_set_rowstream(1)
    assert_exact(_flat(one), _flat(two), "class map, 80 tasks")


@pytest.mark.gpu
def test_the_coverage_region_on_the_gpu():
    r = configs.build_row_filter()
    args = [torch.rand(*sh) - 0.5 for sh in configs.ROW_FILTER_SHAPES]
    one, two = _three_ways(r, *args)
    assert_exact(_flat(one), _flat(two), "row filter")


@pytest.mark.gpu
def test_a_captured_call_takes_the_two_passes_and_replays_follow_their_inputs():
    r = _build("stack", 2)
    dev = torch.device("cuda:0")
    pred, anchors, strides = [t.to(dev) for t in _inputs(800, 80, 2, seed=1)]
    bc = r.bind(pred, anchors, strides)
    bc.launch()
    torch.cuda.synchronize()
    s = torch.cuda.Stream()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.stream(s):
        with torch.cuda.graph(g, stream=s):
            bc.launch(stream=s.cuda_stream)
    for seed in (2, 3, 4):
        new = _inputs(800, 80, 2, seed=seed)[0]
        pred.copy_(new.to(dev))
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        want = _eager("stack", new, anchors.cpu(), strides.cpu())
        tot = bc.totals.tolist()
        for t in range(2):
            assert tot[t] == want[t][2].shape[0]
            assert_close(bc.outs[2][t][:tot[t]].cpu(), want[t][2], "replay seed %d image %d" % (seed, t))


def _list_input_head(batch):
    """The head over a LIST of images: every task's prediction matrix is a tensor of its own."""
    from functs_amd import Region
    r = Region(parallel_degree=batch, is_parallel_map=True)
    p = r.tensor_input(torch.float32, 2, per_task=True)
    anchors = r.tensor_input(torch.float32, 2)
    strides = r.tensor_input(torch.float32, 1)
    pxy, pwh = p.slice(1, 0, 2).sigmoid(), p.slice(1, 2, 4)
    obj, cls = p.select(1, 4).sigmoid(), p.slice(1, 5, None).sigmoid()
    xy = (anchors.slice(1, 0, 2) + anchors.slice(1, 2, None)) * 0.5 + (pxy - 0.5) * strides.unsqueeze(-1)
    wh = (anchors.slice(1, 2, None) - anchors.slice(1, 0, 2)) * 0.5 * pwh.exp()
    r.compact_rows(obj >= 0.3)
    r.output(r.cat([xy - wh, xy + wh], 1))
    r.output(cls)
    r.output(obj)
    return r.finalize()


@pytest.mark.gpu
@pytest.mark.parametrize("batch,n", [(4, 900), (40, 10647), (130, 900)])
def test_a_map_over_a_list_of_images_streams_each_image_once(batch, n):
    """Per-task window pointers (the kernel is the linked one of the `cat` spelling: where a task's
    rows lie is an argument of the launch); the second case has more chunks than the device holds
    workgroups (1 680 of 256 rows), which a map over rows of its own takes in turn; the third
    more per-task buffers (520) than the kernel arguments hold: the build that reads the uploaded
    table."""
    r = _list_input_head(batch)
    g = torch.Generator().manual_seed(9)
    pred = torch.randn(batch, n, 85, generator=g)
    anchors = torch.rand(n, 4, generator=g) * 100
    strides = torch.full((n,), 8.0)
    images = [pred[t].clone() for t in range(batch)]
    dev = torch.device("cuda:0")
    dargs = [[im.to(dev) for im in images], anchors.to(dev), strides.to(dev)]
    assert r.rowstream_info(*dargs)["active"]
    print("list of", batch, "images", flush=True)
    arr, cnt, _ = r._flatten(dargs)
    assert lib.fx_plan_launches(r.plan(arr, cnt).handle) == 1
    one = [[t.cpu() for t in o] for o in r(*dargs)]
    torch.cuda.synchronize()
    lib.fx_set_rowstream(0)
    try:
        two = [[t.cpu() for t in o] for o in r(*dargs)]
        torch.cuda.synchronize()
    finally:
        lib.fx_set_rowstream(1)
    assert_exact(one, two, "list of images: one launch vs two passes")
    assert [o.shape[0] for o in one[0]] == [int((torch.sigmoid(im[:, 4]) >= 0.3).sum()) for im in images]
