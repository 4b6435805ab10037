"""The step in front of the hot path: anchor / stride tables generated inside the region
(the reference's model builds them with arange / repeat / stack / reshape on the host,
functs/benchmark/ai_model/yolov3/yolov3_bbox.py:78-101, and the reference fuses those operators,
fait/fuser/custom_lowering_func.cpp:258-350).  Checked against stock torch on the same inputs."""
import pytest
import torch

from functs_amd import configs
from functs_amd._lib import FxError
from functs_amd.benchmark.programs import yolov3_postproc
from tests.util import run_region, assert_close, assert_boxes_close

LEVELS = configs.GENERATED_ANCHOR_LEVELS
SIZES = (((116, 90), (156, 198), (373, 326)), ((30, 61), (62, 45), (59, 119)), ((10, 13), (16, 30), (33, 23)))


def _inputs(batch, seed):
    g = torch.Generator().manual_seed(seed)
    n = sum(f * f * 3 for f, _ in LEVELS)
    preds = torch.randn(batch, n, 85, generator=g)
    bases = [torch.tensor([[-w / 2, -h / 2, w / 2, h / 2] for w, h in s]) for s in SIZES]
    return preds, bases


def _torch_reference(preds, bases):
    anc, st = [], []
    for b, (f, s) in zip(bases, LEVELS):
        sx = torch.arange(0, f, dtype=torch.float32) * s
        xx = sx.repeat(f)
        yy = sx.view(-1, 1).repeat(1, f).view(-1)
        shifts = torch.stack([xx, yy, xx, yy], -1)
        anc.append((b[None] + shifts[:, None]).reshape(-1, 4))
        st.append(torch.full((f * f * 3,), s))
    anchors, strides = torch.cat(anc), torch.cat(st)
    return [yolov3_postproc(preds[i:i + 1], anchors, strides) for i in range(preds.size(0))]


def test_generated_anchors_equal_torch_on_the_emulator():
    preds, bases = _inputs(2, 3)
    r = configs.build_c5_generated_anchors(2, LEVELS)
    out = run_region("emul", r, preds, *bases)
    ref = _torch_reference(preds, bases)
    for i in range(2):
        assert_boxes_close(out[0][i], ref[i][0], "boxes[%d]" % i)
        assert_close(out[1][i], ref[i][1], "cls[%d]" % i)
        assert_close(out[2][i], ref[i][2], "obj[%d]" % i)


def test_generated_anchors_have_a_key_and_a_source():
    preds, bases = _inputs(2, 3)
    r = configs.build_c5_generated_anchors(2, LEVELS)
    assert r.spec_key(preds, *bases) != 0
    assert "FX_SPEC_COMPACT" in r.spec_source(preds, *bases)


@pytest.mark.gpu
def test_generated_anchors_run_interpreted_in_the_large_lds():
    """The interpreter keeps temporaries in LDS and this region has more of them than fit the
    default 64 KB of a workgroup: the launch asks for what it needs of the 160 KB of a CU, and the
    interpreter gives the compiled kernels' results bit for bit."""
    dev = torch.device("cuda:0")
    preds, bases = _inputs(2, 3)
    r = configs.build_c5_generated_anchors(2, LEVELS)
    args = [preds.to(dev)] + [b.to(dev) for b in bases]
    import functs_amd.aot as aot
    from tests.util import assert_exact
    compiled = [[t.cpu() for t in o] for o in r(*args)]
    torch.cuda.synchronize()
    aot.enable(False)   # as if the compiled kernels of this region were not linked in
    try:
        assert not r.specialized(*args)
        interpreted = [[t.cpu() for t in o] for o in r(*args)]
        torch.cuda.synchronize()
    finally:
        aot.enable(True)
    assert_exact(interpreted, compiled, "interpreter in the large LDS")


@pytest.mark.gpu
def test_generated_anchors_equal_torch_on_the_gpu():
    """Parity of the region with generated anchors on the GPU (its compiled kernels are linked
    into the library: the interpreter's temporaries do not fit LDS for this region)."""
    dev = torch.device("cuda:0")
    preds, bases = _inputs(2, 3)
    r = configs.build_c5_generated_anchors(2, LEVELS)
    args = [preds.to(dev)] + [b.to(dev) for b in bases]
    assert r.specialized(*args), "the compiled kernels of this region are not linked in"
    out = run_region("hip", r, preds, *bases)
    ref = _torch_reference(preds, bases)
    for i in range(2):
        assert_boxes_close(out[0][i], ref[i][0], "boxes[%d]" % i)
        assert_close(out[1][i], ref[i][1], "cls[%d]" % i)
        assert_close(out[2][i], ref[i][2], "obj[%d]" % i)


def test_generated_anchors_have_a_row_stream_form_with_a_linked_kernel():
    """The generation inlines into the rows' own code once (the generator shares what the four
    box columns have in common), so the region runs on the one-launch skeleton like the regions
    that read the tables."""
    preds, bases = _inputs(2, 3)
    info = configs.build_c5_generated_anchors(2, LEVELS).rowstream_info(preds, *bases)
    assert info["ok"] and info["active"] and info["row_elements"] == 85, info


@pytest.mark.gpu
def test_generated_anchors_on_the_row_stream_kernel_equal_the_two_passes_and_torch():
    from functs_amd._lib import lib
    from tests.util import assert_exact
    dev = torch.device("cuda:0")
    preds, bases = _inputs(2, 5)
    r = configs.build_c5_generated_anchors(2, LEVELS)
    args = [preds.to(dev)] + [b.to(dev) for b in bases]
    arr, n, _ = r._flatten(args)
    assert lib.fx_plan_launches(r.plan(arr, n).handle) == 1
    one = [[t.cpu() for t in o] for o in r(*args)]
    torch.cuda.synchronize()
    lib.fx_set_rowstream(0)
    try:
        assert lib.fx_plan_launches(r.plan(arr, n).handle) == 2
        two = [[t.cpu() for t in o] for o in r(*args)]
        torch.cuda.synchronize()
    finally:
        lib.fx_set_rowstream(1)
    assert_exact(one, two, "generated anchors: row-stream kernel vs two passes")
    ref = _torch_reference(preds, bases)
    for i in range(2):
        assert_boxes_close(one[0][i], ref[i][0], "boxes[%d]" % i)
        assert_close(one[1][i], ref[i][1], "cls[%d]" % i)
        assert_close(one[2][i], ref[i][2], "obj[%d]" % i)


@pytest.mark.gpu
def test_generated_anchors_at_the_benchmark_size_equal_the_region_that_reads_the_tables():
    """16 images of 10 647 rows: the same rows as c5 (whose anchors and strides are the tables this
    region generates), one launch."""
    from functs_amd._lib import lib
    from oracle import configs as oc
    dev = torch.device("cuda:0")
    preds, anchors, strides = oc.c5_inputs(0)
    levels = configs.GENERATED_ANCHOR_LEVELS_C5
    sizes = (((116, 90), (156, 198), (373, 326)), ((30, 61), (62, 45), (59, 119)), ((10, 13), (16, 30), (33, 23)))
    bases = [torch.tensor([[-w / 2, -h / 2, w / 2, h / 2] for w, h in s]) for s in sizes]
    r = configs.build_c5_generated_anchors(16, levels)
    args = [preds.to(dev)] + [b.to(dev) for b in bases]
    info = r.rowstream_info(*args)
    assert info["ok"] and info["active"], info
    got = r(*args)
    torch.cuda.synchronize()
    # the tables of the same generator, read from memory by the benchmark's region
    anc, st = [], []
    for b, (f, s) in zip(bases, levels):
        sx = torch.arange(0, f, dtype=torch.float32) * s
        xx, yy = sx.repeat(f), sx.view(-1, 1).repeat(1, f).view(-1)
        shifts = torch.stack([xx, yy, xx, yy], -1)
        anc.append((b[None] + shifts[:, None]).reshape(-1, 4))
        st.append(torch.full((f * f * 3,), s))
    want = configs.build_c5(16)(preds.to(dev), torch.cat(anc).to(dev), torch.cat(st).to(dev))
    torch.cuda.synchronize()
    for t in range(16):
        assert got[2][t].shape == want[2][t].shape
        assert torch.equal(got[2][t], want[2][t]) and torch.equal(got[1][t], want[1][t])
        assert_boxes_close(got[0][t].cpu(), want[0][t].cpu(), "boxes image %d" % t)
