"""The lean dense kernel against the general one.

Dense regions of one task class with one or two outputs of 32-bit elements run a short kernel of
their own when their programs are compiled (fx_dense_lean, the counterpart of the
one-element-per-thread launch of fait/tensorexpr/cuda_codegen_tssa.cpp:1167-1306).  It has to
give the general kernel's results bit for bit: same item geometry, same instruction steps.
The programs here are ones whose compiled kernels are linked into the library: the collapsed
get_started loop (examples/get_started.py:10-15), an elementwise chain (at shapes that end
inside a lane group, inside an item, inside a unit and at both unit sizes), SSD's decode + softmax
and a region with reduction loops."""
import pytest
import torch

from functs_amd import Region, _lib, configs

gpu = pytest.mark.gpu


def _stream_region():
    r = Region()
    x = r.tensor_input(torch.float32, 2)
    r.output((x * 2.0 + 1.0).sigmoid())
    return r.finalize()


SHAPES = [(1, 1), (1, 3), (3, 5), (7, 64), (64, 1000), (257, 255), (1023, 1025), (1024, 1024), (2048, 2049), (4100, 1024)]


def _lean(bound):
    return bool(_lib.lib.fx_plan_dense_lean(bound.plan.handle))


@pytest.fixture
def lean_switch():
    yield
    _lib.lib.fx_set_dense_lean(1)


@gpu
@pytest.mark.parametrize("shape", SHAPES)
def test_collapsed_loop_on_the_lean_kernel(shape, lean_switch):
    dev = torch.device("cuda:0")
    torch.manual_seed(shape[0] * 7919 + shape[1])
    b = torch.randn(*shape, device=dev)
    r = configs.build_c1()
    bc = r.bind(b, shape[0])
    assert _lean(bc), "the collapsed loop is compiled and fits the lean kernel"
    bc.launch()
    lean = bc.results()[0].clone()
    _lib.lib.fx_set_dense_lean(0)
    assert not _lean(r.bind(b, shape[0]))
    general = r(b, shape[0])[0]
    torch.cuda.synchronize()
    assert torch.equal(lean, general)
    assert torch.equal(lean, b + 1)


@gpu
@pytest.mark.parametrize("shape", SHAPES)
def test_elementwise_chain_on_the_lean_kernel(shape, lean_switch):
    dev = torch.device("cuda:0")
    torch.manual_seed(shape[0] * 104729 + shape[1])
    x = torch.randn(*shape, device=dev) * 4
    r = _stream_region()
    bc = r.bind(x)
    assert _lean(bc)
    bc.launch()
    lean = bc.results()[0].clone()
    _lib.lib.fx_set_dense_lean(0)
    general = r(x)[0]
    torch.cuda.synchronize()
    assert torch.equal(lean, general)
    torch.testing.assert_close(lean, torch.sigmoid(x * 2.0 + 1.0), rtol=1e-5, atol=1e-6)


@gpu
def test_partial_loop_keeps_the_other_rows(lean_switch):
    """n below the number of rows: the rows from n on pass through unchanged (a second kind of
    element in the same unit), on both kernels."""
    dev = torch.device("cuda:0")
    torch.manual_seed(5)
    b = torch.randn(300, 77, device=dev)
    r = configs.build_c1()
    lean = r(b, 123)[0].clone()
    _lib.lib.fx_set_dense_lean(0)
    general = r(b, 123)[0]
    torch.cuda.synchronize()
    want = b.clone()
    want[:123] += 1
    assert torch.equal(lean, general)
    assert torch.equal(lean, want)


@gpu
@pytest.mark.parametrize("rows,classes", [(8732, 81), (100, 81), (7, 81), (513, 21)])
def test_rows_that_are_reduced_on_the_lean_kernel(rows, classes, lean_switch):
    """SSD's decode + softmax (functs/benchmark/ai_model/ssd/ssd_bbox.py:121-154, 163-170): the
    scores take one row per segment of a wave and are reduced inside it; two outputs."""
    dev = torch.device("cuda:0")
    torch.manual_seed(rows)
    loc = torch.randn(1, rows, 4, device=dev)
    conf = torch.randn(1, rows, classes, device=dev) * 3
    priors = torch.rand(rows, 4, device=dev)
    r = configs.build_c3_decode()
    bc = r.bind(loc, conf, priors)
    if not r.specialized(loc, conf, priors):
        pytest.skip("no compiled kernels linked for this number of classes")
    assert _lean(bc)
    bc.launch()
    lean = [t.clone() for t in bc.results()]
    _lib.lib.fx_set_dense_lean(0)
    general = r(loc, conf, priors)
    torch.cuda.synchronize()
    assert torch.equal(lean[0], general[0]) and torch.equal(lean[1], general[1])
    torch.testing.assert_close(lean[1], conf[0].softmax(-1), rtol=1e-5, atol=1e-7)


@gpu
def test_reduction_loops_and_a_row_softmax_on_the_lean_kernel(lean_switch):
    dev = torch.device("cuda:0")
    torch.manual_seed(4)
    x = torch.randn(*configs.COLUMN_STANDARDIZE_SHAPE, device=dev)
    r = configs.build_column_standardize()
    bc = r.bind(x)
    assert _lean(bc)
    bc.launch()
    lean = [t.clone() for t in bc.results()]
    _lib.lib.fx_set_dense_lean(0)
    general = r(x)
    torch.cuda.synchronize()
    assert torch.equal(lean[0], general[0]) and torch.equal(lean[1], general[1])


@gpu
def test_interpreted_regions_do_not_take_it(lean_switch):
    """The kernel exists for compiled programs only: a region without a linked kernel runs the
    general kernel through the interpreter and says so."""
    dev = torch.device("cuda:0")
    r = Region()
    x = r.tensor_input(torch.float32, 2)
    r.output((x * 3.0 - 0.25).tanh().relu())
    r = r.finalize()
    xs = torch.randn(100, 50, device=dev)
    bc = r.bind(xs)
    if _lean(bc):
        pytest.skip("a kernel for this program is linked")
    bc.launch()
    torch.testing.assert_close(bc.results()[0], (xs * 3.0 - 0.25).tanh().relu(), rtol=1e-5, atol=1e-6)


def test_switch_is_exported():
    assert hasattr(_lib.lib, "fx_set_dense_lean") and hasattr(_lib.lib, "fx_plan_dense_lean")
