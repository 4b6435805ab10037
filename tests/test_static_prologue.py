"""The step in front of the hot path: anchors generated from the feature-map sizes
(functs/benchmark/ai_model/yolov3/yolov3_bbox.py:78-101, 195-216 in the reference).  What the
static types answer (size, len, dtype; the device when the examples live on a GPU) is folded into
constants when the function is built (FoldStaticTypeQueries), constant propagation then runs the
index arithmetic of the generator once, at build time, and the region reads the anchors as a
table: the decode + score filter stays the region that the detection-head kernel runs.  A function
built that way serves the shapes of its example; other shapes get a graph of their own."""
from typing import List

import pytest
import torch
from torch import Tensor

import functs_amd.aot as aot
import functs_amd.jit as fj
from functs_amd import _C
from functs_amd.benchmark.programs import yolov3_postproc


def _meshgrid(x: Tensor, y: Tensor):
    xx = x.repeat(y.size(0))
    yy = y.reshape(-1, 1).repeat(1, x.size(0)).reshape(-1)
    return xx, yy


def _level_anchors(base: Tensor, feat_h: int, feat_w: int, stride: int, like: Tensor):
    shift_x = torch.arange(0, feat_w, dtype=like.dtype, device=like.device) * stride
    shift_y = torch.arange(0, feat_h, dtype=like.dtype, device=like.device) * stride
    xx, yy = _meshgrid(shift_x, shift_y)
    shifts = torch.stack([xx, yy, xx, yy], dim=-1)
    return (base[None, :, :] + shifts[:, None, :]).reshape(-1, 4)


def generated_anchors(pred: Tensor):
    """Anchors [N, 4] and strides [N] of three levels of s x s cells, s = g, 2g, 4g, three base
    anchors per cell (the base anchors are attributes of the reference's model: constants)."""
    g = int(float(pred.size(1) // 63) ** 0.5 + 0.5)     # N = 3 (g^2 + 4 g^2 + 16 g^2): 13 for the benchmark shape
    base0 = torch.tensor([[-58.0, -45.0, 58.0, 45.0], [-78.0, -99.0, 78.0, 99.0], [-186.5, -163.0, 186.5, 163.0]],
                         dtype=pred.dtype, device=pred.device)
    base1 = torch.tensor([[-15.0, -30.5, 15.0, 30.5], [-31.0, -22.5, 31.0, 22.5], [-29.5, -59.5, 29.5, 59.5]],
                         dtype=pred.dtype, device=pred.device)
    base2 = torch.tensor([[-5.0, -6.5, 5.0, 6.5], [-8.0, -15.0, 8.0, 15.0], [-16.5, -11.5, 16.5, 11.5]],
                         dtype=pred.dtype, device=pred.device)
    a0 = _level_anchors(base0, g, g, 32, pred)
    a1 = _level_anchors(base1, 2 * g, 2 * g, 16, pred)
    a2 = _level_anchors(base2, 4 * g, 4 * g, 8, pred)
    anchors = torch.cat([a0, a1, a2])
    strides = torch.cat([torch.full([a0.size(0)], 32.0, dtype=pred.dtype, device=pred.device),
                         torch.full([a1.size(0)], 16.0, dtype=pred.dtype, device=pred.device),
                         torch.full([a2.size(0)], 8.0, dtype=pred.dtype, device=pred.device)])
    return anchors, strides


def head_with_generated_anchors(pred: Tensor):
    anchors, strides = generated_anchors(pred)
    return yolov3_postproc(pred, anchors, strides)


def _inputs(g=13, seed=0, dev="cpu"):
    gen = torch.Generator().manual_seed(seed)
    n = 3 * (g * g + 4 * g * g + 16 * g * g)
    return [torch.randn(1, n, 85, generator=gen).to(dev)]


def _kinds(block, out=None):
    out = [] if out is None else out
    for n in block.nodes():
        out.append(n.kind())
        for b in n.blocks():
            _kinds(b, out)
    return out


def _all_kinds(graph):
    """Kinds of the graph and of every functor's region."""
    out = _kinds(graph)
    for n in graph.nodes():
        if n.kind() == "tssa::ParallelFunctor":
            out += _kinds(n.g("Subgraph"))
    return out


def test_size_and_dtype_queries_of_static_types_become_constants():
    built = fj.build(fj.script(head_with_generated_anchors), _inputs())
    kinds = _kinds(built.graph)
    params = set(v.debugName() for v in built.graph.inputs())
    asked = [n.inputsAt(0).debugName() for n in built.graph.nodes() if n.kind() in ("aten::size", "prim::dtype")]
    assert not (set(asked) & params)       # (values made inside the graph have no static type: their queries stay)
    # built from CPU examples the device stays a run-time value (what the function creates follows
    # its arguments), so the generator itself still runs per call, as a region of its own
    assert "prim::device" in kinds and "aten::arange" in _all_kinds(built.graph)


def test_the_pass_alone():
    def f(x: Tensor, xs: List[Tensor]):
        return x.size(0) * x.size(-1) + x.dim() + x.numel() + len(xs), xs[1].size(0), x.size()

    g = torch.jit.script(f).graph.copy()
    hints = [fj.extract_type_hint_from_tensor(a) for a in (torch.rand(3, 5), [torch.rand(2), torch.rand(7)])]
    assert _C._jit_pass_fait_pipeline(g, hints)       # True: the graph is specialised to these shapes
    fn = _C._create_function_from_graph("f", g)
    assert not any(k in _kinds(g) for k in ("aten::size", "aten::dim", "aten::numel", "aten::len"))
    assert fn(torch.rand(3, 5), [torch.rand(2), torch.rand(7)]) == (3 * 5 + 2 + 15 + 2, 7, [3, 5])


def test_a_built_function_follows_the_shapes_it_is_called_with():
    def rows_times_two(x: Tensor):
        out: List[Tensor] = []
        for i in range(x.size(0)):
            out.append(x[i] * 2.0 + float(x.size(1)))
        return out

    built = fj.build(fj.script(rows_times_two), [torch.rand(3, 4)])
    assert built._variants is not None and len(built._variants) == 1


@pytest.mark.gpu
def test_generated_anchors_are_folded_and_the_head_kernel_runs():
    dev = torch.device("cuda:0")
    args = _inputs(dev=dev)
    built = fj.build(fj.script(head_with_generated_anchors), args)     # examples on the GPU: the device is static too
    kinds = _all_kinds(built.graph)
    for k in ("aten::arange", "aten::repeat", "aten::stack", "aten::full", "aten::cat", "aten::size", "prim::device"):
        assert k not in kinds, k
    assert "aten::zeros_like" in kinds or "aten::zeros" in kinds     # the box buffer is a fill inside the region, not a constant
    functors = [n for n in built.graph.nodes() if n.kind() == "tssa::ParallelFunctor"]
    assert len(functors) == 1 and functors[0].i("compact_rows") == 1
    total0, _ = aot.launch_stats()
    got = built(*args)
    torch.cuda.synchronize()
    total1, _ = aot.launch_stats()
    assert total1 - total0 == 1                                         # the detection-head kernel, nothing else
    ref = head_with_generated_anchors(*[a.cpu() for a in args])
    assert ref[0].shape[0] > 1000
    assert [tuple(t.shape) for t in got] == [tuple(t.shape) for t in ref]
    torch.testing.assert_close(got[1].cpu(), ref[1], rtol=1e-5, atol=1e-7)
    torch.testing.assert_close(got[2].cpu(), ref[2], rtol=1e-5, atol=1e-7)
    scale = torch.maximum(ref[0][:, :2].abs(), ref[0][:, 2:].abs()).repeat(1, 2)
    assert bool(((got[0].cpu() - ref[0]).abs() <= 1e-7 + 1e-5 * scale).all())


@pytest.mark.gpu
def test_other_shapes_get_a_graph_of_their_own():
    dev = torch.device("cuda:0")
    built = fj.build(fj.script(head_with_generated_anchors), _inputs(13, dev=dev))
    for g, seed in ((13, 1), (7, 2), (13, 3), (10, 4)):
        args = _inputs(g, seed, dev)
        got = built(*args)
        ref = head_with_generated_anchors(*[a.cpu() for a in args])
        assert [tuple(t.shape) for t in got] == [tuple(t.shape) for t in ref], g
        torch.testing.assert_close(got[2].cpu(), ref[2], rtol=1e-5, atol=1e-7)
    assert len(built._variants) == 3


def test_a_constant_of_negative_zeros_keeps_its_sign():
    """A uniform constant tensor becomes a fill inside its region; -0.0 == 0.0, but a fill with
    zeros would lose the sign (1 / x, copysign and bitwise comparisons tell them apart)."""
    def f(x: Tensor):
        # (the literal -0.0 reaches the graph as +0.0: the sign is made by arithmetic)
        return x + torch.full([32], 0.0).neg(), x + torch.tensor([1.0, -1.0] * 16) * 0.0

    g = torch.jit.script(f).graph.copy()
    torch._C._jit_pass_constant_propagation(g)
    assert "aten::full" not in _kinds(g) and "aten::neg" not in _kinds(g)    # both are tensor constants now
    assert _C._jit_pass_uniform_constants_to_fills(g)
    kinds = _kinds(g)
    assert "aten::zeros" not in kinds and kinds.count("aten::full") == 1   # the mixed one stays a constant
    value = list([n for n in g.nodes() if n.kind() == "aten::full"][0].inputs())[1].toIValue()
    import math
    assert value == 0.0 and math.copysign(1.0, value) == -1.0
    fn = torch._C._create_function_from_graph("f", g)
    x = torch.full([32], -0.0)
    a, _ = fn(x)
    assert bool(torch.signbit(a).all())
