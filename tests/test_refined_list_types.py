"""Refined list types (fait/passes/refine_types.cpp:57-81, 175-195; fait/passes/te_op.cpp:43-59):
a list argument whose example is a list of tensors keeps the tuple of its elements' types while
the pipeline runs.  A map functor records the unified element type for it, and len() of the list
is the constant of the example (the pipeline is specialised to the example's shapes)."""
from typing import List

import pytest
import torch
from torch import Tensor

import functs_amd.jit as fj


def over_len(xs: List[Tensor], w: Tensor) -> List[Tensor]:
    out: List[Tensor] = []
    for i in range(len(xs)):
        out.append((xs[i] * w + 1.0).sigmoid())
    return out


def grows(xs: List[Tensor], w: Tensor) -> List[Tensor]:
    xs.append(w)
    out: List[Tensor] = []
    for i in range(len(xs)):
        out.append((xs[i] * w + 1.0).sigmoid())
    return out


def _functors(graph):
    return [n for n in graph.nodes() if n.kind() == "tssa::ParallelFunctor"]


def _kinds(graph):
    return [n.kind() for n in graph.nodes()]


def test_a_map_records_the_element_type_and_len_is_a_constant():
    xs = [torch.rand(5, 3) for _ in range(4)]
    built = fj.build(fj.script(over_len), [xs, torch.rand(3)])
    assert "aten::len" not in _kinds(built.graph)
    (f,) = _functors(built.graph)
    assert f.i("parallel_degree") == 4 and f.i("is_parallel_map") == 1
    assert "input_refine_types=[Float(5, 3, " in str(built.graph)      # not Tensor[]
    t = f.tys("input_refine_types")[0]
    assert t.kind() == "TensorType" and t.sizes() == [5, 3]


def test_ragged_elements_unify():
    xs = [torch.rand(n, 3) for n in (5, 2, 7)]
    built = fj.build(fj.script(over_len), [xs, torch.rand(3)])
    (f,) = _functors(built.graph)
    assert f.i("parallel_degree") == 3
    t = f.tys("input_refine_types")[0]
    assert t.kind() == "TensorType" and t.dim() == 2 and t.sizes() is None      # rows differ from element to element
    assert "input_refine_types=[Float(*, 3, " in str(built.graph)


def test_a_list_that_is_written_is_not_refined():
    xs = [torch.rand(5, 3) for _ in range(4)]
    built = fj.build(fj.script(grows), [xs, torch.rand(5, 3)])
    assert "aten::len" in _kinds(built.graph)


@pytest.mark.gpu
def test_refined_map_equals_eager():
    g = torch.Generator().manual_seed(3)
    xs = [torch.rand(n, 3, generator=g) for n in (5, 2, 7)]
    w = torch.rand(3, generator=g)
    built = fj.build(fj.script(over_len), [xs, w])
    got = built([x.cuda() for x in xs], w.cuda())
    ref = over_len(xs, w)
    assert len(got) == len(ref)
    for a, b in zip(got, ref):
        torch.testing.assert_close(a.cpu(), b, rtol=1e-6, atol=0)
