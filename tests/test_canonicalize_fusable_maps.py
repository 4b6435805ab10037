"""CanonicalizeFusableMaps (fait/passes/parallelize_loops.cpp:458-502, run at
fait/fait_pipeline.cpp:61): the fusion group that is the first node of a ParallelMap takes the
index first, then the map's parameters in the map's order, then the values from outside the map;
the map returns what the group returns, in the group's order.  The functor built from such a map
then has its per-task arguments in front of the shared ones.  CPU tests look at the graphs; the gpu
test runs the built function against eager mode (1e-6 relative: one sigmoid)."""
from typing import List, Tuple

import pytest
import torch
from torch import Tensor

import functs_amd.jit as fj
from functs_amd import _C


def shared_first(w: Tensor, xs: List[Tensor], ys: List[Tensor]) -> Tuple[List[Tensor], List[Tensor]]:
    outs: List[Tensor] = []
    sums: List[Tensor] = []
    for i in range(3):
        t = w * 2.0 + xs[i]
        sums.append(t * ys[i] - w)
        outs.append((t + ys[i]).sigmoid())
    return outs, sums


def _inputs(dev="cpu"):
    g = torch.Generator().manual_seed(11)
    w = torch.rand(4, generator=g).to(dev)
    xs = [torch.rand(4, generator=g).to(dev) for _ in range(3)]
    ys = [torch.rand(4, generator=g).to(dev) for _ in range(3)]
    return [w, xs, ys]


def _functors(graph):
    return [n for n in graph.nodes() if n.kind() == "tssa::ParallelFunctor"]


def test_per_task_arguments_come_first():
    built = fj.build(fj.script(shared_first), _inputs())
    fs = _functors(built.graph)
    assert len(fs) == 1
    f = fs[0]
    assert list(getattr(f, "is")("is_parallel_args")) == [1, 1, 0]
    names = [v.debugName().split(".")[0] for v in f.inputs()]
    assert names == ["xs", "ys", "w"]
    sub = f.g("Subgraph")
    ins = list(sub.inputs())
    assert len(ins) == 4 and str(ins[0].type()) == "int"      # index, xs[i], ys[i], w


def test_the_pass_is_idempotent_on_a_built_graph():
    built = fj.build(fj.script(shared_first), _inputs())
    g = built.graph.copy()
    before = str(g)
    _C._jit_pass_fait_canonicalize_fusable_maps(g)
    assert str(g) == before


@pytest.mark.gpu
def test_reordered_map_equals_eager():
    args = _inputs()
    built = fj.build(fj.script(shared_first), args)
    outs, sums = built(*_inputs("cuda:0"))
    ref_outs, ref_sums = shared_first(*args)
    assert len(outs) == 3 and len(sums) == 3
    for a, b in zip(sums, ref_sums):
        assert torch.equal(a.cpu(), b)                          # products and sums only
    for a, b in zip(outs, ref_outs):
        torch.testing.assert_close(a.cpu(), b, rtol=1e-6, atol=0)
