"""Argument kinds of tssa::ParallelFunctor besides tensors and tensor lists: the reference's
GraphBuilder::prepareRunArgs takes float[], int[], bool[], List[Tuple[int, ...]], List[List[int]]
and scalars (fait/fuser/graph_builder.cpp:736-857).  Here list and tuple values travel as their
elements; per-task ints that shapes depend on split the tasks into classes."""
from typing import List, Tuple

import pytest
import torch

import functs_amd.jit as fj


def size_list_from_a_tensor(x: torch.Tensor, y: torch.Tensor):
    s = y.size()
    return x.reshape(s) * 2 + 1


def per_task_size_lists(x: torch.Tensor, shapes: List[List[int]]):
    out = []
    for i in range(len(shapes)):
        out.append(x[i].reshape(shapes[i]) * 2 + 1)
    return out


def per_task_floats(x: torch.Tensor, scales: List[float]):
    out = []
    for i in range(len(scales)):
        out.append(x[i] * scales[i] + 1)
    return out


def per_task_tuples(x: torch.Tensor, hw: List[Tuple[int, int]]):
    out = []
    for i in range(len(hw)):
        h, w = hw[i]
        out.append(x[i, :h, :w] * 2 + 1)
    return out


def per_task_ints_in_slices(x: torch.Tensor, ks: List[int]):
    out = []
    for i in range(len(ks)):
        out.append(x[i, :ks[i]] * 2 + 1)
    return out


def shared_int_in_a_slice(x: torch.Tensor, k: int):
    return x[:, :k] * 2 + 1


def _rand(*shape):
    return torch.rand(*shape, generator=torch.Generator().manual_seed(11))


CASES = [
    (size_list_from_a_tensor, [_rand(4, 6), _rand(3, 8)], None),
    (per_task_size_lists, [_rand(3, 12), [[3, 4], [2, 6], [4, 3]]], [_rand(3, 12), [[12, 1], [1, 12], [6, 2]]]),
    (per_task_floats, [_rand(3, 5), [1.0, 2.0, 3.0]], [_rand(3, 5), [0.5, -1.0, 4.0]]),
    (per_task_tuples, [_rand(2, 8, 8), [(3, 4), (5, 6)]], [_rand(2, 8, 8), [(8, 1), (2, 7)]]),
    (per_task_ints_in_slices, [_rand(3, 8), [3, 5, 8]], [_rand(3, 8), [1, 2, 7]]),
    (shared_int_in_a_slice, [_rand(3, 8), 5], [_rand(3, 8), 3]),
]


@pytest.mark.parametrize("prog,example,_second", CASES, ids=[c[0].__name__ for c in CASES])
def test_one_region_and_no_loop(prog, example, _second):
    f = fj.build(fj.script(prog), example)
    kinds = [n.kind() for n in f.graph.nodes()]
    assert kinds.count("tssa::ParallelFunctor") == 1 and "prim::Loop" not in kinds and "prim::ParallelMap" not in kinds


@pytest.mark.gpu
@pytest.mark.parametrize("prog,example,second", CASES, ids=[c[0].__name__ for c in CASES])
def test_against_eager(prog, example, second):
    f = fj.build(fj.script(prog), example)
    for args in (example, second):
        if args is None:
            continue
        want = prog(*args)
        got = f(*[a.cuda() if isinstance(a, torch.Tensor) else a for a in args])
        want, got = (want, got) if isinstance(want, list) else ([want], [got])
        assert len(got) == len(want)
        for g, w in zip(got, want):
            assert g.shape == w.shape
            torch.testing.assert_close(g.cpu(), w, rtol=1e-6, atol=0)


@pytest.mark.gpu
def test_lists_of_different_lengths_are_refused():
    f = fj.build(fj.script(per_task_size_lists), [_rand(3, 12), [[3, 4], [2, 6], [4, 3]]])
    with pytest.raises(RuntimeError, match="differ in length"):
        f(_rand(3, 12).cuda(), [[3, 4], [12], [4, 3]])


def causal_scores(q: torch.Tensor):
    return torch.tril(q * 2.0 + 1.0, 0).exp()


@pytest.mark.gpu
def test_tril_through_the_torchscript_route():
    x = _rand(6, 6)
    f = fj.build(fj.script(causal_scores), [x])
    assert [n.kind() for n in f.graph.nodes()].count("tssa::ParallelFunctor") == 1
    torch.testing.assert_close(f(x.cuda()).cpu(), causal_scores(x), rtol=1e-5, atol=1e-6)
