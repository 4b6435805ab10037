"""CanonicalizeOps (fait/passes/canonicalize.cpp:148-157), HoistLoopInvariants
(fait/passes/licm.cpp:55-66) and regions inside prim::If blocks (the values an `if` carries after
functionalization, functs/csrc/jit/passes/convert_to_tensorssa.cpp:356-362).  CPU tests look at
the graphs; the gpu tests run the built functions against eager mode on the same inputs
(bit-exact for copies and products, 1e-6 relative where a transcendental is involved)."""
from typing import List

import pytest
import torch
from torch import Tensor

import functs_amd.jit as fj
from functs_amd import _C


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
        for b in n.blocks():
            for m in b.nodes():
                if m.kind() == "tssa::ParallelFunctor":
                    out += _kinds(m.g("Subgraph"))
    return out


def _canon(fn, args=None):
    g = torch.jit.script(fn).graph.copy()
    if args is not None:
        for v, a in zip(g.inputs(), args):
            if isinstance(a, torch.Tensor):
                v.setType(fj.extract_type_hint_from_tensor(a))
    _C._jit_pass_canonicalize_ops(g)
    torch._C._jit_pass_dce(g)
    return g


# --- programs -------------------------------------------------------------------------------------
def spellings(x: Tensor, y: Tensor):
    a = torch.max(x, y) - torch.min(x, y)              # max.other / min.other
    z = x.new_zeros([x.size(0), x.size(1)]) + x.new_ones([x.size(0), x.size(1)])
    p = x.pow(2) + y.pow(3) + (x * 0.5).pow(5)         # products
    w = x.t().t()[:, :] + y.view(-1).view(x.size(0), x.size(1))
    r = torch.arange(x.size(1), device=x.device).to(torch.float32)   # arange(end), to.dtype
    return a + z + p + w + r + y.to(x)                 # to.other


def integer_spellings(i: Tensor):
    return i.new_zeros([i.size(0)]) + i.pow(2)         # the dtype follows the tensor


def sizes_inside_the_loop(x: Tensor, w: Tensor):
    outs: List[Tensor] = []
    for i in range(x.size(0)):
        scale = float(w.size(0) * 2 + x.size(1))       # the same in every iteration
        outs.append(x[i] * scale + w[i % w.size(0)])
    return outs


def if_in_loop(x: Tensor):
    y = torch.zeros_like(x)
    for i in range(x.size(0)):
        if i % 2 == 0:
            y[i] = x[i].sigmoid()
        else:
            y[i] = x[i] * 3
    return y


def one_sided_if(a: Tensor, k: int):
    a = a.clone()
    v = a[2]
    if k > 0:
        v += 1.5
    return a * 2 + v


def if_with_two_results(x: Tensor, flag: bool):
    x = x.clone()
    if flag:
        x[0] = x[1] * 2.0
        y = x.exp()
    else:
        x[1] = x[0] - 1.0
        y = x.tanh()
    return x + 1.0, y * x


# --- graphs ---------------------------------------------------------------------------------------
def test_spellings_are_rewritten():
    x, y = torch.rand(3, 4), torch.rand(3, 4)
    g = _canon(spellings, (x, y))
    kinds = _kinds(g)
    for gone in ("aten::new_zeros", "aten::new_ones", "aten::pow", "aten::t", "aten::view"):
        assert gone not in kinds, gone
    assert "aten::maximum" in kinds and "aten::minimum" in kinds and "aten::max" not in kinds
    assert kinds.count("aten::transpose") == 2 and kinds.count("aten::reshape") == 2
    assert "aten::zeros" in kinds and "aten::ones" in kinds
    # x.pow(2): 1 product, y.pow(3): 2, pow(5): 3
    assert kinds.count("aten::mul") == 1 + 2 + 3 + 1
    ar = [n for n in g.nodes() if n.kind() == "aten::arange"][0]
    assert len(list(ar.inputs())) == 6 and list(ar.inputs())[0].toIValue() == 0
    # the graph still computes the same
    f = torch._C._create_function_from_graph("f", g)
    assert torch.allclose(f(x, y), spellings(x, y), rtol=1e-6)


def test_new_zeros_takes_the_dtype_from_the_type():
    i = torch.arange(5)
    g = _canon(integer_spellings, (i,))
    z = [n for n in g.nodes() if n.kind() == "aten::zeros"][0]
    assert list(z.inputs())[1].toIValue() == 4   # ScalarType Long, a constant: the region is compiled for it
    f = torch._C._create_function_from_graph("f", g)
    assert torch.equal(f(i), integer_spellings(i))
    # without a static type the dtype is computed at run time, and such an operator stays outside regions
    g = _canon(integer_spellings)
    assert "prim::dtype" in _kinds(g)


def test_slice_with_a_step_and_pow_one_are_left_alone():
    def f(x: Tensor):
        return x[::2] + x[:, :][0:1].pow(1)

    kinds = _kinds(_canon(f))
    assert kinds.count("aten::slice") == 2 and "aten::pow" in kinds


def test_loop_invariants_move_in_front_of_the_loop():
    g = torch.jit.script(sizes_inside_the_loop).graph.copy()
    loop = [n for n in g.nodes() if n.kind() == "prim::Loop"][0]
    inside_before = _kinds(next(loop.blocks()))
    assert inside_before.count("aten::size") >= 2
    assert _C._jit_pass_hoist_loop_invariants(g)
    loop = [n for n in g.nodes() if n.kind() == "prim::Loop"][0]
    inside = _kinds(next(loop.blocks()))
    assert "aten::size" not in inside and "aten::Float" not in inside
    assert "aten::remainder" in inside      # depends on i (and may divide by zero): stays
    f = torch._C._create_function_from_graph("f", g)
    x, w = torch.rand(5, 3), torch.rand(2, 3)
    for a, b in zip(f(x, w), sizes_inside_the_loop(x, w)):
        assert torch.equal(a, b)
    assert not _C._jit_pass_hoist_loop_invariants(g)


def test_the_pipeline_runs_both():
    x, y = torch.rand(3, 4), torch.rand(3, 4)
    built = fj.build(fj.script(spellings), [x, y])
    kinds = _all_kinds(built.graph)
    assert "aten::pow" not in kinds and "aten::new_zeros" not in kinds and "aten::maximum" in kinds


def test_regions_form_inside_if_blocks():
    built = fj.build(fj.script(if_with_two_results), [torch.rand(4, 3), True])
    ifs = [n for n in built.graph.nodes() if n.kind() == "prim::If"]
    assert len(ifs) == 1
    for b in ifs[0].blocks():
        assert [n.kind() for n in b.nodes() if n.kind() != "prim::Constant"] == ["tssa::ParallelFunctor"]


# --- GPU parity -------------------------------------------------------------------------------------
def _run(fn, args):
    built = fj.build(fj.script(fn), list(args))
    dev_args = [a.to("cuda:0") if isinstance(a, torch.Tensor) else a for a in args]
    return built, built(*dev_args)


@pytest.mark.gpu
def test_canonicalized_program_equals_eager():
    g = torch.Generator().manual_seed(1)
    x, y = torch.rand(6, 5, generator=g) + 0.5, torch.rand(6, 5, generator=g) + 0.5
    built, got = _run(spellings, (x, y))
    assert len([n for n in built.graph.nodes() if n.kind() == "tssa::ParallelFunctor"]) >= 1
    assert torch.allclose(got.cpu(), spellings(x, y), rtol=1e-6, atol=0)
    i = torch.arange(7) - 3
    _, got = _run(integer_spellings, (i,))
    assert got.dtype == torch.long and torch.equal(got.cpu(), integer_spellings(i))


@pytest.mark.gpu
def test_hoisted_program_equals_eager():
    g = torch.Generator().manual_seed(2)
    x, w = torch.rand(9, 16, generator=g), torch.rand(4, 16, generator=g)
    built, got = _run(sizes_inside_the_loop, (x, w))
    maps = [n for n in built.graph.nodes() if n.kind() == "tssa::ParallelFunctor" and n.i("is_parallel_map") == 1]
    assert len(maps) == 1                                    # with the sizes outside, the tensor work is one map
    for n in built.graph.nodes():                            # (i % w.size(0), integer work, stays a host loop)
        for b in n.blocks():
            assert "aten::size" not in _kinds(b) and "aten::Float" not in _kinds(b)
    for a, b in zip(got, sizes_inside_the_loop(x, w)):
        assert torch.equal(a.cpu(), b)


@pytest.mark.gpu
@pytest.mark.parametrize("case", ["if_in_loop", "one_sided_if_taken", "one_sided_if_not_taken", "two_results_true",
                                  "two_results_false"])
def test_regions_inside_if_blocks_equal_eager(case):
    g = torch.Generator().manual_seed(3)
    if case == "if_in_loop":
        fn, args = if_in_loop, (torch.rand(7, 33, generator=g),)
    elif case.startswith("one_sided_if"):
        fn, args = one_sided_if, (torch.rand(4, 3, generator=g), 1 if case.endswith("_taken") and "not" not in case else 0)
    else:
        fn, args = if_with_two_results, (torch.rand(5, 40, generator=g), case.endswith("true"))
    want = fn(*[a.clone() if isinstance(a, torch.Tensor) else a for a in args])
    _, got = _run(fn, args)
    want = want if isinstance(want, tuple) else (want,)
    got = got if isinstance(got, tuple) else (got,)
    for a, b in zip(got, want):
        assert torch.allclose(a.cpu(), b, rtol=1e-6, atol=1e-7)
