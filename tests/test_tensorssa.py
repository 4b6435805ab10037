"""Functionalization (ConvertToTensorSSA) on the CPU: the rewritten script,
run by the stock interpreter with the eager immut:: operators, must return what
the original eager program returns.  The first four programs are the ones of the
reference's own test (test/test_basic.py:6-39)."""
import pytest
import torch

import functs_amd.jit as fj


def branch_loop(a: torch.Tensor, c: torch.Tensor, d: torch.Tensor):
    tmp_0 = d.clone()
    tmp_1 = tmp_0[1]
    if a.nonzero().sum():
        tmp_0 = tmp_0 + 1
        for i in range(10):
            tmp_1.copy_(tmp_0[i + 1])
    else:
        tmp_0 = tmp_0 + tmp_1
        tmp_1.copy_(tmp_0[2])
    return tmp_1 + tmp_0


def dataflow(a: torch.Tensor, b: torch.Tensor):
    a[0].copy_(b[0])
    a[1].copy_(b[1])
    a[0:1] = b[0:1]
    return a + a[0:1]


def loop(a: torch.Tensor, b: torch.Tensor):
    for i in range(10):
        a[i].copy_(b[i + 1])
    return a


def branch(a: torch.Tensor, b: torch.Tensor, cond: int):
    tmp_1 = a[1]
    if cond > 0:
        tmp_1.copy_(b[0])
    else:
        tmp_1.copy_(b[1] * 2)
    return a


def carried(a: torch.Tensor, b: torch.Tensor, n: int):
    a = a.clone()
    for i in range(n):
        b = b + 1
        a[i] = b[i] * 2
    return a


def nested_views(a: torch.Tensor, b: torch.Tensor):
    a = a.clone()
    a[1:3, 0].copy_(b[0:2, 1])
    a[0] += 1
    return a + 1


def if_in_loop(x: torch.Tensor):
    y = torch.zeros_like(x)
    for i in range(x.size(0)):
        if i % 2 == 0:
            y[i] = x[i].sigmoid()
        else:
            y[i] = x[i] * 3
    return y


def one_sided_if(a: torch.Tensor, k: int):
    a = a.clone()
    v = a[2]
    if k > 0:
        v += 1.5
    return a * 2 + v


def view_chain(a: torch.Tensor, b: torch.Tensor):
    t = a.clone()
    u = t.permute(1, 0)
    w = u.unsqueeze(0)
    w[0, 1].copy_(b[:, 0])
    s = t.view(-1)
    s[3:5] = 7.0
    return t + u.permute(1, 0)


def live_views(a: torch.Tensor):
    t = a.clone()
    r0 = t[0]
    r1 = t[1]
    r0.add_(1.0)
    t[1].mul_(r0)
    return r0 + r1 + t[0]


def nested_loops(a: torch.Tensor, b: torch.Tensor):
    t = a.clone()
    for i in range(3):
        for j in range(2):
            t[i, j] = b[j, i] + t[i, j + 1]
    return t


def masked_write(a: torch.Tensor):
    t = a.clone()
    t[t > 0.5] = 0.0
    return t


PROGRAMS = [
    (branch_loop, lambda g: (torch.rand(16, 16, generator=g), torch.rand(16, 16, generator=g), torch.rand(16, 16, generator=g))),
    (branch_loop, lambda g: (torch.zeros(16, 16), torch.rand(16, 16, generator=g), torch.rand(16, 16, generator=g))),
    (dataflow, lambda g: (torch.rand(16, 16, generator=g), torch.rand(16, 16, generator=g))),
    (loop, lambda g: (torch.rand(16, 16, generator=g), torch.rand(16, 16, generator=g))),
    (branch, lambda g: (torch.rand(16, 16, generator=g), torch.rand(16, 16, generator=g), 1)),
    (branch, lambda g: (torch.rand(16, 16, generator=g), torch.rand(16, 16, generator=g), -1)),
    (carried, lambda g: (torch.rand(6, 5, generator=g), torch.rand(6, 5, generator=g), 6)),
    (carried, lambda g: (torch.rand(6, 5, generator=g), torch.rand(6, 5, generator=g), 0)),
    (nested_views, lambda g: (torch.rand(4, 3, generator=g), torch.rand(4, 3, generator=g))),
    (if_in_loop, lambda g: (torch.rand(5, 3, generator=g),)),
    (one_sided_if, lambda g: (torch.rand(4, 3, generator=g), 1)),
    (one_sided_if, lambda g: (torch.rand(4, 3, generator=g), 0)),
    (view_chain, lambda g: (torch.rand(4, 3, generator=g), torch.rand(4, 3, generator=g))),
    (live_views, lambda g: (torch.rand(4, 3, generator=g),)),
    (nested_loops, lambda g: (torch.rand(4, 4, generator=g), torch.rand(4, 4, generator=g))),
    (masked_write, lambda g: (torch.rand(4, 4, generator=g),)),
]

_IDS = ["%s-%d" % (p[0].__name__, i) for i, p in enumerate(PROGRAMS)]


def _clone(args):
    return [a.clone() if isinstance(a, torch.Tensor) else a for a in args]


def _kinds(block, out):
    for n in block.nodes():
        out.append(n.kind())
        for b in n.blocks():
            _kinds(b, out)
    return out


@pytest.mark.parametrize("fn,make", PROGRAMS, ids=_IDS)
@pytest.mark.parametrize("add_clone", [False, True])
def test_functionalized_script_matches_eager(fn, make, add_clone):
    gen = torch.Generator().manual_seed(1234)
    args = make(gen)
    want = fn(*_clone(args))
    jit_fn = fj.script(fn, add_clone=add_clone)
    got = jit_fn(*_clone(args))
    assert torch.equal(got, want)
    kinds = _kinds(jit_fn.graph, [])
    assert "tssa::update" not in kinds and "immut::assign" not in kinds


@pytest.mark.parametrize("fn,make", PROGRAMS, ids=_IDS)
def test_owned_buffers_are_fully_functionalized(fn, make):
    """With the arguments cloned on entry every mutated buffer is owned by the
    body, so no in-place operator may survive (masked_write keeps its
    index_put_: mask writes fall back to ATen, convert_to_tensorssa.cpp:422-443)."""
    jit_fn = fj.script(fn, add_clone=True)
    kinds = _kinds(jit_fn.graph, [])
    leftovers = [k for k in kinds if k.startswith("aten::") and k.endswith("_") and k != "aten::index_put_"]
    assert not leftovers, leftovers
    if fn is not masked_write:
        assert any(k.startswith("immut::") for k in kinds)


def test_arguments_are_not_written_when_cloned():
    gen = torch.Generator().manual_seed(7)
    a, b = torch.rand(16, 16, generator=gen), torch.rand(16, 16, generator=gen)
    a0 = a.clone()
    fj.script(loop, add_clone=True)(a, b)
    assert torch.equal(a, a0)


def test_update_nodes_survive_on_request():
    jit_fn = fj.script(carried, remove_update=False, enable_dce_cse=False)
    kinds = _kinds(jit_fn.graph, [])
    assert "tssa::update" in kinds and "immut::select_rev" in kinds


def test_loop_carries_the_mutated_buffer():
    """The version written inside the loop becomes a loop-carried value
    (block propagation, convert_to_tensorssa.cpp:322-364)."""
    jit_fn = fj.script(carried)
    loops = [n for n in jit_fn.graph.nodes() if n.kind() == "prim::Loop"]
    assert len(loops) == 1
    body = next(loops[0].blocks())
    ret = list(body.outputs())
    assert any(v.node().kind() == "immut::select_rev" for v in ret)


def test_registered_but_unused_rev_operators():
    """immut::expand_rev / repeat_rev / expand_as_rev are registered by the reference
    (functs/csrc/jit/ir/symbol_ext.cpp:83-111) and emitted by none of its passes; the bodies
    give the reference's results without touching `self`."""
    x = torch.arange(6.0).reshape(2, 3)
    assert torch.equal(torch.ops.immut.expand_rev(x[:1], [2, 3]), x[:1].expand(2, 3))
    keep = x.clone()
    out = torch.ops.immut.repeat_rev(x, torch.ones(4, 3), [2, 1])
    assert torch.equal(out, keep) and torch.equal(x, keep) and out.data_ptr() != x.data_ptr()
    src = torch.full((3,), 7.0)
    out = torch.ops.immut.expand_as_rev(x, src, torch.zeros(2, 3))
    assert torch.equal(out, src.expand(2, 3)) and torch.equal(x, keep)
    with pytest.raises(RuntimeError, match="single memory location"):
        torch.ops.immut.expand_as_rev(x[:1], torch.ones(2, 3), torch.zeros(2, 3))
