"""Views made by operators that have no immut:: twin (t, transpose, expand_as, narrow, ...) and
operators that may or may not return a view (flatten, to, contiguous): a write to the buffer must
show through a live view exactly as in eager mode.  The reference takes the alias relation from
AliasDb's element map and re-derives every aliasing value after a write
(functs/csrc/jit/passes/convert_to_tensorssa.cpp:80-103, 186-266); eager PyTorch is the pin."""
import pytest
import torch

import functs_amd.jit as fj


def alias_t(a: torch.Tensor):
    x = a + 0.0
    y = x.t()
    x[0] = x[0] + 1.0
    return y.sum(0), x


def alias_transpose(a: torch.Tensor):
    x = a + 0.0
    y = x.transpose(0, 1)
    x[1] = x[1] * 3.0
    return y + 1.0, x


def alias_expand_as(a: torch.Tensor):
    x = a + 0.0
    y = x[0:1].expand_as(x)
    x[0] = x[0] - 2.0
    return y * 2.0, x


def alias_narrow(a: torch.Tensor):
    x = a + 0.0
    y = x.narrow(0, 0, 1)
    x[0] = x[0] + 5.0
    return y + 0.5, x


def alias_flatten(a: torch.Tensor):
    x = a + 0.0
    y = x.flatten()
    x[0] = x[0] + 1.0
    return y.sum(), x


def alias_to_same_dtype(a: torch.Tensor):
    x = a + 0.0
    y = x.to(torch.float32)          # no conversion: a view of x in eager mode
    x[0] = x[0] + 1.0
    return y.sum(), x


def copy_to_other_dtype(a: torch.Tensor):
    x = a + 0.0
    y = x.to(torch.float64)          # a copy: the later write must NOT show
    x[0] = x[0] + 1.0
    return y.sum(), x


def write_through_t(a: torch.Tensor):
    x = a + 0.0
    y = x.t()
    y[0] = y[0] + 1.0                # writes column 0 of x
    return x * 2.0, y


def view_after_the_last_write(a: torch.Tensor):
    x = a + 0.0
    x[0] = x[0] + 1.0
    y = x.contiguous().flatten()     # nothing is written after it: reads the latest version
    return y * 2.0


def alias_in_loop(a: torch.Tensor, n: int):
    x = a + 0.0
    y = x.t()
    for i in range(n):
        x[i] = x[i] + y[:, i]
    return x, y


PROGRAMS = [alias_t, alias_transpose, alias_expand_as, alias_narrow, alias_flatten, alias_to_same_dtype,
            copy_to_other_dtype, write_through_t, view_after_the_last_write]


def _same(got, ref):
    got = got if isinstance(got, tuple) else (got,)
    ref = ref if isinstance(ref, tuple) else (ref,)
    assert len(got) == len(ref)
    for g, r in zip(got, ref):
        assert g.dtype == r.dtype and torch.equal(g, r)


@pytest.mark.parametrize("add_clone", [False, True])
@pytest.mark.parametrize("fn", PROGRAMS, ids=lambda f: f.__name__)
def test_live_alias_sees_the_write(fn, add_clone):
    a = torch.arange(12, dtype=torch.float32).reshape(4, 3) / 7.0
    ref = fn(a.clone())
    jfn = fj.script(fn, add_clone=add_clone)
    _same(jfn(a.clone()), ref)


@pytest.mark.parametrize("add_clone", [False, True])
def test_alias_read_inside_a_loop(add_clone):
    a = torch.arange(16, dtype=torch.float32).reshape(4, 4) / 5.0
    ref = alias_in_loop(a.clone(), 4)
    _same(fj.script(alias_in_loop, add_clone=add_clone)(a.clone(), 4), ref)


def test_plain_views_are_rederived_not_left_stale():
    g = fj.script(alias_t).graph
    s = str(g)
    assert "immut::select_rev" in s          # the write was functionalized ...
    assert s.count("aten::t(") >= 1          # ... and the transposed view is taken from the new version
    t_nodes = [n for n in g.nodes() if n.kind() == "aten::t"]
    rev = [n for n in g.nodes() if n.kind() == "immut::select_rev"]
    assert any(n.input().node() in rev for n in t_nodes)


def test_write_through_a_plain_view_stays_in_place():
    s = str(fj.script(write_through_t).graph)
    assert "aten::copy_" in s and "immut::" not in s
