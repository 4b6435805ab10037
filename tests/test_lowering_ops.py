"""Per-operator parity of fused regions with stock PyTorch.

Mirrors the reference's operator suite (fait/testing/test_lowering.cpp:182-231
over fait/testing/lowering_tests.json, kept as tests/golden/lowering_tests.json)
and its NNC lowering tests (test/test_immut_tensorexpr.py:10-96): build a region
holding the single operator, run it, compare with the same ATen call on the
same random inputs.  Indexing / assignment results must be bit-exact; fp32
arithmetic within 1e-5 relative.

Every test runs twice: on the CPU bytecode emulator (checks shape functions
and lowering without a GPU) and, marked `gpu`, through the C ABI on cuda:0.
"""
import itertools
import json
import os

import pytest
import torch

from functs_amd import Region
from tests.util import assert_close, assert_exact, run_region

HERE = os.path.dirname(os.path.abspath(__file__))
SUITE = json.load(open(os.path.join(HERE, "golden", "lowering_tests.json")))

_DT = {"Float": torch.float32, "Long": torch.int64, "Bool": torch.bool}
_CODE = {4: torch.int64, 6: torch.float32, 11: torch.bool, 3: torch.int32}  # c10::ScalarType numbering


def gen(spec, g):
    """Random input like generateInput (test_lowering.cpp:148-180)."""
    dt = _DT[spec["dtype"]]
    if dt == torch.float32:
        return torch.rand(spec["shape"], generator=g)
    if dt == torch.int64:
        return torch.randint(0, 5, spec["shape"], generator=g)
    return torch.randint(0, 2, spec["shape"], generator=g).bool()


def is_spec(x):
    return isinstance(x, dict) and "shape" in x


class Case:
    """Builds region + reference for one JSON case."""

    def __init__(self, name, args, kwargs):
        self.name, self.args, self.kwargs = name, args, kwargs
        g = torch.Generator().manual_seed(1234)
        self.tensors = []
        self.region = Region()
        self.vals = []  # region values for tensor args, same order as self.tensors

        def conv(a):
            if is_spec(a):
                t = gen(a, g)
                self.tensors.append(t)
                v = self.region.tensor_input(t.dtype, t.dim())
                self.vals.append(v)
                return ("T", len(self.tensors) - 1)
            if isinstance(a, list) and a and is_spec(a[0]):
                return ("L", [conv(x)[1] for x in a])
            return ("S", a)

        self.conv = [conv(a) for a in args]

    def T(self, i):
        kind, idx = self.conv[i]
        assert kind == "T"
        return self.tensors[idx], self.vals[idx]

    def S(self, i, default=None):
        if i >= len(self.conv):
            return default
        return self.conv[i][1]


def build(name, case):
    r = case.region
    kw = case.kwargs
    if name == "tensor":
        v = r.op("SCALAR_TENSOR", case.S(0), dtype=torch.int64)
        return v, torch.tensor(case.S(0))
    if name == "zeros":
        dt = _CODE[kw["dtype"]]
        return r.zeros(case.S(0), dt), torch.zeros(case.S(0), dtype=dt)
    if name == "arange":
        dt = _CODE[kw["dtype"]]
        return r.arange(case.S(0), case.S(1), dt), torch.arange(case.S(0), case.S(1), dtype=dt)
    if name == "to":
        t, v = case.T(0)
        dt = _CODE[case.S(2)]
        return v.to(dt), t.to(dt)
    if name == "triu":
        t, v = case.T(0)
        return r.op("TRIU", v, case.S(1)), torch.triu(t, case.S(1))
    if name in ("add_tensor", "maximum", "minimum"):
        (a, va), (b, vb) = case.T(0), case.T(1)
        op = {"add_tensor": "ADD", "maximum": "MAXIMUM", "minimum": "MINIMUM"}[name]
        fn = {"add_tensor": torch.add, "maximum": torch.maximum, "minimum": torch.minimum}[name]
        return r.op(op, va, vb), fn(a, b)
    if name == "add_scalar":
        t, v = case.T(0)
        return r.op("ADD", v, case.S(1)), t + case.S(1)
    if name == "max":
        t, v = case.T(0)
        keep = bool(case.S(2, False))
        return r.op("MAX_DIM", v, case.S(1), keep), torch.max(t, case.S(1), keep)[0]
    if name == "softmax":
        t, v = case.T(0)
        return v.softmax(case.S(1)), torch.softmax(t, case.S(1))
    if name == "select":
        t, v = case.T(0)
        return v.select(case.S(1), case.S(2)), t.select(case.S(1), case.S(2))
    if name == "slice":
        t, v = case.T(0)
        dim, start, end, step = case.S(1), case.S(2), case.S(3), case.S(4, 1)
        return v.slice(dim, start, end, step), torch.ops.aten.slice(t, dim, start, end, step)
    if name == "unsqueeze":
        t, v = case.T(0)
        return v.unsqueeze(case.S(1)), t.unsqueeze(case.S(1))
    if name == "reshape":
        t, v = case.T(0)
        return v.view(case.S(1)), t.reshape(case.S(1))
    if name == "permute":
        t, v = case.T(0)
        return v.permute(case.S(1)), t.permute(case.S(1))
    if name == "expand":
        t, v = case.T(0)
        return v.expand(case.S(1)), t.expand(case.S(1))
    if name == "expand_as":
        (a, va), (b, vb) = case.T(0), case.T(1)
        return va.expand_as(vb), a.expand_as(b)
    if name == "repeat":
        t, v = case.T(0)
        reps = list(case.S(1))
        # repeats shorter than the rank: ATen refuses, the reference's shape function
        # (shape_func.cpp:206-230) pads with leading ones - follow the reference
        full = [1] * max(t.dim() - len(reps), 0) + reps
        return v.repeat(reps), t.repeat(full)
    if name == "index":
        t, v = case.T(0)
        idx_i = case.conv[1][1][0]
        return v.index(case.vals[idx_i]), t[case.tensors[idx_i]]
    if name in ("cat", "stack"):
        ids = case.conv[0][1]
        ts = [case.tensors[i] for i in ids]
        vs = [case.vals[i] for i in ids]
        if name == "cat":
            return r.cat(vs, case.S(1)), torch.cat(ts, case.S(1))
        return r.stack(vs, case.S(1)), torch.stack(ts, case.S(1))
    raise KeyError(name)


EXACT = {"tensor", "zeros", "arange", "to", "triu", "maximum", "minimum", "max", "select", "slice", "unsqueeze",
         "reshape", "permute", "expand", "expand_as", "repeat", "index", "cat", "stack", "add_tensor", "add_scalar"}

ALL_CASES = [(name, i) for name, suite in SUITE.items() for i in range(len(suite["cases"]))]


@pytest.mark.parametrize("name,idx", ALL_CASES, ids=["%s-%d" % c for c in ALL_CASES])
def test_reference_op_suite(backend, name, idx):
    args, kwargs = SUITE[name]["cases"][idx]
    case = Case(name, args, kwargs)
    out_val, ref = build(name, case)
    case.region.output(out_val)
    case.region.finalize()
    (got,) = run_region(backend, case.region, *case.tensors)
    ref = ref.contiguous()
    if name in EXACT:
        assert_exact(got, ref, name)
    else:
        assert_close(got, ref, name)
        if name == "softmax":  # closed form: rows sum to one
            assert torch.allclose(got.sum(-1), torch.ones(got.shape[0]), atol=1e-6)


# ---------------------------------------------------------------------------
# test/test_immut_tensorexpr.py cases: scalar arguments arrive at run time
# ---------------------------------------------------------------------------


def test_immut_select_runtime_index(backend):
    r = Region()
    x = r.tensor_input(torch.float32, 2)
    i = r.scalar_input("int")
    r.output(x.select(0, i))
    r.finalize()
    t = torch.rand(10, 20)
    for idx in (0, 3, 9):
        (got,) = run_region(backend, r, t, idx)
        assert_exact(got, t.select(0, idx))


def test_immut_select_rev(backend):
    r = Region()
    x = r.tensor_input(torch.float32, 2)
    s = r.tensor_input(torch.float32, 1)
    i = r.scalar_input("int")
    r.output(x.select_rev(s, 1, i))
    r.finalize()
    t, src = torch.rand(3000, 4), torch.rand(3000)
    for idx in (0, 2, 3):
        (got,) = run_region(backend, r, t, src, idx)
        ref = t.clone()
        ref.select(1, idx).copy_(src)
        assert_exact(got, ref)


def test_immut_slice_runtime_bounds(backend):
    r = Region()
    x = r.tensor_input(torch.float32, 2)
    a, b, c = r.scalar_input("int"), r.scalar_input("int"), r.scalar_input("int")
    r.output(x.slice(1, a, b, c))
    r.finalize()
    t = torch.rand(3000, 4)
    (got,) = run_region(backend, r, t, 0, 3, 4)
    assert_exact(got, t[:, 0:3:4])
    assert got.shape == (3000, 1)


def test_immut_slice_rev(backend):
    r = Region()
    x = r.tensor_input(torch.float32, 2)
    s = r.tensor_input(torch.float32, 2)
    a, b, c = r.scalar_input("int"), r.scalar_input("int"), r.scalar_input("int")
    r.output(x.slice_rev(s, 1, a, b, c))
    r.finalize()
    t, src = torch.rand(3000, 4), torch.rand(3000, 1)
    (got,) = run_region(backend, r, t, src, 0, 3, 4)
    ref = t.clone()
    ref[:, 0:3:4] = src
    assert_exact(got, ref)


def test_immut_unsqueeze(backend):
    r = Region()
    x = r.tensor_input(torch.float32, 2)
    r.output(x.unsqueeze(0))
    r.finalize()
    t = torch.rand(3000, 4)
    (got,) = run_region(backend, r, t)
    assert_exact(got, t.unsqueeze(0))


# ---------------------------------------------------------------------------
# brute force over the index arithmetic of select / slice and their *_rev
# (tiny shapes, every dim / index / bound incl. negative, None, out of range)
# ---------------------------------------------------------------------------
SHAPE = (3, 4, 5)


def _select_cases():
    for dim in range(-3, 3):
        n = SHAPE[dim]
        for idx in range(-n, n):
            yield dim, idx


def test_select_and_select_rev_bruteforce(backend):
    g = torch.Generator().manual_seed(7)
    t = torch.rand(SHAPE, generator=g)
    # one region with every case as an output keeps the GPU round trips low
    r = Region()
    x = r.tensor_input(torch.float32, 3)
    srcs, refs = [], []
    for dim, idx in _select_cases():
        r.output(x.select(dim, idx))
        refs.append(t.select(dim, idx).contiguous())
    rev_cases = list(_select_cases())[::3]
    src_vals = []
    for dim, idx in rev_cases:
        s = torch.rand(t.select(dim, idx).shape, generator=g)
        srcs.append(s)
        sv = r.tensor_input(torch.float32, 2)
        src_vals.append(sv)
        r.output(x.select_rev(sv, dim, idx))
        ref = t.clone()
        ref.select(dim, idx).copy_(s)
        refs.append(ref)
    r.finalize()
    got = run_region(backend, r, t, *srcs)
    assert_exact(got, refs)


def _slice_cases():
    bounds = [None, 0, 1, 2, 3, 7, -1, -2, -9]
    for dim in (0, 1, 2, -1):
        for start, end in itertools.product(bounds, bounds):
            for step in (1, 2, 3):
                yield dim, start, end, step


def test_slice_bruteforce(backend):
    t = torch.rand(SHAPE, generator=torch.Generator().manual_seed(8))
    cases = list(_slice_cases())
    # chunks of 64 outputs per region (pointer-slot budget)
    for k in range(0, len(cases), 64):
        r = Region()
        x = r.tensor_input(torch.float32, 3)
        refs = []
        for dim, start, end, step in cases[k:k + 64]:
            r.output(x.slice(dim, start, end, step))
            refs.append(torch.ops.aten.slice(t, dim, start, end, step).contiguous())
        r.finalize()
        assert_exact(run_region(backend, r, t), refs, "slice chunk %d" % k)


def test_slice_rev_bruteforce(backend):
    g = torch.Generator().manual_seed(9)
    t = torch.rand(SHAPE, generator=g)
    cases = [c for i, c in enumerate(_slice_cases()) if i % 5 == 0]
    for k in range(0, len(cases), 24):
        r = Region()
        x = r.tensor_input(torch.float32, 3)
        refs, srcs = [], []
        for dim, start, end, step in cases[k:k + 24]:
            view = torch.ops.aten.slice(t, dim, start, end, step)
            s = torch.rand(view.shape, generator=g)
            srcs.append(s)
            sv = r.tensor_input(torch.float32, 3)
            r.output(x.slice_rev(sv, dim, start, end, step))
            ref = t.clone()
            torch.ops.aten.slice(ref, dim, start, end, step).copy_(s)
            refs.append(ref)
        r.finalize()
        assert_exact(run_region(backend, r, t, *srcs), refs, "slice_rev chunk %d" % k)


# ---------------------------------------------------------------------------
# chains: assignments through views of views, as functionalization emits them
# ---------------------------------------------------------------------------


def test_assign_chain_normalize(backend):
    """examples/kernel_fusion.py:6-16 (README.md:484-507): two select assigns
    swapping channels, then (dup - mean) * scale with run-time float scalars."""
    r = Region()
    src = r.tensor_input(torch.float32, 3)
    mean, scale = r.scalar_input("float"), r.scalar_input("float")
    dup = src.clone()
    dup = dup.select_rev(src.select(2, 2), 2, 0)
    dup = dup.select_rev(src.select(2, 0), 2, 2)
    r.output((dup - mean) * scale)
    r.finalize()
    t = torch.rand(37, 53, 3, generator=torch.Generator().manual_seed(3))
    (got,) = run_region(backend, r, t, 0.25, 1.5)
    ref = t.clone()
    ref[..., 0] = t[..., 2]
    ref[..., 2] = t[..., 0]
    ref = (ref - 0.25) * 1.5
    assert_exact(got, ref)  # sub and mul round identically on both sides


def test_view_of_permute_gather(backend):
    """pred.permute(0,2,3,1).reshape(n,-1,C) (yolov3_bbox.py:209-211): a reshape
    that splits dimensions needs div/mod index code."""
    r = Region()
    x = r.tensor_input(torch.float32, 4)
    r.output(x.permute(0, 2, 3, 1).view(1, -1, 5).sigmoid())
    r.finalize()
    t = torch.randn(1, 15, 3, 4, generator=torch.Generator().manual_seed(4))
    (got,) = run_region(backend, r, t)
    assert_close(got, t.permute(0, 2, 3, 1).reshape(1, -1, 5).sigmoid())


def test_where_clamp_compare(backend):
    r = Region()
    a, b = r.tensor_input(torch.float32, 2), r.tensor_input(torch.float32, 2)
    r.output(r.where(a > b, a.clamp(0.25, 0.75), b * 2.0))
    r.output((a >= 0.5) & (b < 0.5))
    r.finalize()
    g = torch.Generator().manual_seed(5)
    ta, tb = torch.rand(33, 65, generator=g), torch.rand(33, 65, generator=g)
    got = run_region(backend, r, ta, tb)
    assert_exact(got, [torch.where(ta > tb, ta.clamp(0.25, 0.75), tb * 2.0), (ta >= 0.5) & (tb < 0.5)])


@pytest.mark.parametrize("shape", [(0, 4), (1, 1), (63,), (65, 3), (1025,), (257, 9)])
def test_ragged_and_empty_shapes(backend, shape):
    r = Region()
    x = r.tensor_input(torch.float32, len(shape))
    r.output(x * 2.0 + 1.0)
    r.finalize()
    t = torch.rand(shape, generator=torch.Generator().manual_seed(6))
    (got,) = run_region(backend, r, t)
    assert_exact(got, t * 2.0 + 1.0)


def test_strided_input_needs_no_copy(backend):
    """Non-contiguous inputs are read in place (the reference copies them,
    graph_builder.cpp:742-745)."""
    r = Region()
    x = r.tensor_input(torch.float32, 2)
    r.output(x + 1.0)
    r.finalize()
    t = torch.rand(40, 30, generator=torch.Generator().manual_seed(2)).t()[::2]
    assert not t.is_contiguous()
    (got,) = run_region(backend, r, t)
    assert_exact(got, t + 1.0)


def test_int_and_bool_dtypes(backend):
    r = Region()
    a = r.tensor_input(torch.int64, 2)
    b = r.tensor_input(torch.bool, 2)
    r.output(a + 3)
    r.output(a * a - 1)
    r.output(r.op("LOGICAL_NOT", b))
    r.output(a.to(torch.float32) * 0.5)
    r.finalize()
    g = torch.Generator().manual_seed(11)
    ta = torch.randint(-50, 50, (17, 9), generator=g)
    tb = torch.randint(0, 2, (17, 9), generator=g).bool()
    got = run_region(backend, r, ta, tb)
    assert_exact(got, [ta + 3, ta * ta - 1, ~tb, ta.to(torch.float32) * 0.5])


def test_tril_and_triu_over_every_diagonal(backend):
    """aten::tril / aten::triu are both fusable in the reference (fait/passes/fuse_ops.cpp:57-58);
    the library routine is the pin: every diagonal of a non-square matrix, batched."""
    t = (torch.arange(2 * 5 * 7, dtype=torch.float32) + 1).reshape(2, 5, 7)
    diags = list(range(-6, 9))
    r = Region()
    x = r.tensor_input(torch.float32, 3)
    for d in diags:
        r.output(r.op("TRIL", x, d))
        r.output(r.op("TRIU", x, d))
    r.finalize()
    got = run_region(backend, r, t)
    refs = []
    for d in diags:
        refs += [torch.tril(t, d), torch.triu(t, d)]
    assert_exact(got, refs, "tril/triu")


def test_transcendentals_at_the_ends_of_the_range(backend):
    """sigmoid / tanh / exp where exp overflows or underflows, at the infinities and at NaN: the
    eager kernels the reference runs there (ATen) return 0, 1, +-1, inf, NaN, never a NaN made on
    the way."""
    r = Region()
    x = r.tensor_input(torch.float32, 1)
    r.output(x.sigmoid())
    r.output(x.tanh())
    r.output(x.exp())
    r.finalize()
    t = torch.tensor([float("-inf"), -1e30, -200.0, -104.0, -100.0, -90.0, -88.8, -88.0, -20.0, -0.0, 0.0, 20.0, 88.0,
                      88.8, 100.0, 200.0, 1e30, float("inf"), float("nan")] * 7)
    sig, tanh, exp = run_region(backend, r, t)
    for got, ref in ((sig, t.sigmoid()), (tanh, t.tanh()), (exp, t.exp())):
        torch.testing.assert_close(got, ref, rtol=1e-5, atol=1e-37, equal_nan=True)
