"""How a built function is called and what it hands back (functs_amd/jit.py, functs_amd._C):
a graph that is one tssa::ParallelFunctor runs without the TorchScript interpreter
(DirectFunctor); List[Tensor] results may stay the operator's lists (lazy_lists); compacted
results may come back padded with their counts and without a wait (padded_outputs).
Reference contract: GraphBuilder::runKernel allocates, launches and pushes, nothing else
(fait/fuser/graph_builder.cpp:901-927); the reference always goes through the interpreter and
always returns sized lists.

CPU: which graphs take which form.  GPU: every form returns what the plain form returns."""
import pytest
import torch

import functs_amd.jit as fj
from functs_amd import _C
from functs_amd.benchmark import PROGRAMS
from functs_amd.benchmark.inputs import INPUTS


def _cuda(args):
    return [a.cuda() if isinstance(a, torch.Tensor) else a for a in args]


# ---- CPU ----------------------------------------------------------------------------------------
def test_a_single_functor_graph_is_called_directly_and_others_through_the_interpreter():
    for name, small in (("c2", dict(grids=[2, 3, 4])), ("c5", dict(grids=[2, 3, 4], batch=3)), ("c1", dict(size=16, n=8))):
        args = INPUTS[name](0, **small)
        fn = fj.build(fj.script(PROGRAMS[name]), list(args))
        assert type(fn._call).__name__ == "DirectFunctor", name
    args = INPUTS["yolo_head"](0, batch=2, grids=(2, 4, 8))
    fn = fj.build(fj.script(PROGRAMS["yolo_head"]), list(args))
    assert _C._direct_functor(fn.graph) is None and isinstance(fn._call, torch.jit.ScriptFunction)
    with pytest.raises(ValueError, match="one fused region"):
        fj.build(fj.script(PROGRAMS["yolo_head"]), list(args), lazy_lists=True)


def test_wrong_argument_count_is_an_error_of_the_direct_call():
    args = INPUTS["c2"](0, grids=[2, 3, 4])
    fn = fj.build(fj.script(PROGRAMS["c2"]), list(args))
    with pytest.raises(RuntimeError, match="expected 3 arguments"):
        fn._call(args[0])


def test_padded_outputs_retype_the_functor_and_append_the_counts():
    args = INPUTS["c5"](0, grids=[2, 3, 4], batch=3)
    fn = fj.build(fj.script(PROGRAMS["c5"]), list(args), padded_outputs=True)
    f = [n for n in fn.graph.nodes() if n.kind() == "tssa::ParallelFunctor"]
    assert len(f) == 1 and f[0].i("padded_outputs") == 1 and len(list(f[0].outputs())) == 4
    ret = list(fn.graph.outputs())[0]
    assert ret.node().kind() == "prim::TupleConstruct" and len(list(ret.node().inputs())) == 4
    assert str(ret.type()) == "Tuple[Tensor, Tensor, Tensor, Tensor]"
    # a region without compaction is left alone
    args = INPUTS["c1"](0, size=16, n=8)
    fn = fj.build(fj.script(PROGRAMS["c1"]), list(args), padded_outputs=True)
    assert all(not n.hasAttribute("padded_outputs") for n in fn.graph.nodes() if n.kind() == "tssa::ParallelFunctor")


def test_tensor_list_is_a_sequence_of_the_tensors_it_holds():
    ts = [torch.full((2,), float(i)) for i in range(5)]
    g = _C._tensor_list(ts)
    assert len(g) == 5 and "5 tensors" in repr(g)
    assert [float(t[0]) for t in g] == [0.0, 1.0, 2.0, 3.0, 4.0]
    assert g[0].data_ptr() == ts[0].data_ptr() and g[-1].data_ptr() == ts[4].data_ptr()     # the tensors themselves, not copies
    assert isinstance(g[1:3], list) and [float(t[0]) for t in g[1:3]] == [1.0, 2.0] and isinstance(g.tolist(), list)
    for bad in (5, -6):
        with pytest.raises(IndexError):
            g[bad]


# ---- GPU ----------------------------------------------------------------------------------------
def _flat(res):
    out = []
    for r in res if isinstance(res, tuple) else (res,):
        out += list(r) if not isinstance(r, torch.Tensor) else [r]
    return out


@pytest.mark.gpu
@pytest.mark.parametrize("name,small", [("c1", dict(size=64, n=40)), ("c2", dict(grids=[4, 6, 8])), ("c3", dict(n_priors=500, n_cls=9)),
                                        ("c5", dict(grids=[4, 6, 8], batch=5))])
def test_the_direct_call_returns_what_the_interpreter_returns(name, small):
    args = INPUTS[name](1, **small)
    fn = fj.build(fj.script(PROGRAMS[name]), list(args))
    assert type(fn._call).__name__ == "DirectFunctor"
    gargs = _cuda(args)
    print("direct call", name, flush=True)
    a, b = _flat(fn(*gargs)), _flat(fn._aot_script_fn(*gargs))
    assert len(a) == len(b) and all(x.shape == y.shape and torch.equal(x, y) for x, y in zip(a, b))
    # results of an earlier call are not touched by a later one (the next call's memory is
    # allocated ahead, never shared)
    keep = [t.clone() for t in a]
    other = [x.clone() if isinstance(x, torch.Tensor) else x for x in gargs]
    other[0] = other[0].roll(1, 0) if name == "c1" else other[0] * 0.5
    fn(*other)
    fn(*other)
    torch.cuda.synchronize()
    assert all(torch.equal(x, y) for x, y in zip(a, keep))


@pytest.mark.gpu
@pytest.mark.parametrize("name,small", [("c2", dict(grids=[4, 6, 8])), ("c5", dict(grids=[4, 6, 8], batch=5)), ("c3", dict(n_priors=500, n_cls=9))])
def test_kept_row_counts_waited_for_in_the_stream_give_the_same_results(name, small):
    """With a polling budget of 0 the operator does not look for the counts from the host at all:
    it blocks in the stream's synchronisation and finds them afterwards."""
    from functs_amd import _lib
    args = INPUTS[name](4, **small)
    fn = fj.build(fj.script(PROGRAMS[name]), list(args))
    gargs = _cuda(args)
    print("counts from the drained stream", name, flush=True)
    ref = [t.clone() for t in _flat(fn(*gargs))]
    _lib.lib.fx_set_totals_spin_us(0)
    try:
        got = [_flat(fn(*gargs)) for _ in range(3)]
    finally:
        _lib.lib.fx_set_totals_spin_us(2000)
    for g in got:
        assert len(g) == len(ref) and all(x.shape == y.shape and torch.equal(x, y) for x, y in zip(g, ref))


@pytest.mark.gpu
def test_calls_from_two_threads_on_their_own_streams():
    """The direct call keeps the interpreter's lock while it polls for the kept-row counts and makes
    the result lists: two threads calling the same built function get their own results."""
    import threading
    args_a, args_b = INPUTS["c5"](11, grids=[4, 6, 8], batch=5), INPUTS["c5"](12, grids=[4, 6, 8], batch=5)
    fn = fj.build(fj.script(PROGRAMS["c5"]), list(args_a))
    ga, gb = _cuda(args_a), _cuda(args_b)
    ref_a, ref_b = [t.clone() for t in _flat(fn(*ga))], [t.clone() for t in _flat(fn(*gb))]
    torch.cuda.synchronize()
    print("two threads", flush=True)
    bad = []

    def work(gargs, ref, tag):
        stream = torch.cuda.Stream()
        stream.wait_stream(torch.cuda.default_stream())
        with torch.cuda.stream(stream):
            for k in range(100):
                got = _flat(fn(*gargs))
                stream.synchronize()
                if len(got) != len(ref) or not all(x.shape == y.shape and torch.equal(x, y) for x, y in zip(got, ref)):
                    bad.append((tag, k))
                    return

    threads = [threading.Thread(target=work, args=(ga, ref_a, "a")), threading.Thread(target=work, args=(gb, ref_b, "b"))]
    for t in threads:
        t.start()
    for t in threads:
        t.join(timeout=100)
    assert not any(t.is_alive() for t in threads)
    assert not bad, bad


@pytest.mark.gpu
def test_lazy_lists_hold_the_same_tensors():
    args = INPUTS["c5"](2, grids=[4, 6, 8], batch=5)
    plain = fj.build(fj.script(PROGRAMS["c5"]), list(args))
    lazy = fj.build(fj.script(PROGRAMS["c5"]), list(args), lazy_lists=True)
    gargs = _cuda(args)
    ref, got = plain(*gargs), lazy(*gargs)
    assert len(got) == 3 and all(type(g).__name__ == "TensorList" for g in got)
    for r, g in zip(ref, got):
        assert len(g) == len(r) == 5
        assert all(torch.equal(x, y) for x, y in zip(r, g))                  # iteration
        assert all(torch.equal(r[k], g[k]) for k in range(5))                # indexing
        assert torch.equal(g[-1], r[-1]) and torch.equal(g[-5], r[0])
        assert isinstance(g.tolist(), list) and isinstance(g[1:3], list) and len(g[1:3]) == 2
        with pytest.raises(IndexError):
            g[5]
        assert "5 tensors" in repr(g)


@pytest.mark.gpu
@pytest.mark.parametrize("name,small", [("c2", dict(grids=[4, 6, 8])), ("c5", dict(grids=[4, 6, 8], batch=5)), ("c3", dict(n_priors=500, n_cls=9))])
def test_padded_outputs_hold_the_compacted_rows_and_their_counts(name, small):
    args = INPUTS[name](3, **small)
    plain = fj.build(fj.script(PROGRAMS[name]), list(args))
    padded = fj.build(fj.script(PROGRAMS[name]), list(args), padded_outputs=True)
    gargs = _cuda(args)
    print("padded outputs", name, flush=True)
    ref = plain(*gargs)
    got = padded(*gargs)
    counts = got[-1]
    assert counts.dtype == torch.int32 and counts.is_pinned() and not counts.is_cuda
    torch.cuda.synchronize()          # the caller's business: nothing in the call waited
    for r, g in zip(ref, got[:-1]):
        if isinstance(r, torch.Tensor):                       # a single task: the result at full size
            k = int(counts[0])
            assert r.shape[0] == k and g.shape[0] >= k and torch.equal(g[:k], r)
            continue
        assert g.shape[0] == len(r) == counts.numel()
        for t, rt in enumerate(r):
            k = int(counts[t])
            assert rt.shape[0] == k and torch.equal(g[t, :k], rt)
    assert int(counts.sum()) > 0
