"""CollapseRecurrentLoops: the (time, layer) loop nest of a stacked LSTM
(functs/benchmark/ai_model/lstm/lstm.py:79-133) becomes one fx::lstm_stack node inside one
tssa::ParallelFunctor, which runs the persistent kernel.  CPU tests check which graphs are
collapsed and which are left alone; the gpu tests compare the built functions with the oracle
(stock TorchScript on the CPU) on the same inputs at rtol 1e-4 (+ 5e-6 absolute, the rounding
error of a gate's 2 x H products that does not shrink with a result near zero)."""
import ctypes

import pytest
import torch
from torch import Tensor

import functs_amd.jit as fj
from functs_amd import _C
from functs_amd.benchmark import PROGRAMS
from oracle import configs as oc

RTOL = 1e-4
ATOL = 5e-6


def _kinds(block, out=None):
    out = [] if out is None else out
    for n in block.nodes():
        out.append(n.kind())
        for b in n.blocks():
            _kinds(b, out)
    return out


def _functors(graph):
    return [n for n in graph.nodes() if n.kind() == "tssa::ParallelFunctor"]


def _collapsed(built):
    fs = _functors(built.graph)
    return len(fs) == 1 and "fx::lstm_stack" in _kinds(fs[0].g("Subgraph")) and "prim::Loop" not in _kinds(built.graph)


# --- variants of the program ------------------------------------------------------------------
def lstm_with_states(x: Tensor, wih: Tensor, whh: Tensor, bih: Tensor, bhh: Tensor, h0: Tensor, c0: Tensor):
    """Initial states are arguments, operands of the commutative operators the other way round,
    the states updated in the other order, `out` one row longer than the sequence (row T keeps 7)."""
    out = torch.full([x.size(0) + 1, x.size(1), x.size(2)], 7.0, device=x.device)
    state_h = h0.clone()
    state_c = c0.clone()
    for t in range(x.size(0)):
        cur = x[t]
        for j in range(wih.size(0)):
            h = state_h[j]
            c = state_c[j]
            hh = bhh[j] + torch.matmul(h, whh[j])
            ih = bih[j] + torch.matmul(cur, wih[j])
            ingate = torch.sigmoid(hh[0] + ih[0])
            forgetgate = torch.sigmoid(ih[1] + hh[1])
            cellgate = torch.tanh(hh[2] + ih[2])
            outgate = torch.sigmoid(ih[3] + hh[3])
            c2 = (cellgate * ingate) + (c * forgetgate)
            h2 = torch.tanh(c2) * outgate
            state_h[j] = h2
            state_c[j] = c2
            cur = h2
        out[t] = cur
    return out, state_h, state_c


def lstm_first_layer_only(x: Tensor, wih: Tensor, whh: Tensor, bih: Tensor, bhh: Tensor, h0: Tensor, c0: Tensor):
    """Fewer layers than the weights and states hold, fewer steps than x holds: the rest is kept."""
    out = torch.zeros(x.size(0), x.size(1), x.size(2), device=x.device)
    state_h = h0.clone()
    state_c = c0.clone()
    for t in range(x.size(0) - 2):
        cur = x[t]
        for j in range(wih.size(0) - 1):
            ih = torch.matmul(cur, wih[j]) + bih[j]
            hh = torch.matmul(state_h[j], whh[j]) + bhh[j]
            c2 = torch.sigmoid(ih[1] + hh[1]) * state_c[j] + torch.sigmoid(ih[0] + hh[0]) * torch.tanh(ih[2] + hh[2])
            h2 = torch.sigmoid(ih[3] + hh[3]) * torch.tanh(c2)
            state_c[j] = c2
            state_h[j] = h2
            cur = h2
        out[t] = cur
    return out, state_h, state_c


def lstm_with_relu_gate(x: Tensor, wih: Tensor, whh: Tensor, bih: Tensor, bhh: Tensor):
    """Not an LSTM cell (relu in place of the cell gate's tanh): must be left alone."""
    out = torch.zeros(x.size(0), x.size(1), x.size(2), device=x.device)
    state_h = torch.zeros(wih.size(0), x.size(1), x.size(2), device=x.device)
    state_c = torch.zeros(wih.size(0), x.size(1), x.size(2), device=x.device)
    for t in range(x.size(0)):
        cur = x[t]
        for j in range(wih.size(0)):
            ih = torch.matmul(cur, wih[j]) + bih[j]
            hh = torch.matmul(state_h[j], whh[j]) + bhh[j]
            c2 = torch.sigmoid(ih[1] + hh[1]) * state_c[j] + torch.sigmoid(ih[0] + hh[0]) * torch.relu(ih[2] + hh[2])
            h2 = torch.sigmoid(ih[3] + hh[3]) * torch.tanh(c2)
            state_c[j] = c2
            state_h[j] = h2
            cur = h2
        out[t] = cur
    return out, state_h, state_c


def lstm_wrong_gate_order(x: Tensor, wih: Tensor, whh: Tensor, bih: Tensor, bhh: Tensor):
    """Gate 2 where the forget gate (1) belongs: another function, must be left alone."""
    out = torch.zeros(x.size(0), x.size(1), x.size(2), device=x.device)
    state_h = torch.zeros(wih.size(0), x.size(1), x.size(2), device=x.device)
    state_c = torch.zeros(wih.size(0), x.size(1), x.size(2), device=x.device)
    for t in range(x.size(0)):
        cur = x[t]
        for j in range(wih.size(0)):
            ih = torch.matmul(cur, wih[j]) + bih[j]
            hh = torch.matmul(state_h[j], whh[j]) + bhh[j]
            c2 = torch.sigmoid(ih[2] + hh[2]) * state_c[j] + torch.sigmoid(ih[0] + hh[0]) * torch.tanh(ih[1] + hh[1])
            h2 = torch.sigmoid(ih[3] + hh[3]) * torch.tanh(c2)
            state_c[j] = c2
            state_h[j] = h2
            cur = h2
        out[t] = cur
    return out, state_h, state_c


def lstm_reads_the_wrong_state(x: Tensor, wih: Tensor, whh: Tensor, bih: Tensor, bhh: Tensor):
    """The recurrent product reads the cell state instead of the hidden state: left alone."""
    out = torch.zeros(x.size(0), x.size(1), x.size(2), device=x.device)
    state_h = torch.zeros(wih.size(0), x.size(1), x.size(2), device=x.device)
    state_c = torch.zeros(wih.size(0), x.size(1), x.size(2), device=x.device)
    for t in range(x.size(0)):
        cur = x[t]
        for j in range(wih.size(0)):
            ih = torch.matmul(cur, wih[j]) + bih[j]
            hh = torch.matmul(state_c[j], whh[j]) + bhh[j]
            c2 = torch.sigmoid(ih[1] + hh[1]) * state_c[j] + torch.sigmoid(ih[0] + hh[0]) * torch.tanh(ih[2] + hh[2])
            h2 = torch.sigmoid(ih[3] + hh[3]) * torch.tanh(c2)
            state_c[j] = c2
            state_h[j] = h2
            cur = h2
        out[t] = cur
    return out, state_h, state_c


def _states(seed, L, B, H):
    g = torch.Generator().manual_seed(seed + 99)
    return torch.rand(L, B, H, generator=g) * 0.2 - 0.1, torch.rand(L, B, H, generator=g) * 0.2 - 0.1


# --- graphs -----------------------------------------------------------------------------------
def test_the_benchmark_program_becomes_one_functor_around_one_node():
    args = oc.c4_inputs(0)
    built = fj.build(fj.script(PROGRAMS["c4"]), list(args))
    assert _collapsed(built)
    f = _functors(built.graph)[0]
    sub = f.g("Subgraph")
    node = [n for n in sub.nodes() if n.kind() == "fx::lstm_stack"][0]
    ins = list(node.inputs())
    # out, state_h and state_c were zeros that the loops overwrite or start from: no operand, no fill
    assert [i.type().kind() for i in ins[5:8]] == ["NoneType"] * 3
    assert "aten::zeros" not in _kinds(built.graph) and "aten::zeros" not in _kinds(sub)
    assert f.i("parallel_degree") == 1 and f.i("is_parallel_map") == 0
    # 5 tensors; the two trip counts are constants of the static shapes (x.size(0), wih.size(0))
    assert len(list(f.inputs())) == 5 and len(list(f.outputs())) == 3
    assert [i.node().kind() for i in ins[8:10]] == ["prim::Constant"] * 2


def test_a_functionalized_graph_holds_the_node_after_the_pass_alone():
    args = oc.c4_inputs(0, 6, 64, 2, 1)
    g = fj.script(PROGRAMS["c4"]).graph.copy()
    _C._jit_pass_fait_shape_infer(g, [fj.extract_type_hint_from_tensor(a) for a in args], None)
    assert _C._jit_pass_collapse_recurrent_loops(g)
    kinds = _kinds(g)
    assert kinds.count("fx::lstm_stack") == 1 and "prim::Loop" not in kinds
    assert not _C._jit_pass_collapse_recurrent_loops(g)   # nothing left to do


def test_operand_and_update_order_do_not_matter():
    x, wih, whh, bih, bhh = oc.c4_inputs(1, 6, 64, 3, 2)
    h0, c0 = _states(1, 3, 2, 64)
    built = fj.build(fj.script(lstm_with_states), [x, wih, whh, bih, bhh, h0, c0])
    kinds = _kinds(built.graph)
    assert "prim::Loop" not in kinds
    node = [n for f in _functors(built.graph) for n in f.g("Subgraph").nodes() if n.kind() == "fx::lstm_stack"]
    assert len(node) == 1
    # the states are clones of arguments and `out` is longer than the sequence: all three stay operands
    assert [i.type().kind() for i in list(node[0].inputs())[5:8]] == ["TensorType"] * 3


def test_trip_counts_computed_inside_the_time_loop_are_moved_out():
    x, wih, whh, bih, bhh = oc.c4_inputs(4, 9, 64, 3, 1)
    h0, c0 = _states(4, 3, 1, 64)
    args = [x, wih, whh, bih, bhh, h0, c0]
    # the pass alone, on a graph whose size queries are still nodes (the whole pipeline folds them
    # to constants of the static shapes first)
    g = fj.script(lstm_first_layer_only).graph.copy()
    _C._jit_pass_fait_shape_infer(g, [fj.extract_type_hint_from_tensor(a) for a in args], None)
    assert _C._jit_pass_collapse_recurrent_loops(g)
    kinds = _kinds(g)
    assert "prim::Loop" not in kinds and kinds.count("aten::sub") == 2   # T - 2 and L - 1, in front of the node
    assert kinds.index("fx::lstm_stack") > max(i for i, k in enumerate(kinds) if k == "aten::sub")
    built = fj.build(fj.script(lstm_first_layer_only), args)
    kinds = _kinds(built.graph)
    assert "prim::Loop" not in kinds and "aten::sub" not in kinds and len(_functors(built.graph)) == 1


@pytest.mark.parametrize("fn", [lstm_with_relu_gate, lstm_wrong_gate_order, lstm_reads_the_wrong_state])
def test_anything_but_the_lstm_cell_is_left_alone(fn):
    args = oc.c4_inputs(0, 6, 64, 2, 1)
    built = fj.build(fj.script(fn), list(args))
    kinds = _kinds(built.graph)
    assert kinds.count("prim::Loop") == 2
    assert all("fx::lstm_stack" not in _kinds(f.g("Subgraph")) for f in _functors(built.graph))


@pytest.mark.parametrize("seq_len,hidden,layers,batch", [(6, 48, 2, 1), (6, 16, 2, 1), (6, 96, 2, 1), (6, 64, 5, 1), (6, 64, 2, 17),
                                                         (3, 1024, 3, 1)])
def test_shapes_outside_the_kernel_keep_their_loops(seq_len, hidden, layers, batch):
    args = oc.c4_inputs(0, seq_len, hidden, layers, batch)
    built = fj.build(fj.script(PROGRAMS["c4"]), list(args))
    assert _kinds(built.graph).count("prim::Loop") == 2


def test_without_static_shapes_the_loops_stay():
    g = fj.script(PROGRAMS["c4"]).graph.copy()
    assert not _C._jit_pass_collapse_recurrent_loops(g)
    assert _kinds(g).count("prim::Loop") == 2


def test_the_node_refuses_host_tensors():
    """No CPU fallback: the functor of the collapsed loops runs on the GPU only."""
    args = oc.c4_inputs(0, 4, 32, 1, 1)
    built = fj.build(fj.script(PROGRAMS["c4"]), list(args))
    assert _collapsed(built)
    with pytest.raises(RuntimeError, match="GPU only"):
        built(*args)


# --- GPU parity ---------------------------------------------------------------------------------
def _close(got, ref, what):
    for g, r, n in zip(got, ref, ("out", "state_h", "state_c")):
        g = g.cpu()
        assert g.shape == r.shape, (what, n, g.shape, r.shape)
        err = (g.double() - r.double()).abs()
        bad = err > ATOL + RTOL * r.double().abs()
        assert not bool(bad.any()), "%s %s: %d beyond rtol %g (max err %g)" % (what, n, int(bad.sum()), RTOL, err.max())


def _cuda(args):
    return [a.to("cuda:0") for a in args]


@pytest.mark.gpu
@pytest.mark.parametrize("seq_len,hidden,layers,batch", [(64, 512, 2, 1), (7, 32, 1, 1), (9, 128, 3, 4), (12, 512, 4, 2), (5, 1024, 2, 2)])
def test_collapsed_program_equals_the_oracle(seq_len, hidden, layers, batch):
    from functs_amd._lib import lib
    args = oc.c4_inputs(seq_len + hidden, seq_len, hidden, layers, batch)
    ref = oc.run("c4", *args)
    built = fj.build(fj.script(PROGRAMS["c4"]), list(args))
    assert _collapsed(built)
    dev_args = _cuda(args)
    print("collapsed c4 T=%d H=%d L=%d B=%d" % (seq_len, hidden, layers, batch), flush=True)
    _close(built(*dev_args), ref, "first call")
    # calls in a row share the barrier words; one call is one launch of the library
    def launches():
        n = ctypes.c_uint64()
        lib.fx_launch_stats(ctypes.byref(n), None)
        return n.value

    before = launches()
    got = built(*dev_args)
    torch.cuda.synchronize()
    assert launches() - before == 1
    _close(got, ref, "second call")


@pytest.mark.gpu
def test_states_as_arguments_and_a_longer_out_buffer():
    x, wih, whh, bih, bhh = oc.c4_inputs(3, 10, 64, 3, 2)
    h0, c0 = _states(3, 3, 2, 64)
    args = [x, wih, whh, bih, bhh, h0, c0]
    ref = torch.jit.script(lstm_with_states)(*args)
    built = fj.build(fj.script(lstm_with_states), args)
    assert "prim::Loop" not in _kinds(built.graph)
    dev_args = _cuda(args)
    got = built(*dev_args)
    _close(got, ref, "states as arguments")
    assert torch.equal(got[0][10].cpu(), torch.full((2, 64), 7.0))   # the row past the sequence is kept
    assert torch.equal(dev_args[5].cpu(), h0) and torch.equal(dev_args[6].cpu(), c0)   # arguments are never written


@pytest.mark.gpu
def test_fewer_layers_and_steps_than_the_tensors_hold():
    x, wih, whh, bih, bhh = oc.c4_inputs(4, 9, 64, 3, 1)
    h0, c0 = _states(4, 3, 1, 64)
    args = [x, wih, whh, bih, bhh, h0, c0]
    ref = torch.jit.script(lstm_first_layer_only)(*args)
    built = fj.build(fj.script(lstm_first_layer_only), args)
    assert "prim::Loop" not in _kinds(built.graph)
    got = built(*_cuda(args))
    _close(got, ref, "two of three layers, seven of nine steps")
    assert torch.equal(got[1][2].cpu(), h0[2]) and torch.equal(got[0][7:].cpu(), torch.zeros(2, 1, 64))


@pytest.mark.gpu
def test_a_sequence_of_another_length_than_the_example():
    """Regions specialise on the shapes they are called with, not on the example's."""
    args = oc.c4_inputs(0, 6, 64, 2, 1)
    built = fj.build(fj.script(PROGRAMS["c4"]), list(args))
    other = oc.c4_inputs(5, 11, 64, 2, 1)
    _close(built(*_cuda(other)), oc.run("c4", *other), "T=11 through a function built for T=6")
    empty = [torch.zeros(0, 1, 64)] + list(other[1:])
    got = built(*_cuda(empty))
    assert got[0].shape == (0, 1, 64) and not bool(got[1].any()) and got[2].shape == (2, 1, 64)
