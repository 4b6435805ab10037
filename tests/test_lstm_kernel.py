"""The stacked-LSTM recurrence as one persistent kernel (fx_lstm_stack) against the oracle (stock
TorchScript on the CPU, oracle/configs.py c4_fn, itself pinned against torch.nn.LSTM in
tests/test_oracle.py).  Reference loop: functs/benchmark/ai_model/lstm/lstm.py:79-133.
Tolerance: 1e-4 relative, the bound stated for 64 dependent steps of fp32 arithmetic whose sums
are taken in another order than the oracle's BLAS takes them, plus 5e-6 absolute: a gate is a sum
of up to 2 x 1024 products of magnitude 0.1, whose rounding error (a few 1e-6) does not shrink
with the result when that happens to be near zero.
On the CPU, the kernel's schedule (diagonals t + j, two parities of the h buffer) and its
hand-over protocol (values tagged with their step, bounded polls, the tag base carried from launch
to launch) run with one host thread per workgroup (tests/support/lstm_emul.cpp)."""
import ctypes

import pytest
import torch

from oracle import configs as oc

RTOL = 1e-4
ATOL = 5e-6


def _inputs(seed, T, H, L, B):
    x, wih, whh, bih, bhh = oc.c4_inputs(seed, seq_len=T, hidden=H, layers=L, batch=B)
    g = torch.Generator().manual_seed(seed + 99)
    h0 = torch.rand(L, B, H, generator=g) * 0.2 - 0.1
    c0 = torch.rand(L, B, H, generator=g) * 0.2 - 0.1
    return x, wih, whh, bih, bhh, h0, c0


def _reference(x, wih, whh, bih, bhh, h0, c0):
    """The loop nest of the oracle's c4_fn with initial states (c4_fn starts from zeros)."""
    T, B, H = x.shape
    L = wih.size(0)
    out = torch.zeros(T, B, H)
    sh, sc = h0.clone(), c0.clone()
    for t in range(T):
        cur = x[t]
        for j in range(L):
            ih = torch.matmul(cur, wih[j]) + bih[j]
            hh = torch.matmul(sh[j], whh[j]) + bhh[j]
            i, f = torch.sigmoid(ih[0] + hh[0]), torch.sigmoid(ih[1] + hh[1])
            g, o = torch.tanh(ih[2] + hh[2]), torch.sigmoid(ih[3] + hh[3])
            c2 = f * sc[j] + i * g
            h2 = o * torch.tanh(c2)
            sc[j], sh[j] = c2, h2
            cur = h2
        out[t] = cur
    return out, sh, sc


def _close(got, ref, what):
    for g, r, n in zip(got, ref, ("out", "state_h", "state_c")):
        assert g.shape == r.shape, (what, n)
        err = (g.double() - r.double()).abs()
        bad = err > ATOL + RTOL * r.double().abs()
        assert not bool(bad.any()), "%s %s: %d beyond rtol %g (max err %g)" % (what, n, int(bad.sum()), RTOL, err.max())


def test_reference_with_zero_states_is_the_oracle():
    x, wih, whh, bih, bhh, _, _ = _inputs(0, 7, 32, 2, 1)
    z = torch.zeros(2, 1, 32)
    ref = _reference(x, wih, whh, bih, bhh, z, z)
    orc = oc.run("c4", x, wih, whh, bih, bhh)
    for a, b in zip(ref, orc):
        assert torch.allclose(a, b, rtol=1e-6, atol=1e-7)


def _emul(x, wih, whh, bih, bhh, h0, c0, spin=1 << 30, skip=-1, launches=1, base0=0):
    from tests.support import emul
    so = emul.lstm_emul()
    T, B, H = x.shape
    L = wih.size(0)
    out, sh, sc = torch.zeros(T, B, H), torch.zeros(L, B, H), torch.zeros(L, B, H)
    ts = [None if t is None else t.contiguous() for t in (x, wih, whh, bih, bhh, h0, c0)]
    err = so.fx_lstm_emul(*[None if t is None else t.data_ptr() for t in ts], out.data_ptr(), sh.data_ptr(),
                          sc.data_ptr(), T, B, H, L, spin, skip, launches, base0)
    return (out, sh, sc), err


@pytest.mark.parametrize("T,H,L,B", [(1, 32, 1, 1), (5, 32, 2, 1), (9, 64, 3, 2), (4, 32, 4, 3), (12, 96, 2, 1)])
def test_schedule_and_barrier_on_host_threads(T, H, L, B):
    args = _inputs(T * 7 + L, T, H, L, B)
    got, err = _emul(*args)
    assert err == 0
    _close(got, _reference(*args), "emul T=%d H=%d L=%d B=%d" % (T, H, L, B))


def test_launches_in_a_row_share_a_workspace_cleared_once():
    """The last workgroup to leave moves the tag base past the launch's tags (-1: it did not), so
    the values the next launch finds never carry a tag it waits for - also for the shortest
    sequences, whose tags would repeat from launch to launch otherwise."""
    args = _inputs(11, 6, 64, 3, 2)
    got, err = _emul(*args, launches=3)
    assert err == 0
    _close(got, _reference(*args), "third launch")
    args = _inputs(12, 1, 32, 2, 1)
    got, err = _emul(*args, launches=4)
    assert err == 0
    _close(got, _reference(*args), "fourth launch of a one-step sequence")


def test_the_tag_base_starts_over_before_it_wraps():
    args = _inputs(13, 5, 32, 2, 1)
    got, err = _emul(*args, launches=3, base0=0x80000000 - 8)
    assert err == 0
    _close(got, _reference(*args), "launch after the tags were cleared")


def test_no_initial_state_means_zeros():
    x, wih, whh, bih, bhh, _, _ = _inputs(5, 6, 32, 2, 2)
    got, err = _emul(x, wih, whh, bih, bhh, None, None)
    assert err == 0
    z = torch.zeros(2, 2, 32)
    _close(got, _reference(x, wih, whh, bih, bhh, z, z), "zero state")


def test_a_wait_that_cannot_end_is_given_up():
    """One workgroup stops writing: every other one must give up after the poll limit, set the
    error word and return (on the GPU the kernel then ends instead of hanging)."""
    args = _inputs(3, 6, 32, 2, 1)
    _, err = _emul(*args, spin=2000, skip=5)
    assert err == 1


def test_after_a_given_up_wait_the_workspace_refuses_work_until_it_is_cleared():
    """The launch that gives up fills its results with NaN; the next launch on the same workspace
    (whatever the host did with the error report in between) does no step, reports the error
    again and returns NaN; on a cleared workspace the sequence runs."""
    from tests.support import emul
    so = emul.lstm_emul()
    args = _inputs(4, 6, 32, 2, 1)
    x = args[0]
    T, B, H = x.shape
    L = args[1].size(0)
    out, sh, sc = torch.zeros(T, B, H), torch.zeros(L, B, H), torch.zeros(L, B, H)
    ts = [t.contiguous() for t in args]
    bits = so.fx_lstm_emul_give_up(*[t.data_ptr() for t in ts], out.data_ptr(), sh.data_ptr(), sc.data_ptr(),
                                   T, B, H, L, 2000, 5)
    assert bits & 1, "the first launch did not give up"
    assert bits & 2, "the launch that gave up left values that look like results"
    assert bits & 4 and bits & 8, "the launch on the workspace of a given-up wait ran"
    assert bits & 16, "the launch on the cleared workspace failed"
    _close((out, sh, sc), _reference(*args), "launch on the cleared workspace")


def _gpu(x, wih, whh, bih, bhh, h0, c0, launches=1):
    """`launches` calls in a row on one workspace that is cleared once; the last call's results."""
    from functs_amd._lib import check, lib
    dev = torch.device("cuda:0")
    T, B, H = x.shape
    L = wih.size(0)
    ts = [None if t is None else t.contiguous().to(dev) for t in (x, wih, whh, bih, bhh, h0, c0)]
    nbytes = lib.fx_lstm_stack_workspace_bytes(B, H, L)
    ws = torch.zeros(nbytes, dtype=torch.uint8, device=dev)
    assert ws.data_ptr() % 256 == 0
    stream = ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream)
    for _ in range(launches):
        out = torch.full((T, B, H), float("nan"), device=dev)
        sh, sc = torch.full((L, B, H), float("nan"), device=dev), torch.full((L, B, H), float("nan"), device=dev)
        print("fx_lstm_stack T=%d B=%d H=%d L=%d" % (T, B, H, L), flush=True)
        check(lib.fx_lstm_stack(*[None if t is None else t.data_ptr() for t in ts], out.data_ptr(), sh.data_ptr(),
                                sc.data_ptr(), T, B, H, L, ws.data_ptr(), nbytes, stream))
        torch.cuda.synchronize()
        assert lib.fx_async_error(1) == 0
    return out.cpu(), sh.cpu(), sc.cpu()


@pytest.mark.gpu
@pytest.mark.parametrize("T,H,L,B", [(1, 32, 1, 1), (5, 64, 2, 1), (9, 128, 3, 2), (4, 32, 4, 3), (16, 256, 2, 1),
                                     (64, 512, 2, 1), (6, 512, 4, 16), (8, 1024, 1, 2), (7, 1024, 2, 1)])
def test_kernel_against_the_oracle(T, H, L, B):
    args = _inputs(T + H + L, T, H, L, B)
    _close(_gpu(*args), _reference(*args), "gpu T=%d H=%d L=%d B=%d" % (T, H, L, B))


@pytest.mark.gpu
def test_launches_in_a_row_on_one_workspace_and_no_initial_state():
    x, wih, whh, bih, bhh, _, _ = _inputs(21, 10, 128, 2, 2)
    z = torch.zeros(2, 2, 128)
    _close(_gpu(x, wih, whh, bih, bhh, None, None, launches=3), _reference(x, wih, whh, bih, bhh, z, z), "third launch")


@pytest.mark.gpu
def test_benchmark_configuration_against_nn_lstm():
    """T = 64, H = 512, two layers, zero initial states: the library routine as a second opinion."""
    x, wih, whh, bih, bhh = oc.c4_inputs(0)
    z = torch.zeros(2, 1, 512)
    out, sh, sc = _gpu(x, wih, whh, bih, bhh, z, z)
    lstm = torch.nn.LSTM(512, 512, 2)
    with torch.no_grad():
        for l in range(2):
            getattr(lstm, "weight_ih_l%d" % l).copy_(wih[l].transpose(1, 2).reshape(2048, 512))
            getattr(lstm, "weight_hh_l%d" % l).copy_(whh[l].transpose(1, 2).reshape(2048, 512))
            getattr(lstm, "bias_ih_l%d" % l).copy_(bih[l].reshape(2048))
            getattr(lstm, "bias_hh_l%d" % l).copy_(bhh[l].reshape(2048))
        ref, (hn, cn) = lstm(x)
    _close((out, sh, sc), (ref, hn, cn), "nn.LSTM")


@pytest.mark.gpu
def test_unsupported_shapes_are_refused():
    from functs_amd._lib import C, lib
    dev = torch.device("cuda:0")
    t = torch.zeros(1 << 16, device=dev)
    ws = torch.zeros(1 << 20, dtype=torch.uint8, device=dev)
    p = t.data_ptr()
    rc = lib.fx_lstm_stack(p, p, p, p, p, p, p, p, p, p, 4, 1, 48, 2, ws.data_ptr(), 1 << 20, None)   # hidden not a multiple of 32
    assert rc == C["FX_E_UNSUPPORTED"]
    rc = lib.fx_lstm_stack(p, p, p, p, p, p, p, p, p, p, 4, 1, 64, 5, ws.data_ptr(), 1 << 20, None)   # five layers
    assert rc == C["FX_E_UNSUPPORTED"]


def test_sizes_the_kernel_is_built_for():
    from functs_amd._lib import lib
    assert lib.fx_lstm_stack_fits(1, 512, 2) == 1 and lib.fx_lstm_stack_fits(16, 512, 4) == 1
    assert lib.fx_lstm_stack_fits(1, 1024, 2) == 1 and lib.fx_lstm_stack_fits(1, 1024, 3) == 0
    assert lib.fx_lstm_stack_fits(1, 96, 2) == 0 and lib.fx_lstm_stack_fits(17, 64, 2) == 0 and lib.fx_lstm_stack_fits(1, 64, 5) == 0
