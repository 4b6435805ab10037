"""int64 data in regions: programs that only move it are exact for every value (the two 32-bit
words travel separately); integer arithmetic is 32-bit, checked at the loads and reported through
fx_async_error.  The library routine (ATen on the CPU) is the pin; the reference's eager bodies are
dtype-generic (functs/csrc/jit/ir/symbol_ext.cpp:17-117)."""
import pytest
import torch

from functs_amd import Region
from functs_amd._lib import C, FxError, lib
from tests.util import assert_exact, run_region

BIG = 1 << 40


def _big(shape, seed):
    g = torch.Generator().manual_seed(seed)
    t = torch.randint(-(1 << 62), 1 << 62, shape, generator=g)
    t.view(-1)[0] = BIG + 7           # low word 7, high word 256
    t.view(-1)[1] = -BIG - 1          # negative, low word all ones
    t.view(-1)[2] = (1 << 31)         # fits 33 bits, not 32
    t.view(-1)[3] = -1
    return t


def test_compaction_moves_every_int64_value(backend):
    n = 1500 if backend == "hip" else 300
    g = torch.Generator().manual_seed(3)
    x = torch.rand(n, 3, generator=g)
    ids = _big((n,), 5)
    pairs = _big((n, 2), 6)
    r = Region()
    xi = r.tensor_input(torch.float32, 2)
    ii = r.tensor_input(torch.int64, 1)
    pi = r.tensor_input(torch.int64, 2)
    r.output(xi * 2.0)
    r.output(ii)
    r.output(pi)
    r.compact_rows(xi.select(1, 0) > 0.4)
    r.finalize()
    lib.fx_async_error(1)
    got = run_region(backend, r, x, ids, pairs)
    m = x[:, 0] > 0.4
    assert_exact(got, [x[m] * 2.0, ids[m], pairs[m]], "compaction of int64 columns")
    assert lib.fx_async_error(1) == 0


def test_select_rev_slice_rev_where_cat_index_on_int64(backend):
    a = _big((6, 5), 11)
    b = _big((5,), 12)
    c = _big((6, 2), 13)
    idx = torch.tensor([5, 0, 0, 3, -1])
    cond = torch.rand(6, 5, generator=torch.Generator().manual_seed(1)) < 0.5
    r = Region()
    ai = r.tensor_input(torch.int64, 2)
    bi = r.tensor_input(torch.int64, 1)
    ci = r.tensor_input(torch.int64, 2)
    ii = r.tensor_input(torch.int64, 1)
    wi = r.tensor_input(torch.bool, 2)
    r.output(ai.select_rev(bi, 0, 2))
    r.output(ai.slice_rev(ci, 1, 1, 5, 2))
    r.output(r.where(wi, ai, bi))
    r.output(r.cat([ai, ci], 1))
    r.output(ai.index(ii))
    r.output(r.where(wi, ai, r.full([6, 5], BIG * 3 + 1, dtype=torch.int64)))
    r.output(ai.permute(1, 0).select(0, 4))
    r.finalize()
    lib.fx_async_error(1)
    got = run_region(backend, r, a, b, c, idx, cond)
    e0 = a.clone(); e0[2] = b
    e1 = a.clone(); e1[:, 1:5:2] = c
    ref = [e0, e1, torch.where(cond, a, b), torch.cat([a, c], 1), a[idx],
           torch.where(cond, a, torch.full((6, 5), BIG * 3 + 1)), a.t()[4]]
    assert_exact(got, ref, "int64 moves")
    assert lib.fx_async_error(1) == 0


def test_int64_to_float_uses_the_whole_element(backend):
    a = _big((4, 8), 21)
    r = Region()
    ai = r.tensor_input(torch.int64, 2)
    r.output(ai.to(torch.float32) * 0.5)
    r.finalize()
    lib.fx_async_error(1)
    (got,) = run_region(backend, r, a)
    assert_exact(got, a.to(torch.float32) * 0.5)
    assert lib.fx_async_error(1) == 0


def test_int64_arithmetic_is_32_bit_and_says_so(backend):
    r = Region()
    ai = r.tensor_input(torch.int64, 1)
    r.output(ai + 3)
    r.output(r.cat([ai * 2, ai], 0))   # arithmetic and a move in one int64 output
    r.finalize()
    small = torch.tensor([5, -7, (1 << 31) - 4, -(1 << 31)])
    lib.fx_async_error(1)
    got = run_region(backend, r, small)
    assert_exact(got[0], small + 3)
    assert_exact(got[1][4:], small)
    assert_exact(got[1][:2], small[:2] * 2)
    assert lib.fx_async_error(1) == 0
    # an element outside 32 bits enters the addition: the launch is flagged
    big = torch.tensor([5, BIG, 1, 2])
    got = run_region(backend, r, big)
    assert lib.fx_async_error(0) == 1
    assert lib.fx_async_error(1) == 1 and lib.fx_async_error(0) == 0
    assert_exact(got[1][4:], big)      # the moved half of the output is still exact


def test_integer_constants_and_scalars_outside_32_bits_are_refused():
    r = Region()
    ai = r.tensor_input(torch.int64, 1)
    r.output(ai + BIG)
    r.finalize()
    arr, n, _ = r._flatten([torch.zeros(4, dtype=torch.int64)])
    with pytest.raises(FxError) as e:
        r.plan(arr, n)
    assert e.value.code == C["FX_E_UNSUPPORTED"] and "outside 32 bits" in str(e.value)

    from tests.support import emul
    r = Region()
    ai = r.tensor_input(torch.int32, 1)
    k = r.scalar_input("int")
    r.output(ai + k)
    r.finalize()
    (got,) = emul.run(r, torch.arange(4, dtype=torch.int32), 9)
    assert_exact(got, torch.arange(4, dtype=torch.int32) + 9)
    with pytest.raises(FxError) as e:
        emul.run(r, torch.arange(4, dtype=torch.int32), BIG)
    assert e.value.code == C["FX_E_LIMIT"]


def test_the_error_word_is_a_set_of_bits_and_a_caller_takes_only_its_own():
    """fx_async_error_take clears the bits its caller handles and leaves the others to whoever
    handles those; fx_async_error(1) clears everything."""
    from functs_amd._lib import C
    lib.fx_async_error(1)
    lib.fx_async_error_report(C["FX_ASYNC_BARRIER"] | C["FX_ASYNC_NMS_CAPACITY"])
    assert lib.fx_async_error_take(C["FX_ASYNC_NMS_CAPACITY"]) == C["FX_ASYNC_NMS_CAPACITY"]
    assert lib.fx_async_error_take(C["FX_ASYNC_NMS_CAPACITY"]) == 0
    assert lib.fx_async_error(0) == C["FX_ASYNC_BARRIER"]
    assert lib.fx_async_error(1) == C["FX_ASYNC_BARRIER"] and lib.fx_async_error(0) == 0
    assert len({C["FX_ASYNC_INT64"], C["FX_ASYNC_BARRIER"], C["FX_ASYNC_NMS_CAPACITY"]}) == 3
    assert C["FX_ASYNC_INT64"] & C["FX_ASYNC_BARRIER"] == 0 and (C["FX_ASYNC_INT64"] | C["FX_ASYNC_BARRIER"]) & C["FX_ASYNC_NMS_CAPACITY"] == 0


@pytest.mark.gpu
def test_the_operator_raises_on_every_kind_of_report_and_works_again_after_it():
    """Whatever an earlier launch reported (a given-up wait of fx::lstm_stack, an NMS overflow, an
    int64 element outside 32 bits), the next fused-region call raises it; the word is cleared by
    that, so the call after it runs."""
    import functs_amd.jit as fj
    from functs_amd._lib import C
    from torch import Tensor

    def f(a: Tensor):
        b = a.clone()
        b[0] = b[1] * 2.0
        return b.sigmoid()

    x = torch.rand(64, 8)
    fn = fj.build(fj.script(f), [x])
    xg = x.cuda()
    ref = fn(xg).cpu()
    for bits, word in ((C["FX_ASYNC_BARRIER"], "lstm_stack"), (C["FX_ASYNC_NMS_CAPACITY"], "candidates"), (C["FX_ASYNC_INT64"], "int64"),
                       (C["FX_ASYNC_BARRIER"] | C["FX_ASYNC_INT64"], "lstm_stack")):
        lib.fx_async_error(1)
        lib.fx_async_error_report(bits)
        with pytest.raises(RuntimeError, match=word):
            fn(xg)
        assert lib.fx_async_error(0) == 0
        assert torch.equal(fn(xg).cpu(), ref)
