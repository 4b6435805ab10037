"""fx_compact_rows_static (the entry point that allocates nothing) against fx_compact_rows
through the C ABI: two calls in a row on the shared device array, the second smaller."""
import ctypes

import pytest
import torch

from tests.util import assert_exact


def _call(static, mask, cols, outs, total):
    from functs_amd._lib import check, lib
    n = mask.numel()
    k = len(cols)
    src = (ctypes.c_void_p * k)(*[c.data_ptr() for c in cols])
    dst = (ctypes.c_void_p * k)(*[o.data_ptr() for o in outs])
    rowlen = (ctypes.c_int32 * k)(*[c.numel() // n for c in cols])
    elsize = (ctypes.c_int32 * k)(*[c.element_size() for c in cols])
    stream = ctypes.c_void_p(torch.cuda.current_stream(mask.device).cuda_stream)
    m8 = mask.view(torch.uint8)
    if static:
        check(lib.fx_compact_rows_static(m8.data_ptr(), n, src, dst, rowlen, elsize, k, total.data_ptr(), stream))
    else:
        sb = lib.fx_compact_rows_scratch_bytes(n)
        scratch = torch.empty(sb, dtype=torch.uint8, device=mask.device)
        check(lib.fx_compact_rows(m8.data_ptr(), n, src, dst, rowlen, elsize, k, scratch.data_ptr(), sb,
                                  total.data_ptr(), stream))
    torch.cuda.current_stream(mask.device).synchronize()
    t = int(total[0])
    return [o[:t].cpu() for o in outs]


@pytest.mark.gpu
def test_static_matches_caller_scratch_two_calls_in_a_row():
    dev = torch.device("cuda:0")
    total = torch.zeros(1, dtype=torch.int32).pin_memory()
    # the first call takes the scan path (more than 8192 tiles of 256 rows), the second, smaller
    # one the direct path, over tile counts that the first call left in the shared array
    for n in (2200001, 4097):
        g = torch.Generator().manual_seed(n)
        mask = torch.rand(n, generator=g) < 0.5
        a = torch.rand(n, 4, generator=g)
        b = torch.randint(0, 1 << 40, (n,), generator=g)
        c = torch.randint(0, 255, (n, 3), generator=g).to(torch.uint8)
        cols = [a.to(dev), b.to(dev), c.to(dev)]
        m = mask.to(dev)
        # every output is allocated before the call under test
        ref_outs = [torch.empty_like(x) for x in cols]
        got_outs = [torch.empty_like(x) for x in cols]
        ref = _call(False, m, cols, ref_outs, total)
        got = _call(True, m, cols, got_outs, total)
        assert_exact(got, ref, "static vs caller scratch, n=%d" % n)
        assert_exact(got, [a[mask], b[mask], c[mask]], "static vs ATen, n=%d" % n)


@pytest.mark.gpu
def test_static_rejects_sizes_beyond_its_array():
    from functs_amd._lib import C, lib
    dev = torch.device("cuda:0")
    n = C["FX_COMPACT_ROWS_STATIC_MAX"] + 1
    mask = torch.zeros(n, dtype=torch.uint8, device=dev)
    total = torch.zeros(1, dtype=torch.int32).pin_memory()
    rc = lib.fx_compact_rows_static(mask.data_ptr(), n, None, None, None, None, 0, total.data_ptr(), None)
    assert rc == C["FX_E_LIMIT"]
    assert b"above the limit" in lib.fx_last_error()
