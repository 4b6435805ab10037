"""The C-ABI shared library: loads, exports every symbol include/fxhip.h
declares, and reports errors the way the header says (no compute calls here)."""
import ctypes
import re

import pytest
import torch

from functs_amd import Region, _lib
from functs_amd._lib import C, lib


def test_exports_every_declared_symbol():
    names = _lib.exported_symbols()
    assert len(names) >= 30
    for n in names:
        assert hasattr(lib, n), "libfxhip.so does not export %s" % n


def test_version_and_constants():
    assert lib.fx_api_version() == C["FX_API_VERSION"] == 1
    assert C["FX_OP_ACCESS"] == 1
    assert C["FX_OP_TRIL"] + 1 == C["FX_OP__COUNT"]  # new opcodes are appended: numbers of the ABI never move


def test_header_cites_reference_lines():
    text = open(_lib.HEADER_PATH).read()
    for needle in ("cuda_codegen_tssa.cpp:1167-1290", "graph_builder.cpp:259-712", "nnc_ext.cpp:187-212",
                   "te_op.h:13-23"):
        assert needle in text


def test_error_reporting():
    r = Region()
    x = r.tensor_input(torch.float32, 2)
    with pytest.raises(_lib.FxError) as e:
        r.finalize()  # no outputs
    assert e.value.code == C["FX_E_INVALID"]
    r.output(x.select(5, 0))
    r.finalize()
    arr, n, _ = r._flatten([torch.rand(3, 4)])
    with pytest.raises(_lib.FxError) as e:
        r.plan(arr, n)  # dim out of range, found when shapes are known
    assert e.value.code == C["FX_E_INVALID"]
    assert "select" in str(e.value)


def test_wrong_argument_count_and_dtype():
    r = Region()
    x = r.tensor_input(torch.float32, 2)
    r.output(x + 1.0)
    r.finalize()
    with pytest.raises(_lib.FxError):
        r._flatten([torch.rand(2, 2), 3])
    arr, n, _ = r._flatten([torch.rand(2, 2).double().float().to(torch.int64)])
    with pytest.raises(_lib.FxError) as e:
        r.plan(arr, n)
    assert "dtype" in str(e.value)


def test_unsupported_is_reported_not_faked():
    r = Region()
    x = r.tensor_input(torch.float32, 2)
    m = r.tensor_input(torch.bool, 1)
    r.output(x.index(m))  # bool-mask index is not an elementwise gather
    r.finalize()
    arr, n, _ = r._flatten([torch.rand(4, 2), torch.ones(4, dtype=torch.bool)])
    with pytest.raises(_lib.FxError) as e:
        r.plan(arr, n)
    assert e.value.code == C["FX_E_UNSUPPORTED"]


def test_plan_metadata_and_disasm():
    from functs_amd import configs
    from oracle import configs as oc
    r = configs.build_c5(3)
    preds, anchors, strides = oc.c5_inputs(0, [2, 3], 3)
    arr, n, _ = r._flatten([preds, anchors, strides])
    p = r.plan(arr, n)
    # this region is the detection head that has a kernel of its own (one launch); without it
    # two kernels in the two-pass form, one in the streaming form
    assert p.n_out == 3 and p.compact
    assert _lib.lib.fx_plan_launches(p.handle) == 1 and _lib.lib.fx_plan_streaming(p.handle) == 0
    _lib.lib.fx_set_head_kernel(0)
    _lib.lib.fx_set_rowstream(0)
    try:
        assert _lib.lib.fx_plan_launches(p.handle) == 2 and _lib.lib.fx_plan_streaming(p.handle) == 0
        _lib.lib.fx_set_streaming(1)
        try:
            assert _lib.lib.fx_plan_launches(p.handle) == 1 and _lib.lib.fx_plan_streaming(p.handle) == 1
        finally:
            _lib.lib.fx_set_streaming(0)
    finally:
        _lib.lib.fx_set_head_kernel(1)
        _lib.lib.fx_set_rowstream(1)
    assert p.out_meta[1][2] == (torch.float32, (preds.size(1), 80))
    assert p.alg_bytes == (preds.numel() + anchors.numel() + strides.numel()) * 4
    assert p.scratch_bytes > 0
    text = r.disasm(preds, anchors, strides)
    assert "SIGMOID" in text and "mask:" in text
    # the plan is cached by shape signature
    assert r.plan(arr, n) is p


def test_region_without_gpu_fails_loudly():
    if torch.cuda.is_available():
        pytest.skip("GPU present")
    r = Region()
    x = r.tensor_input(torch.float32, 1)
    r.output(x + 1.0)
    r.finalize()
    with pytest.raises(_lib.FxError):
        r(torch.rand(4))  # CPU tensors: no fallback path


def test_polling_for_the_kept_row_counts_never_blocks():
    """fx_region_poll_totals looks at the pinned words only: 0 while a task's count is pending
    (after the time it was given), 1 once every count is there; not for regions that keep all rows."""
    import time
    r = Region(parallel_degree=3, is_parallel_map=True)
    x = r.tensor_input(torch.float32, 2, per_task=True)
    r.compact_rows(x.select(1, 0) > 0.5)
    r.output(x * 2.0)
    r.finalize()
    xs = [torch.rand(10 + k, 4) for k in range(3)]
    arr, n, keep = r._flatten((xs,))
    p = r.plan(arr, n)
    pending = 0xFFFFFFFF
    totals = (ctypes.c_uint32 * 3)(5, pending, 7)
    t0 = time.perf_counter()
    assert lib.fx_region_poll_totals(p.handle, totals, 2000) == 0
    assert 0.0015 < time.perf_counter() - t0 < 0.5
    assert lib.fx_region_poll_totals(p.handle, totals, 0) == 0
    totals[1] = 0
    assert lib.fx_region_poll_totals(p.handle, totals, 0) == 1
    dense = Region()
    d = dense.tensor_input(torch.float32, 2)
    dense.output(d + 1.0)
    dense.finalize()
    arr, n, keep = dense._flatten((torch.rand(4, 4),))
    assert lib.fx_region_poll_totals(dense.plan(arr, n).handle, totals, 0) < 0
