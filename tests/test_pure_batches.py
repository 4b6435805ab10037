"""The batched interpretation of pure program tails (a leading load followed by
elementwise instructions with immediate operands, four items per dispatch) only
starts on complete batches: big dense outputs and wide compacted rows.  These
sizes are too slow for the CPU emulator, so the tests are GPU-only; the same
programs run at small sizes (generic path) in test_lowering_ops.py."""
import pytest
import torch

from functs_amd import Region
from tests.util import assert_close, assert_exact, run_region

pytestmark = pytest.mark.gpu

CHAINS = {
    "sigmoid": (lambda x: x.sigmoid(), lambda t: t.sigmoid()),
    "exp_scale": (lambda x: (x * 0.25).exp() + 1.5, lambda t: (t * 0.25).exp() + 1.5),
    "relu_neg": (lambda x: -((x - 0.5).relu()), lambda t: -((t - 0.5).relu())),
    "rsub_div": (lambda x: (2.0 - x) / 3.0, lambda t: (2.0 - t) / 3.0),
    "clamp": (lambda x: x.clamp(-0.25, 0.75), lambda t: t.clamp(-0.25, 0.75)),
    "sqrt_abs": (lambda x: x.region.op("SQRT", x.region.op("ABS", x)), lambda t: t.abs().sqrt()),
    "rcp": (lambda x: x.region.op("RECIPROCAL", x + 3.0), lambda t: (t + 3.0).reciprocal()),
    "compare": (lambda x: x > 0.125, lambda t: t > 0.125),
    "to_int": (lambda x: (x * 100.0).to(torch.int32), lambda t: (t * 100.0).to(torch.int32)),
    "copy": (lambda x: x.clone(), lambda t: t.clone()),
}


@pytest.mark.parametrize("name", sorted(CHAINS))
def test_dense_pure_chain_large(name):
    build, ref_fn = CHAINS[name]
    # 8 Mi elements and more select four items per wave; the odd last dimension makes
    # the groups at the row ends partial and the 128-bit accesses unaligned
    g = torch.Generator().manual_seed(11)
    x = torch.randn(4100, 2051, generator=g)
    r = Region()
    xi = r.tensor_input(torch.float32, 2)
    r.output(build(xi))
    reg = r.finalize()
    assert "pure=1 unit_items=4" in reg.disasm(x)  # the batched path is the one under test
    (got,) = run_region("hip", reg, x)
    ref = ref_fn(x)
    if ref.dtype.is_floating_point:
        assert_close(got, ref, name)
    else:
        assert_exact(got, ref, name)


def test_dense_pure_chain_strided_source():
    g = torch.Generator().manual_seed(12)
    x = torch.randn(2052, 4100, generator=g)
    r = Region()
    xi = r.tensor_input(torch.float32, 2)
    r.output((xi.transpose(0, 1) * 2.0).sigmoid())
    (got,) = run_region("hip", r.finalize(), x)
    assert_close(got, (x.t() * 2.0).sigmoid(), "transposed source")


@pytest.mark.parametrize("cols", [64, 85, 3])
def test_compacted_pure_outputs_wide_rows(cols):
    g = torch.Generator().manual_seed(13 + cols)
    n = 5000
    x = torch.randn(n, cols, generator=g)
    key = torch.randn(n, generator=g)
    r = Region()
    xi = r.tensor_input(torch.float32, 2)
    ki = r.tensor_input(torch.float32, 1)
    r.output((xi * 0.5).sigmoid())
    r.output(ki.exp())
    r.output(xi)
    r.compact_rows(ki > -0.5)
    reg = r.finalize()
    assert reg.disasm(x, key).count("pure=1") == 3
    got = run_region("hip", reg, x, key)
    m = key > -0.5
    assert got[0].shape[0] == int(m.sum())
    assert_close(got[0], (x[m] * 0.5).sigmoid(), "sigmoid rows")
    assert_close(got[1], key[m].exp(), "exp keys")
    assert_exact(got[2], x[m], "passthrough rows")
