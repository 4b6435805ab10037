"""Order-preserving row compaction (the data-dependent masked select of
detection post-processing).  Contract: ATen `x[mask]` / `nonzero` - kept rows
in ascending source order (the reference leaves these to ATen:
functs/csrc/jit/passes/convert_to_tensorssa.cpp:422-443,
fait/passes/fuse_ops.cpp:173-200).  All results bit-exact.
"""
import pytest
import torch

from functs_amd import Region
from tests.util import assert_exact, run_region


def _region(n_cols_shapes, degree=1):
    r = Region(parallel_degree=degree, is_parallel_map=degree > 1)
    m = r.tensor_input(torch.bool, 1, per_task=degree > 1)
    xs = [r.tensor_input(dt, rank, per_task=degree > 1) for dt, rank in n_cols_shapes]
    for x in xs:
        r.output(x)
    r.compact_rows(m)
    return r.finalize()


@pytest.mark.parametrize("n", [0, 1, 63, 64, 65, 255, 256, 257, 1000, 1025, 4096, 5000])
@pytest.mark.parametrize("density", [0.0, 0.3, 1.0])
def test_region_compaction_sizes(backend, n, density):
    if backend == "emul" and n > 1100:
        pytest.skip("large sizes are exercised on the GPU")
    g = torch.Generator().manual_seed(n * 7 + int(density * 10))
    mask = torch.rand(n, generator=g) < density
    a = torch.rand(n, 5, generator=g)
    b = torch.randint(-9, 9, (n,), generator=g)
    c = torch.rand(n, 2, 3, generator=g)
    r = _region([(torch.float32, 2), (torch.int64, 1), (torch.float32, 3)])
    got = run_region(backend, r, mask, a, b, c)
    assert_exact(got, [a[mask], b[mask], c[mask]], "n=%d density=%g" % (n, density))
    assert got[0].shape[0] == int(mask.sum())


def test_region_compaction_mask_computed_in_region(backend):
    r = Region()
    x = r.tensor_input(torch.float32, 2)
    keep = x.select(1, 0) > 0.5
    r.output(x * 2.0)
    r.output(r.arange(0, r.op("SIZE", x, 0)))   # nonzero(): the kept row indices
    r.compact_rows(keep)
    r.finalize()
    t = torch.rand(777, 3, generator=torch.Generator().manual_seed(1))
    got = run_region(backend, r, t)
    m = t[:, 0] > 0.5
    assert_exact(got, [(t * 2.0)[m], torch.nonzero(m)[:, 0]])
    # invariant: strictly increasing source indices
    assert bool((got[1][1:] > got[1][:-1]).all())


def test_parallel_map_compaction_ragged_tasks(backend):
    """Tasks of different lengths in one ParallelMap (task classes)."""
    sizes = [130, 64, 130, 7]
    g = torch.Generator().manual_seed(5)
    masks = [torch.rand(n, generator=g) < 0.4 for n in sizes]
    xs = [torch.rand(n, 3, generator=g) for n in sizes]
    r = _region([(torch.float32, 2)], degree=4)
    (got,) = run_region(backend, r, masks, xs)
    assert_exact(got, [x[m] for x, m in zip(xs, masks)])


@pytest.mark.gpu
@pytest.mark.parametrize("n", [1, 100, 256, 300000, 700000, 2200000])   # the last one: more tiles than sum their predecessors directly
def test_standalone_compact_rows(n):
    from functs_amd import compact_rows
    dev = torch.device("cuda:0")
    g = torch.Generator().manual_seed(n)
    mask = torch.rand(n, generator=g) < 0.5
    a = torch.rand(n, 4, generator=g)
    b = torch.randint(0, 1 << 40, (n,), generator=g)
    c = torch.randint(0, 255, (n, 3), generator=g).to(torch.uint8)
    got = compact_rows(mask.to(dev), [a.to(dev), b.to(dev), c.to(dev)])
    assert_exact([t.cpu() for t in got], [a[mask], b[mask], c[mask]], "standalone n=%d" % n)


@pytest.mark.gpu
def test_standalone_compact_rows_edge_masks():
    from functs_amd import compact_rows
    dev = torch.device("cuda:0")
    a = torch.arange(1000 * 2, dtype=torch.float32).reshape(1000, 2)
    for mask in (torch.zeros(1000, dtype=torch.bool), torch.ones(1000, dtype=torch.bool)):
        (got,) = compact_rows(mask.to(dev), [a.to(dev)])
        assert_exact(got.cpu(), a[mask])


@pytest.mark.gpu
@pytest.mark.parametrize("n", [300, 70000])
def test_standalone_compact_rows_row_shapes(n):
    """Rows that are whole 16-byte groups (moved as such), rows that are not, single words,
    64-bit elements, and a source that is not 16-byte aligned (moved word by word)."""
    from functs_amd import compact_rows
    dev = torch.device("cuda:0")
    g = torch.Generator().manual_seed(n + 1)
    mask = torch.rand(n, generator=g) < 0.6
    cols = [torch.rand(n, 8, generator=g), torch.rand(n, 85, generator=g), torch.rand(n, generator=g),
            torch.randint(0, 1 << 50, (n, 2), generator=g), torch.rand(n, 20, 4, generator=g),
            torch.rand(n * 12 + 1, generator=g)[1:].view(n, 12)]
    dev_cols = [c.to(dev) for c in cols[:-1]] + [torch.rand(n * 12 + 1, generator=g).to(dev)[1:].view(n, 12)]
    cols[-1] = dev_cols[-1].cpu()
    assert dev_cols[-1].data_ptr() % 16 == 4
    got = compact_rows(mask.to(dev), dev_cols)
    assert_exact([t.cpu() for t in got], [c[mask] for c in cols], "row shapes n=%d" % n)
